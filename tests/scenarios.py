"""Scenarios that compare an engine with the plain implementation; the engine is made by a
factory, so the same scenarios run with the stand-in kernels on the CPU and with the HIP
kernels on the GPU."""
from __future__ import annotations

import torch

from helpers import CONFIGS, plain_logits, plain_model, random_tokens, assert_logits_close
from synaptix_amd.engine.generate import generate, GenerationConfig
import plain_qwen3 as P


def lengths_for(name):
    # the batches named for the two tiny configurations (5/17/11 and 1/33/7/64 tokens), plus lengths around a page's edge
    return {"A": [5, 17, 11, 64, 65], "B": [1, 33, 7, 64, 130], "C": [3, 70, 129, 40, 200],
            "E": [2, 66, 9, 130, 31], "F": [4, 65, 20]}[name]


def requests_for(name, tail=0):
    V = CONFIGS[name]["vocab_size"]
    return {f"r{i}": random_tokens(V, n + tail, 100 + i) for i, n in enumerate(lengths_for(name))}


def whole(make_engine, name, dtype, sharp=False):
    """Each request alone and whole: one step, every position wanted."""
    eng = make_engine(name, dtype, 1024, sharp)
    for rid, toks in requests_for(name).items():
        s = eng.acquire()
        got = eng.step([(s, toks)], want="all")
        assert_logits_close(got, plain_logits(name, toks, sharp), dtype, f"{name} {dtype} {rid} whole", sharp)
        eng.release(s)
    eng.cache.check()


def last_tokens_one_by_one(make_engine, name, dtype, tail=32, sharp=False):
    """The same requests with their last `tail` tokens decoded one by one."""
    eng = make_engine(name, dtype, 2048, sharp)
    for rid, toks in requests_for(name, tail).items():
        want = plain_logits(name, toks, sharp)
        s = eng.acquire()
        head = len(toks) - tail
        got = [eng.step([(s, toks[:head])], want="all")]
        for t in toks[head:]:
            got.append(eng.step([(s, [t])], want="last"))
        assert_logits_close(torch.cat(got), want, dtype, f"{name} {dtype} {rid} last {tail} one by one", sharp)
        eng.release(s)
    eng.cache.check()


def unequal_batches(make_engine, name, dtype, sharp=False, decode=12):
    """Batches of unequal lengths whose shorter requests end earlier, one batch after another so
    that slots and pages are used again; the second batch's order differs from the first's."""
    reqs = requests_for(name, tail=0)
    ids = list(reqs)
    batches = [ids[:3], ids[3:] + ids[:1], list(reversed(ids))]
    eng = make_engine(name, dtype, 64 * 12, sharp)
    for batch in batches:
        slots = {r: eng.acquire() for r in batch}
        head = {r: max(1, len(reqs[r]) - decode) for r in batch}
        got = {r: [] for r in batch}
        lg = eng.step([(slots[r], reqs[r][:head[r]]) for r in batch], want="all")
        off = 0
        for r in batch:
            got[r].append(lg[off:off + head[r]])
            off += head[r]
        fed = dict(head)
        live = [r for r in batch if fed[r] < len(reqs[r])]
        for r in batch:
            if r not in live:
                eng.release(slots[r])
        while live:
            lg = eng.step([(slots[r], [reqs[r][fed[r]]]) for r in live], want="last")
            for i, r in enumerate(live):
                got[r].append(lg[i:i + 1])
                fed[r] += 1
            for r in [r for r in live if fed[r] == len(reqs[r])]:
                eng.release(slots[r])                       # leaves the batch; the others go on
            live = [r for r in live if fed[r] < len(reqs[r])]
        for r in batch:
            assert_logits_close(torch.cat(got[r]), plain_logits(name, reqs[r], sharp), dtype,
                                f"{name} {dtype} {r} in batch {batch}", sharp)
        eng.cache.check()
    assert eng.cache.free_slots == eng.cache.max_slots


def long_decoding(make_engine, name, dtype, n_decode):
    """A short prompt, then many single tokens: positions cross several pages."""
    V = CONFIGS[name]["vocab_size"]
    toks = random_tokens(V, 3 + n_decode, 7)
    want = plain_logits(name, toks)
    eng = make_engine(name, dtype, 1024, False)
    s = eng.acquire()
    got = [eng.step([(s, toks[:3])], want="all")]
    for t in toks[3:]:
        got.append(eng.step([(s, [t])], want="last"))
    got = torch.cat(got)
    assert_logits_close(got, want, dtype, f"{name} {dtype} long decoding")
    # the last positions alone, so that an error that grows with the position is not averaged away
    assert_logits_close(got[-8:], want[-8:], dtype, f"{name} {dtype} long decoding, last positions")


def wide_batch(make_engine, name, dtype, n_seqs=70, n_decode=3):
    """More sequences than 64 in one batch: the products leave the kernels for few rows, the
    captured decode step takes a bucket of 96 rows with 26 of padding."""
    V = CONFIGS[name]["vocab_size"]
    reqs = [random_tokens(V, 2 + (7 * i) % 23 + n_decode, 500 + i) for i in range(n_seqs)]
    eng = make_engine(name, dtype, 64 * n_seqs, False)
    slots = [eng.acquire() for _ in reqs]
    heads = [len(r) - n_decode for r in reqs]
    lg = eng.step([(s, r[:h]) for s, r, h in zip(slots, reqs, heads)], want="last")
    got = [[lg[i:i + 1]] for i in range(n_seqs)]
    runner = eng.decode_runner(n_seqs, 64) if eng.graph_ok else None
    for d in range(n_decode):
        toks = [r[h + d] for r, h in zip(reqs, heads)]
        if runner is not None and d > 0:                  # the first single-token step eagerly, the rest replayed
            _, lg = runner.step(slots, toks)
        else:
            lg = eng.step([(s, [t]) for s, t in zip(slots, toks)], want="last")
        for i in range(n_seqs):
            got[i].append(lg[i:i + 1].clone())
    for i in (0, 1, 17, 33, 64, 65, n_seqs - 1):
        want = plain_logits(name, reqs[i])[heads[i] - 1:]
        assert_logits_close(torch.cat(got[i]), want, dtype, f"{name} {dtype} sequence {i} of {n_seqs}")
    for s in slots:
        eng.release(s)
    eng.cache.check()


def long_context(make_engine, dtype, n_prompt=6000, n_decode=4):
    """Thousands of tokens: page tables wider than 64 pages, attention over ~100 key blocks in the
    prompt and, token by token, over many splits; positions where rounding of angles would show."""
    name = "L"
    V = CONFIGS[name]["vocab_size"]
    toks = random_tokens(V, n_prompt + n_decode, 9)
    want = plain_logits(name, toks)
    eng = make_engine(name, dtype, n_prompt + 128, False)
    s = eng.acquire()
    places = [0, 63, 64, 4095, 4096, n_prompt - 2, n_prompt - 1]
    got = eng.step([(s, toks[:n_prompt])], want=[places])
    assert_logits_close(got, want[places], dtype, f"{dtype} long prompt")
    dec = torch.cat([eng.step([(s, [t])], want="last") for t in toks[n_prompt:]])
    assert_logits_close(dec, want[n_prompt:], dtype, f"{dtype} decoding after a long prompt")
    eng.release(s)


def decode_beside_fresh_prompt(make_engine, name, dtype, sharp=False):
    """One step that holds a sequence in its decode phase (tokens cached, one new token) and a
    prompt that starts; then both decode; then a chunk of several tokens beside a single token."""
    V = CONFIGS[name]["vocab_size"]
    old, new = random_tokens(V, 70 + 5, 31), random_tokens(V, 45 + 2, 32)
    want_old, want_new = plain_logits(name, old, sharp), plain_logits(name, new, sharp)
    eng = make_engine(name, dtype, 1024, sharp)
    a, b = eng.acquire(), eng.acquire()
    got_old = [eng.step([(a, old[:70])], want="all")]
    lg = eng.step([(a, old[70:71]), (b, new[:45])], want="all")      # decode beside a fresh prompt
    got_old.append(lg[:1])
    got_new = [lg[1:]]
    lg = eng.step([(b, new[45:46]), (a, old[71:72])], want="last")   # both decode, order swapped
    got_new.append(lg[:1])
    got_old.append(lg[1:])
    lg = eng.step([(a, old[72:75]), (b, new[46:47])], want="all")    # a chunk of three beside one token
    got_old.append(lg[:3])
    got_new.append(lg[3:])
    assert_logits_close(torch.cat(got_old), want_old, dtype, f"{name} {dtype} the sequence that was decoding", sharp)
    assert_logits_close(torch.cat(got_new), want_new, dtype, f"{name} {dtype} the prompt that joined", sharp)
    eng.release(a)
    eng.release(b)
    eng.cache.check()


def chunked_prompts(make_engine, name, dtype, chunk, sharp=False):
    """Prompts fed in chunks of `chunk` tokens, all unfinished prompts in each step (what the
    generation loop does with prefill_batch): a chunk starts inside a page and may cross pages."""
    reqs = requests_for(name)
    eng = make_engine(name, dtype, 1024, sharp)
    slots = {r: eng.acquire() for r in reqs}
    fed = {r: 0 for r in reqs}
    got = {r: [] for r in reqs}
    while True:
        batch = [r for r in reqs if fed[r] < len(reqs[r])]
        if not batch:
            break
        lg = eng.step([(slots[r], reqs[r][fed[r]:fed[r] + chunk]) for r in batch], want="all")
        off = 0
        for r in batch:
            n = min(chunk, len(reqs[r]) - fed[r])
            got[r].append(lg[off:off + n])
            off += n
            fed[r] += n
    for r in reqs:
        assert_logits_close(torch.cat(got[r]), plain_logits(name, reqs[r], sharp), dtype,
                            f"{name} {dtype} {r} in chunks of {chunk}", sharp)
        eng.release(slots[r])
    eng.cache.check()


def generation_with_chunked_prompt(make_engine, name, dtype, n_prompt=200, prefill_batch=64, n_new=6):
    """The generation loop feeding a prompt in chunks of prefill_batch tokens."""
    V = CONFIGS[name]["vocab_size"]
    prompts = [random_tokens(V, n_prompt, 41), random_tokens(V, 70, 42)]
    plain = plain_model(name)
    eng = make_engine(name, dtype, 1024, False)
    outs, _ = generate(eng, prompts, GenerationConfig(max_new_tokens=n_new, prefill_batch=prefill_batch))
    for p, o in zip(prompts, outs):
        want = P.generate(plain, p, n_new)
        if dtype == "float32":
            assert o.tokens == want
        else:
            check_greedy_path(plain, p, o.tokens, want)
    eng.cache.check()


def long_context_through_graphs(make_engine, dtype, n_prompt=6300, n_decode=3):
    """More than 96 pages a sequence, decoded through captured steps whose page tables are 128
    and 256 pages wide: with one row the keys are cut into 32 and 64 splits, with 32 rows into
    16 (the rule for long contexts); a short sequence beside the long one leaves most of its
    splits empty."""
    from synaptix_amd.kernels import ops
    name = "L"
    V = CONFIGS[name]["vocab_size"]
    nkv = CONFIGS[name]["num_key_value_heads"]
    assert ops.decode_splits(1, nkv, 128) == 32 and ops.decode_splits(1, nkv, 256) == 64
    assert ops.decode_splits(32, nkv, 128) == 16        # the branch for contexts of 96 pages and more
    long_toks = random_tokens(V, n_prompt + 3 * n_decode, 9)
    short_toks = random_tokens(V, 20 + 3 * n_decode, 10)
    want_long, want_short = plain_logits(name, long_toks), plain_logits(name, short_toks)
    eng = make_engine(name, dtype, n_prompt + 256, False)
    if not eng.graph_ok:
        return
    a, b = eng.acquire(), eng.acquire()
    eng.step([(a, long_toks[:n_prompt]), (b, short_toks[:20])], want=None)
    got_long, got_short = [], []
    at = 0
    for rows, cap in ((1, 8192), (1, 16384), (32, 8192)):
        runner = eng.decode_runner(rows, cap)
        assert runner.widths[0] == (128 if cap == 8192 else 256) and runner.rows == rows
        for _ in range(n_decode):
            if rows == 1:                                   # one row: the long sequence alone, the short one eagerly
                _, lg = runner.step([a], [long_toks[n_prompt + at]])
                got_long.append(lg[:1].clone())
                got_short.append(eng.step([(b, [short_toks[20 + at]])], want="last"))
            else:
                _, lg = runner.step([b, a], [short_toks[20 + at], long_toks[n_prompt + at]])
                got_short.append(lg[:1].clone())
                got_long.append(lg[1:2].clone())
            at += 1
    assert_logits_close(torch.cat(got_long), want_long[n_prompt:], dtype, f"{dtype} long sequence through wide graphs")
    assert_logits_close(torch.cat(got_short), want_short[20:], dtype, f"{dtype} short sequence beside it")
    eng.release(a)
    eng.release(b)
    eng.cache.check()


def first_tokens(make_engine, name, dtype):
    """Prompts of one and two tokens; the very first position; a chunk that starts at position 1."""
    V = CONFIGS[name]["vocab_size"]
    eng = make_engine(name, dtype, 512, False)
    toks = random_tokens(V, 4, 8)
    want = plain_logits(name, toks)
    a, b, c = eng.acquire(), eng.acquire(), eng.acquire()
    lg = eng.step([(a, toks[:1]), (b, toks[:2]), (c, toks)], want=[[0], [0, 1], [0, 3]])
    assert_logits_close(lg[0:1], want[0:1], dtype, "one token")
    assert_logits_close(lg[1:3], want[0:2], dtype, "two tokens")
    assert_logits_close(lg[3:5], want[[0, 3]], dtype, "places 0 and 3")
    lg = eng.step([(a, toks[1:])], want="all")                 # positions 1..3 in one step after position 0
    assert_logits_close(lg, want[1:], dtype, "a chunk from position 1")
    lg = eng.step([(b, toks[2:3])], want=None)                 # nothing wanted: the cache still advances
    assert lg.shape[0] == 0 and eng.length(b) == 3
    lg = eng.step([(b, toks[3:])], want="last")
    assert_logits_close(lg, want[3:], dtype, "after a step that wanted nothing")


def greedy_generation(make_engine, name, dtype, n_new=8):
    """Greedy generation through the generation loop equals the plain implementation's."""
    V = CONFIGS[name]["vocab_size"]
    prompts = [random_tokens(V, n, 200 + i) for i, n in enumerate(lengths_for(name)[:4])]
    plain = plain_model(name)
    want = [P.generate(plain, p, n_new) for p in prompts]
    eng = make_engine(name, dtype, 2048, False)
    outs, stats = generate(eng, prompts, GenerationConfig(max_new_tokens=n_new), max_batch=3)
    assert stats.batches == 2
    for p, o, w in zip(prompts, outs, want):
        if dtype == "float32":
            assert o.tokens == w
        else:
            check_greedy_path(plain, p, o.tokens, w)
    eng.cache.check()


def check_greedy_path(plain, prompt, got, want, margin=2e-2):
    """bfloat16 may leave the plain greedy path, but only where the plain logits nearly tie."""
    for i, (g, w) in enumerate(zip(got, want)):
        if g != w:
            row = plain.forward(list(prompt) + want[:i])[-1]
            assert float(row[w] - row[g]) <= margin * max(1.0, float(row.abs().max())), \
                f"token {i}: engine {g}, plain {w}, and the plain logits do not tie"
            return


def generation_with_every_processor(make_engine, name):
    """Penalties over the last tokens, temperature, top-k, top-p and min-p together, two requests with streams of
    their own, in 32-bit: the tokens are the plain implementation's (its processors in the reference's order on
    the plain logits, the same uniform numbers).  What a request's penalties see grows with the tokens it has
    drawn, and a wrong window, a processor out of order or a row's options given to its neighbour changes the
    draws within a few tokens."""
    V = CONFIGS[name]["vocab_size"]
    options = dict(temperature=0.9, k=12, p=0.9, mp=0.02, repetition=1.3, last_n=6, presence=0.2, frequency=0.1)
    cfg = GenerationConfig(max_new_tokens=14, temperature=0.9, top_k=12, top_p=0.9, min_p=0.02, repetition_penalty=1.3,
                           repeat_last_n=6, presence_penalty=0.2, frequency_penalty=0.1, seed=5)
    prompts = [random_tokens(V, n, 400 + i) for i, n in enumerate((9, 30))]
    plain = plain_model(name)
    eng = make_engine(name, "float32", 1024, False)
    outs, _ = generate(eng, prompts, cfg)
    for i, (p, o) in enumerate(zip(prompts, outs)):
        want = P.generate(plain, p, 14, seed=5 + i, **options)
        assert o.tokens == want, f"request {i}: {o.tokens} vs {want}"
    eng.cache.check()


def sampled_generation(make_engine, name, dtype):
    """Temperature sampling with per-sequence streams: the tiny configuration B at temperature 0.7 and seed 1.
    In float32 the tokens are the plain implementation's.  In bfloat16 a draw may fall on the other
    side of a CDF boundary; then the uniform number must lie at that boundary within the
    probabilities' rounding error, and everything before it must agree."""
    V = CONFIGS[name]["vocab_size"]
    T, seed, n_new = 0.7, 1, 12
    prompts = [random_tokens(V, n, 300 + i) for i, n in enumerate(lengths_for(name)[:4])]
    plain = plain_model(name)
    eng = make_engine(name, dtype, 2048, False)
    outs, _ = generate(eng, prompts, GenerationConfig(max_new_tokens=n_new, temperature=T, seed=seed))
    for i, (p, o) in enumerate(zip(prompts, outs)):
        want = P.generate(plain, p, n_new, seed=seed + i, temperature=T)
        if o.tokens == want:
            continue
        assert dtype != "float32", f"request {i}: {o.tokens} vs {want}"
        k = next(j for j, (a, b) in enumerate(zip(o.tokens, want)) if a != b)
        rng = P.PlainPhilox(seed + i)
        for _ in range(k):
            P.uniform_for_multinomial(rng)
        u = P.uniform_for_multinomial(rng)
        row = plain.forward(list(p) + want[:k])[-1] / torch.tensor(T)
        cdf = torch.cumsum(torch.softmax(row, 0), 0)
        lo, hi = sorted((o.tokens[k], want[k]))
        assert all(abs(float(cdf[j]) - u) <= 0.02 for j in range(lo, hi)), \
            f"request {i}, token {k}: engine {o.tokens[k]}, plain {want[k]}, u = {u} is at no boundary between them"
