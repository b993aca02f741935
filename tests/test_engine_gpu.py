"""The engine on the GPU against the plain implementation, in 32-bit and in bfloat16: each
request alone and whole; with the last 32 tokens one by one; in batches of unequal lengths one
after another (slots used again); long decoding; the first tokens; generation; the replay
program as a user runs it."""
import os

import numpy as np
import pytest
import torch

import scenarios
from helpers import (model_folder, CONFIGS, plain_logits, random_tokens, assert_logits_close, run_trace,
                     batched_trace)

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module", autouse=True)
def need_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")


_engines = {}


def make_engine(name, dtype, max_tokens, sharp=False, max_slots=None):
    from synaptix_amd import Engine
    return Engine.load(model_folder(name, sharp), dtype=dtype, max_tokens=max_tokens, max_slots=max_slots)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole(name, dtype):
    scenarios.whole(make_engine, name, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_whole_with_peaked_attention(dtype):
    """q/k gains 3 x larger: attention picks single keys, so a wrong key or page shows."""
    scenarios.whole(make_engine, "C", dtype, sharp=True)
    scenarios.unequal_batches(make_engine, "B", dtype, sharp=True)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_last_32_tokens_one_by_one(name, dtype):
    scenarios.last_tokens_one_by_one(make_engine, name, dtype, tail=32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_unequal_batches_one_after_another(name, dtype):
    scenarios.unequal_batches(make_engine, name, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,n", [("A", 250), ("B", 400), ("C", 300)])
def test_long_decoding(name, n, dtype):
    scenarios.long_decoding(make_engine, name, dtype, n)


@pytest.mark.parametrize("dtype", DTYPES)
def test_awkward_sizes(dtype):
    """A width of 52, head size 80, intermediate size 30, vocabulary 101: every kernel either takes
    the size or hands it to its general form; whole, one by one, and in unequal batches."""
    scenarios.whole(make_engine, "E", dtype)
    scenarios.last_tokens_one_by_one(make_engine, "E", dtype, tail=32)
    scenarios.unequal_batches(make_engine, "E", dtype)


@pytest.mark.parametrize("seed", [0, 1])
def test_random_configurations(seed, tmp_path):
    """Configurations drawn at random, every size odd where it may be (head sizes 16 to 256, groups of 1 to 7 heads,
    widths and intermediate sizes that are multiples of 8 and 2 only, any vocabulary, tied or not): several prompts
    of unequal lengths in one step, then single tokens, against the plain implementation in both types."""
    import random
    from synaptix_amd import Qwen3Config, write_random_model, Engine
    from plain_qwen3 import PlainQwen3
    rnd = random.Random(seed)
    for trial in range(4):
        nkv = rnd.choice([1, 2, 3, 5])
        raw = dict(vocab_size=rnd.randint(20, 700), hidden_size=8 * rnd.randint(3, 40), intermediate_size=2 * rnd.randint(5, 150),
                   num_hidden_layers=rnd.randint(1, 3), num_attention_heads=nkv * rnd.choice([1, 2, 3, 4, 7]),
                   num_key_value_heads=nkv, head_dim=rnd.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 256]),
                   max_position_embeddings=512, rope_theta=rnd.choice([1e4, 1e6]), rms_norm_eps=rnd.choice([1e-6, 1e-5]),
                   tie_word_embeddings=rnd.random() < 0.5, eos_token_id=None)
        folder = str(tmp_path / f"m{trial}")
        write_random_model(folder, Qwen3Config(**raw), seed=100 * seed + trial)
        plain = PlainQwen3.from_folder(folder)
        lens = [rnd.randint(1, 150) for _ in range(rnd.randint(1, 5))]
        seqs = [random_tokens(raw["vocab_size"], n + 3, 7 * trial + i) for i, n in enumerate(lens)]
        want = [plain.forward(q) for q in seqs]
        for dtype in DTYPES:
            eng = Engine.load(folder, dtype=dtype, max_tokens=1024)
            slots = [eng.acquire() for _ in seqs]
            lg = eng.step([(sl, q[:n]) for sl, q, n in zip(slots, seqs, lens)], want="all")
            got, off = [], 0
            for n in lens:
                got.append([lg[off:off + n]])
                off += n
            for d in range(3):
                lg = eng.step([(sl, [q[n + d]]) for sl, q, n in zip(slots, seqs, lens)], want="last")
                for i in range(len(seqs)):
                    got[i].append(lg[i:i + 1].clone())
            for i in range(len(seqs)):
                assert_logits_close(torch.cat(got[i]), want[i], dtype, f"seed {seed} trial {trial} {raw} sequence {i}")
            for sl in slots:
                eng.release(sl)
            eng.cache.check()


def test_head_size_24_runs_in_32_bit_and_is_refused_in_bf16():
    scenarios.whole(make_engine, "F", "float32")
    scenarios.last_tokens_one_by_one(make_engine, "F", "float32", tail=8)
    with pytest.raises(ValueError, match="steps of 16"):
        make_engine("F", "bfloat16", 256)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_wide_batch(name, dtype):
    scenarios.wide_batch(make_engine, name, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_context(dtype):
    scenarios.long_context(make_engine, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_context_through_graphs_of_128_and_256_pages(dtype):
    scenarios.long_context_through_graphs(make_engine, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,sharp", [("B", False), ("C", True)])
def test_decode_beside_a_fresh_prompt(name, sharp, dtype):
    scenarios.decode_beside_fresh_prompt(make_engine, name, dtype, sharp)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk", [2, 50, 64])
def test_prompts_in_chunks(chunk, dtype):
    scenarios.chunked_prompts(make_engine, "C", dtype, chunk, sharp=(chunk == 50))


@pytest.mark.parametrize("dtype", DTYPES)
def test_generation_with_a_prompt_in_chunks_of_64(dtype):
    scenarios.generation_with_chunked_prompt(make_engine, "B", dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens(name, dtype):
    scenarios.first_tokens(make_engine, name, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation(name, dtype):
    scenarios.greedy_generation(make_engine, name, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_sampled_generation(dtype):
    scenarios.sampled_generation(make_engine, "B", dtype)


@pytest.mark.parametrize("name", ["A", "B"])
def test_generation_with_every_processor(name):
    scenarios.generation_with_every_processor(make_engine, name)


def test_batch_rows_do_not_depend_on_their_neighbours():
    """The same request alone, and between others in another slot and other pages."""
    for dtype in DTYPES:
        eng = make_engine("B", dtype, 4096)
        V = CONFIGS["B"]["vocab_size"]
        mine = random_tokens(V, 77, 1)
        s = eng.acquire()
        alone = eng.step([(s, mine)], want="all")
        others = [random_tokens(V, n, 2 + n) for n in (130, 5)]
        a, b, c = eng.acquire(), eng.acquire(), eng.acquire()
        lg = eng.step([(a, others[0]), (b, mine), (c, others[1])], want=[[], list(range(77)), []])
        # no padding and no shared reductions: the rows of a request are the same numbers
        assert float((lg - alone).abs().max()) <= (1e-5 if dtype == "float32" else 2e-2)


def test_middle_sized_model_reaches_the_large_kernels():
    """Hidden 2048, head size 128, vocabulary 33024: prompts of hundreds of tokens take the tiled GEMM,
    single tokens the products cut along K and the wide output product on its deep tiles."""
    name, dtype = "D", "bfloat16"
    V = CONFIGS[name]["vocab_size"]
    reqs = [random_tokens(V, n, 700 + n) for n in (300, 130, 65)]
    eng = make_engine(name, dtype, 2048)
    slots = [eng.acquire() for _ in reqs]
    head = [len(r) - 6 for r in reqs]
    got = [[] for _ in reqs]
    lg = eng.step([(s, r[:h]) for s, r, h in zip(slots, reqs, head)], want=[[h - 2, h - 1] for h in head])
    for i in range(3):
        got[i].append(lg[2 * i:2 * i + 2])
    for j in range(6):
        lg = eng.step([(s, [r[h + j]]) for s, r, h in zip(slots, reqs, head)], want="last")
        for i in range(3):
            got[i].append(lg[i:i + 1])
    for i, r in enumerate(reqs):
        want = plain_logits(name, r)[head[i] - 2:]
        assert_logits_close(torch.cat(got[i]), want, dtype, f"middle-sized model, request {i}")
    # and the 32-bit path of the same model on one short request
    e32 = make_engine(name, "float32", 256)
    s = e32.acquire()
    assert_logits_close(e32.step([(s, reqs[2])], want="last"), plain_logits(name, reqs[2])[-1:], "float32", "middle-sized, 32-bit")


# ----------------------------------------------------------------------------- the replay program
@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_run_whole_one_by_one_and_batched(tmp_path, dtype):
    """bin/trace_run as a user starts it: requests whole; with their last 32 tokens one by one;
    and in batches of unequal lengths, one batch after another, with max-tokens so tight that
    the second batch needs the pages of the first."""
    name = "B"
    folder = model_folder(name)
    V = CONFIGS[name]["vocab_size"]
    reqs = {f"q{i}": random_tokens(V, n, 400 + i) for i, n in enumerate([40, 97, 33, 150, 64])}
    # whole
    steps = [{"step": i, "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))}], "end": [r]}
             for i, (r, t) in enumerate(reqs.items())]
    out = run_trace(folder, dtype, steps, 192, str(tmp_path / "whole"))
    for i, (r, t) in enumerate(reqs.items()):
        assert_logits_close(out[i], plain_logits(name, t), dtype, f"trace whole {r}")
    # last 32 one by one, each request alone
    steps, where = batched_trace(reqs, [[r] for r in reqs], decode=32)
    out = run_trace(folder, dtype, steps, 192, str(tmp_path / "tail"))
    for r, t in reqs.items():
        got = np.stack([out[where[(r, p)][0]][where[(r, p)][1]] for p in range(len(t))])
        assert_logits_close(got, plain_logits(name, t), dtype, f"trace last 32 {r}")
    # unequal batches; q3 (150 tokens, 3 pages) + q0 + q1 (1 + 2 pages) fill 6 pages exactly
    batches = [["q3", "q0", "q1"], ["q2", "q4", "q1"], ["q4", "q3"]]
    steps, where = batched_trace(reqs, batches, decode=32)
    out = run_trace(folder, dtype, steps, 64 * 6, str(tmp_path / "batched"))
    seen = set()
    for (r, p), (st, row) in where.items():
        seen.add(r)
    for r in seen:
        t = reqs[r]
        got = np.stack([out[where[(r, p)][0]][where[(r, p)][1]] for p in range(len(t))])
        assert_logits_close(got, plain_logits(name, t), dtype, f"trace batched {r}")


def test_trace_run_steps_without_wants_write_no_file(tmp_path):
    folder = model_folder("A")
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": [1, 2, 3], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": [4], "want": [0]}], "end": ["x"]},
             {"step": 2, "entries": [], "end": []}]
    out = run_trace(folder, "float32", steps, 64, str(tmp_path / "o"))
    assert sorted(out) == [1]
    assert_logits_close(out[1], plain_logits("A", [1, 2, 3, 4])[3:], "float32", "after a silent step")
    assert not os.path.exists(tmp_path / "o" / "0.f32")


def test_trace_run_names_the_step_it_cannot_run(tmp_path):
    """A step that does not fit the cache, or brings a token outside the vocabulary: the steps before it are
    done, then one line names the step and the reason, exit code 1."""
    import json
    import subprocess
    import sys
    from helpers import ROOT
    folder = model_folder("A")
    for bad, reason in (([1] * 65, "CacheFull"), ([1, 10 ** 6], "vocabulary")):
        steps = [{"step": 0, "entries": [{"id": "x", "tokens": [1, 2, 3], "want": [2]}], "end": ["x"]},
                 {"step": 1, "entries": [{"id": "y", "tokens": bad, "want": [0]}], "end": []}]
        cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
               "--out", str(tmp_path / "o"), "--max-tokens", "64"]
        proc = subprocess.run(cmd, input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True,
                              timeout=300)
        assert proc.returncode == 1
        assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == ["done 0"]
        last = [l for l in proc.stderr.splitlines() if l.startswith("trace_run:")]
        assert len(last) == 1 and "step 1" in last[0] and reason in last[0], proc.stderr[-500:]
        assert "Traceback" not in proc.stderr


# ----------------------------------------------------------------------------- captured decode steps
@pytest.mark.parametrize("dtype", DTYPES)
def test_graph_replays_equal_eager_steps(dtype):
    """Every replay of the captured decode step is checked against the eager step, with eager work
    and synchronisations of the program's own between the replays; rows of padding change nothing."""
    name = "B"
    V = CONFIGS[name]["vocab_size"]
    prompts = [random_tokens(V, n, 500 + n) for n in (20, 70, 3)]
    eager, graph = make_engine(name, dtype, 2048), make_engine(name, dtype, 2048)
    es = [eager.acquire() for _ in prompts]
    gs = [graph.acquire() for _ in prompts]
    tok = eager.sample(eager.step(list(zip(es, prompts)), want="last")).cpu().tolist()
    tok_g = graph.sample(graph.step(list(zip(gs, prompts)), want="last")).cpu().tolist()
    assert tok == tok_g
    runner = graph.decode_runner(3, 200)            # 4 rows: one of padding
    assert runner.rows == 4
    for step in range(70):                          # crosses a page edge for two of the sequences
        want = eager.step([(s, [t]) for s, t in zip(es, tok)], want="last")
        got_tokens, got = runner.step(gs, tok)
        torch.cuda.synchronize()
        assert float((got - want).abs().max()) <= (1e-5 if dtype == "float32" else 2e-2), f"replay {step}"
        tok = eager.sample(want).cpu().tolist()
        if dtype == "float32":
            assert got_tokens == tok, f"replay {step}"
        if step % 7 == 0:                           # eager work of another engine between replays
            other = eager.acquire()
            eager.step([(other, prompts[1])], want="last")
            eager.release(other)
    # a smaller live set in the same graph: the finished sequence's row becomes padding
    want = eager.step([(es[0], [tok[0]]), (es[2], [tok[2]])], want="last")
    _, got = runner.step([gs[0], gs[2]], [tok[0], tok[2]])
    assert float((got - want).abs().max()) <= (1e-5 if dtype == "float32" else 2e-2)
    for e in (eager, graph):
        e.cache.check()


def test_single_tokens_beside_prompts_take_the_kernel_for_single_tokens():
    """A step of two sequences that go on by one token over some hundred cached tokens and one prompt that starts:
    the prompts' attention kernel runs once a layer and leaves the single tokens to the kernel for single tokens,
    which runs once a layer as well; the logits are those of the plain implementation (with peaked attention, so
    that a key out of reach or a row handed to the wrong sequence shows)."""
    from synaptix_amd.kernels import ops
    name, sharp = "C", True
    V, L = CONFIGS[name]["vocab_size"], CONFIGS[name]["num_hidden_layers"]
    olds = [random_tokens(V, 300 + 1, 61), random_tokens(V, 130 + 1, 62)]
    fresh = random_tokens(V, 90, 63)
    eng = make_engine(name, "bfloat16", 2048, sharp)
    a, b, c = eng.acquire(), eng.acquire(), eng.acquire()
    eng.step([(a, olds[0][:300]), (b, olds[1][:130])], want=None)
    with ops.op_timing() as times:
        lg = eng.step([(a, olds[0][300:]), (c, fresh), (b, olds[1][130:])], want="all")
    assert times["syn_attention_prefill_bf16"][1] == L and times["syn_attention_decode_bf16"][1] == L
    assert_logits_close(lg[:1], plain_logits(name, olds[0], sharp)[300:], "bfloat16", "the first single token", sharp)
    assert_logits_close(lg[1:91], plain_logits(name, fresh, sharp), "bfloat16", "the prompt between them", sharp)
    assert_logits_close(lg[91:], plain_logits(name, olds[1], sharp)[130:], "bfloat16", "the second single token", sharp)
    for s_ in (a, b, c):
        eng.release(s_)
    eng.cache.check()


@pytest.mark.parametrize("name", ["B", "C"])
def test_captured_prompt_steps_equal_eager_ones(name):
    """Short prompt steps are replayed from graphs with padding rows behind their own: every replay against
    the eager step of an engine that has the graphs switched off and against the plain implementation;
    several steps through one graph with eager work between them, sequences that go on with a second piece
    of their prompt, a wanted place that is not the last, a slot that is used again, and decode steps after."""
    dtype = "bfloat16"
    V = CONFIGS[name]["vocab_size"]
    eager, graph = make_engine(name, dtype, 4096), make_engine(name, dtype, 4096)
    eager.prompt_graphs = False

    def both(entries_of, want):
        got = graph.step(entries_of(graph), want=want)
        ref = eager.step(entries_of(eager), want=want)
        torch.cuda.synchronize()
        assert got.shape == ref.shape
        err = float((got - ref).abs().max())
        assert err <= 3e-2 * max(1.0, float(ref.abs().max())), f"replayed prompt step differs from the eager one by {err}"
        return got

    slots = {id(e): [] for e in (eager, graph)}

    def acquire(n):
        for e in (eager, graph):
            slots[id(e)] += [e.acquire() for _ in range(n)]

    acquire(3)
    prompts = [random_tokens(V, n, 900 + n) for n in (5, 33, 20)]
    got = both(lambda e: list(zip(slots[id(e)][:3], prompts)), "last")              # 58 tokens: the graph of 64 rows, 4 + 1 sequences
    assert any(k[0] == "prompt" and k[1] == 64 and k[2] == 5 for k in graph._runners if isinstance(k[0], str))
    for i, p in enumerate(prompts):
        assert_logits_close(got[i:i + 1], plain_logits(name, p)[-1:], dtype, f"captured prompt step, sequence {i}")
    # the same graph again with other lengths, and a wanted place in the middle of the first sequence
    acquire(2)
    more = [random_tokens(V, n, 950 + n) for n in (40, 9)]
    got = both(lambda e: list(zip(slots[id(e)][3:5], more)), [[17], [8]])
    assert_logits_close(got[0:1], plain_logits(name, more[0])[17:18], dtype, "a wanted place that is not the last")
    # second pieces of two prompts (tokens cached before), beside a fresh sequence of two tokens (one of a single
    # token would send the step to the kernels launched one by one, where single tokens have a kernel of their own)
    acquire(1)
    tails = [random_tokens(V, n, 970 + n) for n in (30, 12)]
    runners = len(graph._runners)
    got = both(lambda e: [(slots[id(e)][0], tails[0]), (slots[id(e)][3], tails[1]), (slots[id(e)][5], [7, 9])], "last")
    assert len(graph._runners) == runners                      # the graph of 64 rows again
    assert_logits_close(got[0:1], plain_logits(name, prompts[0] + tails[0])[-1:], dtype, "second piece of a prompt")
    assert_logits_close(got[1:2], plain_logits(name, more[0] + tails[1])[-1:], dtype, "second piece of a prompt")
    # a slot that is given back and used again; exactly as many tokens as the graph has rows (no padding rows)
    for e in (eager, graph):
        e.release(slots[id(e)][1])
        slots[id(e)][1] = e.acquire()
    full = random_tokens(V, 16, 990)
    got = both(lambda e: [(slots[id(e)][1], full)], "last")
    assert_logits_close(got, plain_logits(name, full)[-1:], dtype, "a step without padding rows")
    # decode steps after the replayed prompts read what they wrote
    got = both(lambda e: [(slots[id(e)][0], [3]), (slots[id(e)][1], [4])], "last")
    assert_logits_close(got[1:2], plain_logits(name, full + [4])[-1:], dtype, "decode after a captured prompt step")
    for e in (eager, graph):
        e.cache.check()
    assert not any(isinstance(k[0], str) for k in eager._runners)


def test_a_captured_step_keeps_its_own_scratch_memory():
    """A graph holds the addresses of the scratch memory it was captured with.  Larger steps
    afterwards (eager ones and larger captured ones) need more of it; the small runner's must stay
    where it is, and its replays must still give the eager results."""
    name, dtype = "C", "bfloat16"
    V = CONFIGS[name]["vocab_size"]
    eng = make_engine(name, dtype, 64 * 100)
    eager = make_engine(name, dtype, 1024)
    prompt = random_tokens(V, 300, 77)
    s, e = eng.acquire(), eager.acquire()
    tok = eng.sample(eng.step([(s, prompt)], want="last")).cpu().tolist()
    eager.step([(e, prompt)], want="last")
    small = eng.decode_runner(1, 1024)              # 16 pages wide: the keys are cut into 4 splits, merged from scratch memory
    tok2, _ = small.step([s], tok)
    want = eager.step([(e, tok)], want="last")
    before = {k: t.data_ptr() for k, t in small.scratch.tensors.items()}
    assert before and small.scratch.frozen
    # larger steps: 40 sequences decoding eagerly, then through a graph of 64 rows
    many = [eng.acquire() for _ in range(40)]
    eng.step([(m, random_tokens(V, 70, 80 + i)) for i, m in enumerate(many)], want=None)
    eng.step([(m, [1]) for m in many], want="last")
    big = eng.decode_runner(40, 1024)
    big.step(many, [2] * 40)
    held = [torch.empty(1 << 20, device="cuda") for _ in range(8)]     # whoever allocates next gets freed blocks
    for h in held:
        h.fill_(float("nan"))
    assert {k: t.data_ptr() for k, t in small.scratch.tensors.items()} == before
    assert all(small.scratch.tensors[k] is not big.scratch.tensors.get(k) for k in before)
    assert all(small.scratch.tensors[k] is not eng._scratch.tensors.get(k) for k in before)
    _, got = small.step([s], tok2)
    want = eager.step([(e, tok2)], want="last")
    torch.cuda.synchronize()
    assert float((got - want).abs().max()) <= 2e-2
    eng.cache.check()


def test_generation_with_and_without_graph_agree():
    from synaptix_amd.engine.generate import generate, GenerationConfig
    V = CONFIGS["A"]["vocab_size"]
    prompts = [random_tokens(V, n, 600 + n) for n in (5, 40, 64, 9, 2)]
    eng = make_engine("A", "float32", 4096)
    cfgs = [GenerationConfig(max_new_tokens=n, temperature=t, seed=i) for i, (n, t) in
            enumerate([(30, 0.0), (12, 0.8), (70, 0.0), (3, 1.0), (25, 0.0)])]
    a, sa = generate(eng, prompts, cfgs, use_graph=True)
    b, sb = generate(eng, prompts, cfgs, use_graph=False)
    assert [o.tokens for o in a] == [o.tokens for o in b]
    assert [len(o.tokens) for o in a] == [30, 12, 70, 3, 25]
    eng.cache.check()
