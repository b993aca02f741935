#!/usr/bin/env python3
"""Throughput of the engine at a Qwen3 shape with random bf16 weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--shape 8b|4b|32b] [--batch 8] [--layers L]

--shape 8b (the default) and 32b: a step is one decode step of `batch` sequences, each after a
2,048-token prompt of uniform ids, run through the same captured graph and host loop that
generation uses.  One JSON line: decoded tokens a second at the batch, the prefill of one
2,048-token prompt (tokens a second and the fraction of the bf16 MFMA peak), the decode step
against the HBM roofline (every weight it uses once plus the cache of the live requests, over its
time), and decode at batch 1 and 64 (32b: 1 and 32).

--shape 4b (tied embeddings): 16 prompts with seeded lengths uniform in [64, 4096] and 128 greedy
tokens each, through the generation loop itself (engine.generate.generate: its planning, its one
prefill step for all prompts, its captured decode steps and its sampling); a step is one of its
decode steps.  The whole run is done once untimed (it captures the graphs) and once timed.

The default run (8b, without --no-points) measures the other workloads as well and puts them under
`points`: the same 8 sequences through the generation loop (decode_b8_through_generate: the loop's
own clock over its last `steps` decode steps, to stand beside `value`), the 4b workload
(decode_4b_unequal16, its fraction of the HBM roofline and its prompts' rate) and the 32b shape at
8 sequences (decode_32b_b8), each with the sizes it ran at as a text.

Method after the reference's own harnesses (crates/synaptix-models/llm/qwen3/examples/format_perf.rs:41-122,
crates/synaptix-cli/src/commands/bench.rs:35-96): synthetic ids, warm-up first, device synchronised
at both ends of the timed region only.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X, published
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}

_COMMON = dict(num_key_value_heads=8, head_dim=128, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
               max_position_embeddings=8192, eos_token_id=None, bos_token_id=None)
SHAPES = {
    "8b": dict(_COMMON, num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, intermediate_size=12288,
               tie_word_embeddings=False),
    "4b": dict(_COMMON, num_hidden_layers=36, hidden_size=2560, num_attention_heads=32, intermediate_size=9728,
               tie_word_embeddings=True),
    "32b": dict(_COMMON, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, intermediate_size=25600,
                tie_word_embeddings=False),
}
POINTS = {"8b": (1, 64), "32b": (1, 32)}       # the batch sizes beside the main one
QWEN3_8B = SHAPES["8b"]
PROMPT = 2048


def layer_matrix_params(cfg) -> int:
    H, I, nh, nkv, hd = (cfg.hidden_size, cfg.intermediate_size, cfg.num_attention_heads, cfg.num_key_value_heads,
                         cfg.head_dim)
    return H * (nh + 2 * nkv) * hd + nh * hd * H + 3 * H * I


def decode_weight_bytes(cfg) -> int:
    """Every weight a decode step reads, once: the layers' matrices and gains, the final gain and
    the output matrix (the embedding table itself is touched in a few rows only)."""
    L, H, V, hd = cfg.num_hidden_layers, cfg.hidden_size, cfg.vocab_size, cfg.head_dim
    return 2 * (L * (layer_matrix_params(cfg) + 2 * H + 2 * hd) + H + V * H)


def prefill_flops(cfg, lengths) -> int:
    """Matrix products of every token, causal attention of every prompt, the output row of each prompt."""
    L, H, V, hd, nh = cfg.num_hidden_layers, cfg.hidden_size, cfg.vocab_size, cfg.head_dim, cfg.num_attention_heads
    total = 0
    for n in lengths:
        total += 2 * n * L * layer_matrix_params(cfg) + L * 4 * hd * nh * n * (n + 1) // 2 + 2 * V * H
    return total


def unequal_prompts_through_generate(args, shape, emit=True):
    """16 prompts of seeded lengths uniform in [64, 4096], 128 greedy tokens each, through the
    generation loop; its own clocks (GenerationStats) give the numbers.  emit: print the line and return the
    exit code; else return the line."""
    import torch
    from synaptix_amd import Qwen3Config, Engine
    from synaptix_amd.engine.generate import generate, GenerationConfig

    n_prompts, lo, hi = 16, 64, 4096
    new_tokens = args.steps + 1                    # the first token of each sequence comes from the prompts' step
    if new_tokens < 2 or hi + new_tokens > 8192:
        print(f"bench.py: --steps {args.steps} does not fit the context of 8192 beside a prompt of {hi} tokens")
        return 2
    cfg = Qwen3Config.from_dict({**shape, "num_hidden_layers": args.layers})
    g = torch.Generator().manual_seed(0)
    lens = torch.randint(lo, hi + 1, (n_prompts,), generator=g).tolist()
    prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() for n in lens]
    need = sum((n + new_tokens + 63) // 64 * 64 for n in lens)
    eng = Engine.from_config(cfg, seed=0, dtype="bfloat16", max_tokens=need + 64, max_seq=8192)
    gen = GenerationConfig(max_new_tokens=new_tokens, temperature=0.0, eos_token_ids=(-1,))
    for _ in range(max(1, min(args.warmup, 2))):   # whole runs: they build the captured steps that the timed run replays
        generate(eng, prompts, gen, use_graph=not args.no_graph)
    torch.cuda.synchronize()
    outs, st = generate(eng, prompts, gen, use_graph=not args.no_graph)
    torch.cuda.synchronize()
    assert st.batches == 1 and st.decode_steps == args.steps and all(len(o.tokens) == new_tokens for o in outs)
    step_s = st.decode_ms / 1e3 / st.decode_steps
    rate = n_prompts * st.decode_steps / (st.decode_ms / 1e3)
    mean_ctx = sum(lens) / n_prompts + 1 + (st.decode_steps - 1) / 2
    step_bytes = decode_weight_bytes(cfg) + n_prompts * mean_ctx * eng.cache.bytes_per_token()
    achieved = step_bytes / step_s / 1e9
    pre_s = st.prefill_ms / 1e3
    steps_sorted = sorted(st.step_ms)
    line = {
        "metric": "decode tok/s of 16 unequal prompts (64..4096 tokens) through the generation loop, Qwen3-4B shape bf16",
        "value": round(rate, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic: seeded uniform token ids and prompt lengths, random-init weights N(0, 0.02)",
        "config": {"model": "Qwen3-4B shape", "layers": cfg.num_hidden_layers, "model_layers": shape["num_hidden_layers"],
                   "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "global_batch": n_prompts, "seq_len": round(sum(lens) / n_prompts), "min_prompt": min(lens),
                   "max_prompt": max(lens), "context": 8192, "new_tokens": new_tokens, "tie_word_embeddings": True,
                   "rope_theta": 1e6, "rms_norm_eps": 1e-6, "parallelism": "single GPU", "graph": not args.no_graph},
        "prefill": {"value": round(sum(lens) / pre_s, 1), "tokens": sum(lens), "ms": round(pre_s * 1e3, 3),
                    "frac": round(prefill_flops(cfg, lens) / pre_s / MFMA_PEAK["bf16"], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": {"step_ms_median": round(steps_sorted[len(steps_sorted) // 2], 4),
                   "step_ms_max": round(steps_sorted[-1], 4),
                   "end_to_end_tok_s": round(n_prompts * new_tokens / ((st.prefill_ms + st.decode_ms) / 1e3), 1)},
    }
    if not emit:
        del eng
        return line
    print(json.dumps(line))
    return 0


def sizes_text(cfg, layers_run=None) -> str:
    """The sizes a point was measured at, as one text (a record keeps no nested values)."""
    L = cfg.num_hidden_layers if layers_run is None else layers_run
    return (f"{L} of {cfg.num_hidden_layers} layers, hidden {cfg.hidden_size}, {cfg.num_attention_heads} heads / "
            f"{cfg.num_key_value_heads} kv heads of {cfg.head_dim}, intermediate {cfg.intermediate_size}, vocab {cfg.vocab_size}, "
            f"tie {cfg.tie_word_embeddings}")


def through_generate(eng, cfg, batch, prompt_len, warmup, steps, weight_bytes, use_graph=True):
    """`batch` prompts of prompt_len tokens through engine.generate.generate; the loop's own clock over its last
    `steps` decode steps (the first `warmup` are left out: the first run also captures the graph)."""
    import torch
    from synaptix_amd.engine.generate import generate, GenerationConfig
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, cfg.vocab_size, (prompt_len,), generator=g).tolist() for _ in range(batch)]
    gen = GenerationConfig(max_new_tokens=warmup + steps + 1, temperature=0.0, eos_token_ids=(-1,))
    outs, st = generate(eng, prompts, gen, use_graph=use_graph, max_batch=batch)
    torch.cuda.synchronize()
    assert st.batches == 1 and st.decode_steps == warmup + steps
    tail = st.step_ms[-steps:]
    step_s = sum(tail) / 1e3 / steps
    mean_ctx = prompt_len + 1 + warmup + (steps - 1) / 2
    step_bytes = weight_bytes + batch * mean_ctx * eng.cache.bytes_per_token()
    return batch / step_s, step_s, step_bytes


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed decode steps (default 128; 127 for --shape 4b: 128 tokens each)")
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES), help="which Qwen3 shape (default: 8b)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None,
                    help="fewer layers than the model has (same layer sizes); both numbers are reported")
    ap.add_argument("--prompt", type=int, default=PROMPT,
                    help="tokens of every prompt (the contract's run has 2,048; the cache holds 8,192 a sequence)")
    ap.add_argument("--context", type=int, default=8192,
                    help="the longest sequence (positions and cache a sequence; the contract's run has 8,192)")
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64")
    ap.add_argument("--no-graph", action="store_true", help="launch every kernel of a decode step from the host")
    args = ap.parse_args()
    shape = SHAPES[args.shape]
    if args.steps is None:
        args.steps = 127 if args.shape == "4b" else 128
    if args.layers is None:
        args.layers = shape["num_hidden_layers"]
    if args.shape == "4b":
        if args.gpus != 1:
            print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
            return 2
        return unequal_prompts_through_generate(args, shape)
    prompt_len = args.prompt
    if args.context < 64:
        print(f"bench.py: --context {args.context} is too short")
        return 2
    if prompt_len < 1 or prompt_len + args.warmup + args.steps + 8 > args.context:
        print(f"bench.py: --prompt {prompt_len} plus {args.warmup} + {args.steps} + 8 new tokens exceed the context of {args.context}")
        return 2
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    from synaptix_amd import Qwen3Config, Engine
    from synaptix_amd.kernels import ops

    torch.manual_seed(0)
    cfg = Qwen3Config.from_dict({**shape, "num_hidden_layers": args.layers, "max_position_embeddings": args.context})
    batches = [args.batch] if args.no_points else sorted({args.batch, *POINTS[args.shape]})
    new_tokens = args.warmup + args.steps + 8
    per_seq = (prompt_len + new_tokens + 63) // 64 * 64
    eng = Engine.from_config(cfg, seed=0, dtype="bfloat16", max_tokens=max(batches) * per_seq + 64, max_seq=args.context)
    g = torch.Generator().manual_seed(0)

    def prompt():
        return torch.randint(0, cfg.vocab_size, (prompt_len,), generator=g).tolist()

    L, H, I, V = cfg.num_hidden_layers, cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    nh, nkv, hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    weight_bytes = decode_weight_bytes(cfg)
    kv_bytes_per_token = eng.cache.bytes_per_token()

    # ---- prefill of one 2,048-token prompt
    times = []
    for i in range(8):       # (the clocks take some tens of milliseconds of work to settle)
        s = eng.acquire()
        toks = prompt()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.step([(s, toks)], want="last")
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        eng.release(s)
    pre_s = statistics.median(times[3:])
    pre_flops = prefill_flops(cfg, [prompt_len])
    prefill = {"value": round(prompt_len / pre_s, 1), "tokens": prompt_len, "ms": round(pre_s * 1e3, 3),
               "frac": round(pre_flops / pre_s / MFMA_PEAK["bf16"], 4)}

    # ---- decode
    def decode(batch: int, warmup: int, steps: int):
        slots = [eng.acquire() for _ in range(batch)]
        group = max(1, min(8, 65536 // prompt_len))         # prompts go in steps of up to 8 sequences and 65,536 tokens
        for lo in range(0, batch, group):
            part = slots[lo:lo + group]
            lg = eng.step([(s, prompt()) for s in part], want="last")
            first = eng.sample(lg).cpu().tolist()
            if lo == 0:
                tokens = []
            tokens += first
        longest = prompt_len + warmup + steps + 8
        if not args.no_graph:
            # the captured step is built before anything is timed (with a sequence of its own, one
            # token long; the other rows are padding), so that also a run without warm-up times steps only
            spare = eng.acquire()
            eng.step([(spare, [0])], want=None)
            eng.decode_runner(batch, longest).step([spare], [0])
            eng.release(spare)

        def one_step(tokens):
            if args.no_graph:
                lg = eng.step([(s, [t]) for s, t in zip(slots, tokens)], want="last")
                return eng.sample(lg).cpu().tolist()
            return eng.decode_runner(batch, longest).step(slots, tokens)[0]

        for _ in range(warmup):
            tokens = one_step(tokens)
        torch.cuda.synchronize()
        len0 = sum(eng.length(s) for s in slots)
        t0 = time.perf_counter()
        for _ in range(steps):
            tokens = one_step(tokens)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        mean_ctx = len0 / batch + (steps - 1) / 2 + 1       # tokens a sequence holds when a step reads it
        for s in slots:
            eng.release(s)
        step_bytes = weight_bytes + batch * mean_ctx * kv_bytes_per_token
        return batch * steps / dt, dt / steps, step_bytes

    points = {}
    main_rate = main_step = main_bytes = None
    for b in batches:
        k = args.steps if b == args.batch else max(16, min(args.steps, 64))
        w = args.warmup if b == args.batch else max(4, min(args.warmup, 8))
        rate, step_s, step_bytes = decode(b, w, k)
        if b == args.batch:
            main_rate, main_step, main_bytes = rate, step_s, step_bytes
        if b in POINTS[args.shape]:
            points[f"decode_b{b}"] = round(rate, 1)
            points[f"decode_b{b}_hbm_frac"] = round(step_bytes / step_s / 1e9 / HBM_PEAK_GBS, 4)

    if not args.no_points:
        # the same sequences through the generation loop: its planning, its bucket of rows, its sampling
        rate, step_s, step_bytes = through_generate(eng, cfg, args.batch, prompt_len, args.warmup, args.steps, weight_bytes,
                                                    use_graph=not args.no_graph)
        points[f"decode_b{args.batch}_through_generate"] = round(rate, 1)
        points[f"decode_b{args.batch}_through_generate_ms_per_step"] = round(step_s * 1e3, 4)

    achieved = main_bytes / main_step / 1e9
    # what this machine gives to kernels that only read, or only multiply: measured, beside the vendor's peaks
    read_gbs, mfma_tflops = ops.measure_ceilings(eng.device)
    measured = {"hbm_read_GBs": round(read_gbs, 1), "mfma_bf16_TFLOPs": round(mfma_tflops, 1),
                "decode_frac_of_read": round(achieved / read_gbs, 4),
                "prefill_frac_of_mfma": round(pre_flops / pre_s / (mfma_tflops * 1e12), 4)}
    line = {
        "metric": f"decode tok/s at batch {args.batch} (+ batch {'/'.join(str(b) for b in POINTS[args.shape])} in points) "
                  f"and prefill tok/s at {prompt_len} tokens, Qwen3-{args.shape.upper()} shape bf16",
        "value": round(main_rate, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(main_step * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic: seeded uniform token ids, random-init weights N(0, 0.02)",
        "config": {"model": f"Qwen3-{args.shape.upper()} shape", "layers": L, "model_layers": shape["num_hidden_layers"],
                   "hidden": H, "heads": nh, "kv_heads": nkv, "head_dim": hd, "intermediate": I, "vocab": V,
                   "global_batch": args.batch, "seq_len": prompt_len, "context": args.context, "new_tokens": args.steps,
                   "tie_word_embeddings": cfg.tie_word_embeddings, "rope_theta": 1e6, "rms_norm_eps": 1e-6,
                   "parallelism": "single GPU", "graph": not args.no_graph},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
        "measured": measured,
    }
    if not args.no_points and args.shape == "8b" and args.layers == shape["num_hidden_layers"]:
        # the other workloads, each on an engine of its own after this one has gone
        import gc
        del eng
        gc.collect()
        torch.cuda.empty_cache()
        sub = argparse.Namespace(**vars(args))
        sub.steps, sub.warmup, sub.layers = min(args.steps, 127), 1, SHAPES["4b"]["num_hidden_layers"]
        four = unequal_prompts_through_generate(sub, SHAPES["4b"], emit=False)
        points["decode_4b_unequal16"] = four["value"]
        points["decode_4b_unequal16_hbm_frac"] = four["roofline"]["frac"]
        points["prefill_4b_unequal16"] = four["prefill"]["value"]
        points["prefill_4b_unequal16_frac"] = four["prefill"]["frac"]
        points["config_4b_unequal16"] = (sizes_text(Qwen3Config.from_dict(SHAPES["4b"])) +
                                         f", 16 prompts of {four['config']['min_prompt']} to {four['config']['max_prompt']} tokens "
                                         f"({four['prefill']['tokens']} in all), {four['config']['new_tokens']} new tokens each, "
                                         "through engine.generate.generate")
        gc.collect()
        torch.cuda.empty_cache()
        big = Qwen3Config.from_dict(SHAPES["32b"])
        k, w = min(args.steps, 32), min(args.warmup, 4)
        per = (prompt_len + k + w + 8 + 63) // 64 * 64
        eng = Engine.from_config(big, seed=0, dtype="bfloat16", max_tokens=8 * per + 64, max_seq=8192)
        rate, step_s, step_bytes = through_generate(eng, big, 8, prompt_len, w, k, decode_weight_bytes(big))
        points["decode_32b_b8"] = round(rate, 1)
        points["decode_32b_b8_hbm_frac"] = round(step_bytes / step_s / 1e9 / HBM_PEAK_GBS, 4)
        points["config_32b_b8"] = sizes_text(big) + f", 8 prompts of {prompt_len} tokens, {w} + {k} decode steps, through engine.generate.generate"
        del eng
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
