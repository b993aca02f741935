"""Command line in the manner of the reference's `synaptix run` and `synaptix bench`
(crates/synaptix-cli/src/bin/synaptix.rs:60-129, commands/run.rs:289-350, commands/bench.rs:9-96):
the same option names and meanings where this engine has the feature.

    python -m synaptix_amd run MODEL [PROMPT] [--prompt-file F | --prompt-ids 1,2,3 | --prompt-ids-file F]
           [--max-tokens 128] [--temperature 1.0] [--seed 0] [--device cuda] [--max-seq N]
           [--compute-dtype bf16|f32] [--no-graph] [--warmup] [--op-times] [--batch N]
    python -m synaptix_amd run --random CONFIG_JSON ...      (no model folder: random weights drawn with --seed)
    python -m synaptix_amd bench MODEL [--n-tokens 128] [--prompt-tokens 32] [--batch-size 1] [--warmup 3] [--dtype bf16]
    python -m synaptix_amd random CONFIG_JSON OUT_DIR [--seed 0] [--dtype bf16|f32]

Not built, so not offered: --quant, --kv-dtype, --storage-dtype, --lm-head-dtype, --embed-dtype, --attn
(quantized weights and caches, and alternative attention back ends).
"""
from __future__ import annotations

import argparse
import json
import sys
import time


def _ids(text: str) -> list:
    return [int(t) for t in text.replace(",", " ").split()]


def cmd_run(a) -> int:
    from .pipeline import Pipeline
    from .sampling import GenerationConfig

    if a.random is not None:
        # no folder: the configuration alone, weights drawn on the device from --seed; the one positional
        # argument left, if any, is the prompt
        if a.prompt:
            print("synaptix_amd run: with --random CONFIG there is no MODEL argument; give the prompt alone", file=sys.stderr)
            return 1
        a.prompt, a.model = a.model or "", None
        pipe = Pipeline.random(a.random, seed=a.seed, device=a.device, dtype=a.compute_dtype, max_seq=a.max_seq)
    elif not a.model:
        print("synaptix_amd run: a MODEL folder or --random CONFIG_JSON is needed", file=sys.stderr)
        return 1
    else:
        pipe = Pipeline.load(a.model, device=a.device, dtype=a.compute_dtype, max_seq=a.max_seq)
    as_text = False
    if a.prompt_ids is not None:
        prompt = _ids(a.prompt_ids)
    elif a.prompt_ids_file is not None:
        prompt = _ids(open(a.prompt_ids_file).read())
    else:
        text = open(a.prompt_file).read() if a.prompt_file else a.prompt
        if not text:
            print("synaptix_amd run: empty prompt", file=sys.stderr)
            return 1
        prompt = pipe.encode(text)
        as_text = True
    cfg = GenerationConfig(max_new_tokens=a.max_tokens, temperature=a.temperature, seed=a.seed, top_k=a.top_k,
                           top_p=a.top_p, min_p=a.min_p, repetition_penalty=a.repetition_penalty,
                           repeat_last_n=a.repeat_last_n, presence_penalty=a.presence_penalty,
                           frequency_penalty=a.frequency_penalty, max_seq=a.max_seq)
    if a.warmup:       # pays compilation and graph capture before the measured run (the reference: NVRTC)
        import dataclasses
        pipe.generate(prompt, dataclasses.replace(cfg, max_new_tokens=4, temperature=0.0), use_graph=not a.no_graph)
    t0 = time.perf_counter()
    if a.batch > 1:     # the prompt a.batch times in one batch; sequence i draws from the stream of seed + i
        outs, st = pipe.generate_batch([prompt] * a.batch, cfg, use_graph=not a.no_graph)
        ms = (time.perf_counter() - t0) * 1e3
        for o in outs:
            print(pipe.decode(o.tokens) if as_text else " ".join(str(t) for t in o.tokens))
        ids = None
    elif a.op_times:    # the reference's per-op profile (model.rs:22-99): every op synchronised and timed, eager steps
        from .kernels import ops
        with ops.op_timing() as times:
            ids, st = pipe.generate(prompt, cfg, use_graph=False)
        print(times.report(), file=sys.stderr)
    else:
        ids, st = pipe.generate(prompt, cfg, use_graph=not a.no_graph)
    if ids is not None:
        ms = (time.perf_counter() - t0) * 1e3
        print(pipe.decode(ids) if as_text else " ".join(str(t) for t in ids))
    # the reference's line: crates/synaptix-cli/src/commands/run.rs:234
    print(f"synaptix_amd run: {st.prompt_tokens} prompt + {st.new_tokens} new tokens in {ms:.0f} ms | "
          f"prefill {st.prefill_ms:.0f} ms | decode {st.decode_ms:.0f} ms "
          f"({st.new_tokens / max(st.decode_ms, 1.0) * 1e3:.2f} tok/s)", file=sys.stderr)
    return 0


def cmd_bench(a) -> int:
    """Warm-ups, then one greedy run; tok/s = (new - 1) / decode time (bench.rs:84-88), per sequence batch."""
    from .pipeline import Pipeline
    from .sampling import GenerationConfig

    pipe = Pipeline.load(a.model, device=a.device, dtype=a.dtype,
                         max_tokens=a.batch_size * ((a.prompt_tokens + a.n_tokens + 127) // 64 * 64))
    V = pipe.engine.vocab
    prompts = [[((i * 7 + 13 + b) % min(200, V - 5)) + 5 for i in range(a.prompt_tokens)] for b in range(a.batch_size)]
    cfg = GenerationConfig(max_new_tokens=a.n_tokens, temperature=0.0, eos_token_ids=(-1,))     # never stops early
    for _ in range(a.warmup):
        pipe.generate_batch(prompts, cfg)
    outs, st = pipe.generate_batch(prompts, cfg)
    new = sum(len(o.tokens) - 1 for o in outs)
    print(json.dumps({"prompt_tokens": st.prompt_tokens, "new_tokens": st.new_tokens, "batch_size": a.batch_size,
                      "prefill_ms": round(st.prefill_ms, 2), "decode_ms": round(st.decode_ms, 2),
                      "decode_tok_s": round(new / max(st.decode_ms, 1e-9) * 1e3, 2),
                      "prefill_tok_s": round(st.prompt_tokens / max(st.prefill_ms, 1e-9) * 1e3, 2)}))
    return 0


def cmd_random(a) -> int:
    import torch
    from .config import resolve_architecture
    from .weights import write_random_model

    d = json.load(open(a.config))
    cfg = resolve_architecture(d).config_cls.from_dict(d)
    write_random_model(a.out, cfg, a.seed, store_dtype=torch.float32 if a.dtype == "f32" else torch.bfloat16)
    print(a.out)
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="synaptix_amd", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    r = sub.add_parser("run", help="generate from one prompt")
    r.add_argument("model", nargs="?", default="")
    r.add_argument("prompt", nargs="?", default="")
    r.add_argument("--random", metavar="CONFIG_JSON", default=None,
                   help="no model folder: this config.json with random weights drawn from --seed")
    r.add_argument("--batch", type=int, default=1, help="generate this many sequences from the prompt in one batch")
    r.add_argument("--prompt-file")
    r.add_argument("--prompt-ids", help="token ids, separated by commas or blanks (no tokenizer needed)")
    r.add_argument("--prompt-ids-file")
    r.add_argument("--max-tokens", type=int, default=128)
    r.add_argument("--temperature", type=float, default=1.0)
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--device", default="cuda")
    r.add_argument("--max-seq", type=int, default=None)
    r.add_argument("--compute-dtype", default="bf16", choices=["bf16", "f32"])
    r.add_argument("--no-graph", action="store_true")
    r.add_argument("--warmup", action="store_true")
    r.add_argument("--op-times", action="store_true",
                   help="time every kernel entry point with the device synchronised around it (eager steps) and print the table")
    r.add_argument("--top-k", type=int, default=0)
    r.add_argument("--top-p", type=float, default=1.0)
    r.add_argument("--min-p", type=float, default=0.0)
    r.add_argument("--repetition-penalty", type=float, default=1.0)
    r.add_argument("--repeat-last-n", type=int, default=0)
    r.add_argument("--presence-penalty", type=float, default=0.0)
    r.add_argument("--frequency-penalty", type=float, default=0.0)
    r.set_defaults(fn=cmd_run)
    b = sub.add_parser("bench", help="warm-ups and one greedy run")
    b.add_argument("model")
    b.add_argument("--n-tokens", type=int, default=128)
    b.add_argument("--prompt-tokens", type=int, default=32)
    b.add_argument("--batch-size", type=int, default=1)
    b.add_argument("--warmup", type=int, default=3)
    b.add_argument("--device", default="cuda")
    b.add_argument("--dtype", default="bf16", choices=["bf16", "f32"])
    b.set_defaults(fn=cmd_bench)
    m = sub.add_parser("random", help="write a model folder with random weights")
    m.add_argument("config")
    m.add_argument("out")
    m.add_argument("--seed", type=int, default=0)
    m.add_argument("--dtype", default="bf16", choices=["bf16", "f32"])
    m.set_defaults(fn=cmd_random)
    a = ap.parse_args(argv)
    try:
        return a.fn(a)
    except (ValueError, RuntimeError, OSError) as e:     # configuration, weights, cache, kernels, files
        print(f"synaptix_amd {a.cmd}: {type(e).__name__}: {e}", file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(main())
