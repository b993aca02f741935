"""Shared by the tests: the two tiny configurations, model folders made in temporary
directories, traces, and the comparison of logits with their tolerances."""
from __future__ import annotations

import json
import os
import subprocess
import sys
import tempfile

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

from synaptix_amd import Qwen3Config, write_random_model  # noqa: E402
from plain_qwen3 import PlainQwen3  # noqa: E402

# Two configurations that differ in every size and option.
TINY_A = dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
              intermediate_size=176, vocab_size=512, rope_theta=1e4, rms_norm_eps=1e-6, max_position_embeddings=256,
              tie_word_embeddings=True, eos_token_id=None, bos_token_id=None)
TINY_B = dict(num_hidden_layers=3, hidden_size=128, num_attention_heads=8, num_key_value_heads=1, head_dim=32,
              intermediate_size=320, vocab_size=1000, rope_theta=1e6, rms_norm_eps=1e-5, max_position_embeddings=512,
              tie_word_embeddings=False, eos_token_id=None, bos_token_id=None)
# A third one for the GPU tests: sizes that are no power of two, three heads a group, head size 48.
TINY_C = dict(num_hidden_layers=2, hidden_size=120, num_attention_heads=6, num_key_value_heads=2, head_dim=48,
              intermediate_size=200, vocab_size=777, rope_theta=5e5, rms_norm_eps=3e-6, max_position_embeddings=1024,
              tie_word_embeddings=False, eos_token_id=None, bos_token_id=None)
# A middle-sized one: wide enough that the engine takes the kernels which the tiny ones never reach
# (partial sums over slices of K, the deep tiles for wide products, the large GEMM tiles), still seconds on the CPU.
MID_D = dict(num_hidden_layers=2, hidden_size=2048, num_attention_heads=16, num_key_value_heads=4, head_dim=128,
             intermediate_size=2560, vocab_size=33024, rope_theta=1e6, rms_norm_eps=1e-6, max_position_embeddings=2048,
             tie_word_embeddings=True, eos_token_id=None, bos_token_id=None)
# A tiny one for long contexts.  theta is a power of two, so that the rotation's frequencies
# theta^(-2i/16) = 2^(-2i) and with them the angles at any position are exact in 32-bit, whichever
# power routine computes them: at position 6000 a last-bit difference in a frequency would
# otherwise be an angle error of 4e-4, above the 32-bit tolerance of these tests.
LONG_L = dict(TINY_A, rope_theta=65536.0, max_position_embeddings=16384)
# Awkward sizes: a width that is no multiple of 8 (the MFMA products refuse it: plain products), a
# head size with no kernel built ahead of time and no power of two, as many kv heads as heads, an
# intermediate size that cannot be paired, an odd vocabulary.
ODD_E = dict(num_hidden_layers=2, hidden_size=52, num_attention_heads=2, num_key_value_heads=2, head_dim=80,
             intermediate_size=30, vocab_size=101, rope_theta=2e4, rms_norm_eps=2e-5, max_position_embeddings=300,
             tie_word_embeddings=True, eos_token_id=None, bos_token_id=None)
# A head size that only the 32-bit path takes (the bf16 attention kernels take steps of 16).
ODD_F = dict(TINY_A, head_dim=24, num_attention_heads=3, num_key_value_heads=1)
SEEDS = {"A": 0, "B": 1, "C": 2, "D": 3, "L": 4, "E": 5, "F": 6}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": MID_D, "L": LONG_L, "E": ODD_E, "F": ODD_F}

_made = {}
_tmp = None


def model_folder(name: str, sharp: bool = False) -> str:
    """A model folder of the tiny configuration `name` (bf16 weights), made once a process in a
    temporary directory.  sharp: the q/k norm gains are 3 x larger, so that attention is peaked
    and a wrong or lost key changes the logits visibly."""
    global _tmp
    key = (name, sharp)
    if key not in _made:
        if _tmp is None:
            _tmp = tempfile.TemporaryDirectory(prefix="synaptix_amd_models_")
        cfg = Qwen3Config.from_dict(CONFIGS[name])
        folder = os.path.join(_tmp.name, name + ("_sharp" if sharp else ""))
        extra = None
        if sharp:
            g = torch.Generator().manual_seed(99)
            extra = {}
            for l in range(cfg.num_hidden_layers):
                for n in ("q_norm", "k_norm"):
                    extra[f"model.layers.{l}.self_attn.{n}.weight"] = (
                        3.0 + 0.3 * torch.randn(cfg.head_dim, generator=g)).to(torch.bfloat16)
        write_random_model(folder, cfg, SEEDS[name], extra_tensors=extra)
        _made[key] = folder
    return _made[key]


_plain = {}


def plain_model(name: str, sharp: bool = False) -> PlainQwen3:
    key = (name, sharp)
    if key not in _plain:
        _plain[key] = PlainQwen3.from_folder(model_folder(name, sharp))
    return _plain[key]


_plain_logits = {}


def plain_logits(name: str, tokens, sharp: bool = False) -> torch.Tensor:
    key = (name, sharp, tuple(tokens))
    if key not in _plain_logits:
        _plain_logits[key] = plain_model(name, sharp).forward(list(tokens))
    return _plain_logits[key]


def random_tokens(vocab: int, n: int, seed: int) -> list:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def assert_logits_close(got, want, dtype: str, what: str = "", sharp: bool = False) -> None:
    """float32: only the order of sums differs from the plain implementation: 2e-4 of the scale.

    bfloat16: the weights are the same numbers; activations are rounded to 8 bits of mantissa at the
    input of every product, a few times a layer.  What that rounding alone does was measured with
    float32-accumulating torch operations that round at the same places (tests/cpu_kernels.py under
    the engine): for the tiny configurations the error's RMS is 0.3 .. 0.55 % of the logits' RMS and
    its maximum 0.2 .. 0.7 % of the largest logit.  The bounds are 2.5 % for both, a factor of four
    to five.  With `sharp` weights (q/k gains x 3, scores of standard deviation ~9) the same
    measurement gives 2.3 .. 6.9 % RMS and up to 15 % maximum, since a rounding of q or k moves
    whole softmax weights; there the bounds are 20 % and 45 %, which still separates rounding from
    a lost or wrong key (an error of the order of the logits themselves); the exact check of that
    case is the float32 one."""
    got = torch.as_tensor(np.asarray(got), dtype=torch.float32) if not isinstance(got, torch.Tensor) else got.float().cpu()
    want = want.float()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    err = (got - want).abs()
    scale = max(1.0, float(want.abs().max()))
    if dtype == "float32":
        assert float(err.max()) <= 2e-4 * scale, f"{what}: max err {float(err.max()):.3e} at scale {scale:.2f}"
    else:
        rms = max(float(want.pow(2).mean().sqrt()), 0.05)
        b_max, b_rms = (0.45, 0.20) if sharp else (2.5e-2, 2.5e-2)
        assert float(err.max()) <= b_max * scale, f"{what}: max err {float(err.max()):.3e} at scale {scale:.2f}"
        assert float(err.pow(2).mean().sqrt()) <= b_rms * rms, \
            f"{what}: rms err {float(err.pow(2).mean().sqrt()):.3e} vs rms {rms:.3f}"


# ----------------------------------------------------------------------------- traces

def run_trace(folder: str, dtype: str, steps: list, max_tokens: int, out_dir: str, timeout: int = 300) -> dict:
    """Run bin/trace_run over `steps`; returns {step: array [wanted, vocab]}."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens)]
    text = "".join(json.dumps(s) + "\n" for s in steps)
    proc = subprocess.run(cmd, input=text, capture_output=True, text=True, timeout=timeout)
    assert proc.returncode == 0, f"trace_run failed ({proc.returncode}):\n{proc.stderr[-3000:]}"
    done = [l for l in proc.stdout.splitlines() if l.startswith("done ")]
    assert done == [f"done {s['step']}" for s in steps], f"done lines: {done[:5]} ..."
    with open(os.path.join(folder, "config.json")) as f:
        vocab = json.load(f)["vocab_size"]
    out = {}
    for s in steps:
        p = os.path.join(out_dir, f"{s['step']}.f32")
        n_want = sum(len(e.get("want", [])) for e in s["entries"])
        if n_want:
            out[s["step"]] = np.fromfile(p, dtype="<f4").reshape(n_want, vocab)
        else:
            assert not os.path.exists(p)
    return out


def batched_trace(requests: dict, batches: list, decode: int) -> tuple:
    """requests: id -> tokens.  Each batch (a list of ids) starts together: every request's tokens
    but its last `decode` (at least one stays) in the first step, then one token a step; shorter
    requests end earlier.  Everything is wanted.  Returns (steps, where) with where[(id, position)]
    = (step, row)."""
    steps, where, step = [], {}, 0
    for batch in batches:
        head = {r: max(1, len(requests[r]) - decode) for r in batch}
        entries, row = [], 0
        for r in batch:
            n = head[r]
            entries.append({"id": r, "tokens": requests[r][:n], "want": list(range(n))})
            for p in range(n):
                where[(r, p)] = (step, row + p)
            row += n
        fed = dict(head)
        end = [r for r in batch if fed[r] == len(requests[r])]
        steps.append({"step": step, "entries": entries, "end": end})
        step += 1
        live = [r for r in batch if r not in end]
        while live:
            entries = []
            for i, r in enumerate(live):
                entries.append({"id": r, "tokens": [requests[r][fed[r]]], "want": [0]})
                where[(r, fed[r])] = (step, i)
                fed[r] += 1
            end = [r for r in live if fed[r] == len(requests[r])]
            steps.append({"step": step, "entries": entries, "end": end})
            step += 1
            live = [r for r in live if r not in end]
    return steps, where
