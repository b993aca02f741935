"""Greedy generation through the entry points a user has: the Python pipeline and the command line."""
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_qwen3 as P
from helpers import ROOT, model_folder, plain_model, random_tokens, CONFIGS
from scenarios import check_greedy_path

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def need_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_pipeline_generate(dtype):
    import synaptix_amd
    from synaptix_amd import GenerationConfig
    name = "B"
    plain = plain_model(name)
    prompt = random_tokens(CONFIGS[name]["vocab_size"], 21, 9)
    want = P.generate(plain, prompt, 10)
    pipe = synaptix_amd.load(model_folder(name), device="cuda", dtype=dtype, max_seq=256)
    ids, stats = pipe.generate(prompt, GenerationConfig(max_new_tokens=10))
    assert stats.prompt_tokens == 21 and stats.new_tokens == 10
    if dtype == "f32":
        assert ids == want
    else:
        check_greedy_path(plain, prompt, ids, want)
    # the stop token: make the third token of the plain path the stop token
    ids, _ = pipe.generate(prompt, GenerationConfig(max_new_tokens=10, eos_token_id=want[2]))
    if dtype == "f32":
        assert ids == want[:3]
    seen = []
    pipe.generate_streaming(prompt, GenerationConfig(max_new_tokens=4), lambda t: seen.append(t) or True)
    assert len(seen) == 4
    outs, st = pipe.generate_batch([prompt, prompt[:5]], GenerationConfig(max_new_tokens=6))
    assert [len(o.tokens) for o in outs] == [6, 6] and st.batches == 1
    with pytest.raises(FileNotFoundError, match="tokenizer"):
        pipe.encode("text")


def test_command_line_run_and_bench():
    # an untied model with peaked attention: the greedy path depends on far keys, not on the last token alone
    name = "B"
    folder = model_folder(name, sharp=True)
    plain = plain_model(name, sharp=True)
    prompt = random_tokens(CONFIGS[name]["vocab_size"], 12, 10)
    want = P.generate(plain, prompt, 7)
    cmd = [sys.executable, "-m", "synaptix_amd", "run", folder, "--prompt-ids", ",".join(map(str, prompt)),
           "--max-tokens", "7", "--temperature", "0", "--compute-dtype", "f32", "--warmup"]
    proc = subprocess.run(cmd, capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.split()] == want
    assert "12 prompt + 7 new tokens" in proc.stderr and "tok/s" in proc.stderr
    # every sampling option of the command line, in 32-bit: the plain implementation's tokens for the same seed
    want = P.generate(plain, prompt, 9, seed=4, temperature=0.8, k=15, p=0.9, mp=0.01, repetition=1.2, last_n=8,
                      presence=0.1, frequency=0.05)
    cmd = [sys.executable, "-m", "synaptix_amd", "run", folder, "--prompt-ids", ",".join(map(str, prompt)),
           "--max-tokens", "9", "--temperature", "0.8", "--top-k", "15", "--top-p", "0.9", "--min-p", "0.01",
           "--repetition-penalty", "1.2", "--repeat-last-n", "8", "--presence-penalty", "0.1",
           "--frequency-penalty", "0.05", "--seed", "4", "--compute-dtype", "f32"]
    proc = subprocess.run(cmd, capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.split()] == want
    # no folder: a config.json alone with weights drawn from --seed, and the prompt several times in one batch
    cmd = [sys.executable, "-m", "synaptix_amd", "run", "--random", os.path.join(folder, "config.json"), "--seed", "3",
           "--prompt-ids", "5,6,7,8,9", "--max-tokens", "4", "--temperature", "0", "--batch", "3"]
    runs = [subprocess.run(cmd, capture_output=True, text=True, cwd=ROOT, timeout=300) for _ in range(2)]
    assert all(r.returncode == 0 for r in runs), runs[0].stderr[-2000:]
    rows = [[int(t) for t in line.split()] for line in runs[0].stdout.strip().splitlines()]
    assert len(rows) == 3 and rows[0] == rows[1] == rows[2] and len(rows[0]) == 4       # greedy: the same three times
    assert all(0 <= t < CONFIGS[name]["vocab_size"] for t in rows[0]) and runs[0].stdout == runs[1].stdout
    assert "15 prompt + 12 new tokens" in runs[0].stderr
    proc = subprocess.run(cmd[:4] + cmd[6:], capture_output=True, text=True, cwd=ROOT, timeout=60)   # neither MODEL nor --random
    assert proc.returncode == 1 and "MODEL" in proc.stderr
    cmd = [sys.executable, "-m", "synaptix_amd", "bench", folder, "--n-tokens", "16", "--prompt-tokens", "9",
           "--batch-size", "3", "--warmup", "1"]
    proc = subprocess.run(cmd, capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    line = json.loads(proc.stdout.strip().splitlines()[-1])
    assert line["new_tokens"] == 48 and line["prompt_tokens"] == 27 and line["decode_tok_s"] > 0


def test_per_op_times_of_eager_steps_and_their_refusal_under_capture():
    from synaptix_amd import Engine
    from synaptix_amd.kernels import ops
    eng = Engine.load(model_folder("B"), dtype="bfloat16", max_tokens=512)
    eng.prompt_graphs = False                                  # (op by op means launched one by one, both times)
    s = eng.acquire()
    plain = eng.step([(s, [1, 2, 3, 4, 5])], want="last").clone()
    eng.release(s)
    s = eng.acquire()
    with ops.op_timing() as times:
        timed = eng.step([(s, [1, 2, 3, 4, 5])], want="last")
        eng.step([(s, [6])], want="last")
    assert torch.equal(timed, plain)                       # timing changes no result
    L = CONFIGS["B"]["num_hidden_layers"]
    # few rows: only the first norm and the last are kernels of their own; the others ride on the products beside
    # them (all four products of a layer but the first layer's q/k/v and the last layer's down projection)
    assert times["syn_add_rmsnorm"][1] == 2 * 2 and times["syn_embed"][1] == 2
    assert times["syn_gemm_packed_norm"][1] == 2 * (4 * L - 2)
    assert times["syn_attention_prefill_bf16"][1] == L and times["syn_attention_decode_fused_bf16"][1] == L
    assert all(ms > 0 for ms, _ in times.values())
    text = times.report()
    assert text.splitlines()[0].split() == ["op", "ms", "calls", "share"] and "total" in text
    with ops.op_timing():
        with pytest.raises(Exception, match="per-op times need eager steps"):
            eng.decode_runner(1, 256).step([s], [7])
    eng.release(s)
    # the command line's switch
    cmd = [sys.executable, "-m", "synaptix_amd", "run", model_folder("A"), "--prompt-ids", "1,2,3", "--max-tokens", "3",
           "--temperature", "0", "--op-times"]
    proc = subprocess.run(cmd, capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "syn_gemm" in proc.stderr and "share" in proc.stderr


def test_smoke_entry():
    sys.path.insert(0, ROOT)
    import __graft_entry__
    __graft_entry__.smoke()


def test_bench_line_keeps_its_contract():
    """bench.py with one layer of the named shape and a few steps: one JSON line with the agreed keys;
    more than one GPU, or a prompt beyond the context, is refused with exit code 2 and one line."""
    cmd = [sys.executable, f"{ROOT}/bench.py"]
    proc = subprocess.run(cmd + ["--layers", "1", "--steps", "3", "--warmup", "1", "--batch", "2", "--no-points",
                                 "--prompt", "256"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [l for l in proc.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 3 and rec["warmup"] == 1 and rec["dtype"] == "bf16"
    cfg = rec["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())
    assert cfg["layers"] == 1 and cfg["model_layers"] == 36 and cfg["global_batch"] == 2 and cfg["seq_len"] == 256
    assert set(rec["prefill"]) == {"value", "tokens", "ms", "frac"} and rec["prefill"]["tokens"] == 256
    roof = rec["roofline"]
    assert roof["bound"] == "hbm" and roof["unit"] == "GB/s" and roof["peak"] == 8000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert rec["value"] > 0 and abs(rec["value"] - 2 / (rec["ms_per_step"] * 1e-3)) < 0.01 * rec["value"]
    # with points: batch 1 and 64 and the same batch through the generation loop (the other shapes' points come
    # with the whole model only)
    proc = subprocess.run(cmd + ["--layers", "1", "--steps", "3", "--warmup", "1", "--batch", "2", "--prompt", "128"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    pts = json.loads([l for l in proc.stdout.splitlines() if l.strip()][-1])["points"]
    assert pts["decode_b1"] > 0 and pts["decode_b64"] > 0 and pts["decode_b2_through_generate"] > 0
    assert all(not isinstance(v, (dict, list)) for v in pts.values()) and "decode_32b_b8" not in pts
    # the other shapes: the same keys, the shape's own sizes
    proc = subprocess.run(cmd + ["--shape", "4b", "--layers", "1", "--steps", "3", "--warmup", "1"], capture_output=True,
                          text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    rec4 = json.loads([l for l in proc.stdout.splitlines() if l.strip()][-1])
    assert set(rec4) >= set(rec) - {"measured"}
    c4 = rec4["config"]
    assert len(c4) <= 20 and all(not isinstance(v, (dict, list)) for v in c4.values())
    assert (c4["hidden"], c4["intermediate"], c4["heads"], c4["tie_word_embeddings"]) == (2560, 9728, 32, True)
    assert c4["global_batch"] == 16 and c4["new_tokens"] == 4 and 64 <= c4["min_prompt"] <= c4["max_prompt"] <= 4096
    assert abs(rec4["value"] - 16 / (rec4["ms_per_step"] * 1e-3)) < 0.01 * rec4["value"]
    proc = subprocess.run(cmd + ["--shape", "32b", "--layers", "1", "--steps", "3", "--warmup", "1", "--batch", "2",
                                 "--no-points", "--prompt", "128"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    c32 = json.loads([l for l in proc.stdout.splitlines() if l.strip()][-1])["config"]
    assert (c32["hidden"], c32["intermediate"], c32["heads"], c32["model_layers"]) == (5120, 25600, 64, 64)
    for extra in (["--gpus", "2"], ["--prompt", "9000"], ["--shape", "4b", "--gpus", "4"]):
        proc = subprocess.run(cmd + extra, capture_output=True, text=True, timeout=120)
        assert proc.returncode == 2
        assert len([l for l in proc.stdout.splitlines() if l.strip()]) == 1
