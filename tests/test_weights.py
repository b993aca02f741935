"""Safetensors reading and writing, the weight check, kept types, random weights (no GPU)."""
import json
import os

import pytest
import torch

from synaptix_amd import Qwen3Config, WeightError, write_random_model
from synaptix_amd.config import resolve_architecture
from synaptix_amd.weights import (SafetensorsFile, SafetensorsError, FolderSource, DictSource, RandomSource, save_file,
                                  check_source, kept_dtype, load_weights, resolve_shards)
from helpers import TINY_A, TINY_B, model_folder


def test_round_trip_bit_exact_and_against_the_library(tmp_path):
    t = {"a": torch.randn(3, 5).to(torch.bfloat16), "b.c": torch.arange(7, dtype=torch.int32),
         "f": torch.randn(2, 2, 2), "h": torch.randn(4).to(torch.float16), "e": torch.empty(0, 3)}
    p = str(tmp_path / "x.safetensors")
    save_file(t, p, metadata={"k": "v"})
    f = SafetensorsFile(p)
    assert sorted(f.names()) == sorted(t) and f.metadata == {"k": "v"}
    for n, v in t.items():
        got = f.tensor(n)
        assert got.dtype == v.dtype and got.shape == v.shape and torch.equal(got, v)
    assert f.info("a") == ("BF16", (3, 5))
    from safetensors.torch import load_file, save_file as lib_save       # the public library reads ours, we read its
    lib = load_file(p)
    assert all(torch.equal(lib[n], t[n]) for n in t)
    q = str(tmp_path / "y.safetensors")
    lib_save({k: v for k, v in t.items() if v.numel()}, q)
    g = SafetensorsFile(q)
    assert all(torch.equal(g.tensor(n), t[n]) for n in g.names())
    with pytest.raises(SafetensorsError, match="tensor not found: zz"):
        f.tensor("zz")


def test_broken_files(tmp_path):
    p = tmp_path / "bad.safetensors"
    p.write_bytes(b"\x05\x00")
    with pytest.raises(SafetensorsError, match="shorter"):
        SafetensorsFile(str(p))
    p.write_bytes((10 ** 9).to_bytes(8, "little") + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(str(p))
    h = json.dumps({"a": {"dtype": "F8_E4M3", "shape": [1], "data_offsets": [0, 1]}}).encode()
    p.write_bytes(len(h).to_bytes(8, "little") + h + b"\0")
    with pytest.raises(SafetensorsError, match="unsupported dtype F8_E4M3"):
        SafetensorsFile(str(p)).tensor("a")
    with pytest.raises(SafetensorsError, match="no model.safetensors"):
        resolve_shards(str(tmp_path))


def test_shards_through_the_index(tmp_path):
    src = SafetensorsFile(os.path.join(model_folder("A"), "model.safetensors"))
    names = sorted(src.names())
    half = len(names) // 2
    save_file({n: src.tensor(n) for n in names[:half]}, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({n: src.tensor(n) for n in names[half:]}, str(tmp_path / "model-00002-of-00002.safetensors"))
    wm = {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
          for i, n in enumerate(names)}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": wm}))
    folder = FolderSource(str(tmp_path))
    assert sorted(folder.names()) == names
    assert all(torch.equal(folder.tensor(n), src.tensor(n)) for n in names)


def _model(cfg_dict):
    cfg = Qwen3Config.from_dict(cfg_dict)
    return resolve_architecture(cfg.to_dict()).build(cfg)


def test_one_error_lists_missing_unexpected_and_wrong_shapes():
    model = _model(TINY_A)
    specs = model.tensor_specs()
    tensors = {n: torch.zeros(s.shape, dtype=torch.bfloat16) for n, s in specs.items()}
    del tensors["model.norm.weight"]
    del tensors["model.layers.1.mlp.up_proj.weight"]
    tensors["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 65, dtype=torch.bfloat16)
    tensors["model.layers.0.self_attn.k_norm.weight"] = torch.zeros(32, dtype=torch.bfloat16)
    tensors["model.layers.7.stray.weight"] = torch.zeros(1)
    tensors["lm_head.weight"] = torch.zeros(512, 64)          # tied: present in some checkpoints, ignored
    with pytest.raises(WeightError) as e:
        check_source(specs, DictSource(tensors), ignored=model.ignored_tensors())
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"] or \
        sorted(err.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.7.stray.weight"]
    assert sorted(n for n, _, _ in err.wrong_shape) == ["model.layers.0.self_attn.k_norm.weight",
                                                        "model.layers.0.self_attn.q_proj.weight"]
    msg = str(err)
    for needle in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (2)", "file [64, 65], model [64, 64]"):
        assert needle in msg
    # untied: lm_head is wanted
    with pytest.raises(WeightError, match="lm_head.weight"):
        check_source(_model(TINY_B).tensor_specs(), DictSource({}))


def test_kept_types():
    bf, f32 = torch.bfloat16, torch.float32
    assert kept_dtype("BF16", bf) == bf and kept_dtype("F16", bf) == bf
    assert kept_dtype("F32", bf) == f32                     # a tensor stored in 32 bits stays so
    assert kept_dtype("I64", bf) == torch.int32 and kept_dtype("U8", f32) == torch.int32
    assert kept_dtype("BF16", f32) == f32 and kept_dtype("F32", f32) == f32
    with pytest.raises(ValueError):
        kept_dtype("F8_E5M2", bf)


def test_load_hands_parts_their_tensors_in_kept_types():
    model = _model(TINY_A)
    specs = model.tensor_specs()
    src = RandomSource(specs, 3)
    tensors = {n: src.tensor(n) for n in src.names()}
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float()      # stored in 32 bits
    load_weights(model, DictSource(tensors), torch.bfloat16, "cpu")
    assert model.final_norm.gain.dtype == torch.float32
    assert model.blocks[0].norm1.gain.dtype == torch.bfloat16
    att = model.blocks[1].mixer
    assert att.w_qkv.shape == ((4 + 2 * 2) * 16, 64) and att.w_qkv.dtype == torch.bfloat16
    assert att.w_qkv.packed is not None and att.w_qkv.plain is None            # kept once, in fragment order
    assert torch.equal(att.w_qkv.rows()[:64], tensors["model.layers.1.self_attn.q_proj.weight"])
    assert torch.equal(att.w_qkv.rows()[64:96], tensors["model.layers.1.self_attn.k_proj.weight"])
    assert model.head.weight is model.embedding.table        # tied: one buffer
    ff = model.blocks[0].feed_forward
    # bf16: rows of gate and up in turns of 16, for the product that applies the activation itself
    gate, up = tensors["model.layers.0.mlp.gate_proj.weight"], tensors["model.layers.0.mlp.up_proj.weight"]
    assert ff.paired and ff.w_gate_up.shape == (2 * 176, 64)
    gu = ff.w_gate_up.rows()
    assert torch.equal(gu[:16], gate[:16]) and torch.equal(gu[16:32], up[:16])
    assert torch.equal(gu[-32:-16], gate[-16:]) and torch.equal(gu[-16:], up[-16:])
    m32 = _model(TINY_A)
    load_weights(m32, DictSource(tensors), torch.float32, "cpu")
    assert m32.blocks[0].mixer.w_o.dtype == torch.float32
    ff32 = m32.blocks[0].feed_forward                          # 32-bit: one after the other
    assert not ff32.paired and ff32.w_gate_up.packed is None and torch.equal(ff32.w_gate_up.plain[176:], up.float())


def test_random_weights_mode(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_B)
    a = write_random_model(str(tmp_path / "a"), cfg, seed=7)
    b = write_random_model(str(tmp_path / "b"), cfg, seed=7)
    c = write_random_model(str(tmp_path / "c"), cfg, seed=8)
    fa, fb, fc = (SafetensorsFile(os.path.join(x, "model.safetensors")) for x in (a, b, c))
    assert len(fa.names()) == 3 * 11 + 3
    n = "model.layers.2.mlp.down_proj.weight"
    assert torch.equal(fa.tensor(n), fb.tensor(n)) and not torch.equal(fa.tensor(n), fc.tensor(n))
    w = fa.tensor(n).float()
    assert w.shape == (128, 320) and fa.info(n)[0] == "BF16" and abs(float(w.std()) - 0.02) < 0.002
    g = fa.tensor("model.layers.0.input_layernorm.weight").float()
    assert abs(float(g.mean()) - 1.0) < 0.05 and 0.05 < float(g.std()) < 0.15
    d = json.load(open(os.path.join(a, "config.json")))
    assert d["architectures"] == ["Qwen3ForCausalLM"] and d["head_dim"] == 32 and d["rope_theta"] == 1e6
    # a value does not depend on which other tensors are drawn
    specs = _model(TINY_B).tensor_specs()
    only = RandomSource({n: specs[n]}, 7).tensor(n)
    assert torch.equal(only, fa.tensor(n))
