"""Random-weights mode: write a model folder (config.json, model.safetensors) from a
configuration and a seed.

The reference has no such mode for its decoder; its building blocks are a seeded
normal initialiser and the fact that the weight source is a trait
(crates/synaptix-nn/src/init.rs:21-49, crates/synaptix-models/llm/common/src/weights.rs:9-12).
Matrices are N(0, 0.02), norm gains 1 + N(0, 0.1), each tensor from a stream of its own.
"""
from __future__ import annotations

import json
import os

import torch

from .safetensors_io import save_file
from .source import RandomSource


def write_random_model(folder: str, config, seed: int, store_dtype=torch.bfloat16, std=0.02, gain_std=0.1,
                       extra_tensors: dict | None = None) -> str:
    """`config` is a typed configuration of a registered architecture."""
    from ..config.registry import resolve_architecture

    cfg_dict = config.to_dict()
    arch = resolve_architecture(cfg_dict)
    model = arch.build(config)
    src = RandomSource(model.tensor_specs(), seed, store_dtype=store_dtype, std=std, gain_std=gain_std)
    tensors = {n: src.tensor(n) for n in src.names()}
    if extra_tensors:
        tensors.update(extra_tensors)
    os.makedirs(folder, exist_ok=True)
    cfg_dict["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32", torch.float16: "float16"}[store_dtype]
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg_dict, f, indent=1)
    save_file(tensors, os.path.join(folder, "model.safetensors"), metadata={"format": "pt", "seed": seed})
    return folder
