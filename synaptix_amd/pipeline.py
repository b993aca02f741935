"""The Python entry point: a model folder in, token ids out.

In the manner of the reference's pipeline for this model
(crates/synaptix-models/llm/qwen3/src/pipeline.rs:23-158: load / load_with_max_seq /
load_with_precision, encode, decode, generate, generate_streaming) and of its facade's
load_llm(path, device, precision, max_seq) (crates/synaptix/src/facade/llm.rs:1434-1476).
The stop token defaults to config.json's eos_token_id when the caller names none
(pipeline.rs:100-105).  Beyond the reference: `generate_batch` for many prompts at once.
"""
from __future__ import annotations

import dataclasses
import os

from .engine import Engine
from .engine.generate import generate as _generate, GenerationOutput, GenerationStats
from .sampling import GenerationConfig

_DTYPE_NAMES = {"bf16": "bfloat16", "bfloat16": "bfloat16", "f32": "float32", "float32": "float32"}


class Pipeline:
    def __init__(self, engine: Engine, folder: str | None = None):
        self.engine = engine
        self.config = engine.model.config
        self.folder = folder
        self._tokenizer = None

    # ------------------------------------------------------------------ loading
    @classmethod
    def load(cls, path: str, device: str = "cuda", dtype: str = "bf16", max_seq: int | None = None,
             max_tokens: int | None = None, max_batch: int | None = None) -> "Pipeline":
        """path: a folder with config.json and safetensors.  dtype: bf16 (default) or f32, the
        compute type of the whole model.  max_seq: the longest sequence (positions and cache);
        default config.json's max_position_embeddings.  max_tokens: tokens the cache holds in all
        (default: 8 sequences of max_seq, at most 65,536)."""
        if dtype not in _DTYPE_NAMES:
            raise ValueError(f"dtype {dtype!r}: bf16 or f32 (f16 and quantized types are not built)")
        if device == "cuda":
            device = "cuda:0"
        if not device.startswith("cuda"):
            raise ValueError(f"device {device!r}: this engine runs on the GPU only")
        from .config import load_config
        _, cfg = load_config(path)
        longest = max_seq or cfg.max_position_embeddings
        if max_tokens is None:
            max_tokens = min(8 * longest, 65536)
            max_tokens = max(max_tokens, longest)
        eng = Engine.load(path, dtype=_DTYPE_NAMES[dtype], max_tokens=max_tokens, max_slots=max_batch,
                          max_seq=max_seq, device=device)
        return cls(eng, path)

    @classmethod
    def random(cls, config_json: str, seed: int = 0, device: str = "cuda", dtype: str = "bf16", max_seq: int | None = None,
               max_tokens: int | None = None, max_batch: int | None = None) -> "Pipeline":
        """No model folder: the architecture and sizes of `config_json` (a config.json file) with random weights
        drawn on the device from `seed` (for measurements and trials; nothing is written)."""
        import json
        from .config import resolve_architecture
        if dtype not in _DTYPE_NAMES:
            raise ValueError(f"dtype {dtype!r}: bf16 or f32 (f16 and quantized types are not built)")
        if device == "cuda":
            device = "cuda:0"
        with open(config_json) as f:
            d = json.load(f)
        cfg = resolve_architecture(d).config_cls.from_dict(d)
        longest = max_seq or cfg.max_position_embeddings
        if max_tokens is None:
            max_tokens = max(min(8 * longest, 65536), longest)
        eng = Engine.from_config(cfg, seed=seed, dtype=_DTYPE_NAMES[dtype], max_tokens=max_tokens, max_slots=max_batch,
                                 max_seq=max_seq, device=device)
        return cls(eng, None)

    # ------------------------------------------------------------------ text, when the folder has a tokenizer
    def _tok(self):
        if self._tokenizer is None:
            f = os.path.join(self.folder or "", "tokenizer.json")
            if not os.path.isfile(f):
                raise FileNotFoundError(f"{f}: no tokenizer in the model folder; pass token ids")
            from tokenizers import Tokenizer
            self._tokenizer = Tokenizer.from_file(f)
        return self._tokenizer

    def encode(self, text: str) -> list:
        return self._tok().encode(text).ids

    def decode(self, ids) -> str:
        return self._tok().decode(list(ids))

    # ------------------------------------------------------------------ generation
    def _with_stop(self, cfg: GenerationConfig) -> GenerationConfig:
        if cfg.eos_token_id is None and not cfg.eos_token_ids:
            eos = getattr(self.config, "eos_token_id", None)
            if eos is not None:
                cfg = dataclasses.replace(cfg, eos_token_id=eos)
        return cfg

    def generate(self, prompt_ids, cfg: GenerationConfig | None = None, use_graph: bool = True):
        """One prompt: (generated ids, stats)."""
        outs, stats = self.generate_batch([prompt_ids], cfg, use_graph=use_graph)
        return outs[0].tokens, stats

    def generate_streaming(self, prompt_ids, cfg: GenerationConfig | None, on_token, use_graph: bool = True):
        """on_token(token_id) -> bool is called for every token; False cancels."""
        outs, stats = self.generate_batch([prompt_ids], cfg, on_token=lambda r, t: on_token(t), use_graph=use_graph)
        return outs[0].tokens, stats

    def generate_batch(self, prompts, cfg=None, on_token=None, max_batch: int | None = None, use_graph: bool = True):
        """Many prompts: ([GenerationOutput], GenerationStats).  cfg: one for all, or a list."""
        if cfg is None:
            cfg = GenerationConfig()
        cfg = self._with_stop(cfg) if isinstance(cfg, GenerationConfig) else [self._with_stop(c) for c in cfg]
        return _generate(self.engine, prompts, cfg, on_token=on_token, max_batch=max_batch, use_graph=use_graph)


def load(path: str, device: str = "cuda", dtype: str = "bf16", max_seq: int | None = None, **kw) -> Pipeline:
    return Pipeline.load(path, device, dtype, max_seq, **kw)
