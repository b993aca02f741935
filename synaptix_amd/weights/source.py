"""Where weights come from: a folder of safetensors, a dict, or a seeded generator.

A source answers by tensor name, as the reference's `WeightSource` trait does
(crates/synaptix-models/llm/common/src/weights.rs:9-12).
"""
from __future__ import annotations

import hashlib
from dataclasses import dataclass

import torch

from .safetensors_io import SafetensorsFile, resolve_shards, _NAMES


@dataclass(frozen=True)
class TensorSpec:
    """What a part expects under a name.  `kind` only matters to the random generator:
    "matrix" and "table" draw N(0, std), "gain" draws 1 + N(0, gain_std)."""
    shape: tuple
    kind: str = "matrix"


class WeightSource:
    def names(self) -> list:
        raise NotImplementedError

    def info(self, name: str):
        """(dtype name as safetensors spells it, shape)."""
        raise NotImplementedError

    def tensor(self, name: str) -> torch.Tensor:
        raise NotImplementedError

    def contains(self, name: str) -> bool:
        return name in set(self.names())


class FolderSource(WeightSource):
    """All shards of a model folder, mapped; the header of each is parsed once."""

    def __init__(self, folder: str):
        self.folder = folder
        self.files = [SafetensorsFile(p) for p in resolve_shards(folder)]
        self._where = {}
        for f in self.files:
            for n in f.names():
                self._where[n] = f

    def names(self):
        return list(self._where)

    def info(self, name):
        return self._where[name].info(name)

    def tensor(self, name):
        return self._where[name].tensor(name)

    def contains(self, name):
        return name in self._where


class DictSource(WeightSource):
    def __init__(self, tensors: dict):
        self.tensors = tensors

    def names(self):
        return list(self.tensors)

    def info(self, name):
        t = self.tensors[name]
        return _NAMES[t.dtype], tuple(t.shape)

    def tensor(self, name):
        return self.tensors[name]

    def contains(self, name):
        return name in self.tensors


def tensor_seed(seed: int, name: str) -> int:
    """A stream of its own for each tensor, so that values do not depend on the order of loading."""
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFF_FFFF_FFFF_FFFF


class RandomSource(WeightSource):
    """Seeded weights for a set of specs: matrices and tables N(0, std), gains 1 + N(0, gain_std).

    Values are drawn in 32-bit and rounded once to `store_dtype`.  With `device="cpu"` the
    values depend on (seed, name) only; on another device the device's generator is used
    (fast enough for billions of values, but a different stream).
    """

    def __init__(self, specs: dict, seed: int, store_dtype=torch.bfloat16, std=0.02, gain_std=0.1, device="cpu"):
        self.specs = dict(specs)
        self.seed = seed
        self.store_dtype = store_dtype
        self.std = std
        self.gain_std = gain_std
        self.device = torch.device(device)

    def names(self):
        return list(self.specs)

    def info(self, name):
        return _NAMES[self.store_dtype], tuple(self.specs[name].shape)

    def tensor(self, name):
        spec = self.specs[name]
        g = torch.Generator(device=self.device)
        g.manual_seed(tensor_seed(self.seed, name))
        shape = tuple(spec.shape)
        if spec.kind == "gain":
            t = torch.randn(shape, generator=g, device=self.device, dtype=torch.float32) * self.gain_std + 1.0
        elif self.device.type == "cpu" or self.store_dtype == torch.float32:
            t = torch.randn(shape, generator=g, device=self.device, dtype=torch.float32) * self.std
        else:
            # large tensors on the device: draw in the stored type to keep the peak low
            t = torch.randn(shape, generator=g, device=self.device, dtype=self.store_dtype) * self.std
        return t.to(self.store_dtype)

    def contains(self, name):
        return name in self.specs
