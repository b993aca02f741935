"""From rows of logits on the device to one token for each sequence.

Order of the reference's pipeline (crates/synaptix-models/llm/common/src/generate.rs:304-340):
repetition penalty, presence/frequency penalty, temperature, top-k, top-p, min-p, then greedy
(temperature <= 0) or multinomial.  The reference does all of it on the host from a downloaded
vector (generate.rs:124-144); here the logits stay on the device: the processors are one kernel for
the batch (ops.filter_rows), greedy and temperature sampling another (ops.sample_rows).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .params import GenerationConfig
from .philox import Philox4x32


class SequenceSampler:
    """Per-sequence state: the options, a Philox stream of its own and the context so far."""

    def __init__(self, config: GenerationConfig, prompt, seed: int | None = None):
        self.config = config
        self.rng = Philox4x32(config.seed if seed is None else seed)
        self.context = list(prompt) if config.penalties_on else []

    def penalty_ids(self) -> list:
        """The tail of the context that the penalties look at (crates/synaptix-infer/src/sampling/repetition.rs:7-13)."""
        n = self.config.repeat_last_n
        return self.context if n == 0 or n >= len(self.context) else self.context[len(self.context) - n:]

    def commit(self, token: int) -> None:
        if self.config.penalties_on:
            self.context.append(token)


_ZEROED = {}      # device -> int32 counters of the penalties, zero between calls


def _counters(device, n: int) -> torch.Tensor:
    t = _ZEROED.get(str(device))
    if t is None or t.numel() < n:
        t = _ZEROED[str(device)] = torch.zeros(n, dtype=torch.int32, device=device)
    return t


def filter_batch(logits: torch.Tensor, configs: list, penalty_ids: list) -> torch.Tensor:
    """logits [B, V] float on the device through the processors that each row's GenerationConfig switches on
    (ops.filter_rows: one kernel for the batch); returns new rows, divided by the temperature where it is
    positive.  penalty_ids[r]: the tokens that row r's penalties look at."""
    B, V = logits.shape
    dev = logits.device
    ids, starts = [], [0]
    for cfg, row_ids in zip(configs, penalty_ids):
        if cfg.penalties_on:
            ids += [int(t) for t in row_ids]
        starts.append(len(ids))
    # two copies to the device: the float options column after column, and top_k, the rows' offsets and the tokens
    floats = ([float(c.temperature) for c in configs] + [float(c.top_p) for c in configs] + [float(c.min_p) for c in configs]
              + [float(c.repetition_penalty) if c.penalties_on else 1.0 for c in configs]
              + [float(c.presence_penalty) if c.penalties_on else 0.0 for c in configs]
              + [float(c.frequency_penalty) if c.penalties_on else 0.0 for c in configs])
    ints = [int(c.top_k) if 0 < c.top_k < V else 0 for c in configs] + starts + ids
    f = torch.tensor(floats, dtype=torch.float32).to(dev)
    i = torch.tensor(ints, dtype=torch.int32).to(dev)
    temperature, top_p, min_p, repetition, presence, frequency = (f[c * B:(c + 1) * B] for c in range(6))
    out = torch.empty_like(logits)
    ops.filter_rows(logits, out, temperature, i[:B], top_p, min_p, repetition, presence, frequency,
                    i[2 * B + 1:] if ids else None, i[B:2 * B + 1] if ids else None,
                    _counters(dev, B * V) if ids else None)
    return out


def sample_batch(logits: torch.Tensor, samplers: list) -> list:
    """logits [B, V] float on the device, one SequenceSampler a row; returns B token ids."""
    B = logits.shape[0]
    assert B == len(samplers)
    if not all(s.config.plain for s in samplers):
        logits = filter_batch(logits.contiguous(), [s.config for s in samplers], [s.penalty_ids() for s in samplers])
        temps = [1.0 if s.config.temperature > 0 else 0.0 for s in samplers]   # already divided
    else:
        temps = [float(s.config.temperature) for s in samplers]
    out = torch.empty(B, dtype=torch.int32, device=logits.device)
    if all(t <= 0.0 for t in temps):
        ops.sample_rows(logits, None, None, out)
    else:
        u = [s.rng.next_multinomial_uniform() if t > 0.0 else 0.0 for s, t in zip(samplers, temps)]
        t_dev = torch.tensor(temps, dtype=torch.float32).to(logits.device)
        u_dev = torch.tensor(u, dtype=torch.float32).to(logits.device)
        ops.sample_rows(logits, t_dev, u_dev, out)
    tokens = out.cpu().tolist()
    for s, t in zip(samplers, tokens):
        s.commit(t)
    return tokens
