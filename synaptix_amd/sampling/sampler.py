"""From rows of logits on the device to one token for each sequence.

Order of the reference's pipeline (crates/synaptix-models/llm/common/src/generate.rs:304-340):
repetition penalty, presence/frequency penalty, temperature, top-k, top-p, min-p, then greedy
(temperature <= 0) or multinomial.  The reference does all of it on the host from a downloaded
vector (generate.rs:124-144); here the logits stay on the device.  Greedy and temperature
sampling are one hand-written kernel; the filters run as device tensor operations in front of it.
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


def apply_filters(row: torch.Tensor, cfg: GenerationConfig, penalty_ids) -> torch.Tensor:
    """One row of float logits through the processors that are switched on; returns a new row."""
    x = row.clone()
    V = x.numel()
    if cfg.penalties_on and len(penalty_ids):
        ids = torch.as_tensor([t for t in penalty_ids if 0 <= t < V], dtype=torch.long, device=x.device)
        counts = torch.bincount(ids, minlength=V).to(torch.float32)
        seen = counts > 0
        if cfg.repetition_penalty != 1.0:
            # applied once for each occurrence: positive logits are divided, the others multiplied
            # (crates/synaptix-infer/src/sampling/repetition.rs:27-45)
            f = torch.pow(torch.tensor(cfg.repetition_penalty, dtype=torch.float32, device=x.device), counts)
            x = torch.where(seen, torch.where(x > 0, x / f, x * f), x)
        if cfg.presence_penalty != 0.0 or cfg.frequency_penalty != 0.0:
            # repetition.rs:59-77
            x = torch.where(seen, x - (cfg.presence_penalty + cfg.frequency_penalty * counts), x)
    if cfg.temperature > 0.0 and cfg.temperature != 1.0:
        x = x / torch.tensor(cfg.temperature, dtype=torch.float32, device=x.device)
    if 0 < cfg.top_k < V:
        # keep the k largest (crates/synaptix-infer/src/sampling/top_k.rs:8-24); equal values at the
        # k-th place are all kept, where the reference keeps an arbitrary k of them
        kth = torch.topk(x, cfg.top_k).values[-1]
        x = torch.where(x < kth, torch.full_like(x, float("-inf")), x)
    if cfg.top_p < 1.0:
        # sorted by probability, a candidate stays while the sum before it is <= p * total
        # (crates/synaptix-infer/src/sampling/top_p.rs:8-44)
        probs = torch.exp(x - x.max())
        order = torch.argsort(probs, descending=True, stable=True)
        sp = probs[order]
        before = torch.cumsum(sp, 0) - sp
        drop = order[(before > cfg.top_p * probs.sum()) & torch.isfinite(x[order])]
        x[drop] = float("-inf")
    if cfg.min_p > 0.0:
        # crates/synaptix-infer/src/sampling/min_p.rs:8-24
        e = torch.exp(x - x.max())
        pr = e / e.sum()
        x = torch.where(pr < cfg.min_p * pr.max(), torch.full_like(x, float("-inf")), x)
    return x


def sample_batch(logits: torch.Tensor, samplers: list) -> list:
    """logits [B, V] float on the device, one SequenceSampler a row; returns B token ids."""
    B = logits.shape[0]
    assert B == len(samplers)
    if not all(s.config.plain for s in samplers):
        rows = []
        for r, s in enumerate(samplers):
            rows.append(logits[r] if s.config.plain and not (s.config.temperature > 0 and s.config.temperature != 1.0)
                        else apply_filters(logits[r], s.config, s.penalty_ids()))
        logits = torch.stack(rows).contiguous()
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
