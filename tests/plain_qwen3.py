"""A plain, slow statement of the Qwen3 dense decoder, one function per part.

Whole sequences only: no cache, no batching, no kernels.  Every call recomputes
the full sequence.  It shares no code with the package under test; it reads a
model folder through the `safetensors` library and NumPy-style torch CPU ops.

Each function cites the lines of the reference (paths under the reference
checkout) whose formula it states.
"""
from __future__ import annotations

import json
import math
import os

import torch

F32 = torch.float32


# --------------------------------------------------------------------------- parts

def embed(table: torch.Tensor, ids) -> torch.Tensor:
    """x[n, :] = E[id[n], :], no scale and no norm.

    crates/synaptix-ops/src/embed/token_embed.rs:4-15,
    crates/synaptix-models/llm/qwen3/src/config.rs:107-108 (no embed scale/norm).
    """
    ids = torch.as_tensor(ids, dtype=torch.long)
    if ids.numel() and (int(ids.min()) < 0 or int(ids.max()) >= table.shape[0]):
        raise ValueError("token id outside the vocabulary")
    return table[ids]


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """y_i = x_i * (mean_j x_j^2 + eps)^(-1/2) * w_i over the last axis; plain gain.

    crates/synaptix-ops/src/norm/rms_norm.rs:16-26 (square, mean, +eps, sqrt,
    reciprocal, times x, times w).
    """
    var = (x * x).mean(dim=-1, keepdim=True)
    inv = 1.0 / torch.sqrt(var + eps)
    return x * inv * w


def rope_tables(head_dim: int, n_pos: int, theta: float, dtype=F32):
    """cos/sin [n_pos, head_dim/2]; f_i = theta^(-2i/hd); angle = t * f_i.

    crates/synaptix-ops/src/pos/rope_cache.rs:16-38 (f32 powf, f32 product, cos/sin).
    The angle arithmetic is done in `dtype` (float32 as the reference does).
    """
    half = head_dim // 2
    i = torch.arange(half, dtype=dtype)
    expo = -(2.0 * i) / torch.tensor(float(head_dim), dtype=dtype)
    freqs = torch.pow(torch.tensor(float(theta), dtype=dtype), expo)
    t = torch.arange(n_pos, dtype=dtype)
    ang = t[:, None] * freqs[None, :]
    return torch.cos(ang), torch.sin(ang)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions) -> torch.Tensor:
    """Half-split rotation of x [S, n, hd] at the given absolute positions.

    For d < hd/2:  o[d]      = x[d] cos[p,d] - x[d+hd/2] sin[p,d]
                   o[d+hd/2] = x[d] sin[p,d] + x[d+hd/2] cos[p,d]
    crates/synaptix-ops/src/pos/rope.rs:81-97 (Split layout: first half / second half).
    """
    half = x.shape[-1] // 2
    pos = torch.as_tensor(positions, dtype=torch.long)
    c = cos[pos][:, None, :].to(x.dtype)
    s = sin[pos][:, None, :].to(x.dtype)
    a, b = x[..., :half], x[..., half:]
    return torch.cat([a * c - b * s, a * s + b * c], dim=-1)


def attention(q, k, v, scale: float, q_positions, window: int | None = None) -> torch.Tensor:
    """Causal grouped-query attention with an exact two-pass softmax.

    q [S, nh, hd]; k, v [T, nkv, hd]; query s sits at absolute position
    q_positions[s]; key j sits at position j.  Head h reads kv head h // (nh/nkv).
    Key j is visible iff j <= p and (window is None or p < j + window).

    crates/synaptix-kernels-cuda/tests/cuda_flash_decode.rs:32-90 (two-pass softmax,
    h_kv = h / n_rep, causal rule), crates/synaptix-models/llm/common/src/model.rs:2581-2596
    (mask: causal_ok = j <= qi, window_ok = qi < j + w).
    """
    S, nh, hd = q.shape
    T, nkv, _ = k.shape
    g = nh // nkv
    out = torch.zeros(S, nh, v.shape[-1], dtype=q.dtype)
    j = torch.arange(T)
    for s in range(S):
        p = int(q_positions[s])
        visible = j <= p
        if window is not None:
            visible &= p < j + window
        for h in range(nh):
            hk = h // g
            scores = (k[:, hk, :] @ q[s, h, :]) * scale
            scores = torch.where(visible, scores, torch.full_like(scores, -math.inf))
            m = scores.max()
            e = torch.exp(scores - m)
            e = torch.where(visible, e, torch.zeros_like(e))
            out[s, h, :] = (e[:, None] * v[:, hk, :]).sum(0) / e.sum()
    return out


def silu(z: torch.Tensor) -> torch.Tensor:
    """silu(z) = z / (1 + exp(-z)).  crates/synaptix-kernels-cuda/src/cu/fused/mlp/silu_and_mul.cu:11-52."""
    return z / (1.0 + torch.exp(-z))


def swiglu_mlp(h, w_gate, w_up, w_down) -> torch.Tensor:
    """down( silu(gate(h)) * up(h) ).  crates/synaptix-models/llm/common/src/model.rs:1670-1691."""
    return (silu(h @ w_gate.T) * (h @ w_up.T)) @ w_down.T


# --------------------------------------------------------------------------- the model

class PlainQwen3:
    """Weights by name plus the config.json keys; `forward` runs one whole sequence."""

    def __init__(self, cfg: dict, tensors: dict, dtype=F32):
        self.cfg = cfg
        self.dtype = dtype
        self.w = {k: v.to(dtype) for k, v in tensors.items()}
        self.L = cfg["num_hidden_layers"]
        self.nh = cfg["num_attention_heads"]
        self.nkv = cfg["num_key_value_heads"]
        self.hd = cfg["head_dim"]
        self.eps = float(cfg["rms_norm_eps"])
        self.theta = float(cfg["rope_theta"])
        self.tied = bool(cfg.get("tie_word_embeddings", True))
        self.scale = 1.0 / math.sqrt(self.hd)
        self._tables = None
        self.table_dtype = F32        # the reference builds its angles in float32 (tests of invariants widen it)

    @classmethod
    def from_folder(cls, folder: str, dtype=F32) -> "PlainQwen3":
        from safetensors.torch import load_file

        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        tensors = load_file(os.path.join(folder, "model.safetensors"))
        return cls(cfg, tensors, dtype)

    def tables(self, n_pos: int):
        if self._tables is None or self._tables[0].shape[0] < n_pos:
            # angles in float32 as the reference builds them, then widened if asked
            cos, sin = rope_tables(self.hd, n_pos, self.theta, self.table_dtype)
            self._tables = (cos.to(self.dtype), sin.to(self.dtype))
        return self._tables

    def attention_block(self, l: int, xn: torch.Tensor, positions, rope_offset: int = 0) -> torch.Tensor:
        """q/k/v projections, per-head q/k norm, rotation, attention, output projection.

        crates/synaptix-models/llm/common/src/model.rs:1715-1734 (projections, head split,
        q/k norm before the rotation, same eps), 1872-1878 (merge heads, o_proj).
        """
        p = f"model.layers.{l}.self_attn."
        S = xn.shape[0]
        q = (xn @ self.w[p + "q_proj.weight"].T).view(S, self.nh, self.hd)
        k = (xn @ self.w[p + "k_proj.weight"].T).view(S, self.nkv, self.hd)
        v = (xn @ self.w[p + "v_proj.weight"].T).view(S, self.nkv, self.hd)
        q = rms_norm(q, self.w[p + "q_norm.weight"], self.eps)
        k = rms_norm(k, self.w[p + "k_norm.weight"], self.eps)
        turned = [p + rope_offset for p in positions]    # rope_offset: every position moved by as much (for invariants)
        cos, sin = self.tables(int(max(turned)) + 1)
        q = apply_rope(q, cos, sin, turned)
        k = apply_rope(k, cos, sin, turned)
        o = attention(q, k, v, self.scale, positions)
        return o.reshape(S, self.nh * self.hd) @ self.w[p + "o_proj.weight"].T

    def hidden(self, ids, rope_offset: int = 0) -> torch.Tensor:
        """Residual stream after the last block.  model.rs:1179-1199 (pre-norm wiring)."""
        x = embed(self.w["model.embed_tokens.weight"], ids)
        positions = list(range(len(ids)))
        for l in range(self.L):
            p = f"model.layers.{l}."
            x = x + self.attention_block(l, rms_norm(x, self.w[p + "input_layernorm.weight"], self.eps), positions,
                                         rope_offset)
            hn = rms_norm(x, self.w[p + "post_attention_layernorm.weight"], self.eps)
            x = x + swiglu_mlp(hn, self.w[p + "mlp.gate_proj.weight"], self.w[p + "mlp.up_proj.weight"],
                               self.w[p + "mlp.down_proj.weight"])
        return x

    def forward(self, ids, rope_offset: int = 0) -> torch.Tensor:
        """Logits [S, V] at every position of one sequence.

        model.rs:1068-1089 (final norm, lm_head; tied -> the embedding matrix, 757-764).
        """
        h = rms_norm(self.hidden(ids, rope_offset), self.w["model.norm.weight"], self.eps)
        w_out = self.w["model.embed_tokens.weight"] if self.tied else self.w["lm_head.weight"]
        return h @ w_out.T


# --------------------------------------------------------------------------- sampling

_M0, _M1 = 0xD2511F53, 0xCD9E8D57
_W0, _W1 = 0x9E3779B9, 0xBB67AE85
_MASK = 0xFFFFFFFF


def philox4x32(counter, key):
    """Ten rounds of Philox-4x32.  crates/synaptix-ops/src/rng.rs:82-97."""
    c = list(counter)
    k = list(key)
    for _ in range(10):
        p0 = _M0 * c[0]
        p1 = _M1 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & _MASK, p1 & _MASK, ((p0 >> 32) ^ c[3] ^ k[1]) & _MASK, p0 & _MASK]
        k = [(k[0] + _W0) & _MASK, (k[1] + _W1) & _MASK]
    return c


class PlainPhilox:
    """Seed in the key, counter from zero, four words a block.  rng.rs:16-25,32-36,50-58,66-73."""

    def __init__(self, seed: int):
        self.key = [seed & _MASK, (seed >> 32) & _MASK]
        self.counter = [0, 0, 0, 0]
        self.buf = []

    def next_u32(self) -> int:
        if not self.buf:
            self.buf = philox4x32(self.counter, self.key)
            for i in range(4):
                self.counter[i] = (self.counter[i] + 1) & _MASK
                if self.counter[i] != 0:
                    break
        return self.buf.pop(0)


def f32(x: float) -> float:
    return float(torch.tensor(x, dtype=F32))


def uniform_for_multinomial(rng: PlainPhilox) -> float:
    """u = (u32 as f64 as f32) / (u32::MAX as f32).  crates/synaptix-infer/src/sampling/multinomial.rs:30-32."""
    return f32(f32(float(rng.next_u32())) / f32(float(0xFFFFFFFF)))


def greedy(logits: torch.Tensor) -> int:
    """The last of equal maxima (Rust's max_by).  crates/synaptix-infer/src/sampling/greedy.rs:7-13."""
    best, arg = -math.inf, 0
    for i, x in enumerate(logits.tolist()):
        if x >= best:
            best, arg = x, i
    return arg


def multinomial(logits: torch.Tensor, u: float) -> int:
    """softmax, then the first i with u < cumsum_i, else the last index.  multinomial.rs:7-28."""
    x = logits.to(F32)
    e = torch.exp(x - x.max())
    p = e / e.sum()
    c = torch.cumsum(p, 0)
    hit = torch.nonzero(u < c)
    return int(hit[0]) if hit.numel() else x.numel() - 1


def penalty_window(ids, last_n: int):
    """last_n == 0 means all.  crates/synaptix-infer/src/sampling/repetition.rs:7-13."""
    return list(ids) if last_n == 0 or last_n >= len(ids) else list(ids)[len(ids) - last_n:]


def repetition_penalty(logits, ids, penalty: float, last_n: int):
    """Per occurrence: positive logit / penalty, else * penalty.  repetition.rs:27-45."""
    out = logits.clone()
    for t in penalty_window(ids, last_n):
        if t < out.numel():
            out[t] = out[t] / penalty if out[t] > 0 else out[t] * penalty
    return out


def presence_frequency(logits, ids, presence: float, frequency: float, last_n: int):
    """logit -= presence + frequency * count.  repetition.rs:59-77."""
    out = logits.clone()
    counts = {}
    for t in penalty_window(ids, last_n):
        counts[t] = counts.get(t, 0) + 1
    for t, c in counts.items():
        if t < out.numel():
            out[t] -= presence + frequency * c
    return out


def top_k(logits, k: int):
    """Keep the k largest, others -inf; 0 or >= V is off.  sampling/top_k.rs:8-24."""
    if k == 0 or k >= logits.numel():
        return logits.clone()
    out = torch.full_like(logits, -math.inf)
    idx = torch.topk(logits, k).indices
    out[idx] = logits[idx]
    return out


def top_p(logits, p: float):
    """Sort finite candidates by probability; keep while cumsum <= p*sum (the crossing one stays).

    sampling/top_p.rs:8-44.
    """
    if p >= 1.0:
        return logits.clone()
    probs = torch.exp(logits - logits.max())
    total = float(probs.sum())
    cand = [i for i in range(logits.numel()) if math.isfinite(float(logits[i]))]
    cand.sort(key=lambda i: -float(probs[i]))
    thresh = p * total
    cum, cutoff = 0.0, len(cand)
    for pos, i in enumerate(cand):
        if cum > thresh:
            cutoff = pos
            break
        cum = f32(cum + float(probs[i]))
    out = logits.clone()
    for i in cand[cutoff:]:
        out[i] = -math.inf
    return out


def min_p(logits, mp: float):
    """Drop tokens with prob < min_p * max prob.  sampling/min_p.rs:8-24."""
    e = torch.exp(logits - logits.max())
    pr = e / e.sum()
    out = logits.clone()
    out[pr < mp * pr.max()] = -math.inf
    return out


def sample(logits, context_ids, rng: PlainPhilox, temperature=0.0, k=0, p=1.0, mp=0.0,
           repetition=1.0, last_n=0, presence=0.0, frequency=0.0) -> int:
    """Order: repetition, presence/frequency, temperature, top-k, top-p, min-p, sampler.

    crates/synaptix-models/llm/common/src/generate.rs:304-340.
    """
    x = logits.to(F32).clone()
    if repetition != 1.0:
        x = repetition_penalty(x, context_ids, repetition, last_n)
    if presence != 0.0 or frequency != 0.0:
        x = presence_frequency(x, context_ids, presence, frequency, last_n)
    if temperature > 0.0 and temperature != 1.0:
        x = x / torch.tensor(temperature, dtype=F32)
    if k > 0:
        x = top_k(x, k)
    if p < 1.0:
        x = top_p(x, p)
    if mp > 0.0:
        x = min_p(x, mp)
    if temperature <= 0.0:
        return greedy(x)
    return multinomial(x, uniform_for_multinomial(rng))


def generate(model: PlainQwen3, prompt, max_new_tokens: int, stop_ids=(), seed=0, **sampling) -> list:
    """One sequence: first token from the prompt's last logits, then one at a time.

    The stop token is part of the output; the check comes before the next forward;
    at least one token is produced.  generate.rs:276-292.
    """
    rng = PlainPhilox(seed)
    ctx = list(prompt)
    out = []
    tok = sample(model.forward(ctx)[-1], ctx, rng, **sampling)
    out.append(tok)
    ctx.append(tok)
    while len(out) < max_new_tokens and out[-1] not in stop_ids:
        tok = sample(model.forward(ctx)[-1], ctx, rng, **sampling)
        out.append(tok)
        ctx.append(tok)
    return out
