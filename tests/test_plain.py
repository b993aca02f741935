"""What fixes the plain implementation beside the reference's text: vectors the reference's own
tests hold, special cases that reduce to a library routine, and invariants.  Each is chosen so
that a plausible mistake (a wrong sign or pairing, eps outside the root, a norm in the wrong
place) fails it."""
import math

import pytest
import torch

import plain_qwen3 as P
from helpers import plain_model, random_tokens

F64 = torch.float64


def rnd(shape, seed, dtype=torch.float32):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)).to(dtype)


# ----------------------------------------------------------------------------- RMSNorm
def test_rms_norm_reference_vector():
    """crates/synaptix-ops/tests/rms_norm.rs:76-95: shape [2,3,4], x_i = 0.1 i - 1, w = [0.5,-0.25,1,2]."""
    x = torch.tensor([i * 0.1 - 1.0 for i in range(24)]).view(2, 3, 4)
    w = torch.tensor([0.5, -0.25, 1.0, 2.0])
    got = P.rms_norm(x, w, 1e-6)
    xd = x.double()
    want = xd * (1.0 / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-6)) * w.double()
    assert (got.double() - want).abs().max() < 1e-5
    # first row by hand: x = [-1, -.9, -.8, -.7], mean x^2 = 0.735
    r = 1 / math.sqrt(0.735 + 1e-6)
    assert torch.allclose(got[0, 0], torch.tensor([-1 * r * 0.5, 0.9 * r * 0.25, -0.8 * r, -0.7 * r * 2]), atol=1e-6)


def test_rms_norm_properties():
    x = rnd((5, 32), 1)
    y = P.rms_norm(x, torch.ones(32), 1e-12)
    assert torch.allclose((y * y).mean(-1), torch.ones(5), atol=1e-5)            # unit RMS with unit gain
    assert torch.allclose(P.rms_norm(7.0 * x, torch.ones(32), 1e-12), y, atol=1e-5)  # scale invariance
    # eps inside the root: tiny x separates sqrt(m + eps) from sqrt(m) + eps and from no eps at all
    t = torch.full((1, 8), 1e-4)
    assert abs(float(P.rms_norm(t, torch.ones(8), 1e-6)[0, 0]) - 1e-4 / math.sqrt(1e-8 + 1e-6)) < 1e-9
    # plain gain, not 1 + w
    assert torch.allclose(P.rms_norm(x, torch.zeros(32), 1e-6), torch.zeros(5, 32))


# ----------------------------------------------------------------------------- rotation
def test_rope_position_zero_and_norm():
    """crates/synaptix-ops/tests/pos.rs:11-57: position 0 is the identity; norms are kept."""
    cos, sin = P.rope_tables(16, 50, 1e4)
    x = rnd((6, 3, 16), 2)
    assert torch.allclose(P.apply_rope(x, cos, sin, [0] * 6), x, atol=1e-7)
    y = P.apply_rope(x, cos, sin, [3, 7, 11, 19, 30, 49])
    assert torch.allclose((y * y).sum(-1), (x * x).sum(-1), rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("theta,hd", [(1e4, 16), (1e6, 32)])
def test_rope_is_complex_multiplication_of_split_pairs(theta, hd):
    """Pair (d, d + hd/2) turns by p * theta^(-2d/hd): (x_d + i x_{d+hd/2}) * e^{i p f_d}.
    An interleaved pairing, a wrong sign or a wrong exponent fails."""
    cos, sin = P.rope_tables(hd, 40, theta, F64)
    x = rnd((1, 1, hd), 3, F64)
    p = 17
    y = P.apply_rope(x, cos, sin, [p])[0, 0]
    half = hd // 2
    z = torch.complex(x[0, 0, :half], x[0, 0, half:])
    f = torch.tensor([theta ** (-2.0 * d / hd) for d in range(half)], dtype=F64)
    zr = z * torch.exp(1j * p * f)
    assert torch.allclose(y[:half], zr.real, atol=1e-12) and torch.allclose(y[half:], zr.imag, atol=1e-12)


def test_rope_is_the_split_case_that_the_reference_checks_its_own_rotation_against():
    """The reference tests its Split rotation (the only layout its decoder calls,
    crates/synaptix-models/llm/common/src/model.rs:2555-2561) against a case made by
    scripts/reference/gen_pos.py:27-58 (crates/synaptix-ops/tests/ref_pos.rs:13-25, to 1e-5): seed 0, q and k
    [2, 8, 32, 64], full-width tables cos|cos and sin|sin, out = x * cos + cat(-x2, x1) * sin.  The case's data
    file is not among the reference's files; its recipe is, and the plain rotation equals it.  The interleaved
    pairing differs from it by more than 1."""
    torch.manual_seed(0)
    batch, heads, seq, hd = 2, 8, 32, 64
    q = torch.randn(batch, heads, seq, hd, dtype=torch.float32)
    k = torch.randn(batch, heads, seq, hd, dtype=torch.float32)
    theta = 10000.0 ** (-torch.arange(0, hd, 2, dtype=torch.float32) / hd)
    freqs = torch.outer(torch.arange(seq, dtype=torch.float32), theta)
    cos_full, sin_full = freqs.cos().repeat(1, 2), freqs.sin().repeat(1, 2)
    cos, sin = P.rope_tables(hd, seq, 10000.0)
    for x in (q, k):
        half = hd // 2
        want = x * cos_full + torch.cat([-x[..., half:], x[..., :half]], -1) * sin_full
        # the plain function takes [S, n, hd]: tokens first
        got = torch.stack([P.apply_rope(x[b].transpose(0, 1), cos, sin, list(range(seq))).transpose(0, 1)
                           for b in range(batch)])
        assert torch.allclose(got, want, atol=1e-5, rtol=1e-5)
        pairs = x.reshape(batch, heads, seq, half, 2)          # what an interleaved pairing would turn
        c, s_ = freqs.cos(), freqs.sin()
        inter = torch.stack([pairs[..., 0] * c - pairs[..., 1] * s_, pairs[..., 0] * s_ + pairs[..., 1] * c], -1)
        assert (inter.reshape(x.shape) - want).abs().max() > 1.0


def test_rope_scores_depend_on_distance_only():
    cos, sin = P.rope_tables(32, 200, 1e6, F64)
    q, k = rnd((1, 1, 32), 4, F64), rnd((1, 1, 32), 5, F64)
    def score(pq, pk):
        return float((P.apply_rope(q, cos, sin, [pq]) * P.apply_rope(k, cos, sin, [pk])).sum())
    assert abs(score(10, 3) - score(110, 103)) < 1e-9
    assert abs(score(10, 3) - score(3, 10)) > 1e-3      # not symmetric: the sign of the angle matters


# ----------------------------------------------------------------------------- attention
def test_attention_reduces_to_library_softmax_attention():
    """One kv head a q head, no mask effect on the last query: equals torch's SDPA with a causal mask."""
    S, nh, hd = 9, 3, 8
    q, k, v = rnd((S, nh, hd), 6), rnd((S, nh, hd), 7), rnd((S, nh, hd), 8)
    got = P.attention(q, k, v, 1 / math.sqrt(hd), list(range(S)))
    want = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                                            is_causal=True).transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-5)


def test_attention_special_cases():
    hd = 4
    q, k, v = rnd((1, 2, hd), 9), rnd((1, 1, hd), 10), rnd((1, 1, hd), 11)
    # one key: the output is its value, for every head of the group
    o = P.attention(q, k, v, 0.5, [0])
    assert torch.allclose(o[0, 0], v[0, 0]) and torch.allclose(o[0, 1], v[0, 0])
    # equal scores: the mean of the visible values
    T = 6
    kk, vv = torch.zeros(T, 1, hd), rnd((T, 1, hd), 12)
    o = P.attention(rnd((1, 1, hd), 13), kk, vv, 1.0, [3])
    assert torch.allclose(o[0, 0], vv[:4, 0].mean(0), atol=1e-6)
    # a window of 2 sees keys p-1 and p only
    o = P.attention(rnd((1, 1, hd), 13), kk, vv, 1.0, [3], window=2)
    assert torch.allclose(o[0, 0], vv[2:4, 0].mean(0), atol=1e-6)


def test_attention_gqa_is_mha_with_repeated_kv():
    """crates/synaptix-models/llm/common/src/model.rs:2569-2579: kv heads repeated g times, head h -> h // g."""
    S, nh, nkv, hd = 7, 6, 2, 8
    q, k, v = rnd((S, nh, hd), 14), rnd((S, nkv, hd), 15), rnd((S, nkv, hd), 16)
    a = P.attention(q, k, v, 0.3, list(range(S)))
    b = P.attention(q, k.repeat_interleave(3, 1), v.repeat_interleave(3, 1), 0.3, list(range(S)))
    assert torch.allclose(a, b, atol=1e-6)


def test_attention_decode_shape_of_the_reference():
    """(b,nh,nkv,Tq,Tkv,d) = (1,4,2,8,200,64), a chunk of 8 queries at the end of 200 keys:
    q_pos = Tkv - Tq + i (crates/synaptix-kernels-cuda/tests/cuda_flash_decode.rs:32-90,185-240)."""
    nh, nkv, Tq, T, hd = 4, 2, 8, 200, 64
    q, k, v = rnd((Tq, nh, hd), 17), rnd((T, nkv, hd), 18), rnd((T, nkv, hd), 19)
    got = P.attention(q, k, v, 1 / 8.0, [T - Tq + i for i in range(Tq)])
    # the host reference of that test, restated directly
    for i in (0, 7):
        for h in (0, 3):
            qp = T - Tq + i
            s = (k[:qp + 1, h // 2] @ q[i, h]) / 8.0
            want = torch.softmax(s, 0) @ v[:qp + 1, h // 2]
            assert torch.allclose(got[i, h], want, atol=1e-5)


# ----------------------------------------------------------------------------- feed-forward
def test_swiglu():
    z = rnd((20,), 20)
    assert torch.allclose(P.silu(z), z * torch.sigmoid(z), atol=1e-6)
    H, I = 6, 10
    h, wg, wu, wd = rnd((3, H), 21), rnd((I, H), 22), rnd((I, H), 23), rnd((H, I), 24)
    want = (torch.nn.functional.silu(h @ wg.T) * (h @ wu.T)) @ wd.T
    assert torch.allclose(P.swiglu_mlp(h, wg, wu, wd), want, atol=1e-5)
    assert not torch.allclose(P.swiglu_mlp(h, wu, wg, wd), want, atol=1e-3)    # gate and up are not symmetric


# ----------------------------------------------------------------------------- whole model
@pytest.mark.parametrize("name", ["A", "B"])
def test_zeroed_projections_leave_embedding_norm_head(name):
    """o_proj = down_proj = 0: x passes through, logits = RMSNorm(E[id]) . W_out^T: one line that
    checks embedding, final norm, tied or separate output."""
    m = plain_model(name)
    w = dict(m.w)
    for n in list(w):
        if n.endswith("o_proj.weight") or n.endswith("down_proj.weight"):
            w[n] = torch.zeros_like(w[n])
    z = P.PlainQwen3(m.cfg, w)
    ids = random_tokens(m.cfg["vocab_size"], 6, 1)
    E = w["model.embed_tokens.weight"]
    out = E if m.cfg["tie_word_embeddings"] else w["lm_head.weight"]
    want = P.rms_norm(E[ids], w["model.norm.weight"], m.eps) @ out.T
    assert torch.allclose(z.forward(ids), want, atol=1e-6)


@pytest.mark.parametrize("name", ["A", "B"])
def test_causality_and_prefix(name):
    m = plain_model(name)
    ids = random_tokens(m.cfg["vocab_size"], 12, 2)
    full = m.forward(ids)
    assert torch.allclose(m.forward(ids[:7]), full[:7], atol=1e-5)
    other = ids[:7] + random_tokens(m.cfg["vocab_size"], 5, 3)
    assert torch.allclose(m.forward(other)[:7], full[:7], atol=1e-5)


class NormAfterRotation(P.PlainQwen3):
    """The mistake that the invariant below is there to catch: q and k rotated first, normed after."""

    def attention_block(self, l, xn, positions, rope_offset=0):
        p = f"model.layers.{l}.self_attn."
        S = xn.shape[0]
        q = (xn @ self.w[p + "q_proj.weight"].T).view(S, self.nh, self.hd)
        k = (xn @ self.w[p + "k_proj.weight"].T).view(S, self.nkv, self.hd)
        v = (xn @ self.w[p + "v_proj.weight"].T).view(S, self.nkv, self.hd)
        turned = [t + rope_offset for t in positions]
        cos, sin = self.tables(max(turned) + 1)
        q = P.rms_norm(P.apply_rope(q, cos, sin, turned), self.w[p + "q_norm.weight"], self.eps)
        k = P.rms_norm(P.apply_rope(k, cos, sin, turned), self.w[p + "k_norm.weight"], self.eps)
        o = P.attention(q, k, v, self.scale, positions)
        return o.reshape(S, self.nh * self.hd) @ self.w[p + "o_proj.weight"].T


def _uneven_gains(m):
    """Weights of `m` whose q/k gains differ between the two halves of a head (the partners of a rotation)."""
    w = dict(m.w)
    hd = m.hd
    for l in range(m.L):
        for n, lo, hi in (("q_norm", 0.5, 2.0), ("k_norm", 1.5, 0.7)):
            g = torch.cat([torch.full((hd // 2,), lo), torch.full((hd - hd // 2,), hi)])
            w[f"model.layers.{l}.self_attn.{n}.weight"] = g * (1 + 0.05 * rnd((hd,), 40 + l))
    return w


@pytest.mark.parametrize("name", ["A", "B"])
def test_logits_depend_on_distances_only_which_puts_the_qk_norm_before_the_rotation(name):
    """Moving every position by the same amount changes no logit: the rotation is the last thing
    that happens to q and k (crates/synaptix-models/llm/common/src/model.rs:1715-1734).  A gain
    applied after the rotation scales the two partners of a rotated pair differently, and the
    score of (m, n) is then no function of m - n: the variant that norms after rotating fails
    the same check, so the check can tell the two orders apart."""
    m = plain_model(name)
    w = _uneven_gains(m)
    ids = random_tokens(m.cfg["vocab_size"], 9, 4)
    good = P.PlainQwen3(m.cfg, w, dtype=F64)
    good.table_dtype = F64                      # exact angles: what is left is the invariant itself
    base = good.forward(ids)
    for shift in (1, 37, 200):
        assert (good.forward(ids, rope_offset=shift) - base).abs().max() < 1e-9
    bad = NormAfterRotation(m.cfg, w, dtype=F64)
    bad.table_dtype = F64
    assert (bad.forward(ids, rope_offset=37) - bad.forward(ids)).abs().max() > 1e-4
    assert (bad.forward(ids) - base).abs().max() > 1e-4


def test_qk_norm_takes_the_layers_eps_and_its_own_gains(monkeypatch):
    """crates/synaptix-models/llm/qwen3/src/config.rs:89-125: one eps for every norm of the model.
    Config B has eps 1e-5; with activations so small that eps decides the norm's result, another
    eps for q and k alone changes the logits; every call of the norm gets the configured value;
    q_norm and k_norm are two tensors, not one."""
    m = plain_model("B")
    ids = random_tokens(1000, 5, 4)
    seen = []
    real = P.rms_norm

    def spy(x, w, eps):
        seen.append((x.shape[-1], eps))
        return real(x, w, eps)

    monkeypatch.setattr(P, "rms_norm", spy)
    base = m.forward(ids)
    assert {e for _, e in seen} == {1e-5} and any(d == m.hd for d, _ in seen) and any(d == 128 for d, _ in seen)
    # tiny q and k: mean square ~ 1e-10, so the result is x / sqrt(eps) and eps shows in full
    w = dict(m.w)
    for l in range(m.L):
        for n in ("q_proj", "k_proj"):
            w[f"model.layers.{l}.self_attn.{n}.weight"] = m.w[f"model.layers.{l}.self_attn.{n}.weight"] * 1e-4
    tiny = P.PlainQwen3(m.cfg, w)

    def other_eps_for_heads(x, w_, eps):
        return real(x, w_, 1e-6 if x.shape[-1] == m.hd else eps)

    a = tiny.forward(ids)
    monkeypatch.setattr(P, "rms_norm", other_eps_for_heads)
    b = tiny.forward(ids)
    monkeypatch.setattr(P, "rms_norm", real)
    assert (a - b).abs().max() > 1e-6
    w = dict(m.w)
    qn, kn = "model.layers.0.self_attn.q_norm.weight", "model.layers.0.self_attn.k_norm.weight"
    w[qn], w[kn] = m.w[kn], m.w[qn]
    assert (P.PlainQwen3(m.cfg, w).forward(ids) - base).abs().max() > 1e-5


def test_swiglu_vector_of_the_reference():
    """crates/synaptix-ops/tests/ffn.rs:24-55: x = [1,-1,.5,2], gate/up [2,4], down [4,2]; the
    activation sits on the gate product.  Expected values worked out by hand below."""
    x = torch.tensor([[1.0, -1.0, 0.5, 2.0]])
    wg = torch.tensor([0.1, 0.2, 0.3, 0.4, -0.1, 0.0, 0.5, -0.5]).view(2, 4)
    wu = torch.tensor([0.5, -0.5, 0.25, 0.0, 0.1, 0.2, -0.3, 0.4]).view(2, 4)
    wd = torch.tensor([1.0, -1.0, 0.5, 0.25, 0.0, 0.5, -0.5, 1.0]).view(4, 2)
    gate = [0.1 - 0.2 + 0.15 + 0.8, -0.1 + 0.25 - 1.0]              # 0.85, -0.85
    up = [0.5 + 0.5 + 0.125, 0.1 - 0.2 - 0.15 + 0.8]                # 1.125, 0.55
    hid = [g / (1 + math.exp(-g)) * u for g, u in zip(gate, up)]
    want = [hid[0] - hid[1], 0.5 * hid[0] + 0.25 * hid[1], 0.5 * hid[1], -0.5 * hid[0] + hid[1]]
    got = P.swiglu_mlp(x, wg, wu, wd)[0]
    assert torch.allclose(got, torch.tensor(want), atol=1e-6)
    # the activation on the other product gives other numbers
    other = [u / (1 + math.exp(-u)) * g for g, u in zip(gate, up)]
    assert abs(other[0] - hid[0]) > 1e-2


def test_float64_agrees_with_float32():
    m32 = plain_model("A")
    m64 = P.PlainQwen3(m32.cfg, m32.w, dtype=F64)
    ids = random_tokens(512, 20, 5)
    assert (m32.forward(ids).double() - m64.forward(ids)).abs().max() < 2e-5


# ----------------------------------------------------------------------------- sampling
def test_philox_known_answer():
    """crates/synaptix-ops/src/rng.rs:162-167: zero key, zero counter."""
    assert P.philox4x32([0, 0, 0, 0], [0, 0]) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    r = P.PlainPhilox(0)
    assert [r.next_u32() for _ in range(4)] == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert r.counter == [1, 0, 0, 0]


def test_greedy_takes_the_last_of_equal_maxima():
    assert P.greedy(torch.tensor([1.0, 3.0, 2.0, 3.0, 0.0])) == 3
    assert P.greedy(torch.tensor([5.0, 3.0])) == 0


def test_repetition_vector_of_the_reference():
    """crates/synaptix-infer/src/sampling/repetition.rs:88-97: penalty 2, last_n 2 -> [1,1,.5,.5]."""
    got = P.repetition_penalty(torch.ones(4), [0, 1, 2, 3], 2.0, 2)
    assert got.tolist() == [1.0, 1.0, 0.5, 0.5]
    neg = P.repetition_penalty(torch.tensor([-1.0, 1.0]), [0, 0], 2.0, 0)
    assert neg.tolist() == [-4.0, 1.0]                     # once for each occurrence
    pf = P.presence_frequency(torch.zeros(3), [1, 1, 2], 0.5, 0.25, 0)
    assert pf.tolist() == [0.0, -1.0, -0.75]


def test_filters():
    x = torch.tensor([1.0, 4.0, 2.0, 3.0])
    assert P.top_k(x, 2).tolist() == [-math.inf, 4.0, -math.inf, 3.0]
    # probabilities ~ [.03,.64,.09,.24]: p = .7 keeps 4.0 (sum before 0 <= .7) and 3.0 (.64 <= .7), drops the rest
    assert P.top_p(x, 0.7).tolist() == [-math.inf, 4.0, -math.inf, 3.0]
    assert P.min_p(x, 0.2).tolist() == [-math.inf, 4.0, -math.inf, 3.0]    # .24/.64 > .2 > .09/.64
    assert P.multinomial(x, 0.0) == 0 and P.multinomial(x, 0.999999) == 3 and P.multinomial(x, 1.0) == 3


def test_small_temperature_is_greedy():
    x = rnd((50,), 30)
    rng = P.PlainPhilox(3)
    assert all(P.sample(x, [], rng, temperature=1e-3) == int(x.argmax()) for _ in range(5))
