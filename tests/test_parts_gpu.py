"""Each part alone against the plain implementation's function for it, and the framework's
openness: a toy mixer with a state of its own, defined here, is registered, built and stepped
without a change to the package."""
import math

import pytest
import torch

import plain_qwen3 as P
from helpers import assert_logits_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16


@pytest.fixture(scope="module", autouse=True)
def need_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


def tol(dtype):
    return dict(atol=1e-5, rtol=1e-5) if dtype == F32 else dict(atol=3e-2, rtol=2e-2)


def one_sequence_ctx(cache, slot, n_new, dtype):
    """A StepContext for one sequence that brings n_new tokens, as the engine builds it."""
    import numpy as np
    from synaptix_amd.engine.batch import StepLayout, StepContext, ScratchPool, fill_host_buffer
    past = cache.length(slot)
    cache.reserve(slot, n_new)
    layout = StepLayout(n_new, 1, 0, [cache.table_width(g, [slot]) for g in range(len(cache.groups))])
    host = np.zeros(layout.total, dtype=np.int32)
    fill_host_buffer(layout, host, cache, [slot], np.zeros(n_new, dtype=np.int32), [n_new], [])
    return StepContext(layout, torch.from_numpy(host).to(DEV), dtype, [slot], [past], [n_new], ScratchPool(DEV))


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_rms_norm_part(dtype):
    from synaptix_amd.parts import RmsNorm
    n = RmsNorm("g", 72, 1e-5)
    gain = 1 + 0.1 * rnd((72,), 1)
    n.load(lambda name: gain.to(dtype).to(DEV))
    resid, delta = rnd((5, 72), 2), rnd((5, 72), 3)
    r = resid.to(DEV)
    out = n.add_apply(r, delta.to(DEV), dtype)
    want = P.rms_norm(resid + delta, gain.to(dtype).float(), 1e-5)
    assert torch.allclose(out.float().cpu(), want, **tol(dtype))
    assert torch.allclose(r.cpu(), resid + delta, atol=1e-6)
    x = rnd((4, 3, 72), 4).to(dtype)
    assert torch.allclose(n.apply(x.to(DEV)).float().cpu(), P.rms_norm(x.float(), gain.to(dtype).float(), 1e-5),
                          **tol(dtype))


def test_rotary_part_tables():
    from synaptix_amd.parts import RotaryHalfSplit
    r = RotaryHalfSplit(1e6, 32, 300)
    cos, sin = r.tables(DEV)
    c, s = P.rope_tables(32, 300, 1e6)
    assert cos.shape == (300, 16)
    # two float32 power routines may differ by one ulp in a frequency; times a position of up to
    # 300 that is an angle error of 300 * 2^-23 ~ 4e-5
    assert torch.allclose(cos.cpu(), c, atol=1e-4) and torch.allclose(sin.cpu(), s, atol=1e-4)
    assert torch.equal(cos[0].cpu(), torch.ones(16)) and torch.equal(sin[0].cpu(), torch.zeros(16))
    assert torch.allclose(cos[:4].cpu(), c[:4], atol=1e-6)
    with pytest.raises(ValueError):
        RotaryHalfSplit(1e4, 15, 10)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("nh,nkv,hd,rot,qk_norm,window", [(4, 2, 16, 16, True, None), (6, 2, 48, 32, False, None),
                                                           (3, 1, 32, 32, True, 20), (4, 4, 64, 0, True, None)])
def test_attention_part_alone(dtype, nh, nkv, hd, rot, qk_norm, window):
    """GqaAttention with its own sizes and options (partial rotation, no q/k norm, a window, no
    rotation at all), a prompt and then single tokens, against the plain functions."""
    from synaptix_amd.parts import GqaAttention, RotaryHalfSplit, NoPosition, as_delta
    from synaptix_amd.cache import SequenceCache
    H, S, eps = 40, 90, 1e-5
    pos = RotaryHalfSplit(1e4, rot, 256) if rot else NoPosition()
    att = GqaAttention("a.", H, nh, nkv, hd, position=pos, qk_norm_eps=eps if qk_norm else None, window=window)
    w = {n: (rnd(s.shape, 10 + i, 0.3) if s.kind != "gain" else 1 + 0.1 * rnd(s.shape, 10 + i)).to(dtype)
         for i, (n, s) in enumerate(att.tensor_specs().items())}
    att.load(lambda name: w[name].to(DEV))
    x = rnd((S, H), 30).to(dtype)

    # the plain statement of the same part
    xf = x.float()
    q = (xf @ w["a.q_proj.weight"].float().T).view(S, nh, hd)
    k = (xf @ w["a.k_proj.weight"].float().T).view(S, nkv, hd)
    v = (xf @ w["a.v_proj.weight"].float().T).view(S, nkv, hd)
    if qk_norm:
        q, k = P.rms_norm(q, w["a.q_norm.weight"].float(), eps), P.rms_norm(k, w["a.k_norm.weight"].float(), eps)
    if rot:
        cos, sin = P.rope_tables(rot, S, 1e4)
        q = torch.cat([P.apply_rope(q[..., :rot], cos, sin, range(S)), q[..., rot:]], -1)
        k = torch.cat([P.apply_rope(k[..., :rot], cos, sin, range(S)), k[..., rot:]], -1)
    want = P.attention(q, k, v, 1 / math.sqrt(hd), list(range(S)), window=window).reshape(S, nh * hd) \
        @ w["a.o_proj.weight"].float().T

    cache = SequenceCache([att.cache_need()], 256, 2, dtype, DEV)
    slot = cache.acquire()
    got = []
    for lo, hi in [(0, 70)] + [(i, i + 1) for i in range(70, S)]:
        ctx = one_sequence_ctx(cache, slot, hi - lo, dtype)
        got.append(as_delta(att.forward(x[lo:hi].to(DEV), ctx, cache.layer_view(0))))   # few rows: the product may come unrun
        cache.commit(slot, hi - lo)
    got = torch.cat(got).cpu()
    assert got.dtype == F32
    err = (got - want).abs().max()
    assert err <= (2e-4 if dtype == F32 else 4e-2) * max(1.0, float(want.abs().max())), float(err)


@pytest.mark.parametrize("dtype,inter", [(F32, 200), (BF16, 200), (BF16, 2048)])
def test_gated_mlp_part_alone(dtype, inter):
    """With 2048 intermediate values and few rows the last product comes as partial sums over
    slices of K, which the norm that follows adds up."""
    from synaptix_amd.parts import GatedMlp, RmsNorm, as_delta
    ff = GatedMlp("m.", 56, inter)
    w = {n: rnd(s.shape, 40 + i, 0.2).to(dtype) for i, (n, s) in enumerate(ff.tensor_specs().items())}
    ff.load(lambda name: w[name].to(DEV))
    x = rnd((9, 56), 50).to(dtype)
    got = as_delta(ff.forward(x.to(DEV), None))
    if inter >= 2048 and dtype == BF16:
        assert got.dim() == 3 and got.shape[0] > 1
    if got.dim() == 3:
        norm = RmsNorm("g", 56, 1e-6)
        norm.load(lambda name: torch.ones(56, device=DEV))
        resid = torch.zeros((9, 56), device=DEV)
        norm.add_apply(resid, got, torch.float32)           # resid = 0 + sum of the slices
        got = resid
    got = got.cpu()
    want = P.swiglu_mlp(x.float(), w["m.gate_proj.weight"].float(), w["m.up_proj.weight"].float(),
                        w["m.down_proj.weight"].float())
    # bf16: the activations silu(g) * u are rounded once (2^-9 relative) before the last product
    assert (got - want).abs().max() <= (2e-5 if dtype == F32 else 2e-2) * float(want.abs().max())
    with pytest.raises(ValueError, match="gelu"):
        GatedMlp("m.", 8, 8, "gelu")


# ----------------------------------------------------------------------------- a toy architecture
def test_toy_mixer_with_state_registers_builds_and_steps(tmp_path):
    """A decayed running mean of the inputs as 'mixer': state [hidden] for each sequence, zero at
    the start.  It is defined, registered under a name of its own, built from its own config.json,
    loaded and stepped here; whole prompts and single tokens must agree, which they only do if the
    state is kept for each slot, zeroed when a slot is taken, and carried across steps."""
    from dataclasses import dataclass, asdict
    import json
    from synaptix_amd import register_architecture, Engine
    from synaptix_amd.models import DecoderModel, LayerRun, TokenEmbedding, OutputHead
    from synaptix_amd.parts import Mixer, StateNeed, RmsNorm, GatedMlp, PreNormBlock, GqaAttention, RotaryHalfSplit
    from synaptix_amd.weights import TensorSpec, save_file, RandomSource

    class RunningMean(Mixer):
        def __init__(self, prefix, hidden, decay):
            self.prefix, self.hidden, self.decay = prefix, hidden, decay
            self.scale = None

        def tensor_specs(self):
            return {self.prefix + "scale": TensorSpec((self.hidden,), "gain")}

        def load(self, get):
            self.scale = get(self.prefix + "scale").float()

        def cache_need(self):
            return StateNeed((self.hidden,), torch.float32)

        def forward(self, h, ctx, cache, owner=True):
            out = torch.empty(h.shape, dtype=torch.float32, device=h.device)
            start = 0
            for slot, n in zip(ctx.slots, ctx.new_counts):       # tokens of a sequence in order
                s = cache.state[slot]
                for t in range(start, start + n):
                    s.mul_(self.decay).add_(h[t].float())
                    out[t] = s * self.scale
                start += n
            return out

    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int = 97
        hidden_size: int = 48
        intermediate_size: int = 80
        decay: float = 0.5
        max_position_embeddings: int = 128

        @classmethod
        def from_dict(cls, d):
            return cls(**{k: d[k] for k in cls.__dataclass_fields__ if k in d})

        def to_dict(self):
            return {**asdict(self), "architectures": ["ToyRunningMean"]}

    def build(cfg, max_positions=None):
        emb = TokenEmbedding("emb", cfg.vocab_size, cfg.hidden_size)
        rope = RotaryHalfSplit(1e4, 16, cfg.max_position_embeddings)
        blocks = [
            PreNormBlock(RmsNorm("l0.n1", cfg.hidden_size, 1e-5), RunningMean("l0.mix.", cfg.hidden_size, cfg.decay),
                         RmsNorm("l0.n2", cfg.hidden_size, 1e-5), GatedMlp("l0.ff.", cfg.hidden_size, cfg.intermediate_size)),
            PreNormBlock(RmsNorm("l1.n1", cfg.hidden_size, 1e-5),
                         GqaAttention("l1.att.", cfg.hidden_size, 3, 1, 16, position=rope),
                         RmsNorm("l1.n2", cfg.hidden_size, 1e-5), GatedMlp("l1.ff.", cfg.hidden_size, cfg.intermediate_size)),
        ]
        # the stateful block runs twice, each run with a state of its own; the attention block runs once
        schedule = [LayerRun(0, 0), LayerRun(1, 1), LayerRun(0, 2)]
        return DecoderModel(cfg, emb, blocks, schedule, RmsNorm("norm", cfg.hidden_size, 1e-5),
                            OutputHead("head", cfg.vocab_size, cfg.hidden_size))

    register_architecture("ToyRunningMean", ToyConfig, build)
    cfg = ToyConfig()
    model = build(cfg)
    src = RandomSource(model.tensor_specs(), 5, std=0.2)
    save_file({n: src.tensor(n) for n in src.names()}, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))

    for dtype in ("float32", "bfloat16"):
        eng = Engine.load(str(tmp_path), dtype=dtype, max_tokens=512, max_slots=3)
        assert [type(n).__name__ for n in eng.model.cache_needs()] == ["StateNeed", "KvNeed", "StateNeed"]
        toks = [[5, 9, 33, 2, 70, 11, 8], [90, 1, 4]]
        a, b = eng.acquire(), eng.acquire()
        whole = eng.step([(a, toks[0]), (b, toks[1])], want="all")
        eng.release(a), eng.release(b)
        b2, a2 = eng.acquire(), eng.acquire()                   # the same slots again, the other way round
        got = {0: [], 1: []}
        lg = eng.step([(a2, toks[0][:2]), (b2, toks[1][:1])], want="all")
        got[0].append(lg[:2]), got[1].append(lg[2:])
        for i in range(2, 7):
            ent = [(a2, [toks[0][i]])] + ([(b2, [toks[1][i - 1]])] if i - 1 < 3 else [])
            lg = eng.step(ent, want="last")
            got[0].append(lg[:1])
            if len(ent) > 1:
                got[1].append(lg[1:])
        tolerance = 1e-4 if dtype == "float32" else 5e-2
        assert (torch.cat(got[0]) - whole[:7]).abs().max() <= tolerance
        assert (torch.cat(got[1]) - whole[7:]).abs().max() <= tolerance
        # back to a snapshot: the running state is restored with the length, and the same tokens
        # give the same logits again
        eng.release(a2), eng.release(b2)
        c = eng.acquire()
        eng.step([(c, toks[0][:4])], want=None)
        snap = eng.snapshot(c)
        first = eng.step([(c, toks[0][4:])], want="all")
        eng.restore(snap)
        assert eng.length(c) == 4
        again = eng.step([(c, toks[0][4:])], want="all")
        assert torch.equal(first, again)
        assert (first - whole[4:7]).abs().max() <= tolerance


def test_toy_mixer_with_state_is_replayed_from_graphs(tmp_path):
    """The same running mean, written so that its steps may be captured: it finds the state rows of the step's
    sequences through the device arrays of the step (StateLayerView.token_rows), never through slots on the host,
    and says so (capturable).  Prompt steps and decode steps then come from graphs like any other model's: the
    runs that precede a capture must leave no trace in the states (the first replay is checked), every replay
    must advance them once (later replays are checked), padding rows must keep to the spare row (a fourth
    sequence that takes no part in the replayed steps goes on afterwards with the right state), and a slot that
    is used again starts from zero."""
    from dataclasses import dataclass, asdict
    import json
    from synaptix_amd import register_architecture, Engine
    from synaptix_amd.models import DecoderModel, LayerRun, TokenEmbedding, OutputHead
    from synaptix_amd.parts import Mixer, StateNeed, RmsNorm, GatedMlp, PreNormBlock, GqaAttention, RotaryHalfSplit
    from synaptix_amd.weights import TensorSpec, save_file, RandomSource

    class RunningMeanOnDevice(Mixer):
        capturable = True

        def __init__(self, prefix, hidden, decay):
            self.prefix, self.hidden, self.decay = prefix, hidden, decay
            self.scale = None

        def tensor_specs(self):
            return {self.prefix + "scale": TensorSpec((self.hidden,), "gain")}

        def load(self, get):
            self.scale = get(self.prefix + "scale").float()

        def cache_need(self):
            return StateNeed((self.hidden,), torch.float32)

        def forward(self, h, ctx, cache, owner=True):
            rows = cache.token_rows(ctx)                        # on the device; padding tokens: the spare row
            out = torch.empty(h.shape, dtype=torch.float32, device=h.device)
            for t in range(h.shape[0]):                         # tokens of a sequence lie in order
                r = rows[t:t + 1]
                s = cache.state.index_select(0, r) * self.decay + h[t:t + 1].float()
                cache.state.index_copy_(0, r, s)
                out[t:t + 1] = s * self.scale
            return out

    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int = 97
        hidden_size: int = 48
        intermediate_size: int = 80
        decay: float = 0.5
        max_position_embeddings: int = 128

        @classmethod
        def from_dict(cls, d):
            return cls(**{k: d[k] for k in cls.__dataclass_fields__ if k in d})

        def to_dict(self):
            return {**asdict(self), "architectures": ["ToyRunningMeanOnDevice"]}

    def build(cfg, max_positions=None):
        emb = TokenEmbedding("emb", cfg.vocab_size, cfg.hidden_size)
        rope = RotaryHalfSplit(1e4, 16, cfg.max_position_embeddings)
        blocks = [
            PreNormBlock(RmsNorm("l0.n1", cfg.hidden_size, 1e-5), RunningMeanOnDevice("l0.mix.", cfg.hidden_size, cfg.decay),
                         RmsNorm("l0.n2", cfg.hidden_size, 1e-5), GatedMlp("l0.ff.", cfg.hidden_size, cfg.intermediate_size)),
            PreNormBlock(RmsNorm("l1.n1", cfg.hidden_size, 1e-5),
                         GqaAttention("l1.att.", cfg.hidden_size, 3, 1, 16, position=rope),
                         RmsNorm("l1.n2", cfg.hidden_size, 1e-5), GatedMlp("l1.ff.", cfg.hidden_size, cfg.intermediate_size)),
        ]
        schedule = [LayerRun(0, 0), LayerRun(1, 1), LayerRun(0, 2)]
        return DecoderModel(cfg, emb, blocks, schedule, RmsNorm("norm", cfg.hidden_size, 1e-5),
                            OutputHead("head", cfg.vocab_size, cfg.hidden_size))

    register_architecture("ToyRunningMeanOnDevice", ToyConfig, build)
    cfg = ToyConfig()
    src = RandomSource(build(cfg).tensor_specs(), 5, std=0.2)
    save_file({n: src.tensor(n) for n in src.names()}, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))

    seqs = [[5, 9, 33, 2, 70, 11, 8, 41, 3], [90, 1, 4, 17, 60, 2, 2], [7, 7, 52, 13, 88, 21, 30, 6], [64, 12, 95, 3, 18, 44]]
    heads = [5, 3, 4, 3]                                         # tokens that come as prompts
    for dtype in ("float32", "bfloat16"):
        eng = Engine.load(str(tmp_path), dtype=dtype, max_tokens=1024, max_slots=4)
        assert eng.has_states and eng.graph_ok
        tolerance = 1e-4 if dtype == "float32" else 5e-2
        # what every position should give: each sequence whole and alone, launched one by one
        eng.prompt_graphs = False
        whole = []
        for toks in seqs:
            s = eng.acquire()
            whole.append(eng.step([(s, toks)], want="all").clone())
            eng.release(s)
        eng.prompt_graphs = True
        for round_ in range(2):                                  # the second round takes the same slots again
            slots = [eng.acquire() for _ in seqs]
            # the fourth sequence starts before the others and waits while their steps are replayed
            lg = eng.step([(slots[3], seqs[3][:heads[3]])], want="last")
            assert (lg - whole[3][heads[3] - 1:heads[3]]).abs().max() <= tolerance
            live = [0, 1, 2]
            lg = eng.step([(slots[i], seqs[i][:heads[i]]) for i in live], want="last")     # bfloat16: a captured prompt step
            for j, i in enumerate(live):
                assert (lg[j] - whole[i][heads[i] - 1]).abs().max() <= tolerance, (dtype, round_, "prompt", i)
            assert (dtype == "bfloat16") == any(k[0] == "prompt" for k in eng._runners)
            runner = eng.decode_runner(3, 64)                    # 4 rows: one of padding
            d = 0
            while live:
                _, lg = runner.step([slots[i] for i in live], [seqs[i][heads[i] + d] for i in live])
                for j, i in enumerate(live):
                    assert (lg[j] - whole[i][heads[i] + d]).abs().max() <= tolerance, (dtype, round_, "decode", d, i)
                d += 1
                live = [i for i in live if heads[i] + d < len(seqs[i])]      # shorter sequences end earlier
            lg = eng.step([(slots[3], seqs[3][heads[3]:])], want="all")
            assert (lg - whole[3][heads[3]:]).abs().max() <= tolerance, (dtype, round_, "the sequence that waited")
            for s in slots:
                eng.release(s)
        eng.cache.check()


# ----------------------------------------------------------------------------- more toy parts
def test_toy_position_encoding_plugs_into_attention():
    """Another position encoding, defined here: angles that grow linearly with the index of the
    pair, on the first 8 of 16 dims.  The mixer only asks its position part for tables."""
    from synaptix_amd.parts import GqaAttention, Position, as_delta
    from synaptix_amd.cache import SequenceCache

    class LinearFrequencies(Position):
        capacity = 128

        def __init__(self, rotary_dim):
            self.rotary_dim = rotary_dim

        def host(self):
            ang = torch.arange(self.capacity, dtype=F32)[:, None] * (0.05 * (1 + torch.arange(self.rotary_dim // 2, dtype=F32)))[None, :]
            return torch.cos(ang), torch.sin(ang)

        def tables(self, device):
            c, s = self.host()
            return c.to(device), s.to(device)

    H, S, nh, nkv, hd, rot = 24, 40, 2, 1, 16, 8
    pos = LinearFrequencies(rot)
    for dtype in (F32, BF16):
        att = GqaAttention("a.", H, nh, nkv, hd, position=pos)
        w = {n: rnd(s.shape, 40 + i, 0.4).to(dtype) for i, (n, s) in enumerate(att.tensor_specs().items())}
        att.load(lambda name: w[name].to(DEV))
        x = rnd((S, H), 50).to(dtype)
        xf = x.float()
        q = (xf @ w["a.q_proj.weight"].float().T).view(S, nh, hd)
        k = (xf @ w["a.k_proj.weight"].float().T).view(S, nkv, hd)
        v = (xf @ w["a.v_proj.weight"].float().T).view(S, nkv, hd)
        cos, sin = pos.host()
        q = torch.cat([P.apply_rope(q[..., :rot], cos, sin, range(S)), q[..., rot:]], -1)
        k = torch.cat([P.apply_rope(k[..., :rot], cos, sin, range(S)), k[..., rot:]], -1)
        want = P.attention(q, k, v, 1 / math.sqrt(hd), list(range(S))).reshape(S, nh * hd) @ w["a.o_proj.weight"].float().T
        cache = SequenceCache([att.cache_need()], 128, 1, dtype, DEV)
        slot = cache.acquire()
        got = []
        for lo, hi in [(0, 33)] + [(i, i + 1) for i in range(33, S)]:
            ctx = one_sequence_ctx(cache, slot, hi - lo, dtype)
            d = as_delta(att.forward(x[lo:hi].to(DEV), ctx, cache.layer_view(0)))
            got.append(d.sum(0) if d.dim() == 3 else d)
            cache.commit(slot, hi - lo)
        err = (torch.cat(got).cpu() - want).abs().max()
        assert err <= (2e-4 if dtype == F32 else 4e-2) * max(1.0, float(want.abs().max())), float(err)


@pytest.mark.parametrize("softcap", [None, 1.5])
def test_toy_position_scheme_that_acts_on_the_scores(softcap):
    """A position scheme that is no rotation, defined here: a penalty on the scores that grows with the distance
    between query and key, one slope a head (the reference's linear bias, crates/synaptix-ops/src/pos/alibi.rs:5-66),
    with and without a soft cap on the scores.  The mixer asks its position part for the slopes and hands them to
    whichever attention kernel runs: the prompt (whole and in a second chunk), then single tokens, in both types.
    The slopes are steep enough that dropping them changes the result by far more than the tolerance."""
    from synaptix_amd.parts import GqaAttention, Position, as_delta
    from synaptix_amd.cache import SequenceCache

    class DistancePenalty(Position):
        def score_slopes(self, n_heads, device):
            return torch.tensor([2.0 ** (-(h + 1) * 8.0 / n_heads) for h in range(n_heads)], dtype=F32).to(device)

    H, S, nh, nkv, hd = 24, 150, 4, 2, 32
    pos = DistancePenalty()
    slopes = pos.score_slopes(nh, "cpu")
    for dtype in (F32, BF16):
        att = GqaAttention("a.", H, nh, nkv, hd, position=pos, score_softcap=softcap)
        w = {n: rnd(s_.shape, 60 + i, 0.5).to(dtype) for i, (n, s_) in enumerate(att.tensor_specs().items())}
        att.load(lambda name: w[name].to(DEV))
        x = rnd((S, H), 70).to(dtype)
        xf = x.float()
        q = (xf @ w["a.q_proj.weight"].float().T).view(S, nh, hd)
        k = (xf @ w["a.k_proj.weight"].float().T).view(S, nkv, hd)
        v = (xf @ w["a.v_proj.weight"].float().T).view(S, nkv, hd)

        def dense(with_terms):
            out = torch.empty(S, nh, hd)
            dist = (torch.arange(S)[:, None] - torch.arange(S)[None, :]).float()
            for h in range(nh):
                sc = (q[:, h] @ k[:, h // (nh // nkv)].T) / math.sqrt(hd)
                if with_terms:
                    if softcap:
                        sc = softcap * torch.tanh(sc / softcap)
                    sc = sc - slopes[h] * dist
                sc = sc.masked_fill(dist < 0, float("-inf"))
                out[:, h] = torch.softmax(sc, -1) @ v[:, h // (nh // nkv)]
            return out.reshape(S, nh * hd) @ w["a.o_proj.weight"].float().T

        want = dense(True)
        assert float((want - dense(False)).abs().max()) > 0.2 * float(want.abs().max())      # the terms matter
        cache = SequenceCache([att.cache_need()], 256, 1, dtype, DEV)
        slot = cache.acquire()
        got = []
        for lo, hi in [(0, 70), (70, 140)] + [(i, i + 1) for i in range(140, S)]:
            ctx = one_sequence_ctx(cache, slot, hi - lo, dtype)
            d = as_delta(att.forward(x[lo:hi].to(DEV), ctx, cache.layer_view(0)))
            got.append(d.sum(0) if d.dim() == 3 else d)
            cache.commit(slot, hi - lo)
        err = (torch.cat(got).cpu() - want).abs().max()
        assert err <= (2e-4 if dtype == F32 else 4e-2) * max(1.0, float(want.abs().max())), float(err)


def test_toy_feed_forward_with_routing_registers_builds_and_steps(tmp_path):
    """A feed-forward with routing, defined here: a 32-bit router picks one of three gated MLPs
    for each token and scales its output by the router's probability.  Registered, built from its
    own config.json, loaded and stepped without a change to the package; the logits must equal a
    plain statement of the same model and must not depend on the cut of the tokens into steps."""
    from dataclasses import dataclass, asdict
    import json
    from synaptix_amd import register_architecture, Engine
    from synaptix_amd.models import DecoderModel, LayerRun, TokenEmbedding, OutputHead
    from synaptix_amd.parts import FeedForward, RmsNorm, GatedMlp, PreNormBlock, GqaAttention, RotaryHalfSplit
    from synaptix_amd.parts.linear import linear
    from synaptix_amd.weights import TensorSpec, save_file, RandomSource

    class TopOneExperts(FeedForward):
        def __init__(self, prefix, hidden, inter, n_experts):
            self.prefix, self.hidden = prefix, hidden
            self.experts = [GatedMlp(f"{prefix}e{e}.", hidden, inter) for e in range(n_experts)]
            self.router = None

        def tensor_specs(self):
            specs = {self.prefix + "router.weight": TensorSpec((len(self.experts), self.hidden))}
            for e in self.experts:
                specs.update(e.tensor_specs())
            return specs

        def load(self, get):
            self.router = get(self.prefix + "router.weight")
            for e in self.experts:
                e.load(get)

        def forward(self, h, ctx):
            logits = linear(h, self.router, torch.float32)                 # 32-bit router
            prob, pick = torch.softmax(logits, -1).max(-1)
            out = torch.zeros((h.shape[0], self.hidden), dtype=torch.float32, device=h.device)
            for e, expert in enumerate(self.experts):
                rows = torch.nonzero(pick == e).flatten()
                if rows.numel():
                    d = expert.forward(h[rows].contiguous(), ctx)
                    d = d.sum(0) if d.dim() == 3 else d
                    out[rows] = d * prob[rows, None]
            return out

    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int = 61
        hidden_size: int = 32
        intermediate_size: int = 56
        n_experts: int = 3
        max_position_embeddings: int = 64

        @classmethod
        def from_dict(cls, d):
            return cls(**{k: d[k] for k in cls.__dataclass_fields__ if k in d})

        def to_dict(self):
            return {**asdict(self), "architectures": ["ToyRouted"]}

    def build(cfg, max_positions=None):
        H = cfg.hidden_size
        rope = RotaryHalfSplit(1e4, 16, cfg.max_position_embeddings)
        blocks = [PreNormBlock(RmsNorm(f"l{l}.n1", H, 1e-5), GqaAttention(f"l{l}.att.", H, 2, 1, 16, position=rope),
                               RmsNorm(f"l{l}.n2", H, 1e-5),
                               TopOneExperts(f"l{l}.ff.", H, cfg.intermediate_size, cfg.n_experts)) for l in range(2)]
        return DecoderModel(cfg, TokenEmbedding("emb", cfg.vocab_size, H), blocks, [LayerRun(0, 0), LayerRun(1, 1)],
                            RmsNorm("norm", H, 1e-5), OutputHead("head", cfg.vocab_size, H))

    register_architecture("ToyRouted", ToyConfig, build)
    cfg = ToyConfig()
    src = RandomSource(build(cfg).tensor_specs(), 9, std=0.3)
    # the routers are stored in 32-bit and stay so in both modes; everything else is bf16
    tensors = {n: (src.tensor(n).float() if "router" in n else src.tensor(n)) for n in src.names()}
    save_file(tensors, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))

    def plain(ids):
        t = {n: v.float() for n, v in tensors.items()}
        x = t["emb"][ids]
        S, cos_sin = len(ids), P.rope_tables(16, len(ids), 1e4)
        picks = []
        for l in range(2):
            xn = P.rms_norm(x, t[f"l{l}.n1"], 1e-5)
            q = (xn @ t[f"l{l}.att.q_proj.weight"].T).view(S, 2, 16)
            k = (xn @ t[f"l{l}.att.k_proj.weight"].T).view(S, 1, 16)
            v = (xn @ t[f"l{l}.att.v_proj.weight"].T).view(S, 1, 16)
            q, k = P.apply_rope(q, *cos_sin, range(S)), P.apply_rope(k, *cos_sin, range(S))
            x = x + P.attention(q, k, v, 0.25, list(range(S))).reshape(S, 32) @ t[f"l{l}.att.o_proj.weight"].T
            hn = P.rms_norm(x, t[f"l{l}.n2"], 1e-5)
            prob, pick = torch.softmax(hn @ t[f"l{l}.ff.router.weight"].T, -1).max(-1)
            picks.append(pick)
            d = torch.stack([P.swiglu_mlp(hn[i:i + 1], t[f"l{l}.ff.e{int(e)}.gate_proj.weight"],
                                          t[f"l{l}.ff.e{int(e)}.up_proj.weight"],
                                          t[f"l{l}.ff.e{int(e)}.down_proj.weight"])[0] for i, e in enumerate(pick)])
            x = x + d * prob[:, None]
        return P.rms_norm(x, t["norm"], 1e-5) @ t["head"].T, picks

    ids = [3, 17, 44, 9, 60, 21, 5, 38, 12, 50, 7]
    want, picks = plain(ids)
    assert len(set(int(p) for p in torch.cat(picks))) == 3          # every expert is used
    eng = Engine.load(str(tmp_path), dtype="float32", max_tokens=128, max_slots=2)
    a = eng.acquire()
    whole = eng.step([(a, ids)], want="all").cpu()
    assert (whole - want).abs().max() <= 2e-4 * max(1.0, float(want.abs().max()))
    eng.release(a)
    a = eng.acquire()
    cut = [eng.step([(a, ids[:4])], want="all")] + [eng.step([(a, [t])], want="last") for t in ids[4:]]
    assert (torch.cat(cut).cpu() - whole).abs().max() <= 1e-4

    eng = Engine.load(str(tmp_path), dtype="bfloat16", max_tokens=128, max_slots=2)
    assert eng.model.blocks[0].feed_forward.router.dtype == torch.float32 and eng.model.blocks[0].feed_forward.experts[0].w_down.dtype == BF16
    # the routed part waits for the device (it looks at which rows took which expert) and does not say that it may be
    # captured: every step of this model is launched one by one, also the short prompt steps that are replayed elsewhere
    assert not eng.graph_ok
    a = eng.acquire()
    whole16 = eng.step([(a, ids)], want="all").cpu()
    eng.release(a)
    a = eng.acquire()
    last16 = eng.step([(a, ids)], want="last").cpu()
    assert not eng._runners and torch.equal(last16, whole16[-1:])
    eng.release(a)
    a = eng.acquire()
    cut = [eng.step([(a, ids[:4])], want="all")] + [eng.step([(a, [t])], want="last") for t in ids[4:]]
    assert (torch.cat(cut).cpu() - whole16).abs().max() <= 5e-2 * max(1.0, float(whole16.abs().max()))


def test_toy_block_arrangement_and_toy_norm_register_build_and_step(tmp_path):
    """Another arrangement of a layer and another norm, both defined here: a block in which mixer and feed-forward
    read the same normed rows and their sums are added together (x <- x + mixer(n(x)) + ff(n(x))), beside a pre-norm
    block in the same model; and a norm that takes the mean away before it scales (with a gain and a bias).  The
    block keeps to the interface of blocks (the delta it is handed is added by its norm, the delta it returns is added by
    whoever runs next), the norm to that of norms (add_apply with and without rows).  Registered, built from its own
    config.json, loaded and stepped without a change to the package; whole prompts, pieces and single tokens agree
    with a plain statement of the same model in both types."""
    from dataclasses import dataclass, asdict
    import json
    from synaptix_amd import register_architecture, Engine
    from synaptix_amd.models import DecoderModel, LayerRun, TokenEmbedding, OutputHead
    from synaptix_amd.parts import Part, Block, RmsNorm, GatedMlp, PreNormBlock, GqaAttention, RotaryHalfSplit, as_delta
    from synaptix_amd.weights import TensorSpec, save_file, RandomSource

    class CenteredNorm(Part):
        """y = gain * (x - mean) / sqrt(var + eps) + bias, in 32-bit; the residual sum in front of it as the package's norms have it."""
        def __init__(self, name, dim, eps):
            self.name, self.dim, self.eps = name, dim, eps

        def tensor_specs(self):
            return {self.name + ".gain": TensorSpec((self.dim,), "gain"), self.name + ".bias": TensorSpec((self.dim,))}

        def load(self, get):
            self.gain, self.bias = get(self.name + ".gain").float(), get(self.name + ".bias").float()

        def add_apply(self, resid, delta, out_dtype, rows=None):
            delta = as_delta(delta)
            if delta is not None and delta.dim() == 3:
                delta = delta.sum(0)
            if rows is None:
                if delta is not None:
                    resid += delta
                x = resid
            else:
                x = resid[rows.long()] + (0 if delta is None else delta[rows.long()])
            c = x - x.mean(-1, keepdim=True)
            return (self.gain * c * torch.rsqrt(c.square().mean(-1, keepdim=True) + self.eps) + self.bias).to(out_dtype)

    class ParallelBlock(Block):
        def __init__(self, norm, mixer, feed_forward):
            self.norm, self.mixer, self.feed_forward = norm, mixer, feed_forward

        def _parts(self):
            return (self.norm, self.mixer, self.feed_forward)

        def tensor_specs(self):
            return {k: v for p in self._parts() for k, v in p.tensor_specs().items()}

        def load(self, get):
            for p in self._parts():
                p.load(get)

        def forward(self, resid, pending, ctx, cache, owner=True):
            h = self.norm.add_apply(resid, pending, ctx.act_dtype)              # the delta of the layer before is added here
            both = [as_delta(self.mixer.forward(h, ctx, cache, owner)), as_delta(self.feed_forward.forward(h, ctx))]
            both = [d.sum(0) if d.dim() == 3 else d for d in both]                # (products may come as partial sums)
            return both[0] + both[1]                                              # added by the norm that runs next

    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int = 83
        hidden_size: int = 48
        intermediate_size: int = 64
        max_position_embeddings: int = 128

        @classmethod
        def from_dict(cls, d):
            return cls(**{k: d[k] for k in cls.__dataclass_fields__ if k in d})

        def to_dict(self):
            return {**asdict(self), "architectures": ["ToyParallel"]}

    def build(cfg, max_positions=None):
        H = cfg.hidden_size
        rope = RotaryHalfSplit(1e4, 16, cfg.max_position_embeddings)
        blocks = [ParallelBlock(CenteredNorm("l0.n", H, 1e-5), GqaAttention("l0.att.", H, 3, 1, 16, position=rope),
                                GatedMlp("l0.ff.", H, cfg.intermediate_size)),
                  PreNormBlock(RmsNorm("l1.n1", H, 1e-5), GqaAttention("l1.att.", H, 3, 3, 16, position=rope),
                               CenteredNorm("l1.n2", H, 1e-5), GatedMlp("l1.ff.", H, cfg.intermediate_size)),
                  ParallelBlock(RmsNorm("l2.n", H, 1e-5), GqaAttention("l2.att.", H, 3, 1, 16, position=rope),
                                GatedMlp("l2.ff.", H, cfg.intermediate_size))]
        return DecoderModel(cfg, TokenEmbedding("emb", cfg.vocab_size, H), blocks, [LayerRun(l, l) for l in range(3)],
                            CenteredNorm("norm", H, 1e-5), OutputHead("head", cfg.vocab_size, H))

    register_architecture("ToyParallel", ToyConfig, build)
    cfg = ToyConfig()
    src = RandomSource(build(cfg).tensor_specs(), 21, std=0.25)
    tensors = {n: src.tensor(n) for n in src.names()}
    save_file(tensors, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))

    def plain(ids):
        t = {n: v.float() for n, v in tensors.items()}
        S, cos_sin = len(ids), P.rope_tables(16, len(ids), 1e4)

        def centered(x, name):
            c = x - x.mean(-1, keepdim=True)
            return t[name + ".gain"] * c * torch.rsqrt(c.square().mean(-1, keepdim=True) + 1e-5) + t[name + ".bias"]

        def attend(xn, pre, nkv):
            q = (xn @ t[pre + "q_proj.weight"].T).view(S, 3, 16)
            k = (xn @ t[pre + "k_proj.weight"].T).view(S, nkv, 16)
            v = (xn @ t[pre + "v_proj.weight"].T).view(S, nkv, 16)
            q, k = P.apply_rope(q, *cos_sin, range(S)), P.apply_rope(k, *cos_sin, range(S))
            return P.attention(q, k, v, 0.25, list(range(S))).reshape(S, 48) @ t[pre + "o_proj.weight"].T

        def mlp(xn, pre):
            return P.swiglu_mlp(xn, t[pre + "gate_proj.weight"], t[pre + "up_proj.weight"], t[pre + "down_proj.weight"])

        x = t["emb"][ids]
        n = centered(x, "l0.n")
        x = x + attend(n, "l0.att.", 1) + mlp(n, "l0.ff.")
        x = x + attend(P.rms_norm(x, t["l1.n1"], 1e-5), "l1.att.", 3)
        x = x + mlp(centered(x, "l1.n2"), "l1.ff.")
        n = P.rms_norm(x, t["l2.n"], 1e-5)
        x = x + attend(n, "l2.att.", 1) + mlp(n, "l2.ff.")
        return centered(x, "norm") @ t["head"].T

    ids = [3, 17, 44, 9, 60, 21, 5, 38, 12, 50, 7, 80, 2]
    want = plain(ids)
    for dtype, tol in (("float32", 3e-4), ("bfloat16", 6e-2)):
        eng = Engine.load(str(tmp_path), dtype=dtype, max_tokens=256, max_slots=2)
        assert not eng.graph_ok                        # parts from elsewhere: every step is launched one by one
        a = eng.acquire()
        whole = eng.step([(a, ids)], want="all").cpu()
        assert (whole - want).abs().max() <= tol * max(1.0, float(want.abs().max())), dtype
        last = eng.step([(eng.acquire(), ids)], want=[[4, 12]]).cpu()             # wanted rows: the last norm with rows
        assert (last - whole[[4, 12]]).abs().max() <= (1e-5 if dtype == "float32" else 2e-2)
        eng.release(a)
        a = eng.acquire()
        cut = [eng.step([(a, ids[:5])], want="all"), eng.step([(a, ids[5:9])], want="all")]
        cut += [eng.step([(a, [tok])], want="last") for tok in ids[9:]]
        assert (torch.cat(cut).cpu() - whole).abs().max() <= (1e-4 if dtype == "float32" else 5e-2 * max(1.0, float(whole.abs().max())))
