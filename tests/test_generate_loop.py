"""The generation loop's decisions, with a counter in place of a model (no weights, no GPU):
argmax = (token + 1) mod V, the pattern of crates/synaptix-infer/tests/engine_ops.rs:19-37."""
import pytest
import torch

import cpu_kernels
from synaptix_amd.cache import SequenceCache
from synaptix_amd.engine.generate import generate, plan_batch, GenerationConfig
from synaptix_amd.parts import KvNeed
from synaptix_amd.sampling import Philox4x32, SequenceSampler, filter_batch
import plain_qwen3 as P

V = 50


class CounterEngine:
    """Has the engine's surface; the 'model' answers (last token + 1) mod V with certainty."""

    def __init__(self, max_tokens=64 * 8, max_slots=4, max_positions=None):
        self.cache = SequenceCache([KvNeed(1, 16)], max_tokens, max_slots, torch.float32, "cpu",
                                   max_positions=max_positions)
        self.max_positions = max_positions
        self.steps = []

    def acquire(self):
        return self.cache.acquire()

    def release(self, s):
        self.cache.release(s)

    def step(self, entries, want="last"):
        assert want == "last"
        self.steps.append([(s, len(t)) for s, t in entries])
        rows = []
        for s, toks in entries:
            self.cache.reserve(s, len(toks))
            self.cache.commit(s, len(toks))
            row = torch.zeros(V)
            row[(toks[-1] + 1) % V] = 10.0
            rows.append(row)
        return torch.stack(rows)


@pytest.fixture(autouse=True)
def kernels_on_cpu(monkeypatch):
    cpu_kernels.install(monkeypatch)


def test_stop_token_is_part_of_the_output_and_ends_the_sequence():
    eng = CounterEngine()
    outs, st = generate(eng, [[3]], GenerationConfig(max_new_tokens=20, eos_token_id=7))
    assert outs[0].tokens == [4, 5, 6, 7] and outs[0].finish_reason == "stop"
    assert st.new_tokens == 4 and st.prompt_tokens == 1 and st.decode_steps == 3
    outs, _ = generate(eng, [[3]], GenerationConfig(max_new_tokens=20, eos_token_ids=(9, 5), eos_token_id=30))
    assert outs[0].tokens == [4, 5]
    outs, _ = generate(eng, [[6]], GenerationConfig(max_new_tokens=3, eos_token_id=7))
    assert outs[0].tokens == [7]                       # the first token already stops


def test_length_limit_and_at_least_one_token():
    eng = CounterEngine()
    outs, _ = generate(eng, [[0]], GenerationConfig(max_new_tokens=5))
    assert outs[0].tokens == [1, 2, 3, 4, 5] and outs[0].finish_reason == "length"
    outs, _ = generate(eng, [[0]], GenerationConfig(max_new_tokens=0))
    assert outs[0].tokens == [1]                       # as the reference: no check before the first token
    with pytest.raises(ValueError, match="empty prompt"):
        generate(eng, [[1], []], GenerationConfig())


def test_unequal_batch_shorter_ones_leave_and_slots_come_back():
    eng = CounterEngine(max_slots=3)
    prompts = [[10], [20, 21, 22], [40, 41]]
    cfgs = [GenerationConfig(max_new_tokens=2), GenerationConfig(max_new_tokens=6, eos_token_id=25),
            GenerationConfig(max_new_tokens=4)]
    outs, st = generate(eng, prompts, cfgs)
    assert [o.tokens for o in outs] == [[11, 12], [23, 24, 25], [42, 43, 44, 45]]
    assert [o.finish_reason for o in outs] == ["length", "stop", "length"]
    # first step: all prompts together with their own lengths; then the batch shrinks
    assert eng.steps[0] == [(0, 1), (1, 3), (2, 2)]
    assert [len(s) for s in eng.steps[1:]] == [3, 2, 1]
    assert eng.cache.free_slots == 3
    eng.cache.check()


def test_more_requests_than_slots_run_batch_after_batch():
    eng = CounterEngine(max_slots=2)
    prompts = [[i] for i in range(5)]
    outs, st = generate(eng, prompts, GenerationConfig(max_new_tokens=3))
    assert [o.tokens for o in outs] == [[i + 1, i + 2, i + 3] for i in range(5)]
    assert st.batches == 3
    firsts = [s for s in eng.steps if all(n == 1 for _, n in s)]
    used = {slot for s in eng.steps for slot, _ in s}
    assert used == {0, 1}                              # the same two slots, again and again
    eng.cache.check()
    assert eng.cache.groups[0].pool.free_pages == 8


def test_max_batch_and_page_budget():
    assert plan_batch([0, 1, 2], [10, 10, 10], [5, 5, 5], free_slots=8, free_pages=100, max_batch=2, capacity=None) == [0, 1]
    # 100 + 100 tokens need 4 pages each
    assert plan_batch([0, 1, 2], [100] * 3, [100] * 3, free_slots=8, free_pages=9, max_batch=None, capacity=None) == [0, 1]
    assert plan_batch([3, 4], [0, 0, 0, 64, 1], [0, 0, 0, 1, 1], 8, 2, None, None) == [3]      # 65 tokens: two pages
    assert plan_batch([0], [500], [500], 1, 4, None, capacity=256) == [0]                        # capped by the range
    with pytest.raises(ValueError, match="does not fit"):
        plan_batch([0], [1000], [10], 4, 3, None, None)
    eng = CounterEngine(max_tokens=64 * 2, max_slots=4)
    outs, st = generate(eng, [[1] * 60, [2] * 60, [3]], GenerationConfig(max_new_tokens=3))
    assert st.batches == 2 and outs[2].tokens == [4, 5, 6]


def test_batches_are_planned_for_each_group_of_cache_layers():
    """A group that keeps a window has a small pool of its own (with a promise about the longest step); the plan counts
    each group's pages against that group's pool, so long prompts in chunks start together although the small pool
    could never hold them whole."""
    assert plan_batch([0, 1], [300, 300], [20, 20], free_slots=4, free_pages=[40, 8], max_batch=None, capacity=None,
                      group_need=lambda r, total: [5, 4]) == [0, 1]
    assert plan_batch([0, 1], [300, 300], [20, 20], free_slots=4, free_pages=[40, 7], max_batch=None, capacity=None,
                      group_need=lambda r, total: [5, 4]) == [0]
    eng = CounterEngine(max_tokens=64 * 40, max_slots=2)
    eng.cache = SequenceCache([KvNeed(1, 16), KvNeed(1, 16, window=70)], 64 * 40, 2, torch.float32, "cpu", max_step_tokens=64)
    assert eng.cache.groups[1].n_pages == 8
    prompts = [[(3 * i) % V for i in range(300)], [(5 * i + 1) % V for i in range(290)]]
    outs, st = generate(eng, prompts, GenerationConfig(max_new_tokens=20, prefill_batch=64))
    assert st.batches == 1 and all(len(o.tokens) == 20 for o in outs)
    assert eng.steps[0] == [(0, 64), (1, 64)]
    eng.cache.check()
    assert eng.cache.groups[1].pool.free_pages == 8 and eng.cache.groups[0].pool.free_pages == 40


def test_capacity_ends_a_sequence():
    eng = CounterEngine(max_positions=6)
    outs, _ = generate(eng, [[1, 2, 3, 4]], GenerationConfig(max_new_tokens=50))
    # positions 0..5: four prompt tokens, then two generated tokens can be fed; the third has no place
    assert outs[0].tokens == [5, 6, 7] and outs[0].finish_reason == "capacity"
    outs, _ = generate(eng, [[1, 2]], GenerationConfig(max_new_tokens=50, max_seq=4))
    assert outs[0].tokens == [3, 4, 5] and outs[0].finish_reason == "capacity"
    with pytest.raises(ValueError, match="position range"):
        generate(eng, [[0] * 7], GenerationConfig())


def test_streaming_callback_can_cancel():
    eng = CounterEngine()
    seen = []

    def on_token(req, tok):
        seen.append((req, tok))
        return not (req == 0 and tok == 3)

    outs, _ = generate(eng, [[0], [10]], GenerationConfig(max_new_tokens=5), on_token=on_token)
    assert outs[0].tokens == [1, 2, 3] and outs[0].finish_reason == "cancelled"
    assert outs[1].tokens == [11, 12, 13, 14, 15]
    assert (1, 15) in seen and (0, 4) not in seen


def test_chunked_prompt():
    eng = CounterEngine()
    outs, _ = generate(eng, [[1, 2, 3, 4, 5], [9]], GenerationConfig(max_new_tokens=2, prefill_batch=2))
    assert [o.tokens for o in outs] == [[6, 7], [10, 11]]
    assert eng.steps[:3] == [[(0, 2), (1, 1)], [(0, 2)], [(0, 1)]]


def test_a_failing_step_gives_the_slots_back():
    eng = CounterEngine(max_tokens=128, max_slots=2)

    def boom(entries, want="last"):
        raise RuntimeError("boom")

    eng.step = boom
    with pytest.raises(RuntimeError):
        generate(eng, [[1]], GenerationConfig())
    assert eng.cache.free_slots == 2


# ----------------------------------------------------------------------------- sampling pieces
def test_philox_matches_the_known_answer_and_the_plain_stream():
    r = Philox4x32(0)
    assert [r.next_u32() for _ in range(4)] == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    a, b = Philox4x32(2 ** 40 + 5), P.PlainPhilox(2 ** 40 + 5)
    assert [a.next_u32() for _ in range(9)] == [b.next_u32() for _ in range(9)]
    assert Philox4x32(1).next_multinomial_uniform() == P.uniform_for_multinomial(P.PlainPhilox(1))
    u = Philox4x32(3).next_f32_uniform()
    assert 0.0 <= u < 1.0


def test_options_reach_the_filters_as_the_plain_ones_apply_them(monkeypatch):
    """What a GenerationConfig and a context become on their way to the filter kernel (here its stand-in on the
    CPU): which tokens the penalties see (the last repeat_last_n), which options are on, row by row of a batch
    whose rows have different options."""
    import cpu_kernels
    cpu_kernels.install(monkeypatch)
    g = torch.Generator().manual_seed(0)
    for trial in range(10):
        rows, cfgs, ctxs = [], [], []
        for r in range(3):
            t = 3 * trial + r
            rows.append(torch.randn(200, generator=g) * 3)
            ctxs.append(torch.randint(0, 200, (30,), generator=g).tolist())
            cfgs.append(GenerationConfig(temperature=[0.8, 1.0, 0.0][r], top_k=[0, 17][t % 2], top_p=[1.0, 0.85][(t // 2) % 2],
                                         min_p=[0.0, 0.02][(t // 4) % 2], repetition_penalty=[1.2, 1.0][r % 2],
                                         presence_penalty=0.3, frequency_penalty=[0.1, 0.0][t % 2], repeat_last_n=[0, 10][t % 2]))
        samplers = [SequenceSampler(c, ids) for c, ids in zip(cfgs, ctxs)]
        got = filter_batch(torch.stack(rows), cfgs, [s.penalty_ids() for s in samplers])
        for r, (x, cfg, ids) in enumerate(zip(rows, cfgs, ctxs)):
            want = x.clone()
            if cfg.repetition_penalty != 1.0:
                want = P.repetition_penalty(want, ids, cfg.repetition_penalty, cfg.repeat_last_n)
            want = P.presence_frequency(want, ids, cfg.presence_penalty, cfg.frequency_penalty, cfg.repeat_last_n)
            if cfg.temperature > 0 and cfg.temperature != 1.0:
                want = want / torch.tensor(cfg.temperature)
            if cfg.top_k:
                want = P.top_k(want, cfg.top_k)
            if cfg.top_p < 1:
                want = P.top_p(want, cfg.top_p)
            if cfg.min_p > 0:
                want = P.min_p(want, cfg.min_p)
            assert torch.equal(torch.isinf(got[r]), torch.isinf(want)), (trial, r)
            keep = ~torch.isinf(want)
            assert torch.allclose(got[r][keep], want[keep], atol=1e-6)
