"""The engine's own logic (packing, page tables, slots, order of layers, generation) with the
stand-in kernels on the CPU, against the plain implementation."""
import pytest
import torch

import cpu_kernels
import scenarios
from helpers import model_folder, CONFIGS
from synaptix_amd import StepError, CacheError, CacheFull


@pytest.fixture(autouse=True)
def kernels_on_cpu(monkeypatch):
    cpu_kernels.install(monkeypatch)


def make_engine(name, dtype, max_tokens, sharp=False, max_slots=None):
    return cpu_kernels.CpuEngine.load(model_folder(name, sharp), dtype=dtype, max_tokens=max_tokens, device="cpu",
                                      max_slots=max_slots)


@pytest.mark.parametrize("name", ["A", "B"])
def test_whole(name):
    scenarios.whole(make_engine, name, "float32")


def test_whole_sharp_attention():
    scenarios.whole(make_engine, "C", "float32", sharp=True)


@pytest.mark.parametrize("name", ["A", "B"])
def test_last_tokens_one_by_one(name):
    scenarios.last_tokens_one_by_one(make_engine, name, "float32", tail=8)


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("B", "bfloat16")])
def test_unequal_batches(name, dtype):
    scenarios.unequal_batches(make_engine, name, dtype, decode=5)


def test_first_tokens():
    scenarios.first_tokens(make_engine, "B", "float32")


def test_decode_beside_a_fresh_prompt_and_prompts_in_chunks():
    scenarios.decode_beside_fresh_prompt(make_engine, "B", "float32")
    scenarios.chunked_prompts(make_engine, "C", "float32", 50, sharp=True)
    scenarios.generation_with_chunked_prompt(make_engine, "A", "float32", n_prompt=150, prefill_batch=64, n_new=3)


def test_greedy_and_sampled_generation():
    scenarios.greedy_generation(make_engine, "A", "float32", n_new=5)
    scenarios.sampled_generation(make_engine, "B", "float32")
    scenarios.generation_with_every_processor(make_engine, "A")


def test_step_errors():
    eng = make_engine("A", "float32", 256, max_slots=2)
    s = eng.acquire()
    with pytest.raises(StepError, match="vocabulary"):
        eng.step([(s, [1, 512])])
    with pytest.raises(StepError, match="vocabulary"):
        eng.step([(s, [-1])])
    with pytest.raises(StepError, match="at least one token"):
        eng.step([(s, [])])
    with pytest.raises(StepError, match="at least one sequence"):
        eng.step([])
    with pytest.raises(StepError, match="twice"):
        eng.step([(s, [1]), (s, [2])])
    with pytest.raises(CacheError, match="not live"):
        eng.step([(1, [1])])
    with pytest.raises(StepError, match="place 3"):
        eng.step([(s, [1, 2, 3])], want=[[3]])
    with pytest.raises(StepError, match="one list of places"):
        eng.step([(s, [1, 2, 3])], want=[[0], [1]])
    assert eng.length(s) == 0                                   # nothing of the above touched the cache
    with pytest.raises(CacheError, match="KV overflow"):
        eng.step([(s, [1] * 257)])                              # max_position_embeddings = 256
    t = eng.acquire()
    eng.step([(s, [1] * 200)])
    with pytest.raises(CacheFull):
        eng.step([(t, [1] * 65)])                               # 4 pages in all; s holds 4... none left
    assert eng.length(t) == 0 and eng.length(s) == 200
    eng.cache.check()


def test_batch_rows_do_not_depend_on_their_neighbours():
    """Permuting a batch permutes its logits bit for bit (no padding, nothing shared between rows)."""
    eng = make_engine("A", "float32", 1024)
    V = CONFIGS["A"]["vocab_size"]
    prompts = [scenarios.random_tokens(V, n, 50 + n) for n in (9, 2, 30)]
    a = [eng.acquire() for _ in prompts]
    x = eng.step(list(zip(a, prompts)), want="last")
    b = [eng.acquire() for _ in prompts]
    y = eng.step(list(zip(b, prompts))[::-1], want="last")
    assert torch.equal(x, y.flip(0))


def test_a_head_size_without_a_kernel_is_refused_when_the_engine_is_made(tmp_path):
    """Head size 24: the bf16 attention kernels take steps of 16; the 32-bit path takes any even size."""
    from synaptix_amd import Qwen3Config, write_random_model
    from helpers import TINY_A
    cfg = Qwen3Config.from_dict(dict(TINY_A, head_dim=24))
    write_random_model(str(tmp_path), cfg, 1)
    with pytest.raises(ValueError, match="steps of 16"):
        cpu_kernels.CpuEngine.load(str(tmp_path), dtype="bfloat16", max_tokens=128, device="cpu")
    eng = cpu_kernels.CpuEngine.load(str(tmp_path), dtype="float32", max_tokens=128, device="cpu")
    s = eng.acquire()
    assert eng.step([(s, [1, 2, 3])], want="last").shape == (1, cfg.vocab_size)


def test_every_weight_is_kept_once():
    """A bf16 matrix whose sizes allow it lies in fragment order and nowhere else; the others in plain rows;
    both are the matrix of the model's folder (the order is a layout, not another model)."""
    from safetensors.torch import load_file
    import os
    eng = make_engine("A", "bfloat16", 256)
    stored = load_file(os.path.join(model_folder("A"), "model.safetensors"))
    mixer, ff = eng.model.blocks[0].mixer, eng.model.blocks[0].feed_forward
    for m in (mixer.w_qkv, mixer.w_o, ff.w_gate_up, ff.w_down, eng.model.head.weight, eng.model.embedding.table):
        assert (m.packed is None) != (m.plain is None)
        N, K = m.shape
        assert (m.packed is not None) == (N % 16 == 0 and K % 32 == 0)
        assert m.nbytes() == N * K * 2
    assert torch.equal(mixer.w_o.rows(), stored["model.layers.0.self_attn.o_proj.weight"])
    assert torch.equal(eng.model.embedding.table.rows(), stored["model.embed_tokens.weight"])
    if CONFIGS["A"].get("tie_word_embeddings"):
        assert eng.model.head.weight is eng.model.embedding.table


def test_generation_that_resumes_a_kept_prefix_equals_a_fresh_one():
    """The reference's prefix_cache_resume_matches_fresh (crates/synaptix-models/llm/qwen3/src/pipeline.rs:395-424): half
    of the prompt is run into a slot beforehand; generation that resumes there runs only the other half and gives
    the fresh run's greedy tokens.  A slot that holds more than the prompt is cut back to prompt - 1 tokens; the
    slot stays with the caller and holds everything that was run."""
    from synaptix_amd.engine.generate import generate, GenerationConfig
    eng = make_engine("C", "float32", 1024, sharp=True)
    V = CONFIGS["C"]["vocab_size"]
    full = scenarios.random_tokens(V, 90, 4)          # crosses a page edge
    other = scenarios.random_tokens(V, 20, 5)
    cfg = GenerationConfig(max_new_tokens=6, temperature=0.0)
    fresh, _ = generate(eng, [full, other], cfg)
    slot = eng.acquire()
    eng.step([(slot, full[:45])], want=None)
    steps = []
    step = eng.step
    eng.step = lambda entries, want="last": (steps.append([(s_, len(t)) for s_, t in entries]), step(entries, want))[1]
    resumed, st = generate(eng, [full, other], cfg, resume={0: slot})
    assert [o.tokens for o in resumed] == [o.tokens for o in fresh]
    assert (slot, 45) in steps[0] and st.prompt_tokens == 110           # only the tail of the resumed prompt was run
    assert eng.length(slot) == 90 + 5                                   # the last token has not been run yet
    # the slot now holds more than the prompt: all but the prompt's last token is kept, one token is run
    steps.clear()
    again, _ = generate(eng, [full], cfg, resume={0: slot})
    assert again[0].tokens == fresh[0].tokens and steps[0] == [(slot, 1)]
    eng.release(slot)
    eng.cache.check()
    assert not eng.cache.live_slots
    with pytest.raises(CacheError):
        generate(eng, [full], cfg, resume={0: slot})                    # a slot that is not held
