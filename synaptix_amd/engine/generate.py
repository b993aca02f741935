"""The generation loop above the step function.

For one sequence it behaves as the reference's loop
(crates/synaptix-models/llm/common/src/generate.rs:237-302): the first token comes from the
prompt's last logits; then, while fewer than max_new_tokens are out, stop if the last token is
a stop token (the stop token stays in the output), else run one token and sample the next.  At
least one token is produced, also for max_new_tokens == 0.

What the reference does not have: batches.  Requests are taken in order; as many as fit (slots,
pages for prompt and new tokens, max_batch) start together with all prompts in one step; then
every step brings one token for each sequence that is still alive; a sequence that ends gives
its slot back at once and leaves the step's table; when the batch is over the next requests
start in the slots that came free.  The bookkeeping follows the shape of the reference's
generic engine (crates/synaptix-infer/src/session.rs:72-125, batch.rs:22-33, engine.rs:165-185).
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field

import torch

from ..cache import pages_for
from ..sampling import GenerationConfig, SequenceSampler, sample_batch


@dataclass
class GenerationOutput:
    tokens: list
    finish_reason: str          # "stop" (a stop token), "length" (max_new_tokens), "capacity", "cancelled"
    prompt_tokens: int


@dataclass
class GenerationStats:
    """prompt_tokens / new_tokens / prefill_ms / decode_ms as generate.rs:59-65, over all requests."""
    prompt_tokens: int = 0
    new_tokens: int = 0
    prefill_ms: float = 0.0
    decode_ms: float = 0.0
    decode_steps: int = 0
    batches: int = 0
    step_ms: list = field(default_factory=list)

    @property
    def decode_tokens_per_s(self) -> float:
        """Tokens that decode steps produced per second of decode time (the first token of each
        sequence belongs to the prefill: crates/synaptix-cli/src/commands/bench.rs:84-88)."""
        n = self.new_tokens - self.batches_first_tokens
        return n / (self.decode_ms / 1000.0) if self.decode_ms > 0 else 0.0

    batches_first_tokens: int = 0


def plan_batch(waiting: list, prompt_lens: list, max_new: list, free_slots: int, free_pages,
               max_batch: int | None, capacity: int | None, held: dict | None = None, group_need=None) -> list:
    """Which of the waiting requests (indices, in order) start together now.

    A request needs a slot and pages for its prompt and all tokens it may produce, so that a
    batch never runs out of pages half way.  Requests are not reordered: the first that does not
    fit ends the batch.  A request that can never fit raises ValueError.
    held: {request: tokens it keeps in a slot of its own}: such a request needs no slot and only the pages
    beyond those that its kept tokens lie in.
    free_pages: one number, or one for each group of cache layers together with group_need(request, total tokens)
    -> the pages of each group that the request can hold at once (groups that keep a window need fewer).
    """
    many = isinstance(free_pages, (list, tuple))
    free = list(free_pages) if many else [free_pages]
    chosen, pages, slots = [], [0] * len(free), 0
    for r in waiting:
        total = prompt_lens[r] + max(max_new[r], 1)
        if capacity is not None:
            total = min(total, capacity)
        need = list(group_need(r, total)) if (many and group_need is not None) else [pages_for(total)] * len(free)
        own_slot = held is not None and r in held
        if own_slot:
            need = [max(0, n - pages_for(held[r])) for n in need]
        if max_batch is not None and len(chosen) >= max_batch:
            break
        if (not own_slot and slots >= free_slots) or any(p + n > f for p, n, f in zip(pages, need, free)):
            break
        chosen.append(r)
        pages = [p + n for p, n in zip(pages, need)]
        slots += 0 if own_slot else 1
    if not chosen and waiting:
        r = waiting[0]
        raise ValueError(f"request {r} ({prompt_lens[r]} prompt tokens + {max_new[r]} new) does not fit the cache "
                         f"({min(free)} pages of 64 tokens and {free_slots} slots are free)")
    return chosen


def graph_step(engine, live, longest):
    """One decode step through the captured graph; sampling runs inside it when every sequence
    samples greedily or by temperature alone, else on the graph's logits."""
    runner = engine.decode_runner(len(live), longest)
    slots, last = [s.slot for s in live], [s.out[-1] for s in live]
    if all(s.config.plain for s in live):
        temps = [float(s.config.temperature) for s in live]
        if all(t <= 0.0 for t in temps):
            tokens, _ = runner.step(slots, last)
        else:
            u = [s.sampler.rng.next_multinomial_uniform() if t > 0.0 else 0.0 for s, t in zip(live, temps)]
            tokens, _ = runner.step(slots, last, temps, u)
        for s, t in zip(live, tokens):
            s.sampler.commit(t)
        return tokens
    _, logits = runner.step(slots, last)
    return sample_batch(logits, [s.sampler for s in live])


class _Live:
    def __init__(self, request, slot, prompt, config, sampler, kept=0, owned=True):
        self.request, self.slot, self.prompt, self.config, self.sampler = request, slot, prompt, config, sampler
        self.kept, self.owned = kept, owned     # prompt tokens that the slot already holds; whether the loop gives the slot back
        self.out = []
        self.stop = config.stop_set()
        self.finish = None


def generate(engine, prompts, config=None, on_token=None, max_batch: int | None = None, use_graph: bool = True,
             resume: dict | None = None):
    """prompts: a list of token-id lists.  config: one GenerationConfig for all, or one each
    (with one for all, request i draws from the stream of seed + i).  on_token(request, token)
    -> bool: False cancels that request.  use_graph: decode steps are replayed from a captured
    graph where the engine allows it (the reference's --no-graph switches the same thing off).
    resume: {request: slot}: the caller holds that slot, and the tokens it caches are the beginning of the
    request's prompt (the caller vouches for that, as in the reference's generate_streaming_resume,
    crates/synaptix-models/llm/common/src/generate.rs:233-250): min(cached, prompt - 1) of them are kept, only
    the rest of the prompt is run, new tokens go into the same slot, and the slot stays with the caller.
    Returns ([GenerationOutput], GenerationStats)."""
    resume = dict(resume or {})
    for r, slot in resume.items():
        if not (0 <= r < len(prompts)):
            raise ValueError(f"resume names request {r}; there are {len(prompts)}")
        engine.length(slot)                       # raises for a slot that is not held
    if len(set(resume.values())) != len(resume):
        raise ValueError("resume: two requests name the same slot")
    if config is None:
        config = GenerationConfig()
    shared = isinstance(config, GenerationConfig)
    configs = [config] * len(prompts) if shared else list(config)
    if len(configs) != len(prompts):
        raise ValueError("one GenerationConfig for all requests, or one for each")
    for i, p in enumerate(prompts):
        if len(p) == 0:
            raise ValueError(f"request {i}: empty prompt")            # generate.rs:225-227
        cap = engine.max_positions
        if cap is not None and len(p) > cap:
            raise ValueError(f"request {i}: prompt of {len(p)} tokens exceeds the position range {cap}")
    outputs = [None] * len(prompts)
    stats = GenerationStats()
    waiting = list(range(len(prompts)))
    lens = [len(p) for p in prompts]
    max_new = [c.max_new_tokens for c in configs]

    def limit(seq: _Live):
        caps = [c for c in (engine.max_positions, seq.config.max_seq) if c is not None]
        return min(caps) if caps else None

    def kept_tokens(r):
        return min(engine.length(resume[r]), lens[r] - 1)

    def group_need(r, total):
        step = configs[r].prefill_batch if configs[r].prefill_batch > 0 else lens[r]
        return engine.cache.pages_for_sequence(total, min(step, lens[r]))

    while waiting:
        free_pages = [g.pool.free_pages for g in engine.cache.groups] if engine.cache.groups else [1 << 30]
        batch = plan_batch(waiting, lens, max_new, engine.cache.free_slots, free_pages, max_batch,
                           engine.max_positions, held={r: kept_tokens(r) for r in waiting if r in resume},
                           group_need=group_need if engine.cache.groups else None)
        waiting = waiting[len(batch):]
        stats.batches += 1
        live = []
        for r in batch:
            seed = configs[r].seed + r if shared else configs[r].seed
            sampler = SequenceSampler(configs[r], prompts[r], seed)
            if r in resume:
                kept = kept_tokens(r)
                if kept < engine.length(resume[r]):
                    if getattr(engine, "has_states", False):     # a running state cannot be rewound by a length
                        raise ValueError(f"request {r}: its slot holds {engine.length(resume[r])} tokens and a state of "
                                         f"fixed size; restore a snapshot taken at {kept} tokens or fewer first")
                    engine.cache.truncate(resume[r], kept)
                live.append(_Live(r, resume[r], list(prompts[r]), configs[r], sampler, kept=kept, owned=False))
            else:
                live.append(_Live(r, engine.acquire(), list(prompts[r]), configs[r], sampler))
        try:
            # ---- the prompts, in one step (or in chunks of prefill_batch tokens each)
            t0 = time.perf_counter()
            fed = [s.kept for s in live]
            logits_rows = {}
            while True:
                entries, who = [], []
                for i, s in enumerate(live):
                    if fed[i] < len(s.prompt):
                        n = len(s.prompt) - fed[i]
                        if s.config.prefill_batch > 0:
                            n = min(n, s.config.prefill_batch)
                        entries.append((s.slot, s.prompt[fed[i]:fed[i] + n]))
                        who.append(i)
                        fed[i] += n
                if not entries:
                    break
                lg = engine.step(entries, want="last")
                for j, i in enumerate(who):
                    if fed[i] == len(live[i].prompt):
                        logits_rows[i] = lg[j]
            first = torch.stack([logits_rows[i] for i in range(len(live))]).contiguous()
            tokens = sample_batch(first, [s.sampler for s in live])
            stats.prefill_ms += (time.perf_counter() - t0) * 1000.0
            stats.prompt_tokens += sum(len(s.prompt) for s in live)
            stats.batches_first_tokens += len(live)
            for s, t in zip(live, tokens):
                s.out.append(t)
                if on_token is not None and on_token(s.request, t) is False:
                    s.finish = "cancelled"

            # ---- one token a step for each live sequence
            graph = use_graph and getattr(engine, "graph_ok", False)
            longest = max(len(s.prompt) + max(s.config.max_new_tokens, 1) for s in live)
            t1 = time.perf_counter()
            while True:
                still = []
                for s in live:
                    if s.finish is None:
                        cap = limit(s)
                        if len(s.out) >= s.config.max_new_tokens:
                            s.finish = "length"
                        elif s.out[-1] in s.stop:
                            s.finish = "stop"
                        elif cap is not None and len(s.prompt) + len(s.out) > cap:
                            s.finish = "capacity"      # the last token has no place left in the cache
                    if s.finish is None:
                        still.append(s)
                    else:
                        outputs[s.request] = GenerationOutput(s.out, s.finish, len(s.prompt))
                        if s.owned:
                            engine.release(s.slot)       # at once: the slot is free for the next batch
                        s.slot = None
                live = still
                if not live:
                    break
                ts = time.perf_counter()
                if graph:
                    tokens = graph_step(engine, live, longest)
                else:
                    lg = engine.step([(s.slot, [s.out[-1]]) for s in live], want="last")
                    tokens = sample_batch(lg, [s.sampler for s in live])
                stats.step_ms.append((time.perf_counter() - ts) * 1000.0)
                stats.decode_steps += 1
                for s, t in zip(live, tokens):
                    s.out.append(t)
                    if on_token is not None and on_token(s.request, t) is False:
                        s.finish = "cancelled"
            stats.decode_ms += (time.perf_counter() - t1) * 1000.0
        finally:
            for s in live:
                if s.slot is not None and s.owned:
                    engine.release(s.slot)
    stats.new_tokens = sum(len(o.tokens) for o in outputs if o is not None)
    return outputs, stats
