"""Options of generation, with the names, meanings and defaults of the reference's
GenerationConfig (crates/synaptix-models/llm/common/src/generate.rs:17-56)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class GenerationConfig:
    max_new_tokens: int = 64
    temperature: float = 0.0            # <= 0: greedy; 1 leaves the logits as they are
    top_k: int = 0                      # 0: off
    top_p: float = 1.0                  # >= 1: off
    min_p: float = 0.0                  # 0: off
    repetition_penalty: float = 1.0     # 1: off
    repeat_last_n: int = 0              # window of the penalties over the context's tail; 0: all of it
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    seed: int = 0
    eos_token_id: Optional[int] = None
    eos_token_ids: tuple = ()
    max_seq: Optional[int] = None       # stop when a sequence holds this many tokens
    prefill_batch: int = 0              # prompt tokens a step for each sequence; 0: the whole prompt

    def stop_set(self) -> frozenset:
        """eos_token_ids and eos_token_id together (generate.rs:202-208)."""
        s = set(int(t) for t in self.eos_token_ids)
        if self.eos_token_id is not None:
            s.add(int(self.eos_token_id))
        return frozenset(s)

    @property
    def penalties_on(self) -> bool:
        return self.repetition_penalty != 1.0 or self.presence_penalty != 0.0 or self.frequency_penalty != 0.0

    @property
    def plain(self) -> bool:
        """Greedy or temperature only: the sampling kernel alone does it."""
        return not (self.penalties_on or self.top_k > 0 or self.top_p < 1.0 or self.min_p > 0.0)
