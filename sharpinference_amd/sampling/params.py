"""Sampling options of one request."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Optional, Sequence, Tuple


@dataclass
class SamplingParams:
    """Names, meanings and defaults follow the reference's record
    (reference: src/SharpInference.Engine/Sampler.cs:648-741): temperature <= 0 is greedy;
    top_k 0, top_p 1 and min_p 0 switch their filters off; repetition_penalty 1 and
    frequency / presence 0 switch the penalties off; the penalties look at the last
    ``penalty_last_n`` tokens (0 = all), the prompt included if ``penalty_seed_from_prompt``.
    ``stop_token_ids`` None means the model's end-of-generation tokens; a tuple (an empty one
    too) replaces them; ``additional_stop_token_ids`` are added to either (reference:
    Sampler.cs:724-741)."""

    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    min_p: float = 0.0
    repetition_penalty: float = 1.0
    frequency_penalty: float = 0.0
    presence_penalty: float = 0.0
    penalty_last_n: int = 256
    penalty_seed_from_prompt: bool = True
    logit_bias: Optional[Dict[int, float]] = None
    max_new_tokens: int = 512
    stop_token_ids: Optional[Tuple[int, ...]] = None
    additional_stop_token_ids: Tuple[int, ...] = ()
    seed: int = 0

    def __post_init__(self):
        if self.stop_token_ids is not None:
            self.stop_token_ids = tuple(int(t) for t in self.stop_token_ids)
        self.additional_stop_token_ids = tuple(int(t) for t in (self.additional_stop_token_ids or ()))
        if self.max_new_tokens < 0:
            raise ValueError("max_new_tokens must not be negative")
        if self.top_k < 0:
            raise ValueError("top_k must not be negative")
        if self.repetition_penalty <= 0:
            raise ValueError("repetition_penalty must be positive")

    def stop_set(self, end_of_generation: Sequence[int] = ()) -> frozenset:
        """The tokens that end this request, given the model's end-of-generation tokens."""
        base = end_of_generation if self.stop_token_ids is None else self.stop_token_ids
        return frozenset(int(t) for t in base) | frozenset(self.additional_stop_token_ids)

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0

    @property
    def has_penalties(self) -> bool:
        return self.repetition_penalty != 1.0 or self.frequency_penalty != 0.0 or self.presence_penalty != 0.0

    @property
    def edits_logits(self) -> bool:
        return self.has_penalties or bool(self.logit_bias)
