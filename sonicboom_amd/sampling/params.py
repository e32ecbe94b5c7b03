"""Sampling options: the names, meanings and neutral values of the reference's
``boom_llm_sampling`` (/root/reference/capi/include/sonicboom/capi.h:627-677;
defaults /root/reference/core/include/sonicboom/nn/sampling.h:47-57)."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0        # 0: greedy, the first maximum
    top_p: float = 1.0              # 1: no nucleus truncation
    top_k: int = 0                  # 0: no top-k truncation
    seed: int = 0                   # Philox key of the draws
    max_tokens: int = 16            # output cap
    min_p: float = 0.0
    repeat_penalty: float = 1.0     # 0 reads as 1 (off)
    repeat_last_n: int = 64         # 0 disables every penalty
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0

    def validated(self) -> "SamplingParams":
        """Range checks of /root/reference/capi/src/capi.cpp:2634-2660."""
        if not self.temperature >= 0.0:
            raise ValueError("temperature must be >= 0")
        if not 0.0 <= self.top_p <= 1.0:
            raise ValueError("top_p must be in [0, 1]")
        if not 0.0 <= self.min_p <= 1.0:
            raise ValueError("min_p must be in [0, 1]")
        if self.top_k < 0 or self.repeat_last_n < 0 or self.max_tokens < 0:
            raise ValueError("top_k, repeat_last_n and max_tokens must not be negative")
        if self.repeat_penalty < 0.0:
            raise ValueError("repeat_penalty must not be negative")
        if not 0 <= self.seed < 2 ** 64:
            raise ValueError("seed must fit 64 bits")
        if self.repeat_penalty == 0.0:
            return SamplingParams(**{**self.__dict__, "repeat_penalty": 1.0})
        return self

    @property
    def has_penalties(self) -> bool:
        return self.repeat_last_n > 0 and (self.repeat_penalty != 1.0 or self.presence_penalty != 0.0
                                           or self.frequency_penalty != 0.0)
