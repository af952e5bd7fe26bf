"""The options of sampling, with the reference's names, defaults and ranges
(engine/sampler.h:7-17; validation engine/sampler.cpp:222-260)."""
from __future__ import annotations

import math
from dataclasses import dataclass


class SamplingError(ValueError):
    pass


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.6        # 0 = greedy
    top_k: int = 50                 # 0 = disabled
    top_p: float = 0.9              # 0 or 1 = disabled
    min_p: float = 0.0              # probability relative to the best token
    repeat_penalty: float = 1.0     # 1 = disabled
    repeat_last_n: int = 64         # window for all penalties; -1 = full context, 0 = disabled
    presence_penalty: float = 0.0   # [-2, 2]
    frequency_penalty: float = 0.0  # [-2, 2]
    seed: int = 42

    def validate(self) -> None:
        def finite(v):
            return isinstance(v, (int, float)) and math.isfinite(v)
        if not finite(self.temperature) or not 0.0 <= self.temperature <= 2.0:
            raise SamplingError("temperature must be between 0 and 2")
        if self.top_k < 0:
            raise SamplingError("top_k must be non-negative")
        if not finite(self.top_p) or not 0.0 <= self.top_p <= 1.0:
            raise SamplingError("top_p must be between 0 and 1")
        if not finite(self.min_p) or not 0.0 <= self.min_p <= 1.0:
            raise SamplingError("min_p must be between 0 and 1")
        if not finite(self.repeat_penalty) or self.repeat_penalty <= 0.0:
            raise SamplingError("repeat_penalty must be greater than 0")
        if self.repeat_last_n < -1:
            raise SamplingError("repeat_last_n must be -1 or non-negative")
        if not finite(self.presence_penalty) or not -2.0 <= self.presence_penalty <= 2.0:
            raise SamplingError("presence_penalty must be between -2 and 2")
        if not finite(self.frequency_penalty) or not -2.0 <= self.frequency_penalty <= 2.0:
            raise SamplingError("frequency_penalty must be between -2 and 2")
        if self.seed < 0:
            raise SamplingError("seed must be non-negative")

    @property
    def penalties_enabled(self) -> bool:
        # engine/sampler.cpp:305-309
        return self.repeat_last_n != 0 and (self.repeat_penalty != 1.0 or self.presence_penalty != 0.0
                                            or self.frequency_penalty != 0.0)

    @property
    def greedy(self) -> bool:
        # engine/sampler.cpp:171-172
        return self.temperature <= 0.0 or self.top_k == 1

    @property
    def plain_argmax(self) -> bool:
        # engine/sampler.cpp:293-302
        return self.greedy and not self.penalties_enabled


GREEDY = SamplingParams(temperature=0.0, top_k=0, top_p=0.0)
