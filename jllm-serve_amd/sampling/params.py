"""Decoding parameters (sampling/SamplingParams.java:19-56): names, meanings, defaults and checks."""
from __future__ import annotations

import math
from dataclasses import dataclass, replace
from typing import Optional, Tuple


@dataclass(frozen=True)
class SamplingParams:
    """temperature 0 = greedy; top_k 0 = off; top_p 1 = off; min_p 0 = off (keep weights >= min_p of the top
    token's); repetition_penalty 1 = off (HF style, over prompt and output); presence / frequency penalties
    OpenAI style over generated tokens; seed -1 = a fresh random seed; max_tokens caps the output.
    Defaults are the reference's (Qwen3's generation_config values, SamplingParams.java:53-56).
    logprobs: report every generated token's log-probability under the raw logits, with top_logprobs (0 to 20)
    alternatives per position (engine/Engine.java:88-98, engine/TokenLogprob.java). prompt_logprobs: report the
    prompt tokens' log-probabilities too; the whole prompt is then computed, nothing of it is taken from shared
    pages (engine/Engine.java:93-94)."""

    temperature: float = 0.6
    top_k: int = 20
    top_p: float = 0.95
    min_p: float = 0.0
    repetition_penalty: float = 1.0
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    seed: int = -1
    max_tokens: int = 2048
    logit_bias: Optional[Tuple[Tuple[int, float], ...]] = None
    ignore_eos: bool = False
    logprobs: bool = False
    top_logprobs: int = 0
    prompt_logprobs: bool = False

    def __post_init__(self):
        floats = (self.temperature, self.top_p, self.min_p, self.repetition_penalty, self.presence_penalty,
                  self.frequency_penalty)
        if not all(isinstance(v, (int, float)) and math.isfinite(v) for v in floats):
            raise ValueError(f"sampling parameters must be finite numbers: {self.describe()}")
        if (self.temperature < 0 or self.top_k < 0 or self.top_p <= 0 or self.top_p > 1 or self.min_p < 0
                or self.min_p > 1 or self.repetition_penalty <= 0):
            raise ValueError("invalid sampling parameters (temperature >= 0, top_k >= 0, 0 < top_p <= 1, "
                             f"0 <= min_p <= 1, repetition_penalty > 0): {self.describe()}")
        if self.max_tokens < 0:
            raise ValueError(f"max_tokens must not be negative, got {self.max_tokens}")
        if not 0 <= self.top_logprobs <= 20:
            raise ValueError(f"top_logprobs must be between 0 and 20, got {self.top_logprobs}")
        if isinstance(self.logit_bias, dict):
            object.__setattr__(self, "logit_bias", tuple(sorted((int(k), float(v)) for k, v in self.logit_bias.items())))

    def describe(self) -> str:
        return (f"temperature={self.temperature}, top_k={self.top_k}, top_p={self.top_p}, min_p={self.min_p}, "
                f"repetition_penalty={self.repetition_penalty}, presence_penalty={self.presence_penalty}, "
                f"frequency_penalty={self.frequency_penalty}")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0 or self.top_k == 1

    @property
    def plain(self) -> bool:
        """No penalties and no bias: the logits go to the selection kernel as they are (Sampler.java:66-69)."""
        return (self.repetition_penalty == 1 and self.presence_penalty == 0 and self.frequency_penalty == 0
                and not self.logit_bias)

    def with_seed(self, seed: int) -> "SamplingParams":
        return replace(self, seed=seed)

    def with_max_tokens(self, n: int) -> "SamplingParams":
        return replace(self, max_tokens=n)

    @staticmethod
    def greedy_params(max_tokens: int = 2048, **kw) -> "SamplingParams":
        return SamplingParams(temperature=0.0, top_k=0, top_p=1.0, max_tokens=max_tokens, **kw)
