"""The sampler: per-request state on the host, selection on the device.

sampling/Sampler.java keeps one sampler per request: the tokens seen (prompt and output), how often each was
generated, and a seeded random stream; ``sample(logits)`` applies penalties and bias, then greedy or the
filtered draw (:72-77, :346-432). Here the state is the same, the arithmetic over the vocabulary runs in
the selection kernel, and the random stream is counter based: draw number i of a request with seed s uses
``uniform(s, i)``, so neither batching nor a preemption that replays the request changes what is drawn.
"""
from __future__ import annotations

import os
from typing import Dict, List, Sequence

import torch

from ..kernels import ops
from .params import SamplingParams

_M64 = (1 << 64) - 1


def uniform(seed: int, counter: int) -> float:
    """A number in [0, 1) from (seed, counter): a 64-bit mix (add-shift-multiply finaliser), top 53 bits."""
    x = ((seed & _M64) * 0x9E3779B97F4A7C15 + ((counter + 1) & _M64) * 0xD1B54A32D192ED03) & _M64
    x ^= x >> 30
    x = (x * 0xBF58476D1CE4E5B9) & _M64
    x ^= x >> 27
    x = (x * 0x94D049BB133111EB) & _M64
    x ^= x >> 31
    return (x >> 11) * (1.0 / (1 << 53))


class SamplerState:
    """What one request's sampler remembers (Sampler.java:37-61)."""

    def __init__(self, params: SamplingParams, vocab: int, prompt: Sequence[int]):
        self.params = params
        self.vocab = vocab
        self.seed = params.seed if params.seed >= 0 else int.from_bytes(os.urandom(7), "little")
        self.draws = 0
        self.seen = {t for t in prompt if 0 <= t < vocab} if not params.plain else set()
        self.generated: Dict[int, int] = {}

    def accept(self, token: int) -> None:
        """Records a generated token so the penalties see it (Sampler.java:55-61)."""
        if not self.params.plain and 0 <= token < self.vocab:
            self.seen.add(token)
            self.generated[token] = self.generated.get(token, 0) + 1

    def next_uniform(self) -> float:
        u = uniform(self.seed, self.draws)
        self.draws += 1
        return u


def sample_rows(logits: torch.Tensor, states: List[SamplerState]) -> List[int]:
    """One token for each row of fp32 ``logits`` [n, vocab] with the row's sampler; the logits of rows with
    penalties or bias are changed in place, as in the reference."""
    n = logits.shape[0]
    assert n == len(states)
    dev = logits.device
    for i, st in enumerate(states):
        p = st.params
        if p.plain:
            continue
        ids = sorted(st.seen)
        seen = torch.tensor(ids, dtype=torch.int32, device=dev) if ids else None
        counts = torch.tensor([st.generated.get(t, 0) for t in ids], dtype=torch.int32, device=dev) if ids else None
        b_ids = b_vals = None
        if p.logit_bias:
            b_ids = torch.tensor([b[0] for b in p.logit_bias], dtype=torch.int32, device=dev)
            b_vals = torch.tensor([b[1] for b in p.logit_bias], dtype=torch.float32, device=dev)
        ops.adjust_logits(logits[i], seen, counts, p.repetition_penalty, p.presence_penalty, p.frequency_penalty,
                          b_ids, b_vals)
    return select_rows(logits, states).tolist()


def select_rows(logits: torch.Tensor, states: List[SamplerState]) -> torch.Tensor:
    """The selection alone (greedy or the filtered draw), left on the device as int32 [n]: what ``sample_rows`` does
    after penalties and bias. Advances the draw counters of the rows that draw."""
    dev = logits.device
    if all(st.params.greedy for st in states):
        return ops.argmax(logits)
    temps = torch.tensor([0.0 if st.params.greedy else st.params.temperature for st in states], dtype=torch.float32)
    top_k = torch.tensor([st.params.top_k for st in states], dtype=torch.int32)
    top_p = torch.tensor([st.params.top_p for st in states], dtype=torch.float32)
    min_p = torch.tensor([st.params.min_p for st in states], dtype=torch.float32)
    u = torch.tensor([0.0 if st.params.greedy else st.next_uniform() for st in states], dtype=torch.float64)
    return ops.sample(logits, temps.to(dev), top_k.to(dev), top_p.to(dev), min_p.to(dev), u.to(dev))
