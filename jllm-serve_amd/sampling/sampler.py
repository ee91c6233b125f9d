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

import numpy as np
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


class _ParamUpload:
    """The selection's per-row numbers go up as one small buffer that a kernel in the stream copies out of pinned host
    memory (``ops.copy_words``): a copy from ordinary host memory makes the host wait until the stream has reached
    it, that is for the whole pass that made the logits, and the look-ahead of the engine would be gone (0.3 ms per
    step at batch 8). Three buffers take turns; one is written again only when the copy out of it has run."""

    TURNS = 3

    def __init__(self, device):
        self.device = device
        self.turn = 0
        self.slots = [None] * self.TURNS  # (pinned host, device, event after the copy)

    def put(self, words: "np.ndarray") -> torch.Tensor:
        n = int(words.size)
        self.turn = (self.turn + 1) % self.TURNS
        slot = self.slots[self.turn]
        if slot is None or slot[0].numel() < n:
            if slot is not None:
                # the copy kernel that reads the old pinned block may still be queued, and the host allocator that
                # gets the block back knows nothing of kernels: wait for it before letting go
                slot[2].synchronize()
            size = max(64, 1 << (n - 1).bit_length())
            slot = (torch.empty(size, dtype=torch.int32).pin_memory(),
                    torch.empty(size, dtype=torch.int32, device=self.device), torch.cuda.Event())
            self.slots[self.turn] = slot
        else:
            slot[2].synchronize()
        host, dev, copied = slot
        host.numpy()[:n] = words
        ops.copy_words(host[:n], dev[:n])
        copied.record()
        return dev[:n]


_uploads: Dict[torch.device, _ParamUpload] = {}


def select_rows(logits: torch.Tensor, states: List[SamplerState]) -> torch.Tensor:
    """The selection alone (greedy or the filtered draw), left on the device as int32 [n]: what ``sample_rows`` does
    after penalties and bias. Advances the draw counters of the rows that draw."""
    dev = logits.device
    if all(st.params.greedy for st in states):
        return ops.argmax(logits)
    n = len(states)
    # one buffer of 32-bit words: the uniform numbers (64-bit, first: aligned), temperatures, top-k, top-p, min-p
    words = np.empty(6 * n, np.int32)
    words[:2 * n].view(np.float64)[:] = [0.0 if st.params.greedy else st.next_uniform() for st in states]
    words[2 * n:3 * n].view(np.float32)[:] = [0.0 if st.params.greedy else st.params.temperature for st in states]
    words[3 * n:4 * n] = [st.params.top_k for st in states]
    words[4 * n:5 * n].view(np.float32)[:] = [st.params.top_p for st in states]
    words[5 * n:].view(np.float32)[:] = [st.params.min_p for st in states]
    if dev.type == "cuda":
        up = _uploads.get(dev)
        if up is None:
            up = _uploads[dev] = _ParamUpload(dev)
        d = up.put(words)
    else:
        d = torch.from_numpy(words).to(dev)
    return ops.sample(logits, d[2 * n:3 * n].view(torch.float32), d[3 * n:4 * n], d[4 * n:5 * n].view(torch.float32),
                      d[5 * n:].view(torch.float32), d[:2 * n].view(torch.float64))
