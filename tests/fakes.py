"""A model stand-in for host-side tests: the real cache manager and step bookkeeping, no GPU.

Its "logits" put all mass on one token that is a hash of the request's whole token history up to the row, so
any mistake in cutting, ordering, preempting or replaying a request changes the generated tokens.
"""
import torch

from jllm_serve_amd.cache.manager import CacheEntryPlan, CacheManager, KvSpec
from jllm_serve_amd.engine.step import ModelRunner


def next_token(history, vocab):
    h = 1469598103
    for t in history:
        h = (h * 1000003 + t + 1) % 2147483647
    return h % vocab


class FakeConfig:
    def __init__(self, vocab):
        self.vocab = vocab


class FakeModel:
    def __init__(self, vocab=97, layers=2, window=0):
        self.config = FakeConfig(vocab)
        self.device = torch.device("cpu")
        self.history = {}
        self.calls = []  # [(rid, position of first row, rows)] per forward
        self.layers = layers
        self.window = window

    def cache_plans(self):
        plans = [CacheEntryPlan(kv=KvSpec(1, 4, 0)) for _ in range(self.layers)]
        if self.window:
            plans.append(CacheEntryPlan(kv=KvSpec(1, 4, self.window)))
        return plans

    def forward(self, step, slots):
        tok = step.token_ids.tolist()
        rows = {}
        call = []
        for s in step.segments:
            h = self.history.setdefault(s.rid, [])
            assert len(h) == s.pos0, f"request {s.rid}: the step starts at {s.pos0} but {len(h)} tokens were fed"
            call.append((s.rid, s.pos0, s.n))
            for i in range(s.n):
                h.append(tok[s.row0 + i])
                rows[s.row0 + i] = next_token(h, self.config.vocab)
        self.calls.append(call)
        out = torch.zeros((step.n_selected, self.config.vocab))
        for j, r in enumerate(step.selected.tolist()):
            out[j, rows[r]] = 1.0
        return out


class FakeRunner(ModelRunner):
    def __init__(self, vocab=97, page_size=4, pool_tokens=64, max_requests=4, max_positions=256, window=0):
        model = FakeModel(vocab, window=window)
        cache = CacheManager(model.cache_plans(), page_size, pool_tokens, max_requests, allocate=False)
        super().__init__(model, cache, max_positions)

    def finish(self, rid):
        super().finish(rid)
        self.model.history.pop(rid, None)


def argmax_sampler(logits, states):
    return torch.argmax(logits, dim=-1).tolist()


def expected_generation(prompt, n, vocab, eos=()):
    """What greedy generation must give with the fake model, however the engine cuts and replays."""
    h = list(prompt)
    out = []
    for _ in range(n):
        t = next_token(h, vocab)
        if t in eos:
            return out, "stop"
        out.append(t)
        h.append(t)
    return out, "length"
