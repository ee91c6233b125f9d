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
    """With ``read_pages`` the model keeps what a real cache keeps: the token of every row, stored where the
    step's slot index says, and a row's history is read back through the step's block table, as attention reads
    keys. A page shared, copied or reused wrongly then shows as a wrong token."""

    def __init__(self, vocab=97, layers=2, window=0, read_pages=False, page_size=4):
        self.config = FakeConfig(vocab)
        self.device = torch.device("cpu")
        self.history = {}
        self.calls = []  # [(rid, position of first row, rows)] per forward
        self.layers = layers
        self.window = window
        self.read_pages = read_pages
        self.page_size = page_size
        self.rows_of_page = {}  # page -> [token or None] * page_size

    def copy_page(self, src, dst, rows):
        page = self.rows_of_page.setdefault(dst, [None] * self.page_size)
        page[:rows] = self.rows_of_page[src][:rows]

    def _forward_pages(self, step):
        B = self.page_size
        tok = step.token_ids.tolist()
        slots = step.groups[0].slots.tolist()
        table = step.groups[0].block_table.tolist()
        rows = {}
        call = []
        for s in step.segments:
            call.append((s.rid, s.pos0, s.n))
            for i in range(s.n):  # store first, as the kernels do
                slot = slots[s.row0 + i]
                self.rows_of_page.setdefault(slot // B, [None] * B)[slot % B] = tok[s.row0 + i]
            for i in range(s.n):
                h = [self.rows_of_page[table[s.index][j // B]][j % B] for j in range(s.pos0 + i + 1)]
                assert None not in h, f"request {s.rid}: a row of its cache was never written"
                rows[s.row0 + i] = next_token(h, self.config.vocab)
        self.calls.append(call)
        out = torch.zeros((step.n_selected, self.config.vocab))
        for j, r in enumerate(step.selected.tolist()):
            out[j, rows[r]] = 1.0
        return out

    def cache_plans(self):
        plans = [CacheEntryPlan(kv=KvSpec(1, 4, 0)) for _ in range(self.layers)]
        if self.window:
            plans.append(CacheEntryPlan(kv=KvSpec(1, 4, self.window)))
        return plans

    def forward(self, step, slots):
        if self.read_pages:
            return self._forward_pages(step)
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
    def __init__(self, vocab=97, page_size=4, pool_tokens=64, max_requests=4, max_positions=256, window=0,
                 prefix_share=False, read_pages=False):
        model = FakeModel(vocab, window=window, read_pages=read_pages or prefix_share, page_size=page_size)
        cache = CacheManager(model.cache_plans(), page_size, pool_tokens, max_requests, allocate=False,
                             prefix_share=prefix_share)
        cache.copy_page = lambda gi, src, dst, rows: model.copy_page(src, dst, rows)
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
