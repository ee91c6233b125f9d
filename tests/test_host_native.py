"""The native host library against plain Python formulations of the same: the page pool under random orders, the
step layout (token ids, positions, row -> request, state slots, selected rows, cache slots, block tables) for random
batches with windows (table entries given back), padding to a captured size and a wider table than needed."""
import ctypes
import random

import numpy as np
import pytest

from jllm_serve_amd import host
from jllm_serve_amd.cache.pages import OutOfPages, PagePool
from jllm_serve_amd.cache.tables import TableArena


def test_pool_against_a_plain_model_under_random_orders():
    rng = random.Random(5)
    pool = PagePool(37, 16)
    refs = {}
    for step in range(4000):
        op = rng.random()
        if op < 0.45:
            if len(refs) == 37:
                with pytest.raises(OutOfPages):
                    pool.alloc()
            else:
                p = pool.alloc()
                assert p not in refs
                refs[p] = 1
        elif op < 0.6 and refs:
            p = rng.choice(sorted(refs))
            pool.retain(p)
            refs[p] += 1
        elif refs:
            p = rng.choice(sorted(refs))
            pool.release(p)
            refs[p] -= 1
            if not refs[p]:
                del refs[p]
        if step % 97 == 0:
            pool.shuffle_free(rng)
            pool.check()
        assert pool.used_pages == len(refs) and pool.free_pages == 37 - len(refs)
    assert all(pool.refs(p) == n for p, n in refs.items())
    free = pool.free_list()
    assert sorted(free + sorted(refs)) == list(range(37))
    assert pool.high_water <= 37 and pool.allocations >= pool.high_water
    for bad in (-1, 37):
        with pytest.raises(ValueError):
            pool.release(bad)
    unheld = free[0]
    with pytest.raises(ValueError):
        pool.release(unheld)
    with pytest.raises(ValueError):
        pool.retain(unheld)


def plain_layout(entries, tables, B, pad_rows, width):
    """entries: (tokens, pos0, state slot, want); tables[g][i]: list of page ids of entry i in group g."""
    n_real = sum(len(e[0]) for e in entries)
    T = max(n_real, pad_rows)
    R = len(entries) + (T - n_real)
    tok, pos = np.zeros(T, np.int32), np.zeros(T, np.int32)
    req = np.arange(R - T, R, dtype=np.int32)
    sel, row, max_ctx = [], 0, 1
    for i, (t, p0, _, want) in enumerate(entries):
        n = len(t)
        tok[row:row + n], pos[row:row + n], req[row:row + n] = t, np.arange(p0, p0 + n), i
        sel += [row + w for w in want]
        max_ctx = max(max_ctx, p0 + n)
        row += n
    if pad_rows:
        sel = list(range(T))
    width = max(width, 1, -(-max_ctx // B))
    slots_of = np.zeros(R, np.int32)
    slots_of[:len(entries)] = [e[2] for e in entries]
    parts = [tok, pos, req, slots_of, np.asarray(sel, np.int32)]
    for g in range(len(tables)):
        slots = np.full(T, -1, np.int32)
        table = np.zeros((R, width), np.int32)
        row = 0
        for i, (t, p0, _, _) in enumerate(entries):
            tb = np.asarray(tables[g][i], np.int32)
            table[i, :len(tb)] = np.maximum(tb, 0)
            p = np.arange(p0, p0 + len(t))
            slots[row:row + len(t)] = tb[p // B] * B + p % B
            row += len(t)
        parts += [slots, table.reshape(-1)]
    return np.concatenate(parts), (T, R, len(sel), width, max_ctx)


def native_layout(entries, arenas, B, pad_rows, width):
    lib = host.library()
    i32 = lambda v: np.asarray(v, np.int32)
    counts, starts, slots = i32([len(e[0]) for e in entries]), i32([e[1] for e in entries]), i32([e[2] for e in entries])
    want_counts = i32([len(e[3]) for e in entries])
    tokens, wants = i32([t for e in entries for t in e[0]]), i32([w for e in entries for w in e[3]])
    G = len(arenas)
    ap = (ctypes.c_void_p * max(1, G))(*[a.data.ctypes.data for a in arenas])
    st = (ctypes.c_int64 * max(1, G))(*[a.data.shape[1] for a in arenas])
    lp = (ctypes.c_void_p * max(1, G))(*[a.lens.ctypes.data for a in arenas])
    sizes = host.StepSizes()
    call = lambda out, cap: lib.jllm_step_layout(len(entries), counts.ctypes.data, starts.ctypes.data, slots.ctypes.data,
                                                 tokens.ctypes.data, want_counts.ctypes.data, wants.ctypes.data, pad_rows, width, B,
                                                 G, ap, st, slots.ctypes.data, lp, out.ctypes.data, cap, ctypes.byref(sizes))
    small = np.full(4, 77, np.int32)
    assert call(small, 0) == -1 and (small == 77).all(), "too small a buffer: sizes only, nothing written"
    total = 3 * sizes.T + sizes.R + sizes.S + G * (sizes.T + sizes.R * sizes.width)
    out = np.full(total + 3, -99, np.int32)
    got = call(out, total)
    return got, out, (sizes.T, sizes.R, sizes.S, sizes.width, sizes.max_context)


@pytest.mark.parametrize("seed", range(12))
def test_step_layout_against_a_plain_formulation(seed):
    rng = random.Random(seed)
    B = rng.choice([1, 4, 16])
    G = rng.choice([0, 1, 2])
    slots_free = list(range(9))
    rng.shuffle(slots_free)
    arenas = [TableArena(9, cols=2) for _ in range(G)]
    entries, tables = [], [[] for _ in range(G)]
    decode_only = rng.random() < 0.4
    for i in range(rng.randint(1, 6)):
        n = 1 if decode_only else rng.choice([1, 2, 5, 33])
        p0 = rng.randint(0, 70)
        slot = slots_free.pop()
        want = sorted(rng.sample(range(n), rng.randint(0, min(n, 3))))
        entries.append(([rng.randrange(1000) for _ in range(n)], p0, slot, want))
        for g in range(G):
            need = -(-(p0 + n) // B)
            gone = rng.randint(0, p0 // B) if g == 1 else 0  # the windowed group has given back its first pages
            pages = [-1] * gone + [rng.randrange(500) for _ in range(need - gone)]
            t = arenas[g].table(slot)
            for p in pages:
                t.append(p)
            assert t == pages and len(t) == need
            tables[g].append(pages)
    pad = rng.choice([0, 0, 8, 64]) if decode_only else 0
    pad = max(pad, len(entries)) if pad else 0
    width = rng.choice([0, 0, 40])
    want_flat, want_sizes = plain_layout(entries, tables, B, pad, width)
    got, out, sizes = native_layout(entries, arenas, B, pad, width)
    assert sizes == want_sizes and got == want_flat.size
    assert np.array_equal(out[:got], want_flat) and (out[got:] == -99).all()


def test_step_layout_refuses_a_row_in_a_page_that_was_given_back():
    arena = TableArena(2)
    t = arena.table(1)
    for p in (-1, 7):
        t.append(p)
    for pos0, n, bad in ((4, 2, False), (3, 2, True), (6, 3, True)):  # page size 4: positions 0..3 are gone, 8.. not there yet
        got, _, _ = native_layout([([1] * n, pos0, 1, [])], [arena], 4, 0, 0)
        assert (got == -2) == bad
