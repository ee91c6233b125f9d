"""The native host library against plain Python formulations of the same: the page pool under random orders, the
step layout (token ids, positions, row -> request, state slots, selected rows, cache slots, block tables) for random
batches with windows (table entries given back), padding to a captured size and a wider table than needed."""
import ctypes
import os
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


def plain_layout(entries, tables, B, pad_rows, width, pad_slot=0):
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
    slots_of = np.full(R, pad_slot, np.int32)
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


def native_layout(entries, arenas, B, pad_rows, width, pad_slot=0):
    i32 = lambda v: np.asarray(v, np.int32)
    counts, starts, slots = i32([len(e[0]) for e in entries]), i32([e[1] for e in entries]), i32([e[2] for e in entries])
    want_counts = i32([len(e[3]) for e in entries])
    tokens, wants = i32([t for e in entries for t in e[0]]), i32([w for e in entries for w in e[3]])
    G = len(arenas)
    call = lambda out, cap: host.step_layout(counts, starts, slots, tokens, want_counts, wants, pad_rows, pad_slot, width, B,
                                             arenas, slots, out, cap)
    small = np.full(4, 77, np.int32)
    rc, sizes = call(small, 0)
    if rc == -3:
        return rc, small, None
    assert rc == -1 and (small == 77).all(), "too small a buffer: sizes only, nothing written"
    total = 3 * sizes.T + sizes.R + sizes.S + G * (sizes.T + sizes.R * sizes.width)
    out = np.full(total + 3, -99, np.int32)
    got, sizes = call(out, total)
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
    want_flat, want_sizes = plain_layout(entries, tables, B, pad, width, pad_slot=9)
    got, out, sizes = native_layout(entries, arenas, B, pad, width, pad_slot=9)
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


def test_padding_rows_get_a_state_row_that_no_request_holds():
    """A captured step of 8 rows with 2 live requests, one of them in state slot 0: the 6 padding requests all name
    the row beyond the request slots, never slot 0 (a mixer that updates its state per row would otherwise write
    into a live request's state from the padding rows)."""
    arena = TableArena(4)
    entries = []
    for slot, p0 in ((0, 5), (3, 17)):
        t = arena.table(slot)
        for p in range(-(-(p0 + 1) // 4)):
            t.append(10 + p)
        entries.append(([7], p0, slot, [0]))
    got, out, sizes = native_layout(entries, [arena], 4, 8, 0, pad_slot=4)
    T, R, S, width, _ = sizes
    assert (T, R, S) == (8, 8, 8) and got > 0
    slots_of = out[3 * T:3 * T + R]
    assert slots_of.tolist() == [0, 3] + [4] * 6


def test_step_layout_refuses_a_batch_that_contradicts_itself():
    """The builder trusts no length it was not given: a wanted place outside its entry, a table row outside the
    arena, a table that claims more entries than its row has, counts below one, a page size that is no power of two."""
    def one(n=3, p0=2, slot=1, want=(2,), B=4, rows=2, lens=None):
        arena = TableArena(rows, cols=4)
        if 0 <= slot < rows:
            t = arena.table(slot)
            for p in range(-(-(p0 + max(n, 1)) // max(B, 1))):
                t.append(p)
            if lens is not None:
                arena.lens[slot] = lens
        return native_layout([([1] * n, p0, slot, list(want))], [arena], B, 0, 0)[0]
    assert one() > 0
    assert one(want=(3,)) == -3 and one(want=(-1,)) == -3            # a place outside the entry's tokens
    assert one(want=(2,), n=3) > 0 and one(want=(0, 2)) > 0          # the last place is fine
    assert one(slot=2) == -3 and one(slot=-1) == -3                  # a table row outside the arena
    assert one(lens=5) == -3                                         # more entries than the row holds
    assert one(p0=-1) == -3 and one(B=3) == -3 and one(B=0) == -3
    assert one(p0=13, n=3, B=4) > 0                                  # a table used up to its last column (4 entries)
    # the sums of the counts must be the lengths of the token and want lists
    arena = TableArena(1)
    arena.table(0).append(0)
    i32 = lambda v: np.asarray(v, np.int32)
    out = np.zeros(64, np.int32)
    rc, _ = host.step_layout(i32([2]), i32([0]), i32([0]), i32([1, 2, 3]), i32([0]), i32([]), 0, 1, 0, 4, [arena], i32([0]), out)
    assert rc == -3
    rc, _ = host.step_layout(i32([2]), i32([0]), i32([0]), i32([1, 2]), i32([1]), i32([]), 0, 1, 0, 4, [arena], i32([0]), out)
    assert rc == -3


@pytest.mark.parametrize("seed", [1, 2])
def test_host_library_under_sanitizers(tmp_path, seed):
    """The pool and the step layout, built with AddressSanitizer and UndefinedBehaviorSanitizer, hammered by their C++
    driver with random work: wanted places at the last token, tables used up to their last column, buffers of
    exactly the stated lengths, and batches made wrong in one place (refused, not read). CPU only."""
    import subprocess
    from jllm_serve_amd.kernels import build
    try:
        exe = build.build_host_check(str(tmp_path))
    except RuntimeError as e:
        if "sanitize" in str(e) or "asan" in str(e).lower():
            pytest.skip(f"this compiler has no sanitizer runtime: {str(e)[-200:]}")
        raise
    r = subprocess.run([exe, str(seed), "2000"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120,
                       env=dict(os.environ, ASAN_OPTIONS="detect_leaks=1", UBSAN_OPTIONS="print_stacktrace=1"))
    assert r.returncode == 0 and "hammer ok" in r.stdout, r.stdout[-3000:]
