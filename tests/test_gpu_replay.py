"""Trace replay through bin/trace_run against the plain implementation: every request whole, with the last 32
tokens one by one, in portions of changing size down to two tokens, and mixed with other requests on so few
pages that they are used again; float32 and bfloat16; the tiny configurations and one of a realistic width."""
import numpy as np
import pytest

import replay
import tiny

pytestmark = pytest.mark.gpu


def build_trace(name):
    t = replay.Trace(page=tiny.CONFIGS[name][2])
    lens = {"A": [5, 17, 33, 150],  # 150 > max_position_embeddings of A: the runtime context may exceed the trained one
             "B": [1, 9, 40, 100], "C": [3, 31, 64, 97], "D": [5, 40, 150, 300], "E": [7, 70, 130, 260]}[name]
    toks = {f"r{n}": tiny.prompt(name, n) for n in lens}
    longest = toks[f"r{lens[-1]}"]
    replay.whole(t, "whole", longest)
    replay.tail_one_by_one(t, "tail", longest)
    replay.portions(t, "cut", longest)
    for rid, tk in toks.items():
        replay.whole(t, "w" + rid, tk)
    more = dict(toks)
    more["x1"] = tiny.prompt(name, 45, seed=1)
    more["x2"] = tiny.prompt(name, 2, seed=2)
    more["x3"] = tiny.prompt(name, 66, seed=3)
    replay.mixed(t, more, seed=len(name))
    req_tokens = {"whole": longest, "tail": longest, "cut": longest, **{"w" + k: v for k, v in toks.items()}, **more}
    return t, req_tokens


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_replay_matches_plain(name, dtype, model_folders, plain_logits, tmp_path):
    cfg, _, page = tiny.CONFIGS[name]
    trace, req_tokens = build_trace(name)
    # the pool is exactly the pages of the busiest step, so later requests reuse the pages of ended ones; the free
    # pages are reordered before every step, so page ids follow neither positions nor requests
    got = replay.run(model_folders[name], dtype, trace, str(tmp_path), page_size=page, max_tokens=trace.peak,
                     shuffle_free=len(name) + 7)
    V = cfg["vocab_size"]
    worst = 0.0
    for step, rows in trace.rows.items():
        arr = got[step].reshape(len(rows), V)
        for i, (rid, pos) in enumerate(rows):
            ref = plain_logits(name, req_tokens[rid])[pos]
            tol = tiny.tolerance(dtype, ref)
            err = float(np.abs(arr[i].astype(np.float64) - ref.numpy()).max())
            worst = max(worst, err / tol)
            assert err <= tol, f"{name} {dtype}: step {step} request {rid} position {pos}: |diff| {err:.3g} > {tol:.3g}"
            if dtype == "float32":
                assert int(arr[i].argmax()) == int(ref.argmax())
    if dtype == "float32":
        # the 32-bit kernels add in an order that depends on a row's own position only: whole, with the tail one by
        # one, cut into portions, or mixed with other requests, a position's logits are the same to the last bit
        by_place = {}
        for step, rows in trace.rows.items():
            arr = got[step].reshape(len(rows), V)
            for i, (rid, pos) in enumerate(rows):
                by_place[(rid, pos)] = arr[i]
        pairs = [("whole", other) for other in ("tail", "cut")] + [("w" + rid, rid) for rid in req_tokens if "w" + rid in req_tokens]
        compared = 0
        for a, b in pairs:
            for pos in range(len(req_tokens[a])):
                assert np.array_equal(by_place[(a, pos)], by_place[(b, pos)]), \
                    f"{name}: position {pos} of '{b}' differs in bits from the same position of '{a}'"
                compared += 1
        assert compared >= 2 * len(req_tokens["whole"]) + sum(len(req_tokens[b]) for _, b in pairs[2:])
    print(f"{name} {dtype}: worst error / tolerance = {worst:.3f} over {sum(len(r) for r in trace.rows.values())} rows")
