"""CPU-only: the rule by which the scan and by-key kernels reproduce the SERIAL fold of
thrust::maximum over floating-point values that contain NaNs.

maximum(a, b) = a < b ? b : a (thrust/functional.h) is not associative once NaNs take part: in the
serial fold (thrust/system/detail/sequential/scan.h:54-72, scan_by_key.h:46-142, reduce_by_key.h:43-95)
a NaN that STARTS a fold stays (NaN < x is false, the accumulator is kept), a NaN met later is skipped
(acc < NaN is false as well).  A parallel scan regroups the fold, so the kernels first replace
every NaN that cannot start a fold by the operator's identity (all but element 0 of an inclusive scan;
all but segment heads in inclusive_scan_by_key and reduce_by_key; every NaN in the exclusive forms,
whose folds start from `init`).  After that a NaN only ever appears as the LEFT operand of the
operator, where it is kept whatever the grouping.  The plain scan cannot carry a leading NaN through
its identity-padded wave scans and handles it apart: if the fold's first value (element 0, or `init`)
is a NaN, every result is that NaN.

thrust::minimum(a, b) = a < b ? a : b behaves differently: a NaN element becomes the accumulator and
the next element replaces it (NaN < x is false, b is taken), so every NaN RESTARTS the fold.  The raw
operator does that by itself wherever values are folded in input order.  Where PIECES are combined,
a piece says besides its raw fold whether it holds a NaN (after its last segment head): nothing to
its left survives that NaN.  The empty piece is a state of its own, because the identity +inf is none
for a NaN accumulator (minimum(NaN, +inf) = +inf) and accumulators are shown as they are (exclusive
results, the value of a run that ends with a NaN).  Results are formed by one more raw fold from the
accumulator before each piece.

This test states the rule in numpy — partial aggregates of random pieces, combined in random
groupings, results formed from the pieces' prefixes, exactly the steps the kernels take — and checks
it against the oracle's serial folds.  The GPU tests check the kernels themselves."""
import numpy as np
import pytest

import oracle

OPS = {"maximum": (lambda a, b: b if a < b else a, -np.inf)}


def tree_reduce(items, comb, rng):
    """comb-fold of `items` in their order with a random grouping."""
    if len(items) == 1:
        return items[0]
    cut = int(rng.integers(1, len(items)))
    return comb(tree_reduce(items[:cut], comb, rng), tree_reduce(items[cut:], comb, rng))


def pieces(n, rng):
    cuts = sorted(set(rng.integers(0, n + 1, size=max(1, n // 3)).tolist()) | {0, n})
    return [(a, b) for a, b in zip(cuts[:-1], cuts[1:]) if b > a]


def same(a, b):
    return np.array_equal(np.asarray(a, np.float32).view(np.uint32), np.asarray(b, np.float32).view(np.uint32))


def model_scan(x, opname, exclusive, init, rng):
    op, ident = OPS[opname]
    n = len(x)
    lead = np.float32(init) if exclusive else x[0]
    m = np.where(np.isnan(x), np.float32(ident), x).astype(np.float32)  # every NaN -> identity
    parts = pieces(n, rng)
    aggs = []
    for a, b in parts:
        acc = np.float32(ident)
        for i in range(a, b):
            acc = op(acc, m[i])
        aggs.append(acc)
    out = np.empty(n, np.float32)
    for p, (a, b) in enumerate(parts):
        prefix = tree_reduce(aggs[:p], op, rng) if p else np.float32(ident)
        acc = op(np.float32(init), prefix) if exclusive else prefix
        for i in range(a, b):
            if exclusive:
                out[i] = acc
                acc = op(acc, m[i])
            else:
                acc = op(acc, m[i])
                out[i] = acc
    if np.isnan(lead):
        out[:] = lead
    return out


def model_by_key(keys, vals, opname, mode, init, rng):
    """mode: 'inclusive', 'exclusive' (scan_by_key) or 'reduce' (reduce_by_key)."""
    op, ident = OPS[opname]
    n = len(keys)
    head = np.ones(n, bool)
    head[1:] = keys[1:] != keys[:-1]
    nan = np.isnan(vals)
    skip = nan if mode == "exclusive" else (nan & ~head)
    m = np.where(skip, np.float32(ident), vals).astype(np.float32)

    def comb(a, b):  # (heads seen, value of the open segment)
        return (a[0] + b[0], b[1] if b[0] else op(a[1], b[1]))

    parts = pieces(n, rng)
    aggs = []
    for a, b in parts:
        agg = (0, np.float32(ident))
        for i in range(a, b):
            agg = (agg[0] + 1, m[i]) if head[i] else (agg[0], op(agg[1], m[i]))
        aggs.append(agg)
    out = np.empty(n, np.float32)
    run_keys, run_vals = [], []
    for p, (a, b) in enumerate(parts):
        off = tree_reduce(aggs[:p], comb, rng) if p else (0, np.float32(ident))
        open_ = off[1]
        for i in range(a, b):
            if mode == "exclusive":
                out[i] = np.float32(init) if head[i] else op(np.float32(init), open_)
            if head[i]:
                if mode == "reduce" and i > 0:
                    run_vals.append(open_)
                if mode == "reduce":
                    run_keys.append(keys[i])
                open_ = m[i]
            else:
                open_ = op(open_, m[i])
            if mode == "inclusive":
                out[i] = open_
        if mode == "reduce" and b == n:
            run_vals.append(open_)
    if mode == "reduce":
        return np.array(run_keys, keys.dtype), np.array(run_vals, np.float32)
    return out


EMPTY = 2  # state of a piece without elements


def min_op(a, b):
    return a if a < b else b


def restart_piece(vals, head=None):
    """(heads, state, raw fold) of a piece; state: 0 no NaN after the last head, 1 a NaN, EMPTY."""
    c, r, v = 0, EMPTY, np.float32(np.inf)
    for i, x in enumerate(vals):
        h = bool(head[i]) if head is not None else False
        fresh = h or r == EMPTY
        c += 1 if h else 0
        v = x if fresh else min_op(v, x)
        r = (0 if fresh else r) | (1 if np.isnan(x) else 0)
    return (c, r, v)


def restart_comb(a, b):
    if b[1] == EMPTY:
        return a
    if a[1] == EMPTY:
        return b
    return (a[0] + b[0], b[1] if b[0] else (a[1] | b[1]), b[2] if (b[0] or b[1]) else min_op(a[2], b[2]))


def model_min_scan(x, exclusive, init, rng):
    n = len(x)
    parts = pieces(n, rng)
    aggs = [restart_piece(x[a:b]) for a, b in parts]
    out = np.empty(n, np.float32)
    for p, (a, b) in enumerate(parts):
        before = [restart_piece([np.float32(init)])] if exclusive else []
        before += aggs[:p]
        acc = tree_reduce(before, restart_comb, rng)[2] if before else np.float32(np.inf)
        for i in range(a, b):
            if exclusive:
                out[i] = acc
            acc = min_op(acc, x[i])
            if not exclusive:
                out[i] = acc
    return out


def model_min_by_key(keys, vals, mode, init, rng):
    n = len(keys)
    head = np.ones(n, bool)
    head[1:] = keys[1:] != keys[:-1]
    parts = pieces(n, rng)
    aggs = [restart_piece(vals[a:b], head[a:b]) for a, b in parts]
    out = np.empty(n, np.float32)
    run_keys, run_vals = [], []
    for p, (a, b) in enumerate(parts):
        off = tree_reduce(aggs[:p], restart_comb, rng) if p else (0, EMPTY, np.float32(np.inf))
        open_, restarted = off[2], off[1] == 1
        for i in range(a, b):
            if mode == "exclusive":
                out[i] = np.float32(init) if head[i] else (open_ if restarted else min_op(np.float32(init), open_))
            if head[i]:
                if mode == "reduce" and i > 0:
                    run_vals.append(open_)
                if mode == "reduce":
                    run_keys.append(keys[i])
                open_ = vals[i]
            else:
                open_ = min_op(open_, vals[i])
            restarted = (restarted and not head[i]) or bool(np.isnan(vals[i]))
            if mode == "inclusive":
                out[i] = open_
        if mode == "reduce" and b == n:
            run_vals.append(open_)
    if mode == "reduce":
        return np.array(run_keys, keys.dtype), np.array(run_vals, np.float32)
    return out


def inputs(rng, n, nan_at):
    x = rng.uniform(-5, 5, n).astype(np.float32)
    x[rng.random(n) < 0.1] = np.float32(-np.inf)
    for i in nan_at:
        if i < n:
            x[i] = np.nan
    return x


CASES = [(), (0,), (3,), (0, 1, 2), (5, 9, 10), tuple(range(40))]


@pytest.mark.parametrize("opname", ["maximum"])
def test_scan_rule_reproduces_the_serial_fold(opname):
    rng = np.random.default_rng(1)
    for n in (1, 2, 7, 40):
        for nan_at in CASES:
            x = inputs(rng, n, nan_at)
            for _ in range(6):
                assert same(model_scan(x, opname, False, None, rng), oracle.scan(x, op=opname)), (n, nan_at)
                for init in (np.float32(0.5), np.float32(np.nan), np.float32(-np.inf)):
                    assert same(model_scan(x, opname, True, init, rng), oracle.scan(x, op=opname, exclusive=True, init=init)), (n, nan_at, init)


@pytest.mark.parametrize("opname", ["maximum"])
def test_by_key_rule_reproduces_the_serial_folds(opname):
    rng = np.random.default_rng(2)
    for n in (1, 2, 9, 40):
        for nan_at in CASES:
            for mean in (1, 3, 50):
                keys = np.cumsum(rng.random(n) < 1.0 / mean).astype(np.int32)
                vals = inputs(rng, n, nan_at)
                for _ in range(4):
                    assert same(model_by_key(keys, vals, opname, "inclusive", None, rng), oracle.scan_by_key(keys, vals, op=opname)), (n, nan_at, mean)
                    for init in (np.float32(1.5), np.float32(np.nan)):
                        assert same(model_by_key(keys, vals, opname, "exclusive", init, rng),
                                    oracle.scan_by_key(keys, vals, op=opname, exclusive=True, init=init)), (n, nan_at, mean, init)
                    rk, rv = model_by_key(keys, vals, opname, "reduce", None, rng)
                    ek, ev = oracle.reduce_by_key(keys, vals, op=opname)
                    assert np.array_equal(rk, ek) and same(rv, ev), (n, nan_at, mean)


def test_minimum_with_nans_is_a_restarting_fold():
    x = np.array([1, np.nan, 5, 3, np.nan, np.nan, 7, 9], np.float32)
    got = oracle.scan(x, op="minimum")
    want = np.array([1, np.nan, 5, 3, np.nan, np.nan, 7, 7], np.float32)
    assert same(got, want)


def min_inputs(rng, n, nan_at):
    x = rng.uniform(-5, 5, n).astype(np.float32)
    x[rng.random(n) < 0.1] = np.float32(np.inf)  # the identity as a value
    x[rng.random(n) < 0.1] = np.float32(0.0)
    x[rng.random(n) < 0.1] = np.float32(-0.0)
    for i in nan_at:
        if i < n:
            x[i] = np.nan
    nan = np.isnan(x)
    x.view(np.uint32)[nan] ^= rng.integers(0, 1 << 20, int(nan.sum())).astype(np.uint32)  # NaNs that differ
    return x


def test_minimum_scan_rule_reproduces_the_serial_fold():
    rng = np.random.default_rng(3)
    for n in (1, 2, 7, 40):
        for nan_at in CASES + [(6,), (1, 39), (38, 39)]:
            x = min_inputs(rng, n, nan_at)
            for _ in range(6):
                assert same(model_min_scan(x, False, None, rng), oracle.scan(x, op="minimum")), (n, nan_at)
                for init in (np.float32(0.5), np.float32(np.nan), np.float32(np.inf), np.float32(-0.0)):
                    assert same(model_min_scan(x, True, init, rng), oracle.scan(x, op="minimum", exclusive=True, init=init)), (n, nan_at, init)


def test_minimum_by_key_rule_reproduces_the_serial_folds():
    rng = np.random.default_rng(4)
    for n in (1, 2, 9, 40):
        for nan_at in CASES + [(8,), (1, 39)]:
            for mean in (1, 3, 50):
                keys = np.cumsum(rng.random(n) < 1.0 / mean).astype(np.int32)
                vals = min_inputs(rng, n, nan_at)
                for _ in range(4):
                    assert same(model_min_by_key(keys, vals, "inclusive", None, rng), oracle.scan_by_key(keys, vals, op="minimum")), (n, nan_at, mean)
                    for init in (np.float32(1.5), np.float32(np.nan), np.float32(-0.0)):
                        assert same(model_min_by_key(keys, vals, "exclusive", init, rng),
                                    oracle.scan_by_key(keys, vals, op="minimum", exclusive=True, init=init)), (n, nan_at, mean, init)
                    rk, rv = model_min_by_key(keys, vals, "reduce", None, rng)
                    ek, ev = oracle.reduce_by_key(keys, vals, op="minimum")
                    assert np.array_equal(rk, ek) and same(rv, ev), (n, nan_at, mean)


def test_the_empty_state_is_needed():
    """With +inf standing in for "no elements", a NaN accumulator would be lost: minimum(NaN, +inf) is +inf."""
    assert min_op(np.float32(np.nan), np.float32(np.inf)) == np.float32(np.inf)
    nan_piece = restart_piece([np.float32(np.nan)])
    assert np.isnan(restart_comb(nan_piece, (0, EMPTY, np.float32(np.inf)))[2])
