"""An elementwise op behind a matmul in the same task (the reference runs the ops of a task one
after the other over the task's tile, ark/codegen.cpp:160-238) is folded into the matmul's store
where the operands allow: the result must be the bits of the two ops run apart, which round the
matmul's output to the tensor type in between, and agree with the oracle's composition."""
import json

import numpy as np
import pytest

from helpers import make
from test_executor_gpu import close, run_model

pytestmark = pytest.mark.gpu


def _folded(plan):
    from ark_amd import plan_analysis
    return [s["FoldedIntoStore"] for s in plan_analysis(plan)["Steps"] if s["Kind"] == "Tasks"]


def _close_sum(oracle, ref, got, dtype):
    """Sums cancel: one rounding step of the matmul's output (whose summation order differs from the
    oracle's) is not small relative to a single result; the error is bounded by the largest result and
    in rms instead."""
    t, g = (oracle.to_f32(a, dtype).astype(np.float64) for a in (ref, got))
    assert np.abs(t - g).max() <= 1e-2 * np.abs(t).max()
    assert np.sqrt(((t - g) ** 2).mean()) <= 2e-3 * np.sqrt((t * t).mean())


def _both_ways(monkeypatch, build, feeds_of):
    """Runs the model `build(m)` makes with the fold on and off; returns (plan, folded flags, results)."""
    from ark_amd import Model
    res = []
    for on in ("1", "0"):
        monkeypatch.setenv("ARKMI_GEMM_FOLD_STORE", on)
        m = Model()
        tensors, outs = build(m)
        plan = m.plan(device_id=0)
        got, _, _ = run_model(m, feeds_of(tensors), outs, iters=2, plan=plan)
        res.append((plan, _folded(plan), got))
    return res


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("kind,c_first", [("add", False), ("add", True), ("sub", False), ("sub", True),
                                          ("mul", True), ("div", True), ("div", False)])
def test_arithmetic_behind_a_matmul(oracle, monkeypatch, dtype, kind, c_first):
    M, N, K = 512, 768, 256
    x = make(oracle, (M, K), dtype, 301)
    w = make(oracle, (N, K), dtype, 302, "normal", scale=0.05)
    r = make(oracle, (M, N), dtype, 303, "uniform", 0.5, 2.0)

    def build(m):
        tx, tw, tr = m.tensor(x.shape, dtype), m.tensor(w.shape, dtype), m.tensor(r.shape, dtype)
        with m.planner_context(sync=False):
            y = m.matmul(tx, tw, trans_other=True)
            o = getattr(m, kind)(y, tr) if c_first else getattr(m, kind)(tr, y)
        return (tx, tw, tr), [o, y]

    (plan, on_flags, on), (_, off_flags, off) = _both_ways(
        monkeypatch, build, lambda t: {t[0]: x, t[1]: w, t[2]: r})
    assert len(json.loads(plan)["TaskInfos"]) == 1 and on_flags == [True] and off_flags == [False]
    assert np.array_equal(on[0], off[0]) and np.array_equal(on[1], off[1])  # the op's result, and C itself
    y = oracle.matmul(x, w, dtype, trans_b=True)
    ref = oracle.binary(y, r, kind, dtype) if c_first else oracle.binary(r, y, kind, dtype)
    if kind == "div" and not c_first:
        # r / y with y near zero: compare where the quotient is tame
        ok = np.abs(oracle.to_f32(y, dtype)) > 0.05
        t, g = oracle.to_f32(ref, dtype)[ok], oracle.to_f32(on[0], dtype)[ok]
        assert ok.mean() > 0.5 and np.abs(t - g).max() <= 5e-2 * np.abs(t).max()
    elif kind in ("add", "sub"):
        _close_sum(oracle, ref, on[0], dtype)
    else:
        close(oracle, ref, on[0], dtype, 1e-2)


def test_bias_row_and_a_column_operand(oracle, monkeypatch):
    """A [1, N] operand (one row for all) folds; a [M, 1] operand (one value per row) does not,
    and runs as the pass of its own it was."""
    dtype = "bf16"
    M, N, K = 512, 512, 128
    x = make(oracle, (M, K), dtype, 311)
    w = make(oracle, (K, N), dtype, 312, "normal", scale=0.05)
    for shape, folds in (((1, N), True), ((M, 1), False)):
        b = make(oracle, shape, dtype, 313)

        def build(m):
            tx, tw, tb = m.tensor(x.shape, dtype), m.tensor(w.shape, dtype), m.tensor(b.shape, dtype)
            with m.planner_context(sync=False):
                o = m.add(m.matmul(tx, tw), tb)
            return (tx, tw, tb), [o]

        (plan, on_flags, on), (_, off_flags, off) = _both_ways(
            monkeypatch, build, lambda t: {t[0]: x, t[1]: w, t[2]: b})
        assert len(json.loads(plan)["TaskInfos"]) == 1 and on_flags == [folds] and off_flags == [False]
        assert np.array_equal(on[0], off[0])
        ref = oracle.binary(oracle.matmul(x, w, dtype), np.broadcast_to(b, (M, N)), "add", dtype)
        _close_sum(oracle, ref, on[0], dtype)


@pytest.mark.parametrize("heads,hd", [(4, 128), (8, 64)])
def test_rope_through_a_reshape(oracle, monkeypatch, heads, hd):
    dtype = "bf16"
    S, K = 512, 256
    x = make(oracle, (1, S, K), dtype, 321)
    w = make(oracle, (heads * hd, K), dtype, 322, "normal", scale=0.05)
    f = make(oracle, (1, S, 1, hd), dtype, 323)

    def build(m):
        tx, tw, tf = m.tensor(x.shape, dtype), m.tensor(w.shape, dtype), m.tensor(f.shape, dtype)
        with m.planner_context(sync=False):
            o = m.rope(m.reshape(m.matmul(tx, tw, trans_other=True), [1, S, heads, hd]), tf)
        return (tx, tw, tf), [o]

    (plan, on_flags, on), (_, off_flags, off) = _both_ways(
        monkeypatch, build, lambda t: {t[0]: x, t[1]: w, t[2]: f})
    assert on_flags == [True] and off_flags == [False]
    assert np.array_equal(on[0], off[0])
    y = oracle.matmul(x, w, dtype, trans_b=True).reshape(1, S, heads, hd)
    ref = oracle.rope(y, np.broadcast_to(f, y.shape), dtype)
    _close_sum(oracle, ref, on[0], dtype)


def test_residual_add_behind_a_split_matmul(oracle, monkeypatch):
    """2048 x 4096 x 4096 is planned with K split in two: the tile's finisher folds the add."""
    dtype = "bf16"
    M, N, K = 2048, 4096, 4096
    x = make(oracle, (M, K), dtype, 331, "normal")
    w = make(oracle, (N, K), dtype, 332, "normal", scale=0.02)
    r = make(oracle, (M, N), dtype, 333, "normal")

    def build(m):
        tx, tw, tr = m.tensor(x.shape, dtype), m.tensor(w.shape, dtype), m.tensor(r.shape, dtype)
        with m.planner_context(sync=False):
            o = m.add(tr, m.matmul(tx, tw, trans_other=True))
        return (tx, tw, tr), [o]

    (plan, on_flags, on), (_, off_flags, off) = _both_ways(
        monkeypatch, build, lambda t: {t[0]: x, t[1]: w, t[2]: r})
    assert json.loads(plan)["TaskInfos"][0]["Ops"][0]["Config"].get("SplitK") == 2
    assert on_flags == [True] and off_flags == [False]
    assert np.array_equal(on[0], off[0])
    pick = np.sort(np.random.default_rng(7).choice(M, 32, replace=False))
    pick[0], pick[-1] = 0, M - 1
    ref = oracle.binary(np.ascontiguousarray(r[pick]),
                        oracle.matmul(np.ascontiguousarray(x[pick]), w, dtype, trans_b=True), "add", dtype)
    _close_sum(oracle, ref, on[0][pick], dtype)


@pytest.mark.parametrize("onto", ["other", "c"])
def test_result_written_over_an_operand(oracle, monkeypatch, onto):
    """The op's output may be one of its inputs: the residual it adds (h <- h + x @ w, the way a decoder
    layer updates its hidden state in place) or the matmul's own result.  A lane loads its segment of the
    other operand before it stores the same addresses, and stores C before the result."""
    dtype = "bf16"
    M, N, K = 512, 512, 256
    x = make(oracle, (M, K), dtype, 351)
    w = make(oracle, (N, K), dtype, 352, "normal", scale=0.05)
    r = make(oracle, (M, N), dtype, 353)

    def build(m):
        tx, tw, tr = m.tensor(x.shape, dtype), m.tensor(w.shape, dtype), m.tensor(r.shape, dtype)
        with m.planner_context(sync=False):
            y = m.matmul(tx, tw, trans_other=True)
            o = m.add(tr, y, tr if onto == "other" else y)
        return (tx, tw, tr), [o]

    (plan, on_flags, on), (_, off_flags, off) = _both_ways(
        monkeypatch, build, lambda t: {t[0]: x, t[1]: w, t[2]: r})
    assert len(json.loads(plan)["TaskInfos"]) == 1 and on_flags == [True] and off_flags == [False]
    assert np.array_equal(on[0], off[0])
    # (two iterations: written over the residual, the second adds the product to the first's result)
    y = oracle.matmul(x, w, dtype, trans_b=True)
    ref = oracle.binary(r, y, "add", dtype)
    if onto == "other":
        ref = oracle.binary(ref, y, "add", dtype)
    _close_sum(oracle, ref, on[0], dtype)
