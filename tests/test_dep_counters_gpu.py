"""Dependency counters in place of grid barriers (the loop kernel's per-row-block counters in
device memory): each graph runs with the counters and with every barrier kept
(ARKMI_DEP_COUNTERS=0, the default).  The run with counters is checked against the CPU oracle
(the graph evaluated op by op, one rounding per op), and the two runs must agree bit for bit over
several iterations, in the resident loop kernel and in one-shot launches; the executor must
report which barriers it replaced.
The reference orders the same chains with one sync_gpu per op boundary (ark/codegen.cpp:109-158)."""
import numpy as np
import pytest

import llama_ref as R
from helpers import make

pytestmark = pytest.mark.gpu


def _run(m, feeds, fetch, iters, loop_mode=True):
    from ark_amd import Executor
    ex = Executor(m.plan(device_id=0), device_id=0, loop_mode=loop_mode).compile()
    for t, a in feeds.items():
        ex.tensor_write(t, a)
    ex.launch()
    ex.run(iters)
    ex.wait()
    outs = [ex.tensor_read(t) for t in fetch]
    info = ex.info()
    ex.stop()
    return outs, info


def rows_gemm_gemm(m, dt):
    x, w1, w2 = m.tensor([1024, 1024], dt), m.tensor([1024, 2048], dt), m.tensor([2048, 1024], dt)
    return [x, w1, w2], [m.matmul(m.matmul(m.rmsnorm(x), w1), w2)], 2


def gemm_rows_gemm(m, dt):
    x, w1, w2 = m.tensor([1024, 512], dt), m.tensor([512, 1024], dt), m.tensor([1024, 512], dt)
    h = m.matmul(x, w1)
    return [x, w1, w2], [m.matmul(m.softmax(h), w2), m.reduce_sum(h, -1)], 2


def gemm_with_follower_feeds_gemm(m, dt):
    x, w1, w2, r = (m.tensor([1024, 1024], dt), m.tensor([1024, 1024], dt), m.tensor([1024, 1024], dt),
                    m.tensor([1024, 1024], dt))
    with m.planner_context(sync=False):
        h = m.add(r, m.matmul(x, w1))
    return [x, w1, w2, r], [m.matmul(h, w2, trans_other=True)], 1


def projections_attention_projection(m, dt):
    seq, heads, hd = 512, 4, 128
    dim = heads * hd
    x = m.tensor([1, seq, dim], dt)
    wq, wk, wv, wo = (m.tensor([dim, dim], dt) for _ in range(4))
    q = m.reshape(m.matmul(x, wq, trans_other=True), [1, seq, heads, hd])
    k = m.reshape(m.matmul(x, wk, trans_other=True), [1, seq, heads, hd])
    v = m.reshape(m.matmul(x, wv, trans_other=True), [1, seq, heads, hd])
    a = m.reshape(m.attention(q, k, v, hd ** -0.5, causal=True), [1, seq, dim])
    return [x, wq, wk, wv, wo], [m.matmul(a, wo, trans_other=True)], 2


def in_place_residual_loop(m, dt):
    """x <- x + rmsnorm(x) @ w: every iteration reads what the previous one wrote, so the boundary
    between iterations keeps its grid barrier.  (At this size the ops run on sub-ranges of the
    workgroups, whose barriers are never replaced: the graph checks that nothing else changes.)"""
    x, w = m.tensor([512, 512], dt), m.tensor([512, 512], dt)
    h = m.matmul(m.rmsnorm(x), w)
    out = m.add(x, m.mul(h, 0.01), output=x)
    return [x, w], [out], 0


# ---- the same graphs on the oracle: inputs in the order the graph functions list them ----------
def _ref_rows_gemm_gemm(O, v, dt):
    x, w1, w2 = v
    return [O.matmul(O.matmul(O.rmsnorm(x, None, dt), w1, dt), w2, dt)]


def _ref_gemm_rows_gemm(O, v, dt):
    x, w1, w2 = v
    h = O.matmul(x, w1, dt)
    return [O.matmul(O.softmax(h, dt), w2, dt), O.reduce(h, -1, "sum", dt)]


def _ref_gemm_with_follower_feeds_gemm(O, v, dt):
    x, w1, w2, r = v
    return [O.matmul(O.binary(r, O.matmul(x, w1, dt), "add", dt), w2, dt, trans_b=True)]


def _ref_projections_attention_projection(O, v, dt):
    x, wq, wk, wv, wo = v
    return [R.attention(O, x, wq, wk, wv, wo, None, _causal(x.shape[1]), 4, dt)]


def _causal(seq):
    mask = np.zeros((1, 1, seq, seq), np.float32)
    mask[0, 0][np.triu_indices(seq, 1)] = -np.inf
    return mask


def _ref_in_place_residual_loop(O, v, dt, iters=4):
    x, w = v
    for _ in range(iters):
        h = O.matmul(O.rmsnorm(x, None, dt), w, dt)
        x = O.binary(x, O.scalar(h, 0.01, "mul", dt), "add", dt)
    return [x]


GRAPHS = {f.__name__: f for f in (rows_gemm_gemm, gemm_rows_gemm, gemm_with_follower_feeds_gemm,
                                  projections_attention_projection, in_place_residual_loop)}


@pytest.mark.parametrize("loop_mode", [True, False])
@pytest.mark.parametrize("graph", sorted(GRAPHS))
def test_counters_give_the_barriers_results(oracle, graph, loop_mode, monkeypatch):
    from ark_amd import Model
    dtype = "bf16" if "attention" in graph else "fp16"
    results = {}
    for counters in ("0", "1"):
        monkeypatch.setenv("ARKMI_DEP_COUNTERS", counters)
        m = Model()
        ins, fetch, least = GRAPHS[graph](m, dtype)
        feeds = {t: make(oracle, tuple(t.shape), dtype, 700 + i, "uniform", -0.5, 0.5) for i, t in enumerate(ins)}
        outs, info = _run(m, feeds, fetch, iters=4, loop_mode=loop_mode)
        if counters == "0":
            assert info["barriers_counted"] == 0
        else:
            assert info["barriers_counted"] >= least, info
            assert least == 0 or info["iteration_sync"] == 2
        results[counters] = outs
    for a, b in zip(results["0"], results["1"]):
        assert np.array_equal(a, b), graph
    # against the oracle: the counter run, judged like every composite (largest and rms difference
    # relative to the reference's; a missed dependency reads stale or unwritten rows, an O(1) error)
    refs = globals()["_ref_" + graph](oracle, [feeds[t] for t in ins], dtype)
    for ref, got in zip(refs, results["1"]):
        mx, rms = R.composite_error(oracle, ref.reshape(got.shape), got, dtype)
        tol = 3e-2 if "attention" in graph else 1e-2
        assert mx <= tol and rms <= tol, (graph, mx, rms)


def test_counters_across_commands_and_relaunch(oracle, monkeypatch):
    """The counters count iterations since the kernel's launch: several run() commands on one
    resident kernel, then a stop and a second launch (counters start from zero again)."""
    from ark_amd import Model, Executor
    dtype = "fp16"
    m = Model()
    ins, fetch, _ = rows_gemm_gemm(m, dtype)
    feeds = {t: make(oracle, tuple(t.shape), dtype, 800 + i, "uniform", -0.5, 0.5) for i, t in enumerate(ins)}
    monkeypatch.setenv("ARKMI_DEP_COUNTERS", "0")
    (want,), _ = _run(m, feeds, fetch, iters=1)
    monkeypatch.setenv("ARKMI_DEP_COUNTERS", "1")
    ex = Executor(m.plan(device_id=0), device_id=0).compile()
    assert ex.info()["barriers_counted"] >= 2
    for t, a in feeds.items():
        ex.tensor_write(t, a)
    for launch in range(2):
        ex.launch()
        for n in (1, 3, 2):
            ex.tensor_write(fetch[0], np.zeros(fetch[0].shape, np.float16))
            ex.run(n)
            ex.wait()
            assert np.array_equal(ex.tensor_read(fetch[0]), want), (launch, n)
        ex.stop()


@pytest.mark.parametrize("fused", [True, "attention", "side_by_side"])
def test_decoder_layer_with_counters(oracle, fused, monkeypatch):
    """The fused Llama decoder layer (RMSNorm -> projections with the rotation on their tiles ->
    attention -> output projection with the residual -> RMSNorm -> SwiGLU -> down projection with the
    residual): with counters every barrier of the chain is replaced; results bit for bit."""
    import test_llama_gpu as L
    from ark_amd import Model
    dtype, seq, dim, heads, hidden = "bf16", 2048, 4096, 32, 11008  # the size at which every op fills the grid
    results = {}
    for counters in ("0", "1"):
        monkeypatch.setenv("ARKMI_DEP_COUNTERS", counters)
        m = Model()
        blk, vals, x, freqs, mask = L._layer_case(oracle, m, seq, dim, heads, hidden, dtype, 400)  # the inputs of the oracle-checked full-size test
        tx = m.tensor([1, seq, dim], dtype)
        tf = m.tensor([1, seq, 1, dim // heads], dtype)
        tm = m.tensor([1, 1, seq, seq], dtype)
        side_by_side = fused == "side_by_side"  # query and key projections on the two halves of the processors
        kind = "attention" if side_by_side else fused
        out = blk.forward(tx, tf, tm, fused=bool(kind), causal=(kind == "attention"), pair_on=256 if side_by_side else None)
        feeds = {tx: x, tf: oracle.to_storage(freqs, dtype), tm: oracle.to_storage(mask, dtype)}
        if kind == "attention":
            del feeds[tm]
        feeds.update({t: vals[name] for name, t in blk.params().items()})
        (got,), info = _run(m, feeds, [out], iters=2)
        if counters == "1":
            assert info["barriers_counted"] >= 4, info
        results[counters] = got
    assert np.array_equal(results["0"], results["1"])
    # the run with counters against the reference composition on the oracle, on 64 sampled positions
    pick = np.sort(np.random.default_rng(11).choice(seq, 64, replace=False))
    pick[0], pick[-1] = 0, seq - 1
    ref = R.transformer_block(oracle, x, vals, freqs, mask, heads, dtype, q_rows=pick)
    mx, rms = R.composite_error(oracle, ref, results["1"][:, pick], dtype)
    assert mx <= 1e-2 and rms <= 1e-2, (mx, rms)
