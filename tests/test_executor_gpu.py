"""GPU tests of the Model -> Planner -> Executor path (the persistent loop
kernel), through the C ABI, against the CPU oracle.

Mirrors how the reference tests ops: build a model, run one iteration in the
executor, compare with the op's host baseline (ark/ops/ops_test_common.cpp:
34-224).  Shapes follow ark/ops/ops_{arithmetic,math,scalar,cast,rope,
transpose,reduce,matmul}_test.cpp.
"""
import json

import numpy as np
import pytest

from helpers import make

pytestmark = pytest.mark.gpu


def run_model(m, feeds, fetches, iters=1, loop_mode=True, trace=False, plan=None):
    from ark_amd import Executor
    plan = plan or m.plan(device_id=0)
    ex = Executor(plan, device_id=0, loop_mode=loop_mode, trace=trace)
    ex.compile()
    for t, a in feeds.items():
        ex.tensor_write(t, a)
    ex.launch()
    ex.run(iters)
    ex.wait()
    outs = [ex.tensor_read(t) for t in fetches]
    ex.stop()
    return outs, ex, plan


def close(oracle, ref, got, dtype, tol):
    rel, abs_rest, mx = oracle.max_rel_error(ref, got, dtype)
    assert rel <= tol and abs_rest <= tol * max(mx, 1e-30), (rel, abs_rest, mx)


# ---------------------------------------------------------------- elementwise
@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("kind", ["add", "sub", "mul", "div"])
def test_arithmetic(oracle, kind, dtype):
    from ark_amd import Model
    # exact (ops_arithmetic_test.cpp asserts max_diff == 0), incl. broadcasting
    for sa, sb in [((2, 3, 64, 96), (2, 3, 64, 96)), ((4, 1024), (1,)), ((3, 1, 1024), (1, 4, 1)),
                   ((1, 5, 33), (7, 1, 33)), ((8192,), (8192,))]:
        m = Model()
        a = make(oracle, sa, dtype, 1, "uniform", -2, 2)
        b = make(oracle, sb, dtype, 2, "uniform", 0.5, 2)
        ta, tb = m.tensor(sa, dtype), m.tensor(sb, dtype)
        out = getattr(m, kind)(ta, tb)
        (got,), _, _ = run_model(m, {ta: a, tb: b}, [out])
        ref = oracle.binary(a, b, kind, dtype)
        assert got.shape == ref.shape
        assert np.array_equal(got, ref), (kind, dtype, sa, sb)


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("kind,tol", [("exp", 1e-5), ("gelu", 1e-6), ("relu", 0), ("rsqrt", 1e-4),
                                      ("sigmoid", 1e-5), ("sqrt", 1e-6)])
def test_math(oracle, kind, tol, dtype):
    from ark_amd import Model
    m = Model()
    shape = (4, 2, 1024)
    lo = 0.1 if kind in ("rsqrt", "sqrt") else -3.0
    x = make(oracle, shape, dtype, 3, "uniform", lo, 3.0)
    t = m.tensor(shape, dtype)
    out = getattr(m, kind)(t)
    (got,), _, _ = run_model(m, {t: x}, [out])
    ref = oracle.unary(x, kind, dtype)
    if tol == 0:
        assert np.array_equal(got, ref)
    else:
        # The reference asserts on the maximum absolute difference
        # (ops_math_test.cpp:120-366) for inputs in (-0.1, 0.1); here inputs
        # reach 3, so the bound scales with the result magnitude, plus one
        # storage ulp where the fp32 results differ in the last bit.
        r, g = oracle.to_f32(ref, dtype).astype(np.float64), oracle.to_f32(got, dtype).astype(np.float64)
        ulp = {"fp32": 0.0, "fp16": 2.0 ** -10, "bf16": 2.0 ** -7}[dtype]
        bound = tol * np.maximum(1.0, np.abs(r)) + ulp * np.abs(r)
        assert np.all(np.abs(r - g) <= bound), float(np.max(np.abs(r - g) - bound))


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_scalar_ops(oracle, dtype):
    from ark_amd import Model
    m = Model()
    shape = (4, 2, 50)
    x = make(oracle, shape, dtype, 4)
    t = m.tensor(shape, dtype)
    o1 = m.add(t, 0.7)
    o2 = m.sub(t, 0.7)
    o3 = m.mul(t, 0.7)
    o4 = m.div(t, 0.7)
    c = m.constant(7.0, (3, 5), dtype)
    (g1, g2, g3, g4, gc), _, _ = run_model(m, {t: x}, [o1, o2, o3, o4, c])
    assert np.array_equal(g1, oracle.scalar(x, 0.7, "add", dtype))
    assert np.array_equal(g2, oracle.scalar(x, -0.7, "add", dtype))
    assert np.array_equal(g3, oracle.scalar(x, 0.7, "mul", dtype))
    assert np.array_equal(g4, oracle.scalar(x, np.float32(1) / np.float32(0.7), "mul", dtype))
    assert np.array_equal(gc, oracle.to_storage(np.full((3, 5), 7.0, np.float32), dtype))


@pytest.mark.parametrize("src,dst", [("fp32", "fp16"), ("fp16", "fp32"), ("fp32", "bf16"),
                                     ("bf16", "fp32"), ("fp16", "bf16"), ("int32", "fp32"),
                                     ("fp32", "int32"), ("fp16", "int32"), ("int32", "fp16")])
def test_cast(oracle, src, dst):
    from ark_amd import Model
    m = Model()
    shape = (4, 2, 1000)
    if src == "int32":
        x = np.random.default_rng(5).integers(-1000, 1000, shape).astype(np.int32)
        xf = x.astype(np.float32)
    else:
        x = make(oracle, shape, src, 5, "uniform", -100, 100)
        xf = oracle.to_f32(x, src)
    t = m.tensor(shape, src)
    out = m.cast(t, dst)
    (got,), _, _ = run_model(m, {t: x}, [out])
    ref = np.trunc(xf).astype(np.int32) if dst == "int32" else oracle.to_storage(xf, dst)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_rope(oracle, dtype):
    from ark_amd import Model
    m = Model()
    a = make(oracle, (1, 32, 32, 256), dtype, 6)
    b = make(oracle, (1, 32, 1, 256), dtype, 7)
    ta, tb = m.tensor(a.shape, dtype), m.tensor(b.shape, dtype)
    out = m.rope(ta, tb)
    (got,), _, _ = run_model(m, {ta: a, tb: b}, [out])
    ref = oracle.rope(a, np.broadcast_to(b, a.shape), dtype)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("perm", [(0, 2, 1, 3), (0, 2, 3, 1), (0, 1, 3, 2), (3, 2, 1, 0), (1, 0, 2, 3)])
def test_transpose(oracle, perm):
    from ark_amd import Model
    m = Model()
    x = make(oracle, (2, 5, 24, 40), "fp16", 8)
    t = m.tensor(x.shape, "fp16")
    out = m.transpose(t, perm)
    (got,), _, _ = run_model(m, {t: x}, [out])
    assert np.array_equal(got, np.transpose(x, perm))


# ---------------------------------------------------------------- row ops and matmul
@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_reduce_and_fused_rows(oracle, dtype):
    from ark_amd import Model
    tol = {"fp32": 1e-3, "fp16": 1e-3, "bf16": 2.0 ** -7}[dtype]
    m = Model()
    shape = (7, 2, 4, 1024)
    x = make(oracle, shape, dtype, 9)
    w = np.random.default_rng(1).uniform(0.5, 1.5, 1024).astype(np.float32)
    t = m.tensor(shape, dtype)
    tw = m.tensor((1, 1, 1024), "fp32")
    outs = [m.reduce_sum(t, -1), m.reduce_max(t, 3, keepdims=False), m.reduce_mean(t, -1),
            m.softmax(t), m.layernorm(t, 1e-6), m.rmsnorm(t, tw, 1e-6)]
    got, _, _ = run_model(m, {t: x, tw: w.reshape(1, 1, 1024)}, outs)
    refs = [oracle.reduce(x, -1, "sum", dtype), oracle.reduce(x, -1, "max", dtype, keepdims=False),
            oracle.reduce(x, -1, "mean", dtype), oracle.softmax(x, dtype),
            oracle.layernorm(x, dtype, 1e-6), oracle.rmsnorm(x, w, dtype, 1e-6)]
    assert np.array_equal(got[1], refs[1])
    for g, r in zip(got, refs):
        assert g.shape == r.shape
        close(oracle, r, g, dtype, tol)


def test_softmax_composition_matches_fused(oracle):
    """The reference's 5-op softmax (python/ark/ops.py:491-500) as separate ops."""
    from ark_amd import Model
    dtype = "fp32"
    m = Model()
    x = make(oracle, (64, 512), dtype, 10)
    t = m.tensor(x.shape, dtype)
    mx = m.reduce_max(t, -1)
    o = m.sub(t, mx)
    o = m.exp(o, o)
    s = m.reduce_sum(o, -1)
    o = m.div(o, s, o)
    (got,), _, _ = run_model(m, {t: x}, [o])
    close(oracle, oracle.softmax(x, dtype), got, dtype, 1e-5)


@pytest.mark.parametrize("dtype", ["fp16", "bf16", "fp32"])
@pytest.mark.parametrize("cols", [256, 2048, 200])
def test_softmax_scaled_masked(oracle, dtype, cols):
    """softmax(x * scale + mask) as one op equals the reference's chain
    ScalarMul -> Add(mask) -> softmax (examples/llama/model.py:426-433) evaluated
    on the oracle; the mask ([1, 1, rows, cols], -inf above the diagonal)
    broadcasts over the two leading axes."""
    from ark_amd import Model
    n, c, rows = 2, 3, 64
    x = make(oracle, (n, c, rows, cols), dtype, 41)
    mask = np.zeros((1, 1, rows, cols), np.float32)
    mask[0, 0][np.triu_indices(rows, k=1, m=cols)] = -np.inf
    mask_s = oracle.to_storage(mask, dtype)
    scale = 0.0883883
    m = Model()
    t, tm = m.tensor(x.shape, dtype), m.tensor(mask.shape, dtype)
    o = m.softmax(t, mask=tm, scale=scale)
    o2 = m.softmax(t, scale=scale)
    (got, got2), _, _ = run_model(m, {t: x, tm: mask_s}, [o, o2])
    scaled = oracle.scalar(x, scale, "mul", dtype)
    ref = oracle.softmax(oracle.binary(scaled, mask_s, "add", dtype), dtype)
    ref2 = oracle.softmax(scaled, dtype)
    tol = 1e-5 if dtype == "fp32" else 1e-2  # the chain rounds twice before the softmax, the fused op never
    close(oracle, ref, got, dtype, tol)
    close(oracle, ref2, got2, dtype, tol)
    assert np.all(oracle.to_f32(got, dtype)[..., np.triu_indices(rows, k=1, m=cols)[0], np.triu_indices(rows, k=1, m=cols)[1]] == 0)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("trans_other", [False, True])
def test_matmul(oracle, dtype, trans_other):
    from ark_amd import Model
    for (bs, M, N, K) in [((), 256, 256, 128), ((3,), 128, 256, 64), ((2, 2), 128, 128, 192)]:
        m = Model()
        a = make(oracle, bs + (M, K), dtype, 11, "uniform")
        b = make(oracle, (N, K) if trans_other else (K, N), dtype, 12, "uniform")
        ta, tb = m.tensor(a.shape, dtype), m.tensor(b.shape, dtype)
        c = m.matmul(ta, tb, trans_other=trans_other)
        (got,), _, _ = run_model(m, {ta: a, tb: b}, [c])
        ref = oracle.matmul(a, b, dtype, trans_b=trans_other)
        assert got.shape == ref.shape
        close(oracle, ref, got, dtype, 1e-2)


@pytest.mark.parametrize("trans_other", [False, True])
def test_matmul_transposed_input(oracle, trans_other):
    """tn / tt through the plan (ops_matmul_test.cpp:457-511), batched."""
    from ark_amd import Model
    dtype = "fp16"
    for (bs, M, N, K) in [((), 128, 128, 64), ((2,), 256, 384, 128)]:
        m = Model()
        a = make(oracle, bs + (K, M), dtype, 15, "uniform")
        b = make(oracle, (N, K) if trans_other else (K, N), dtype, 16, "uniform")
        ta, tb = m.tensor(a.shape, dtype), m.tensor(b.shape, dtype)
        c = m.matmul(ta, tb, trans_input=True, trans_other=trans_other)
        (got,), _, _ = run_model(m, {ta: a, tb: b}, [c])
        ref = oracle.matmul(a, b, dtype, trans_a=True, trans_b=trans_other)
        assert got.shape == ref.shape
        close(oracle, ref, got, dtype, 1e-2)


def test_matmul_fp32(oracle):
    """fp32 matmul through the plan (ops_matmul_test.cpp:364-397: 128x64 . 64x256), batched too."""
    from ark_amd import Model
    dtype = "fp32"
    for (bs, M, N, K) in [((), 128, 256, 64), ((3,), 256, 128, 128)]:
        m = Model()
        a = make(oracle, bs + (M, K), dtype, 17, "uniform")
        b = make(oracle, (K, N), dtype, 18, "uniform")
        ta, tb = m.tensor(a.shape, dtype), m.tensor(b.shape, dtype)
        c = m.matmul(ta, tb)
        (got,), _, _ = run_model(m, {ta: a, tb: b}, [c])
        close(oracle, oracle.matmul(a, b, dtype), got, dtype, 1e-4)


def test_matmul_padded(oracle):
    """A 2x9 result inside a 128x128 padded tile (ops_matmul_test.cpp:527-543)."""
    from ark_amd import Model
    dtype = "fp16"
    m = Model()
    a = make(oracle, (2, 64), dtype, 13, "uniform")
    b = make(oracle, (64, 9), dtype, 14, "uniform")
    ta = m.tensor((2, 64), dtype, strides=(128, 64), padded_shape=(128, 64))
    tb = m.tensor((64, 9), dtype, strides=(64, 128), padded_shape=(64, 128))
    c = m.matmul(ta, tb)
    assert c.shape == [2, 9] and c.padded_shape == [128, 128]
    (got,), _, _ = run_model(m, {ta: a, tb: b}, [c])
    close(oracle, oracle.matmul(a, b, dtype), got, dtype, 1e-2)


# ---------------------------------------------------------------- plans, schedule, life cycle
def test_fused_context_and_trace(oracle):
    """ScalarMul + Add fused into one task by a PlannerContext with sync(False)
    (ark/api/planner_test.cpp:285-319), and task placement recorded by the
    kernel equal to the task_seq formula, bit for bit."""
    import json
    from ark_amd import Model, plan_schedule
    dtype = "fp32"
    m = Model()
    t0 = m.tensor((1024, 64), dtype)
    t1 = m.tensor((1024, 64), dtype)
    cfg = {"NumWarps": 8, "SramBytes": 0, "Tile": [8, 64], "NumTasks": 128}
    with m.planner_context(processor_range=[0, 48], sync=False, config=cfg):
        t2 = m.mul(t0, 0.7)
        t3 = m.add(t2, t1)
    t4 = m.relu(t3)
    x0, x1 = make(oracle, (1024, 64), dtype, 15), make(oracle, (1024, 64), dtype, 16)
    (got,), ex, plan = run_model(m, {t0: x0, t1: x1}, [t4], trace=True)
    pj = json.loads(plan)
    assert len(pj["TaskInfos"]) == 2 and len(pj["TaskInfos"][0]["Ops"]) == 2
    ref = oracle.unary(oracle.binary(oracle.scalar(x0, 0.7, "mul", dtype), x1, "add", dtype), "relu", dtype)
    assert np.array_equal(got, ref)
    sch = plan_schedule(plan)
    grid = sch["NumProcessors"]
    gi = 0
    for st in sch["Steps"]:
        if st["Kind"] != "TaskSeq":
            continue
        pb, pe, ps, pc, tb, te, ts, gran, nslots, sw, ss, tid = st["Args"]
        trace = ex.read_trace(gi)
        expect = {}
        for block in range(grid):
            for k in range(nslots):
                for order, task in enumerate(oracle.task_seq(block, grid, (pb, pe, ps), pc, (tb, te, ts),
                                                             gran, nslots, k)):
                    assert task not in expect
                    expect[task] = (block, k, order)
        assert sorted(expect) == list(range(tb, te, ts))  # every task exactly once
        for i, task in enumerate(range(tb, te, ts)):
            assert trace[i] == expect[task], (gi, task, trace[i], expect[task])
        gi += 1
    assert gi == 2


def test_lifecycle(oracle):
    from ark_amd import Model, Executor, ArkmiError
    dtype = "fp32"
    m = Model()
    t = m.tensor((4, 64), dtype)
    o = m.add(t, 1.0, t)  # in place: every run adds 1
    plan = m.plan(device_id=0)
    ex = Executor(plan)
    with pytest.raises(ArkmiError) as e:
        ex.launch()  # not compiled
    assert e.value.kind == "InvalidUsageError"
    ex.compile()
    x = np.zeros((4, 64), np.float32)
    ex.tensor_write(t, x)
    ex.launch()
    ex.launch()  # second launch is ignored with a warning
    ex.run(3)
    ex.wait()
    assert np.all(ex.tensor_read(o) == 3)
    ex.run(2)
    ex.run(1)  # blocks until the previous run is done
    ms = ex.stop()
    assert ms > 0
    assert np.all(ex.tensor_read(o) == 6)
    ex.launch()  # re-launch after stop
    ex.run(1)
    ex.stop()
    assert np.all(ex.tensor_read(o) == 7)
    assert ex.info()["iterations_done"] == 1
    with pytest.raises(ArkmiError) as e:
        ex._copy(t, x.ctypes.data, 16, True)  # size mismatch
    assert e.value.kind == "InvalidUsageError"
    ex.destroy()
    assert ex.info()["destroyed"] == 1
    # no-loop mode: one kernel launch per run()
    ex2 = Executor(plan, loop_mode=False).compile()
    ex2.tensor_write(t, x)
    ex2.launch()
    ex2.run(4)
    ex2.wait()
    assert np.all(ex2.tensor_read(o) == 4)
    ex2.stop()


def test_idle_exit_and_resume(oracle, monkeypatch):
    """The loop kernel leaves by itself when no command arrives within its idle
    limit, and run() brings it back."""
    import time
    from ark_amd import Model, Executor
    monkeypatch.setenv("ARKMI_IDLE_EXIT_MS", "200")
    m = Model()
    t = m.tensor((2, 64), "fp32")
    o = m.add(t, 1.0, t)
    ex = Executor(m.plan(device_id=0)).compile()
    ex.tensor_write(t, np.zeros((2, 64), np.float32))
    ex.launch()
    ex.run(1)
    ex.wait()
    time.sleep(0.6)  # idle limit passes, kernel exits
    ex.run(2)
    ex.wait()
    assert np.all(ex.tensor_read(o) == 3)
    ex.stop()


def test_strided_tensor_io(oracle):
    """tensor_write / tensor_read on offset, strided views (executor_test.cpp:95-148)."""
    from ark_amd import Model
    m = Model()
    base = m.tensor((4, 8, 64), "fp32")
    view = m.refer(base, shape=(2, 4, 32), strides=(4, 8, 64), offsets=(1, 2, 16))
    out = m.mul(view, 2.0)
    m.noop(base)
    x = make(oracle, (2, 4, 32), "fp32", 17)
    (got, whole), _, _ = run_model(m, {view: x}, [out, base])
    assert np.array_equal(got, x * 2)
    expect = np.zeros((4, 8, 64), np.float32)  # arena is zero-filled
    expect[1:3, 2:6, 16:48] = x
    assert np.array_equal(whole, expect)


def test_unsupported_and_invalid_plans():
    import json
    from ark_amd import Model, Executor, ArkmiError
    with pytest.raises(ArkmiError) as e:
        Executor("not json")
    assert e.value.kind == "PlanError"
    with pytest.raises(ArkmiError) as e:
        Executor("{}", device_id=99)
    assert e.value.kind == "InvalidUsageError"
    m = Model()
    t = m.tensor((128, 64), "int32")
    m.matmul(t, m.tensor((64, 128), "int32"))
    with pytest.raises(ArkmiError) as e:
        m.plan(device_id=0)  # no integer GEMM on this backend
    assert e.value.kind == "PlanError"


def test_elementwise_chain_uses_local_syncs(oracle):
    """A chain of same-shape elementwise ops (SiLU * up: sigmoid -> mul -> mul)
    depends only on what each workgroup wrote itself: the grid barriers between
    the steps become workgroup-local syncs, and the result stays exact."""
    from ark_amd import Model, Executor
    dtype = "bf16"
    g = make(oracle, (512, 1024), dtype, 61)
    u = make(oracle, (512, 1024), dtype, 62)
    m = Model()
    tg, tu = m.tensor(g.shape, dtype), m.tensor(u.shape, dtype)
    sig = m.sigmoid(tg, m.tensor(g.shape, dtype))
    silu = m.mul(tg, sig)
    out = m.mul(silu, tu)
    (got,), ex, _ = run_model(m, {tg: g, tu: u}, [out], iters=3)
    info = ex.info()
    assert info["barriers_local"] == 2, info
    ref = oracle.binary(oracle.binary(g, oracle.unary(g, "sigmoid", dtype), "mul", dtype), u, "mul", dtype)
    close(oracle, ref, got, dtype, 1e-2)


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_silu_mul(oracle, dtype):
    """silu(g) * u as one op against the reference's chain sigmoid -> mul -> mul
    (examples/llama/model.py:281-293, 329-331) on the oracle; the chain rounds
    to the storage type three times, the fused op once."""
    from ark_amd import Model
    g = make(oracle, (3, 64, 520), dtype, 71)
    u = make(oracle, (3, 64, 520), dtype, 72)
    m = Model()
    tg, tu = m.tensor(g.shape, dtype), m.tensor(u.shape, dtype)
    o = m.silu_mul(tg, tu)
    (got,), _, _ = run_model(m, {tg: g, tu: u}, [o])
    ref = oracle.binary(oracle.binary(g, oracle.unary(g, "sigmoid", dtype), "mul", dtype), u, "mul", dtype)
    close(oracle, ref, got, dtype, 1e-5 if dtype == "fp32" else 2e-2)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("heads,hd", [(8, 128), (6, 64), (4, 96)])
def test_rope_rides_on_gemm_tiles_through_reshape(oracle, dtype, heads, hd):
    """Matmul -> reshape [1, S, heads, hd] -> Rope with a [1, S, 1, hd] table in one
    sync(False) context: the rotation runs per GEMM tile over the GEMM's [S, heads * hd]
    view, the table wrapping every hd columns.  Same results as the two ops apart
    (bit-exact: the GEMM's rounded output is the rotation's input either way)."""
    from ark_amd import Model
    S, K = 384, 256
    x = make(oracle, (1, S, K), dtype, 41)
    w = make(oracle, (heads * hd, K), dtype, 42, "normal", 0, 0.05)
    f = make(oracle, (1, S, 1, hd), dtype, 43)
    outs = []
    for fuse in (False, True):
        m = Model()
        tx, tw, tf = m.tensor(x.shape, dtype), m.tensor(w.shape, dtype), m.tensor(f.shape, dtype)
        if fuse:
            with m.planner_context(sync=False):
                o = m.rope(m.reshape(m.matmul(tx, tw, trans_other=True), [1, S, heads, hd]), tf)
        else:
            o = m.rope(m.reshape(m.matmul(tx, tw, trans_other=True), [1, S, heads, hd]), tf)
        (got,), _, plan = run_model(m, {tx: x, tw: w, tf: f}, [o], iters=2)
        tasks = json.loads(plan)["TaskInfos"]
        assert len(tasks) == (1 if fuse else 2)
        if fuse:
            assert "ViewAs" in tasks[0]["Ops"][1]["Config"]
        outs.append(got)
    assert np.array_equal(outs[0], outs[1])
    y = oracle.matmul(x, w, dtype, trans_b=True).reshape(1, S, heads, hd)
    ref = oracle.rope(y, np.broadcast_to(f, y.shape), dtype)
    # a0 b0 - a1 b1 cancels, so one rounding step of the GEMM's output (whose summation
    # order differs from the oracle's) is not small relative to a single result: bound
    # the error relative to the largest result and in rms instead
    t, g = (oracle.to_f32(a, dtype).astype(np.float64) for a in (ref, outs[1]))
    assert np.abs(t - g).max() <= 1e-2 * np.abs(t).max()
    assert np.sqrt(((t - g) ** 2).mean()) <= 2e-3 * np.sqrt((t * t).mean())


# ------------------------------------------------ what separates two iterations of one run(n)
def test_iterations_without_shared_data_run_without_barrier(oracle, monkeypatch):
    """Independent row ops over the same input: an iteration only rewrites its own
    outputs, task by task on the same workgroups, so iterations of one run(n) can be
    separated by a workgroup-local sync, and many iterations give the one-iteration
    result.  (Streaming-only bodies keep the barrier by default, for speed: the
    variable asks for what the data allows.)"""
    from ark_amd import Model
    monkeypatch.setenv("ARKMI_ITERATION_BARRIER", "0")
    dtype = "fp16"
    x = make(oracle, (4096, 1024), dtype, 5)
    m = Model()
    tx = m.tensor(x.shape, dtype)
    o1, o2 = m.softmax(tx), m.reduce_sum(tx, -1)
    (g1, g2), ex, _ = run_model(m, {tx: x}, [o1, o2], iters=7)
    assert ex.info()["iteration_sync"] == 1, ex.info()
    close(oracle, oracle.softmax(x, dtype), g1, dtype, 1e-3)
    close(oracle, oracle.reduce(x, -1, "sum", dtype), g2, dtype, 1e-3)


def test_iteration_with_own_data_only_in_place(oracle, monkeypatch):
    """x <- x + 1 in place: every task re-reads what the same lanes wrote one iteration
    earlier; n iterations add n."""
    from ark_amd import Model
    monkeypatch.setenv("ARKMI_ITERATION_BARRIER", "0")
    x = make(oracle, (256, 2048), "fp32", 6)
    m = Model()
    tx = m.tensor(x.shape, "fp32")
    m.add(tx, 1.0, tx)
    (got,), ex, _ = run_model(m, {tx: x}, [tx], iters=9)
    assert ex.info()["iteration_sync"] == 1, ex.info()
    want = x.copy()
    for _ in range(9):
        want = oracle.scalar(want, 1.0, "add", "fp32")
    assert np.array_equal(got, want)


def test_iteration_that_feeds_other_workgroups_keeps_barrier(oracle, monkeypatch):
    """y <- transpose(x); x <- y + 1: the next iteration's transpose reads elements other
    workgroups wrote, so the grid barrier between iterations stays; the result after n
    iterations matches n applications on the host."""
    from ark_amd import Model
    monkeypatch.setenv("ARKMI_ITERATION_BARRIER", "0")
    x = make(oracle, (1, 1, 512, 512), "fp32", 7)
    m = Model()
    tx = m.tensor(x.shape, "fp32")
    ty = m.transpose(tx, [0, 1, 3, 2])
    m.add(ty, 1.0, tx)
    n = 5
    (got,), ex, _ = run_model(m, {tx: x}, [tx], iters=n)
    assert ex.info()["iteration_sync"] == 2, ex.info()
    want = x.copy()
    for _ in range(n):
        want = np.ascontiguousarray(want.transpose(0, 1, 3, 2)) + np.float32(1.0)
    assert np.array_equal(got, want)


def test_skinny_matmul_keeps_iteration_barrier(oracle, monkeypatch):
    """The skinny matmul finishes split-K partial sums in scratch memory shared between
    workgroups: iterations stay separated by the grid barrier."""
    from ark_amd import Model
    monkeypatch.setenv("ARKMI_ITERATION_BARRIER", "0")
    dtype = "bf16"
    x = make(oracle, (1, 4096), dtype, 8)
    w = make(oracle, (4096, 4096), dtype, 9, "normal", 0, 0.02)
    m = Model()
    tx, tw = m.tensor(x.shape, dtype), m.tensor(w.shape, dtype)
    o = m.matmul(tx, tw)
    (got,), ex, _ = run_model(m, {tx: x, tw: w}, [o], iters=6)
    assert ex.info()["iteration_sync"] == 2, ex.info()
    close(oracle, oracle.matmul(x, w, dtype), got, dtype, 1e-2)


def test_gemm_iterations_run_without_barrier(oracle):
    """A GEMM rewrites each output tile on the workgroup that wrote it before: no grid
    barrier between iterations by default, same result after many."""
    from ark_amd import Model
    dtype = "fp16"
    a = make(oracle, (512, 256), dtype, 11)
    b = make(oracle, (256, 512), dtype, 12)
    m = Model()
    ta, tb = m.tensor(a.shape, dtype), m.tensor(b.shape, dtype)
    o = m.matmul(ta, tb)
    (got,), ex, _ = run_model(m, {ta: a, tb: b}, [o], iters=8)
    assert ex.info()["iteration_sync"] == 1, ex.info()
    close(oracle, oracle.matmul(a, b, dtype), got, dtype, 1e-2)


# ---------------------------------------------------------------- reductions over any axis
@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("shape,axis,keep", [((7, 2, 4, 1024), 0, True), ((1, 2, 4, 1024), 1, True),
                                             ((1, 1, 7, 8192), 2, True), ((7, 2, 4, 1024), 1, False),
                                             ((3, 5, 6, 40), 2, False), ((5, 33), 0, True), ((4, 3, 130), -2, False)])
def test_reduce_over_leading_axes(oracle, shape, axis, keep, dtype):
    """ops_reduce_test.cpp:215-252, 282-295 (axes 0, 1, 2 of 4-D tensors, fp32 and fp16) plus
    shapes of lower rank and ragged extents; sum, max and mean share the walk."""
    from ark_amd import Model
    x = make(oracle, shape, dtype, 21)
    m = Model()
    t = m.tensor(shape, dtype)
    outs = [m.reduce_sum(t, axis, keepdims=keep), m.reduce_max(t, axis, keepdims=keep),
            m.reduce_mean(t, axis, keepdims=keep)]
    got, _, _ = run_model(m, {t: x}, outs)
    tol = {"fp32": 1e-3, "fp16": 1e-3, "bf16": 2.0 ** -7}[dtype]
    for g, kind in zip(got, ("sum", "max", "mean")):
        ref = oracle.reduce(x, axis, kind, dtype, keepdims=keep)
        assert g.shape == ref.shape
        if kind == "max":
            assert np.array_equal(g, ref)
        else:
            close(oracle, ref, g, dtype, tol)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("shape", [(128, 128, 64), (256, 384, 192), (512, 1280, 256), (2, 384, 256, 128)])
def test_swiglu_matches_chain(oracle, dtype, shape):
    """silu(x w1^T) * (x w3^T) as one op against the reference's chain (two matmuls,
    sigmoid, mul, mul: examples/llama/model.py:326-331) on the oracle.  The chain rounds
    both products and two more intermediates to the storage type, the op rounds once:
    bounds on max|diff| / max|ref| and rms(diff) / rms(ref), and the op must be at least
    as close to float64 as the chain."""
    from ark_amd import Model
    *bs, M, H, K = shape
    x = make(oracle, tuple(bs) + (M, K), dtype, 31)
    w1 = make(oracle, (H, K), dtype, 32, "normal", 0, 0.05)
    w3 = make(oracle, (H, K), dtype, 33, "normal", 0, 0.05)
    m = Model()
    tx, t1, t3 = m.tensor(x.shape, dtype), m.tensor(w1.shape, dtype), m.tensor(w3.shape, dtype)
    o = m.swiglu(tx, t1, t3)
    (got,), _, plan = run_model(m, {tx: x, t1: w1, t3: w3}, [o], iters=2)
    assert len(json.loads(plan)["TaskInfos"]) == 1
    g = oracle.matmul(x, w1, dtype, trans_b=True)
    u = oracle.matmul(x, w3, dtype, trans_b=True)
    ref = oracle.binary(oracle.binary(g, oracle.unary(g, "sigmoid", dtype), "mul", dtype), u, "mul", dtype)
    xf, w1f, w3f = (oracle.to_f32(a, dtype).astype(np.float64) for a in (x, w1, w3))
    gf, uf = xf @ w1f.T, xf @ w3f.T
    exact = gf / (1.0 + np.exp(-gf)) * uf
    def err(a):
        d = oracle.to_f32(a, dtype).astype(np.float64) - exact
        return np.abs(d).max() / np.abs(exact).max(), np.sqrt((d * d).mean() / (exact * exact).mean())
    assert got.shape == ref.shape
    emx, erms = err(got)
    cmx, crms = err(ref)
    tol = {"fp16": 2e-3, "bf16": 1e-2}[dtype]
    assert emx <= tol and erms <= tol, (emx, erms)
    assert erms <= 1.25 * crms, (erms, crms)


def test_fused_ops_with_different_task_counts_are_refused():
    """An op that cannot take its producer's tiles (here: behind the SwiGLU op, whose result tiles are
    half its GEMM tiles) keeps its own tiling; fused into the same task it would run for the wrong
    task ids, so compile() refuses the plan instead."""
    from ark_amd import Model, Executor, ArkmiError
    m = Model()
    x = m.tensor([1, 256, 256], "bf16")
    w1, w3 = m.tensor([512, 256], "bf16"), m.tensor([512, 256], "bf16")
    r = m.tensor([1, 256, 512], "bf16")
    with m.planner_context(sync=False):
        m.add(r, m.swiglu(x, w1, w3))
    with pytest.raises(ArkmiError) as e:
        Executor(m.plan(device_id=0), device_id=0).compile()
    assert e.value.kind == "PlanError" and "NumTasks" in str(e.value)


# ---------------------------------------------------------------- barriers that must stay
@pytest.mark.parametrize("n", [1024, 4096])
def test_gemm_feeding_gemm_keeps_grid_barrier(oracle, n):
    """(X @ W1) @ W2 with square operands: both GEMMs cut equal output shapes into the same tiles on
    the same workgroups and Y1 is seen through one view, but task t of the second GEMM reads a whole
    row panel of Y1, written by other workgroups on other L2s.  The barrier between them must stay a
    grid barrier.  Checked on sampled rows against the oracle."""
    from ark_amd import Model
    dtype = "fp16"
    x = make(oracle, (n, n), dtype, 81, "uniform")
    w1 = make(oracle, (n, n), dtype, 82, "normal", scale=1.0 / np.sqrt(n))
    w2 = make(oracle, (n, n), dtype, 83, "normal", scale=1.0 / np.sqrt(n))
    m = Model()
    tx, t1, t2 = (m.tensor([n, n], dtype) for _ in range(3))
    y2 = m.matmul(m.matmul(tx, t1), t2)
    (got,), ex, _ = run_model(m, {tx: x, t1: w1, t2: w2}, [y2], iters=2)
    info = ex.info()
    assert info["barriers_local"] == 0 and info["barriers_elided"] == 0, info
    pick = np.sort(np.random.default_rng(3).choice(n, 16, replace=False))
    pick[0], pick[-1] = 0, n - 1
    y1 = oracle.matmul(np.ascontiguousarray(x[pick]), w1, dtype)
    # The intermediate is rounded to fp16 on both sides, after sums in different orders: single
    # elements of Y1 differ by an ulp, which is not small relative to the smallest results.  Judged
    # against the largest result and in rms; a missing barrier gives errors of order one.
    t, g = (oracle.to_f32(a, dtype).astype(np.float64) for a in (oracle.matmul(y1, w2, dtype), got[pick]))
    assert np.abs(t - g).max() <= 1e-3 * np.abs(t).max()
    assert np.sqrt(((t - g) ** 2).mean()) <= 1e-3 * np.sqrt((t * t).mean())


def test_iterated_gemm_plus_one_keeps_iteration_barrier(oracle, monkeypatch):
    """X <- (X @ W) * 0.5 + ... in place across iterations: the next iteration's GEMM reads row
    panels of X that other workgroups' elementwise tasks wrote, so iterations stay separated by the
    grid barrier even though the add rides on the GEMM's tiles."""
    from ark_amd import Model
    monkeypatch.setenv("ARKMI_ITERATION_BARRIER", "0")
    dtype, n = "fp16", 512
    x = make(oracle, (n, n), dtype, 84, "uniform")
    w = make(oracle, (n, n), dtype, 85, "normal", scale=1.0 / np.sqrt(n))
    m = Model()
    tx, tw = m.tensor([n, n], dtype), m.tensor([n, n], dtype)
    y = m.matmul(tx, tw)
    m.add(y, 1.0, tx)
    iters = 4
    (got,), ex, _ = run_model(m, {tx: x, tw: w}, [tx], iters=iters)
    assert ex.info()["iteration_sync"] == 2, ex.info()
    want = x
    for _ in range(iters):
        want = oracle.scalar(oracle.matmul(want, w, dtype), 1.0, "add", dtype)
    # four rounds of rounding in different summation orders: judged against the largest value
    t, g = (oracle.to_f32(a, dtype).astype(np.float64) for a in (want, got))
    assert np.abs(t - g).max() <= 1e-2 * np.abs(t).max()


def _chain_graphs():
    """Small multi-op graphs whose dependencies cross workgroups in different ways."""
    def gemm_gemm(m, dt):
        a, b, c = m.tensor([512, 512], dt), m.tensor([512, 512], dt), m.tensor([512, 512], dt)
        return [a, b, c], [m.matmul(m.matmul(a, b), c)]

    def ewise_gemm(m, dt):
        a, b = m.tensor([512, 512], dt), m.tensor([512, 512], dt)
        return [a, b], [m.matmul(m.mul(a, 0.5), b)]

    def gemm_reduce(m, dt):
        a, b = m.tensor([512, 256], dt), m.tensor([256, 512], dt)
        y = m.matmul(a, b)
        return [a, b], [m.reduce_sum(y, -1), m.softmax(y)]

    def gemm_ewise_transpose(m, dt):
        a, b = m.tensor([256, 256], dt), m.tensor([256, 256], dt)
        y = m.relu(m.matmul(a, b))
        return [a, b], [m.transpose(y, [1, 0]), m.add(y, y)]

    def rows_then_gemm(m, dt):
        a, b = m.tensor([256, 512], dt), m.tensor([512, 256], dt)
        return [a, b], [m.matmul(m.softmax(a), b)]

    return {"gemm_gemm": gemm_gemm, "ewise_gemm": ewise_gemm, "gemm_reduce": gemm_reduce,
            "gemm_ewise_transpose": gemm_ewise_transpose, "rows_then_gemm": rows_then_gemm}


@pytest.mark.parametrize("graph", sorted(_chain_graphs()))
def test_elided_barriers_give_the_reference_placements_results(oracle, graph, monkeypatch):
    """Each graph runs twice, with the barriers this backend keeps and with every barrier the
    reference places (ARKMI_KEEP_ALL_BARRIERS=1): outputs must agree bit for bit, over several
    iterations."""
    from ark_amd import Model
    dtype = "fp16"
    outs = []
    for keep in ("1", "0"):
        monkeypatch.setenv("ARKMI_KEEP_ALL_BARRIERS", keep)
        m = Model()
        ins, fetch = _chain_graphs()[graph](m, dtype)
        feeds = {t: make(oracle, tuple(t.shape), dtype, 90 + i, "uniform", -0.25, 0.25) for i, t in enumerate(ins)}
        got, ex, _ = run_model(m, feeds, fetch, iters=3)
        if keep == "1":
            assert ex.info()["barriers_elided"] == 0 and ex.info()["barriers_local"] == 0
        outs.append(got)
    for a, b in zip(*outs):
        assert np.array_equal(a, b), graph


# ---------------------------------------------------------------- remaining single-GPU ops
@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_embedding(oracle, dtype):
    """ops_embedding_test.cpp:43-96: indices [8, 3, 64] into a [100, 4096] table, every ninth index
    negative (counted from the end of the table); exact."""
    from ark_amd import Model
    num_emb, dim = 100, 4096
    rng = np.random.default_rng(12)
    idx = rng.integers(0, num_emb, (8, 3, 64)).astype(np.int32)
    flat = idx.reshape(-1)
    flat[::9] = -flat[::9]
    w = make(oracle, (num_emb, dim), dtype, 13, "uniform")
    m = Model()
    ti, tw = m.tensor(idx.shape, "int32"), m.tensor(w.shape, dtype)
    out = m.embedding(ti, tw)
    assert out.shape == [8, 3, 64, dim]
    (got,), ex, _ = run_model(m, {ti: idx, tw: w}, [out], iters=2)
    assert np.array_equal(got, oracle.embedding(idx, w))


def test_embedding_index_outside_the_table_is_clamped(oracle):
    """Indices a table of 100 rows has no row for (100, 101, 2**31 - 1, -101, -2**31): the reference
    reads outside the table there; here they take the last or the first row and never leave it."""
    from ark_amd import Model
    num_emb, dim = 100, 256
    idx = np.array([[0, 99, 100, 101, 2**31 - 1, -1, -100, -101, -2**31, 7]], dtype=np.int32)
    w = make(oracle, (num_emb, dim), "fp16", 14, "uniform")
    m = Model()
    ti, tw = m.tensor(idx.shape, "int32"), m.tensor(w.shape, "fp16")
    out = m.embedding(ti, tw)
    (got,), ex, _ = run_model(m, {ti: idx, tw: w}, [out])
    want = oracle.embedding(idx, w, clamp=True)
    assert np.array_equal(want[0, [2, 3, 4]], np.stack([w[99]] * 3)) and np.array_equal(want[0, [7, 8]], np.stack([w[0]] * 2))
    assert np.array_equal(got.reshape(want.shape), want)


def test_embedding_ragged_rows_and_other_ops_in_one_plan(oracle):
    """A table whose rows are not whole 16-byte vectors (scalar path), a 1-D index vector, and a
    matmul on the gathered rows in the same plan."""
    from ark_amd import Model
    dtype = "fp16"
    idx = np.array([3, -1, 0, 7, -8, 5, 5, 2, 1], np.int32)
    w = make(oracle, (8, 50), dtype, 14, "uniform")
    w2 = make(oracle, (16, 128), dtype, 15, "uniform")
    b = make(oracle, (128, 128), dtype, 16, "uniform")
    idx2 = np.arange(-128, 0, dtype=np.int32).reshape(128) % 16 - 16  # all negative
    m = Model()
    ti, tw = m.tensor(idx.shape, "int32"), m.tensor(w.shape, dtype)
    ti2, tw2, tb = m.tensor(idx2.shape, "int32"), m.tensor(w2.shape, dtype), m.tensor(b.shape, dtype)
    o1 = m.embedding(ti, tw)
    g2 = m.embedding(ti2, tw2)
    assert o1.shape == [1, 1, 9, 50] and g2.shape == [1, 1, 128, 128]
    o2 = m.matmul(m.reshape(g2, [128, 128]), tb)
    (got1, got2), _, _ = run_model(m, {ti: idx, tw: w, ti2: idx2, tw2: w2, tb: b}, [o1, o2])
    assert np.array_equal(got1.reshape(9, 50), oracle.embedding(idx, w))
    close(oracle, oracle.matmul(oracle.embedding(idx2, w2), b, dtype), got2, dtype, 1e-2)


def _all_permutations():
    import itertools
    return [p for p in itertools.permutations(range(4)) if p != (0, 1, 2, 3)]


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_transpose_all_permutations(oracle, dtype):
    """All 23 non-identity permutations of a 4-D tensor (the reference instantiates one kernel per
    permutation, ark/include/kernels/transpose.h, and tests 0132 and 0231 in three types,
    ops_transpose_test.cpp:154-160); one plan per type holds all of them.  Exact."""
    from ark_amd import Model
    x = make(oracle, (3, 4, 24, 40), dtype, 18)
    m = Model()
    t = m.tensor(x.shape, dtype)
    outs = [m.transpose(t, list(p)) for p in _all_permutations()]
    got, _, _ = run_model(m, {t: x}, outs)
    for p, g in zip(_all_permutations(), got):
        assert np.array_equal(g, np.transpose(x, p)), p
    # the two shapes the reference tests: [5, 3, 32, 128] as 0132 and 0231
    y = make(oracle, (5, 3, 32, 128), dtype, 19)
    m = Model()
    t = m.tensor(y.shape, dtype)
    outs = [m.transpose(t, [0, 1, 3, 2]), m.transpose(t, [0, 2, 3, 1])]
    got, _, _ = run_model(m, {t: y}, outs)
    assert np.array_equal(got[0], np.transpose(y, (0, 1, 3, 2)))
    assert np.array_equal(got[1], np.transpose(y, (0, 2, 3, 1)))


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "int32"])
def test_cast_through_bytes(oracle, dtype):
    """Casts to and from BYTE reinterpret the buffer (ops_cast_test.cpp:141-233, ops_cast.cpp:107-132):
    a tensor seen as bytes, a byte tensor seen as `dtype`, and a real op on the reinterpreted view so
    that the plan reads it on the GPU."""
    from ark_amd import Model
    elem = 2 if dtype == "fp16" else 4
    rng = np.random.default_rng(20)
    raw = rng.integers(0, 256, (4, 2, 1024), dtype=np.uint8)
    if dtype != "int32":
        # keep the reinterpreted floats finite: clear the top exponent bit of every element
        raw.reshape(-1, elem)[:, elem - 1] &= 0xBF
    m = Model()
    tb = m.tensor(raw.shape, "byte")
    as_t = m.cast(tb, dtype)            # view: [4, 2, 1024 / elem]
    assert as_t.shape == [4, 2, 1024 // elem] and as_t.buffer_id == tb.buffer_id
    back = m.cast(as_t, "byte")         # and back: the original bytes
    assert back.shape == list(raw.shape) and back.buffer_id == tb.buffer_id
    copied = m.copy(as_t)               # a kernel that reads the reinterpreted view
    m.noop(back)
    (g_t, g_back, g_copy), _, _ = run_model(m, {tb: raw}, [as_t, back, copied])
    np_t = {"fp32": np.float32, "fp16": np.float16, "int32": np.int32}[dtype]
    want = raw.view(np_t)
    assert np.array_equal(g_t.view(np.uint8), raw) and g_t.shape == want.shape
    assert np.array_equal(g_back, raw)
    assert np.array_equal(g_copy.view(np.uint8).reshape(raw.shape), raw)


# ---------------------------------------------------------------- matmul with K split in two
@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("trans_other", [False, True])
@pytest.mark.parametrize("K,skew", [(8192, None), (4096, None), (4096, "0"), (1024, "100000")])
def test_matmul_split_k(oracle, monkeypatch, dtype, trans_other, K, skew):
    """An output that gives 256x256 tiles to half of the CUs only (2048 x 4096, the decoder layer's
    projections) is planned with SplitK 2 from K = 4096 on: two tasks per tile, one multiplying the
    upper part of K and sending its partial sums, the other the lower part, adding the two and
    finishing the tile.  Several iterations reuse the tiles' full/empty words; the split point is
    moved (equal parts; the shortest sender's part a short K allows); checked on sampled rows
    against the oracle, and bit for bit against the same plan run one kernel per op."""
    import torch
    from ark_amd import Model, Executor
    M, N = 2048, 4096
    if skew is not None:
        monkeypatch.setenv("ARKMI_SPLITK_SKEW", skew)
    a = make(oracle, (M, K), dtype, 111, "uniform")
    b = make(oracle, (N, K) if trans_other else (K, N), dtype, 112, "normal", scale=0.05)
    m = Model()
    ta, tb = m.tensor(a.shape, dtype), m.tensor(b.shape, dtype)
    c = m.matmul(ta, tb, trans_other=trans_other)
    split = {"NumWarps": 8, "SramBytes": 131072, "TileShapeMNK": [256, 256, 64], "SplitK": 2, "NumTasks": 256}
    plan = m.plan(device_id=0, config_rules=[lambda op, arch: json.dumps(split)] if K < 4096 else ())
    cfg = json.loads(plan)["TaskInfos"][0]["Ops"][0]["Config"]
    assert cfg["SplitK"] == 2 and cfg["TileShapeMNK"][:2] == [256, 256] and cfg["NumTasks"] == 2 * 8 * 16, cfg
    (got,), ex, _ = run_model(m, {ta: a, tb: b}, [c], iters=3, plan=plan)
    assert ex.info()["iteration_sync"] == 2 and (ex.info()["kernel_families"] & 64), ex.info()
    pick = np.sort(np.random.default_rng(5).choice(M, 32, replace=False))
    pick[0], pick[-1] = 0, M - 1
    close(oracle, oracle.matmul(np.ascontiguousarray(a[pick]), b, dtype, trans_b=trans_other), got[pick], dtype, 1e-2)
    ex2 = Executor(plan, device_id=0, loop_mode=False).compile()
    ex2.tensor_write(ta, a)
    ex2.tensor_write(tb, b)
    ex2.run_separate(2)
    torch.cuda.synchronize()
    assert np.array_equal(ex2.tensor_read(c), got)


def test_matmul_split_k_with_follower_and_neighbours(oracle):
    """The residual add fused behind a split matmul belongs to the workgroup that finishes the tile; the
    ops before and after it keep their grid barriers (a split tile's sender is another workgroup)."""
    from ark_amd import Model
    dtype = "bf16"
    M, N, K = 2048, 4096, 8192
    x = make(oracle, (M, K), dtype, 113, "normal")
    w = make(oracle, (N, K), dtype, 114, "normal", scale=0.02)
    r = make(oracle, (M, N), dtype, 115, "normal")
    m = Model()
    tx, tw, tr = m.tensor(x.shape, dtype), m.tensor(w.shape, dtype), m.tensor(r.shape, dtype)
    xs = m.mul(tx, 0.5)
    with m.planner_context(sync=False):
        h = m.add(tr, m.matmul(xs, tw, trans_other=True))
    out = m.relu(h)
    plan = m.plan(device_id=0)
    tasks = json.loads(plan)["TaskInfos"]
    assert len(tasks) == 3 and len(tasks[1]["Ops"]) == 2 and tasks[1]["Ops"][0]["Config"].get("SplitK") == 2
    assert tasks[1]["Ops"][1]["Config"]["NumTasks"] * 2 == tasks[1]["Ops"][0]["Config"]["NumTasks"]
    (got,), ex, _ = run_model(m, {tx: x, tw: w, tr: r}, [out], iters=2, plan=plan)
    assert ex.info()["barriers_local"] == 0 and ex.info()["barriers_elided"] == 0, ex.info()
    pick = np.sort(np.random.default_rng(6).choice(M, 24, replace=False))
    pick[0], pick[-1] = 0, M - 1
    xs_ref = oracle.scalar(np.ascontiguousarray(x[pick]), 0.5, "mul", dtype)
    ref = oracle.unary(oracle.binary(np.ascontiguousarray(r[pick]), oracle.matmul(xs_ref, w, dtype, trans_b=True),
                                     "add", dtype), "relu", dtype)
    close(oracle, ref, got[pick], dtype, 1e-2)


# ---------------------------------------------------------------- caches across iterations
def test_follower_sees_this_iterations_tile_not_a_cached_one(oracle):
    """x <- 0.5 * relu(x @ w), the relu fused behind the matmul: every iteration the follower reads a
    tile its own workgroup has just rewritten with new values, small enough to sit in the CU's L1 from
    the iteration before.  A stale read would feed the previous iteration's tile forward."""
    from ark_amd import Model
    dtype, n = "fp16", 128
    x = make(oracle, (n, n), dtype, 121, "uniform")
    w = make(oracle, (n, n), dtype, 122, "normal", scale=2.0 / np.sqrt(n))
    m = Model()
    tx, tw = m.tensor([n, n], dtype), m.tensor([n, n], dtype)
    with m.planner_context(sync=False):
        z = m.relu(m.matmul(tx, tw))
    m.mul(z, 0.5, tx)
    iters = 6
    (got,), ex, plan = run_model(m, {tx: x, tw: w}, [tx], iters=iters)
    assert len(json.loads(plan)["TaskInfos"][0]["Ops"]) == 2
    want = x
    for _ in range(iters):
        want = oracle.scalar(oracle.unary(oracle.matmul(want, w, dtype), "relu", dtype), 0.5, "mul", dtype)
    t, g = (oracle.to_f32(a, dtype).astype(np.float64) for a in (want, got))
    assert np.abs(t).max() > 1e-3  # the sequence has not died out
    assert np.abs(t - g).max() <= 1e-2 * np.abs(t).max()


def test_grid_barrier_drops_other_workgroups_old_lines_from_the_l1(oracle):
    """a <- transpose(a) + 1 on a 16 KB tensor cut into 8 tasks: every workgroup re-reads, each
    iteration, a few lines that other workgroups have rewritten since, and that still sit in its own L1
    from the iteration before.  The grid barrier between the two ops must drop them."""
    from ark_amd import Model
    a = make(oracle, (1, 1, 64, 64), "fp32", 123)
    cfg = {"NumWarps": 8, "SramBytes": 0, "Tile": [8, 64], "NumTasks": 8}
    m = Model()
    ta = m.tensor(a.shape, "fp32")
    with m.planner_context(config=cfg):
        tb = m.transpose(ta, [0, 1, 3, 2])
    with m.planner_context(config=cfg):
        m.add(tb, 1.0, ta)
    iters = 7
    (got,), ex, _ = run_model(m, {ta: a}, [ta], iters=iters)
    assert ex.info()["iteration_sync"] == 2 and ex.info()["barriers_local"] == 0
    want = a.copy()
    for _ in range(iters):
        want = np.ascontiguousarray(want.transpose(0, 1, 3, 2)) + np.float32(1.0)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- several slots per workgroup
def test_fused_task_in_two_warp_slots(oracle):
    """Tasks of two warps run four to a workgroup, each slot on its own waves; the ops of a fused
    task then meet on the slot's own barrier (ark/include/kernels/common/sync.h:81-130), not on
    the workgroup's.  500 tasks over 4 slots x 256 workgroups leaves slots with unequal task
    counts, so a workgroup-wide barrier inside the task would pair the wrong waves."""
    from ark_amd import Model
    dtype = "fp16"
    m = Model()
    t0, t1 = m.tensor((4000, 256), dtype), m.tensor((4000, 256), dtype)
    cfg = {"NumWarps": 2, "SramBytes": 0, "Tile": [8, 256], "NumTasks": 500}
    with m.planner_context(sync=False, config=cfg):
        t2 = m.mul(t0, 0.5)
        t3 = m.add(t2, t1)
        t4 = m.relu(t3)
    x0, x1 = make(oracle, (4000, 256), dtype, 31), make(oracle, (4000, 256), dtype, 32)
    (got,), ex, plan = run_model(m, {t0: x0, t1: x1}, [t4], iters=3)
    pj = json.loads(plan)
    assert len(pj["TaskInfos"]) == 1 and len(pj["TaskInfos"][0]["Ops"]) == 3
    assert pj["TaskInfos"][0]["NumWarps"] == 2
    ref = oracle.unary(oracle.binary(oracle.scalar(x0, 0.5, "mul", dtype), x1, "add", dtype), "relu", dtype)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("warps", [1, 2, 4])
def test_rmsnorm_with_staged_weights_in_narrow_slots(oracle, warps):
    """RMSNorm stages its fp32 weights in the slot's LDS window and syncs the slot around the copy:
    with 8 / warps slots per workgroup each slot has a window and a barrier of its own."""
    from ark_amd import Model
    dtype, rows, cols = "bf16", 1000, 2048
    m = Model()
    x, w = m.tensor((rows, cols), dtype), m.tensor((1, cols), "fp32")
    cfg = {"NumWarps": warps, "SramBytes": cols * 4, "RowsPerWave": 2, "NumTasks": -(-rows // (warps * 2))}
    with m.planner_context(config=cfg):
        y = m.rmsnorm(x, w, eps=1e-6)
    xs = make(oracle, (rows, cols), dtype, 41)
    ws = make(oracle, (1, cols), "fp32", 42, "uniform", 0.5, 1.5)
    (got,), ex, plan = run_model(m, {x: xs, w: ws}, [y], iters=2)
    assert json.loads(plan)["TaskInfos"][0]["NumWarps"] == warps
    close(oracle, oracle.rmsnorm(xs, ws.reshape(-1), dtype, eps=1e-6), got, dtype, 1e-2)
