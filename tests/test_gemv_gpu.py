"""GPU parity of the skinny matmul ("decode GEMV": at most 16 rows times W[K,N])
against the CPU oracle's textbook fp32-accumulate matmul, through the C ABI and
through Model -> plan -> Executor.

The reference has no separate GEMV: these shapes go through its Matmul op
(ark/ops/ops_matmul.cpp:13-252), so the cases restate ops_matmul_test.cpp for
skinny inputs: the all-0.1 known answer (:349-359), random operands, a one-hot
X that must pick a row of W bit for bit, ragged K and N.  Tolerance: max
relative error <= 1e-2 over elements above 1e-3 * max|ref| plus the reference's
reduction_abs_error_bound for the rest (ops_test_common.hpp:52-69).
"""
import numpy as np
import pytest
import torch

from helpers import make, to_gpu, to_np

pytestmark = pytest.mark.gpu


def _check(oracle, ref, got, dtype, max_abs, k):
    rel, abs_rest, mx = oracle.max_rel_error(ref, got, dtype)
    assert rel <= 1e-2, (rel, abs_rest, mx)
    bound = oracle.reduction_abs_error_bound(dtype, max_abs, min(k, 1 << (oracle.FRAC_BITS[dtype] + 1)))
    assert abs_rest <= bound, (abs_rest, bound)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("m", [1, 3, 8, 16])
@pytest.mark.parametrize("n,k,tasks", [(256, 256, 0), (512, 1024, 16), (512, 1024, 5), (512, 1024, 1),
                                       (1024, 4096, 0), (264, 300, 0), (264, 300, 3), (8, 16, 0),
                                       (4096, 11008, 0), (4096, 11008, 77)])
def test_gemv_shapes(oracle, dtype, m, n, k, tasks):
    from ark_amd import ops
    if k > 4096 and m not in (1, 8):
        pytest.skip("large case runs for the two benchmark batch sizes")
    kp = (k + 7) // 8 * 8  # row pitch of X must be a multiple of 8 elements
    x = make(oracle, (m, kp), dtype, seed=11, dist="normal")
    w = make(oracle, (k, n), dtype, seed=12, dist="normal")
    w = oracle.to_storage(oracle.to_f32(w, dtype) * 0.05, dtype)
    ref = oracle.matmul(np.ascontiguousarray(x[:, :k]), w, dtype)
    xg = to_gpu(x, dtype)[:, :k]
    got = to_np(ops.gemv(xg, to_gpu(w, dtype), num_tasks=tasks), dtype)
    _check(oracle, ref, got, dtype, 4.0 * 0.25, k)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_gemv_known_answer(oracle, dtype):
    """All-0.1 inputs: every output is K * (0.1 rounded)^2, rounded once."""
    from ark_amd import ops
    m, n, k = 8, 512, 2048
    x = oracle.to_storage(np.full((m, k), 0.1, np.float32), dtype)
    w = oracle.to_storage(np.full((k, n), 0.1, np.float32), dtype)
    got = oracle.to_f32(to_np(ops.gemv(to_gpu(x, dtype), to_gpu(w, dtype)), dtype), dtype)
    v = float(oracle.to_f32(x, dtype)[0, 0])
    assert np.all(got == got[0, 0])
    assert abs(got[0, 0] - k * v * v) <= oracle.reduction_abs_error_bound(
        dtype, 0.1, min(k, 256 if dtype == "bf16" else 2048))


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_gemv_one_hot_picks_rows(oracle, dtype):
    """X rows that are one-hot select rows of W bit for bit (pins operand
    orientation, the K split and the order the partial sums are added in)."""
    from ark_amd import ops
    m, n, k = 5, 768, 2048
    w = make(oracle, (k, n), dtype, seed=5, dist="normal")
    x = np.zeros((m, k), np.float32)
    picks = [0, 17, 1023, 1024, 2047]
    for i, p in enumerate(picks):
        x[i, p] = 1.0
    got = to_np(ops.gemv(to_gpu(oracle.to_storage(x, dtype), dtype), to_gpu(w, dtype), num_tasks=37), dtype)
    assert np.array_equal(got, w[picks])


def test_gemv_repeated_calls_share_workspace(oracle):
    """The arrival counters return to zero: back-to-back calls agree bit for bit."""
    from ark_amd import ops
    x = to_gpu(make(oracle, (8, 4096), "bf16", seed=1, dist="normal"), "bf16")
    w = to_gpu(make(oracle, (4096, 1024), "bf16", seed=2, dist="normal"), "bf16")
    first = ops.gemv(x, w, num_tasks=100).clone()
    for _ in range(5):
        assert torch.equal(ops.gemv(x, w, num_tasks=100), first)


def test_gemv_rejects_bad_arguments(oracle):
    from ark_amd import ops
    x = torch.zeros(17, 256, device="cuda", dtype=torch.float16)
    w = torch.zeros(256, 256, device="cuda", dtype=torch.float16)
    with pytest.raises(Exception):
        ops.gemv(x, w)  # more than 16 rows
    with pytest.raises(Exception):
        ops.gemv(x[:4], w, num_tasks=-1)  # negative task count
    with pytest.raises(Exception):
        ops.gemv(x[:4], torch.zeros(256, 260, device="cuda", dtype=torch.float16))  # n % 8


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("m", [1, 8])
def test_gemv_in_loop_kernel(oracle, dtype, m):
    """Model.matmul on a skinny input is planned onto the GEMV body and run by
    the loop kernel; several iterations reuse the split-K counters."""
    import json
    from ark_amd import Model, Executor
    n, k = 1536, 2048
    x = make(oracle, (m, k), dtype, seed=21, dist="normal")
    w = oracle.to_storage(oracle.to_f32(make(oracle, (k, n), dtype, seed=22, dist="normal"), dtype) * 0.05, dtype)
    mod = Model()
    tx, tw = mod.tensor([m, k], dtype), mod.tensor([k, n], dtype)
    ty = mod.matmul(tx, tw)
    plan = mod.plan(device_id=0)
    cfg = json.loads(plan)["TaskInfos"][0]["Ops"][0]["Config"]
    assert cfg["TileShapeMNK"] == [16, 256, 128]
    ex = Executor(plan).compile()
    assert ex.info()["kernel_families"] == 8
    ex.tensor_write(tx, x)
    ex.tensor_write(tw, w)
    ex.launch()
    ex.run(3)
    ex.wait()
    got = ex.tensor_read(ty)
    ex.stop()
    ref = oracle.matmul(x, w, dtype)
    _check(oracle, ref, got, dtype, 4.0 * 0.25, k)


def _sampled_columns_check(oracle, x, w, got, dtype, cols):
    """Oracle on sampled output columns (all rows of X against those columns of W)."""
    ref = oracle.matmul(x, np.ascontiguousarray(w[:, cols]), dtype)
    _check(oracle, ref, np.ascontiguousarray(got[:, cols]), dtype, 4.0 * 0.25, x.shape[1])


@pytest.mark.parametrize("m", [1, 8])
@pytest.mark.parametrize("n,k", [(12288, 4096), (22016, 4096), (4096, 4096)])
def test_gemv_decode_projection_shapes(oracle, m, n, k):
    """The remaining Llama-2-7B decode shapes (W_qkv, W_gate/up, W_o; W_down is in test_gemv_shapes),
    bf16, batch 1 and 8; the oracle evaluates 512 sampled columns plus the first and last."""
    from ark_amd import ops
    dtype = "bf16"
    x = make(oracle, (m, k), dtype, seed=31, dist="normal")
    w = make(oracle, (k, n), dtype, seed=32, dist="normal", scale=0.02)
    got = to_np(ops.gemv(to_gpu(x, dtype), to_gpu(w, dtype)), dtype)
    cols = np.sort(np.random.default_rng(4).choice(n, 512, replace=False))
    cols[0], cols[-1] = 0, n - 1
    _sampled_columns_check(oracle, x, w, got, dtype, cols)


@pytest.mark.parametrize("batch", [1, 8])
def test_decode_step_four_projections_in_one_plan(oracle, batch):
    """The decode step the benchmark times: x[B,4096] against W_qkv[4096,12288], W_o[4096,4096],
    W_gate/up[4096,22016] and x2[B,11008] against W_down[11008,4096], bf16, as four skinny matmuls of
    one plan in the loop kernel, three iterations.  All four outputs against the oracle on sampled
    columns (512 per matrix)."""
    from ark_amd import Model, Executor
    dtype = "bf16"
    shapes = [(4096, 12288), (4096, 4096), (4096, 22016), (11008, 4096)]
    mod = Model()
    xs, ws, ys, vals = [], [], [], {}
    for i, (k, n) in enumerate(shapes):
        tx, tw = mod.tensor([batch, k], dtype), mod.tensor([k, n], dtype)
        vals[tx] = make(oracle, (batch, k), dtype, seed=40 + i, dist="normal")
        vals[tw] = make(oracle, (k, n), dtype, seed=50 + i, dist="normal", scale=0.02)
        xs.append(tx); ws.append(tw); ys.append(mod.matmul(tx, tw))
    ex = Executor(mod.plan(device_id=0)).compile()
    assert ex.info()["kernel_families"] == 8 and ex.info()["gemv_chains"] == 1 and ex.info()["gemv_claimed"] == 1
    for t, a in vals.items():
        ex.tensor_write(t, a)
    ex.launch()
    ex.run(3)
    ex.wait()
    got = [ex.tensor_read(t) for t in ys]
    ex.stop()
    for (k, n), tx, tw, g in zip(shapes, xs, ws, got):
        cols = np.sort(np.random.default_rng(n).choice(n, 512, replace=False))
        cols[0], cols[-1] = 0, n - 1
        _sampled_columns_check(oracle, vals[tx], vals[tw], g, dtype, cols)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("claimed", [False, True])
def test_consecutive_skinny_matmuls_run_as_one_stream(oracle, dtype, claimed, monkeypatch):
    """Independent skinny matmuls that follow one another are streamed as one sequence by the loop
    kernel (the next one's weights are loaded while the current one adds up its tiles), and when all
    of them are deep enough the workgroups claim their stretches at run time instead of getting fixed
    shares.  Shapes with ragged K and N, different row counts, few stretches (most workgroups have
    nothing to do for that matmul) and many: every output against the oracle, and bit for bit
    against the same plan with fixed shares (ARKMI_GEMV_CLAIM=0), with the matmuls run one by one
    (ARKMI_GEMV_CHAIN=0) and as one kernel per op: the partial sums are per stretch and added in a
    fixed order, whoever streams them."""
    from ark_amd import Model, Executor
    if claimed:
        shapes = [(1, 2048, 1536), (3, 424, 264), (8, 4096, 512), (16, 1024, 8), (2, 384, 4096), (1, 11008, 1024)]
    else:  # a matmul of one or two units keeps the run on fixed shares
        shapes = [(1, 2048, 1536), (3, 296, 264), (8, 4096, 512), (16, 1024, 8), (2, 16, 4096), (1, 11008, 1024)]
    mod = Model()
    vals, ys = {}, []
    for i, (m, k, n) in enumerate(shapes):
        tx, tw = mod.tensor([m, k], dtype), mod.tensor([k, n], dtype)
        vals[tx] = make(oracle, (m, k), dtype, seed=60 + i, dist="normal")
        vals[tw] = make(oracle, (k, n), dtype, seed=70 + i, dist="normal", scale=0.05)
        ys.append((mod.matmul(tx, tw), tx, tw, k))
    plan = mod.plan(device_id=0)

    def run(separate=False, iters=3):
        ex = Executor(plan, device_id=0, loop_mode=not separate).compile()
        info = ex.info()
        for t, a in vals.items():
            ex.tensor_write(t, a)
        if separate:
            ex.run_separate(2)
            torch.cuda.synchronize()
        else:
            ex.launch()
            ex.run(iters)
            ex.wait()
            ex.run(2)  # (a second command: the claim counters alternate by iteration across commands)
            ex.wait()
        got = [ex.tensor_read(y) for y, _, _, _ in ys]
        if not separate:
            ex.stop()
        return got, info

    first, info = run()
    assert info["kernel_families"] == 8 and info["gemv_chains"] == 1 and info["gemv_claimed"] == int(claimed)
    for g, (_, tx, tw, k) in zip(first, ys):
        _check(oracle, oracle.matmul(vals[tx], vals[tw], dtype), g, dtype, 4.0 * 0.25, k)
    # who streams what does not matter: another run of the same plan gives the same bits
    again, _ = run(iters=4)
    for a, b in zip(first, again):
        assert np.array_equal(a, b)
    # fixed shares: the plan's tasks, the same in a run, one by one and as one kernel per op
    monkeypatch.setenv("ARKMI_GEMV_CLAIM", "0")
    fixed, info = run()
    assert info["gemv_chains"] == 1 and info["gemv_claimed"] == 0
    monkeypatch.setenv("ARKMI_GEMV_CHAIN", "0")
    one_by_one, info = run()
    assert info["gemv_chains"] == 0 and info["gemv_claimed"] == 0
    one_kernel_per_op, _ = run(separate=True)
    for a, b, c in zip(fixed, one_by_one, one_kernel_per_op):
        assert np.array_equal(a, b) and np.array_equal(a, c)
    for g, (_, tx, tw, k) in zip(fixed, ys):
        _check(oracle, oracle.matmul(vals[tx], vals[tw], dtype), g, dtype, 4.0 * 0.25, k)
    if not claimed:
        for a, b in zip(first, fixed):
            assert np.array_equal(a, b)
    # every matmul by itself, its stretches claimed where it is deep enough (cut differently from
    # the run: other partial sums, same tolerance)
    monkeypatch.delenv("ARKMI_GEMV_CLAIM")
    alone, info = run()
    assert info["gemv_chains"] == 0 and info["gemv_claimed"] == (6 if claimed else 5)
    for g, (_, tx, tw, k) in zip(alone, ys):
        _check(oracle, oracle.matmul(vals[tx], vals[tw], dtype), g, dtype, 4.0 * 0.25, k)


@pytest.mark.parametrize("num_processors", [256, 40])
def test_dependent_skinny_matmuls_claim_their_stretches(oracle, num_processors, monkeypatch):
    """y = ((x W1) W2) W3 with 2 rows: every matmul waits for the one before it (the grid barriers
    stay), and each is cut into stretches that the workgroups claim at run time, with their two claim
    counters alternating over the iterations of several commands.  On the full grid and on 40
    processors (more stretches than twice the workgroups: most are claimed, few are the fixed first
    two).  Against the oracle and the plan's fixed shares (three bf16 roundings deep, a last-bit
    difference of an intermediate value moves a result by an ulp or two: judged by the largest
    difference against the largest value, 1e-2), and bit for bit against a second run."""
    from ark_amd import Model, Executor
    dtype = "bf16"
    dims = [(2048, 3072), (3072, 1024), (1024, 2048)]
    mod = Model()
    tx = mod.tensor([2, dims[0][0]], dtype)
    vals = {tx: make(oracle, (2, dims[0][0]), dtype, seed=90, dist="normal")}
    ws, y = [], tx
    for i, (k, n) in enumerate(dims):
        tw = mod.tensor([k, n], dtype)
        vals[tw] = make(oracle, (k, n), dtype, seed=91 + i, dist="normal", scale=0.03)
        ws.append(tw)
        y = mod.matmul(y, tw)
    plan = mod.plan(arch="ROCM_950", num_processors=num_processors)

    def run(commands):
        ex = Executor(plan, device_id=0).compile()
        info = ex.info()
        for t, a in vals.items():
            ex.tensor_write(t, a)
        ex.launch()
        for n in commands:
            ex.run(n)
            ex.wait()
        got = ex.tensor_read(y)
        ex.stop()
        return got, info

    got, info = run([1, 2, 3])
    assert info["gemv_chains"] == 0 and info["gemv_claimed"] == 3 and info["iteration_sync"] == 2
    assert info["num_processors"] <= num_processors  # (a plan names the processors it uses)
    ref = vals[tx]
    for tw in ws:
        ref = oracle.matmul(ref, vals[tw], dtype)
    ref32 = oracle.to_f32(ref, dtype)

    def close(a):
        return float(np.abs(oracle.to_f32(a, dtype) - ref32).max()) <= 1e-2 * float(np.abs(ref32).max())
    assert close(got)
    again, _ = run([4])
    assert np.array_equal(got, again)
    monkeypatch.setenv("ARKMI_GEMV_CLAIM", "0")
    fixed, info = run([2])
    assert info["gemv_claimed"] == 0
    assert close(fixed)
