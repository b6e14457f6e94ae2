"""GPU parity of the MFMA GEMM against the CPU oracle (textbook fp32-accumulate
matmul, one rounding), through the C ABI.

Cases follow ark/ops/ops_matmul_test.cpp: the all-0.1 known answer (:349-359,
every C element = K * 0.01 before rounding), layouts nn / nt (:429-470), batched
with broadcast (:472-525).  Tolerance: max relative error <= 1e-2 over elements
above 1e-3 * max|ref|, and the reference's reduction_abs_error_bound for the
rest (ops_test_common.hpp:52-69).
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
@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("mnk,tile", [((256, 256, 64), (256, 256)), ((256, 512, 256), (128, 256)),
                                      ((512, 256, 128), (256, 128)), ((384, 640, 192), (128, 128)),
                                      ((512, 512, 512), (0, 0))])
def test_matmul_layouts(oracle, dtype, trans_b, mnk, tile):
    from ark_amd import ops
    m, n, k = mnk
    a = make(oracle, (m, k), dtype, seed=1, dist="uniform")
    b = make(oracle, (n, k) if trans_b else (k, n), dtype, seed=2, dist="uniform")
    ref = oracle.matmul(a, b, dtype, trans_b=trans_b)
    got = to_np(ops.matmul(to_gpu(a, dtype), to_gpu(b, dtype), trans_b=trans_b, tile=tile), dtype)
    _check(oracle, ref, got, dtype, 1.0, k)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("mnk", [(128, 128, 64), (384, 640, 192), (256, 128, 4096)])
def test_matmul_transposed_input(oracle, dtype, trans_b, mnk):
    """tn and tt (ops_matmul_test.cpp:457-511): A given as [k, m]."""
    from ark_amd import ops
    m, n, k = mnk
    a = make(oracle, (k, m), dtype, seed=5, dist="uniform")
    b = make(oracle, (n, k) if trans_b else (k, n), dtype, seed=6, dist="uniform")
    ref = oracle.matmul(a, b, dtype, trans_a=True, trans_b=trans_b)
    got = to_np(ops.matmul(to_gpu(a, dtype), to_gpu(b, dtype), trans_a=True, trans_b=trans_b), dtype)
    _check(oracle, ref, got, dtype, 1.0, k)


@pytest.mark.parametrize("trans_a", [False, True])
@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("mnk", [(128, 128, 64), (256, 384, 192), (128, 256, 2048)])
def test_matmul_fp32(oracle, trans_a, trans_b, mnk):
    """fp32 operands (ops_matmul_test.cpp:364-397), all four layouts."""
    from ark_amd import ops
    dtype = "fp32"
    m, n, k = mnk
    a = make(oracle, (k, m) if trans_a else (m, k), dtype, seed=7, dist="uniform")
    b = make(oracle, (n, k) if trans_b else (k, n), dtype, seed=8, dist="uniform")
    ref = oracle.matmul(a, b, dtype, trans_a=trans_a, trans_b=trans_b)
    got = to_np(ops.matmul(to_gpu(a, dtype), to_gpu(b, dtype), trans_a=trans_a, trans_b=trans_b), dtype)
    _check(oracle, ref, got, dtype, 1.0, k)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_matmul_known_answer(oracle, dtype):
    """All-0.1 inputs: every output is K * (0.1 rounded)^2, rounded once."""
    from ark_amd import ops
    m, n, k = 256, 512, 2048
    a = oracle.to_storage(np.full((m, k), 0.1, np.float32), dtype)
    b = oracle.to_storage(np.full((k, n), 0.1, np.float32), dtype)
    got = oracle.to_f32(to_np(ops.matmul(to_gpu(a, dtype), to_gpu(b, dtype)), dtype), dtype)
    v = float(oracle.to_f32(a, dtype)[0, 0])
    exact = k * v * v
    assert np.all(got == got[0, 0])
    assert abs(got[0, 0] - exact) <= oracle.reduction_abs_error_bound(dtype, 0.1, min(k, 256 if dtype == "bf16" else 2048))


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_matmul_batched_broadcast(oracle, dtype):
    from ark_amd import ops
    a = make(oracle, (3, 128, 64), dtype, seed=3, dist="uniform")
    b = make(oracle, (1, 64, 256), dtype, seed=4, dist="uniform")
    ref = oracle.matmul(a, b, dtype)
    got = to_np(ops.matmul(to_gpu(a, dtype), to_gpu(b, dtype)), dtype)
    _check(oracle, ref, got, dtype, 1.0, 64)
    b2 = make(oracle, (3, 256, 64), dtype, seed=5, dist="uniform")
    ref = oracle.matmul(a, b2, dtype, trans_b=True)
    got = to_np(ops.matmul(to_gpu(a, dtype), to_gpu(b2, dtype), trans_b=True), dtype)
    _check(oracle, ref, got, dtype, 1.0, 64)


def test_matmul_identity_picks_columns(oracle):
    """B = identity: C must equal A bit for bit (pins operand orientation)."""
    from ark_amd import ops
    dtype = "fp16"
    a = make(oracle, (256, 256), dtype, seed=9)
    eye = oracle.to_storage(np.eye(256, dtype=np.float32), dtype)
    for tb in (False, True):
        got = to_np(ops.matmul(to_gpu(a, dtype), to_gpu(eye, dtype), trans_b=tb), dtype)
        assert np.array_equal(got, a)
    # a permutation matrix distinguishes B from B^T
    perm = np.roll(np.eye(256, dtype=np.float32), 1, axis=1)  # P[i, i+1] = 1
    p = oracle.to_storage(perm, dtype)
    got = to_np(ops.matmul(to_gpu(a, dtype), to_gpu(p, dtype)), dtype)
    assert np.array_equal(got, np.roll(a, 1, axis=1))
    got = to_np(ops.matmul(to_gpu(a, dtype), to_gpu(p, dtype), trans_b=True), dtype)
    assert np.array_equal(got, np.roll(a, -1, axis=1))


def test_matmul_full_size_config(oracle):
    """C[4096,4096] = A.B fp16, U[-1,1): checked on 256 sampled rows x all
    columns against the oracle, the rest through linearity: C(2A) == 2 C(A)."""
    from ark_amd import ops
    dtype = "fp16"
    a = make(oracle, (4096, 4096), dtype, seed=21, dist="uniform")
    b = make(oracle, (4096, 4096), dtype, seed=22, dist="uniform")
    ta, tb = to_gpu(a, dtype), to_gpu(b, dtype)
    c = ops.matmul(ta, tb)
    got = to_np(c, dtype)
    rows = np.random.default_rng(0).choice(4096, 256, replace=False)
    ref = oracle.matmul(np.ascontiguousarray(a[rows]), b, dtype)
    _check(oracle, ref, got[rows], dtype, 1.0, 2048)
    # scaling an operand by two scales every fp32 partial sum exactly; only
    # results in fp16's subnormal range may round differently
    c2 = ops.matmul(ta * 2, tb)
    assert float((c2.float() - 2 * c.float()).abs().max()) <= 2.0 ** -22


@pytest.mark.parametrize("trans_b", [False, True])
def test_matmul_full_size_through_the_plan(oracle, trans_b):
    """The same configuration the way the benchmark runs it: Model -> Planner -> plan -> Executor ->
    loop kernel (256x256 tiles, the XCD-aware tile order on), two iterations; 256 sampled rows x
    all columns against the oracle.  With the second operand stored [N, K] too: the layout of every
    weight matmul in the FFN and the decoder layer."""
    from ark_amd import Model, Executor, plan_analysis
    dtype = "fp16"
    a = make(oracle, (4096, 4096), dtype, seed=21, dist="uniform")
    b = make(oracle, (4096, 4096), dtype, seed=22, dist="uniform")
    m = Model()
    ta, tb = m.tensor([4096, 4096], dtype), m.tensor([4096, 4096], dtype)
    out = m.matmul(ta, tb, trans_other=trans_b)
    plan = m.plan(device_id=0)
    assert plan_analysis(plan)["GemmXcdOrdered"] == 1
    ex = Executor(plan, device_id=0).compile()
    ex.tensor_write(ta, a)
    ex.tensor_write(tb, b)
    ex.launch()
    ex.run(2)
    ex.wait()
    got = ex.tensor_read(out)
    ex.stop()
    rows = np.random.default_rng(1).choice(4096, 256, replace=False)
    ref = oracle.matmul(np.ascontiguousarray(a[rows]), b, dtype, trans_b=trans_b)
    _check(oracle, ref, got[rows], dtype, 1.0, 2048)


def test_matmul_errors():
    from ark_amd import ops, ArkmiError
    a = torch.zeros(100, 64, dtype=torch.float16, device="cuda")
    b = torch.zeros(64, 128, dtype=torch.float16, device="cuda")
    with pytest.raises(ArkmiError) as e:
        ops.matmul(a, b)
    assert e.value.kind == "UnsupportedError"
    with pytest.raises(ValueError):
        ops.matmul(torch.zeros(128, 64, dtype=torch.float16, device="cuda"),
                   torch.zeros(128, 128, dtype=torch.float16, device="cuda"))
