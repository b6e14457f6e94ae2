"""Pins the CPU oracle against independent facts: reference test vectors,
closed forms, invariants and independent libraries (numpy / torch / scipy).
None of these checks retypes the oracle's own formula."""
import ctypes

import numpy as np
import pytest
import torch


# ---------------------------------------------------------------- fp16 / bf16
def test_half_all_patterns_round_trip(oracle):
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    for b in range(0, 65536, 1):
        f = L.orc_half_to_float(ctypes.c_uint16(b))
        r = ref[b]
        if np.isnan(r):
            assert np.isnan(f)
            continue
        assert f == r, (b, f, r)
        assert L.orc_float_to_half(ctypes.c_float(f)) == b


def test_float_to_half_rne_against_numpy(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 10,
        (rng.standard_normal(5000) * 1e-5).astype(np.float32),   # subnormal range
        (rng.standard_normal(2000) * 7e4).astype(np.float32),    # overflow range
        np.array([65504, 65519.99, 65520, 1e9, -1e9, 2 ** -24, 2 ** -25, 2 ** -25 * 1.0001,
                  1 + 2 ** -11, 1 + 3 * 2 ** -11, 0.0, -0.0, np.inf, -np.inf], dtype=np.float32)])
    want = xs.astype(np.float16).view(np.uint16)
    for x, w in zip(xs, want):
        assert L.orc_float_to_half(ctypes.c_float(float(x))) == w, (x, w)


def test_bf16_against_torch(oracle):
    rng = np.random.default_rng(1)
    xs = np.concatenate([rng.standard_normal(50000).astype(np.float32) * 100,
                         np.array([1 + 2 ** -8, 1 + 3 * 2 ** -8, 3.3895314e38, 1e-40, -0.0, np.inf],
                                  dtype=np.float32)])
    ours = oracle.to_bf16(xs)
    ref = torch.from_numpy(xs).to(torch.bfloat16).view(torch.uint16).numpy()
    assert np.array_equal(ours, ref)
    L = oracle.lib()
    for x, w in zip(xs[:2000], ref[:2000]):
        assert L.orc_float_to_bf16(ctypes.c_float(float(x))) == w
    assert np.array_equal(oracle.from_bf16(ref), torch.from_numpy(ref).view(torch.bfloat16).float().numpy())


# ---------------------------------------------------------------- reductions
@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("axis", [0, 1, 2, 3])
def test_reduce_axes_against_float64(oracle, dtype, axis):
    rng = np.random.default_rng(2)
    x = oracle.to_storage(rng.uniform(-0.1, 0.1, (3, 5, 7, 64)).astype(np.float32), dtype)
    xf = oracle.to_f32(x, dtype).astype(np.float64)
    n = x.shape[axis]
    bound = oracle.reduction_abs_error_bound(dtype, 0.1, n)
    for kind, ref in (("sum", xf.sum(axis, keepdims=True)), ("mean", xf.mean(axis, keepdims=True)),
                      ("max", xf.max(axis, keepdims=True))):
        got = oracle.to_f32(oracle.reduce(x, axis, kind, dtype), dtype)
        assert got.shape == ref.shape
        if kind == "max":
            assert np.array_equal(got, ref.astype(np.float32))  # exact (ops_reduce_test.cpp:432)
        else:
            assert np.max(np.abs(got - ref)) <= bound
    assert oracle.reduce(x, axis, "sum", dtype, keepdims=False).ndim == 3


def test_reduce_reference_bf16_vector(oracle):
    """Deterministic input of ops_reduce_test.cpp:311-314: (i % 1000) * 1e-4."""
    n = 7 * 2 * 4 * 1024
    x = oracle.to_bf16(((np.arange(n) % 1000) * 1e-4).astype(np.float32)).reshape(7, 2, 4, 1024)
    xf = oracle.from_bf16(x).astype(np.float64)
    got = oracle.from_bf16(oracle.reduce(x, -1, "sum", "bf16"))
    # the exact sum rounded once to bf16 differs from sequential float32
    # accumulation by far less than the reference bound
    assert np.max(np.abs(got - xf.sum(-1, keepdims=True))) <= oracle.reduction_abs_error_bound("bf16", 0.1, 256) * 4


def test_error_bound_formula_value(oracle):
    # 2 * K * 2 * max_abs / 2^(frac+1): fp16, K=2048, 0.1 -> 0.4
    assert abs(oracle.reduction_abs_error_bound("fp16", 0.1, 2048) - 0.4) < 1e-12
    assert abs(oracle.reduction_abs_error_bound("fp32", 1.0, 64) - 64 * 4 / 2 ** 24) < 1e-15
    with pytest.raises(AssertionError):
        oracle.reduction_abs_error_bound("bf16", 0.1, 257)


# ---------------------------------------------------------------- matmul
def test_matmul_known_answer_all_tenths(oracle):
    """ops_matmul_test.cpp:349-359: all-0.1 inputs, K = 2048."""
    a = np.full((64, 2048), 0.1, np.float32).astype(np.float16)
    b = np.full((2048, 32), 0.1, np.float32).astype(np.float16)
    c = oracle.matmul(a, b, "fp16").astype(np.float32)
    v = float(np.float16(0.1))
    assert np.all(c == c[0, 0])
    assert abs(c[0, 0] - 2048 * v * v) <= oracle.reduction_abs_error_bound("fp16", 0.1, 2048)
    assert abs(c[0, 0] - 20.48) < 0.02


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_matmul_layouts_against_float64(oracle, dtype, ta, tb):
    rng = np.random.default_rng(3)
    M, N, K = 33, 17, 96
    a = oracle.to_storage(rng.uniform(-1, 1, (K, M) if ta else (M, K)).astype(np.float32), dtype)
    b = oracle.to_storage(rng.uniform(-1, 1, (N, K) if tb else (K, N)).astype(np.float32), dtype)
    af, bf = oracle.to_f32(a, dtype).astype(np.float64), oracle.to_f32(b, dtype).astype(np.float64)
    ref = (af.T if ta else af) @ (bf.T if tb else bf)
    got = oracle.to_f32(oracle.matmul(a, b, dtype, trans_a=ta, trans_b=tb), dtype)
    assert np.max(np.abs(got - ref)) <= oracle.reduction_abs_error_bound(dtype, 1.0, K)


def test_matmul_batch_broadcast_and_permutation(oracle):
    rng = np.random.default_rng(4)
    a = rng.uniform(-1, 1, (3, 7, 8, 16)).astype(np.float32)
    b = rng.uniform(-1, 1, (1, 7, 16, 4)).astype(np.float32)
    got = oracle.matmul(a, b, "fp32")
    assert got.shape == (3, 7, 8, 4)
    assert np.allclose(got, a.astype(np.float64) @ b.astype(np.float64), atol=1e-5)
    p = np.roll(np.eye(16, dtype=np.float32), 1, axis=1)
    x = rng.standard_normal((8, 16)).astype(np.float32)
    assert np.array_equal(oracle.matmul(x, p, "fp32"), np.roll(x, 1, axis=1))
    assert np.array_equal(oracle.matmul(x, p, "fp32", trans_b=True), np.roll(x, -1, axis=1))


# ---------------------------------------------------------------- row compositions
def test_softmax_closed_form_and_invariants(oracle):
    import scipy.special
    x = np.log(np.array([[1, 2, 3, 4]], dtype=np.float64)).astype(np.float32)
    assert np.allclose(oracle.softmax(x, "fp32"), [[0.1, 0.2, 0.3, 0.4]], atol=1e-7)
    rng = np.random.default_rng(5)
    y = rng.standard_normal((16, 333)).astype(np.float32) * 3
    s = oracle.softmax(y, "fp32")
    assert np.allclose(s.sum(-1), 1, atol=1e-5)
    assert np.allclose(s, oracle.softmax(y + 5.0, "fp32"), atol=1e-6)           # shift invariance
    assert np.allclose(oracle.softmax(np.full((2, 50), 7.0, np.float32), "fp32"), 1 / 50)
    assert np.allclose(s, scipy.special.softmax(y.astype(np.float64), axis=-1), atol=1e-6)
    assert np.all(np.diff(np.take_along_axis(s, np.argsort(y, -1), -1), axis=-1) >= 0)  # monotone
    # the stepwise (storage-rounded) variant stays within a few fp16 ulps of it
    h = y.astype(np.float16)
    d = np.abs(oracle.softmax(h, "fp16").astype(np.float32) - oracle.softmax(h, "fp16", stepwise=True).astype(np.float32))
    assert d.max() < 4e-3


def test_layernorm_properties(oracle):
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((8, 512)) * 3 + 2).astype(np.float32)
    y = oracle.layernorm(x, "fp32", eps=0.0).astype(np.float64)
    assert np.allclose(y.mean(-1), 0, atol=1e-5) and np.allclose(y.var(-1), 1, atol=1e-4)
    assert np.allclose(oracle.layernorm(2 * x + 7, "fp32", eps=0.0), y, atol=1e-4)  # affine invariance
    two = oracle.layernorm(np.array([[1.0, 3.0]], np.float32), "fp32", eps=0.0)
    assert np.allclose(two, [[-1, 1]], atol=1e-6)
    # eps enters as 1/sqrt(var + eps): a row of variance 1 shrinks by 1/sqrt(1 + eps)
    z = oracle.layernorm(np.array([[-1.0, 1.0]], np.float32), "fp32", eps=3.0)
    assert np.allclose(z, [[-0.5, 0.5]], atol=1e-6)


def test_rmsnorm_properties(oracle):
    rng = np.random.default_rng(7)
    x = rng.standard_normal((8, 256)).astype(np.float32)
    y = oracle.rmsnorm(x, None, "fp32", eps=0.0).astype(np.float64)
    assert np.allclose(np.sqrt((y ** 2).mean(-1)), 1, atol=1e-5)
    assert np.allclose(oracle.rmsnorm(-3 * x, None, "fp32", eps=0.0), -y, atol=1e-5)
    one_hot = np.zeros((1, 16), np.float32)
    one_hot[0, 5] = -2.0
    out = oracle.rmsnorm(one_hot, None, "fp32", eps=0.0)
    assert np.allclose(out[0, 5], -4.0) and np.count_nonzero(out) == 1   # -2 / (2/sqrt(16))
    w = rng.uniform(0.5, 1.5, 256).astype(np.float32)
    assert np.allclose(oracle.rmsnorm(x, w, "fp32", eps=0.0), y * w, atol=1e-5)
    # eps is added to the mean square: ones with eps = 3 -> 1/sqrt(1+3)
    assert np.allclose(oracle.rmsnorm(np.ones((1, 8), np.float32), None, "fp32", eps=3.0), 0.5)


# ---------------------------------------------------------------- elementwise
def test_unary_closed_forms_and_torch(oracle):
    f = np.float32
    assert oracle.unary(np.array([0, np.log(2)], f), "exp", "fp32").tolist() == pytest.approx([1, 2], abs=1e-6)
    assert oracle.unary(np.array([0.0], f), "sigmoid", "fp32")[0] == 0.5
    assert oracle.unary(np.array([4.0], f), "rsqrt", "fp32")[0] == 0.5
    assert oracle.unary(np.array([9.0], f), "sqrt", "fp32")[0] == 3.0
    assert oracle.unary(np.array([-1.5, 0, 2], f), "relu", "fp32").tolist() == [0, 0, 2]
    x = np.random.default_rng(8).uniform(-4, 4, 4096).astype(f)
    t = torch.from_numpy(x)
    for kind, ref, tol in (("exp", torch.exp(t), 1e-5), ("sigmoid", torch.sigmoid(t), 1e-6),
                           ("gelu", torch.nn.functional.gelu(t, approximate="tanh"), 1e-6),
                           ("relu", torch.relu(t), 0)):
        got = oracle.unary(x, kind, "fp32")
        assert np.max(np.abs(got - ref.numpy()) / np.maximum(1, np.abs(ref.numpy()))) <= tol, kind
    xp = np.abs(x) + 0.1
    assert np.allclose(oracle.unary(xp, "sqrt", "fp32"), np.sqrt(xp))
    assert np.allclose(oracle.unary(xp, "rsqrt", "fp32"), 1 / np.sqrt(xp.astype(np.float64)), rtol=1e-6)
    # storage types: result is the fp32 value rounded once
    h = x.astype(np.float16)
    assert np.array_equal(oracle.unary(h, "relu", "fp16"), np.maximum(h, 0))
    assert np.array_equal(oracle.unary(h, "exp", "fp16"), np.exp(h.astype(np.float32)).astype(np.float16))


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_binary_broadcast_against_numpy(oracle, dtype):
    rng = np.random.default_rng(9)
    for sa, sb in [((2, 3, 4, 8), (2, 3, 4, 8)), ((4, 8), (1,)), ((3, 1, 8), (1, 4, 1)), ((1, 5, 6), (7, 1, 6))]:
        a = oracle.to_storage(rng.uniform(-2, 2, sa).astype(np.float32), dtype)
        b = oracle.to_storage(rng.uniform(0.5, 2, sb).astype(np.float32), dtype)
        af, bf = oracle.to_f32(a, dtype), oracle.to_f32(b, dtype)
        for kind, ref in (("add", af + bf), ("sub", af - bf), ("mul", af * bf), ("div", af / bf)):
            got = oracle.binary(a, b, kind, dtype)
            assert np.array_equal(got, oracle.to_storage(ref.astype(np.float32), dtype)), (kind, sa, sb)


def test_scalar_factor_is_cast_first(oracle):
    # 0.7 in fp16 is 0.7001953125; 1 + that = 1.7001953125 -> fp16 1.7001953125
    one = np.ones(4, np.float16)
    assert float(oracle.scalar(one, 0.7, "add", "fp16")[0]) == float(np.float16(1 + float(np.float16(0.7))))
    assert float(oracle.scalar(one * 3, 0.7, "mul", "fp16")[0]) == float(np.float16(3 * float(np.float16(0.7))))
    assert np.all(oracle.scalar(one, 7.0, "assign", "fp16") == 7)
    x = np.array([1.0], np.float32)
    assert oracle.scalar(x, 0.7, "mul", "fp32")[0] == np.float32(0.7)


def test_rope_is_complex_multiplication(oracle):
    a = np.array([1, 2, 0.5, -1], np.float32)
    b = np.array([3, 4, 2, 2], np.float32)
    assert oracle.rope(a, b, "fp32").tolist() == [-5, 10, 3, -1]   # (1+2i)(3+4i), (.5-i)(2+2i)
    rng = np.random.default_rng(10)
    x, y = rng.standard_normal((4, 64)).astype(np.float32), rng.standard_normal((4, 64)).astype(np.float32)
    z = (x[..., 0::2] + 1j * x[..., 1::2]).astype(np.complex128) * (y[..., 0::2] + 1j * y[..., 1::2])
    got = oracle.rope(x, y, "fp32")
    assert np.allclose(got[..., 0::2], z.real, atol=1e-6) and np.allclose(got[..., 1::2], z.imag, atol=1e-6)
    h = oracle.rope(x.astype(np.float16), y.astype(np.float16), "fp16").astype(np.float32)
    assert np.max(np.abs(h[..., 0::2] - z.real)) < 2e-2   # ops_rope_test.cpp:57-70 loose bound


def test_cast_against_numpy_and_torch(oracle):
    x = np.random.default_rng(11).uniform(-100, 100, 5000).astype(np.float32)
    assert np.array_equal(oracle.cast(x, "fp32", "fp16"), x.astype(np.float16))
    assert np.array_equal(oracle.cast(x, "fp32", "bf16"),
                          torch.from_numpy(x).to(torch.bfloat16).view(torch.uint16).numpy())
    h = x.astype(np.float16)
    assert np.array_equal(oracle.cast(h, "fp16", "fp32"), h.astype(np.float32))


def test_tensor_compare_fields(oracle):
    a = np.array([1.0, 2.0, 0.0, -4.0], np.float32)
    b = np.array([1.0, 2.5, 0.0, -3.0], np.float32)
    r = oracle.tensor_compare(a, b, "fp32")
    assert r["max_diff"] == 1.0 and r["num_wrong"] == 2 and r["num_total"] == 4
    assert abs(r["mse"] - (0.25 + 1.0) / 4) < 1e-7
    assert abs(r["max_error_rate"] - 0.25) < 1e-7      # |4-3| / max(4,3)


# ---------------------------------------------------------------- task_seq
def test_task_seq_round_robin_closed_form(oracle):
    # granularity 1, one slot: processor p runs p, p+n, p+2n, ...
    for grid, ntasks in [(4, 10), (8, 8), (5, 3), (108, 172)]:
        seen = []
        for block in range(grid):
            ids = oracle.task_seq(block, grid, (0, grid, 1), 0, (0, ntasks, 1), 1, 1, 0)
            assert ids == list(range(block, ntasks, grid))
            seen += ids
        assert sorted(seen) == list(range(ntasks))


def test_task_seq_granularity_and_slots_every_task_once(oracle):
    import itertools
    for grid, pb, pe, ntasks, gran, nslots, cur in itertools.product(
            [6, 8], [0, 2], [4, 6], [1, 7, 23, 48], [1, 2, 3], [1, 2, 4], [0, 1]):
        if pb >= pe or pe > grid:
            continue
        pc = pb + cur % (pe - pb)
        if pc != pb and pb != 0:
            continue  # the wrap through gridDim only stays in range for ranges starting at 0
        seen = []
        for block in range(grid):
            for k in range(nslots):
                ids = oracle.task_seq(block, grid, (pb, pe, 1), pc, (0, ntasks, 1), gran, nslots, k)
                assert ids == sorted(ids)
                seen += ids
        if pc == pb or pe - pb == grid:
            assert sorted(seen) == list(range(ntasks)), (grid, pb, pe, ntasks, gran, nslots, pc)


def test_task_seq_documented_formula(oracle):
    """codegen.cpp:318-385: the t-th task of processor index p is
    task_b + task_s*(p*gran + t//gran*gran*n_procs + t%gran)."""
    grid, gran, nprocs = 4, 3, 4
    for p in range(nprocs):
        ids = oracle.task_seq(p, grid, (0, 4, 1), 0, (0, 40, 1), gran, 1, 0)
        want = [p * gran + t // gran * gran * nprocs + t % gran for t in range(40)]
        want = want[:len(ids)]
        assert ids == want and all(i < 40 for i in ids)
    # rotation: proc_cur = 1 makes block 1 the first dealer
    assert oracle.task_seq(1, 4, (0, 4, 1), 1, (0, 8, 1), 1, 1, 0) == [0, 4]
    assert oracle.task_seq(0, 4, (0, 4, 1), 1, (0, 8, 1), 1, 1, 0) == [3, 7]


def test_plan_oracle_task_ids_agree_with_c(oracle):
    from oracle import plan_oracle as P
    step = ("tasks", 0, 6, 1, 2, 0, 50, 1, 2, 2, 4, 0, 0)
    for block in range(8):
        for k in range(2):
            assert P.task_ids(step, block, 8, k) == oracle.task_seq(block, 8, (0, 6, 1), 2, (0, 50, 1), 2, 2, k)


def test_embedding_oracle_by_brute_force(oracle):
    """The gather restated from ark/ops/ops_embedding_test.cpp:11-41, checked element by element
    with plain loops on a tiny case, negative indices (counted from the end of the table) included,
    and against the one-hot matrix product that defines an embedding lookup."""
    rng = np.random.default_rng(3)
    table = rng.standard_normal((7, 5)).astype(np.float32)
    idx = np.array([[0, 6, -1], [3, -7, 2]], dtype=np.int32)
    got = oracle.embedding(idx, table)
    assert got.shape == (2, 3, 5)
    for i in range(2):
        for j in range(3):
            row = int(idx[i, j])
            row = row + 7 if row < 0 else row
            for c in range(5):
                assert got[i, j, c] == table[row, c]
    onehot = np.zeros((6, 7), np.float32)
    flat = np.where(idx.reshape(-1) < 0, idx.reshape(-1) + 7, idx.reshape(-1))
    onehot[np.arange(6), flat] = 1.0
    assert np.array_equal(got.reshape(6, 5), onehot @ table)


def test_int32_arithmetic_by_python_integers(oracle):
    """INT32 add/sub/mul/div of the oracle against Python's unbounded integers reduced to 32-bit
    two's complement, on values that overflow, and C's truncation toward zero for the quotient."""
    rng = np.random.default_rng(3)
    a = rng.integers(-2 ** 31, 2 ** 31, 4096, dtype=np.int64).astype(np.int32)
    b = rng.integers(-2 ** 31, 2 ** 31, 4096, dtype=np.int64).astype(np.int32)
    b[:64] = rng.integers(-9, 10, 64)  # small divisors, zeros among them
    a[64:72] = -2 ** 31
    b[64:72] = -1

    def wrap(v):
        v &= 0xFFFFFFFF
        return v - (1 << 32) if v >= 1 << 31 else v

    def cdiv(x, y):
        if y == 0 or (x == -2 ** 31 and y == -1):
            return 0
        q = abs(x) // abs(y)
        return -q if (x < 0) != (y < 0) else q
    for kind, f in (("add", lambda x, y: wrap(x + y)), ("sub", lambda x, y: wrap(x - y)),
                    ("mul", lambda x, y: wrap(x * y)), ("div", cdiv)):
        want = np.array([f(int(x), int(y)) for x, y in zip(a, b)], np.int64).astype(np.int32)
        assert np.array_equal(oracle.binary(a, b, kind, "int32"), want), kind
    assert list(oracle.binary(np.array([7, -7, 7, -7], np.int32), np.array([2, 2, -2, -2], np.int32), "div", "int32")) == [3, -3, -3, 3]
    assert list(oracle.scalar(np.array([5, -5], np.int32), 2.9, "mul", "int32")) == [10, -10]
    assert list(oracle.scalar(np.array([5, -5], np.int32), -2.9, "add", "int32")) == [3, -7]
    assert list(oracle.scalar(np.array([5, -5], np.int32), 7.0, "assign", "int32")) == [7, 7]
