"""GPU parity of the row ops (reduce / softmax / layernorm / RMSNorm) against
the CPU oracle on the same seeded inputs, through the C ABI.

Shapes follow the reference's reduce tests (ark/ops/ops_reduce_test.cpp:
254-377: [7,2,4,1024], [1,1,2,8192] ...), plus ragged lengths for the general
path, and the full benchmark shape X[16384,4096].

Tolerances: reductions and normalisations accumulate in fp32 on both sides, so
results may differ only by summation order and one rounding to storage:
max relative error <= 1e-3 (fp32/fp16 storage; bf16 storage has an 8-bit
significand, its bound is one output ulp = 2^-7), reduce_max is exact
(ops_reduce_test.cpp:432).
"""
import numpy as np
import pytest
import torch

from helpers import make, to_gpu, to_np

pytestmark = pytest.mark.gpu

REL_TOL = {"fp32": 1e-3, "fp16": 1e-3, "bf16": 2.0 ** -7}
SHAPES = [(7, 2, 4, 1024), (1, 1, 2, 8192), (3, 5, 1000), (64, 4096), (9, 333),
          (2, 3, 2056), (4, 17000), (130, 8), (5, 1)]


def _check(oracle, ref, got, dtype, exact=False):
    if exact:
        assert np.array_equal(ref, got)
        return
    rel, abs_rest, mx = oracle.max_rel_error(ref, got, dtype)
    assert rel <= REL_TOL[dtype], (rel, abs_rest, mx)
    assert abs_rest <= REL_TOL[dtype] * max(mx, 1e-30), (rel, abs_rest, mx)


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("kind", ["sum", "max", "mean"])
def test_reduce(oracle, kind, shape, dtype):
    from ark_amd import ops
    x = make(oracle, shape, dtype, seed=hash((kind, shape)) % 2**31)
    ref = oracle.reduce(x, -1, kind, dtype)
    got = to_np(ops.row_op("reduce_" + kind, to_gpu(x, dtype)), dtype)
    assert got.shape == ref.shape
    _check(oracle, ref, got, dtype, exact=(kind == "max"))


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES)
def test_softmax(oracle, shape, dtype):
    from ark_amd import ops
    x = make(oracle, shape, dtype, seed=11, scale=2.0)
    ref = oracle.softmax(x, dtype)
    got = to_np(ops.softmax(to_gpu(x, dtype)), dtype)
    _check(oracle, ref, got, dtype)
    rows = oracle.to_f32(got, dtype).reshape(-1, shape[-1]).sum(-1)
    # rows sum to 1 up to one storage rounding per element
    assert np.allclose(rows, 1.0, atol=4 * REL_TOL[dtype])


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_softmax_in_place(oracle, dtype):
    from ark_amd import ops
    for shape in [(33, 2048), (7, 999)]:
        x = make(oracle, shape, dtype, seed=5)
        ref = oracle.softmax(x, dtype)
        t = to_gpu(x, dtype)
        ops.softmax(t, out=t)
        _check(oracle, ref, to_np(t, dtype), dtype)


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES[:-1])
def test_layernorm(oracle, shape, dtype):
    from ark_amd import ops
    x = make(oracle, shape, dtype, seed=12)
    x = oracle.to_storage(oracle.to_f32(x, dtype) + 0.5, dtype)
    ref = oracle.layernorm(x, dtype, eps=1e-6)
    got = to_np(ops.layernorm(to_gpu(x, dtype), eps=1e-6), dtype)
    _check(oracle, ref, got, dtype)


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("wkind", ["none", "fp32", "same"])
def test_rmsnorm(oracle, shape, dtype, wkind):
    from ark_amd import ops
    x = make(oracle, shape, dtype, seed=13)
    cols = shape[-1]
    w = np.random.default_rng(14).uniform(0.5, 1.5, cols).astype(np.float32)
    wt = None
    wref = None
    if wkind == "fp32":
        wt = torch.from_numpy(w).cuda()
        wref = w
    elif wkind == "same":
        ws = oracle.to_storage(w, dtype)
        wt = to_gpu(ws, dtype)
        wref = oracle.to_f32(ws, dtype)
    for eps in (0.0, 1e-6):
        ref = oracle.rmsnorm(x, wref, dtype, eps=eps)
        got = to_np(ops.rmsnorm(to_gpu(x, dtype), wt, eps=eps), dtype)
        _check(oracle, ref, got, dtype)


def test_strided_rows(oracle):
    """Row pitch larger than the row length (a padded / offset view)."""
    from ark_amd import ops
    dtype = "fp16"
    full = make(oracle, (40, 1536), dtype, seed=3)
    t = to_gpu(full, dtype)[:, 256:256 + 1024]
    ref = oracle.softmax(np.ascontiguousarray(full[:, 256:1280]), dtype)
    out = torch.empty(40, 1024, dtype=torch.float16, device="cuda")
    ops.softmax(t, out=out)
    _check(oracle, ref, to_np(out, dtype), dtype)
    ref = oracle.reduce(np.ascontiguousarray(full[:, 256:1280]), -1, "sum", dtype)
    _check(oracle, ref, to_np(ops.reduce_sum(t), dtype), dtype)


def test_full_size_config(oracle):
    """X[16384,4096] fp16 ~ N(0,1): all three row ops of the benchmark config."""
    from ark_amd import ops
    dtype = "fp16"
    x = make(oracle, (16384, 4096), dtype, seed=2024)
    w = np.random.default_rng(7).uniform(0.5, 1.5, 4096).astype(np.float32)
    t = to_gpu(x, dtype)
    _check(oracle, oracle.reduce(x, -1, "sum", dtype), to_np(ops.reduce_sum(t), dtype), dtype)
    _check(oracle, oracle.softmax(x, dtype), to_np(ops.softmax(t), dtype), dtype)
    _check(oracle, oracle.rmsnorm(x, w, dtype, eps=1e-6),
           to_np(ops.rmsnorm(t, torch.from_numpy(w).cuda(), eps=1e-6), dtype), dtype)


def test_errors():
    from ark_amd import ops, ArkmiError
    x = torch.zeros(4, 8, dtype=torch.int32, device="cuda")
    with pytest.raises(TypeError):
        ops.softmax(x)
    with pytest.raises(ValueError):
        ops.softmax(torch.zeros(4, 8))


def test_row_ops_over_one_tensor_cached_and_streamed_inputs_agree(oracle, monkeypatch):
    """reduce_sum, softmax and RMSNorm over the same X in one plan: the first two fetch X through
    the caches because a later op reads it again, the last one streams it.  The load policy changes
    no value: the same bits with every input streamed (ARKMI_ROW_CACHED_INPUT=0), and the softmax
    against the oracle."""
    from ark_amd import Model, Executor
    dtype = "fp16"
    x = make(oracle, (2048, 4096), dtype, seed=77, dist="normal")
    w = np.random.default_rng(5).uniform(0.5, 1.5, 4096).astype(np.float32)

    def run():
        m = Model()
        tx, tw = m.tensor([2048, 4096], dtype), m.tensor([4096], "fp32")
        outs = [m.reduce_sum(tx, -1), m.softmax(tx), m.rmsnorm(tx, tw, 1e-6)]
        ex = Executor(m.plan(device_id=0)).compile()
        ex.tensor_write(tx, x)
        ex.tensor_write(tw, w)
        ex.launch()
        ex.run(2)
        ex.wait()
        got = [ex.tensor_read(t) for t in outs]
        ex.stop()
        return got

    a = run()
    monkeypatch.setenv("ARKMI_ROW_CACHED_INPUT", "0")
    b = run()
    for p, q in zip(a, b):
        assert np.array_equal(p, q)
    ref = oracle.softmax(x, dtype)
    assert np.abs(oracle.to_f32(a[1], dtype) - oracle.to_f32(ref, dtype)).max() <= 1e-3
