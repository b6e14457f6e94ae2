"""ctypes front end of oracle/oracle.c plus numpy-only helpers.

TEST INFRASTRUCTURE ONLY: the checker for the HIP path and the timed CPU
baseline; never part of the product path.

Arrays in fp16 are numpy float16; arrays in bf16 are numpy uint16 bit patterns
(see `to_bf16` / `from_bf16`).  dtype names: "fp32", "fp16", "bf16".
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

DT = {"fp32": 0, "fp16": 1, "bf16": 2}
NP_STORAGE = {"fp32": np.float32, "fp16": np.float16, "bf16": np.uint16}
FRAC_BITS = {"fp32": 23, "fp16": 10, "bf16": 7}
SUBNORMAL_QUANTUM = {"fp32": 2.0 ** -149, "fp16": 2.0 ** -24, "bf16": 2.0 ** -133}


def build():
    """Compile oracle.c into liboracle.so (gcc, a second or two)."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
        _LIB.orc_half_to_float.restype = ctypes.c_float
        _LIB.orc_half_to_float.argtypes = [ctypes.c_uint16]
        _LIB.orc_float_to_half.restype = ctypes.c_uint16
        _LIB.orc_float_to_half.argtypes = [ctypes.c_float]
        _LIB.orc_bf16_to_float.restype = ctypes.c_float
        _LIB.orc_bf16_to_float.argtypes = [ctypes.c_uint16]
        _LIB.orc_float_to_bf16.restype = ctypes.c_uint16
        _LIB.orc_float_to_bf16.argtypes = [ctypes.c_float]
        _LIB.orc_num_threads.restype = ctypes.c_int
        _LIB.orc_task_seq.restype = ctypes.c_int64
    return _LIB


def num_threads():
    return int(lib().orc_num_threads())


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _i64x4(v):
    return (ctypes.c_int64 * 4)(*[int(x) for x in v])


def _c(a, dtype):
    a = np.ascontiguousarray(a)
    assert a.dtype == NP_STORAGE[dtype], (a.dtype, dtype)
    return a


def dims4(shape):
    """Left-pad a shape with 1s to 4 dims (ark/api/dims.cpp:59-68)."""
    shape = [int(s) for s in shape]
    assert len(shape) <= 4
    return [1] * (4 - len(shape)) + shape


# ---------------------------------------------------------------- dtypes
def to_bf16(x):
    """float32 array -> bf16 bit patterns (uint16), round to nearest even."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return r.astype(np.uint16)


def from_bf16(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def to_storage(x, dtype):
    """float32 values -> storage array of `dtype` (one RNE rounding)."""
    x = np.asarray(x, dtype=np.float32)
    if dtype == "fp32":
        return np.ascontiguousarray(x)
    if dtype == "fp16":
        return x.astype(np.float16)
    return to_bf16(x)


def to_f32(a, dtype):
    if dtype == "bf16":
        return from_bf16(a)
    return np.asarray(a).astype(np.float32)


def reduction_abs_error_bound(dtype, max_abs, length):
    """ark/ops/ops_test_common.hpp:52-69."""
    fb = FRAC_BITS[dtype]
    assert length <= (1 << (fb + 1)), "reduction length is too large"
    return length * 2 * max_abs * 1.0 / (1 << (fb + 1)) * 2


# ------------------------------------------------------------- C wrappers
def reduce(x, axis, kind, dtype, keepdims=True):
    """kind in {"sum","max","mean"}; x of any rank <= 4."""
    x = _c(x, dtype)
    nd = x.ndim
    axis = axis % nd
    sh4 = dims4(x.shape)
    ax4 = axis + (4 - nd)
    osh = list(sh4)
    osh[ax4] = 1
    out = np.empty(osh, dtype=NP_STORAGE[dtype])
    lib().orc_reduce(_p(x), _p(out), _i64x4(sh4), ctypes.c_int(ax4),
                     ctypes.c_int({"sum": 0, "max": 1, "mean": 2}[kind]),
                     ctypes.c_int(DT[dtype]))
    oshape = list(x.shape)
    if keepdims:
        oshape[axis] = 1
    else:
        del oshape[axis]
    return out.reshape(oshape)


def softmax(x, dtype, stepwise=False):
    x = _c(x, dtype)
    cols = x.shape[-1]
    rows = x.size // cols
    out = np.empty_like(x)
    fn = lib().orc_softmax_rows_stepwise if stepwise else lib().orc_softmax_rows
    fn(_p(x), _p(out), ctypes.c_int64(rows), ctypes.c_int64(cols),
       ctypes.c_int(DT[dtype]))
    return out


def layernorm(x, dtype, eps=1e-6):
    x = _c(x, dtype)
    cols = x.shape[-1]
    rows = x.size // cols
    out = np.empty_like(x)
    lib().orc_layernorm_rows(_p(x), _p(out), ctypes.c_int64(rows),
                             ctypes.c_int64(cols), ctypes.c_float(eps),
                             ctypes.c_int(DT[dtype]))
    return out


def rmsnorm(x, weight, dtype, eps=0.0):
    x = _c(x, dtype)
    cols = x.shape[-1]
    rows = x.size // cols
    out = np.empty_like(x)
    if weight is not None:
        weight = np.ascontiguousarray(weight, dtype=np.float32).reshape(-1)
        assert weight.size == cols
    lib().orc_rmsnorm_rows(_p(x), _p(weight) if weight is not None else None,
                           _p(out), ctypes.c_int64(rows), ctypes.c_int64(cols),
                           ctypes.c_float(eps), ctypes.c_int(DT[dtype]))
    return out


def matmul(a, b, dtype, trans_a=False, trans_b=False):
    """Batched matmul with NumPy broadcasting of the batch dims; 2-D+ inputs."""
    a = _c(a, dtype)
    b = _c(b, dtype)
    if a.ndim == 1:
        a = a.reshape(1, -1)
    M, K = (a.shape[-1], a.shape[-2]) if trans_a else (a.shape[-2], a.shape[-1])
    N = b.shape[-2] if trans_b else b.shape[-1]
    Kb = b.shape[-1] if trans_b else b.shape[-2]
    assert K == Kb, (a.shape, b.shape, trans_a, trans_b)
    ba, bb = a.shape[:-2], b.shape[:-2]
    bshape = np.broadcast_shapes(ba, bb)
    nb = int(np.prod(bshape)) if bshape else 1
    out = np.empty(tuple(bshape) + (M, N), dtype=NP_STORAGE[dtype])
    a3 = np.ascontiguousarray(np.broadcast_to(a, tuple(bshape) + a.shape[-2:])).reshape((nb,) + a.shape[-2:])
    b3 = np.ascontiguousarray(np.broadcast_to(b, tuple(bshape) + b.shape[-2:])).reshape((nb,) + b.shape[-2:])
    lib().orc_matmul(_p(a3), _p(b3), _p(out), ctypes.c_int64(nb),
                     ctypes.c_int64(M), ctypes.c_int64(N), ctypes.c_int64(K),
                     ctypes.c_int64(a3.shape[-1]), ctypes.c_int64(b3.shape[-1]),
                     ctypes.c_int64(N), ctypes.c_int64(a3.shape[-1] * a3.shape[-2]),
                     ctypes.c_int64(b3.shape[-1] * b3.shape[-2]),
                     ctypes.c_int64(M * N), ctypes.c_int(int(trans_a)),
                     ctypes.c_int(int(trans_b)), ctypes.c_int(DT[dtype]))
    return out


_UNARY = {"exp": 0, "gelu": 1, "relu": 2, "rsqrt": 3, "sigmoid": 4, "sqrt": 5, "copy": 6}
_BINARY = {"add": 0, "sub": 1, "mul": 2, "div": 3}
_SCALAR = {"assign": 0, "add": 1, "mul": 2}


def unary(x, kind, dtype):
    x = _c(x, dtype)
    out = np.empty_like(x)
    lib().orc_unary(_p(x), _p(out), ctypes.c_int64(x.size),
                    ctypes.c_int(_UNARY[kind]), ctypes.c_int(DT[dtype]))
    return out


def _int32_op(a, b, kind):
    """INT32 arithmetic as C computes it on two's-complement words: + - * wrap around, / truncates
    toward zero (the reference's functors are `a + b` ... `a / b` on the element type,
    ark/include/kernels/common/type_intrinsics.h:174-252; a scalar op casts its float value to the
    element type first, ark/include/kernels/scalar.h:13-41).  x / 0 and INT_MIN / -1, undefined in C, are 0 here."""
    a64, b64 = np.asarray(a, np.int32).astype(np.int64), np.asarray(b, np.int32).astype(np.int64)
    if kind == "add":
        r = a64 + b64
    elif kind == "sub":
        r = a64 - b64
    elif kind == "mul":
        r = a64 * b64  # |product| < 2^62: exact in int64
    else:
        bad = (b64 == 0) | ((a64 == -2 ** 31) & (b64 == -1))
        safe = np.where(bad, 1, b64)
        q = np.abs(a64) // np.abs(safe)
        r = np.where(bad, 0, np.where((a64 < 0) != (safe < 0), -q, q))
    return (r & 0xFFFFFFFF).astype(np.uint32).view(np.int32)


def binary(a, b, kind, dtype):
    if dtype == "int32":
        a, b = np.broadcast_arrays(np.asarray(a, np.int32), np.asarray(b, np.int32))
        return _int32_op(a, b, kind)
    a = _c(a, dtype)
    b = _c(b, dtype)
    oshape = np.broadcast_shapes(a.shape, b.shape)
    out = np.empty(oshape, dtype=NP_STORAGE[dtype])
    nd = len(oshape)
    ash = dims4((1,) * (nd - a.ndim) + a.shape)
    bsh = dims4((1,) * (nd - b.ndim) + b.shape)
    lib().orc_binary(_p(a), _i64x4(ash), _p(b), _i64x4(bsh), _p(out),
                     _i64x4(dims4(oshape)), ctypes.c_int(_BINARY[kind]),
                     ctypes.c_int(DT[dtype]))
    return out


def scalar(x, factor, kind, dtype):
    if dtype == "int32":  # the factor is converted like a C cast (toward zero)
        x = np.asarray(x, np.int32)
        f = np.full(x.shape, int(np.float32(factor)), np.int32)
        return f if kind == "assign" else _int32_op(x, f, kind)
    x = _c(x, dtype)
    out = np.empty_like(x)
    lib().orc_scalar(_p(x), _p(out), ctypes.c_int64(x.size),
                     ctypes.c_float(factor), ctypes.c_int(_SCALAR[kind]),
                     ctypes.c_int(DT[dtype]))
    return out


def rope(x, other, dtype):
    x = _c(x, dtype)
    other = _c(np.broadcast_to(other, x.shape), dtype)
    out = np.empty_like(x)
    lib().orc_rope(_p(x), _p(other), _p(out), ctypes.c_int64(x.size),
                   ctypes.c_int(DT[dtype]))
    return out


def cast(x, src, dst):
    x = _c(x, src)
    out = np.empty(x.shape, dtype=NP_STORAGE[dst])
    lib().orc_convert(_p(x), ctypes.c_int(DT[src]), _p(out),
                      ctypes.c_int(DT[dst]), ctypes.c_int64(x.size))
    return out


def embedding(indices, weight, clamp=False):
    """out[..., :] = weight[indices[...], :], negative indices counted from the end of the
    table (the host baseline of ark/ops/ops_embedding_test.cpp:11-41).  Pure data movement:
    works on the storage bits of any type.  An index outside [-rows, rows) has no meaning in the
    reference (its baseline and its kernel both read outside the table); with `clamp` such an
    index takes the nearest row after the wrap, which is what the device code here does."""
    idx = np.asarray(indices, dtype=np.int64)
    idx = np.where(idx < 0, idx + weight.shape[0], idx)
    if clamp:
        idx = np.clip(idx, 0, weight.shape[0] - 1)
    return np.ascontiguousarray(weight[idx])


def tensor_compare(truth, got, dtype):
    """Returns dict(mse, max_diff, max_error_rate, num_wrong, num_total)."""
    truth = _c(truth, dtype)
    got = _c(got, dtype)
    assert truth.shape == got.shape, (truth.shape, got.shape)
    res = (ctypes.c_double * 4)()
    lib().orc_tensor_compare(_p(truth), _p(got), ctypes.c_int64(truth.size),
                             ctypes.c_int(DT[dtype]), res)
    return dict(mse=res[0], max_diff=res[1], max_error_rate=res[2],
                num_wrong=int(res[3]), num_total=truth.size)


def max_rel_error(truth, got, dtype, floor_frac=1e-3):
    """The acceptance metric: max |a-b|/max(|a|,|b|) over elements whose
    reference magnitude exceeds floor_frac * max|ref| (near-zero elements are
    judged by absolute difference instead; cf. examples/llama/model_test.py:231-233)."""
    t = to_f32(truth, dtype).astype(np.float64).ravel()
    g = to_f32(got, dtype).astype(np.float64).ravel()
    assert np.all(np.isfinite(g)), "non-finite values in result"
    mx = np.max(np.abs(t)) if t.size else 0.0
    sel = np.abs(t) > floor_frac * mx
    denom = np.maximum(np.abs(t), np.abs(g))
    rel = np.zeros_like(t)
    # a difference of one subnormal quantum of the storage format is a
    # rounding flip, not an arithmetic error (fp16: 2^-24)
    diff = np.abs(t - g)
    diff = np.where(diff <= SUBNORMAL_QUANTUM[dtype], 0.0, diff)
    np.divide(diff, denom, out=rel, where=denom > 0)
    rel_sel = float(rel[sel].max()) if sel.any() else 0.0
    abs_rest = float(np.abs(t - g)[~sel].max()) if (~sel).any() else 0.0
    return rel_sel, abs_rest, float(mx)


def task_seq(block, grid, proc, proc_cur, task, gran, n_slots, k):
    """Task ids run by (block, slot k) per kernel_template.in:11-27.
    proc = (b, e, s), task = (b, e, s)."""
    cap = max(1, (task[1] - task[0]) // max(1, task[2]) + 1)
    buf = (ctypes.c_int64 * cap)()
    i64 = ctypes.c_int64
    n = lib().orc_task_seq(i64(block), i64(grid), i64(proc[0]), i64(proc[1]),
                           i64(proc[2]), i64(proc_cur), i64(task[0]),
                           i64(task[1]), i64(task[2]), i64(gran), i64(n_slots),
                           i64(k), buf, i64(cap))
    return list(buf[:n])
