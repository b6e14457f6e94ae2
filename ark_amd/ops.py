"""Stand-alone op launchers over the C ABI, on torch device tensors.

Each function enqueues one kernel on torch's current stream and returns the
output tensor.  Tensors carry memory only; all compute is in libarkmi.so.
"""
import ctypes

import torch

from ._lib import lib, check, DTYPES

_TORCH_DT = {torch.float32: "fp32", torch.float16: "fp16", torch.bfloat16: "bf16"}
ROW_KINDS = {"reduce_sum": 0, "reduce_max": 1, "reduce_mean": 2, "softmax": 3,
             "layernorm": 4, "rmsnorm": 5}


def _dt(t):
    try:
        return DTYPES[_TORCH_DT[t.dtype]]
    except KeyError:
        raise TypeError(f"unsupported tensor dtype {t.dtype}")


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def _require_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("ark_amd ops run on the GPU only; got a CPU tensor")


def row_op(kind, x, weight=None, eps=0.0, out=None):
    """kind in ROW_KINDS; x: [..., cols] with a dense last axis and uniform row pitch."""
    _require_cuda(x, weight, out)
    cols = x.shape[-1]
    x2 = x.reshape(-1, cols)
    if x2.stride(-1) != 1:
        raise ValueError("last axis must be dense")
    rows = x2.shape[0]
    is_reduce = ROW_KINDS[kind] <= 2
    if out is None:
        out = torch.empty(x.shape[:-1] + (1,) if is_reduce else x.shape,
                          dtype=x.dtype, device=x.device)
    o2 = out.reshape(rows, -1)
    wfp32 = 0
    if weight is not None:
        if weight.numel() != cols:
            raise ValueError("weight length must equal the row length")
        wfp32 = 1 if weight.dtype == torch.float32 else 0
        if not wfp32 and weight.dtype != x.dtype:
            raise TypeError("weight must be fp32 or the tensor dtype")
        weight = weight.contiguous()
    check(lib().arkmi_row_op(
        ctypes.c_int(ROW_KINDS[kind]), ctypes.c_int(_dt(x)), _ptr(x2), _ptr(o2),
        _ptr(weight), ctypes.c_int(wfp32), ctypes.c_int64(rows), ctypes.c_int64(cols),
        ctypes.c_int64(x2.stride(0) if rows > 1 else cols),
        ctypes.c_int64(o2.stride(0) if rows > 1 else o2.shape[-1]),
        ctypes.c_float(eps), _stream()))
    return out


def reduce_sum(x, out=None):
    return row_op("reduce_sum", x, out=out)


def reduce_max(x, out=None):
    return row_op("reduce_max", x, out=out)


def reduce_mean(x, out=None):
    return row_op("reduce_mean", x, out=out)


def softmax(x, out=None):
    return row_op("softmax", x, out=out)


def layernorm(x, eps=1e-6, out=None):
    return row_op("layernorm", x, eps=eps, out=out)


def rmsnorm(x, weight=None, eps=0.0, out=None):
    return row_op("rmsnorm", x, weight=weight, eps=eps, out=out)


def matmul(a, b, out=None, trans_b=False, tile=(0, 0), trans_a=False):
    """C = A @ B (A^T when trans_a: A given as [..., k, m]; B^T when trans_b: B given
    as [..., n, k]); 2-D or batched 3-D/4-D operands whose batch dims are equal or
    broadcast (size 1)."""
    _require_cuda(a, b, out)
    if a.dtype != b.dtype:
        raise TypeError("operand dtypes differ")
    m, k = (a.shape[-1], a.shape[-2]) if trans_a else (a.shape[-2], a.shape[-1])
    n = b.shape[-2] if trans_b else b.shape[-1]
    kb = b.shape[-1] if trans_b else b.shape[-2]
    if k != kb:
        raise ValueError(f"inner dimensions differ: {tuple(a.shape)} x {tuple(b.shape)}")
    ba, bb = a.shape[:-2], b.shape[:-2]
    bshape = torch.broadcast_shapes(ba, bb)
    nb = 1
    for s_ in bshape:
        nb *= s_
    a3 = a.reshape((-1,) + tuple(a.shape[-2:]))
    b3 = b.reshape((-1,) + tuple(b.shape[-2:]))
    if a3.shape[0] not in (1, nb) or b3.shape[0] not in (1, nb):
        raise ValueError("only full or size-1 batch broadcasting is supported")
    if a3.stride(-1) != 1 or b3.stride(-1) != 1:
        raise ValueError("innermost axis must be dense")
    if out is None:
        out = torch.empty(tuple(bshape) + (m, n), dtype=a.dtype, device=a.device)
    o3 = out.reshape(-1, m, n)
    check(lib().arkmi_gemm(
        ctypes.c_int(_dt(a)), _ptr(a3), _ptr(b3), _ptr(o3), ctypes.c_int(nb),
        ctypes.c_int(m), ctypes.c_int(n), ctypes.c_int(k),
        ctypes.c_int64(a3.stride(1)), ctypes.c_int64(b3.stride(1)), ctypes.c_int64(o3.stride(1)),
        ctypes.c_int64(a3.stride(0) if a3.shape[0] > 1 else 0),
        ctypes.c_int64(b3.stride(0) if b3.shape[0] > 1 else 0),
        ctypes.c_int64(o3.stride(0) if nb > 1 else 0),
        ctypes.c_int(int(trans_a)), ctypes.c_int(int(trans_b)), ctypes.c_int(tile[0]), ctypes.c_int(tile[1]),
        _stream()))
    return out


_GEMV_WS = {}


def gemv(x, w, out=None, num_tasks=0):
    """Y = X @ W for a skinny X: x [m, k] with 1 <= m <= 16 (or 1-D [k]), w [k, n]
    row-major, n % 8 == 0.  num_tasks: workgroups W is dealt to, 0 = one per CU."""
    _require_cuda(x, w, out)
    if x.dtype != w.dtype:
        raise TypeError("operand dtypes differ")
    x2 = x.reshape(1, -1) if x.dim() == 1 else x
    m, k = x2.shape
    if w.shape[0] != k:
        raise ValueError(f"inner dimensions differ: {tuple(x.shape)} x {tuple(w.shape)}")
    n = w.shape[1]
    if x2.stride(-1) != 1 or w.stride(-1) != 1:
        raise ValueError("innermost axis must be dense")
    ntasks, need = ctypes.c_int(), ctypes.c_size_t()
    check(lib().arkmi_gemv_plan(ctypes.c_int(m), ctypes.c_int(n), ctypes.c_int(k),
                                ctypes.c_int(num_tasks), ctypes.byref(ntasks), ctypes.byref(need)))
    ws = None
    if need.value:
        # one zeroed workspace per (device, stream, size): the kernel leaves its counters zero
        key = (x.device.index, torch.cuda.current_stream().cuda_stream, need.value)
        ws = _GEMV_WS.get(key)
        if ws is None:
            ws = torch.zeros(need.value, dtype=torch.uint8, device=x.device)
            _GEMV_WS[key] = ws
    if out is None:
        out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    o2 = out.reshape(m, n)
    check(lib().arkmi_gemv(
        ctypes.c_int(_dt(x2)), _ptr(x2), _ptr(w), _ptr(o2), ctypes.c_int(m), ctypes.c_int(n),
        ctypes.c_int(k), ctypes.c_int64(x2.stride(0)), ctypes.c_int64(w.stride(0)),
        ctypes.c_int64(o2.stride(0)), ctypes.c_int(ntasks.value), _ptr(ws),
        ctypes.c_size_t(need.value), _stream()))
    return out.reshape(n) if x.dim() == 1 and out.dim() == 2 and out.shape[0] == 1 else out


def gemv_static(x, w, out, num_tasks=0):
    """gemv() through the entry point that allocates nothing: the workspace is a fixed array inside
    the library (arkmi_gemv_static_limit() bytes per GPU) and `out` must be given.  Calls on one GPU
    share that array and must not overlap in time."""
    _require_cuda(x, w, out)
    if x.dtype != w.dtype:
        raise TypeError("operand dtypes differ")
    x2 = x.reshape(1, -1) if x.dim() == 1 else x
    m, k = x2.shape
    if w.shape[0] != k:
        raise ValueError(f"inner dimensions differ: {tuple(x.shape)} x {tuple(w.shape)}")
    n = w.shape[1]
    if x2.stride(-1) != 1 or w.stride(-1) != 1:
        raise ValueError("innermost axis must be dense")
    o2 = out.reshape(m, n)
    check(lib().arkmi_gemv_static(
        ctypes.c_int(_dt(x2)), _ptr(x2), _ptr(w), _ptr(o2), ctypes.c_int(m), ctypes.c_int(n),
        ctypes.c_int(k), ctypes.c_int64(x2.stride(0)), ctypes.c_int64(w.stride(0)),
        ctypes.c_int64(o2.stride(0)), ctypes.c_int(num_tasks), _stream()))
    return out


def gemv_static_limit():
    lib().arkmi_gemv_static_limit.restype = ctypes.c_size_t
    return int(lib().arkmi_gemv_static_limit())
