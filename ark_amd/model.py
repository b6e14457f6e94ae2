"""Python host side of the model / planner API over the C ABI.

Names and argument meaning follow the reference's Python frontend
(python/ark/ops.py, planner.py) one level down: a `Model` object instead of a
global singleton, tensors as light handles.  Everything is executed by
libarkmi.so; nothing here computes.
"""
import ctypes
import json
import math

from ._lib import lib, check, DTYPES, InvalidUsageError

_DT_NAMES = {v: k for k, v in DTYPES.items()}


class TensorInfo(ctypes.Structure):
    _fields_ = [("id", ctypes.c_int64), ("buffer_id", ctypes.c_int64),
                ("dtype", ctypes.c_int), ("ndims", ctypes.c_int),
                ("shape", ctypes.c_int64 * 4), ("strides", ctypes.c_int64 * 4),
                ("offsets", ctypes.c_int64 * 4), ("padded_shape", ctypes.c_int64 * 4)]


CONFIG_RULE = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_void_p)


def _i64(v):
    if v is None or len(v) == 0:
        return None
    return (ctypes.c_int64 * len(v))(*[int(x) for x in v])


def reset_ids():
    """Restart the process-global tensor / buffer id counters."""
    lib().arkmi_reset_ids()


class Tensor:
    def __init__(self, model, tid):
        self._model = model
        self.id = tid
        info = TensorInfo()
        check(lib().arkmi_model_tensor_info(model._h, ctypes.c_int64(tid), ctypes.byref(info)))
        n = info.ndims
        self.buffer_id = info.buffer_id
        self.dtype = _DT_NAMES[info.dtype]
        self.shape = list(info.shape[:n])
        self.strides = list(info.strides[:n])
        self.offsets = list(info.offsets[:n])
        self.padded_shape = list(info.padded_shape[:n])

    def nelems(self):
        n = 1
        for s in self.shape:
            n *= s
        return n

    def __repr__(self):
        return f"Tensor(id={self.id}, {self.dtype}, shape={self.shape})"


class PlannerContext:
    """`with model.planner_context(sync=False, config={...}):` — ops created
    inside share one planner context (python/ark/planner.py:110-170)."""

    def __init__(self, model, processor_range=None, warp_range=None, sram_range=None,
                 sync=None, config=None):
        self._model = model
        self._kw = dict(processor_range=processor_range, warp_range=warp_range,
                        sram_range=sram_range, sync=sync, config=config)

    def __enter__(self):
        h = self._model._h
        check(lib().arkmi_model_context_enter(h))
        try:
            for member, val in self._kw.items():
                if val is None:
                    continue
                check(lib().arkmi_model_context_call(h, member.encode(), json.dumps(val).encode()))
        except Exception:
            lib().arkmi_model_context_exit(h)
            raise
        return self

    def __exit__(self, *exc):
        check(lib().arkmi_model_context_exit(self._model._h))
        return False

    def call(self, member, value):
        """Invoke a PlannerContext member on this (innermost) context."""
        check(lib().arkmi_model_context_call(self._model._h, member.encode(),
                                             json.dumps(value).encode()))

    def get(self, key):
        out = ctypes.c_char_p()
        check(lib().arkmi_model_context_get(self._model._h, key.encode(), ctypes.byref(out)))
        try:
            return ctypes.string_at(out).decode()
        finally:
            lib().arkmi_free(out)


class Model:
    def __init__(self, rank=0, world_size=1):
        self._h = ctypes.c_void_p()
        check(lib().arkmi_model_create(ctypes.c_int(rank), ctypes.c_int(world_size),
                                       ctypes.byref(self._h)))

    @classmethod
    def from_json(cls, text):
        """A model rebuilt from the text Model.serialize() writes (the reference's model
        file, docs/model_file.md); tensors keep the ids of the file."""
        self = cls.__new__(cls)
        self._h = ctypes.c_void_p()
        check(lib().arkmi_model_from_json(text.encode(), ctypes.byref(self._h)))
        return self

    def tensor_by_id(self, tid):
        return Tensor(self, tid)

    def __del__(self):
        if getattr(self, "_h", None):
            lib().arkmi_model_destroy(self._h)
            self._h = None

    # ---- tensors ------------------------------------------------------------
    def tensor(self, shape, dtype, strides=None, offsets=None, padded_shape=None, rank=-1, name=""):
        out = ctypes.c_int64()
        check(lib().arkmi_model_tensor(self._h, ctypes.c_int(len(shape)), _i64(shape),
                                       ctypes.c_int(DTYPES[dtype]), _i64(strides), _i64(offsets),
                                       _i64(padded_shape), ctypes.c_int(rank), name.encode(),
                                       ctypes.byref(out)))
        return Tensor(self, out.value)

    def _op(self, op, inputs, output=None, name="", **args):
        ins = [t.id for t in inputs if t is not None]
        res = (ctypes.c_int64 * 64)()
        n = ctypes.c_int()
        args = {k: v for k, v in args.items() if v is not None}
        for k, v in args.items():
            # a plan file is JSON, which has no spelling for inf or nan
            if isinstance(v, float) and not math.isfinite(v):
                raise InvalidUsageError(f"op {op}: argument {k} = {v} is not finite")
        check(lib().arkmi_model_op(self._h, op.encode(), _i64(ins), ctypes.c_int(len(ins)),
                                   ctypes.c_int64(output.id if output is not None else -1),
                                   json.dumps(args).encode(), name.encode(), res, ctypes.c_int(64),
                                   ctypes.byref(n)))
        return [Tensor(self, res[i]) for i in range(n.value)]

    def _op1(self, *a, **k):
        return self._op(*a, **k)[0]

    # ---- ops (same names as ark::Model) ---------------------------------------
    def matmul(self, input, other, output=None, trans_input=False, trans_other=False, name=""):
        return self._op1("matmul", [input, other], output, name, trans_input=trans_input,
                         trans_other=trans_other)

    def reduce_sum(self, input, axis, keepdims=True, output=None, name=""):
        return self._op1("reduce_sum", [input], output, name, axis=axis, keepdims=keepdims)

    def reduce_mean(self, input, axis, keepdims=True, output=None, name=""):
        return self._op1("reduce_mean", [input], output, name, axis=axis, keepdims=keepdims)

    def reduce_max(self, input, axis, keepdims=True, output=None, name=""):
        return self._op1("reduce_max", [input], output, name, axis=axis, keepdims=keepdims)

    def softmax(self, input, output=None, name="", mask=None, scale=1.0):
        """Softmax over the last axis; with mask / scale: softmax(input * scale + mask)."""
        if mask is None and scale == 1.0:
            return self._op1("softmax", [input], output, name)
        return self._op1("softmax", [input, mask], output, name, scale=float(scale))

    def layernorm(self, input, eps=1e-6, output=None, name=""):
        return self._op1("layernorm", [input], output, name, eps=eps)

    def rmsnorm(self, input, weight=None, eps=0.0, output=None, name=""):
        return self._op1("rmsnorm", [input, weight], output, name, eps=eps)

    def _arith(self, op, input, other, output, name):
        if isinstance(other, Tensor):
            return self._op1(op, [input, other], output, name)
        return self._op1(op, [input], output, name, value=float(other))

    def add(self, input, other, output=None, name=""):
        return self._arith("add", input, other, output, name)

    def sub(self, input, other, output=None, name=""):
        return self._arith("sub", input, other, output, name)

    def mul(self, input, other, output=None, name=""):
        return self._arith("mul", input, other, output, name)

    def div(self, input, other, output=None, name=""):
        return self._arith("div", input, other, output, name)

    def exp(self, input, output=None, name=""):
        return self._op1("exp", [input], output, name)

    def sqrt(self, input, output=None, name=""):
        return self._op1("sqrt", [input], output, name)

    def rsqrt(self, input, output=None, name=""):
        return self._op1("rsqrt", [input], output, name)

    def relu(self, input, output=None, name=""):
        return self._op1("relu", [input], output, name)

    def gelu(self, input, output=None, name=""):
        return self._op1("gelu", [input], output, name)

    def sigmoid(self, input, output=None, name=""):
        return self._op1("sigmoid", [input], output, name)

    def copy(self, input, output=None, name=""):
        if isinstance(input, Tensor):
            return self._op1("copy", [input], output, name)
        return self._op1("copy", [], output, name, value=float(input))

    def constant(self, value, shape, dtype, name=""):
        return self._op1("constant", [], None, name, value=float(value), shape=list(shape),
                         data_type=dtype.upper())

    def cast(self, input, dtype, output=None, name=""):
        return self._op1("cast", [input], output, name, data_type=dtype.upper())

    def attention(self, q, k, v, scale, causal=False, output=None, name=""):
        """softmax(q k^T * scale [+ causal mask]) v over [batch, seq, heads, head_dim] tensors."""
        return self._op1("attention", [q, k, v], output, name, scale=float(scale), causal=bool(causal))

    def swiglu(self, input, gate, up, output=None, name=""):
        """silu(input @ gate.T) * (input @ up.T), weights stored [hidden, dim], as one op."""
        return self._op1("swiglu", [input, gate, up], output, name)

    def silu_mul(self, input, other, output=None, name=""):
        """silu(input) * other in one pass (SwiGLU gate)."""
        return self._op1("silu_mul", [input, other], output, name)

    def rope(self, input, other, output=None, name=""):
        return self._op1("rope", [input, other], output, name)

    def embedding(self, input, weight, output=None, name=""):
        return self._op1("embedding", [input, weight], output, name)

    def transpose(self, input, permutation, output=None, name=""):
        return self._op1("transpose", [input], output, name, permutation=list(permutation))

    def reshape(self, input, shape, allowzero=False, name=""):
        return self._op1("reshape", [input], None, name, shape=list(shape), allowzero=allowzero)

    def refer(self, input, shape=None, strides=None, offsets=None, padded_shape=None, name=""):
        return self._op1("refer", [input], None, name, shape=shape, strides=strides,
                         offsets=offsets, padded_shape=padded_shape)

    def identity(self, input, deps=(), name=""):
        return self._op1("identity", [input] + list(deps), None, name)

    def sharding(self, input, axis, dim_per_shard, name=""):
        return self._op("sharding", [input], None, name, axis=axis, dim_per_shard=dim_per_shard)

    def noop(self, input, name=""):
        self._op("noop", [input], None, name)

    # ---- graph ------------------------------------------------------------------
    def planner_context(self, **kw):
        return PlannerContext(self, **kw)

    def serialize(self, pretty=True):
        out = ctypes.c_char_p()
        check(lib().arkmi_model_serialize(self._h, ctypes.c_int(int(pretty)), ctypes.byref(out)))
        try:
            return ctypes.string_at(out).decode()
        finally:
            lib().arkmi_free(out)

    def dump(self, compressed=False, with_context=False):
        """Parsed JSON of the model (or of a compressed copy)."""
        out = ctypes.c_char_p()
        check(lib().arkmi_model_dump(self._h, ctypes.c_int(int(compressed)),
                                     ctypes.c_int(int(with_context)), ctypes.c_int(0),
                                     ctypes.byref(out)))
        try:
            return json.loads(ctypes.string_at(out).decode())
        finally:
            lib().arkmi_free(out)

    def compress(self):
        """Compresses in place (drops virtual ops) and returns self."""
        check(lib().arkmi_model_compress(self._h))
        return self

    def verify(self):
        ok = ctypes.c_int()
        check(lib().arkmi_model_verify(self._h, ctypes.byref(ok)))
        return bool(ok.value)

    def plan(self, device_id=0, arch=None, num_processors=0, config_rules=(), pretty=True):
        """Planner(model, device).plan(); with `arch` given, plans for that
        architecture / processor count without touching a GPU."""
        keep = []

        def wrap(rule):
            def cb(op_json, arch_name, _user):
                r = rule(op_json.decode(), arch_name.decode())
                buf = ctypes.create_string_buffer((r or "").encode())
                keep.append(buf)
                return ctypes.addressof(buf)
            return CONFIG_RULE(cb)

        cbs = [wrap(r) for r in config_rules]
        arr = (CONFIG_RULE * len(cbs))(*cbs) if cbs else None
        out = ctypes.c_char_p()
        check(lib().arkmi_model_plan(self._h, ctypes.c_int(device_id),
                                     arch.encode() if arch else None, ctypes.c_int(num_processors),
                                     arr, None, ctypes.c_int(len(cbs)), ctypes.c_int(int(pretty)),
                                     ctypes.byref(out)))
        try:
            return ctypes.string_at(out).decode()
        finally:
            lib().arkmi_free(out)
