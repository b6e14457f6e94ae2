"""Data types, tensors, the global model and the op functions of the `ark` surface.

Follows python/ark/data_type.py, tensor.py, model.py and ops.py in names, argument order and
error behaviour.  Two ops differ in how they are built, not in what they mean: `softmax` and
`layernorm` emit one fused row op each (the reference composes them from reduce / arithmetic
ops, python/ark/ops.py:491-513), because the fused bodies read every row once.
"""
import types

import numpy as np

from .. import model as _m
from .._lib import DTYPES, InvalidUsageError

__all__ = ["DataType", "fp32", "fp16", "bf16", "int32", "uint32", "int8", "uint8", "byte",
           "Dims", "Tensor", "Parameter", "NullTensor", "Model",
           "tensor", "parameter", "add", "sub", "mul", "div", "cast", "constant", "copy",
           "embedding", "exp", "gelu", "identity", "matmul", "noop", "reduce_max", "reduce_mean",
           "reduce_sum", "relu", "reshape", "rope", "rsqrt", "sharding", "sigmoid", "sqrt",
           "transpose", "mean", "ones", "zeros", "softmax", "layernorm", "rmsnorm", "attention",
           "swiglu", "silu_mul", "refer"]


# ---- data types ---------------------------------------------------------------------------------
class _CoreDataType:
    """The tag `DataType.ctype()` returns (`ark.core.FP32` ...): name, C ABI code, byte size."""

    def __init__(self, name, size):
        self._name, self._size = name, size
        self.code = DTYPES[name.lower()]

    def name(self):
        return self._name

    def bytes(self):
        return self._size

    def __repr__(self):
        return f"core.{self._name}"


_NUMPY = {"fp32": np.float32, "fp16": np.float16, "bf16": None, "int32": np.int32,
          "uint32": np.uint32, "int8": np.int8, "uint8": np.uint8, "byte": np.uint8}
_SIZES = {"fp32": 4, "fp16": 2, "bf16": 2, "int32": 4, "uint32": 4, "int8": 1, "uint8": 1, "byte": 1}
core = types.SimpleNamespace(CoreDataType=_CoreDataType,
                             **{n.upper(): _CoreDataType(n.upper(), s) for n, s in _SIZES.items()})


class DataType:
    """Base of the type tags; the tags are classes used without instantiation (`ark.fp16`)."""
    _name = None

    @staticmethod
    def from_numpy(np_type):
        if not isinstance(np_type, np.dtype):
            raise InvalidUsageError(f"Expected a numpy data type, but got {type(np_type)}")
        for name, t in _NUMPY.items():
            if t is not None and name != "byte" and np.dtype(t) == np_type:
                return _TAGS[name]
        raise InvalidUsageError(f"Undefined conversion from numpy data type {np_type} to ark data type.")

    @staticmethod
    def from_name(type_name):
        try:
            return _TAGS[type_name]
        except (KeyError, TypeError):
            raise InvalidUsageError(f"Undefined data type {type_name}") from None

    @staticmethod
    def from_ctype(ctype):
        if not isinstance(ctype, _CoreDataType):
            raise InvalidUsageError(f"Expected a core data type, but got {type(ctype)}")
        return DataType.from_name(ctype.name().lower())

    @classmethod
    def to_numpy(cls):
        """numpy type of the storage; bf16 has none in numpy and travels as uint16 bit patterns."""
        return np.uint16 if cls._name == "bf16" else _NUMPY[cls._name]

    @classmethod
    def ctype(cls):
        return getattr(core, cls._name.upper())

    @classmethod
    def element_size(cls):
        return _SIZES[cls._name]


def _tag(name):
    return type(name, (DataType,), {"_name": name, "__doc__": f"{name} element type"})


fp32, fp16, bf16, int32 = _tag("fp32"), _tag("fp16"), _tag("bf16"), _tag("int32")
uint32, int8, uint8, byte = _tag("uint32"), _tag("int8"), _tag("uint8"), _tag("byte")
_TAGS = {t._name: t for t in (fp32, fp16, bf16, int32, uint32, int8, uint8, byte)}


# ---- tensors -------------------------------------------------------------------------------------
class Dims(list):
    """Up to four extents (ark::Dims)."""

    def __init__(self, *dims):
        if len(dims) == 1 and isinstance(dims[0], (list, tuple)):
            dims = dims[0]
        if len(dims) > 4:
            raise InvalidUsageError("Only support tensors with up to 4 dimensions")
        super().__init__(int(d) for d in dims)

    def vector(self):
        return list(self)

    def ndims(self):
        return len(self)

    def nelems(self):
        n = 1
        for d in self:
            n *= d
        return n


NullTensor = None


class Tensor:
    """Handle of a model tensor; data moves only once the runtime is launched
    (python/ark/tensor.py:15-92)."""

    def __init__(self, _tensor):
        self._tensor = _tensor

    def shape(self):
        return list(self._tensor.shape)

    def strides(self):
        return list(self._tensor.strides)

    def nelems(self):
        return self._tensor.nelems()

    def dtype(self):
        return _TAGS[self._tensor.dtype]

    def to_numpy(self, ndarray=None, stream=0):
        from .session import Runtime
        np_type = self.dtype().to_numpy()
        rt = Runtime.get_runtime()
        if not rt.launched():
            return np.ndarray(self.shape(), dtype=np_type, buffer=None)
        if ndarray is None:
            ndarray = np.zeros(self.shape(), dtype=np_type)
        elif not ndarray.flags["C_CONTIGUOUS"]:
            raise ValueError("ndarray is not contiguous in memory")
        elif list(ndarray.shape) != self.shape():
            raise ValueError("ndarray shape does not match the tensor")
        elif ndarray.dtype != np_type:
            raise ValueError("ndarray dtype does not match the tensor")
        rt.executor.tensor_read(self, ndarray, stream)
        return ndarray

    def from_numpy(self, ndarray, stream=0):
        from .session import Runtime
        rt = Runtime.get_runtime()
        if not rt.launched():
            raise RuntimeError("Tensor is not allocated yet. `Tensor.from_numpy()` is "
                               "usable only after you call `Runtime.launch()`.")
        ndarray = np.ascontiguousarray(ndarray.astype(self.dtype().to_numpy(), copy=False))
        if ndarray.nbytes != self.nelems() * self.dtype().element_size():
            raise ValueError("ndarray size does not match the tensor")
        rt.executor.tensor_write(self, ndarray, stream)
        return self

    def __repr__(self):
        return f"ark.Tensor({self._tensor.dtype}, shape={self.shape()})"


class Parameter(Tensor):
    """A tensor a Module lists in its state dict."""


# ---- the global model ---------------------------------------------------------------------------
class _ModelState:
    model = None
    rank = 0
    world_size = 1


class Model(_m.Model):
    """The one model the op functions append to (python/ark/model.py:13-74)."""

    @staticmethod
    def get_model():
        if _ModelState.model is None:
            _ModelState.model = Model(_ModelState.rank, _ModelState.world_size)
        return _ModelState.model

    @staticmethod
    def get_rank():
        return _ModelState.rank

    @staticmethod
    def get_world_size():
        return _ModelState.world_size

    @staticmethod
    def set_rank(rank):
        _ModelState.rank = rank

    @staticmethod
    def set_world_size(world_size):
        _ModelState.world_size = world_size

    @staticmethod
    def reset():
        _ModelState.model = None
        _ModelState.rank = 0
        _ModelState.world_size = 1


# ---- ops -------------------------------------------------------------------------------------------
def _seq(v, what):
    if not isinstance(v, (list, tuple)):
        raise InvalidUsageError(f"{what} should be a list or tuple of integers")
    if len(v) > 4:
        raise InvalidUsageError("Only support tensors with up to 4 dimensions")
    return list(v)


def _raw(t):
    return t._tensor if t is not None else None


def _g():
    return Model.get_model()


def _new(cls, shape, dtype, strides, offsets, padded_shape, rank, name):
    shape = _seq(shape, "shape")
    strides, offsets = _seq(strides, "strides"), _seq(offsets, "offsets")
    padded_shape = _seq(padded_shape, "padded_shape")
    return cls(_g().tensor(shape, dtype._name, strides or None, offsets or None,
                           padded_shape or None, rank, name))


def tensor(shape, dtype=fp32, strides=(), offsets=(), padded_shape=(), rank=-1, name=""):
    return _new(Tensor, shape, dtype, strides, offsets, padded_shape, rank, name)


def parameter(shape, dtype=fp32, strides=(), offsets=(), padded_shape=(), name=""):
    return _new(Parameter, shape, dtype, strides, offsets, padded_shape, -1, name)


def _binary(op, pyop, commutes):
    def f(input, other, output=NullTensor, name=op):
        ti, to = isinstance(input, Tensor), isinstance(other, Tensor)
        if not ti and not to:
            # two numbers: plain arithmetic, or a constant fill of `output`
            # (python/ark/ops.py:96-120)
            v = pyop(input, other)
            if output is NullTensor:
                return v
            return Tensor(_g().copy(v, _raw(output), name))
        if not ti:
            if not commutes:
                raise InvalidUsageError(f"{op}: the first operand must be a tensor")
            input, other = other, input
        rhs = other._tensor if isinstance(other, Tensor) else other
        return Tensor(getattr(_g(), op)(input._tensor, rhs, _raw(output), name))
    f.__name__ = op
    return f


add = _binary("add", lambda a, b: a + b, True)
sub = _binary("sub", lambda a, b: a - b, False)
mul = _binary("mul", lambda a, b: a * b, True)
div = _binary("div", lambda a, b: a / b, False)


def _unary(op):
    def f(input, output=NullTensor, name=op):
        return Tensor(getattr(_g(), op)(input._tensor, _raw(output), name))
    f.__name__ = op
    return f


exp, gelu, relu, rsqrt, sigmoid, sqrt = (_unary(n) for n in
                                         ("exp", "gelu", "relu", "rsqrt", "sigmoid", "sqrt"))


def cast(input, dtype, output=NullTensor, name="cast"):
    return Tensor(_g().cast(input._tensor, dtype._name, _raw(output), name))


def constant(value, shape, dtype=fp32, name="constant"):
    return Tensor(_g().constant(value, _seq(shape, "shape"), dtype._name, name))


def ones(shape, dtype=fp32, name="ones"):
    return constant(1, shape, dtype, name)


def zeros(shape, dtype=fp32, name="zeros"):
    return constant(0, shape, dtype, name)


def copy(input, output=NullTensor, name="copy"):
    return Tensor(_g().copy(input._tensor if isinstance(input, Tensor) else input, _raw(output), name))


def embedding(input, weight, output=NullTensor, name="embedding"):
    return Tensor(_g().embedding(input._tensor, weight._tensor, _raw(output), name))


def identity(input, deps=(), name="identity"):
    for d in deps:
        if not isinstance(d, Tensor):
            raise InvalidUsageError("All dependencies should be a tensor")
    return Tensor(_g().identity(input._tensor, [d._tensor for d in deps], name))


def matmul(input, other, output=NullTensor, transpose_input=False, transpose_other=False,
           name="matmul"):
    return Tensor(_g().matmul(input._tensor, other._tensor, _raw(output), transpose_input,
                              transpose_other, name))


def noop(input, name="noop"):
    _g().noop(input._tensor, name)


def _reduce(op):
    def f(input, axis, keepdims=True, output=NullTensor, name=op):
        return Tensor(getattr(_g(), op)(input._tensor, axis, keepdims, _raw(output), name))
    f.__name__ = op
    return f


reduce_max, reduce_mean, reduce_sum = _reduce("reduce_max"), _reduce("reduce_mean"), _reduce("reduce_sum")


def mean(input, axis, keepdims=True, output=NullTensor, name="mean"):
    return reduce_mean(input, axis, keepdims, output, name)


def reshape(input, shape, allowzero=False, name="reshape"):
    return Tensor(_g().reshape(input._tensor, _seq(shape, "shape"), allowzero, name))


def refer(input, shape=None, strides=None, offsets=None, padded_shape=None, name="refer"):
    return Tensor(_g().refer(input._tensor, shape, strides, offsets, padded_shape, name))


def rope(input, other, output=NullTensor, name="rope"):
    return Tensor(_g().rope(input._tensor, other._tensor, _raw(output), name))


def sharding(input, axis, dim_per_shard, name="sharding"):
    return [Tensor(t) for t in _g().sharding(input._tensor, axis, dim_per_shard, name)]


def transpose(input, perm, output=NullTensor, name="transpose"):
    if not isinstance(perm, (list, tuple)):
        raise InvalidUsageError("perm should be a list or tuple of integers")
    if len(perm) > 4:
        raise InvalidUsageError("Only support perm up to 4 dimensions")
    return Tensor(_g().transpose(input._tensor, list(perm), _raw(output), name))


def softmax(input, output=NullTensor, name="softmax"):
    return Tensor(_g().softmax(input._tensor, _raw(output), name))


def layernorm(input, eps=1e-6, output=NullTensor, name="layernorm"):
    return Tensor(_g().layernorm(input._tensor, eps, _raw(output), name))


# fused ops this backend adds to the model API
def rmsnorm(input, weight=NullTensor, eps=0.0, output=NullTensor, name="rmsnorm"):
    return Tensor(_g().rmsnorm(input._tensor, _raw(weight), eps, _raw(output), name))


def attention(q, k, v, scale, causal=False, output=NullTensor, name="attention"):
    return Tensor(_g().attention(q._tensor, k._tensor, v._tensor, scale, causal, _raw(output), name))


def swiglu(input, gate, up, output=NullTensor, name="swiglu"):
    return Tensor(_g().swiglu(input._tensor, gate._tensor, up._tensor, _raw(output), name))


def silu_mul(input, other, output=NullTensor, name="silu_mul"):
    return Tensor(_g().silu_mul(input._tensor, other._tensor, _raw(output), name))
