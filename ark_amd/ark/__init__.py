"""`import ark_amd.ark as ark` — the reference's Python frontend, name for name.

Module-level op functions over one global model, `Runtime` with its three-state
life cycle, `Module` with state dicts, `Tensor.from_numpy/to_numpy`, `Planner` /
`Plan` / `PlannerContext`, the data type tags and the error classes
(python/ark/__init__.py:9-39 lists the surface).  Everything below the function
signatures is the C ABI of libarkmi.so; nothing here computes.
"""
from .._lib import lib as _lib
from .._lib import (BaseError, InternalError, InvalidUsageError, ModelError, PlanError,  # noqa: F401
                    UnsupportedError, SystemError, GpuError)
from . import error  # noqa: F401
from .frontend import *  # noqa: F401,F403
from .frontend import Model, core  # noqa: F401
from .session import *  # noqa: F401,F403


def version():
    """Version string of the native library."""
    return _lib().arkmi_version().decode()


__version__ = None


def set_rank(rank):
    Model.set_rank(rank)


def set_world_size(world_size):
    Model.set_world_size(world_size)
