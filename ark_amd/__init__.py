"""ark_amd — MI355X (gfx950) execution backend for the ARK model API.

The product is the native library `libarkmi.so` (HIP kernels, host runtime and
the C ABI declared in include/arkmi.h).  This package is the thin Python host
side over that ABI; PyTorch is used only for device memory and streams.
"""
from ._lib import lib, check, ArkmiError, DTYPES, device_info  # noqa: F401
from . import ops  # noqa: F401
from .model import Model, Tensor, PlannerContext, reset_ids  # noqa: F401
from .executor import Executor, plan_schedule, plan_analysis, schedule_tasks  # noqa: F401


def init():
    """ark::init(): read the ARK_* environment variables again."""
    check(lib().arkmi_init())
