"""`ark.error.<Class>`: the error classes under the module name the reference's tests use
(python/ark/error.py:4-22)."""
from .._lib import (BaseError, InternalError, InvalidUsageError, ModelError, PlanError,  # noqa: F401
                    UnsupportedError, SystemError, GpuError)

__all__ = ["BaseError", "InternalError", "InvalidUsageError", "ModelError", "PlanError",
           "UnsupportedError", "SystemError", "GpuError"]
