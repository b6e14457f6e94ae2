// Loop-kernel variant: GEMM.
#define ARKMI_BODY __device__ __forceinline__
#include "loop_kernel_impl.h"
namespace arkmi {
ARKMI_LOOP_KERNEL_VARIANT(4)
ARKMI_STEP_KERNEL_VARIANT(4)
}
