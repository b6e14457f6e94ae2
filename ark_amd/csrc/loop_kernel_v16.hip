// Loop-kernel variant: attention.
// Bodies inlined: a function that needs most vector registers saves and restores over a hundred
// of them per call (~8 us), too much beside a body that runs for 20-100 us.
#define ARKMI_BODY __device__ __forceinline__
#include "loop_kernel_impl.h"
namespace arkmi {
ARKMI_LOOP_KERNEL_VARIANT(16)
ARKMI_STEP_KERNEL_VARIANT(16)
}
