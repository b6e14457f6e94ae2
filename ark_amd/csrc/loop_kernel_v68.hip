// Loop-kernel variant: GEMM incl. the split of K.
#define ARKMI_BODY __device__ __forceinline__
#include "loop_kernel_impl.h"
namespace arkmi {
ARKMI_LOOP_KERNEL_VARIANT(68)
}
