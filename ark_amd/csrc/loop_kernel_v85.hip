// Loop-kernel variant: rows + GEMM incl. the split of K + attention (a decoder layer whose elementwise ops are all folded into matmul stores).
// Bodies inlined: this variant mixes long-running and small bodies, and with the long ones as
// functions the register allocation of the small ones around the call sites was measured worse.
#define ARKMI_BODY __device__ __forceinline__
#include "loop_kernel_impl.h"
namespace arkmi {
ARKMI_LOOP_KERNEL_VARIANT(85)
}
