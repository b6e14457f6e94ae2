// Loop-kernel variant: elementwise + GEMM incl. the split of K.
#include "loop_kernel_impl.h"
namespace arkmi {
ARKMI_LOOP_KERNEL_VARIANT(70)
ARKMI_STEP_KERNEL_VARIANT(70)
}
