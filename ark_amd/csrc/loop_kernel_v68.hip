// Loop-kernel variant: GEMM incl. the split of K.
#include "loop_kernel_impl.h"
namespace arkmi {
ARKMI_LOOP_KERNEL_VARIANT(68)
}
