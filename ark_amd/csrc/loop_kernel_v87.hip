// Loop-kernel variant: rows + elementwise + GEMM incl. the split of K + attention (a decoder layer).
#include "loop_kernel_impl.h"
namespace arkmi {
ARKMI_LOOP_KERNEL_VARIANT(87)
}
