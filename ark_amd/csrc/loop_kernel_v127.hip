// Loop-kernel variant: every op family.
#include "loop_kernel_impl.h"
namespace arkmi {
ARKMI_LOOP_KERNEL_VARIANT(127)
}
