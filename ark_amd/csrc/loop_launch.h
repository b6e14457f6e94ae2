// Host-callable entry points of loop_kernel.hip.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace arkmi {

struct LoopProgram;
struct LoopControl;
struct HostMailbox;

constexpr int kLoopMaxThreads = 512;  // 8 waves: one resident slot per CU

// The loop kernel is compiled in several variants, each carrying a subset of
// the op families (OpFamily bits).  Returns the smallest compiled variant that
// covers `families`; *chosen receives its family set.
const void *loop_kernel_select(int families, int *chosen);
// The one-task-group kernel of the smallest variant that covers `families`,
// and its launch (one kernel per op, for the separate-kernel comparison).
const void *step_kernel_select(int families);
void step_kernel_launch(const void *kernel, const LoopProgram &prog, LoopControl *ctl, HostMailbox *mb_dev,
                        int group, int grid, int threads, int lds_bytes, uint64_t wait_ticks, hipStream_t stream);
void loop_kernel_prepare(const void *kernel, int lds_bytes);
int loop_kernel_max_blocks_per_cu(const void *kernel, int threads, int lds_bytes);
int loop_kernel_lds_reserved();
void loop_kernel_launch(const void *kernel, const LoopProgram &prog, LoopControl *ctl,
                        HostMailbox *mb_dev, int grid, int threads, int lds_bytes,
                        int one_shot_iters, uint64_t idle_ticks, uint64_t wait_ticks,
                        hipStream_t stream);

}  // namespace arkmi
