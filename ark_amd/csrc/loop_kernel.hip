// Host side of the persistent loop kernel: the table of compiled variants and
// the launch helpers (called from executor.hip).  The kernel itself is the
// template in loop_kernel_impl.h; loop_kernel_v*.hip instantiate it.
#include "host_common.h"
#include "kernels/loop.h"
#include "loop_launch.h"

namespace arkmi {

const void *loop_kernel_variant_1();   // rows
const void *loop_kernel_variant_2();   // elementwise
const void *loop_kernel_variant_3();   // rows + elementwise
const void *loop_kernel_variant_4();   // GEMM
const void *loop_kernel_variant_6();   // elementwise + GEMM
const void *loop_kernel_variant_7();   // rows + elementwise + GEMM
const void *loop_kernel_variant_8();   // skinny matmul (GEMV)
const void *loop_kernel_variant_11();  // rows + elementwise + GEMV
const void *loop_kernel_variant_16();  // attention
const void *loop_kernel_variant_23();  // rows + elementwise + GEMM + attention
const void *loop_kernel_variant_31();  // every common family
const void *loop_kernel_variant_32();  // the rarely used bodies alone
const void *loop_kernel_variant_63();  // everything but the split of K
const void *loop_kernel_variant_68();  // GEMM incl. the split of K
const void *loop_kernel_variant_70();  // elementwise + GEMM incl. the split of K
const void *loop_kernel_variant_85();  // rows + GEMM incl. the split of K + attention (elementwise ops all folded)
const void *loop_kernel_variant_87();  // rows + elementwise + GEMM incl. the split of K + attention
const void *loop_kernel_variant_127(); // everything

const void *step_kernel_variant_1();
const void *step_kernel_variant_2();
const void *step_kernel_variant_3();
const void *step_kernel_variant_4();
const void *step_kernel_variant_6();
const void *step_kernel_variant_8();
const void *step_kernel_variant_16();
const void *step_kernel_variant_32();
const void *step_kernel_variant_70();

const void *step_kernel_select(int families) {
    struct Variant { int fam; const void *(*get)(); };
    static const Variant table[] = {
        {1, step_kernel_variant_1}, {2, step_kernel_variant_2}, {8, step_kernel_variant_8}, {16, step_kernel_variant_16},
        {32, step_kernel_variant_32},
        {3, step_kernel_variant_3}, {4, step_kernel_variant_4}, {6, step_kernel_variant_6},
        {70, step_kernel_variant_70},
    };
    for (const Variant &v : table)
        if ((families & ~v.fam) == 0) return v.get();
    ARKMI_FAIL(ARKMI_UNSUPPORTED, "no one-op kernel holds the op families ", families, " of a fused task");
}

void step_kernel_launch(const void *kernel, const LoopProgram &prog, LoopControl *ctl, HostMailbox *mb_dev,
                        int group, int grid, int threads, int lds_bytes, uint64_t wait_ticks, hipStream_t stream) {
    LoopArgs a{};
    a.prog = prog;
    // a body's bounded wait (the split of K) needs the abort word and the limit here too
    a.ctl = ctl; a.mb = mb_dev;
    a.wait_ticks = wait_ticks;
    // kernel boundaries order the ops: no dependency counters
    a.prog.waits = nullptr; a.prog.wait_spans = nullptr; a.prog.signal_map = nullptr; a.prog.dep_counters = nullptr;
    a.group = group;
    void *args[] = {&a};
    ARKMI_HIP(hipLaunchKernel(kernel, dim3(grid), dim3(threads), args, (size_t)lds_bytes, stream));
}

const void *loop_kernel_select(int families, int *chosen) {
    // cheapest first: the register need of a variant is that of its largest body
    struct Variant { int fam; const void *(*get)(); };
    static const Variant table[] = {
        {1, loop_kernel_variant_1},   {2, loop_kernel_variant_2},   {8, loop_kernel_variant_8},
        {16, loop_kernel_variant_16}, {32, loop_kernel_variant_32},
        {3, loop_kernel_variant_3},   {11, loop_kernel_variant_11}, {4, loop_kernel_variant_4},
        {6, loop_kernel_variant_6},   {7, loop_kernel_variant_7},   {23, loop_kernel_variant_23},
        {31, loop_kernel_variant_31}, {63, loop_kernel_variant_63},
        {68, loop_kernel_variant_68}, {70, loop_kernel_variant_70}, {85, loop_kernel_variant_85},
        {87, loop_kernel_variant_87},
        {127, loop_kernel_variant_127},
    };
    for (const Variant &v : table) {
        if ((families & ~v.fam) == 0) {
            if (chosen) *chosen = v.fam;
            return v.get();
        }
    }
    if (chosen) *chosen = FAM_ALL;
    return loop_kernel_variant_127();
}

void loop_kernel_prepare(const void *kernel, int lds_bytes) {
    ARKMI_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes));
}

int loop_kernel_max_blocks_per_cu(const void *kernel, int threads, int lds_bytes) {
    int n = 0;
    ARKMI_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, threads, (size_t)lds_bytes));
    return n;
}

void loop_kernel_launch(const void *kernel, const LoopProgram &prog, LoopControl *ctl,
                        HostMailbox *mb_dev, int grid, int threads, int lds_bytes,
                        int one_shot_iters, uint64_t idle_ticks, uint64_t wait_ticks,
                        hipStream_t stream) {
    LoopArgs a{};
    a.prog = prog;
    a.ctl = ctl; a.mb = mb_dev;
    a.idle_ticks = idle_ticks; a.wait_ticks = wait_ticks;
    a.one_shot_iters = one_shot_iters;
    a.group = -1;  // all of them
    void *args[] = {&a};
    ARKMI_HIP(hipLaunchKernel(kernel, dim3(grid), dim3(threads), args, (size_t)lds_bytes, stream));
}

int loop_kernel_lds_reserved() { return kLdsReserved; }

}  // namespace arkmi
