// Data structures of the persistent loop kernel: the device "program" a plan
// compiles to, the grid-barrier state and the host mailbox.
//
// The reference generates CUDA/HIP source per plan and JIT-compiles it
// (ark/codegen.cpp:79-180, ark/include/kernels/kernel_template.in).  Here the
// plan compiles to tables interpreted by one ahead-of-time compiled kernel:
//   steps[]  : the body, in plan order — grid barriers over processor ranges
//              and task groups (one per task_seq<> of the reference);
//   groups[] : the task_seq<> parameters, bit for bit;
//   ops[]    : descriptors of the op bodies a task runs, with absolute device
//              addresses (the reference bakes arena offsets in as literals).
#pragma once
#include <stdint.h>

#include "ewise.h"
#include "gemm.h"
#include "gemm_f32.h"
#include "attn.h"
#include "gemv.h"
#include "row_ops.h"

namespace arkmi {

enum DevOpKind : int32_t { DEV_NOOP = 0, DEV_ROW = 1, DEV_GEMM = 2, DEV_EWISE = 3, DEV_GEMV = 4, DEV_ATTN = 5, DEV_EMBED = 6 };

// Op families as a bit set: which bodies a loop-kernel variant carries, and
// which a compiled plan needs.
// FAM_EXT holds the bodies few plans use (fp32 and transposed-first-operand matmuls,
// reductions over an axis other than the last, the embedding gather): kept out of the common variants, whose
// register allocation and code size every other body shares.
// FAM_SPLITK adds the matmul body that splits K in two (256x256 tiles only) to a variant
// that carries FAM_GEMM.
enum OpFamily : int32_t { FAM_ROW = 1, FAM_EWISE = 2, FAM_GEMM = 4, FAM_GEMV = 8, FAM_ATTN = 16, FAM_EXT = 32,
                          FAM_SPLITK = 64, FAM_ALL = 127 };

struct DevOp {
    int32_t kind;
    int32_t gemm_tile_m, gemm_tile_n;  // DEV_GEMM: which compiled tile body
    int32_t pad_;
    union {
        RowOpDesc row;
        GemmDesc gemm;
        GemvDesc gemv;
        AttnDesc attn;
        EwiseDesc ew;
        EmbedDesc emb;
    };
};

// Parameters of one task_seq<> (kernel_template.in:6-29).
struct DevTaskGroup {
    int32_t proc_b, proc_e, proc_s, proc_cur;
    int32_t task_b, task_e, task_s, gran;
    int32_t n_slots, slot_warps, slot_sram;
    int32_t op_begin, op_count;
    int32_t trace_offset;  // first trace record of this group, -1 if not traced
    // Dependency counters (the fields are dead when LoopProgram::dep_counters is null).
    // As a consumer: before task index i runs, the counters [lo, hi] of each of the group's
    // n_waits producers must have reached expect * iteration; (lo, hi) of wait w are the words
    // wait_spans[span_begin + 2 * (i * n_waits + w)] and the next one.
    int32_t n_waits, wait_begin, span_begin;
    // As a producer: task index i completes row block signal_map[signal_begin + i] and adds one
    // to counter signal_base + that block; signal_begin < 0: the group signals nothing.
    int32_t signal_begin, signal_base;
    // A group of skinny-matmul tasks runs from tables the host lays out in LoopProgram::gemv_seq
    // (stretches of units, GemvSeqEntry).  The one-op kernels run the group by itself: workgroup
    // b's stretches are the entries from seq_begin + b * seq_stride up to the first one with
    // op < 0.  The loop kernel streams runs of groups that follow one another with nothing to wait
    // for in between as one sequence (the next matmul's weights are on their way while the current
    // one adds up its tiles): chain = n > 1 on the first group of such a run (the groups gi ..
    // gi + n - 1), -1 on the others, which the loop kernel skips, 0 on a group by itself.  The
    // sequence of the run (or of the group by itself) is
    //   claim < 0:  per workgroup, the entries from run_begin + b * run_stride as above;
    //   claim >= 0: the run_stride entries from run_begin on, shared: workgroup b takes entries
    //               b and b + grid and claims further ones from claim counter `claim` as it gets
    //               free (LoopProgram::gemv_claims).
    int32_t chain;
    int32_t seq_begin, seq_stride;
    int32_t run_begin, run_stride;
    int32_t claim;
};

// One producer a task group waits for.
struct DevWait {
    int32_t counter_base;  // first counter of the producer's row blocks
    int32_t expect;        // tasks per row block, i.e. what one iteration adds to each counter
};

constexpr int kDepStride = 16;  // words between two dependency counters: one per 64-byte line

// STEP_LOCAL_SYNC: the next group depends only on what this workgroup itself wrote
enum DevStepKind : int32_t { STEP_BARRIER = 0, STEP_TASKS = 1, STEP_LOCAL_SYNC = 2 };

struct DevStep {
    int32_t kind;
    // STEP_BARRIER: blocks b, b+s, ... < e synchronise on barrier `index`
    // STEP_TASKS:   `index` names the task group
    int32_t index;
    int32_t b, e, s;
    int32_t count;  // number of blocks in the barrier
    int32_t pad_[2];
};

struct GridBarrier {
    unsigned int count;
    unsigned int generation;
    unsigned int pad_[14];  // one barrier per 64-byte line
};

constexpr int kMaxBarriers = 64;
constexpr int kMaxXcds = 16;

// Device-resident control block, zeroed before every launch.
struct LoopControl {
    int32_t iter;    // command broadcast to all blocks
    int32_t abort;   // set when a bounded wait expired; every spin loop exits on it
    int32_t pad_[14];
    GridBarrier all;  // flat barrier over every block of the grid (set-up only)
    GridBarrier bars[kMaxBarriers];
    // Two-level barrier over every block of the grid: one counter per XCD, and
    // one on top that the XCDs' last arrivers meet on.
    GridBarrier xcd[kMaxXcds];
    GridBarrier top;
    unsigned int xcd_blocks[kMaxXcds];  // workgroups resident on each XCD, counted at kernel start
};

// One record per executed task when tracing is on.
struct TraceRecord {
    int32_t block, slot, order;
};

struct LoopProgram {
    const DevStep *steps;
    const DevTaskGroup *groups;
    const DevOp *ops;
    TraceRecord *trace;  // null unless tracing
    // null unless tracing: per block, the wall-clock ticks at which it entered
    // each step of the last iteration, plus one entry for the end of the body
    // ([num_blocks][num_steps + 1])
    unsigned long long *step_clock;
    // Dependency counters in place of some grid barriers; all four null when the plan has none
    // (and in the one-op kernels, where kernel boundaries order everything).  The counters are
    // zeroed before every launch and only grow.
    const DevWait *waits;
    const int32_t *wait_spans;
    const int32_t *signal_map;
    unsigned int *dep_counters;
    const GemvSeqEntry *gemv_seq;  // the sequences of the skinny matmuls, null if there are none
    // Claim counters of the skinny matmuls whose stretches are claimed at run time: two words per
    // counter, kDepStride apart, used by alternating iterations (the one not in use is zeroed
    // during the other's iteration; a grid barrier separates iterations).  Zero at every launch.
    unsigned int *gemv_claims;
    int32_t num_steps;
    int32_t num_blocks;
    // what separates two iterations of the body inside one command:
    // 2 a grid barrier, 1 a workgroup-local sync, 0 nothing
    int32_t iter_sync;
    int32_t pad_;
};

struct HostMailbox;

// The one kernel parameter of the loop kernel and of the one-op kernels.  The kernels read it
// through the kernel-argument segment whenever a field is needed instead of keeping the fields
// in registers across the op bodies.
struct LoopArgs {
    LoopProgram prog;
    LoopControl *ctl;
    HostMailbox *mb;
    uint64_t idle_ticks, wait_ticks;
    int32_t one_shot_iters;  // loop kernel: > 0 runs that many iterations and returns
    int32_t group;           // one-op kernel: the task group to run; loop kernel: -1
};

// Mapped, pinned host memory shared with the kernel.
struct HostMailbox {
    volatile int32_t cmd;     // host -> device: 0 idle, n > 0 run n iterations, < 0 exit
    volatile int32_t alive;   // device -> host: 1 while the loop kernel is resident
    volatile int32_t status;  // 0 ok, 1 left after the idle limit, 2 a bounded wait expired
    volatile int32_t done;    // iterations completed since launch (diagnostic)
};

// LDS ahead of the slots' windows: control words of the loop itself (barrier
// verdicts).
constexpr int kLdsControl = 128;
constexpr int kLdsReserved = 256;

enum MailboxStatus : int32_t { MB_OK = 0, MB_IDLE_EXIT = 1, MB_ABORTED = 2 };

}  // namespace arkmi
