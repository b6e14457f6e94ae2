// The persistent loop kernel, as a template over the op families it can run:
// one workgroup per CU interprets the compiled
// plan (kernels/loop.h), polling a mapped host mailbox for "run N iterations"
// commands.  Counterpart of ark/include/kernels/kernel_template.in:6-78 and
// ark/include/kernels/common/sync.h:36-66.
//
// Every wait in here is bounded: the command poll ends after an idle limit
// (the host relaunches on the next run), and a grid barrier that does not
// complete within its limit raises `abort`, which every spin loop observes, so
// the grid always drains.
#pragma once
#include "host_common.h"
#include "kernels/loop.h"
#include "loop_launch.h"

namespace arkmi {

extern __shared__ __attribute__((aligned(16))) char g_loop_lds[];

#define AGENT __HIP_MEMORY_SCOPE_AGENT
#define SYSTEM __HIP_MEMORY_SCOPE_SYSTEM

__device__ __forceinline__ bool in_range(int x, int b, int e, int s) {
    return x >= b && x < e && ((x - b) % s) == 0;
}

// Sense-free counting barrier over `nblocks` workgroups.  Agent-scope release /
// acquire fences order the blocks' global writes across the XCDs' L2s.
// Returns false (uniformly per block) once `abort` has been raised.
__device__ __forceinline__ bool grid_barrier(GridBarrier *bar, unsigned nblocks, LoopControl *ctl,
                             uint64_t limit_ticks) {
    int *lds_flag = reinterpret_cast<int *>(g_loop_lds);
    // every wave's stores are acknowledged by the L2 before thread 0 writes the L2 back
    drain_stores_then_barrier();
    if (threadIdx.x == 0) {
        int ok = 1;
        if (nblocks > 1) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
            unsigned gen = __hip_atomic_load(&bar->generation, __ATOMIC_RELAXED, AGENT);
            // release: the generation must be read before this arrival is counted,
            // or a wake-up between the two could be missed
            unsigned prev = __hip_atomic_fetch_add(&bar->count, 1u, __ATOMIC_ACQ_REL, AGENT);
            if (prev == nblocks - 1) {
                __hip_atomic_store(&bar->count, 0u, __ATOMIC_RELAXED, AGENT);
                // release: the reset of `count` is visible before anyone is woken
                __hip_atomic_fetch_add(&bar->generation, 1u, __ATOMIC_RELEASE, AGENT);
            } else {
                const uint64_t t0 = wall_clock64();
                unsigned polls = 0;
                // relaxed polls: an acquire load would invalidate this XCD's L2 on
                // every poll and slow the workgroups that are still computing;
                // the fences around the loop carry the ordering
                while (__hip_atomic_load(&bar->generation, __ATOMIC_RELAXED, AGENT) == gen) {
                    __builtin_amdgcn_s_sleep(4);
                    if ((++polls & 63u) == 0) {
                        if (__hip_atomic_load(&ctl->abort, __ATOMIC_RELAXED, AGENT)) break;
                        if (wall_clock64() - t0 > limit_ticks) {
                            __hip_atomic_store(&ctl->abort, 1, __ATOMIC_RELAXED, AGENT);
                            break;
                        }
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        }
        if (__hip_atomic_load(&ctl->abort, __ATOMIC_RELAXED, AGENT)) ok = 0;
        *lds_flag = ok;
    }
    __syncthreads();
    const bool ok = (*lds_flag != 0);
    return ok;
}

// Where this workgroup runs: its XCD and how many of the grid's workgroups share
// it.  The XCDs' L2 caches are not coherent with each other, so a barrier that
// orders global memory has to write back and invalidate them.  Each such cache
// operation walks the whole L2 and the requests of one XCD's 32 workgroups are
// served one after another: a flat barrier in which every workgroup fences costs
// about 20 us.  The two-level barrier below writes each L2 back once (by the
// XCD's last arriver, after every workgroup of the XCD has seen its stores
// acknowledged by that L2) and costs 5-6 us.
struct XcdInfo {
    unsigned x;     // XCC_ID of this workgroup
    unsigned nx;    // workgroups of the grid on this XCD
    unsigned nxcd;  // XCDs that hold at least one workgroup
    unsigned epoch; // full-grid barriers passed since the launch
};

__device__ __forceinline__ unsigned xcc_id() {
    // s_getreg_b32 hwreg(HW_REG_XCC_ID, 0, 4)
    return __builtin_amdgcn_s_getreg(20 | (3 << 11)) & (kMaxXcds - 1);
}

// Polls *word until it has reached `target` (counters only grow; the comparison
// is safe across 32-bit wrap-around); false once `abort` is raised or the time
// limit has passed (then `abort` is raised for everyone).
__device__ __forceinline__ bool poll_reached(unsigned *word, unsigned target, LoopControl *ctl, uint64_t limit_ticks) {
    const uint64_t t0 = wall_clock64();
    unsigned polls = 0;
    // relaxed polls: an acquire load would invalidate this XCD's L2 on every
    // poll and slow the workgroups that are still computing
    while ((int)(__hip_atomic_load(word, __ATOMIC_RELAXED, AGENT) - target) < 0) {
        __builtin_amdgcn_s_sleep(1);
        if ((++polls & 63u) == 0) {
            if (__hip_atomic_load(&ctl->abort, __ATOMIC_RELAXED, AGENT)) return false;
            if (wall_clock64() - t0 > limit_ticks) {
                __hip_atomic_store(&ctl->abort, 1, __ATOMIC_RELAXED, AGENT);
                return false;
            }
        }
    }
    return true;
}

// Barrier over every workgroup of the grid.  Counters only grow: barrier number e
// (counted per launch, identically by every workgroup) is complete on an XCD
// when its counter reaches e * nx, and on the chip when the top counter
// reaches e * nxcd, so an arrival is one atomic and nothing is ever reset.
// Returns false (uniformly per block) once `abort` has been raised.
__device__ __forceinline__ bool grid_barrier_xcd(LoopControl *ctl, XcdInfo &xi, uint64_t limit_ticks) {
    int *lds_flag = reinterpret_cast<int *>(g_loop_lds);
    xi.epoch += 1u;
    // every wave waits until the L2 has acknowledged its stores, then the workgroup
    // meets: the arrival below may be what lets the XCD's last arriver write the L2
    // back, and a store still in flight then would stay dirty in this L2 only
    drain_stores_then_barrier();
    if (threadIdx.x == 0) {
        GridBarrier *xb = &ctl->xcd[xi.x];
        const unsigned prev = __hip_atomic_fetch_add(&xb->count, 1u, __ATOMIC_RELAXED, AGENT);
        if (prev + 1u == xi.epoch * xi.nx) {
            // last of this XCD: its L2 now holds every store of the XCD's workgroups
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");  // one write-back of this L2
            __hip_atomic_fetch_add(&ctl->top.count, 1u, __ATOMIC_RELAXED, AGENT);
            poll_reached(&ctl->top.count, xi.epoch * xi.nxcd, ctl, limit_ticks);
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");  // invalidates this L2 (and this CU's L1)
            __hip_atomic_store(&xb->generation, xi.epoch, __ATOMIC_RELAXED, AGENT);
        } else {
            poll_reached(&xb->generation, xi.epoch, ctl, limit_ticks);
            // This CU's L1 only: the XCD's L2 has just been invalidated by its last arriver,
            // and an agent-scope acquire here would walk that L2 once more per workgroup.
            asm volatile("buffer_inv sc0" ::: "memory");
        }
        *lds_flag = __hip_atomic_load(&ctl->abort, __ATOMIC_RELAXED, AGENT) ? 0 : 1;
    }
    __syncthreads();
    return *lds_flag != 0;
}

// The plan's tables (steps, task groups, op descriptors) are written by the host
// before the launch and never by the device, and every address into them is
// uniform across the workgroup.  They are read through the constant address
// space: scalar loads into scalar registers, served by the scalar cache, which
// the barriers' L2 invalidations do not touch.  A body receives its descriptor
// by value and reads no field from memory afterwards.
#define ARKMI_CONST __attribute__((address_space(4)))

template <typename D>
__device__ __forceinline__ D load_const(const D *p) {
    static_assert(sizeof(D) % 4 == 0, "table entries are whole words");
    D d;
    uint32_t w[sizeof(D) / 4];
    const ARKMI_CONST uint32_t *src = (const ARKMI_CONST uint32_t *)p;
#pragma unroll
    for (size_t i = 0; i < sizeof(D) / 4; ++i) w[i] = src[i];
    __builtin_memcpy(&d, w, sizeof(D));
    return d;
}

// FAM is the set of op families compiled into this kernel variant.  A plan runs on the
// smallest variant that holds its families.

// The small bodies (elementwise ops, row ops, the embedding gather) for one task, inlined.
template <int FAM>
__device__ __forceinline__ void run_small(const DevOp *op, int task, const Slot &s) {
    const int kind = load_const(&op->kind);
    if (kind == DEV_EWISE) {
        if constexpr ((FAM & FAM_EWISE) != 0) {
            const EwiseDesc d = load_const(&op->ew);
            ewise_dispatch(d, task, s);
        }
    } else if (kind == DEV_ROW) {
        if (load_const(&op->row.red_len) > 0) {
            if constexpr ((FAM & FAM_EXT) != 0) {
                const RowOpDesc d = load_const(&op->row);
                reduce_axis_dispatch(d, task, s);
            }
        } else if constexpr ((FAM & FAM_ROW) != 0) {
            const RowOpDesc d = load_const(&op->row);
            row_op_dispatch(d, task, s);
        }
    } else if (kind == DEV_EMBED) {
        if constexpr ((FAM & FAM_EXT) != 0) {
            const EmbedDesc d = load_const(&op->emb);
            embedding_task(d, task, s);
        }
    }
}

// An elementwise op fused behind a matmul in the same task (the host admits no other kind
// there).  The thread index is made opaque per task: the per-lane addresses the body derives
// from it would otherwise be lifted out of the task loop and stay in registers across the matmul.
template <int FAM>
__device__ __forceinline__ void run_follower(const DevOp *op, int task, const Slot &s_in) {
    if constexpr ((FAM & FAM_EWISE) != 0) {
        Slot s = s_in;
        asm volatile("" : "+v"(s.tid));
        const EwiseDesc d = load_const(&op->ew);
        ewise_dispatch(d, task, s);
    }
}

// The kernel's one parameter, read where a field is needed: the pointer to the kernel-argument
// segment is made opaque on every access, so no load from it is shared with an earlier one or
// lifted out of a loop, and no field occupies a scalar register across an op body.  The pointer
// is handed down as `ka`: the kernel takes it from the hardware, a non-inlined function gets it
// as an argument (inside a function the intrinsic yields a null pointer).
using KArgs = const ARKMI_CONST LoopArgs *;

__device__ __forceinline__ KArgs kernel_kargs() { return (KArgs)__builtin_amdgcn_kernarg_segment_ptr(); }

__device__ __forceinline__ KArgs launder(KArgs p) {
    asm volatile("" : "+s"(p));
    return p;
}

template <typename D>
__device__ __forceinline__ D load_karg(const ARKMI_CONST D *p) {
    static_assert(sizeof(D) % 4 == 0, "kernel-argument fields are whole words");
    D d;
    uint32_t w[sizeof(D) / 4];
    const ARKMI_CONST uint32_t *src = (const ARKMI_CONST uint32_t *)p;
#pragma unroll
    for (size_t i = 0; i < sizeof(D) / 4; ++i) w[i] = src[i];
    __builtin_memcpy(&d, w, sizeof(D));
    return d;
}
#define KARG(field) load_karg(&launder(ka)->field)  // needs a `KArgs ka` in scope

// The tasks of one task_seq<> of the reference (kernel_template.in:11-27: task ids dealt to
// processors and slots by the formula): the group's parameters and this workgroup's share.
struct TaskDeal {
    DevTaskGroup g;
    int64_t base;   // id of this workgroup's first task
    int64_t round;  // id step per full deal
    bool mine;      // this workgroup is in the group's processor range
};

__device__ __forceinline__ TaskDeal deal_of(const DevTaskGroup *groups, int gi) {
    TaskDeal d;
    d.g = load_const(groups + gi);
    const DevTaskGroup &g = d.g;
    const int block = blockIdx.x, grid = gridDim.x;
    d.mine = in_range(block, g.proc_b, g.proc_e, g.proc_s);
    const int n_procs = (g.proc_e - g.proc_b + g.proc_s - 1) / g.proc_s;
    const int p = ((block + grid - g.proc_cur) % grid) / g.proc_s;
    // Task ids fit 32 bits (the host rejects larger plans); 64-bit products only
    // where the formula could overflow before the range check.
    d.base = g.task_b + (int64_t)p * g.task_s * g.gran;
    d.round = (int64_t)g.task_s * g.gran * n_procs;
    return d;
}

__device__ __forceinline__ int64_t task_id(const TaskDeal &d, unsigned t) {
    if (d.g.gran == 1) return d.base + d.round * t;
    const unsigned q = t / (unsigned)d.g.gran, r = t - q * (unsigned)d.g.gran;
    return d.base + (int64_t)d.g.task_s * r + d.round * q;
}

__device__ __forceinline__ int task_index(const DevTaskGroup &g, int64_t id) {
    return ((int)id - g.task_b) / g.task_s;
}

// Before task index `ti` of a consumer group: wait until the producers' row blocks it reads
// are complete in this iteration.  The data is then read through this XCD's L2 without
// invalidating it: the host admits the wait in place of a barrier only where no workgroup can
// have fetched these lines since the last barrier (rows own whole cache lines, and every reader
// in between waits like this one).  False (uniformly) once `abort` is raised.  Whole-workgroup
// slots only (checked on the host).
__device__ __forceinline__ bool wait_for_rows(KArgs ka, const DevTaskGroup &g, int ti, int tid, int nthreads,
                                              unsigned epoch, lds_ptr control) {
    // (`control`: the start of the workgroup's LDS; a body function gets it from its slot window)
    volatile __attribute__((address_space(3))) int *fail = (volatile __attribute__((address_space(3))) int *)control + 1;
    const DevWait *waits = KARG(prog.waits) + g.wait_begin;
    const int32_t *spans = KARG(prog.wait_spans) + g.span_begin + 2 * (ti * g.n_waits);
    unsigned *counters = KARG(prog.dep_counters);
    LoopControl *ctl = KARG(ctl);
    const uint64_t limit = KARG(wait_ticks);
    bool ok = true;
    for (int w = 0; w < g.n_waits; ++w) {
        const DevWait dw = load_const(waits + w);
        const int lo = load_const(spans + 2 * w), hi = load_const(spans + 2 * w + 1);
        const unsigned target = (unsigned)dw.expect * epoch;
        for (int c = lo + tid; c <= hi; c += nthreads)
            ok = poll_reached(counters + (size_t)(dw.counter_base + c) * kDepStride, target, ctl, limit) && ok;
    }
    if (!ok) *fail = 1;
    __syncthreads();
    return *fail == 0;
}

// After task index `ti` of a producer group: every wave's stores have been acknowledged by the
// L2, the L2 is written back (the release), then the row block's counter grows by one.
__device__ __forceinline__ void signal_rows(KArgs ka, const DevTaskGroup &g, int ti) {
    drain_stores_then_barrier();
    if (threadIdx.x == 0) {
        const int block = load_const(KARG(prog.signal_map) + g.signal_begin + ti);
        __hip_atomic_fetch_add(KARG(prog.dep_counters) + (size_t)(g.signal_base + block) * kDepStride, 1u,
                               __ATOMIC_RELEASE, AGENT);
    }
}

// ---- the long-running bodies -----------------------------------------------------------------
// Matmul tiles, the skinny matmul and attention are functions of their own, not inlined into
// the kernel: each gets its own register allocation and instruction schedule, the same in every
// variant, in the loop kernel and in the one-op kernels alike.  (Inlined, the K loop of a
// matmul tile came out differently depending on what surrounded it: in the loop kernel its
// loads were issued later and it carried five more waits than in a kernel of its own, and ran
// 10-15 % slower.)  A function that needs most of the vector registers saves and restores the
// callee-saved half of them around its body (~6 us for a 256x256 tile), so the task loop runs
// inside the function: it returns when the group's tasks are done, or after one task when ops
// are fused behind the matmul (those run in the kernel).  Arguments arrive in vector registers;
// what is uniform is moved to scalar registers first.
#ifndef ARKMI_BODY
#define ARKMI_BODY __device__ __attribute__((noinline))
#endif

constexpr int kTasksDone = -2;     // returned by a body: the group has no more tasks for this workgroup
constexpr int kTasksAborted = -3;  // a dependency wait gave up
static_assert(kGemmAborted == kTasksAborted, "a matmul body reports an expired wait with the task loop's value");

__device__ __forceinline__ KArgs uniform_kargs(KArgs p) {
    const uint64_t a = (uint64_t)(uintptr_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
    return (KArgs)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

// A long-running op owns the whole workgroup (checked on the host): slot 0, all waves.
__device__ __forceinline__ Slot body_slot(int tid, lds_ptr lds) {
    Slot s;
    s.tid = tid;
    s.nthreads = kLoopMaxThreads;  // (not read by these bodies)
    s.lds = (lds_ptr)(uintptr_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds);
    s.lds_bytes = 0;
    s.whole_block = true;
    return s;
}

// The task loop of a group whose first op is long-running, from this workgroup's task number
// `t0` on.  `one(op, task)` runs the op for one task and returns the task the fused followers
// run for (-1: none, a split of K that another workgroup finishes).  Nothing of the group's
// parameters is kept across the op: they are read again for every task.  Returns kTasksDone,
// kTasksAborted, or -- for a group with followers, after one task -- that task's follow value.
template <typename One>
__device__ __forceinline__ int long_task_loop(KArgs ka, int gi, int t0, int tid, unsigned epoch, lds_ptr control,
                                              One one) {
    for (unsigned t = (unsigned)t0;; ++t) {
        int follow;
        {
            const TaskDeal d = deal_of(KARG(prog.groups), gi);
            const DevTaskGroup &g = d.g;
            const int64_t id = task_id(d, t);
            if (id >= g.task_e) return kTasksDone;
#ifndef ARKMI_NO_TRACE
            TraceRecord *trace = KARG(prog.trace);
            if (trace && g.trace_offset >= 0 && tid == 0) {
                TraceRecord rec{(int)blockIdx.x, 0, (int)t};
                trace[g.trace_offset + task_index(g, id)] = rec;
            }
#endif
            if (KARG(prog.dep_counters) != nullptr && g.n_waits > 0 &&
                !wait_for_rows(ka, g, task_index(g, id), tid, kLoopMaxThreads, epoch, control))
                return kTasksAborted;
            follow = one(KARG(prog.ops) + g.op_begin, (int)id);
            if (follow == kTasksAborted) return kTasksAborted;
        }
        const DevTaskGroup g = load_const(KARG(prog.groups) + gi);
        if (g.op_count > 1) return follow;  // the kernel runs the followers, signals, and calls again
        // (a matmul that splits K signals for the tile this workgroup finished, if any)
        if (KARG(prog.dep_counters) != nullptr && g.signal_begin >= 0 && follow >= 0)
            signal_rows(ka, g, task_index(g, follow));
    }
}

template <typename T, int BM, int BN, bool TRANS_B, bool TRANS_A = false, bool DUAL_B = false, bool SPLIT = false>
ARKMI_BODY int gemm_body(KArgs ka_in, int gi, int t0, int tid, lds_ptr lds, unsigned epoch) {
    const KArgs ka = uniform_kargs(ka_in);
    const Slot s = body_slot(tid, lds);
    return long_task_loop(ka, __builtin_amdgcn_readfirstlane(gi), __builtin_amdgcn_readfirstlane(t0), tid,
                          __builtin_amdgcn_readfirstlane(epoch), s.lds - kLdsReserved, [&](const DevOp *op, int task) {
                              const GemmDesc g = load_const(&op->gemm);
                              if constexpr (SPLIT) {
                                  auto poll = [&](unsigned int *word, unsigned int want) {
                                      return poll_equals(word, want, BodyWait{&KARG(ctl)->abort, KARG(wait_ticks)});
                                  };
                                  return gemm_tile<T, BM, BN, TRANS_B, EpilogueStore, TRANS_A, DUAL_B, SPLIT>(
                                      g, task, s, EpilogueStore(), poll);
                              } else {
                                  return gemm_tile<T, BM, BN, TRANS_B, EpilogueStore, TRANS_A, DUAL_B, SPLIT>(
                                      g, task, s, EpilogueStore());
                              }
                          });
}

ARKMI_BODY int gemm_f32_body(KArgs ka_in, int gi, int t0, int tid, lds_ptr lds, unsigned epoch) {
    const KArgs ka = uniform_kargs(ka_in);
    const Slot s = body_slot(tid, lds);
    return long_task_loop(ka, __builtin_amdgcn_readfirstlane(gi), __builtin_amdgcn_readfirstlane(t0), tid,
                          __builtin_amdgcn_readfirstlane(epoch), s.lds - kLdsReserved, [&](const DevOp *op, int task) {
                              const GemmDesc g = load_const(&op->gemm);
                              gemm_f32_dispatch(g, task, s);
                              return task;
                          });
}

// Where the loop kernel's skinny-matmul stretches come from (the `Source` of gemv_stream).
// This workgroup's row of one of the host's tables:
struct GemvTableSource {
    KArgs ka;
    const GemvSeqEntry *entry;  // the next one
    int tid;
    __device__ __forceinline__ bool next(GemvDesc &d, int &nb, int &ku, int &units, int &part, int &parts) {
        const GemvSeqEntry e = load_const(entry);
        if (e.op < 0) return false;
        ++entry;
#ifndef ARKMI_NO_TRACE
        TraceRecord *trace = KARG(prog.trace);
        if (trace && e.trace_index >= 0 && tid == 0) {
            TraceRecord rec{(int)blockIdx.x, 0, e.order};
            trace[e.trace_index] = rec;
        }
#endif
        d = load_const(&(KARG(prog.ops) + e.op)->gemv);
        nb = e.nb; ku = e.ku; units = e.units; part = e.part; parts = e.parts;
        return true;
    }
    __device__ __forceinline__ void fold_begins(int) {}
    __device__ __forceinline__ void fold_ends(int) {}
};

// A list of stretches shared by the grid: workgroup b streams entries b and b + grid, and while
// it folds its k-th stretch it claims the one it will stream as its (k+2)-th from a counter, so a
// workgroup that streams more slowly (its share of the HBM bandwidth varies) ends up with fewer.
// Thread 0 claims; the claimed index reaches the other waves through a ring of four words in
// the body's LDS control area, published by the barrier that ends the fold.  The load cursor,
// two units ahead, reads position k when it leaves stretch k - 1, which is after the fold of
// stretch k - 2 as long as every stretch has at least 3 units (the host checks).
struct GemvClaimSource {
    KArgs ka;
    const GemvSeqEntry *entries;
    int n;
    unsigned *counter;  // of this iteration
    unsigned *other;    // of the next one: zeroed meanwhile
    lds_u32_ptr ring;
    int k = 0;          // position of the next stretch in this workgroup's sequence
    unsigned pending = 0;
    __device__ __forceinline__ bool next(GemvDesc &d, int &nb, int &ku, int &units, int &part, int &parts) {
        unsigned id;
        if (k < 2) id = blockIdx.x + (unsigned)k * gridDim.x;
        else id = __builtin_amdgcn_readfirstlane(ring[k & 3]);
        ++k;
        if (id >= (unsigned)n) return false;
        const GemvSeqEntry e = load_const(entries + id);
        d = load_const(&(KARG(prog.ops) + e.op)->gemv);
        nb = e.nb; ku = e.ku; units = e.units; part = e.part; parts = e.parts;
        return true;
    }
    // (called on the multiply cursor: k - 1 is the position of the stretch being folded)
    __device__ __forceinline__ void fold_begins(int tid) {
        if (tid == 0) {
            pending = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, AGENT);
            if (blockIdx.x == 0 && k == 1) __hip_atomic_store(other, 0u, __ATOMIC_RELAXED, AGENT);
        }
    }
    __device__ __forceinline__ void fold_ends(int tid) {
        if (tid == 0) ring[(k + 1) & 3] = pending + 2u * gridDim.x;
    }
};

// (Skinny matmuls take no part in the dependency counters: the host keeps the barriers around
// them, so there is nothing to wait for or to signal here.)
ARKMI_BODY int gemv_body(KArgs ka_in, int gi_in, int t0, int tid, lds_ptr lds, unsigned epoch_in) {
    const KArgs ka = uniform_kargs(ka_in);
    const Slot s = body_slot(tid, lds);
    const int gi = __builtin_amdgcn_readfirstlane(gi_in);
    const unsigned epoch = __builtin_amdgcn_readfirstlane(epoch_in);
    const DevTaskGroup *g = KARG(prog.groups) + gi;
    // the loop kernel streams a run of groups from the first one; the one-op kernels (which name
    // their group in the kernel arguments) run every group by itself
    const bool loop = KARG(group) < 0;
    const int begin = loop ? load_const(&g->run_begin) : load_const(&g->seq_begin);
    const int stride = loop ? load_const(&g->run_stride) : load_const(&g->seq_stride);
    const int claim = loop ? load_const(&g->claim) : -1;
    const GemvSeqEntry *seq = KARG(prog.gemv_seq) + begin;
    // (one element type per sequence: checked on the host)
    if (claim >= 0) {
        if (stride <= 0) return kTasksDone;
        unsigned *counters = KARG(prog.gemv_claims) + (size_t)claim * 2 * kDepStride;
        GemvClaimSource src{ka, seq, stride, counters + (epoch & 1u) * kDepStride,
                            counters + ((epoch + 1u) & 1u) * kDepStride, (lds_u32_ptr)(s.lds + 16)};
        if (load_const(&(KARG(prog.ops) + load_const(&seq->op))->gemv.dtype) == 1) gemv_stream<f16>(s, src);
        else gemv_stream<bf16>(s, src);
        return kTasksDone;
    }
    seq += (size_t)blockIdx.x * stride;
    const int op = load_const(&seq->op);
    if (op >= 0) {
        GemvTableSource src{ka, seq, tid};
        if (load_const(&(KARG(prog.ops) + op)->gemv.dtype) == 1) gemv_stream<f16>(s, src);
        else gemv_stream<bf16>(s, src);
    }
    return kTasksDone;
}

ARKMI_BODY int attn_body(KArgs ka_in, int gi, int t0, int tid, lds_ptr lds, unsigned epoch) {
    const KArgs ka = uniform_kargs(ka_in);
    const Slot s = body_slot(tid, lds);
    return long_task_loop(ka, __builtin_amdgcn_readfirstlane(gi), __builtin_amdgcn_readfirstlane(t0), tid,
                          __builtin_amdgcn_readfirstlane(epoch), s.lds - kLdsReserved, [&](const DevOp *op, int task) {
                              const AttnDesc d = load_const(&op->attn);
                              attn_dispatch(d, task, s);
                              return task;
                          });
}

#define ARKMI_BODY_ARGS ka, gi, t0, tid, lds, epoch

template <int FAM, typename T, bool TRANS_B>
__device__ __forceinline__ int gemm_by_tile(const DevOp *op, KArgs ka, int gi, int t0, int tid, lds_ptr lds,
                                            unsigned epoch) {
    const int tm = load_const(&op->gemm_tile_m), tn = load_const(&op->gemm_tile_n);
    if (load_const(&op->gemm.split_k) == 2) {  // 256x256 tiles only (checked on the host)
        if constexpr ((FAM & FAM_SPLITK) != 0)
            return gemm_body<T, 256, 256, TRANS_B, false, false, true>(ARKMI_BODY_ARGS);
        else
            return kTasksDone;
    }
    if constexpr (TRANS_B) {
        if (load_const(&op->gemm.b2) != nullptr) {  // gate/up pair: 256-wide tiles only (checked on the host)
            if (tm == 256) return gemm_body<T, 256, 256, true, false, true>(ARKMI_BODY_ARGS);
            return gemm_body<T, 128, 256, true, false, true>(ARKMI_BODY_ARGS);
        }
    }
    if (tm == 256 && tn == 256) return gemm_body<T, 256, 256, TRANS_B>(ARKMI_BODY_ARGS);
    if (tm == 128 && tn == 256) return gemm_body<T, 128, 256, TRANS_B>(ARKMI_BODY_ARGS);
    if (tm == 256 && tn == 128) return gemm_body<T, 256, 128, TRANS_B>(ARKMI_BODY_ARGS);
    return gemm_body<T, 128, 128, TRANS_B>(ARKMI_BODY_ARGS);
}

// Hands the group's tasks from number t0 on to the body of its first op (of the long-running
// kind KIND).  Returns (uniformly) what the body returned.
template <int FAM, int KIND>
__device__ __forceinline__ int run_long(const DevOp *op, KArgs ka, int gi, int t0, int tid, lds_ptr lds,
                                        unsigned epoch) {
    int r = kTasksDone;
    if constexpr (KIND == DEV_GEMM) {
        const int dtype = load_const(&op->gemm.dtype);
        const bool trans_a = load_const(&op->gemm.trans_a) != 0, trans_b = load_const(&op->gemm.trans_b) != 0;
        if (dtype == 0 || trans_a) {
            if constexpr ((FAM & FAM_EXT) != 0) {
                if (dtype == 0) r = gemm_f32_body(ARKMI_BODY_ARGS);
                else if (dtype == 1)
                    r = trans_b ? gemm_body<f16, 128, 128, true, true>(ARKMI_BODY_ARGS)
                                : gemm_body<f16, 128, 128, false, true>(ARKMI_BODY_ARGS);
                else
                    r = trans_b ? gemm_body<bf16, 128, 128, true, true>(ARKMI_BODY_ARGS)
                                : gemm_body<bf16, 128, 128, false, true>(ARKMI_BODY_ARGS);
            }
        } else if constexpr ((FAM & FAM_GEMM) != 0) {
            if (dtype == 1)
                r = trans_b ? gemm_by_tile<FAM, f16, true>(op, ARKMI_BODY_ARGS) : gemm_by_tile<FAM, f16, false>(op, ARKMI_BODY_ARGS);
            else
                r = trans_b ? gemm_by_tile<FAM, bf16, true>(op, ARKMI_BODY_ARGS) : gemm_by_tile<FAM, bf16, false>(op, ARKMI_BODY_ARGS);
        }
    } else if constexpr (KIND == DEV_GEMV) {
        if constexpr ((FAM & FAM_GEMV) != 0) r = gemv_body(ARKMI_BODY_ARGS);
    } else if constexpr (KIND == DEV_ATTN) {
        if constexpr ((FAM & FAM_ATTN) != 0) r = attn_body(ARKMI_BODY_ARGS);
    }
    return __builtin_amdgcn_readfirstlane(r);
}

// The task loop of a group of small ops: the program's and the group's parameters stay in
// registers (`P` was read once for the step).
template <int FAM>
__device__ __forceinline__ bool run_small_tasks(KArgs ka, const LoopProgram &P, const TaskDeal &d, const Slot &s,
                                                int slot_k, unsigned epoch) {
    const DevTaskGroup &g = d.g;
    const DevOp *ops = P.ops + g.op_begin;
    const bool deps = P.dep_counters != nullptr;
    const bool waits = deps && g.n_waits > 0, signals = deps && g.signal_begin >= 0;
    int order = 0;
    for (unsigned t = (unsigned)slot_k;; t += (unsigned)g.n_slots, ++order) {
        const int64_t id = task_id(d, t);
        if (id >= g.task_e) break;
        const int ti = (waits || signals) ? task_index(g, id) : 0;
#ifndef ARKMI_NO_TRACE
        if (P.trace && g.trace_offset >= 0 && s.tid == 0) {
            TraceRecord rec{(int)blockIdx.x, slot_k, order};
            P.trace[g.trace_offset + task_index(g, id)] = rec;
        }
#endif
        if (waits && !wait_for_rows(ka, g, ti, s.tid, s.nthreads, epoch, (lds_ptr)g_loop_lds)) return false;
        for (int o = 0; o < g.op_count; ++o) {
            // later ops of a fused task read what earlier ones of the same slot wrote: the slot's
            // waves meet (they share one L1, which sees their stores)
            if (o > 0) s.sync();
            run_small<FAM>(ops + o, (int)id, s);
        }
        if (signals) signal_rows(ka, g, ti);
    }
    return true;
}

// A group whose first op is long-running (KIND: matmul, skinny matmul, attention): the body
// function runs the tasks; it comes back after each task when ops are fused behind a matmul,
// which then run here.
template <int FAM, int KIND>
__device__ __forceinline__ bool run_long_tasks(KArgs ka, int gi, const Slot &s, unsigned epoch) {
    for (int t = 0;; ++t) {
        const DevOp *first = KARG(prog.ops) + load_const(&(KARG(prog.groups) + gi)->op_begin);
        const int follow = run_long<FAM, KIND>(first, ka, gi, t, s.tid, s.lds, epoch);
        if (follow == kTasksDone) return true;
        if (follow == kTasksAborted) return false;
        // one task of a group with followers was run; `follow` is the tile they run for
        const DevTaskGroup g = load_const(KARG(prog.groups) + gi);
        if constexpr (KIND == DEV_GEMM) {
            const DevOp *ops = KARG(prog.ops) + g.op_begin;
            for (int o = 1; o < g.op_count && follow >= 0; ++o) {
                s.sync();
                run_follower<FAM>(ops + o, follow, s);
            }
        }
        if (KARG(prog.dep_counters) != nullptr && g.signal_begin >= 0 && follow >= 0)
            signal_rows(ka, g, task_index(g, follow));
    }
}

// Does this variant hold a long-running body?  If not, nothing competes for scalar registers
// and the program's parameters are read once per launch instead of once per step.
template <int FAM>
constexpr bool kHasLongBodies = (FAM & (FAM_GEMM | FAM_SPLITK | FAM_EXT | FAM_GEMV | FAM_ATTN)) != 0;

constexpr int kLdsSlotCounters = 64;  // byte offset of the slots' arrival counters in the control area

template <int FAM>
__device__ __forceinline__ bool run_group(KArgs ka, const LoopProgram &P, int gi, unsigned epoch) {
    const TaskDeal d = deal_of(P.groups, gi);
    const DevTaskGroup &g = d.g;
    if constexpr ((FAM & FAM_GEMV) != 0) {
        if (KARG(group) < 0) {
            // a skinny matmul that the first group of its run has already streamed
            if (g.chain < 0) return true;
            // the first group of a run, or stretches claimed at run time: the host's tables say
            // what this workgroup does, whether or not it has a task of the (first) matmul
            if (g.chain > 1 || g.claim >= 0) {
                const Slot s0 = body_slot(threadIdx.x, (lds_ptr)g_loop_lds + kLdsReserved);
                return run_long_tasks<FAM, DEV_GEMV>(ka, gi, s0, epoch);
            }
        }
    }
    if (!d.mine) return true;
    const int slot_threads = g.slot_warps * kWave;
    const int k = threadIdx.x / slot_threads;
    if (k >= g.n_slots) return true;
    Slot s;
    s.tid = threadIdx.x - k * slot_threads;
    // Opaque per task group: what the bodies derive from the thread index alone (per-lane
    // address parts) is loop-invariant for the compiler, which would lift it out of the step and
    // iteration loops for every body at once and keep it live across all of them and across the
    // calls of the long-running bodies, where only the callee-saved registers survive (one
    // variant spilled 51 000 vector registers that way).  Inside the group's task loop it may
    // still be lifted.
    asm volatile("" : "+v"(s.tid));
    s.nthreads = slot_threads;
    s.lds = (lds_ptr)g_loop_lds + kLdsReserved + k * g.slot_sram;
    s.lds_bytes = g.slot_sram;
    s.whole_block = (slot_threads == (int)blockDim.x);
    s.arrivals = s.whole_block ? nullptr : (lds_u32_ptr)((lds_ptr)g_loop_lds + kLdsSlotCounters) + k;
    // one task loop per long-running kind of first op, one for the tasks of small ops
    // (a variant holds the loops of the families it was built for)
    const int first = load_const(&(P.ops + g.op_begin)->kind);
    if constexpr ((FAM & (FAM_GEMM | FAM_SPLITK | FAM_EXT)) != 0) {
        if (first == DEV_GEMM) return run_long_tasks<FAM, DEV_GEMM>(ka, gi, s, epoch);
    }
    if constexpr ((FAM & FAM_GEMV) != 0) {
        if (first == DEV_GEMV) return run_long_tasks<FAM, DEV_GEMV>(ka, gi, s, epoch);
    }
    if constexpr ((FAM & FAM_ATTN) != 0) {
        if (first == DEV_ATTN) return run_long_tasks<FAM, DEV_ATTN>(ka, gi, s, epoch);
    }
    if constexpr ((FAM & (FAM_ROW | FAM_EWISE | FAM_EXT)) != 0) {
        if (first != DEV_GEMM && first != DEV_GEMV && first != DEV_ATTN)
            return run_small_tasks<FAM>(ka, P, d, s, k, epoch);
    }
    return true;
}

// The control words at the start of the workgroup's LDS: [0] the barriers' verdict, [1] raised
// when a dependency wait gave up, from byte kLdsSlotCounters one arrival counter per slot.
__device__ __forceinline__ void init_lds_control() {
    if (threadIdx.x == 0) reinterpret_cast<volatile int *>(g_loop_lds)[1] = 0;
    if (threadIdx.x < 8) reinterpret_cast<volatile unsigned *>(g_loop_lds + kLdsSlotCounters)[threadIdx.x] = 0u;
    __syncthreads();
}

// One iteration of the plan's body; `epoch` counts the iterations since the launch from 1.
template <int FAM>
__device__ __forceinline__ bool run_body(KArgs ka, const LoopProgram &P0, XcdInfo &xi, unsigned epoch) {
    const int num_steps = kHasLongBodies<FAM> ? KARG(prog.num_steps) : P0.num_steps;
    for (int si = 0; si < num_steps; ++si) {
        // (one read of the whole parameter block per step where long bodies want the registers)
        const LoopProgram P = kHasLongBodies<FAM> ? KARG(prog) : P0;
        const DevStep st = load_const(P.steps + si);
        if (P.step_clock && threadIdx.x == 0) P.step_clock[(size_t)blockIdx.x * (P.num_steps + 1) + si] = wall_clock64();
        if (st.kind == STEP_BARRIER) {
            LoopControl *ctl = KARG(ctl);
            if ((unsigned)st.count == gridDim.x) {
                if (!grid_barrier_xcd(ctl, xi, KARG(wait_ticks))) return false;
            } else if (in_range(blockIdx.x, st.b, st.e, st.s)) {
                if (!grid_barrier(&ctl->bars[st.index], (unsigned)st.count, ctl, KARG(wait_ticks))) return false;
            }
        } else if (st.kind == STEP_LOCAL_SYNC) {
            // the next group reads only what this workgroup itself wrote: its waves share one
            // L1, which sees their own stores, so the workgroup only has to meet
            __syncthreads();
        } else {
            if (!run_group<FAM>(ka, P, st.index, epoch)) return false;
        }
    }
    unsigned long long *clock = KARG(prog.step_clock);
    if (clock && threadIdx.x == 0) clock[(size_t)blockIdx.x * (num_steps + 1) + num_steps] = wall_clock64();
    return true;
}

template <int FAM>
__global__ __launch_bounds__(kLoopMaxThreads) void arkmi_loop_kernel(LoopArgs) {
    const KArgs ka = kernel_kargs();
    const unsigned nblocks = gridDim.x;
    const bool leader = (blockIdx.x == 0 && threadIdx.x == 0);
    init_lds_control();
    // count the workgroups per XCD (the control block is zeroed before every launch)
    XcdInfo xi;
    xi.epoch = 0;
    xi.x = xcc_id();
    {
        LoopControl *ctl = KARG(ctl);
        HostMailbox *mb = KARG(mb);
        if (threadIdx.x == 0) __hip_atomic_fetch_add(&ctl->xcd_blocks[xi.x], 1u, __ATOMIC_RELAXED, AGENT);
        if (!grid_barrier(&ctl->all, nblocks, ctl, KARG(wait_ticks))) {
            if (threadIdx.x == 0) {
                __hip_atomic_store(&mb->status, (int)MB_ABORTED, __ATOMIC_RELAXED, SYSTEM);
                if (blockIdx.x == 0) __hip_atomic_store(&mb->alive, 0, __ATOMIC_RELEASE, SYSTEM);
            }
            return;
        }
        xi.nx = __hip_atomic_load(&ctl->xcd_blocks[xi.x], __ATOMIC_RELAXED, AGENT);
        xi.nxcd = 0;
        for (int i = 0; i < kMaxXcds; ++i)
            xi.nxcd += __hip_atomic_load(&ctl->xcd_blocks[i], __ATOMIC_RELAXED, AGENT) ? 1u : 0u;
    }
    unsigned epoch = 0;  // iterations of the body started since the launch
    const LoopProgram P0 = KARG(prog);
    for (;;) {
        int iter;
        const int one_shot_iters = KARG(one_shot_iters);
        if (one_shot_iters > 0) {
            iter = one_shot_iters;
        } else {
            LoopControl *ctl = KARG(ctl);
            if (leader) {
                HostMailbox *mb = KARG(mb);
                const uint64_t idle_ticks = KARG(idle_ticks);
                const uint64_t t0 = wall_clock64();
                int cmd;
                unsigned polls = 0;
                while ((cmd = __hip_atomic_load(&mb->cmd, __ATOMIC_RELAXED, SYSTEM)) == 0) {
                    __builtin_amdgcn_s_sleep(8);
                    if ((++polls & 15u) == 0 && wall_clock64() - t0 > idle_ticks) {
                        cmd = -2;  // nobody is driving this kernel any more
                        break;
                    }
                }
                __hip_atomic_store(&ctl->iter, cmd, __ATOMIC_RELAXED, AGENT);
            }
            if (!grid_barrier_xcd(ctl, xi, KARG(wait_ticks))) break;
            iter = __hip_atomic_load(&ctl->iter, __ATOMIC_RELAXED, AGENT);
            if (iter < 0) {
                if (leader) {
                    HostMailbox *mb = KARG(mb);
                    if (iter == -2) __hip_atomic_store(&mb->status, (int)MB_IDLE_EXIT, __ATOMIC_RELAXED, SYSTEM);
                    __hip_atomic_store(&mb->alive, 0, __ATOMIC_RELEASE, SYSTEM);
                }
                return;
            }
        }
        bool ok = true;
        for (int i = 0; i < iter && ok; ++i) {
            if (i > 0) {
                // the host has compared the end of the body with its start: a barrier
                // when another workgroup's data is involved, a local sync when only
                // this workgroup's own, nothing when the iterations share no data
                const int iter_sync = KARG(prog.iter_sync);
                if (iter_sync == 2) {
                    ok = grid_barrier_xcd(KARG(ctl), xi, KARG(wait_ticks));
                } else if (iter_sync == 1) {
                    __syncthreads();
                }
            }
            ++epoch;
            if (ok) ok = run_body<FAM>(ka, P0, xi, epoch);
        }
        if (!ok) break;
        // results must be visible to the host before the command is cleared: every
        // wave's stores are in the L2 before thread 0's system-scope release
        drain_stores_then_barrier();
        if (threadIdx.x == 0) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
        if (!grid_barrier_xcd(KARG(ctl), xi, KARG(wait_ticks))) break;
        if (one_shot_iters > 0) return;
        if (leader) {
            HostMailbox *mb = KARG(mb);
            __hip_atomic_store(&mb->done, mb->done + iter, __ATOMIC_RELAXED, SYSTEM);
            __hip_atomic_store(&mb->cmd, 0, __ATOMIC_RELEASE, SYSTEM);
        }
    }
    // a bounded wait expired somewhere: report and leave
    if (threadIdx.x == 0) {
        HostMailbox *mb = KARG(mb);
        __hip_atomic_store(&mb->status, (int)MB_ABORTED, __ATOMIC_RELAXED, SYSTEM);
        if (blockIdx.x == 0) __hip_atomic_store(&mb->alive, 0, __ATOMIC_RELEASE, SYSTEM);
    }
}

// One task group as a kernel of its own (no loop, no barriers): the same op
// bodies launched the conventional way, one kernel per op, for comparison with
// the persistent loop kernel.  The host passes no dependency counters here: kernel
// boundaries order everything.
template <int FAM>
__global__ __launch_bounds__(kLoopMaxThreads) void arkmi_step_kernel(LoopArgs) {
    const KArgs ka = kernel_kargs();
    init_lds_control();
    const LoopProgram P = KARG(prog);
    if (!run_group<FAM>(ka, P, KARG(group), 1u) && threadIdx.x == 0) {
        // a body's bounded wait expired: report it the way the loop kernel does
        HostMailbox *mb = KARG(mb);
        if (mb) __hip_atomic_store(&mb->status, (int)MB_ABORTED, __ATOMIC_RELAXED, SYSTEM);
    }
}

// Defines the host-visible handles of one kernel variant; each variant is its own
// translation unit so the variants compile in parallel.
#define ARKMI_LOOP_KERNEL_VARIANT(FAM)                                        \
    const void *loop_kernel_variant_##FAM() {                                 \
        return reinterpret_cast<const void *>(&arkmi_loop_kernel<FAM>);       \
    }
// The one-op kernels exist for the variants a single task group can need.
#define ARKMI_STEP_KERNEL_VARIANT(FAM)                                        \
    const void *step_kernel_variant_##FAM() {                                 \
        return reinterpret_cast<const void *>(&arkmi_step_kernel<FAM>);       \
    }

}  // namespace arkmi
