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
static __device__ bool grid_barrier(GridBarrier *bar, unsigned nblocks, LoopControl *ctl,
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
static __device__ bool poll_reached(unsigned *word, unsigned target, LoopControl *ctl, uint64_t limit_ticks) {
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
static __device__ bool grid_barrier_xcd(LoopControl *ctl, XcdInfo &xi, uint64_t limit_ticks) {
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
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");  // this CU's L1
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

// Returns the task index the ops fused behind the matmul run for (the tile this workgroup
// finished), -1 when another workgroup finishes the tile (a split of K).
template <int FAM, typename T, bool TRANS_B>
__device__ __forceinline__ int gemm_by_tile(const DevOp *op, int task, const Slot &s) {
    const GemmDesc g = load_const(&op->gemm);
    const int tm = load_const(&op->gemm_tile_m), tn = load_const(&op->gemm_tile_n);
    if (g.split_k == 2) {  // 256x256 tiles only (checked on the host)
        if constexpr ((FAM & FAM_SPLITK) != 0)
            return gemm_tile<T, 256, 256, TRANS_B, EpilogueStore, false, false, true>(g, task, s, EpilogueStore());
        else
            return -1;
    }
    if constexpr (TRANS_B) {
        if (g.b2) {  // gate/up pair: 256-wide tiles only (checked on the host)
            if (tm == 256) return gemm_tile<T, 256, 256, true, EpilogueStore, false, true>(g, task, s, EpilogueStore());
            return gemm_tile<T, 128, 256, true, EpilogueStore, false, true>(g, task, s, EpilogueStore());
        }
    }
    if (tm == 256 && tn == 256) return gemm_tile<T, 256, 256, TRANS_B>(g, task, s, EpilogueStore());
    if (tm == 128 && tn == 256) return gemm_tile<T, 128, 256, TRANS_B>(g, task, s, EpilogueStore());
    if (tm == 256 && tn == 128) return gemm_tile<T, 256, 128, TRANS_B>(g, task, s, EpilogueStore());
    return gemm_tile<T, 128, 128, TRANS_B>(g, task, s, EpilogueStore());
}

// FAM is the set of op families compiled into this kernel variant.  The families
// differ widely in register need (a 256x256 GEMM tile takes nearly the whole
// budget of a two-waves-per-SIMD workgroup); compiled together they share one
// register allocation, and the row and elementwise bodies then spill values
// that live across the task loop and reload them in their inner loops.  A
// plan runs on the smallest variant that holds its families.
// Returns the task index for the ops that follow in the same fused task: `task` itself, except
// behind a matmul that splits K, where it is the tile this workgroup finished or -1 (none).
template <int FAM>
__device__ __forceinline__ int run_op(const DevOp *op, int task, const Slot &s_in) {
    // For the long-running bodies the thread index is made opaque per task: the per-lane
    // addresses they derive from it would otherwise be hoisted out of the task and step
    // loops as invariants and stay in registers across every other body.  The short
    // bodies keep theirs hoisted (they run many tasks per step).
    Slot s = s_in;
    const int kind = load_const(&op->kind);
    if (kind == DEV_GEMM || kind == DEV_ATTN || kind == DEV_GEMV) asm volatile("" : "+v"(s.tid));
    switch (kind) {
        case DEV_ROW:
            if (load_const(&op->row.red_len) > 0) {
                if constexpr ((FAM & FAM_EXT) != 0) {
                    const RowOpDesc d = load_const(&op->row);
                    reduce_axis_dispatch(d, task, s);
                }
            } else if constexpr ((FAM & FAM_ROW) != 0) {
                const RowOpDesc d = load_const(&op->row);
                row_op_dispatch(d, task, s);
            }
            break;
        case DEV_EWISE:
            if constexpr ((FAM & FAM_EWISE) != 0) {
                const EwiseDesc d = load_const(&op->ew);
                ewise_dispatch(d, task, s);
            }
            break;
        case DEV_GEMM:
            if (load_const(&op->gemm.dtype) == 0 || load_const(&op->gemm.trans_a) != 0) {
                if constexpr ((FAM & FAM_EXT) != 0) {
                    const GemmDesc g = load_const(&op->gemm);
                    if (g.dtype == 0) gemm_f32_dispatch(g, task, s);
                    else if (g.dtype == 1) {
                        if (g.trans_b) gemm_tile<f16, 128, 128, true, EpilogueStore, true>(g, task, s, EpilogueStore());
                        else gemm_tile<f16, 128, 128, false, EpilogueStore, true>(g, task, s, EpilogueStore());
                    } else {
                        if (g.trans_b) gemm_tile<bf16, 128, 128, true, EpilogueStore, true>(g, task, s, EpilogueStore());
                        else gemm_tile<bf16, 128, 128, false, EpilogueStore, true>(g, task, s, EpilogueStore());
                    }
                }
            } else if constexpr ((FAM & FAM_GEMM) != 0) {
                const bool trans_b = load_const(&op->gemm.trans_b) != 0;
                if (load_const(&op->gemm.dtype) == 1) {
                    if (trans_b) return gemm_by_tile<FAM, f16, true>(op, task, s);
                    return gemm_by_tile<FAM, f16, false>(op, task, s);
                } else {
                    if (trans_b) return gemm_by_tile<FAM, bf16, true>(op, task, s);
                    return gemm_by_tile<FAM, bf16, false>(op, task, s);
                }
            }
            break;
        case DEV_GEMV:
            if constexpr ((FAM & FAM_GEMV) != 0) {
                const GemvDesc d = load_const(&op->gemv);
                gemv_dispatch(d, task, s);
            }
            break;
        case DEV_EMBED:
            if constexpr ((FAM & FAM_EXT) != 0) {
                const EmbedDesc d = load_const(&op->emb);
                embedding_task(d, task, s);
            }
            break;
        case DEV_ATTN:
            if constexpr ((FAM & FAM_ATTN) != 0) {
                const AttnDesc d = load_const(&op->attn);
                attn_dispatch(d, task, s);
            }
            break;
        default: break;
    }
    return task;
}

// task_seq<> of the reference, parameters read from the table
// (kernel_template.in:11-27).
template <int FAM>
__device__ __forceinline__ void run_group(const LoopProgram &prog, const DevTaskGroup *gptr) {
    const DevTaskGroup g = load_const(gptr);
    const int block = blockIdx.x;
    if (!in_range(block, g.proc_b, g.proc_e, g.proc_s)) return;
    const DevOp *ops = prog.ops + g.op_begin;
    const int slot_threads = g.slot_warps * kWave;
    const int k = threadIdx.x / slot_threads;
    if (k >= g.n_slots) return;
    const int n_procs = (g.proc_e - g.proc_b + g.proc_s - 1) / g.proc_s;
    const int grid = gridDim.x;
    const int p = ((block + grid - g.proc_cur) % grid) / g.proc_s;
    Slot s;
    s.tid = threadIdx.x - k * slot_threads;
    s.nthreads = slot_threads;
    s.lds = (lds_ptr)g_loop_lds + kLdsReserved + k * g.slot_sram;
    s.lds_bytes = g.slot_sram;
    s.whole_block = (slot_threads == (int)blockDim.x);
    // Task ids fit 32 bits (the host rejects larger plans); 64-bit products only
    // where the formula could overflow before the range check.
    const int64_t base = g.task_b + (int64_t)p * g.task_s * g.gran;
    const int64_t round = (int64_t)g.task_s * g.gran * n_procs;  // id step per full deal
    int order = 0;
    for (unsigned t = (unsigned)k;; t += (unsigned)g.n_slots, ++order) {
        int64_t id;
        if (g.gran == 1) {
            id = base + round * t;
        } else {
            const unsigned q = t / (unsigned)g.gran, r = t - q * (unsigned)g.gran;
            id = base + (int64_t)g.task_s * r + round * q;
        }
        if (id >= g.task_e) break;
#ifndef ARKMI_NO_TRACE
        if (prog.trace && g.trace_offset >= 0 && s.tid == 0) {
            TraceRecord rec{block, k, order};
            prog.trace[g.trace_offset + (int)((id - g.task_b) / g.task_s)] = rec;
        }
#endif
        int follow = (int)id;  // uniform across the workgroup
        for (int o = 0; o < g.op_count && follow >= 0; ++o) {
            if (o > 0) {
                // later ops of a fused task read what earlier ones wrote: the stores
                // have reached the L2, and the L1 must not serve older copies
                s.sync();
                if (s.tid == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
                s.sync();
            }
            follow = run_op<FAM>(ops + o, follow, s);
        }
    }
}

template <int FAM>
__device__ __forceinline__ bool run_body(const LoopProgram &prog, LoopControl *ctl, XcdInfo &xi,
                                          uint64_t wait_ticks) {
    const bool clocked = prog.step_clock && threadIdx.x == 0;
    unsigned long long *clk = prog.step_clock + (size_t)blockIdx.x * (prog.num_steps + 1);
    for (int si = 0; si < prog.num_steps; ++si) {
        const DevStep st = load_const(prog.steps + si);
        if (clocked) clk[si] = wall_clock64();
        if (st.kind == STEP_BARRIER) {
            if ((unsigned)st.count == gridDim.x) {
                if (!grid_barrier_xcd(ctl, xi, wait_ticks)) return false;
            } else if (in_range(blockIdx.x, st.b, st.e, st.s)) {
                if (!grid_barrier(&ctl->bars[st.index], (unsigned)st.count, ctl, wait_ticks))
                    return false;
            }
        } else if (st.kind == STEP_LOCAL_SYNC) {
            // this workgroup's stores have reached the L2 it shares with nobody else
            // for these lines; drop what its L1 still holds of them
            __syncthreads();
            if (threadIdx.x == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            __syncthreads();
        } else {
            run_group<FAM>(prog, prog.groups + st.index);
        }
    }
    if (clocked) clk[prog.num_steps] = wall_clock64();
    return true;
}

template <int FAM>
__global__ __launch_bounds__(kLoopMaxThreads) void arkmi_loop_kernel(
    LoopProgram prog, LoopControl *ctl, HostMailbox *mb, int one_shot_iters, uint64_t idle_ticks,
    uint64_t wait_ticks) {
    const unsigned nblocks = gridDim.x;
    const bool leader = (blockIdx.x == 0 && threadIdx.x == 0);
    // count the workgroups per XCD (the control block is zeroed before every launch)
    XcdInfo xi;
    xi.epoch = 0;
    xi.x = xcc_id();
    if (threadIdx.x == 0) __hip_atomic_fetch_add(&ctl->xcd_blocks[xi.x], 1u, __ATOMIC_RELAXED, AGENT);
    if (!grid_barrier(&ctl->all, nblocks, ctl, wait_ticks)) {
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
    for (;;) {
        int iter;
        if (one_shot_iters > 0) {
            iter = one_shot_iters;
        } else {
            if (leader) {
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
            if (!grid_barrier_xcd(ctl, xi, wait_ticks)) break;
            iter = __hip_atomic_load(&ctl->iter, __ATOMIC_RELAXED, AGENT);
            if (iter < 0) {
                if (leader) {
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
                if (prog.iter_sync == 2) {
                    ok = grid_barrier_xcd(ctl, xi, wait_ticks);
                } else if (prog.iter_sync == 1) {
                    __syncthreads();
                    if (threadIdx.x == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
                    __syncthreads();
                }
            }
            if (ok) ok = run_body<FAM>(prog, ctl, xi, wait_ticks);
        }
        if (!ok) break;
        // results must be visible to the host before the command is cleared: every
        // wave's stores are in the L2 before thread 0's system-scope release
        drain_stores_then_barrier();
        if (threadIdx.x == 0) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
        if (!grid_barrier_xcd(ctl, xi, wait_ticks)) break;
        if (one_shot_iters > 0) return;
        if (leader) {
            __hip_atomic_store(&mb->done, mb->done + iter, __ATOMIC_RELAXED, SYSTEM);
            __hip_atomic_store(&mb->cmd, 0, __ATOMIC_RELEASE, SYSTEM);
        }
    }
    // a bounded wait expired somewhere: report and leave
    if (threadIdx.x == 0) {
        __hip_atomic_store(&mb->status, (int)MB_ABORTED, __ATOMIC_RELAXED, SYSTEM);
        if (blockIdx.x == 0) __hip_atomic_store(&mb->alive, 0, __ATOMIC_RELEASE, SYSTEM);
    }
}

// One task group as a kernel of its own (no loop, no barriers): the same op
// bodies launched the conventional way, one kernel per op, for comparison with
// the persistent loop kernel.
template <int FAM>
__global__ __launch_bounds__(kLoopMaxThreads) void arkmi_step_kernel(LoopProgram prog, int group) {
    run_group<FAM>(prog, prog.groups + group);
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
