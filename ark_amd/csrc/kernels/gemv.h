// Skinny matmul ("decode GEMV") for gfx950: Y[M,N] = X[M,K] . W[K,N] with
// M <= 16 rows, fp16 or bf16 operands, fp32 accumulate, one rounding to the
// storage type.  The work is reading W once, so the body is built around the
// HBM stream: W is fetched in its natural [K,N] layout with 128-bit loads,
// 512 contiguous bytes per row, and never re-read.
//
// The product runs on the matrix cores with the operands swapped,
// Y^T[n,m] = sum_k W^T[n,k] X^T[k,m], as v_mfma_f32_16x16x16: the 16 columns
// of the MFMA are the (zero-padded) rows of X, so M = 1 and M = 16 cost the
// same.  The MFMA wants 4 consecutive k per lane while W has n contiguous;
// each wave parks its 16 x 256 slab of W in a private LDS window and reads
// it back through ds_read_b64_tr_b16, which transposes on the way out.  (The
// depth-16 MFMA keeps a step at 8 loads per lane; the depth-32 one doubles the
// staging registers for no gain in a kernel that waits on HBM.)
//
// Work is cut stream-K style.  A unit is 256 columns x 128 rows of W (16 rows
// per wave, one MFMA step).  A workgroup streams stretches of consecutive units
// of one column block, the next unit's loads always in flight, also across the
// end of a stretch; at the end of a stretch the 8 waves add their tiles through
// LDS and either store Y (the stretch covered the block's whole K) or store an
// fp32 partial and count arrivals in an HBM-resident counter; the workgroup that
// arrives last adds the partials in the order of the parts (so the result does
// not depend on arrival order) and stores Y.  Who streams which stretch is the
// caller's matter (`Source`): the stand-alone op deals the units to T tasks in
// contiguous ranges, so with T = the number of CUs every CU streams the same
// number of bytes (+-1 unit) whatever the shape; the loop kernel works from the
// host's tables, or lets the workgroups claim stretches as they get free.
//
// The reference runs this shape through its general GEMM
// (ark/include/kernels/matmul.h:36-115) with a 128-row tile, 127/128 of it
// padding at batch 1.
#pragma once
#include "dev_common.h"
#include "gemm.h"

namespace arkmi {

struct GemvDesc {
    const void *x;   // [m, k], row pitch ldx
    const void *w;   // [k, n], row pitch ldw
    void *y;         // [m, n], row pitch ldy
    float *partial;  // [n_blocks][max_parts][m][256] fp32
    unsigned int *counters;  // [n_blocks], zero between uses
    int32_t m, n, k;
    int32_t ldx, ldw, ldy;
    int32_t n_blocks;   // ceil(n / 256)
    int32_t k_units;    // ceil(k / 128): units per column block
    int32_t num_tasks;  // T <= n_blocks * k_units
    int32_t max_parts;  // most tasks that share one column block
    int32_t dtype;      // 1 fp16, 2 bf16
};

typedef float f32x4 __attribute__((ext_vector_type(4)));
using lds_f32x4 = __attribute__((address_space(3))) f32x4;
using lds_f32 = __attribute__((address_space(3))) float;
using lds_i32 = __attribute__((address_space(3))) int;

typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

template <typename T>
__device__ __forceinline__ f32x4 mfma16(u32x2 a, u32x2 b, f32x4 c);
template <>
__device__ __forceinline__ f32x4 mfma16<f16>(u32x2 a, u32x2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a),
                                                 __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4 mfma16<bf16>(u32x2 a, u32x2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a),
                                                     __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
}

constexpr int kGemvCols = 256;   // columns per unit
constexpr int kGemvStepK = 16;   // rows of W per wave per unit (one MFMA depth)
constexpr int kGemvWaves = 8;
constexpr int kGemvUnitK = kGemvStepK * kGemvWaves;  // rows per unit
constexpr int kGemvRowBytes = kGemvCols * 2 + 32;  // LDS pitch of a staged W row
constexpr int kGemvStageBytes = kGemvStepK * kGemvRowBytes;           // per wave
constexpr int kGemvRedPitch = kGemvCols + 4;                          // floats
constexpr int kGemvRedBytes = 16 * kGemvRedPitch * 4;                 // per wave
constexpr int kGemvWaveBytes = kGemvStageBytes > kGemvRedBytes ? kGemvStageBytes : kGemvRedBytes;
constexpr int kGemvLdsBytes = 64 + kGemvWaves * kGemvWaveBytes;

inline size_t gemv_counter_bytes(int n_blocks) { return 256 * (((size_t)n_blocks * 4 + 255) / 256); }

// First unit of task t, and the task that owns unit u (its inverse), for U
// units dealt to T <= U tasks.
__host__ __device__ inline int64_t gemv_task_begin(int64_t t, int64_t U, int64_t T) { return t * U / T; }
__host__ __device__ inline int64_t gemv_task_of(int64_t u, int64_t U, int64_t T) {
    return ((u + 1) * T - 1) / U;
}

// Fills the partition fields of a descriptor whose m, n, k are set, for
// `tasks` tasks (clamped to the number of units); returns the bytes of
// workspace (counters, then partials) the op needs.
inline size_t gemv_partition(GemvDesc &d, int tasks) {
    d.n_blocks = (d.n + kGemvCols - 1) / kGemvCols;
    d.k_units = (d.k + kGemvUnitK - 1) / kGemvUnitK;
    const int64_t U = (int64_t)d.n_blocks * d.k_units;
    d.num_tasks = (int)(tasks < 1 ? 1 : (tasks > U ? U : tasks));
    d.max_parts = 1;
    for (int nb = 0; nb < d.n_blocks; ++nb) {
        const int parts = (int)(gemv_task_of((int64_t)(nb + 1) * d.k_units - 1, U, d.num_tasks) -
                                gemv_task_of((int64_t)nb * d.k_units, U, d.num_tasks)) + 1;
        if (parts > d.max_parts) d.max_parts = parts;
    }
    return gemv_counter_bytes(d.n_blocks) +
           (size_t)d.n_blocks * d.max_parts * d.m * kGemvCols * sizeof(float);
}

// A stretch of consecutive units inside one column block: what a workgroup streams in one go and
// folds at the end.  The host cuts every skinny matmul of a plan into these and lays out who
// streams which.  `op < 0` ends a sequence.
struct GemvSeqEntry {
    int32_t op;
    int32_t nb, ku;       // first unit: column block, K-chunk inside it
    int32_t units;        // > 0, all inside block nb
    int32_t part, parts;  // the block's K is covered by `parts` stretches; this is number `part`
    int32_t trace_index;  // where the trace record of the stretch's task goes, -1: nowhere
    int32_t order;        // the task's number on its workgroup within its group
};

// Where a workgroup is in the units it has to stream.  Two of these walk the same sequence of
// stretches, the one that issues loads two units ahead of the one that multiplies.  `Source`
// hands out the stretches: `next(d, nb, ku, units, part, parts)` (false at the end); the fold at
// the end of a stretch calls its `fold_begins(tid)` and `fold_ends(tid)`.
template <typename Source>
struct GemvCursor {
    Source src;
    GemvDesc d;
    int nb = 0, ku = 0;  // the current unit
    int left = 0;        // units of the current stretch still to go, this one included; 0: the end
    int part = 0, parts = 1;
    __device__ __forceinline__ explicit GemvCursor(const Source &s) : src(s) {}
};

// Streams a sequence of stretches through one workgroup.  Between two stretches the loads never
// stop: while one is added up across the waves and stored, the first two units of the next one
// (of the same matmul or the next) are already in flight.
template <typename T, typename Source>
__device__ __forceinline__ void gemv_stream(const Slot &s, const Source &source) {
    const int tid = s.tid, lane = tid & 63, wave = tid >> 6;

    lds_i32 *flag = (lds_i32 *)s.lds;
    const lds_ptr wlds = s.lds + 64 + wave * kGemvWaveBytes;

    // global -> registers: instruction i fetches rows 2i and 2i+1 of the wave's
    // 16, lanes 0-31 the first, lanes 32-63 the second, 8 columns per lane
    const int lrow = lane >> 5, lcol = (lane & 31) * 8;
    const int wdst = lrow * kGemvRowBytes + lcol * 2;

    // X fragment (B operand): lane holds x[m = lane%16][k = k0 + (lane/16)*4 .. +3]
    const int xm = lane & 15, xk = (lane >> 4) * 4;

    // W^T fragment (A operand) through the transposing read: inside each block
    // of 16 lanes (one k-group of 4), lane i supplies the address of 4
    // consecutive n at row i/4 and receives 4 consecutive k of column i
    const int i16 = lane & 15;
    const int wfrag = ((lane >> 4) * 4 + (i16 >> 2)) * kGemvRowBytes + (i16 & 3) * 8;

    using Cursor = GemvCursor<Source>;
    auto seek = [&](Cursor &c) {  // to the first unit of the next stretch
        if (!c.src.next(c.d, c.nb, c.ku, c.left, c.part, c.parts)) c.left = 0;
    };
    auto advance = [&](Cursor &c) {
        if (--c.left <= 0) seek(c);
        else ++c.ku;
    };

    constexpr int NG = kGemvCols / 16;  // 16 MFMA tiles per wave
    f32x4 acc[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};

    constexpr int NLD = kGemvStepK / 2;  // load instructions per unit
    // two units are kept in flight per wave (16 KB), in two register sets
    u32x4 stage_a[NLD], stage_b[NLD];
    u32x2 x_a, x_b;
    auto gload = [&](const Cursor &c, u32x4(&stage)[NLD], u32x2 &xf) {
        const GemvDesc &d = c.d;
        gptr<const T> W = as_global(static_cast<const T *>(d.w));
        gptr<const T> xsrc = as_global(static_cast<const T *>(d.x)) + (int64_t)xm * d.ldx + xk;
        const int nb = c.nb, ku = c.ku;
        const int k0 = ku * kGemvUnitK + wave * kGemvStepK;  // this wave's first row
        // Loads are unconditional: a column past N is clamped to the last
        // vector of the row (its products are never stored) and a row past K to
        // the last row, whose values are then replaced by zeros.
        const int col = min(nb * kGemvCols + lcol, d.n - 8);  // n is a multiple of 8
        const int row0 = k0 + lrow;
        gptr<const T> src = W + col;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int row = row0 + 2 * i;
            u32x4 v = __builtin_nontemporal_load(
                (const ARKMI_GLOBAL u32x4 *)(src + (int64_t)min(row, d.k - 1) * d.ldw));
            if (row >= d.k) v = u32x4{0u, 0u, 0u, 0u};
            stage[i] = v;
        }
        u32x2 xv{0u, 0u};
        if (xm < d.m) {
            // the last k-group of a ragged K may reach past the row: fetch by element
            if (k0 + xk + 4 <= d.k) {
                xv = *(const ARKMI_GLOBAL u32x2 *)(xsrc + k0);
            } else {
                uint16_t e[4];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    e[j] = (k0 + xk + j < d.k) ? *((gptr<const uint16_t>)(xsrc + k0) + j) : (uint16_t)0;
                __builtin_memcpy(&xv, e, 8);
            }
        }
        xf = xv;
    };

    Cursor L(source);  // loads run two units ahead of the products
    seek(L);
    if (L.left <= 0) return;
    Cursor C = L;
    gload(L, stage_a, x_a);
    advance(L);
    if (L.left > 0) {
        gload(L, stage_b, x_b);
        advance(L);
    }
    // One unit: park it in LDS, refill its register set with the unit after
    // next, multiply, and fold the tiles when the column block is left.
    auto consume = [&](u32x4(&stage)[NLD], u32x2 &xf) {
        // only this wave touches its window, and LDS serves one wave's requests
        // in order, so a wave-level fence is enough
#pragma unroll
        for (int i = 0; i < NLD; ++i)
            *(lds_u32x4 *)(wlds + wdst + 2 * i * kGemvRowBytes) = stage[i];
        const u32x2 xcur = xf;
        if (L.left > 0) {
            gload(L, stage, xf);
            advance(L);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // four transposed reads, then their four MFMAs: deep enough to cover the
        // LDS latency without spending the registers the loads in flight need
#pragma unroll
        for (int g0 = 0; g0 < NG; g0 += 4) {
            s16x4 wt[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                wt[i] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(wlds + wfrag + (g0 + i) * 32));
#pragma unroll
            for (int i = 0; i < 4; ++i)
                acc[g0 + i] = mfma16<T>(__builtin_bit_cast(u32x2, wt[i]), xcur, acc[g0 + i]);
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        if (C.left > 1) return;

        // ---- end of a stretch: add the 8 waves' tiles through LDS ------------------------
        // accumulator layout of 16x16x16: lane holds column (lane%16) = m and rows
        // 4*(lane/16) + r = n inside the tile
        const GemvDesc &d = C.d;
        const int nb = C.nb;
        gptr<T> Y = as_global(static_cast<T *>(d.y));
        s.sync();  // every wave is done with its staging window
        C.src.fold_begins(tid);
        {
            lds_f32 *red = (lds_f32 *)wlds;
            const int m = lane & 15, nq = (lane >> 4) * 4;
            const bool live = m < d.m;  // (the other lanes hold products of X's zero padding)
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                if (live) *(lds_f32x4 *)(red + m * kGemvRedPitch + g * 16 + nq) = acc[g];
                acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
        s.sync();
        // a thread adds up four consecutive columns of one row (a wave one row of the block, the
        // workgroup eight rows at a time) over the eight waves' windows
        const int c4 = (tid & 63) * 4, mrow = tid >> 6;
        const int col = nb * kGemvCols + c4;  // n is a multiple of 8: col < n means col + 4 <= n
        f32x4 sums[2];
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            const int m = mrow + 8 * pass;
            f32x4 v{0.f, 0.f, 0.f, 0.f};
            if (m < d.m) {
#pragma unroll
                for (int w = 0; w < kGemvWaves; ++w)
                    v += *(const lds_f32x4 *)(s.lds + 64 + w * kGemvWaveBytes + (m * kGemvRedPitch + c4) * 4);
            }
            sums[pass] = v;
        }
        const bool vec_ok = ((d.ldy & 3) == 0) && (((uintptr_t)d.y & 7) == 0);
        auto store_y = [&](int m, f32x4 v) {
            gptr<T> p = Y + (int64_t)m * d.ldy + col;
            T o[4] = {from_f32<T>(v[0]), from_f32<T>(v[1]), from_f32<T>(v[2]), from_f32<T>(v[3])};
            if (vec_ok) {
                u32x2 w;
                __builtin_memcpy(&w, o, 8);
                *(ARKMI_GLOBAL u32x2 *)p = w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) p[e] = o[e];
            }
        };
        if (C.parts == 1) {
            if (col < d.n) {
#pragma unroll
                for (int pass = 0; pass < 2; ++pass) {
                    const int m = mrow + 8 * pass;
                    if (m < d.m) store_y(m, sums[pass]);
                }
            }
        } else {
            // K of this block is shared with other stretches: partial + arrival counter.
            // Partials travel as 16-byte buffer stores and loads with the agent-scope
            // bit (written through to memory, read past this XCD's L2), so no
            // cache-wide write-back or invalidate is needed: those are serialised
            // per L2 and cost more than the op itself when every task issues them.
            // Ordering: every wave waits for its stores to be acknowledged (vmcnt 0)
            // before the workgroup barrier, the counter is bumped after it, and the
            // partials are read only after the counter has been seen full.
            constexpr int kAgentScope = 16;  // cache-policy bit sc1 of the buffer instructions
            const int parts = C.parts;
            const int part_bytes = d.m * kGemvCols * 4;
            float *Pb = d.partial + (int64_t)nb * d.max_parts * d.m * kGemvCols;
            const __amdgpu_buffer_rsrc_t rsrc =
                __builtin_amdgcn_make_buffer_rsrc(Pb, 0, d.max_parts * part_bytes, 0x00020000);
#pragma unroll
            for (int pass = 0; pass < 2; ++pass) {
                const int m = mrow + 8 * pass;
                if (m < d.m)
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, sums[pass]), rsrc,
                                                           C.part * part_bytes + (m * kGemvCols + c4) * 4,
                                                           0, kAgentScope);
            }
            drain_stores_then_barrier();
            if (tid == 0) {
                const unsigned prev = __hip_atomic_fetch_add(d.counters + nb, 1u, __ATOMIC_RELAXED,
                                                             __HIP_MEMORY_SCOPE_AGENT);
                *flag = (prev == (unsigned)parts - 1u) ? 1 : 0;
            }
            s.sync();
            if (*flag) {
                if (col < d.n) {
#pragma unroll
                    for (int pass = 0; pass < 2; ++pass) {
                        const int m = mrow + 8 * pass;
                        if (m < d.m) {
                            // eight loads in flight per row (the accumulator registers are
                            // free here), added in the order of the parts
                            constexpr int kInFlight = 8;
                            f32x4 v{0.f, 0.f, 0.f, 0.f};
                            for (int q0 = 0; q0 < parts; q0 += kInFlight) {
                                u32x4 t[kInFlight];
#pragma unroll
                                for (int i = 0; i < kInFlight; ++i)
                                    t[i] = (q0 + i < parts)
                                               ? __builtin_amdgcn_raw_buffer_load_b128(
                                                     rsrc, (q0 + i) * part_bytes + (m * kGemvCols + c4) * 4, 0,
                                                     kAgentScope)
                                               : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
                                for (int i = 0; i < kInFlight; ++i)
                                    if (q0 + i < parts) v += __builtin_bit_cast(f32x4, t[i]);
                            }
                            store_y(m, v);
                        }
                    }
                }
                if (tid == 0)
                    __hip_atomic_store(d.counters + nb, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        C.src.fold_ends(tid);
        s.sync();  // the windows (and the flag) are reused by the next stretch
    };
    for (;;) {
        consume(stage_a, x_a);
        advance(C);
        if (C.left <= 0) break;
        consume(stage_b, x_b);
        advance(C);
        if (C.left <= 0) break;
    }
}

// The stretches of the tasks first, first + stride, ... < end of one skinny matmul whose units are
// dealt to d.num_tasks tasks in contiguous ranges (gemv_partition): a task's range, cut at the
// column-block boundaries.
struct GemvTaskSource {
    const GemvDesc *d;
    int t, stride, end;
    int u = 0, u_end = 0;
    __device__ __forceinline__ GemvTaskSource(const GemvDesc *desc, int first, int step, int last)
        : d(desc), t(first - step), stride(step), end(last) {}
    __device__ __forceinline__ bool next(GemvDesc &out, int &nb, int &ku, int &units, int &part, int &parts) {
        const int64_t U = (int64_t)d->n_blocks * d->k_units;
        while (u >= u_end) {
            t += stride;
            if (t >= end) return false;
            u = (int)gemv_task_begin(t, U, d->num_tasks);
            u_end = (int)gemv_task_begin(t + 1, U, d->num_tasks);
        }
        out = *d;
        nb = u / d->k_units;
        ku = u - nb * d->k_units;
        units = min(u_end - u, d->k_units - ku);
        const int t_first = (int)gemv_task_of((int64_t)nb * d->k_units, U, d->num_tasks);
        const int t_last = (int)gemv_task_of((int64_t)(nb + 1) * d->k_units - 1, U, d->num_tasks);
        part = t - t_first;
        parts = t_last - t_first + 1;
        u += units;
        return true;
    }
    __device__ __forceinline__ void fold_begins(int) {}
    __device__ __forceinline__ void fold_ends(int) {}
};

template <typename T>
__device__ __forceinline__ void gemv_tasks(const GemvDesc &d, int first, int stride, int end, const Slot &s) {
    gemv_stream<T>(s, GemvTaskSource(&d, first, stride, end));
}

}  // namespace arkmi
