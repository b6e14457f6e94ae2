// Row-wise ops over the last axis: reduce_{sum,max,mean}, softmax, layernorm,
// RMSNorm.  One wavefront owns one row: 64 lanes x 16-byte loads are fully
// coalesced (1 KiB per wave instruction), the row is held in registers so HBM
// sees one read and (for the normalising ops) one write, accumulation is fp32,
// and the cross-lane step is a wave64 DPP reduction.
//
// Replaces ark/include/kernels/reduce.h:341-444 (WwiseReduce, storage-dtype
// accumulation, one wave per CU) and the multi-op compositions
// python/ark/ops.py:491-513 and examples/llama/model.py:92-99.
#pragma once
#include <type_traits>

#include "dev_common.h"

namespace arkmi {

enum RowKind : int32_t {
    ROW_SUM = 0,
    ROW_MAX = 1,
    ROW_MEAN = 2,
    ROW_SOFTMAX = 3,
    ROW_LAYERNORM = 4,
    ROW_RMSNORM = 5,
};

// Rows are the (n, c, h) positions of a 4-D tensor whose last axis is dense.
struct RowOpDesc {
    const void *in;
    void *out;
    const void *weight;   // RMSNorm scale, length cols; softmax: additive mask (may be null)
    int64_t rows;         // N * C * H
    int32_t cols;         // W
    int32_t dim_c, dim_h;
    int32_t rows_per_wave;  // rows a wave handles per task (0 and 1: one)
    int64_t in_s[3];      // element strides of n, c, h in the input
    int64_t out_s[3];     // element strides of n, c, h in the output
    float eps;
    int32_t kind;
    int32_t dtype;        // 0 fp32, 1 fp16, 2 bf16
    int32_t weight_fp32;  // 1: weight is float, 0: weight has the tensor dtype
    // softmax(x * scale + mask): the mask has the tensor dtype and these element
    // strides of n, c, h (0 where it broadcasts); its rows are dense
    int64_t w_s[3];
    float scale;
    int32_t prescale;     // 1: scale and/or mask are applied before the softmax
    int32_t weight_lds;   // RMSNorm with several rows per wave: the fp32 weights are staged in the slot's LDS
    // Reduction over an axis other than the last (red_len > 0): rows, dim_c, dim_h and
    // cols describe the OUTPUT (the reduced axis has extent 1), one output per thread,
    // which walks red_len inputs red_stride elements apart.
    int32_t red_len;
    int64_t red_stride;
    // 1: a later op of the plan reads the input again (before anything overwrites it): fetch it
    // through the caches instead of streaming past them
    int32_t in_read_again;
    // The row op that runs next on the same workgroups with the same dealing of rows (the host knows;
    // pf_base null: none): while a wave finishes its last row of this task it touches the lines of
    // its first row of that op, pf_base + first row * pf_row_bytes, pf_len bytes, so that the next
    // task's first loads, which nothing overlaps, find them in the L2.
    int32_t pf_len;
    const void *pf_base;
    int64_t pf_row_bytes;
};

__device__ __forceinline__ int64_t row_offset(int64_t r, int dim_c, int dim_h,
                                              const int64_t s[3]) {
    // row counts fit 32 bits (checked on the host): 32-bit division is an
    // order of magnitude cheaper than the 64-bit sequence
    const unsigned ru = (unsigned)r;
    const unsigned t = ru / (unsigned)dim_h, h = ru - t * (unsigned)dim_h;
    const unsigned n = t / (unsigned)dim_c, c = t - n * (unsigned)dim_c;
    return (int64_t)n * s[0] + (int64_t)c * s[1] + (int64_t)h * s[2];
}

// ---------------------------------------------------------------------------
// Per-element arithmetic shared by the three code paths below.
// ---------------------------------------------------------------------------
template <int KIND>
struct RowMath {
    static constexpr bool IS_REDUCE = (KIND == ROW_SUM || KIND == ROW_MAX || KIND == ROW_MEAN);
    static constexpr bool IS_MAX = (KIND == ROW_MAX || KIND == ROW_SOFTMAX);
    __device__ static __forceinline__ float init() { return IS_MAX ? -3.402823466e+38f : 0.f; }
    __device__ static __forceinline__ float acc1(float acc, float x) {
        if (IS_MAX) return fmaxf(acc, x);
        if (KIND == ROW_RMSNORM) return acc + x * x;
        return acc + x;
    }
    __device__ static __forceinline__ float wave1(float acc) {
        return IS_MAX ? wave_allreduce(acc, OpMax()) : wave_allreduce(acc, OpSum());
    }
    // second statistic: softmax denominator / layernorm variance
    __device__ static __forceinline__ float acc2(float acc, float x, float s1) {
        if (KIND == ROW_SOFTMAX) return acc + __expf(x - s1);
        float dlt = x - s1;
        return acc + dlt * dlt;
    }
};

template <typename T>
__device__ __forceinline__ void load_weight(const RowOpDesc &d, int idx, float (&w)[Vec16<T>::N]) {
    constexpr int VN = Vec16<T>::N;
    if (d.weight_fp32) {
        gptr<const float> wp = as_global(static_cast<const float *>(d.weight) + idx);
#pragma unroll
        for (int j = 0; j < VN; ++j) w[j] = wp[j];
    } else {
        gptr<const T> wp = as_global(static_cast<const T *>(d.weight) + idx);
#pragma unroll
        for (int j = 0; j < VN; ++j) w[j] = to_f32(wp[j]);
    }
}

// ---------------------------------------------------------------------------
// Path 1: the row is exactly NC full chunks (64 lanes x 16 B each) and 16-byte
// aligned, and fits in at most 64 fp32 registers per lane.  Straight-line
// code: all NC loads are issued back to back, the row is widened to fp32 once
// and stays in registers for every pass.
// ---------------------------------------------------------------------------
// Softmax input transform x * scale + mask[idx..] on one vector of values.
template <typename T>
__device__ __forceinline__ void softmax_pre(gptr<const T> mask, float scale, int idx, float (&x)[Vec16<T>::N]) {
    constexpr int VN = Vec16<T>::N;
    if (mask) {
        Vec16<T> mv = load16<T>(mask + idx);
#pragma unroll
        for (int j = 0; j < VN; ++j) x[j] = x[j] * scale + to_f32(mv.v[j]);
    } else {
#pragma unroll
        for (int j = 0; j < VN; ++j) x[j] *= scale;
    }
}

// `again`: another op of the plan reads this input after this one (the host knows): the row is
// then fetched with ordinary loads and stays in the caches for that op; a row that nobody reads
// again streams past them.  (Three row ops over one 128 MiB X: 456 us with the first two reading
// X this way against 512 us with all three streaming; one op over four such tensors is 3-8 %
// faster streaming.)
template <typename T, int NC>
__device__ __forceinline__ void row_exact_load(gptr<const T> in, int lane, Vec16<T> (&reg)[NC], bool again = false) {
    constexpr int VN = Vec16<T>::N;
    if (again) {
#pragma unroll
        for (int c = 0; c < NC; ++c) reg[c] = load16<T>(in + c * (kWave * VN) + lane * VN);
    } else {
        // (the empty statements keep the compiler from merging the two branches' loads into one
        // set of ordinary loads: merged instructions lose the streaming hint)
        asm volatile("" ::: "memory");
#pragma unroll
        for (int c = 0; c < NC; ++c) reg[c] = load16_nt<T>(in + c * (kWave * VN) + lane * VN);
        asm volatile("" ::: "memory");
    }
}

// Everything after the loads: `reg` holds the row as it was fetched.
// RMSNorm weights: `w_lds` (fp32, staged in LDS by the task), else `w_reg` (of the tensor's
// type, fetched once per task into registers), else loaded from memory chunk by chunk.
// (`w_reg`: per chunk the lane's VN weights, as Vec16<T> or as fp32 values)
template <int N>
struct F32Vec {
    float v[N];
};
template <typename T, int KIND, int NC, typename WReg>
__device__ __forceinline__ void row_exact_finish(const RowOpDesc &d, const Vec16<T> (&reg)[NC], gptr<T> out,
                                                 int lane, gptr<const T> mask, lds_ptr w_lds,
                                                 const WReg (&w_reg)[NC], bool w_in_regs) {
    using M = RowMath<KIND>;
    constexpr int VN = Vec16<T>::N;
    constexpr int PER_CHUNK = kWave * VN;
    static_assert(NC * VN <= 64, "row does not fit the register budget");
    const int cols = NC * PER_CHUNK;
    float x[NC][VN];
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int j = 0; j < VN; ++j) x[c][j] = to_f32(reg[c].v[j]);
    if (KIND == ROW_SOFTMAX && d.prescale) {
#pragma unroll
        for (int c = 0; c < NC; ++c) softmax_pre<T>(mask, d.scale, c * PER_CHUNK + lane * VN, x[c]);
    }
    float acc = M::init();
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int j = 0; j < VN; ++j) acc = M::acc1(acc, x[c][j]);
    acc = M::wave1(acc);
    if (M::IS_REDUCE) {
        if (KIND == ROW_MEAN) acc /= (float)cols;
        if (lane == 0) out[0] = from_f32<T>(acc);
        return;
    }
    float scale;
    if (KIND == ROW_RMSNORM) {
        scale = 1.0f / sqrtf(acc / (float)cols + d.eps);
    } else {
        const float s1 = (KIND == ROW_SOFTMAX) ? acc : acc / (float)cols;
        float a2 = 0.f;
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int j = 0; j < VN; ++j) {
                // keep exp(x - max) / (x - mean) for the output pass
                x[c][j] = (KIND == ROW_SOFTMAX) ? __expf(x[c][j] - s1) : x[c][j] - s1;
                a2 += (KIND == ROW_SOFTMAX) ? x[c][j] : x[c][j] * x[c][j];
            }
        a2 = wave_allreduce(a2, OpSum());
        scale = (KIND == ROW_SOFTMAX) ? 1.0f / a2 : 1.0f / sqrtf(a2 / (float)cols + d.eps);
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int idx = c * PER_CHUNK + lane * VN;
        Vec16<T> o;
        if (KIND == ROW_RMSNORM && d.weight) {
            float w[VN];
            if (w_lds) {
                // fp32 weights staged by the task: VN floats from LDS
                typedef float row_f4 __attribute__((ext_vector_type(4)));
                using lds_f4 = __attribute__((address_space(3))) const row_f4;
#pragma unroll
                for (int q = 0; q < VN / 4; ++q) {
                    const row_f4 v = *(lds_f4 *)(w_lds + (idx + 4 * q) * 4);
                    w[4 * q] = v.x; w[4 * q + 1] = v.y; w[4 * q + 2] = v.z; w[4 * q + 3] = v.w;
                }
            } else if (w_in_regs) {
#pragma unroll
                for (int j = 0; j < VN; ++j) w[j] = to_f32(w_reg[c].v[j]);  // (identity for fp32 weights)
            } else {
                load_weight<T>(d, idx, w);
            }
#pragma unroll
            for (int j = 0; j < VN; ++j) o.v[j] = from_f32<T>(x[c][j] * scale * w[j]);
        } else {
#pragma unroll
            for (int j = 0; j < VN; ++j) o.v[j] = from_f32<T>(x[c][j] * scale);
        }
        store16_nt<T>(out + idx, o);
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <typename T, int KIND, int NC>
__device__ __forceinline__ void row_op_exact(const RowOpDesc &d, gptr<const T> in, gptr<T> out, int lane,
                                             gptr<const T> mask) {
    Vec16<T> reg[NC];
    row_exact_load<T, NC>(in, lane, reg);
    // Every load is issued before the first value is consumed: without
    // this fence the scheduler may pull a conversion of chunk 0 between
    // the loads, and the wave then waits a full memory round trip with only
    // half of its loads in flight.
    __builtin_amdgcn_sched_barrier(0);
    row_exact_finish<T, KIND, NC>(d, reg, out, lane, mask, nullptr, reg, false);
}

// ---------------------------------------------------------------------------
// Path 2: any length that is a multiple of the vector width, 16-byte aligned.
// Streams the row once per pass with 16-byte loads; passes after the first hit
// L2 (a row is a few KiB), so HBM still sees one read and one write.
// ---------------------------------------------------------------------------
template <typename T, int KIND>
__device__ __forceinline__ void row_op_vec(const RowOpDesc &d, gptr<const T> in, gptr<T> out, int lane,
                                           gptr<const T> mask) {
    using M = RowMath<KIND>;
    constexpr int VN = Vec16<T>::N;
    constexpr int PER_CHUNK = kWave * VN;
    const int cols = d.cols;
    const bool pre = (KIND == ROW_SOFTMAX) && d.prescale;
    // the row's values at idx, widened (and transformed, for a scaled / masked softmax)
    auto fetch = [&](int idx, float (&x)[VN]) {
        Vec16<T> v = load16<T>(in + idx);
#pragma unroll
        for (int j = 0; j < VN; ++j) x[j] = to_f32(v.v[j]);
        if (pre) softmax_pre<T>(mask, d.scale, idx, x);
    };
    float acc = M::init();
    for (int idx = lane * VN; idx < cols; idx += PER_CHUNK) {
        float x[VN];
        fetch(idx, x);
#pragma unroll
        for (int j = 0; j < VN; ++j) acc = M::acc1(acc, x[j]);
    }
    acc = M::wave1(acc);
    if (M::IS_REDUCE) {
        if (KIND == ROW_MEAN) acc /= (float)cols;
        if (lane == 0) out[0] = from_f32<T>(acc);
        return;
    }
    float shift = 0.f, scale;
    if (KIND == ROW_RMSNORM) {
        scale = 1.0f / sqrtf(acc / (float)cols + d.eps);
    } else {
        const float s1 = (KIND == ROW_SOFTMAX) ? acc : acc / (float)cols;
        float a2 = 0.f;
        for (int idx = lane * VN; idx < cols; idx += PER_CHUNK) {
            float x[VN];
            fetch(idx, x);
#pragma unroll
            for (int j = 0; j < VN; ++j) a2 = M::acc2(a2, x[j], s1);
        }
        a2 = wave_allreduce(a2, OpSum());
        shift = s1;
        scale = (KIND == ROW_SOFTMAX) ? 1.0f / a2 : 1.0f / sqrtf(a2 / (float)cols + d.eps);
    }
    // In-place use is safe: all statistics are complete (the wave reductions
    // above are convergence points) and each lane re-reads only what it
    // overwrites itself.
    for (int idx = lane * VN; idx < cols; idx += PER_CHUNK) {
        float xv[VN];
        fetch(idx, xv);
        Vec16<T> o;
        float w[VN];
#pragma unroll
        for (int j = 0; j < VN; ++j) w[j] = 1.f;
        if (KIND == ROW_RMSNORM && d.weight) load_weight<T>(d, idx, w);
#pragma unroll
        for (int j = 0; j < VN; ++j) {
            float x = xv[j];
            o.v[j] = from_f32<T>(KIND == ROW_SOFTMAX ? __expf(x - shift) * scale
                                                     : (x - shift) * scale * w[j]);
        }
        store16<T>(out + idx, o);
    }
}

// ---------------------------------------------------------------------------
// Path 3: any length / alignment, element by element.
// ---------------------------------------------------------------------------
template <typename T, int KIND>
__device__ __forceinline__ void row_op_scalar(const RowOpDesc &d, gptr<const T> in, gptr<T> out, int lane,
                                              gptr<const T> mask) {
    using M = RowMath<KIND>;
    const int cols = d.cols;
    const bool pre = (KIND == ROW_SOFTMAX) && d.prescale;
    auto fetch = [&](int i) {
        float x = to_f32(in[i]);
        if (pre) x = mask ? x * d.scale + to_f32(mask[i]) : x * d.scale;
        return x;
    };
    float acc = M::init();
    for (int i = lane; i < cols; i += kWave) acc = M::acc1(acc, fetch(i));
    acc = M::wave1(acc);
    if (M::IS_REDUCE) {
        if (KIND == ROW_MEAN) acc /= (float)cols;
        if (lane == 0) out[0] = from_f32<T>(acc);
        return;
    }
    float shift = 0.f, scale;
    if (KIND == ROW_RMSNORM) {
        scale = 1.0f / sqrtf(acc / (float)cols + d.eps);
    } else {
        const float s1 = (KIND == ROW_SOFTMAX) ? acc : acc / (float)cols;
        float a2 = 0.f;
        for (int i = lane; i < cols; i += kWave) a2 = M::acc2(a2, fetch(i), s1);
        a2 = wave_allreduce(a2, OpSum());
        shift = s1;
        scale = (KIND == ROW_SOFTMAX) ? 1.0f / a2 : 1.0f / sqrtf(a2 / (float)cols + d.eps);
    }
    for (int i = lane; i < cols; i += kWave) {
        float x = fetch(i);
        float y;
        if (KIND == ROW_SOFTMAX) {
            y = __expf(x - shift) * scale;
        } else {
            float w = 1.f;
            if (KIND == ROW_RMSNORM && d.weight)
                w = d.weight_fp32 ? as_global(static_cast<const float *>(d.weight))[i]
                                  : to_f32(as_global(static_cast<const T *>(d.weight))[i]);
            y = (x - shift) * scale * w;
        }
        out[i] = from_f32<T>(y);
    }
}

template <typename T, int KIND>
__device__ __forceinline__ void row_op_wave(const RowOpDesc &d, int64_t row, int lane) {
    constexpr int VN = Vec16<T>::N;
    constexpr int PER_CHUNK = kWave * VN;
    constexpr bool IS_REDUCE = RowMath<KIND>::IS_REDUCE;
    const int cols = d.cols;
    gptr<const T> in = as_global(static_cast<const T *>(d.in) + row_offset(row, d.dim_c, d.dim_h, d.in_s));
    gptr<T> out = as_global(static_cast<T *>(d.out) + row_offset(row, d.dim_c, d.dim_h, d.out_s));
    gptr<const T> mask = nullptr;
    if (KIND == ROW_SOFTMAX && d.weight)
        mask = as_global(static_cast<const T *>(d.weight) + row_offset(row, d.dim_c, d.dim_h, d.w_s));
    const bool w_ok = (KIND == ROW_RMSNORM && d.weight) ? aligned16(d.weight) : (!mask || aligned16(mask));
    const bool vec_ok = (cols % VN == 0) && aligned16(in) && (IS_REDUCE || aligned16(out)) && w_ok;
    if (!vec_ok) return row_op_scalar<T, KIND>(d, in, out, lane, mask);
    // rows of 1, 2, 4, ... full chunks (up to 4096 elements) take the
    // register-resident path
    constexpr int MAXNC = 64 / VN;
    if (cols == 1 * PER_CHUNK) return row_op_exact<T, KIND, 1>(d, in, out, lane, mask);
    if (cols == 2 * PER_CHUNK) return row_op_exact<T, KIND, 2>(d, in, out, lane, mask);
    if (cols == 4 * PER_CHUNK) return row_op_exact<T, KIND, 4>(d, in, out, lane, mask);
    if (cols == 8 * PER_CHUNK) return row_op_exact<T, KIND, 8>(d, in, out, lane, mask);
    if (MAXNC >= 16 && cols == 16 * PER_CHUNK)
        return row_op_exact<T, KIND, (MAXNC >= 16 ? 16 : 8)>(d, in, out, lane, mask);
    return row_op_vec<T, KIND>(d, in, out, lane, mask);
}

// The register-resident rows of one wave for one task: the next row's loads are in
// flight while the current one is reduced and stored.  With `stage`, the task's
// fp32 RMSNorm weights (the same cols floats for every row) are first copied to
// the slot's LDS, and read from there: the copy is issued ahead of the first row's
// loads and written to LDS while those are still in flight.  `stage` and the choice
// of this path depend on the descriptor only, so every wave of the slot runs the
// barriers below, also a wave that has no row (count 0).
template <typename T, int KIND, int NC>
__device__ __forceinline__ void row_op_pipelined(const RowOpDesc &d, int64_t row0, int stride, int count,
                                                 const Slot &s, bool stage) {
    constexpr int VN = Vec16<T>::N;
    constexpr int NVEC = NC * kWave * VN / 4;  // 16-byte vectors in the fp32 weights
    constexpr int WV = (NVEC + 511) / 512;     // per thread of a 512-thread slot
    typedef uint32_t row_u4 __attribute__((ext_vector_type(4)));
    using l_u4 = __attribute__((address_space(3))) row_u4;
    const int lane = s.lane();
    const bool in_regs = stage && s.nthreads == 512;
    row_u4 wv[WV];
    if (stage) {
        s.sync();  // readers of the previous task's copy are done
        if (in_regs) {
#pragma unroll
            for (int u = 0; u < WV; ++u)
                if (s.tid + u * 512 < NVEC) wv[u] = ((const ARKMI_GLOBAL row_u4 *)d.weight)[s.tid + u * 512];
            __builtin_amdgcn_sched_barrier(0);
        } else {
            for (int i = s.tid; i < NVEC; i += s.nthreads)
                ((l_u4 *)s.lds)[i] = ((const ARKMI_GLOBAL row_u4 *)d.weight)[i];
        }
    }
    Vec16<T> cur[NC], nxt[NC];
    if (count > 0)
        row_exact_load<T, NC>(
            as_global(static_cast<const T *>(d.in) + row_offset(row0, d.dim_c, d.dim_h, d.in_s)), lane, cur,
            d.in_read_again != 0);
    lds_ptr w_lds = nullptr;
    if (stage) {
        if (in_regs) {
#pragma unroll
            for (int u = 0; u < WV; ++u)
                if (s.tid + u * 512 < NVEC) ((l_u4 *)s.lds)[s.tid + u * 512] = wv[u];
        }
        s.sync();
        w_lds = s.lds;
    }
    uint32_t touched = 0;
    auto finish = [&](int64_t row) {
        gptr<T> out = as_global(static_cast<T *>(d.out) + row_offset(row, d.dim_c, d.dim_h, d.out_s));
        gptr<const T> mask = nullptr;
        if (KIND == ROW_SOFTMAX && d.weight)
            mask = as_global(static_cast<const T *>(d.weight) + row_offset(row, d.dim_c, d.dim_h, d.w_s));
        row_exact_finish<T, KIND, NC>(d, cur, out, lane, mask, w_lds, cur, false);
    };
    // every row but the last: the next row's loads are issued, then this one is reduced and stored
    for (int j = 0; j + 1 < count; ++j) {
        const int64_t row = row0 + (int64_t)j * stride;
        row_exact_load<T, NC>(
            as_global(static_cast<const T *>(d.in) + row_offset(row + stride, d.dim_c, d.dim_h, d.in_s)), lane, nxt,
            d.in_read_again != 0);
        __builtin_amdgcn_sched_barrier(0);
        finish(row);
#pragma unroll
        for (int c = 0; c < NC; ++c) cur[c] = nxt[c];
    }
    // the last row (kept out of the loop above, which then has no branch inside): in place of a next
    // row's loads, one word of every 128-byte line of the next op's first row for this wave
    if (count > 0) {
        if (d.pf_base) {
            const ARKMI_GLOBAL char *p = (const ARKMI_GLOBAL char *)d.pf_base + row0 * d.pf_row_bytes;
            for (int b = lane * 128; b < d.pf_len; b += kWave * 128) touched ^= *(const ARKMI_GLOBAL uint32_t *)(p + b);
        }
        __builtin_amdgcn_sched_barrier(0);
        finish(row0 + (int64_t)(count - 1) * stride);
    }
    asm volatile("" ::"v"(touched));  // (the touches are waited for here, behind the last row's stores)
}

// RMSNorm of 16-bit rows: the weights (the same NC vectors per lane for every row) go straight to
// registers, fetched beside the first row, instead of one dependent load per chunk after the
// reduction or a copy through LDS with two workgroup barriers per task (2048 rows of 4096 bf16,
// one row per wave, in the loop kernel: 13.0 us with fp32 weights staged in LDS, 11.6 loaded
// chunk by chunk, 8.3 with the weights in registers).
template <typename T, int NC, bool W32>
__device__ __forceinline__ void rmsnorm_rows_weight_in_regs(const RowOpDesc &d, int64_t row0, int stride, int count,
                                                            int lane) {
    constexpr int VN = Vec16<T>::N;
    using WReg = typename std::conditional<W32, F32Vec<VN>, Vec16<T>>::type;
    WReg wreg[NC];
    if constexpr (W32) {
        typedef float row_f4 __attribute__((ext_vector_type(4)));
        const ARKMI_GLOBAL row_f4 *wp = (const ARKMI_GLOBAL row_f4 *)d.weight;
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int q = 0; q < VN / 4; ++q) {
                const row_f4 v = wp[(c * (kWave * VN) + lane * VN) / 4 + q];
                wreg[c].v[4 * q] = v.x; wreg[c].v[4 * q + 1] = v.y; wreg[c].v[4 * q + 2] = v.z; wreg[c].v[4 * q + 3] = v.w;
            }
    } else {
        gptr<const T> wp = as_global(static_cast<const T *>(d.weight));
#pragma unroll
        for (int c = 0; c < NC; ++c) wreg[c] = load16<T>(wp + c * (kWave * VN) + lane * VN);
    }
    // the rows as in row_op_pipelined: the next row's loads ahead of this row's reduction, the
    // last row outside the loop, with the touches of the next op's first row in its place
    Vec16<T> cur[NC], nxt[NC];
    if (count > 0)
        row_exact_load<T, NC>(as_global(static_cast<const T *>(d.in) + row_offset(row0, d.dim_c, d.dim_h, d.in_s)),
                              lane, cur, d.in_read_again != 0);
    uint32_t touched = 0;
    auto finish = [&](int64_t row) {
        row_exact_finish<T, ROW_RMSNORM, NC>(
            d, cur, as_global(static_cast<T *>(d.out) + row_offset(row, d.dim_c, d.dim_h, d.out_s)), lane, nullptr,
            nullptr, wreg, true);
    };
    for (int j = 0; j + 1 < count; ++j) {
        const int64_t row = row0 + (int64_t)j * stride;
        row_exact_load<T, NC>(
            as_global(static_cast<const T *>(d.in) + row_offset(row + stride, d.dim_c, d.dim_h, d.in_s)), lane, nxt,
            d.in_read_again != 0);
        __builtin_amdgcn_sched_barrier(0);
        finish(row);
#pragma unroll
        for (int c = 0; c < NC; ++c) cur[c] = nxt[c];
    }
    if (count > 0) {
        if (d.pf_base) {
            const ARKMI_GLOBAL char *p = (const ARKMI_GLOBAL char *)d.pf_base + row0 * d.pf_row_bytes;
            for (int b = lane * 128; b < d.pf_len; b += kWave * 128) touched ^= *(const ARKMI_GLOBAL uint32_t *)(p + b);
        }
        __builtin_amdgcn_sched_barrier(0);
        finish(row0 + (int64_t)(count - 1) * stride);
    }
    asm volatile("" ::"v"(touched));
}

// One task = rows_per_wave rows per wave of the slot.  With R rows per wave and W
// waves, task t covers rows [t*R*W, (t+1)*R*W); at each step the W waves work on W
// adjacent rows.
template <typename T, int KIND>
__device__ __forceinline__ void row_op_task(const RowOpDesc &d, int task, const Slot &s) {
    constexpr int VN = Vec16<T>::N;
    constexpr int PER_CHUNK = kWave * VN;
    constexpr bool IS_REDUCE = RowMath<KIND>::IS_REDUCE;
    const int R = d.rows_per_wave > 1 ? d.rows_per_wave : 1;
    const int nw = s.nwaves();
    const int64_t row0 = (int64_t)task * R * nw + s.wave();
    const int count = row0 < d.rows ? (int)min((int64_t)R, (d.rows - row0 + nw - 1) / nw) : 0;
    // every row equally aligned: the base and all row strides are whole vectors
    auto whole = [](const void *p, const int64_t (&st)[3]) {
        return aligned16(p) && (st[0] % VN) == 0 && (st[1] % VN) == 0 && (st[2] % VN) == 0;
    };
    bool ok = whole(d.in, d.in_s) && (IS_REDUCE || whole(d.out, d.out_s));
    if (KIND == ROW_RMSNORM && d.weight) ok = ok && aligned16(d.weight);
    if (KIND == ROW_SOFTMAX && d.weight) ok = ok && whole(d.weight, d.w_s);
    // `ok` and `stage` depend on the descriptor alone: the whole slot takes the same path
    const bool stage = (KIND == ROW_RMSNORM) && d.weight_lds != 0;
    if constexpr (KIND == ROW_RMSNORM && sizeof(T) == 2) {
        // (decided by the descriptor alone: the whole slot takes this path, which has no barrier)
        if (ok && d.weight) {
            if (d.weight_fp32) {
                if (d.cols == 4 * PER_CHUNK) return rmsnorm_rows_weight_in_regs<T, 4, true>(d, row0, nw, count, s.lane());
                if (d.cols == 8 * PER_CHUNK) return rmsnorm_rows_weight_in_regs<T, 8, true>(d, row0, nw, count, s.lane());
            } else {
                if (d.cols == 4 * PER_CHUNK) return rmsnorm_rows_weight_in_regs<T, 4, false>(d, row0, nw, count, s.lane());
                if (d.cols == 8 * PER_CHUNK) return rmsnorm_rows_weight_in_regs<T, 8, false>(d, row0, nw, count, s.lane());
            }
        }
    }
    if (ok && d.cols == 4 * PER_CHUNK) return row_op_pipelined<T, KIND, 4>(d, row0, nw, count, s, stage);
    if (ok && d.cols == 8 * PER_CHUNK) return row_op_pipelined<T, KIND, 8>(d, row0, nw, count, s, stage);
    for (int j = 0; j < count; ++j) row_op_wave<T, KIND>(d, row0 + (int64_t)j * nw, s.lane());
}

// Reduction over an axis other than the last (ark/include/kernels/reduce.h:236-339,
// the reference's element-wise reduce): one output element per thread, adjacent
// threads on adjacent elements of the last axis, fp32 accumulation in index order.
template <typename T, int KIND>
__device__ __forceinline__ void reduce_axis_task(const RowOpDesc &d, int task, const Slot &s) {
    using M = RowMath<KIND>;
    const int64_t id = (int64_t)task * s.nthreads + s.tid;
    if (id >= d.rows * d.cols) return;
    const int64_t row = id / d.cols;
    const int w = (int)(id - row * d.cols);
    gptr<const T> in = as_global(static_cast<const T *>(d.in) + row_offset(row, d.dim_c, d.dim_h, d.in_s) + w);
    gptr<T> out = as_global(static_cast<T *>(d.out) + row_offset(row, d.dim_c, d.dim_h, d.out_s) + w);
    float acc = M::init();
    for (int r = 0; r < d.red_len; ++r) acc = M::acc1(acc, to_f32(in[(int64_t)r * d.red_stride]));
    if (KIND == ROW_MEAN) acc /= (float)d.red_len;
    out[0] = from_f32<T>(acc);
}

template <typename T>
__device__ __forceinline__ void reduce_axis_dispatch_kind(const RowOpDesc &d, int task, const Slot &s) {
    switch (d.kind) {
        case ROW_SUM: reduce_axis_task<T, ROW_SUM>(d, task, s); break;
        case ROW_MAX: reduce_axis_task<T, ROW_MAX>(d, task, s); break;
        default: reduce_axis_task<T, ROW_MEAN>(d, task, s); break;
    }
}

// descriptors with red_len > 0
__device__ __forceinline__ void reduce_axis_dispatch(const RowOpDesc &d, int task, const Slot &s) {
    if (d.dtype == 0)
        reduce_axis_dispatch_kind<float>(d, task, s);
    else if (d.dtype == 1)
        reduce_axis_dispatch_kind<f16>(d, task, s);
    else
        reduce_axis_dispatch_kind<bf16>(d, task, s);
}

template <typename T>
__device__ __forceinline__ void row_op_dispatch_kind(const RowOpDesc &d, int task, const Slot &s) {
    switch (d.kind) {
        case ROW_SUM: row_op_task<T, ROW_SUM>(d, task, s); break;
        case ROW_MAX: row_op_task<T, ROW_MAX>(d, task, s); break;
        case ROW_MEAN: row_op_task<T, ROW_MEAN>(d, task, s); break;
        case ROW_SOFTMAX: row_op_task<T, ROW_SOFTMAX>(d, task, s); break;
        case ROW_LAYERNORM: row_op_task<T, ROW_LAYERNORM>(d, task, s); break;
        default: row_op_task<T, ROW_RMSNORM>(d, task, s); break;
    }
}

__device__ __forceinline__ void row_op_dispatch(const RowOpDesc &d, int task, const Slot &s) {
    if (d.dtype == 0)
        row_op_dispatch_kind<float>(d, task, s);
    else if (d.dtype == 1)
        row_op_dispatch_kind<f16>(d, task, s);
    else
        row_op_dispatch_kind<bf16>(d, task, s);
}

}  // namespace arkmi
