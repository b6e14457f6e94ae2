// Elementwise ops with NumPy broadcasting over 4-D strided views: add/sub/mul/
// div, exp/gelu/relu/rsqrt/sigmoid/sqrt, copy, cast, scalar assign/add/mul,
// rope, and (through permuted input strides) transpose.
//
// One task = one [tile_h x tile_w] tile of the output at a fixed (n, c).
// Threads walk the tile in groups of 8 consecutive elements along W: operands
// whose innermost stride is 1 move as one vector (16 B for 2-byte types),
// broadcast operands are read once and splat, anything else is gathered.
// Arithmetic is fp32 on the exact stored values with one rounding to storage,
// which is what the reference's host baselines do
// (ark/ops/ops_arithmetic_test.cpp:6-128, ops_math_test.cpp:10-94,
// ops_scalar_test.cpp:9-60, ops_cast_test.cpp, ops_rope_test.cpp:8-34).
//
// Replaces ark/include/kernels/common/broadcast.h:378-524 and the per-op
// functors in arithmetic.h / math_functions.h / scalar.h / cast.h / copy.h /
// embedding.h:14-37 (rope) / transpose.h.
#pragma once
#include "dev_common.h"

namespace arkmi {

enum EwOp : int32_t {
    EW_ADD = 0, EW_SUB, EW_MUL, EW_DIV, EW_SILU_MUL, EW_ROPE,  // binary
    EW_EXP, EW_GELU, EW_RELU, EW_RSQRT, EW_SIGMOID, EW_SQRT,  // unary
    EW_COPY, EW_CAST,
    EW_SCALAR_ASSIGN, EW_SCALAR_ADD, EW_SCALAR_MUL,
    // INT32 tensors: the same ops on the bits (the values travel through the float registers of
    // the common paths unconverted; the host selects these for dt_in == dt_out == int32)
    EW_IADD, EW_ISUB, EW_IMUL, EW_IDIV, EW_ISCALAR_ASSIGN, EW_ISCALAR_ADD, EW_ISCALAR_MUL,
};

constexpr bool ew_is_binary(int op) { return op <= EW_ROPE || (op >= EW_IADD && op <= EW_IDIV); }
constexpr bool ew_has_no_input(int op) { return op == EW_SCALAR_ASSIGN || op == EW_ISCALAR_ASSIGN; }

struct EwTensor {
    void *ptr;
    int64_t s[4];  // element strides per output dim; 0 where the operand broadcasts
};

struct EwiseDesc {
    EwTensor out, in0, in1;
    int32_t shape[4];  // output N, C, H, W
    int32_t tile_h, tile_w;
    int32_t tiles_h, tiles_w;
    int32_t op;
    int32_t dt_in, dt_out;  // 0 fp32, 1 fp16, 2 bf16, 3 int32
    float param;            // scalar ops: the factor / value
    int32_t fast;           // set by the host when ewise_fast's conditions hold
    int32_t in1_period;     // > 0: in1 is addressed with (w mod in1_period) along W (a multiple of 8)
};

constexpr int kEwGroup = 8;   // elements per thread step
constexpr int kEwUnroll = 4;  // steps a thread keeps in flight

template <typename T>
__device__ __forceinline__ float ew_to_f32(T v) { return static_cast<float>(v); }
template <typename T>
__device__ __forceinline__ T ew_from_f32(float v) { return static_cast<T>(v); }
// fp -> int32 truncates toward zero like a C cast
template <>
__device__ __forceinline__ int32_t ew_from_f32<int32_t>(float v) { return (int32_t)v; }

// round to the storage type and back (host half types round after every op)
template <typename T>
__device__ __forceinline__ float ew_round(float v) { return ew_to_f32<T>(ew_from_f32<T>(v)); }

template <typename T>
__device__ __forceinline__ void ew_load(const EwTensor &t, int64_t base, bool full, int valid,
                                        float (&x)[kEwGroup]) {
    gptr<const T> p = as_global(static_cast<const T *>(t.ptr) + base);
    const int64_t sw = t.s[3];
    if (sw == 0) {
        float v = ew_to_f32<T>(p[0]);
#pragma unroll
        for (int j = 0; j < kEwGroup; ++j) x[j] = v;
    } else if (sw == 1 && full && (((uintptr_t)p & (sizeof(T) * kEwGroup - 1)) == 0)) {
        using raw = uint32_t __attribute__((ext_vector_type(sizeof(T) * kEwGroup / 4)));
        // an operand that is read once (no broadcast along any axis) streams past the caches
        const bool stream = t.s[0] != 0 && t.s[1] != 0 && t.s[2] != 0;
        raw r = stream ? __builtin_nontemporal_load((const ARKMI_GLOBAL raw *)p) : *(const ARKMI_GLOBAL raw *)p;
        T v[kEwGroup];
        __builtin_memcpy(v, &r, sizeof(v));
#pragma unroll
        for (int j = 0; j < kEwGroup; ++j) x[j] = ew_to_f32<T>(v[j]);
    } else {
#pragma unroll
        for (int j = 0; j < kEwGroup; ++j) x[j] = (j < valid) ? ew_to_f32<T>(p[j * sw]) : 0.f;
    }
}

template <typename T>
__device__ __forceinline__ void ew_store(const EwTensor &t, int64_t base, bool full, int valid,
                                         const float (&y)[kEwGroup]) {
    gptr<T> p = as_global(static_cast<T *>(t.ptr) + base);
    const int64_t sw = t.s[3];
    if (sw == 1 && full && (((uintptr_t)p & (sizeof(T) * kEwGroup - 1)) == 0)) {
        using raw = uint32_t __attribute__((ext_vector_type(sizeof(T) * kEwGroup / 4)));
        T v[kEwGroup];
#pragma unroll
        for (int j = 0; j < kEwGroup; ++j) v[j] = ew_from_f32<T>(y[j]);
        raw r;
        __builtin_memcpy(&r, v, sizeof(v));
        __builtin_nontemporal_store(r, (ARKMI_GLOBAL raw *)p);
    } else {
#pragma unroll
        for (int j = 0; j < kEwGroup; ++j)
            if (j < valid) p[j * sw] = ew_from_f32<T>(y[j]);
    }
}

// One group of 8 results.
template <typename TO, int OP>
__device__ __forceinline__ void ew_compute(const float (&a)[kEwGroup], const float (&b)[kEwGroup], float param,
                                           float (&y)[kEwGroup]) {
#pragma unroll
    for (int j = 0; j < kEwGroup; ++j) {
        const float x = a[j];
        float r;
        switch (OP) {
            case EW_ADD: r = x + b[j]; break;
            case EW_SUB: r = x - b[j]; break;
            case EW_MUL: r = x * b[j]; break;
            case EW_DIV: r = x / b[j]; break;
            case EW_SILU_MUL: r = x / (1.f + expf(-x)) * b[j]; break;
            case EW_ROPE: {
                // (a0 + i a1)(b0 + i b1) on adjacent pairs, rounded to the
                // storage type after every operation like the host types;
                // no FMA contraction, so fp32 matches a plain C evaluation
#pragma clang fp contract(off)
                const int e = j & ~1;
                const float a0 = a[e], a1 = a[e + 1], b0 = b[e], b1 = b[e + 1];
                const float p0 = ew_round<TO>((j & 1) ? a0 * b1 : a0 * b0);
                const float p1 = ew_round<TO>((j & 1) ? a1 * b0 : a1 * b1);
                r = (j & 1) ? p0 + p1 : p0 - p1;
                break;
            }
            case EW_EXP: r = expf(x); break;
            case EW_GELU:
                r = 0.5f * x * (1.f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
                break;
            case EW_RELU: r = x > 0.f ? x : 0.f; break;
            case EW_RSQRT: r = 1.0f / sqrtf(x); break;
            case EW_SIGMOID: r = 1.f / (1.f + expf(-x)); break;
            case EW_SQRT: r = sqrtf(x); break;
            case EW_SCALAR_ASSIGN: r = param; break;
            case EW_SCALAR_ADD: r = x + param; break;
            case EW_SCALAR_MUL: r = x * param; break;
            // INT32: two's-complement wrap-around for + - *, C's truncating division (x / 0 and
            // INT_MIN / -1 give 0 here), the scalar converted like a C cast
            case EW_IADD: case EW_ISUB: case EW_IMUL: case EW_IDIV:
            case EW_ISCALAR_ASSIGN: case EW_ISCALAR_ADD: case EW_ISCALAR_MUL: {
                const bool scalar = OP >= EW_ISCALAR_ASSIGN;
                const uint32_t ua = __builtin_bit_cast(uint32_t, x);
                const uint32_t ub = scalar ? (uint32_t)(int32_t)param : __builtin_bit_cast(uint32_t, b[j]);
                uint32_t ur;
                if (OP == EW_IADD || OP == EW_ISCALAR_ADD) ur = ua + ub;
                else if (OP == EW_ISUB) ur = ua - ub;
                else if (OP == EW_IMUL || OP == EW_ISCALAR_MUL) ur = ua * ub;
                else if (OP == EW_ISCALAR_ASSIGN) ur = ub;
                else {
                    const int32_t ia = (int32_t)ua, ib = (int32_t)ub;
                    ur = (ib == 0 || (ia == INT32_MIN && ib == -1)) ? 0u : (uint32_t)(ia / ib);
                }
                r = __builtin_bit_cast(float, ur);
                break;
            }
            default: r = x; break;  // copy, cast
        }
        y[j] = r;
    }
}

// The common case: every operand either dense along W (stride 1, 16-byte
// aligned groups) or broadcast along W, no ragged group, and an (n, c) slice
// under 4 GB.  Wave64 VALU instructions take four cycles each, so at HBM rate
// a workgroup can spend only a few hundred of them per 64 KB moved: the walk
// over the tile uses no division and no 64-bit arithmetic after its first
// step, offsets advance by uniform constants.
// PERIODIC: in1 wraps along W with a power-of-two period (in1_period).
template <typename TI, typename TO, int OP, bool PERIODIC = false>
__device__ __forceinline__ void ewise_fast(const EwiseDesc &d, int n, int c, int h0, int h1, int w0, int w1,
                                           const Slot &s) {
    constexpr bool BINARY = ew_is_binary(OP);
    constexpr bool NO_INPUT = ew_has_no_input(OP);
    constexpr int U = kEwUnroll;
    using rawi = uint32_t __attribute__((ext_vector_type(sizeof(TI) * kEwGroup / 4)));
    using rawo = uint32_t __attribute__((ext_vector_type(sizeof(TO) * kEwGroup / 4)));
    const int gw = (w1 - w0) / kEwGroup;  // groups per row
    const int items = (h1 - h0) * gw;
    const int nt = s.nthreads;
    const float param = ew_round<TO>(d.param);  // the factor is cast to the tensor type first

    gptr<const char> p0 = as_global(reinterpret_cast<const char *>(
        static_cast<const TI *>(d.in0.ptr) + n * d.in0.s[0] + c * d.in0.s[1] + h0 * d.in0.s[2] + w0 * d.in0.s[3]));
    gptr<const char> p1 = as_global(reinterpret_cast<const char *>(
        static_cast<const TI *>(d.in1.ptr) + n * d.in1.s[0] + c * d.in1.s[1] + h0 * d.in1.s[2] +
        (PERIODIC ? 0 : w0) * d.in1.s[3]));
    const int pmask = PERIODIC ? d.in1_period / kEwGroup - 1 : 0;  // in groups
    const int pcol0 = PERIODIC ? w0 / kEwGroup : 0;
    gptr<char> po = as_global(reinterpret_cast<char *>(
        static_cast<TO *>(d.out.ptr) + n * d.out.s[0] + c * d.out.s[1] + h0 * d.out.s[2] + w0 * d.out.s[3]));
    // byte strides per row and per group (0 for an operand broadcast along W)
    const uint32_t r0 = (uint32_t)(d.in0.s[2] * sizeof(TI)), g0 = (uint32_t)(d.in0.s[3] * sizeof(TI) * kEwGroup);
    const uint32_t r1 = (uint32_t)(d.in1.s[2] * sizeof(TI)), g1 = (uint32_t)(d.in1.s[3] * sizeof(TI) * kEwGroup);
    const uint32_t ro = (uint32_t)(d.out.s[2] * sizeof(TO)), go = (uint32_t)(sizeof(TO) * kEwGroup);
    const bool stream0 = d.in0.s[0] != 0 && d.in0.s[1] != 0 && d.in0.s[2] != 0 && g0 != 0;
    const bool stream1 = d.in1.s[0] != 0 && d.in1.s[1] != 0 && d.in1.s[2] != 0 && g1 != 0;

    // this thread's first group, and the uniform step to its next one
    int row = s.tid / gw;
    int col = s.tid - row * gw;
    const int drow = nt / gw, dcol = nt - drow * gw;
    uint32_t o0 = row * r0 + col * g0, o1 = row * r1 + col * g1, oo = row * ro + col * go;
    const uint32_t st0 = drow * r0 + dcol * g0, st1 = drow * r1 + dcol * g1, sto = drow * ro + dcol * go;
    const uint32_t wr0 = r0 - gw * g0, wr1 = r1 - gw * g1, wro = ro - gw * go;  // a step that wraps to the next row

    for (int it0 = s.tid; it0 < items; it0 += nt * U) {
        uint32_t a0[U], a1[U], ao[U];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            ok[u] = it0 + u * nt < items;
            a0[u] = o0; ao[u] = oo;
            a1[u] = PERIODIC ? row * r1 + ((pcol0 + col) & pmask) * g1 : o1;
            col += dcol;
            const bool wrap = col >= gw;
            col -= wrap ? gw : 0;
            if (PERIODIC) row += drow + (wrap ? 1 : 0);
            o0 += st0 + (wrap ? wr0 : 0u);
            o1 += st1 + (wrap ? wr1 : 0u);
            oo += sto + (wrap ? wro : 0u);
        }
        rawi va[U], vb[U];
        TI ea[U], eb[U];
        if (!NO_INPUT) {
            if (g0 != 0) {
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (ok[u]) {
                        const ARKMI_GLOBAL rawi *p = (const ARKMI_GLOBAL rawi *)(p0 + (size_t)a0[u]);
                        va[u] = stream0 ? __builtin_nontemporal_load(p) : *p;
                    }
            } else {
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (ok[u]) ea[u] = *(gptr<const TI>)(p0 + (size_t)a0[u]);
            }
        }
        if (BINARY) {
            if (g1 != 0) {
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (ok[u]) {
                        const ARKMI_GLOBAL rawi *p = (const ARKMI_GLOBAL rawi *)(p1 + (size_t)a1[u]);
                        vb[u] = stream1 ? __builtin_nontemporal_load(p) : *p;
                    }
            } else {
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (ok[u]) eb[u] = *(gptr<const TI>)(p1 + (size_t)a1[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (!ok[u]) continue;
            float a[kEwGroup], b[kEwGroup], y[kEwGroup];
            if (!NO_INPUT) {
                if (g0 != 0) {
                    TI v[kEwGroup];
                    __builtin_memcpy(v, &va[u], sizeof(v));
#pragma unroll
                    for (int j = 0; j < kEwGroup; ++j) a[j] = ew_to_f32<TI>(v[j]);
                } else {
#pragma unroll
                    for (int j = 0; j < kEwGroup; ++j) a[j] = ew_to_f32<TI>(ea[u]);
                }
            }
            if (BINARY) {
                if (g1 != 0) {
                    TI v[kEwGroup];
                    __builtin_memcpy(v, &vb[u], sizeof(v));
#pragma unroll
                    for (int j = 0; j < kEwGroup; ++j) b[j] = ew_to_f32<TI>(v[j]);
                } else {
#pragma unroll
                    for (int j = 0; j < kEwGroup; ++j) b[j] = ew_to_f32<TI>(eb[u]);
                }
            }
            ew_compute<TO, OP>(a, b, param, y);
            TO v[kEwGroup];
#pragma unroll
            for (int j = 0; j < kEwGroup; ++j) v[j] = ew_from_f32<TO>(y[j]);
            rawo r;
            __builtin_memcpy(&r, v, sizeof(v));
            __builtin_nontemporal_store(r, (ARKMI_GLOBAL rawo *)(po + (size_t)ao[u]));
        }
    }
}

template <typename TI, typename TO, int OP>
__device__ __forceinline__ void ewise_task(const EwiseDesc &d, int task, const Slot &s) {
    constexpr bool BINARY = ew_is_binary(OP);
    constexpr bool NO_INPUT = ew_has_no_input(OP);
    const int tw_i = task % d.tiles_w;
    int t = task / d.tiles_w;
    const int th_i = t % d.tiles_h;
    t /= d.tiles_h;
    const int c = t % d.shape[1];
    const int n = t / d.shape[1];
    const int h0 = th_i * d.tile_h, w0 = tw_i * d.tile_w;
    const int h1 = min(h0 + d.tile_h, d.shape[2]);
    const int w1 = min(w0 + d.tile_w, d.shape[3]);
    if (d.fast) {
        if (OP == EW_ROPE && d.in1_period > 0)
            ewise_fast<TI, TO, OP, (OP == EW_ROPE)>(d, n, c, h0, h1, w0, w1, s);
        else
            ewise_fast<TI, TO, OP>(d, n, c, h0, h1, w0, w1, s);
        return;
    }
    const int groups_w = (w1 - w0 + kEwGroup - 1) / kEwGroup;
    const int items = (h1 - h0) * groups_w;
    const float param = ew_round<TO>(d.param);  // the factor is cast to the tensor type first

    // Each thread keeps kEwUnroll groups in flight: all their loads are issued
    // before the first result is needed.
    for (int it0 = s.tid; it0 < items; it0 += s.nthreads * kEwUnroll) {
        float a[kEwUnroll][kEwGroup], b[kEwUnroll][kEwGroup];
#pragma unroll
        for (int u = 0; u < kEwUnroll; ++u) {
            const int it = it0 + u * s.nthreads;
            if (it >= items) break;
            const int h = h0 + it / groups_w;
            const int w = w0 + (it % groups_w) * kEwGroup;
            const int valid = min(kEwGroup, w1 - w);
            const bool full = (valid == kEwGroup);
            if (!NO_INPUT) {
                int64_t off = n * d.in0.s[0] + c * d.in0.s[1] + h * d.in0.s[2] + w * d.in0.s[3];
                ew_load<TI>(d.in0, off, full, valid, a[u]);
            }
            if (BINARY) {
                const int w1m = d.in1_period > 0 ? w % d.in1_period : w;
                int64_t off = n * d.in1.s[0] + c * d.in1.s[1] + h * d.in1.s[2] + w1m * d.in1.s[3];
                ew_load<TI>(d.in1, off, full, valid, b[u]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < kEwUnroll; ++u) {
            const int it = it0 + u * s.nthreads;
            if (it >= items) break;
            const int h = h0 + it / groups_w;
            const int w = w0 + (it % groups_w) * kEwGroup;
            const int valid = min(kEwGroup, w1 - w);
            const bool full = (valid == kEwGroup);
            float y[kEwGroup];
            ew_compute<TO, OP>(a[u], b[u], param, y);
            int64_t off = n * d.out.s[0] + c * d.out.s[1] + h * d.out.s[2] + w * d.out.s[3];
            ew_store<TO>(d.out, off, full, valid, y);
        }
    }
}

template <typename T>
__device__ __forceinline__ void ewise_same_type(const EwiseDesc &d, int task, const Slot &s) {
    switch (d.op) {
        case EW_ADD: ewise_task<T, T, EW_ADD>(d, task, s); break;
        case EW_SUB: ewise_task<T, T, EW_SUB>(d, task, s); break;
        case EW_MUL: ewise_task<T, T, EW_MUL>(d, task, s); break;
        case EW_DIV: ewise_task<T, T, EW_DIV>(d, task, s); break;
        case EW_SILU_MUL: ewise_task<T, T, EW_SILU_MUL>(d, task, s); break;
        case EW_ROPE: ewise_task<T, T, EW_ROPE>(d, task, s); break;
        case EW_EXP: ewise_task<T, T, EW_EXP>(d, task, s); break;
        case EW_GELU: ewise_task<T, T, EW_GELU>(d, task, s); break;
        case EW_RELU: ewise_task<T, T, EW_RELU>(d, task, s); break;
        case EW_RSQRT: ewise_task<T, T, EW_RSQRT>(d, task, s); break;
        case EW_SIGMOID: ewise_task<T, T, EW_SIGMOID>(d, task, s); break;
        case EW_SQRT: ewise_task<T, T, EW_SQRT>(d, task, s); break;
        case EW_SCALAR_ASSIGN: ewise_task<T, T, EW_SCALAR_ASSIGN>(d, task, s); break;
        case EW_SCALAR_ADD: ewise_task<T, T, EW_SCALAR_ADD>(d, task, s); break;
        case EW_SCALAR_MUL: ewise_task<T, T, EW_SCALAR_MUL>(d, task, s); break;
        default: ewise_task<T, T, EW_COPY>(d, task, s); break;
    }
}

template <typename TI>
__device__ __forceinline__ void ewise_cast_from(const EwiseDesc &d, int task, const Slot &s) {
    switch (d.dt_out) {
        case 0: ewise_task<TI, float, EW_CAST>(d, task, s); break;
        case 1: ewise_task<TI, f16, EW_CAST>(d, task, s); break;
        case 2: ewise_task<TI, bf16, EW_CAST>(d, task, s); break;
        default: ewise_task<TI, int32_t, EW_CAST>(d, task, s); break;
    }
}

// ---- embedding gather ---------------------------------------------------------------
// out[n, c, h, :] = weight[idx[n, c, h], :] with negative indices counted from the end of
// the table (ark/include/kernels/embedding.h:107-143).  An index outside [-num_emb, num_emb)
// names no row: it is clamped to the nearest one (row 0 or the last), so that index data
// from a user can never make the gather read outside the table; the reference reads
// whatever lies there.  One wave per output row: the
// index is a uniform load, the row moves as 16-byte vectors when both rows are aligned.
struct EmbedDesc {
    const int32_t *idx;
    const void *weight;
    void *out;
    int64_t rows;          // N * C * H of the output
    int32_t dim_c, dim_h;  // output C and H, to unflatten a row number
    int64_t idx_s[3];      // element strides of the index tensor along N, C, H
    int64_t out_s[3];      // element strides of the output rows
    int64_t w_pitch;       // elements between rows of the table
    int32_t emb_dim, num_emb;
    int32_t elem;          // bytes per element (2 or 4)
    int32_t pad_;
};

__device__ __forceinline__ void embedding_task(const EmbedDesc &d, int task, const Slot &s) {
    const int64_t row = (int64_t)task * s.nwaves() + s.wave();
    if (row >= d.rows) return;
    const int lane = s.lane();
    const int64_t h = row % d.dim_h, c = (row / d.dim_h) % d.dim_c, n = row / ((int64_t)d.dim_h * d.dim_c);
    int e = as_global(d.idx)[n * d.idx_s[0] + c * d.idx_s[1] + h * d.idx_s[2]];
    if (e < 0) e += d.num_emb;
    e = min(max(e, 0), d.num_emb - 1);
    e = __builtin_amdgcn_readfirstlane(e);
    gptr<const char> src = as_global(static_cast<const char *>(d.weight)) + (int64_t)e * d.w_pitch * d.elem;
    gptr<char> dst = as_global(static_cast<char *>(d.out)) +
                     (n * d.out_s[0] + c * d.out_s[1] + h * d.out_s[2]) * d.elem;
    const int bytes = d.emb_dim * d.elem;
    if ((((uintptr_t)src | (uintptr_t)dst | (uintptr_t)bytes) & 15) == 0) {
        for (int b = lane * 16; b < bytes; b += 64 * 16)
            store16<char>(dst + b, load16<char>(src + b));
    } else if (d.elem == 4) {
        for (int i = lane; i < d.emb_dim; i += 64) ((gptr<uint32_t>)dst)[i] = ((gptr<const uint32_t>)src)[i];
    } else {
        for (int i = lane; i < d.emb_dim; i += 64) ((gptr<uint16_t>)dst)[i] = ((gptr<const uint16_t>)src)[i];
    }
}

__device__ __forceinline__ void ewise_dispatch(const EwiseDesc &d, int task, const Slot &s) {
    if (d.op == EW_CAST || d.dt_in != d.dt_out) {
        switch (d.dt_in) {
            case 0: ewise_cast_from<float>(d, task, s); break;
            case 1: ewise_cast_from<f16>(d, task, s); break;
            case 2: ewise_cast_from<bf16>(d, task, s); break;
            default: ewise_cast_from<int32_t>(d, task, s); break;
        }
        return;
    }
    switch (d.dt_in) {
        case 0: ewise_same_type<float>(d, task, s); break;
        case 1: ewise_same_type<f16>(d, task, s); break;
        case 2: ewise_same_type<bf16>(d, task, s); break;
        // int32: the bits travel untouched as 4-byte words (through a float conversion values
        // above 2^24 would round); the arithmetic ops work on the bits
        default:
            switch (d.op) {
                case EW_ADD: ewise_task<float, float, EW_IADD>(d, task, s); break;
                case EW_SUB: ewise_task<float, float, EW_ISUB>(d, task, s); break;
                case EW_MUL: ewise_task<float, float, EW_IMUL>(d, task, s); break;
                case EW_DIV: ewise_task<float, float, EW_IDIV>(d, task, s); break;
                case EW_SCALAR_ASSIGN: ewise_task<float, float, EW_ISCALAR_ASSIGN>(d, task, s); break;
                case EW_SCALAR_ADD: ewise_task<float, float, EW_ISCALAR_ADD>(d, task, s); break;
                case EW_SCALAR_MUL: ewise_task<float, float, EW_ISCALAR_MUL>(d, task, s); break;
                default: ewise_task<float, float, EW_COPY>(d, task, s); break;
            }
            break;
    }
}

}  // namespace arkmi
