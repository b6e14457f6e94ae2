// MFMA GEMM for gfx950: C[M,N] = A[M,K] . B, fp16 or bf16 operands, fp32
// accumulate, one rounding to the storage type.
//
// One task = one BM x BN output tile, computed by the 8 waves of a workgroup
// (2 x 4 wave grid) with v_mfma_f32_16x16x32 (at the chip's power limit that shape
// sustains about 15 % more flops than 32x32x16: a quarter of the accumulator
// traffic per instruction for half the flops).  A and B tiles of depth BK
// travel from global memory straight into LDS (global_load_lds_dwordx4 through
// direct_load16, no staging registers, no LDS store instructions) into a ring of S stage
// buffers; the loads of the next S-1 tiles are in flight while the current one
// is multiplied, and there is one workgroup barrier per tile.
//
// A wave-level direct load writes 1 KB of consecutive LDS, so rows cannot be
// padded against bank conflicts.  Instead every lane fetches the 16-byte chunk
// that belongs at its LDS position under an XOR swizzle:
//   K-contiguous tiles (A, and B stored [N,K]): rows of BK/8 chunks, the chunk of
//     k-group c of row r sits at position c ^ swz(r), with swz(r) =
//     (r & 7) ^ ((r >> 3) & 1) for 128-byte rows and (r >> 2) & 3 for 64-byte
//     rows; a ds_read_b128 of 16 consecutive rows at one k-group then touches
//     every bank once;
//   N-contiguous tiles (B stored [K,N]): rows of BN/8 chunks, chunk n of row k at
//     position n ^ ((k & 3) << 2); ds_read_b64_tr_b16 transposes on the way out
//     and the four k-rows a 16-lane block reads fall into different banks.
//
// Replaces ark/include/kernels/matmul.h:36-115 -> gemm_ck.h:375-526 (CK
// DeviceGemm_Xdl_CShuffle, 4 waves, 128x256x32 tiles, single-stage 24.6 KB LDS).
// Tile index semantics follow ark/include/kernels/common/unit_op.h:73-92:
// task -> (batch, m_tile, n_tile) row-major with the N tile fastest.
#pragma once
#include <type_traits>

#include "ewise.h"
#include "dev_common.h"

namespace arkmi {

struct GemmDesc {
    const void *a;
    const void *b;
    void *c;
    int32_t m, n, k;           // problem size (padded: multiples of the tile)
    int32_t lda, ldb, ldc;     // leading dimensions in elements
    // The batch is the (N, C) pair of a 4-D view: batch index -> n = idx /
    // batch_c, c = idx % batch_c; a stride of 0 broadcasts the operand.
    int64_t a_bs[2], b_bs[2], c_bs[2];
    int32_t batch_c;
    int32_t batch_total;       // number of (N, C) batches
    int32_t trans_b;           // 1: B stored [N,K]; 0: B stored [K,N]
    int32_t trans_a;           // 1: A stored [K,M] (128x128 tiles only); 0: A stored [M,K]
    // Gate/up pair (b2 != null, trans_b): C[M, n/2] = silu(A . B^T) * (A . B2^T) with B, B2 stored
    // [n/2, K].  The tile's n columns alternate in groups of 32 between B and B2 rows, so the two
    // products of an output column sit in the same lane of adjacent accumulator tiles.
    const void *b2;
    int32_t dtype;             // 1 fp16, 2 bf16; 0 fp32 (kernels/gemm_f32.h, 128x128 tiles)
    int32_t tiles_m, tiles_n;  // ceil(m/BM), ceil(n/BN)
    int32_t store_m, store_n;  // rows/cols of C that exist (unpadded shape)
    // Two-way split of K (split_k == 2): task t multiplies K from split_at on for tile t and
    // leaves its fp32 accumulators in `partial`; task t + tiles multiplies K below split_at,
    // adds those and finishes the tile.  `arrivals[t]` is the full/empty word of the tile's
    // partial sums: 0 empty (the sender may write), 1 full (the finisher may read).  The
    // sender's part of K is the shorter one, so that its partial sums are on their way while
    // the finisher still multiplies.
    int32_t split_k;           // 1 or 2
    // XCD-aware order of the tiles (gemm_tile): xcd_round > 0 turns it on
    int32_t xcd_round, xcd_band;
    int32_t split_at;          // split_k == 2: where the sender's part of K begins
    float *partial;            // [tiles][MT * NT][512 threads] x 4 floats
    unsigned int *arrivals;    // [tiles], zero between launches
    // An elementwise op folded into the store of C (fuse_kind != 0; the host sets it only where
    // every tile takes the staged store of gemm_tile): the values of C, rounded to the tensor
    // type as they are stored, meet the op's other operand, 16 bytes per lane, and the result
    // goes to fuse_out.  C itself is stored as always.
    const void *fuse_other;
    void *fuse_out;
    int32_t fuse_kind;         // 0: none; else 1 + EwOp (EW_ADD, EW_SUB, EW_MUL, EW_DIV, EW_ROPE)
    int32_t fuse_c_second;     // 1: C is the op's second input and the other operand its first
    int32_t fuse_ld_other;     // elements between rows of the other operand (0: one row for all)
    int32_t fuse_ld_out;       // elements between rows of the result
    int32_t fuse_period;       // > 0: the other operand's column is taken modulo this (a multiple of 8)
    int32_t pad2_;
};

// Eight values of C (as stored) and eight of the other operand through elementwise op `op`,
// with the arithmetic and the roundings of the op's own body (ew_compute).
template <typename T>
__device__ __forceinline__ uint32_t __attribute__((ext_vector_type(4)))
fused_store_values(int op, bool c_second, uint32_t __attribute__((ext_vector_type(4))) cv,
                   uint32_t __attribute__((ext_vector_type(4))) ov) {
    T c[kEwGroup], o[kEwGroup], r[kEwGroup];
    __builtin_memcpy(c, &cv, 16);
    __builtin_memcpy(o, &ov, 16);
    float a[kEwGroup], b[kEwGroup], y[kEwGroup];
#pragma unroll
    for (int j = 0; j < kEwGroup; ++j) {
        const float fc = ew_to_f32<T>(c[j]), fo = ew_to_f32<T>(o[j]);
        a[j] = c_second ? fo : fc;
        b[j] = c_second ? fc : fo;
    }
    switch (op) {
        case EW_ADD: ew_compute<T, EW_ADD>(a, b, 0.f, y); break;
        case EW_SUB: ew_compute<T, EW_SUB>(a, b, 0.f, y); break;
        case EW_MUL: ew_compute<T, EW_MUL>(a, b, 0.f, y); break;
        case EW_DIV: ew_compute<T, EW_DIV>(a, b, 0.f, y); break;
        default: ew_compute<T, EW_ROPE>(a, b, 0.f, y); break;
    }
#pragma unroll
    for (int j = 0; j < kEwGroup; ++j) r[j] = ew_from_f32<T>(y[j]);
    uint32_t __attribute__((ext_vector_type(4))) out;
    __builtin_memcpy(&out, r, 16);
    return out;
}

// What a bounded wait inside a body needs: the kernel's abort word and the tick limit.
struct BodyWait {
    int32_t *abort;
    uint64_t limit_ticks;
};
constexpr int kGemmAborted = -3;  // gemm_tile: a bounded wait gave up (the kernel's abort word is set)

// Polls *word until it reads `want`; false once the abort word is set or the limit has passed
// (then the abort word is set for everyone).
__device__ __forceinline__ bool poll_equals(unsigned int *word, unsigned int want, const BodyWait &w) {
    const uint64_t t0 = wall_clock64();
    unsigned polls = 0;
    while (__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != want) {
        __builtin_amdgcn_s_sleep(1);
        if ((++polls & 63u) == 0 && w.abort != nullptr) {  // (no abort word: nothing bounds the wait)
            if (__hip_atomic_load(w.abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) return false;
            if (wall_clock64() - t0 > w.limit_ticks) {
                __hip_atomic_store(w.abort, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                return false;
            }
        }
    }
    return true;
}

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
using lds_u32x4 = __attribute__((address_space(3))) u32x4;
using lds_s16x4 = __attribute__((address_space(3))) s16x4;
using lds_void = __attribute__((address_space(3))) void;
using lds_i32x = __attribute__((address_space(3))) int;

typedef float f32x4 __attribute__((ext_vector_type(4)));
template <typename T>
__device__ __forceinline__ f32x4 mfma16x32(u32x4 a, u32x4 b, f32x4 c);
template <>
__device__ __forceinline__ f32x4 mfma16x32<f16>(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                  0);
}
template <>
__device__ __forceinline__ f32x4 mfma16x32<bf16>(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
}

constexpr int kGemmThreads = 512;
constexpr int kGemmLoadBytes = 1024;  // LDS bytes one wave-level direct load fills

// Depth of a K tile and number of stage buffers for an output tile: the ring
// has to fit the 160 KB of LDS next to the loop kernel's own control words.
template <int BM, int BN>
struct GemmShape {
#ifdef ARKMI_GEMM_BK
    static constexpr int BK = ARKMI_GEMM_BK;
    static constexpr int STAGES = ARKMI_GEMM_STAGES;
#else
    static constexpr int BK = (BM + BN >= 512) ? 32 : 64;
    static constexpr int STAGES = (BM + BN >= 512) ? 4 : ((BM + BN >= 384) ? 3 : 4);
#endif
};
constexpr int kGemmMinK = 64;  // K must be a multiple of this for every tile shape

template <int BM, int BN>
struct GemmLds {
    static constexpr int BK = GemmShape<BM, BN>::BK;
    static constexpr int A_BYTES = BM * BK * 2;
    static constexpr int B_BYTES = BN * BK * 2;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int TOTAL_BYTES = GemmShape<BM, BN>::STAGES * STAGE_BYTES;
};

// s_waitcnt vmcnt(N) with the other counters left alone (gfx9 encoding: vmcnt in
// bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8).
template <int N>
__device__ __forceinline__ void wait_vmcnt_then_barrier() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}

// Epilogue hook: called once per accumulator element with its coordinates.
struct EpilogueStore {
    __device__ __forceinline__ float operator()(float v, int, int) const { return v; }
};

// Returns the tile this workgroup finished (its followers — the elementwise ops fused behind the
// matmul — run for that tile index), -1 when the other half of a split tile will finish it, or
// kGemmAborted.
// `poll(word, want)` is the bounded wait of the split (poll_equals with the kernel's abort word
// and tick limit, which the caller reads where it waits rather than carry them through the K loop).
struct NoPoll {
    __device__ __forceinline__ bool operator()(unsigned int *, unsigned int) const { return true; }
};
template <typename T, int BM, int BN, bool TRANS_B, typename Epi, bool TRANS_A = false, bool DUAL_B = false,
          bool SPLIT = false, typename Poll = NoPoll>
__device__ __forceinline__ int gemm_tile(const GemmDesc &d, int task_in, const Slot &s, Epi epi, Poll poll = Poll()) {
    static_assert(!SPLIT || !std::is_same<Poll, NoPoll>::value, "the split of K needs a bounded wait");
    static_assert(!DUAL_B || (TRANS_B && !TRANS_A), "the gate/up pair takes K-contiguous operands");
    static_assert(!SPLIT || (!DUAL_B && !TRANS_A), "the split of K exists for plain matmuls");
    // split: tasks [0, tiles) send the part of K from split_at on, tasks [tiles, 2 tiles) multiply
    // the part below it and finish the tile.  A workgroup runs its tasks in rising order, so a
    // sender never stands behind a finisher that waits for it.
    int task = task_in, k_begin = 0, k_len = d.k, half = 0;
    if constexpr (SPLIT) {
        const int tiles = d.tiles_m * d.tiles_n * d.batch_total;
        half = task_in >= tiles ? 0 : 1;
        task = task_in >= tiles ? task_in - tiles : task_in;
        k_begin = half ? d.split_at : 0;
        k_len = half ? d.k - d.split_at : d.split_at;
    }
    constexpr int BK = GemmShape<BM, BN>::BK;
    constexpr int S = GemmShape<BM, BN>::STAGES;
    constexpr int WGM = 2, WGN = 4;                // wave grid
    constexpr int WTM = BM / WGM, WTN = BN / WGN;  // wave tile
    constexpr int MT = WTM / 16, NT = WTN / 16;    // 16x16 MFMA tiles per wave
    static_assert(MT >= 1 && NT >= 1, "tile too small for the wave grid");
    static_assert(BK == 32 || BK == 64, "K tile depth");
    using L = GemmLds<BM, BN>;
    constexpr int ROW_B = 2 * BK;                    // bytes per row of a K-contiguous tile
    constexpr int CPR_K = BK / 8;                    // 16-byte chunks per such row
    constexpr int RPB_K = kGemmLoadBytes / ROW_B;    // rows one direct load covers
    constexpr int AK_LD = BM / (8 * RPB_K);          // direct loads per wave per K tile
    constexpr int BT_LD = BN / (8 * RPB_K);
    constexpr int RB_N = BN * 2;                     // bytes per k-row of an N-contiguous B tile
    constexpr int RPI_N = kGemmLoadBytes / RB_N;     // k-rows one direct load covers
    constexpr int CPR_N = BN / 8;                    // 16-byte chunks per k-row
    constexpr int BN_LD = BK / (8 * RPI_N);
    constexpr int B_LD = TRANS_B ? BT_LD : BN_LD;
    constexpr int RB_M = BM * 2;                     // the same for an M-contiguous A tile ([k][m])
    constexpr int RPI_M = kGemmLoadBytes / RB_M;
    constexpr int CPR_M = BM / 8;
    constexpr int AM_LD = BK / (8 * RPI_M);
    constexpr int A_LD = TRANS_A ? AM_LD : AK_LD;
    constexpr int LOADS = A_LD + B_LD;               // per wave per K tile
    static_assert(A_LD >= 1 && B_LD >= 1, "tile too small for 8 waves of direct loads");

    const int tid = s.tid;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;

    const int tiles_per_batch = d.tiles_m * d.tiles_n;
    const int bidx = task / tiles_per_batch;
    const int t2 = task % tiles_per_batch;
    int tm = t2 / d.tiles_n, tn = t2 % d.tiles_n;
    if (d.xcd_round > 0) {
        // Workgroups go to the chip's eight XCDs round robin and every XCD has its own L2, so
        // with tasks dealt in tile order an XCD's concurrent tiles are strewn over the whole
        // output and its L2 fetches nearly all of A.  Here the tile index is permuted so that the
        // R / 8 tiles an XCD works on at a time form a block of xcd_band tile rows by
        // R / (8 xcd_band) tile columns (R = xcd_round: the tasks that run at once).  The tiles are
        // ordered in bands of xcd_band rows, column by column inside a band; task index t2 of a
        // full round takes position ((round * 8 + xcd) * R / 8 + number within the XCD) of that
        // order; the tasks of an incomplete last round keep their positions.  (The host sets this
        // only where tiles_m is a multiple of xcd_band and task t runs on workgroup t mod R.)
        const int R = d.xcd_round, per = R >> 3, bm = d.xcd_band;
        int p = t2;
        if (t2 < (tiles_per_batch / R) * R) {
            const int r = t2 / R, q = t2 - r * R;
            p = (r * 8 + (q & 7)) * per + (q >> 3);
        }
        const int band = bm * d.tiles_n, b = p / band, w = p - b * band;
        tn = w / bm;
        tm = b * bm + (w - tn * bm);
        // the tile's own index from here on: partial tiles, arrivals and the ops fused behind
        // the matmul go by it
        task = bidx * tiles_per_batch + tm * d.tiles_n + tn;
    }
    const int m0 = tm * BM, n0 = tn * BN;

    const int bn = bidx / d.batch_c, bc = bidx % d.batch_c;
    // k_begin moves both operands along K (only the plain layouts can be split)
    gptr<const T> A = as_global(static_cast<const T *>(d.a) + bn * d.a_bs[0] + bc * d.a_bs[1] + k_begin);
    gptr<const T> B = as_global(static_cast<const T *>(d.b) + bn * d.b_bs[0] + bc * d.b_bs[1] +
                                (TRANS_B ? (int64_t)k_begin : (int64_t)k_begin * d.ldb));
    gptr<T> C = as_global(static_cast<T *>(d.c) + bn * d.c_bs[0] + bc * d.c_bs[1]);

    const lds_ptr lds = s.lds;

    // ---- global -> LDS -------------------------------------------------------------
    // Load i of a wave fills LDS block (i*8 + wave): RPB_K rows of a K-contiguous
    // tile.  The lane at LDS position (row lr, chunk pos) fetches k-group
    // pos ^ swz(row); swz depends on lr and the wave only, whatever i is.
    const int lr = lane / CPR_K;
    const int swl = (BK == 64) ? (lr ^ (wave & 1)) : (BK == 32) ? ((lr >> 2) & 3) : ((lr >> 3) & 1);
    const int kc = (lane % CPR_K) ^ swl;
    gptr<const T> a_src;
    int64_t a_step, a_kstep;  // elements between a wave's loads, and between K tiles
    if (TRANS_A) {
        // as for an N-contiguous B below, with m in the place of n
        const int kr = lane / CPR_M;
        const int krow = wave * RPI_M + kr;
        const int mc = (lane % CPR_M) ^ ((krow & 3) << 2);
        a_src = A + (int64_t)krow * d.lda + m0 + mc * 8;
        a_step = (int64_t)8 * RPI_M * d.lda;
        a_kstep = (int64_t)BK * d.lda;
    } else {
        a_src = A + (int64_t)(m0 + wave * RPB_K + lr) * d.lda + kc * 8;
        a_step = (int64_t)8 * RPB_K * d.lda;
        a_kstep = BK;
    }
    gptr<const T> b_src;
    int64_t b_step, b_kstep;
    gptr<const T> b_dual[DUAL_B ? B_LD : 1];  // DUAL_B: source of each of the wave's B loads
    if (DUAL_B) {
        gptr<const T> B2 = as_global(static_cast<const T *>(d.b2) + bn * d.b_bs[0] + bc * d.b_bs[1]);
        const int n0h = tn * (BN / 2);  // first row of the tile in B and in B2
#pragma unroll
        for (int l = 0; l < B_LD; ++l) {
            const int row = (l * 8 + wave) * RPB_K + lr;  // column of the tile
            const int q = row >> 5;                       // its group of 32: even from B, odd from B2
            b_dual[l] = ((q & 1) ? B2 : B) + (int64_t)(n0h + (q >> 1) * 32 + (row & 31)) * d.ldb + kc * 8;
        }
        b_src = B;
        b_step = 0;
        b_kstep = BK;
    } else if (TRANS_B) {
        b_src = B + (int64_t)(n0 + wave * RPB_K + lr) * d.ldb + kc * 8;
        b_step = (int64_t)8 * RPB_K * d.ldb;
        b_kstep = BK;
    } else {
        // block (i*8 + wave) holds RPI_N k-rows; the lane at (k-row, chunk pos) fetches
        // n-chunk pos ^ ((krow & 3) << 2); krow & 3 does not depend on i
        const int kr = lane / CPR_N;
        const int krow = wave * RPI_N + kr;
        const int nc = (lane % CPR_N) ^ ((krow & 3) << 2);
        b_src = B + (int64_t)krow * d.ldb + n0 + nc * 8;
        b_step = (int64_t)8 * RPI_N * d.ldb;
        b_kstep = (int64_t)BK * d.ldb;
    }
    // load l of a K tile: l < A_LD fills a block of A, the rest blocks of B
    auto issue_one = [&](int kt, int stage, int l) {
        const lds_ptr base = lds + stage * L::STAGE_BYTES + wave * kGemmLoadBytes;
        if (l < A_LD)
            direct_load16(a_src + l * a_step + kt * a_kstep, base + l * 8 * kGemmLoadBytes);
        else if (DUAL_B)
            direct_load16(b_dual[l - A_LD] + kt * b_kstep, base + L::A_BYTES + (l - A_LD) * 8 * kGemmLoadBytes);
        else
            direct_load16(b_src + (l - A_LD) * b_step + kt * b_kstep,
                          base + L::A_BYTES + (l - A_LD) * 8 * kGemmLoadBytes);
    };
    auto issue = [&](int kt, int stage) {
#pragma unroll
        for (int l = 0; l < LOADS; ++l) issue_one(kt, stage, l);
    };

    // ---- LDS fragment addresses -------------------------------------------------------
    // v_mfma_f32_16x16x32 takes, per lane, 8 consecutive k of one row (first operand) or one
    // column (second operand): lane -> row/column lane%16, k-group lane/16.  The operands are
    // swapped — the B fragment goes in first, the A fragment second — so the accumulator tile is
    // C^T: lane (lane%16 = m, lane/16 = g) holds C[m][4g .. 4g+3] of its 16x16 tile, four
    // consecutive columns, which leave as one 8-byte store.
    // K-contiguous tiles: the fragment of 16 consecutive rows at one k-group; wave and MFMA tile
    // offsets are multiples of 16 rows, so the swizzle depends on the lane alone.
    const int l16 = lane & 15, g4 = lane >> 4;
    const int sw = (BK == 64) ? ((l16 & 7) ^ ((l16 >> 3) & 1)) : (BK == 32) ? ((l16 >> 2) & 3) : 0;
    constexpr int KS = BK / 32;  // MFMA k-steps per K tile
    int kx[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kx[ks] = ((ks * 4 + g4) ^ sw) << 4;
    const int a_frag = (wm * WTM + l16) * ROW_B;
    const int bt_frag = L::A_BYTES + (wn * WTN + l16) * ROW_B;
    // N-contiguous B tile ([k][n]) through ds_read_b64_tr_b16: inside each block of 16 lanes,
    // lane i supplies the address of 4 consecutive n at k-row (i/4) and receives 4 consecutive
    // k for column i.  Block g covers k-rows 8g .. 8g+7 of the k-step in two reads (rows 0-3
    // and 4-7 of its group), all four blocks the same 16 columns.
    int bn_frag[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int nchunk = (wn * WTN + j * 16) / 8 + ((l16 & 3) >> 1);
        bn_frag[j] = L::A_BYTES + (g4 * 8 + (l16 >> 2)) * RB_N + ((nchunk ^ (((l16 >> 2) & 3) << 2)) << 4) +
                     (l16 & 1) * 8;
    }
    // A operand from an M-contiguous tile ([k][m]): the same transposing reads, m for n
    int am_frag[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int mchunk = (wm * WTM + i * 16) / 8 + ((l16 & 3) >> 1);
        am_frag[i] = (g4 * 8 + (l16 >> 2)) * RB_M + ((mchunk ^ (((l16 >> 2) & 3) << 2)) << 4) + (l16 & 1) * 8;
    }

    f32x4 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto read_a = [&](int stage, int ks, int i) -> u32x4 {
        const lds_ptr base = lds + stage * L::STAGE_BYTES;
        if constexpr (TRANS_A) {
            const lds_ptr p = base + am_frag[i] + ks * 32 * RB_M;
            s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)p);
            s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p + 4 * RB_M));
            u32x2 lo2 = __builtin_bit_cast(u32x2, lo), hi2 = __builtin_bit_cast(u32x2, hi);
            return u32x4{lo2.x, lo2.y, hi2.x, hi2.y};
        } else {
            return *(const lds_u32x4 *)(base + a_frag + i * 16 * ROW_B + kx[ks]);
        }
    };
    auto read_b = [&](int stage, int ks, int j) -> u32x4 {
        const lds_ptr base = lds + stage * L::STAGE_BYTES;
        if constexpr (TRANS_B) {
            return *(const lds_u32x4 *)(base + bt_frag + j * 16 * ROW_B + kx[ks]);
        } else {
            const lds_ptr p = base + bn_frag[j] + ks * 32 * RB_N;
            s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)p);
            s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p + 4 * RB_N));
            u32x2 lo2 = __builtin_bit_cast(u32x2, lo), hi2 = __builtin_bit_cast(u32x2, hi);
            return u32x4{lo2.x, lo2.y, hi2.x, hi2.y};
        }
    };

    // ---- main loop -----------------------------------------------------------------
    // At the top of tile kt one barrier establishes two facts: tile kt+1 has landed for every
    // wave (each waited for its own loads first), and every wave is done reading tile kt-1,
    // whose stage is refilled right away.  Because tile kt+1 is already complete, the fragments
    // of its first k-step are read during the last k-step of tile kt: the MFMA queue stays fed
    // across the barrier.  Tiles kt+2 .. kt+S-1 are in flight meanwhile.  A tile index past the
    // last one is clamped: the extra loads land in a stage nobody reads again and keep the
    // number of outstanding loads the same in every iteration, so one constant vmcnt bound
    // serves the whole loop.
    //
    static_assert(S >= 3, "the ring needs the current, the next and one tile in flight");
    const int KT = k_len / BK;
    constexpr int B_DS = TRANS_B ? 1 : 2, A_DS = TRANS_A ? 2 : 1;  // LDS reads per fragment

    s.sync();  // the previous task is done with the stage buffers
#pragma unroll
    for (int p = 0; p < S - 1; ++p) issue(min(p, KT - 1), p);
    wait_vmcnt_then_barrier<(S - 2) * LOADS>();  // tile 0 is complete

    constexpr int A_SET = (MT >= 8 && NT >= 4) ? MT / 2 : MT;  // A fragments per register set (see below)
    u32x4 af[2][A_SET], bf[2][NT];
#pragma unroll
    for (int i = 0; i < A_SET; ++i) af[0][i] = read_a(0, 0, i);
#pragma unroll
    for (int j = 0; j < NT; ++j) bf[0][j] = read_b(0, 0, j);

    int stage = 0, fill = S - 1;  // fill: the free stage (tile kt-1's), refilled at the top of tile kt
    int refill = 0, next_stage = 0;
    auto tile_top = [&](int kt) {
        wait_vmcnt_then_barrier<(S - 3) * LOADS>();
        refill = min(kt + S - 1, KT - 1);
        next_stage = (stage + 1 == S) ? 0 : stage + 1;
    };
    auto tile_end = [&]() {
        stage = next_stage;
        fill = (fill + 1 == S) ? 0 : fill + 1;
    };
    // A k-step of a 256x256 tile runs in two phases, the upper and the lower half of the wave's
    // row tiles (PH = 2).  Phase H multiplies A fragment set H by the k-step's B fragments (set
    // CUR) and meanwhile reads A set H^1 for the phase after it plus half of the next k-step's B
    // fragments (set CUR^1): 16 fragments in registers instead of 24, which is what lets the body
    // share a kernel with others without spilling.  Smaller tiles run a k-step as one phase
    // (PH = 1) that reads the whole next k-step (their phases would be too short to cover the
    // LDS latency).  The reads are issued in the phase's first row tiles, the next phase's first
    // operands first, and its last row tile reads nothing, so every read has returned when the
    // phase ends (also at the barrier on top of a K tile).
    constexpr int PH = (MT >= 8 && NT >= 4) ? 2 : 1;
    constexpr int MH = MT / PH;              // row tiles per phase
    constexpr int NBH = (NT + PH - 1) / PH;  // B fragments read per phase
    constexpr int NREADS = MH + NBH;         // fragments read per phase
    constexpr int NRT = MH > 2 ? MH - (PH == 2 ? 1 : 2) : 1;  // row tiles of a phase that issue reads
    static_assert(MT % PH == 0, "the wave's row tiles split evenly over the phases");
    // fragment read R of phase H: a0 first, then the phase's B fragments, then the other A fragments
    auto read_one = [&](auto cur_c, auto h_c, auto r_c, int astage, int aks, int bstage, int bks) {
        constexpr int CUR = decltype(cur_c)::value, H = decltype(h_c)::value, R = decltype(r_c)::value;
        constexpr int ASET = PH == 2 ? (H ^ 1) : (CUR ^ 1);      // the A set being filled
        constexpr int AROW = PH == 2 ? (H ^ 1) * MH : 0;          // its first row tile
        constexpr int BJ0 = H * NBH;                              // first B fragment this phase reads
        if constexpr (R == 0) {
            af[ASET][0] = read_a(astage, aks, AROW);
        } else if constexpr (R <= NBH) {
            if constexpr (BJ0 + R - 1 < NT) bf[CUR ^ 1][BJ0 + R - 1] = read_b(bstage, bks, BJ0 + R - 1);
        } else {
            af[ASET][R - NBH] = read_a(astage, aks, AROW + R - NBH);
        }
    };
    auto row_tile = [&](auto cur_c, auto ks_c, auto h_c, auto i_c, int astage, int aks, int bstage, int bks) {
        constexpr int CUR = decltype(cur_c)::value, KS_I = decltype(ks_c)::value, H = decltype(h_c)::value,
                      I = decltype(i_c)::value;
        constexpr int ASET = PH == 2 ? H : CUR;
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[H * MH + I][j] = mfma16x32<T>(bf[CUR][j], af[ASET][I], acc[H * MH + I][j]);
        constexpr int R0 = I < NRT ? (I * NREADS) / NRT : NREADS, R1 = I < NRT ? ((I + 1) * NREADS) / NRT : NREADS;
        static_for<R1 - R0>([&](auto r_c) {
            read_one(cur_c, h_c, std::integral_constant<int, R0 + decltype(r_c)::value>{}, astage, aks, bstage, bks);
        });
        // LDS instructions of those reads
        constexpr int DS = [&]() constexpr {
            int n = 0;
            for (int r = R0; r < R1; ++r)
                n += (r == 0 || r > NBH) ? A_DS : ((H * NBH + r - 1 < NT) ? B_DS : 0);
            return n;
        }();
        // this row tile's share of the refill of the stage tile kt-1 used
        constexpr int P = KS_I * PH + H, NP = KS * PH;  // phase index inside the K tile
        constexpr int PL0 = (P * LOADS) / NP, PL1 = ((P + 1) * LOADS) / NP;
        constexpr int L0 = PL0 + (I * (PL1 - PL0)) / MH, L1 = PL0 + ((I + 1) * (PL1 - PL0)) / MH;
#pragma unroll
        for (int l = L0; l < L1; ++l) issue_one(refill, fill, l);
        // Issue order: the LDS reads and direct loads of a row tile sit between its MFMAs.  All
        // waves leave the barrier together; if each first issued its loads and reads back to
        // back, they would queue at the CU's one memory pipeline while the matrix cores wait.
        constexpr int HEAD = NT >= 2 ? NT / 2 : NT;
        __builtin_amdgcn_sched_group_barrier(0x008, HEAD, 0);  // MFMA
        if constexpr (DS > 0) __builtin_amdgcn_sched_group_barrier(0x100, DS, 0);  // LDS reads
        if constexpr (NT - HEAD > 0) __builtin_amdgcn_sched_group_barrier(0x008, NT - HEAD, 0);
        if constexpr (L1 - L0 > 0) __builtin_amdgcn_sched_group_barrier(0x020, L1 - L0, 0);  // direct loads
    };
    auto kstep = [&](auto cur_c, auto ks_c) {
        constexpr int KS_I = decltype(ks_c)::value;
        constexpr bool last = (KS_I + 1 == KS);
        const int nstage = last ? next_stage : stage;
        constexpr int nks = last ? 0 : KS_I + 1;
        if constexpr (PH == 2) {
            // phase 0 reads A for phase 1 of this k-step, phase 1 for phase 0 of the next one
            static_for<MH>([&](auto i_c) {
                row_tile(cur_c, ks_c, std::integral_constant<int, 0>{}, i_c, stage, KS_I, nstage, nks);
            });
            static_for<MH>([&](auto i_c) {
                row_tile(cur_c, ks_c, std::integral_constant<int, 1>{}, i_c, nstage, nks, nstage, nks);
            });
        } else {
            static_for<MH>([&](auto i_c) {
                row_tile(cur_c, ks_c, std::integral_constant<int, 0>{}, i_c, nstage, nks, nstage, nks);
            });
        }
    };
    using std::integral_constant;
    if constexpr (KS == 1) {
        // the B buffers alternate from tile to tile: two tiles per trip (K is a multiple of 64)
        for (int kt = 0; kt < KT; kt += 2) {
            tile_top(kt);
            kstep(integral_constant<int, 0>{}, integral_constant<int, 0>{});
            tile_end();
            tile_top(kt + 1);
            kstep(integral_constant<int, 1>{}, integral_constant<int, 0>{});
            tile_end();
        }
    } else {
        static_assert(KS == 2, "K tiles are 32 or 64 deep");
        for (int kt = 0; kt < KT; ++kt) {
            tile_top(kt);
            kstep(integral_constant<int, 0>{}, integral_constant<int, 0>{});
            kstep(integral_constant<int, 1>{}, integral_constant<int, 1>{});
            tile_end();
        }
    }
    // the clamped loads still in flight target LDS: they must land before the
    // buffers are used again (by the next task or another op body)
    wait_vmcnt_then_barrier<0>();

    // The wave's output: NTO column tiles of 16 per 16-row strip.  For the gate/up pair accumulator
    // tiles j and j + NT/2 of a wave hold the gate and the up product of the same 16 output columns.
    static_assert(!DUAL_B || NT % 2 == 0, "the gate/up pair needs an even number of column tiles per wave");
    constexpr int NTO = DUAL_B ? NT / 2 : NT;
    const int col_w = DUAL_B ? tn * (BN / 2) + wn * (WTN / 2) : n0 + wn * WTN;  // the wave's first output column
    const int out_n0 = DUAL_B ? tn * (BN / 2) : n0, out_bn = DUAL_B ? BN / 2 : BN;
    // Whole tiles of an aligned C go through LDS, strip by strip: a wave writes a strip of 16 rows
    // x (16 NTO) columns (8 bytes per lane and column tile) into a window of its own and reads it
    // back as 16 bytes per lane, LPR lanes to a row: every store instruction then writes whole row
    // segments (128 bytes, a cache line, for four column tiles), where the accumulator layout by
    // itself gives 32 bytes per row and instruction and the L2 writes some lines back more than
    // once.  No barrier inside: a wave's LDS operations complete in order and the window is the
    // wave's own (the stage ring is free: the K loop ended with every load landed and every wave
    // past its last fragment read).
    constexpr int SEG_B = NTO * 16 * 2;           // bytes of a strip's row
    constexpr int SPITCH = SEG_B + 16;            // padded: rows 16 bytes apart modulo the bank span
    constexpr int LPR = SEG_B / 16;               // lanes per row when reading back
    constexpr int RPP = 64 / LPR;                 // rows per pass
    constexpr bool kStaged = (64 % LPR == 0) && (RPP <= 16) && (16 % RPP == 0);
    // An elementwise op folded into the store (fuse_kind): the other operand's segments are
    // requested four strips ahead of their use (a strip takes a fraction of a memory round trip:
    // fetched one strip ahead, every strip waited for its segment).  The first four strips' here;
    // for a split tile two of them here, before the finisher waits for and adds the sender's
    // partial sums, and two after (the registers do not hold more beside the sums being added).
    constexpr int PASSES = kStaged ? 16 / RPP : 1;
    const int rrow = lane / LPR, rchunk = lane % LPR;
    const bool fuse = !DUAL_B && kStaged && d.fuse_kind != 0 && (!SPLIT || half == 0);
    // (four strips: with all eight of a 256-row tile requested at once, 64 more registers, the
    // kernel spilled 17 registers to scratch in every variant, and a plain 4096^3 matmul lost 4 %)
    constexpr int FW = MT < 4 ? MT : 4;  // strips requested ahead
    u32x4 oth[FW][PASSES];
    gptr<const T> other = as_global(static_cast<const T *>(d.fuse_other));
    gptr<T> fout = as_global(static_cast<T *>(d.fuse_out));
    int ocol = col_w + rchunk * 8;
    if (fuse && d.fuse_period > 0) ocol %= d.fuse_period;
    auto other_load = [&](int i, u32x4(&dst)[PASSES]) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int row = m0 + wm * WTM + i * 16 + p * RPP + rrow;
            dst[p] = *(const ARKMI_GLOBAL u32x4 *)(other + (int64_t)row * d.fuse_ld_other + ocol);
        }
    };
    constexpr int FIRST = SPLIT ? (FW < 2 ? FW : 2) : FW;
    if (fuse) {
#pragma unroll
        for (int i = 0; i < FIRST; ++i) other_load(i, oth[i]);
    }

    if constexpr (SPLIT) {
        // The partial sums cross from one XCD to another, whose L2s do not see each other:
        // 16-byte buffer stores and loads with the agent-scope bit (sc1), written through to
        // memory and read past this XCD's L2.  Ordering: every wave of the sender waits for its
        // stores to be acknowledged before the workgroup barrier, the word is set to full after
        // it; the finisher reads only after it has seen full, and sets empty only after its
        // last load has returned.
        constexpr int PER_THREAD = MT * NT;  // f32x4 values
        constexpr int kAgentScope = 16;      // cache-policy bit sc1 of the buffer instructions
        const int64_t tile_bytes = (int64_t)kGemmThreads * PER_THREAD * 16;
        char *tile_base = reinterpret_cast<char *>(d.partial) + (int64_t)task * tile_bytes;
        const __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc(tile_base, 0, (int)tile_bytes, 0x00020000);
        // [row tile * NT + column tile][thread]: a wave's store covers 1 KB in one piece
        const int at = tid * 16;
        unsigned int *word = d.arrivals + task;
        lds_i32x *verdict = (lds_i32x *)lds;
        if (tid == 0) *verdict = poll(word, half ? 0u : 1u) ? 1 : 0;
        s.sync();
        const bool go = *verdict != 0;
        s.sync();  // the verdict word is part of the stage buffers the next task refills
        if (!go) return kGemmAborted;
        if (half) {
#pragma unroll
            for (int i = 0; i < MT; ++i) {
#pragma unroll
                for (int j = 0; j < NT; ++j)
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[i][j]), rsrc,
                                                           at + (i * NT + j) * kGemmThreads * 16, 0, kAgentScope);
                __builtin_amdgcn_sched_barrier(0);  // row tile by row tile: no pile of addresses and values
            }
            drain_stores_then_barrier();
            if (tid == 0) __hip_atomic_store(word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return -1;
        }
        // the finisher: AHEAD row tiles of loads in flight while one is added
        constexpr int AHEAD = MT < 4 ? MT : 4;
        u32x4 in[AHEAD][NT];
#pragma unroll
        for (int i = 0; i < AHEAD; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
                in[i][j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, at + (i * NT + j) * kGemmThreads * 16, 0,
                                                                 kAgentScope);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
#pragma unroll
            for (int j = 0; j < NT; ++j) acc[i][j] += __builtin_bit_cast(f32x4, in[i % AHEAD][j]);
            if (i + AHEAD < MT) {
#pragma unroll
                for (int j = 0; j < NT; ++j)
                    in[i % AHEAD][j] = __builtin_amdgcn_raw_buffer_load_b128(
                        rsrc, at + ((i + AHEAD) * NT + j) * kGemmThreads * 16, 0, kAgentScope);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        wait_vmcnt_then_barrier<0>();
        if (tid == 0) __hip_atomic_store(word, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    if (fuse) {
#pragma unroll
        for (int i = FIRST; i < FW; ++i) other_load(i, oth[i]);
    }

    // ---- epilogue: lane (m = lane%16, g = lane/16) holds C[m][4g .. 4g+3] of each 16x16 tile ----
    // (store4 takes finished values: the epilogue hook or the gate/up product has been applied)
    const bool vec_ok = ((d.ldc & 3) == 0) && (((uintptr_t)d.c & 7) == 0) && ((d.c_bs[0] & 3) == 0) &&
                        ((d.c_bs[1] & 3) == 0);
    auto store4 = [&](int row, int col, float v0, float v1, float v2, float v3) {
        if (row >= d.store_m) return;
        gptr<T> p = C + (int64_t)row * d.ldc + col;
        if (vec_ok && col + 4 <= d.store_n) {
            T o[4] = {from_f32<T>(v0), from_f32<T>(v1), from_f32<T>(v2), from_f32<T>(v3)};
            u32x2 w;
            __builtin_memcpy(&w, o, 8);
            *(ARKMI_GLOBAL u32x2 *)p = w;
        } else {
            const float v[4] = {v0, v1, v2, v3};
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (col + e < d.store_n) p[e] = from_f32<T>(v[e]);
        }
    };
    auto value4 = [&](int i, int j, int row, int col, float *o) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if constexpr (DUAL_B) {
                const float g = acc[i][j][e], u = acc[i][j + NT / 2][e];
                o[e] = g / (1.f + __expf(-g)) * u;
            } else {
                o[e] = epi(acc[i][j][e], row, col + e);
            }
        }
    };
    if (kStaged && vec_ok && (d.ldc & 7) == 0 && (((uintptr_t)d.c & 15) == 0) && (d.c_bs[0] & 7) == 0 &&
        (d.c_bs[1] & 7) == 0 && m0 + BM <= d.store_m && out_n0 + out_bn <= d.store_n) {
        const lds_ptr win = lds + wave * (2 * 16 * SPITCH);
        // (two copies of the strip loop, chosen per tile: with the folded op's branches inside the
        // one loop its stores no longer ran together, and a matmul with nothing folded lost 2 %)
        auto strips = [&](auto folded_c) {
            constexpr bool FOLDED = decltype(folded_c)::value;
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const lds_ptr buf = win + (i & 1) * 16 * SPITCH;
                const int row = m0 + wm * WTM + i * 16 + l16;
#pragma unroll
                for (int j = 0; j < NTO; ++j) {
                    float o[4];
                    value4(i, j, row, col_w + j * 16 + 4 * g4, o);
                    T t[4] = {from_f32<T>(o[0]), from_f32<T>(o[1]), from_f32<T>(o[2]), from_f32<T>(o[3])};
                    u32x2 w;
                    __builtin_memcpy(&w, t, 8);
                    *(__attribute__((address_space(3))) u32x2 *)(buf + l16 * SPITCH + j * 32 + g4 * 8) = w;
                }
#pragma unroll
                for (int p = 0; p < 16 / RPP; ++p) {
                    const int r = p * RPP + rrow;
                    const u32x4 v = *(const lds_u32x4 *)(buf + r * SPITCH + rchunk * 16);
                    const int row_g = m0 + wm * WTM + i * 16 + r;
                    *(ARKMI_GLOBAL u32x4 *)(C + (int64_t)row_g * d.ldc + col_w + rchunk * 8) = v;
                    if constexpr (FOLDED)
                        *(ARKMI_GLOBAL u32x4 *)(fout + (int64_t)row_g * d.fuse_ld_out + col_w + rchunk * 8) =
                            fused_store_values<T>(d.fuse_kind - 1, d.fuse_c_second != 0, v, oth[i % FW][p]);
                }
                if constexpr (FOLDED) {
                    if (i + FW < MT) other_load(i + FW, oth[i % FW]);
                }
            }
        };
        if (fuse) strips(std::true_type{});
        else strips(std::false_type{});
        s.sync();  // the windows lie in the stage ring, which the next task (or another op body) fills
        return task;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int row = m0 + wm * WTM + i * 16 + l16;
#pragma unroll
        for (int j = 0; j < NTO; ++j) {
            const int col = col_w + j * 16 + 4 * g4;
            float o[4];
            value4(i, j, row, col, o);
            store4(row, col, o[0], o[1], o[2], o[3]);
        }
    }
    return task;
}

}  // namespace arkmi
