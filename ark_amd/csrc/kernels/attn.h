// Scaled-dot-product attention for gfx950, one pass over the keys per query
// block (online softmax): O = softmax(Q K^T * scale [+ causal mask]) V, head
// dimension 128, fp16 or bf16 operands, fp32 scores and accumulators, the
// probabilities rounded to the storage type before they meet V.
//
// It replaces the chain the reference's attention builds per layer
// (examples/llama/model.py:421-443): transpose q / k / v, Matmul(q, k^T) ->
// ScalarMul -> Add(mask) -> softmax (5 ops) -> Matmul(scores, v) -> transpose,
// which writes and re-reads the [heads, seq, seq] score tensor several times.
// Q, K, V and O are addressed through (batch, position, head) strides, so the
// [batch, seq, heads, head_dim] tensors the projections and RoPE produce are
// consumed as they are and no transpose is needed on either side.
//
// One task = 128 consecutive query positions of one (batch, head).  The eight
// waves form two groups of four; a wave owns 32 queries (two MFMA column tiles),
// and the two groups split the keys: keys are walked in steps of 128, group 0
// takes the lower 64 of a step, group 1 the upper 64, each with a running
// maximum, denominator and output of its own, and the two halves are merged
// once at the end of the task.  So every K and V fragment read from LDS feeds
// two MFMAs (32 queries per wave), while a task stays 128 queries, small enough
// to pair a long and a short one per workgroup under a causal mask.
//
// Everything is computed transposed so that a query's scores live in one
// lane's registers and the softmax needs almost no cross-lane traffic:
//   S^T[key, q] = K[key, :] . Q[q, :]     v_mfma_f32_16x16x32: A = K rows from
//                                         LDS, B = Q rows held in registers;
//   lane (q = lane%16, g = lane/16) then holds keys 4g..4g+3 of every 16-key tile;
//   O^T[d, q] += V^T[d, key] P^T[key, q]  A = V^T through ds_read_b64_tr_b16
//                                         from the [key][d] tile, B = P^T
//                                         straight from the score registers;
//   l[q]      += 1^T[., key] P^T[key, q]  the denominator from one more MFMA whose
//                                         A operand is all ones: the sum of the
//                                         rounded probabilities, no vector-ALU adds.
// The contraction order of the second product is "keys 4g..4g+3 of an even
// tile, then of the odd tile" per lane group, the same on both operands.
//
// K and V steps travel global -> LDS directly (global_load_lds_dwordx4), double
// buffered; a wave-level direct load fills 1 KB of consecutive LDS (four rows of
// 256 bytes), so instead of padding rows every lane fetches the 16-byte chunk that
// belongs at its LDS position under an XOR swizzle: chunk c of K row r sits at
// position c ^ (r & 15) (a ds_read_b128 of 16 rows at one chunk touches every bank
// once), chunk c of V row r at c ^ ((r & 7) << 1) (the transposing read's eight
// rows of 32 bytes per half wave fall into different banks).
//
// Vector-ALU work per score is what bounds this kernel next to the matrix cores
// (v_exp_f32 runs at quarter rate), so: the mask is applied only in steps that
// cross a query's last visible key, the accumulators are rescaled only when some
// lane's running maximum moved, and the scale is folded into the exponent's FMA.
// With a causal mask the steps above the diagonal are skipped, a wave skips a
// block none of its queries sees, and tasks are numbered so that a workgroup's
// two tasks are a long and a short query block of different heads.
#pragma once
#include "dev_common.h"
#include "gemm.h"

namespace arkmi {

struct AttnDesc {
    const void *q, *k, *v;
    void *o;
    int64_t q_s[3], k_s[3], v_s[3], o_s[3];  // element strides of batch, position, head
    int32_t batch, heads, seq_q, seq_k;
    float scale;
    int32_t causal;   // 1: key j is visible to query i iff j <= i + (seq_k - seq_q)
    int32_t dtype;    // 1 fp16, 2 bf16
    int32_t q_blocks; // ceil(seq_q / 128)
    // > 0: the tasks that run at once (task t on workgroup t mod xcd_round); the task index is then
    // permuted so that the query blocks an XCD (t mod 8) works on at a time belong to the same few
    // heads, whose K and V its L2 then fetches once instead of every XCD fetching every head's
    int32_t xcd_round;
};

constexpr int kAttnD = 128;        // head dimension
constexpr int kAttnQBlock = 128;   // query positions per task (32 per wave, four waves per group)
constexpr int kAttnKBlock = 64;    // keys per group and step
constexpr int kAttnStep = 2 * kAttnKBlock;            // keys per step of the workgroup
constexpr int kAttnRowBytes = kAttnD * 2;             // a K or V row in LDS
constexpr int kAttnTileBytes = kAttnStep * kAttnRowBytes;  // the K (or V) rows of a step
constexpr int kAttnStageBytes = 2 * kAttnTileBytes;   // K rows, then V rows
constexpr int kAttnLdsBytes = 2 * kAttnStageBytes;    // two stages: 128 KB

typedef float f32x2 __attribute__((ext_vector_type(2)));

template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    T v[2] = {from_f32<T>(lo), from_f32<T>(hi)};
    uint32_t r;
    __builtin_memcpy(&r, v, 4);
    return r;
}

template <typename T>
__device__ __forceinline__ uint32_t packed_ones();
template <>
__device__ __forceinline__ uint32_t packed_ones<f16>() { return 0x3C003C00u; }
template <>
__device__ __forceinline__ uint32_t packed_ones<bf16>() { return 0x3F803F80u; }

// max of three floats as one instruction; the operands are never NaN here, and the library's
// fmaxf would first canonicalise each of them with an instruction of its own
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// Number of tasks of an attention op.
inline int attn_num_tasks(int batch, int heads, int seq_q) {
    return batch * heads * ((seq_q + kAttnQBlock - 1) / kAttnQBlock);
}

template <typename T>
__device__ __forceinline__ void attn_task(const AttnDesc &d, int task_in, const Slot &s) {
    int task = task_in;
    if (d.xcd_round > 0) {
        // position ((round * 8 + xcd) * R / 8 + number within the XCD) of the (head, query block)
        // order below for a task of a full round of R; t and t + R keep their distance, so the
        // pairing of long and short query blocks on a workgroup stands
        const int R = d.xcd_round, total = d.batch * d.heads * d.q_blocks;
        if (task < (total / R) * R) {
            const int r = task / R, q = task - r * R;
            task = (r * 8 + (q & 7)) * (R >> 3) + (q >> 3);
        }
    }
    const int tid = s.tid, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2, wq = wave & 3;  // key half, and which 32 queries of the task
    const int qi = lane & 15, g = lane >> 4;
    const int QB = d.q_blocks;
    // task -> (batch*head, query block).  For the upper half of the (batch, head)
    // pairs the query blocks run backwards: with the tasks dealt round-robin, a
    // workgroup's task t and task t + ntasks/2 then add up to the same number of
    // key steps under a causal mask.
    int bh = task / QB, qb = task - bh * QB;
    if (d.causal && bh >= (d.batch * d.heads + 1) / 2) qb = QB - 1 - qb;
    const int b = bh / d.heads, h = bh - b * d.heads;
    const int q0 = qb * kAttnQBlock;

    gptr<const T> Q = as_global(static_cast<const T *>(d.q) + b * d.q_s[0] + h * d.q_s[2]);
    gptr<const T> K = as_global(static_cast<const T *>(d.k) + b * d.k_s[0] + h * d.k_s[2]);
    gptr<const T> V = as_global(static_cast<const T *>(d.v) + b * d.v_s[0] + h * d.v_s[2]);
    gptr<T> O = as_global(static_cast<T *>(d.o) + b * d.o_s[0] + h * d.o_s[2]);

    // ---- this lane's two query rows, as the B operands of the first product --------------
    const int wrow0 = q0 + wq * 32;  // the wave's first query row
    int qrow[2];
    u32x4 qf[2][kAttnD / 32];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        qrow[qt] = wrow0 + qt * 16 + qi;
        gptr<const T> qp = Q + (int64_t)min(qrow[qt], d.seq_q - 1) * d.q_s[1] + 8 * g;
#pragma unroll
        for (int ds = 0; ds < kAttnD / 32; ++ds) qf[qt][ds] = *(const ARKMI_GLOBAL u32x4 *)(qp + ds * 32);
    }
    // the last key each query may see; what the whole wave sees; what the whole task needs
    const int shift = d.seq_k - d.seq_q;
    int last_key[2];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) last_key[qt] = d.causal ? min(d.seq_k - 1, qrow[qt] + shift) : d.seq_k - 1;
    const int wave_last = d.causal ? min(d.seq_k - 1, wrow0 + 31 + shift) : d.seq_k - 1;   // uniform
    const int wave_first_last = d.causal ? min(d.seq_k - 1, wrow0 + shift) : d.seq_k - 1;  // uniform
    const int task_keys = d.causal ? min(d.seq_k, min(q0 + kAttnQBlock, d.seq_q) + shift) : d.seq_k;
    const int nsteps = (task_keys + kAttnStep - 1) / kAttnStep;

    // ---- global -> LDS ------------------------------------------------------------------------
    // A step's K tile is 128 rows = 32 wave-level loads of four rows, its V tile likewise: wave w
    // issues loads w, w + 8, w + 16, w + 24 of each.  The lane at (row lr of the four, position
    // pos) fetches the chunk that the swizzle puts there.
    // Addresses: a scalar base per load (uniform: step, load and wave pick the four rows) plus a
    // per-lane byte offset that holds for the whole task (the row of the four and the swizzled
    // chunk: the swizzle depends on (4 wave + lr) & 15 only), so a load costs no vector ALU work.
    // Only a step that reaches past the last key clamps its rows lane by lane.
    const int lr = lane >> 4, pos = lane & 15;
    const int row_lo = (wave * 4 + lr) & 15;
    const uint32_t k_lane = (uint32_t)((pos ^ row_lo) * 16), v_lane = (uint32_t)((pos ^ ((row_lo & 7) << 1)) * 16);
    const int k_pitch2 = (int)d.k_s[1] * 2, v_pitch2 = (int)d.v_s[1] * 2;  // bytes between rows
    // part i (0..3) of a step's loads: one load of K and one of V per wave
    auto issue_part = [&](int step, int stage, int i) {
        const lds_ptr kdst = s.lds + stage * kAttnStageBytes + wave * kGemmLoadBytes;
        const lds_ptr vdst = kdst + kAttnTileBytes;
        // rows key .. key + 3, those past the last key replaced by the last one (their scores are masked)
        const int key = min(step * kAttnStep + (i * 8 + wave) * 4, d.seq_k - 1);  // uniform
        const int dr = min(lr, d.seq_k - 1 - key);
        direct_load16_at(K + (int64_t)key * d.k_s[1], (uint32_t)(dr * k_pitch2) + k_lane, kdst + i * 8 * kGemmLoadBytes);
        direct_load16_at(V + (int64_t)key * d.v_s[1], (uint32_t)(dr * v_pitch2) + v_lane, vdst + i * 8 * kGemmLoadBytes);
    };
    auto issue_step = [&](int step, int stage) {
#pragma unroll
        for (int i = 0; i < 4; ++i) issue_part(step, stage, i);
    };

    // ---- running state: per query (lane%16), two queries per lane -----------------------------------
    const float c2 = d.scale * 1.4426950408889634f;  // scores are kept raw; exp(x*scale) = exp2(x*c2)
    constexpr float kNothing = -1.0e30f;  // below every score; finite, so that (kNothing * c2) stays finite
    float m_run[2] = {kNothing, kNothing};  // running maximum of the raw scores a query has seen
    f32x4 acc_o[2][kAttnD / 16], acc_l[2];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        acc_l[qt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < kAttnD / 16; ++dt) acc_o[qt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const uint32_t one2 = packed_ones<T>();
    const u32x4 ones = u32x4{one2, one2, one2, one2};

    // K fragment (A operand): key row = lane%16 of the 16-key tile, d = 32*ds + 8g .. +7, i.e.
    // chunk 4*ds + g, which sits at position (4*ds + g) ^ (row & 15) = (4*ds + g) ^ qi
    const int k_row = (grp * kAttnKBlock + qi) * kAttnRowBytes;
    int kx[kAttnD / 32];
#pragma unroll
    for (int ds = 0; ds < kAttnD / 32; ++ds) kx[ds] = ((4 * ds + g) ^ qi) << 4;
    // V^T fragment through the transposing read: in lane group g, lane i supplies the address of
    // d = 16*dt + 4*(i%4) .. +3 at key row 4g + i/4 and receives keys 4g..4g+3 for d = 16*dt + i.
    // Those 8 bytes lie in chunk 2*dt + (i%4)/2, at position (2*dt + (i%4)/2) ^ ((row & 7) << 1)
    // = 2*(dt ^ (row & 7)) + (i%4)/2.
    const int v_row = (grp * kAttnKBlock + 4 * g + (qi >> 2)) * kAttnRowBytes + (qi & 3) * 8;
    const int v_sw = ((4 * g + (qi >> 2)) & 7) << 5;

    s.sync();  // the previous task is done with the stage buffers
    if (nsteps > 0) issue_step(0, 0);
    for (int st = 0; st < nsteps; ++st) {
        // this step's tiles have landed for every wave, and every wave is done with the other stage
        wait_vmcnt_then_barrier<0>();
        if (st + 1 < nsteps) issue_step(st + 1, (st + 1) & 1);
        const int key_base = st * kAttnStep + grp * kAttnKBlock;  // this group's first key
        if (key_base > wave_last) continue;  // none of the wave's queries sees the block
        const lds_ptr kbase = s.lds + (st & 1) * kAttnStageBytes;
        const lds_ptr vbase = kbase + kAttnTileBytes;

        // ---- S^T = K Q^T for the block's four 16-key tiles, both query tiles ------------------
        // The K fragments of the next key tile are read while the current one is multiplied, and
        // the first V fragments of the second product are requested ahead of the softmax: the
        // compiler by itself waits for every handful of reads right before their first use.
        f32x4 sc[kAttnKBlock / 16][2];
        u32x4 kf[2][kAttnD / 32];
        auto read_k = [&](int kt, u32x4 *dst) {
#pragma unroll
            for (int ds = 0; ds < kAttnD / 32; ++ds)
                dst[ds] = *(const lds_u32x4 *)(kbase + k_row + kt * 16 * kAttnRowBytes + kx[ds]);
        };
        read_k(0, kf[0]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kt = 0; kt < kAttnKBlock / 16; ++kt) {
            if (kt + 1 < kAttnKBlock / 16) read_k(kt + 1, kf[(kt + 1) & 1]);
            sc[kt][0] = f32x4{0.f, 0.f, 0.f, 0.f};
            sc[kt][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ds = 0; ds < kAttnD / 32; ++ds) {
                sc[kt][0] = mfma16x32<T>(kf[kt & 1][ds], qf[0][ds], sc[kt][0]);
                sc[kt][1] = mfma16x32<T>(kf[kt & 1][ds], qf[1][ds], sc[kt][1]);
            }
            // one LDS read behind every second MFMA
            if (kt + 1 < kAttnKBlock / 16) {
#pragma unroll
                for (int i = 0; i < kAttnD / 32; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // V^T fragments: VG tiles of d per group, the next group in flight while one is multiplied
        constexpr int VG = 4, NVG = 2 * (kAttnD / 16) / VG;  // groups per block: (pr, dt / VG)
        u32x4 vf[2][VG];
        auto read_v = [&](int grp_i, u32x4 *dst) {
            const int pr = grp_i / (NVG / 2), dt0 = (grp_i % (NVG / 2)) * VG;
#pragma unroll
            for (int t = 0; t < VG; ++t) {
                const lds_ptr p = vbase + pr * 32 * kAttnRowBytes + v_row + (v_sw ^ ((dt0 + t) << 5));
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)p);
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p + 16 * kAttnRowBytes));
                const u32x2 lo2 = __builtin_bit_cast(u32x2, lo), hi2 = __builtin_bit_cast(u32x2, hi);
                dst[t] = u32x4{lo2.x, lo2.y, hi2.x, hi2.y};
            }
        };
        read_v(0, vf[0]);
        __builtin_amdgcn_sched_barrier(0);
        // ---- mask (only a block that reaches past some query's last key), running maximum ------
        if (key_base + kAttnKBlock - 1 > wave_first_last) {
            const int key0 = key_base + 4 * g;  // this lane's first key of tile 0
#pragma unroll
            for (int qt = 0; qt < 2; ++qt)
#pragma unroll
                for (int kt = 0; kt < kAttnKBlock / 16; ++kt)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (key0 + kt * 16 + r > last_key[qt]) sc[kt][qt][r] = -__builtin_inff();
        }
        float nm[2];  // -(new maximum) * c2
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
            float m_blk = max3_raw(max3_raw(sc[0][qt][0], sc[0][qt][1], sc[0][qt][2]), sc[0][qt][3], sc[1][qt][0]);
            m_blk = max3_raw(max3_raw(m_blk, sc[1][qt][1], sc[1][qt][2]), sc[1][qt][3], sc[2][qt][0]);
            m_blk = max3_raw(max3_raw(m_blk, sc[2][qt][1], sc[2][qt][2]), sc[2][qt][3], sc[3][qt][0]);
            m_blk = max3_raw(max3_raw(m_blk, sc[3][qt][1], sc[3][qt][2]), sc[3][qt][3], m_blk);
            m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 16, 64));
            m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 32, 64));
            const float m_new = fmaxf(m_run[qt], m_blk);
            if (m_new != m_run[qt]) {
                // (rare once a query has seen a few hundred keys)
                const float alpha = __builtin_amdgcn_exp2f((m_run[qt] - m_new) * c2);
                m_run[qt] = m_new;
                acc_l[qt] *= alpha;
#pragma unroll
                for (int dt = 0; dt < kAttnD / 16; ++dt) acc_o[qt][dt] *= alpha;
            }
            nm[qt] = -m_new * c2;
        }
        // ---- probabilities: exp2(score * c2 - max * c2); a masked score gives exp2(-inf) = 0 ----------
        u32x4 pf[2][kAttnKBlock / 32];
#pragma unroll
        for (int qt = 0; qt < 2; ++qt)
#pragma unroll
            for (int pr = 0; pr < kAttnKBlock / 32; ++pr) {
                float p[8];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    p[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[2 * pr][qt][r], c2, nm[qt]));
                    p[4 + r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[2 * pr + 1][qt][r], c2, nm[qt]));
                }
                pf[qt][pr] = u32x4{pack2<T>(p[0], p[1]), pack2<T>(p[2], p[3]), pack2<T>(p[4], p[5]), pack2<T>(p[6], p[7])};
            }
        // ---- O^T += V^T P^T, l += 1^T P^T ---------------------------------------------------------------
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int gi = 0; gi < NVG; ++gi) {
            const int pr = gi / (NVG / 2), dt0 = (gi % (NVG / 2)) * VG;
            if (gi + 1 < NVG) read_v(gi + 1, vf[(gi + 1) & 1]);
            if (dt0 == 0) {
                acc_l[0] = mfma16x32<T>(ones, pf[0][pr], acc_l[0]);
                acc_l[1] = mfma16x32<T>(ones, pf[1][pr], acc_l[1]);
            }
#pragma unroll
            for (int t = 0; t < VG; ++t) {
                acc_o[0][dt0 + t] = mfma16x32<T>(vf[gi & 1][t], pf[0][pr], acc_o[0][dt0 + t]);
                acc_o[1][dt0 + t] = mfma16x32<T>(vf[gi & 1][t], pf[1][pr], acc_o[1][dt0 + t]);
            }
            if (gi + 1 < NVG) {
#pragma unroll
                for (int i = 0; i < VG; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // ---- merge the two key halves ------------------------------------------------------------------
    // Group 0 finishes d = 0..63 of the task's outputs, group 1 d = 64..127: a wave leaves the
    // half it does not finish, with its maximum and denominator, in LDS for its partner (the
    // wave of the other group with the same queries).
    s.sync();  // every wave is done reading the stage buffers
    constexpr int HALF = kAttnD / 32;  // accumulator tiles per half of d
    {
        // [wave][query tile][tile of the half][lane] x 16 bytes, then [wave][query tile][lane] x 8 bytes
        const lds_ptr obase = s.lds + ((wave * 2) * HALF * 64 + lane) * 16;
        const lds_ptr mbase = s.lds + 8 * 2 * HALF * 64 * 16 + ((wave * 2) * 64 + lane) * 8;
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
#pragma unroll
            for (int t = 0; t < HALF; ++t)
                // (selected, not indexed: an index that is not a constant would put the accumulators in memory)
                *(__attribute__((address_space(3))) f32x4 *)(obase + (qt * HALF + t) * 64 * 16) =
                    grp ? acc_o[qt][t] : acc_o[qt][HALF + t];
            *(__attribute__((address_space(3))) f32x2 *)(mbase + qt * 64 * 8) = f32x2{m_run[qt], acc_l[qt][0]};
        }
    }
    s.sync();
    {
        const int pw = wave ^ 4;  // the partner
        const lds_ptr obase = s.lds + ((pw * 2) * HALF * 64 + lane) * 16;
        const lds_ptr mbase = s.lds + 8 * 2 * HALF * 64 * 16 + ((pw * 2) * 64 + lane) * 8;
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
            const f32x2 ml = *(__attribute__((address_space(3))) f32x2 *)(mbase + qt * 64 * 8);
            const float m = fmaxf(m_run[qt], ml.x);
            const float wa = __builtin_amdgcn_exp2f((m_run[qt] - m) * c2), wb = __builtin_amdgcn_exp2f((ml.x - m) * c2);
            const float l = acc_l[qt][0] * wa + ml.y * wb;
            const float inv = l > 0.f ? 1.0f / l : 0.f;
            const float fa = wa * inv, fb = wb * inv;
            if (qrow[qt] < d.seq_q) {
                gptr<T> op = O + (int64_t)qrow[qt] * d.o_s[1] + grp * (kAttnD / 2) + 4 * g;
#pragma unroll
                for (int t = 0; t < HALF; ++t) {
                    const f32x4 other = *(__attribute__((address_space(3))) f32x4 *)(obase + (qt * HALF + t) * 64 * 16);
                    const f32x4 mine = grp ? acc_o[qt][HALF + t] : acc_o[qt][t];
                    // the lane holds d = 64*grp + 16*t + 4g + r, r = 0..3: one 8-byte store
                    const u32x2 pk{pack2<T>(mine[0] * fa + other[0] * fb, mine[1] * fa + other[1] * fb),
                                   pack2<T>(mine[2] * fa + other[2] * fb, mine[3] * fa + other[3] * fb)};
                    *(ARKMI_GLOBAL u32x2 *)(op + t * 16) = pk;
                }
            }
        }
    }
    // (the next task's first barrier comes before anything writes the stage buffers again)
}

__device__ __forceinline__ void attn_dispatch(const AttnDesc &d, int task, const Slot &s) {
    if (d.dtype == 1) attn_task<f16>(d, task, s);
    else attn_task<bf16>(d, task, s);
}

}  // namespace arkmi
