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
// One task = 128 consecutive query positions of one (batch, head): 16 per
// wave.  Everything is computed transposed so that a query's scores live in
// one lane's registers and the softmax needs almost no cross-lane traffic:
//   S^T[key, q] = K[key, :] . Q[q, :]     v_mfma_f32_16x16x32: A = K rows from
//                                         LDS, B = Q rows held in registers;
//   lane (q = lane%16, g = lane/16) then holds keys 4g..4g+3 of every 16-key tile;
//   O^T[d, q] += V^T[d, key] P^T[key, q]  A = V^T through ds_read_b64_tr_b16
//                                         from the [key][d] tile, B = P^T
//                                         straight from the score registers.
// The contraction order of the second product is "keys 4g..4g+3 of an even
// tile, then of the odd tile" per lane group, the same on both operands.
// Keys are walked in blocks of 64; K and V blocks are staged through LDS
// (double buffered), shared by the 8 waves.  With a causal mask the blocks
// above the diagonal are skipped, and tasks are numbered so that a workgroup's
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
constexpr int kAttnQBlock = 128;   // query positions per task (16 per wave)
constexpr int kAttnKBlock = 64;    // keys per step
constexpr int kAttnKPitch = kAttnD * 2 + 16;  // LDS row pitch of the K tile (bytes)
constexpr int kAttnVPitch = kAttnD * 2 + 32;  // LDS row pitch of the V tile (bytes)
constexpr int kAttnStageBytes = kAttnKBlock * (kAttnKPitch + kAttnVPitch);
constexpr int kAttnLdsBytes = 2 * kAttnStageBytes;

using f32x4v = f32x4;  // the 16x16x32 MFMA wrappers live in gemm.h

template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    T v[2] = {from_f32<T>(lo), from_f32<T>(hi)};
    uint32_t r;
    __builtin_memcpy(&r, v, 4);
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
    const int qi = lane & 15, g = lane >> 4;
    const int QB = d.q_blocks;
    // task -> (batch*head, query block).  For the upper half of the (batch, head)
    // pairs the query blocks run backwards: with the tasks dealt round-robin, a
    // workgroup's task t and task t + ntasks/2 then add up to the same number of
    // key blocks under a causal mask.
    int bh = task / QB, qb = task - bh * QB;
    if (d.causal && bh >= (d.batch * d.heads + 1) / 2) qb = QB - 1 - qb;
    const int b = bh / d.heads, h = bh - b * d.heads;
    const int q0 = qb * kAttnQBlock;

    gptr<const T> Q = as_global(static_cast<const T *>(d.q) + b * d.q_s[0] + h * d.q_s[2]);
    gptr<const T> K = as_global(static_cast<const T *>(d.k) + b * d.k_s[0] + h * d.k_s[2]);
    gptr<const T> V = as_global(static_cast<const T *>(d.v) + b * d.v_s[0] + h * d.v_s[2]);
    gptr<T> O = as_global(static_cast<T *>(d.o) + b * d.o_s[0] + h * d.o_s[2]);

    // ---- this lane's query row, as the B operand of the first product ------------------
    const int qrow = q0 + wave * 16 + qi;
    const bool q_ok = qrow < d.seq_q;
    u32x4 qf[kAttnD / 32];
    {
        gptr<const T> qp = Q + (int64_t)min(qrow, d.seq_q - 1) * d.q_s[1] + 8 * g;
#pragma unroll
        for (int ds = 0; ds < kAttnD / 32; ++ds) qf[ds] = *(const ARKMI_GLOBAL u32x4 *)(qp + ds * 32);
    }
    // the last key this query may see
    const int shift = d.seq_k - d.seq_q;
    const int last_key = d.causal ? min(d.seq_k - 1, qrow + shift) : d.seq_k - 1;
    // keys the whole task needs (uniform): up to the last query row's diagonal
    const int task_keys = d.causal ? min(d.seq_k, min(q0 + kAttnQBlock, d.seq_q) + shift) : d.seq_k;
    const int nblocks = (task_keys + kAttnKBlock - 1) / kAttnKBlock;

    // ---- global -> registers -> LDS staging of a K and a V block ------------------------
    // 64 rows x 256 B each: 1024 chunks of 16 B per tile, two per thread
    u32x4 kreg[2], vreg[2];
    const int ld_row = tid >> 4, ld_chunk = tid & 15;  // rows ld_row and ld_row + 32
    auto gload = [&](int kb) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int key = min(kb * kAttnKBlock + ld_row + 32 * i, d.seq_k - 1);
            kreg[i] = *(const ARKMI_GLOBAL u32x4 *)(K + (int64_t)key * d.k_s[1] + ld_chunk * 8);
            vreg[i] = *(const ARKMI_GLOBAL u32x4 *)(V + (int64_t)key * d.v_s[1] + ld_chunk * 8);
        }
    };
    auto lstore = [&](int stage) {
        const lds_ptr kbase = s.lds + stage * kAttnStageBytes;
        const lds_ptr vbase = kbase + kAttnKBlock * kAttnKPitch;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            *(lds_u32x4 *)(kbase + (ld_row + 32 * i) * kAttnKPitch + ld_chunk * 16) = kreg[i];
            *(lds_u32x4 *)(vbase + (ld_row + 32 * i) * kAttnVPitch + ld_chunk * 16) = vreg[i];
        }
    };

    // ---- running state: per query (lane%16) ----------------------------------------------
    const float c2 = d.scale * 1.4426950408889634f;  // scores are kept raw; exp(x*scale) = exp2(x*c2)
    float m_run = -3.0e38f;   // running maximum of the raw scores this query has seen
    float l_run = 0.f;        // this lane's share of the running denominator
    f32x4v acc_o[kAttnD / 16];
#pragma unroll
    for (int dt = 0; dt < kAttnD / 16; ++dt) acc_o[dt] = f32x4v{0.f, 0.f, 0.f, 0.f};

    const int i16 = lane & 15;
    // K fragment (A operand): key row = lane%16 of the 16-key tile, d = 32*ds + 8g .. +7
    const int k_frag = qi * kAttnKPitch + g * 16;
    // V^T fragment through the transposing read: in lane group g, lane i supplies
    // the address of d = 16*dt + 4*(i%4) .. +3 at key row 4g + i/4 and receives
    // keys 4g..4g+3 for d = 16*dt + i
    const int v_frag = (4 * g + (i16 >> 2)) * kAttnVPitch + (i16 & 3) * 8;

    s.sync();  // the previous task is done with the stage buffers
    if (nblocks > 0) {
        gload(0);
        lstore(0);
    }
    s.sync();
    for (int kb = 0; kb < nblocks; ++kb) {
        const int stage = kb & 1;
        if (kb + 1 < nblocks) gload(kb + 1);
        const lds_ptr kbase = s.lds + stage * kAttnStageBytes;
        const lds_ptr vbase = kbase + kAttnKBlock * kAttnKPitch;

        // ---- S^T = K Q^T for the block's four 16-key tiles ----------------------------------
        f32x4v sc[kAttnKBlock / 16];
#pragma unroll
        for (int kt = 0; kt < kAttnKBlock / 16; ++kt) {
            sc[kt] = f32x4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ds = 0; ds < kAttnD / 32; ++ds) {
                const u32x4 kf = *(const lds_u32x4 *)(kbase + kt * 16 * kAttnKPitch + k_frag + ds * 64);
                sc[kt] = mfma16x32<T>(kf, qf[ds], sc[kt]);
            }
        }
        // ---- mask, running maximum -------------------------------------------------------------
        const int key0 = kb * kAttnKBlock + 4 * g;  // this lane's first key of tile 0
        float m_blk = -3.0e38f;
#pragma unroll
        for (int kt = 0; kt < kAttnKBlock / 16; ++kt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = key0 + kt * 16 + r;
                if (key > last_key) sc[kt][r] = -3.0e38f;
                m_blk = fmaxf(m_blk, sc[kt][r]);
            }
        m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 16, 64));
        m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 32, 64));
        const float m_new = fmaxf(m_run, m_blk);
        const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c2);
        m_run = m_new;
        // ---- probabilities -----------------------------------------------------------------------
        float l_blk = 0.f;
        u32x4 pf[kAttnKBlock / 32];
#pragma unroll
        for (int pr = 0; pr < kAttnKBlock / 32; ++pr) {
            float p[8];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                // a masked score stays at -3e38: exp2 of it is 0 whatever m_new is
                p[r] = __builtin_amdgcn_exp2f((sc[2 * pr][r] - m_new) * c2);
                p[4 + r] = __builtin_amdgcn_exp2f((sc[2 * pr + 1][r] - m_new) * c2);
            }
            if (m_new <= -3.0e38f) {
#pragma unroll
                for (int e = 0; e < 8; ++e) p[e] = 0.f;  // nothing visible yet: exp2(0) would count masked keys
            }
            // the denominator sums the rounded probabilities, the values the second product uses
            pf[pr] = u32x4{pack2<T>(p[0], p[1]), pack2<T>(p[2], p[3]), pack2<T>(p[4], p[5]), pack2<T>(p[6], p[7])};
            T pv[8];
            __builtin_memcpy(pv, &pf[pr], 16);
#pragma unroll
            for (int e = 0; e < 8; ++e) l_blk += to_f32(pv[e]);
        }
        l_run = l_run * alpha + l_blk;
#pragma unroll
        for (int dt = 0; dt < kAttnD / 16; ++dt) acc_o[dt] *= alpha;
        // ---- O^T += V^T P^T ---------------------------------------------------------------------------
#pragma unroll
        for (int pr = 0; pr < kAttnKBlock / 32; ++pr) {
#pragma unroll
            for (int dt = 0; dt < kAttnD / 16; ++dt) {
                const lds_ptr p = vbase + pr * 32 * kAttnVPitch + v_frag + dt * 32;
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)p);
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p + 16 * kAttnVPitch));
                const u32x2 lo2 = __builtin_bit_cast(u32x2, lo), hi2 = __builtin_bit_cast(u32x2, hi);
                acc_o[dt] = mfma16x32<T>(u32x4{lo2.x, lo2.y, hi2.x, hi2.y}, pf[pr], acc_o[dt]);
            }
        }
        if (kb + 1 < nblocks) lstore(stage ^ 1);
        s.sync();
    }
    // ---- epilogue: O[q, d] = O^T[d, q] / l ------------------------------------------------------
    float l_tot = l_run + __shfl_xor(l_run, 16, 64);
    l_tot += __shfl_xor(l_tot, 32, 64);
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    if (q_ok) {
        gptr<T> op = O + (int64_t)qrow * d.o_s[1] + 4 * g;
#pragma unroll
        for (int dt = 0; dt < kAttnD / 16; ++dt) {
            // the lane holds d = 16*dt + 4g + r, r = 0..3: one 8-byte store
            const u32x2 pk{pack2<T>(acc_o[dt][0] * inv, acc_o[dt][1] * inv),
                           pack2<T>(acc_o[dt][2] * inv, acc_o[dt][3] * inv)};
            *(ARKMI_GLOBAL u32x2 *)(op + dt * 16) = pk;
        }
    }
}

__device__ __forceinline__ void attn_dispatch(const AttnDesc &d, int task, const Slot &s) {
    if (d.dtype == 1) attn_task<f16>(d, task, s);
    else attn_task<bf16>(d, task, s);
}

}  // namespace arkmi
