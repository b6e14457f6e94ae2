// Device-side building blocks shared by every op body: storage types, 128-bit
// vector access, wave64 reductions, slot context.  gfx950 only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>
#include <utility>

namespace arkmi {

using f16 = _Float16;
using bf16 = __bf16;

constexpr int kWave = 64;

// ---- compile-time loops ---------------------------------------------------------
// static_for<N>(f) calls f(std::integral_constant<int, I>{}) for I = 0 .. N-1: for bodies whose
// instructions need the index as a constant (scheduling hints, register-array slots).
template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F &&f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// ---- storage <-> float ----------------------------------------------------
template <typename T>
__device__ __forceinline__ float to_f32(T v) {
    return static_cast<float>(v);
}
template <typename T>
__device__ __forceinline__ T from_f32(float v) {
    return static_cast<T>(v);  // RNE: v_cvt_f16_f32 / v_cvt_pk_bf16_f32
}

// ---- global address space ------------------------------------------------------
// Tensor data always lives in device (global) memory.  Pointers that reach an
// op body through a descriptor read from memory have no known address space,
// and the compiler would fall back to flat_load/flat_store, which also tie up
// the LDS counters; casting to address space 1 gives global_load/global_store.
#define ARKMI_GLOBAL __attribute__((address_space(1)))
template <typename T>
using gptr = ARKMI_GLOBAL T *;
template <typename T>
__device__ __forceinline__ gptr<T> as_global(T *p) {
    return (gptr<T>)p;
}

// ---- 16-byte vectors --------------------------------------------------------
template <typename T>
struct Vec16 {
    static constexpr int N = 16 / sizeof(T);
    T v[N];
};

template <typename T>
__device__ __forceinline__ Vec16<T> load16(gptr<const T> p) {
    using raw = __attribute__((ext_vector_type(4))) uint32_t;
    raw r = *(const ARKMI_GLOBAL raw *)p;
    Vec16<T> o;
    __builtin_memcpy(&o, &r, 16);
    return o;
}
// Streaming (read-once) variant: non-temporal hint keeps the row out of L2's
// way for data that is not reused.
template <typename T>
__device__ __forceinline__ Vec16<T> load16_nt(gptr<const T> p) {
    using raw = __attribute__((ext_vector_type(4))) uint32_t;
    raw r = __builtin_nontemporal_load((const ARKMI_GLOBAL raw *)p);
    Vec16<T> o;
    __builtin_memcpy(&o, &r, 16);
    return o;
}
template <typename T>
__device__ __forceinline__ void store16(gptr<T> p, const Vec16<T> &v) {
    using raw = __attribute__((ext_vector_type(4))) uint32_t;
    raw r;
    __builtin_memcpy(&r, &v, 16);
    *(ARKMI_GLOBAL raw *)p = r;
}
template <typename T>
__device__ __forceinline__ void store16_nt(gptr<T> p, const Vec16<T> &v) {
    using raw = __attribute__((ext_vector_type(4))) uint32_t;
    raw r;
    __builtin_memcpy(&r, &v, 16);
    __builtin_nontemporal_store(r, (ARKMI_GLOBAL raw *)p);
}

template <typename P>
__device__ __forceinline__ bool aligned16(P p) {
    return ((uintptr_t)p & 15) == 0;
}

// ---- wave64 all-reduce ------------------------------------------------------
// Steps 1,2,4,8 run on the DPP crossbar inside a row of 16 lanes (quad_perm,
// row_half_mirror, row_mirror); steps 16 and 32 cross rows through
// ds_bpermute (no LDS memory is touched).  Every lane ends with the result.
struct OpSum {
    __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
struct OpMax {
    __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};

template <int Ctrl>
__device__ __forceinline__ float dpp_move(float v) {
    int x = __builtin_bit_cast(int, v);
    int y = __builtin_amdgcn_update_dpp(x, x, Ctrl, 0xf, 0xf, false);
    return __builtin_bit_cast(float, y);
}

template <typename Op>
__device__ __forceinline__ float wave_allreduce(float v, Op op) {
    v = op(v, dpp_move<0xB1>(v));   // quad_perm:[1,0,3,2]
    v = op(v, dpp_move<0x4E>(v));   // quad_perm:[2,3,0,1]
    v = op(v, dpp_move<0x141>(v));  // row_half_mirror
    v = op(v, dpp_move<0x140>(v));  // row_mirror
    v = op(v, __shfl_xor(v, 16, 64));
    v = op(v, __shfl_xor(v, 32, 64));
    return v;
}

// ---- stores complete, then the workgroup meets ---------------------------------
// A workgroup barrier alone does not wait for a wave's global stores: the compiler
// emits no wait for a workgroup-scope release, and s_barrier does not drain the
// memory counters.  Where one thread goes on to tell other workgroups that this
// workgroup's data is in the L2 (an arrival atomic, a flag), every wave first waits
// until its own stores are acknowledged (vmcnt counts loads and stores on gfx9) and
// its LDS traffic is done, and only then joins the barrier.
__device__ __forceinline__ void drain_stores_then_barrier() {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---- slot context -----------------------------------------------------------
// A task runs on one "slot": a contiguous group of waves of the workgroup with
// its own LDS window.  With one resident slot per CU (the gfx950 default) the
// slot is the whole workgroup and sync() is a plain s_barrier.  A plan may run
// several narrower slots side by side (tasks of fewer warps than the workgroup
// has); their waves then meet on a counter in LDS, one per slot, as the
// reference does on this architecture (ark/include/kernels/common/sync.h:108-127).
using lds_ptr = __attribute__((address_space(3))) char *;
using lds_u32_ptr = __attribute__((address_space(3))) unsigned int *;

// ---- global -> LDS direct loads ----------------------------------------------------
// One wave-level load of 16 bytes per lane straight into LDS: lane i's bytes land at
// dst + 16 i (dst is uniform; it travels in M0).  Written as an instruction of its own
// rather than through the compiler's builtin: with loads of that builtin outstanding the
// compiler puts s_waitcnt vmcnt(0) in front of every ds_read_b64_tr_b16 (it cannot tell
// which LDS bytes a transposing read touches), which drains a ring's prefetch several times
// per tile in every layout that reads through the transposing instruction.  Completion is
// tracked by hand with vmcnt waits, as it has to be for the builtin too.  M0 is put back:
// the compiler owns that register.
template <typename P>
__device__ __forceinline__ void direct_load16(P src, lds_ptr dst) {
    const uint32_t m0v = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)dst);
    uint32_t keep;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(keep)
                 : "v"(src), "s"(m0v)
                 : "memory");
}
// The same with the address as a uniform base plus a 32-bit byte offset per lane.
template <typename P>
__device__ __forceinline__ void direct_load16_at(P base, uint32_t lane_bytes, lds_ptr dst) {
    const uint32_t m0v = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)dst);
    const uint64_t b = (uint64_t)base;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b), hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
    const uint64_t sb = ((uint64_t)hi << 32) | lo;
    uint32_t keep;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b32 m0, %0"
                 : "=&s"(keep)
                 : "v"(lane_bytes), "s"(sb), "s"(m0v)
                 : "memory");
}

constexpr unsigned kSlotSyncSpinLimit = 1u << 26;  // polls before a slot barrier gives up waiting

struct Slot {
    int tid;        // thread index inside the slot
    int nthreads;   // threads in the slot (multiple of 64)
    lds_ptr lds;    // slot's LDS window
    int lds_bytes;  // bytes in the window
    bool whole_block;
    // The slot's arrival counter (null for a slot that spans the workgroup).  It only
    // grows: with W waves per slot, barrier number g is complete when it reaches g * W.
    lds_u32_ptr arrivals = nullptr;
    __device__ __forceinline__ int lane() const { return tid & 63; }
    __device__ __forceinline__ int wave() const { return tid >> 6; }
    __device__ __forceinline__ int nwaves() const { return nthreads >> 6; }
    __device__ __forceinline__ void sync() const {
        if (whole_block || arrivals == nullptr) {
            __syncthreads();
            return;
        }
        if (nthreads <= 64) {  // one wave: nothing to meet, only this wave's own memory order
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
            __builtin_amdgcn_wave_barrier();
            return;
        }
        // this wave's LDS and global traffic is complete before it counts as arrived
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        if (lane() == 0) {
            const unsigned w = (unsigned)nwaves();
            const unsigned old = __hip_atomic_fetch_add(arrivals, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            const unsigned target = (old / w + 1u) * w;
            unsigned spins = 0;
            while ((int)(__hip_atomic_load(arrivals, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) - target) < 0) {
                __builtin_amdgcn_s_sleep(1);
                if (++spins > kSlotSyncSpinLimit) break;  // never hang the CU
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
        __builtin_amdgcn_wave_barrier();
    }
};

__device__ __forceinline__ Slot block_slot(lds_ptr lds, int lds_bytes) {
    Slot s;
    s.tid = threadIdx.x;
    s.nthreads = blockDim.x;
    s.lds = lds;
    s.lds_bytes = lds_bytes;
    s.whole_block = true;
    return s;
}

}  // namespace arkmi
