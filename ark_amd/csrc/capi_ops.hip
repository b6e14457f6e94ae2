// Stand-alone launchers of the op bodies (one kernel launch per op).
#include <atomic>

#include "host_common.h"
#include "host/ops.hpp"
#include "kernels/gemm.h"
#include "kernels/gemm_f32.h"
#include "kernels/gemv.h"
#include "kernels/row_ops.h"

namespace arkmi {

constexpr int kBlock = 512;  // 8 waves: one resident slot per CU in the loop kernel

template <typename T, int KIND>
__global__ __launch_bounds__(kBlock) void row_op_kernel(RowOpDesc d, int ntasks) {
    Slot s = block_slot(nullptr, 0);
    for (int t = blockIdx.x; t < ntasks; t += gridDim.x) row_op_task<T, KIND>(d, t, s);
}

template <typename T>
static void launch_row_op(const RowOpDesc &d, int ntasks, int grid, hipStream_t st) {
#define ARKMI_ROW_CASE(K)                                                                  \
    case K:                                                                                \
        hipLaunchKernelGGL((row_op_kernel<T, K>), dim3(grid), dim3(kBlock), 0, st, d, ntasks); \
        break;
    switch (d.kind) {
        ARKMI_ROW_CASE(ROW_SUM)
        ARKMI_ROW_CASE(ROW_MAX)
        ARKMI_ROW_CASE(ROW_MEAN)
        ARKMI_ROW_CASE(ROW_SOFTMAX)
        ARKMI_ROW_CASE(ROW_LAYERNORM)
        ARKMI_ROW_CASE(ROW_RMSNORM)
    }
#undef ARKMI_ROW_CASE
}

extern __shared__ __attribute__((aligned(16))) char g_dyn_lds[];

__device__ __forceinline__ lds_ptr dyn_lds() { return (lds_ptr)g_dyn_lds; }

template <typename T, int BM, int BN, bool TRANS_B, bool TRANS_A = false>
__global__ __launch_bounds__(kGemmThreads) void gemm_kernel(GemmDesc d, int ntasks) {
    Slot s = block_slot(dyn_lds(), GemmLds<BM, BN>::TOTAL_BYTES);
    for (int t = blockIdx.x; t < ntasks; t += gridDim.x)
        gemm_tile<T, BM, BN, TRANS_B, EpilogueStore, TRANS_A>(d, t, s, EpilogueStore());
}

template <typename T, int BM, int BN, bool TRANS_B, bool TRANS_A = false>
static void launch_gemm_variant(const GemmDesc &d, int ntasks, int grid, hipStream_t st) {
    auto kern = gemm_kernel<T, BM, BN, TRANS_B, TRANS_A>;
    constexpr int lds = GemmLds<BM, BN>::TOTAL_BYTES;
    static bool attr_set = false;  // per instantiation
    if (!attr_set) {
        ARKMI_HIP(hipFuncSetAttribute((const void *)kern,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kGemmThreads), lds, st, d, ntasks);
}

template <typename T, bool TRANS_B>
static void launch_gemm_tile(const GemmDesc &d, int bm, int bn, int ntasks, int grid,
                             hipStream_t st) {
    if (d.trans_a) {
        if (bm != 128 || bn != 128)
            ARKMI_FAIL(ARKMI_UNSUPPORTED, "a transposed first operand needs 128x128 tiles, got ", bm, "x", bn);
        launch_gemm_variant<T, 128, 128, TRANS_B, true>(d, ntasks, grid, st);
    } else if (bm == 256 && bn == 256)
        launch_gemm_variant<T, 256, 256, TRANS_B>(d, ntasks, grid, st);
    else if (bm == 128 && bn == 256)
        launch_gemm_variant<T, 128, 256, TRANS_B>(d, ntasks, grid, st);
    else if (bm == 256 && bn == 128)
        launch_gemm_variant<T, 256, 128, TRANS_B>(d, ntasks, grid, st);
    else if (bm == 128 && bn == 128)
        launch_gemm_variant<T, 128, 128, TRANS_B>(d, ntasks, grid, st);
    else
        ARKMI_FAIL(ARKMI_UNSUPPORTED, "no GEMM kernel for tile ", bm, "x", bn);
}

__global__ __launch_bounds__(kGemmThreads) void gemm_f32_kernel(GemmDesc d, int ntasks) {
    Slot s = block_slot(dyn_lds(), kGemmF32LdsBytes);
    for (int t = blockIdx.x; t < ntasks; t += gridDim.x) gemm_f32_dispatch(d, t, s);
}

static int env_int(const char *name, int dflt) {
    const char *v = getenv(name);
    return v ? atoi(v) : dflt;
}

}  // namespace arkmi

using namespace arkmi;

extern "C" int arkmi_row_op(int kind, int dtype, const void *in, void *out,
                            const void *weight, int weight_fp32, int64_t rows,
                            int64_t cols, int64_t in_ld, int64_t out_ld, float eps,
                            void *stream) {
    return guard([&] {
        if (kind < 0 || kind > 5) ARKMI_FAIL(ARKMI_INVALID_USAGE, "unknown row op kind ", kind);
        if (dtype != ARKMI_FP32 && dtype != ARKMI_FP16 && dtype != ARKMI_BF16)
            ARKMI_FAIL(ARKMI_UNSUPPORTED, "row ops support fp32/fp16/bf16, got dtype ", dtype);
        if (rows < 0 || cols <= 0 || cols > INT32_MAX)
            ARKMI_FAIL(ARKMI_INVALID_USAGE, "bad shape rows=", rows, " cols=", cols);
        if (rows == 0) return;
        if (!in || !out) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null tensor pointer");
        if (in_ld < cols) ARKMI_FAIL(ARKMI_INVALID_USAGE, "in_ld ", in_ld, " < cols ", cols);
        const bool is_reduce = kind <= 2;
        if (out_ld < (is_reduce ? 1 : cols))
            ARKMI_FAIL(ARKMI_INVALID_USAGE, "out_ld ", out_ld, " too small");
        RowOpDesc d{};
        d.in = in;
        d.out = out;
        d.weight = weight;
        d.rows = rows;
        d.cols = (int32_t)cols;
        d.dim_c = 1;
        d.dim_h = (int32_t)std::min<int64_t>(rows, INT32_MAX);
        if (rows > INT32_MAX) ARKMI_FAIL(ARKMI_UNSUPPORTED, "too many rows");
        d.in_s[0] = d.in_s[1] = 0;
        d.in_s[2] = in_ld;
        d.out_s[0] = d.out_s[1] = 0;
        d.out_s[2] = out_ld;
        d.eps = eps;
        d.kind = kind;
        d.dtype = dtype;
        d.weight_fp32 = weight_fp32;
        const int waves = kBlock / 64;
        int64_t ntasks = (rows + waves - 1) / waves;
        const auto &facts = device_facts(current_device());
        int per_cu = env_int("ARKMI_ROW_BLOCKS_PER_CU", 2);
        int grid = (int)std::min<int64_t>(ntasks, (int64_t)facts.num_cu * per_cu);
        if (dtype == ARKMI_FP32)
            launch_row_op<float>(d, (int)ntasks, grid, (hipStream_t)stream);
        else if (dtype == ARKMI_FP16)
            launch_row_op<f16>(d, (int)ntasks, grid, (hipStream_t)stream);
        else
            launch_row_op<bf16>(d, (int)ntasks, grid, (hipStream_t)stream);
        ARKMI_HIP(hipGetLastError());
    });
}

extern "C" int arkmi_gemm(int dtype, const void *a, const void *b, void *c, int batch, int m,
                          int n, int k, int64_t lda, int64_t ldb, int64_t ldc,
                          int64_t batch_stride_a, int64_t batch_stride_b,
                          int64_t batch_stride_c, int trans_a, int trans_b, int tile_m,
                          int tile_n, void *stream) {
    return guard([&] {
        if (dtype != ARKMI_FP16 && dtype != ARKMI_BF16 && dtype != ARKMI_FP32)
            ARKMI_FAIL(ARKMI_UNSUPPORTED, "MFMA GEMM supports fp32/fp16/bf16, got dtype ", dtype);
        const bool f32 = (dtype == ARKMI_FP32);
        if (batch < 0 || m < 0 || n < 0 || k < 0) ARKMI_FAIL(ARKMI_INVALID_USAGE, "negative size");
        if (batch == 0 || m == 0 || n == 0) return;
        if (!a || !b || !c) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null tensor pointer");
        if (k % kGemmMinK != 0 || k == 0)
            ARKMI_FAIL(ARKMI_UNSUPPORTED, "K must be a positive multiple of ", kGemmMinK, ", got ", k);
        // the one tile shape of a transposed A and of fp32 operands
        if ((trans_a || f32) && (tile_m == 0 || tile_n == 0)) tile_m = tile_n = 128;
        if (f32 && (tile_m != 128 || tile_n != 128))
            ARKMI_FAIL(ARKMI_UNSUPPORTED, "fp32 operands need 128x128 tiles, got ", tile_m, "x", tile_n);
        if (tile_m == 0 || tile_n == 0) {
            // largest tile that divides the problem and still fills the chip
            const int cand[4][2] = {{256, 256}, {128, 256}, {256, 128}, {128, 128}};
            const auto &facts = device_facts(current_device());
            tile_m = tile_n = 0;
            for (auto &t : cand) {
                if (m % t[0] || n % t[1]) continue;
                int64_t tasks = (int64_t)batch * (m / t[0]) * (n / t[1]);
                if (tile_m == 0) { tile_m = t[0]; tile_n = t[1]; }
                if (tasks >= facts.num_cu) { tile_m = t[0]; tile_n = t[1]; break; }
            }
            if (tile_m == 0)
                ARKMI_FAIL(ARKMI_UNSUPPORTED, "M and N must be multiples of 128 (got ", m, "x", n,
                           "); pad the tensors as the plan format allows");
        }
        if (m % tile_m || n % tile_n)
            ARKMI_FAIL(ARKMI_INVALID_USAGE, "tile ", tile_m, "x", tile_n, " does not divide ", m, "x", n);
        if (lda < (trans_a ? m : k) || ldc < n || ldb < (trans_b ? k : n))
            ARKMI_FAIL(ARKMI_INVALID_USAGE, "leading dimension too small");
        const int vec = f32 ? 4 : 8;  // elements per 16-byte vector
        if ((lda % vec) || (ldb % vec) || ((uintptr_t)a & 15) || ((uintptr_t)b & 15))
            ARKMI_FAIL(ARKMI_UNSUPPORTED,
                       "operands must be 16-byte aligned with leading dimensions of whole 16-byte vectors");
        GemmDesc d{};
        d.a = a; d.b = b; d.c = c;
        d.m = m; d.n = n; d.k = k;
        d.lda = (int)lda; d.ldb = (int)ldb; d.ldc = (int)ldc;
        d.a_bs[0] = d.b_bs[0] = d.c_bs[0] = 0;
        d.a_bs[1] = batch_stride_a; d.b_bs[1] = batch_stride_b; d.c_bs[1] = batch_stride_c;
        d.batch_c = batch; d.batch_total = batch; d.split_k = 1; d.trans_b = trans_b; d.trans_a = trans_a ? 1 : 0; d.dtype = dtype;
        d.tiles_m = m / tile_m; d.tiles_n = n / tile_n;
        d.store_m = m; d.store_n = n;
        int64_t ntasks = (int64_t)batch * d.tiles_m * d.tiles_n;
        if (ntasks > INT32_MAX) ARKMI_FAIL(ARKMI_UNSUPPORTED, "too many tiles");
        const auto &facts = device_facts(current_device());
        int grid = (int)std::min<int64_t>(ntasks, facts.num_cu);
        hipStream_t st = (hipStream_t)stream;
        if (f32) {
            hipLaunchKernelGGL(gemm_f32_kernel, dim3(grid), dim3(kGemmThreads), kGemmF32LdsBytes, st, d, (int)ntasks);
        } else if (dtype == ARKMI_FP16) {
            if (trans_b) launch_gemm_tile<f16, true>(d, tile_m, tile_n, (int)ntasks, grid, st);
            else launch_gemm_tile<f16, false>(d, tile_m, tile_n, (int)ntasks, grid, st);
        } else {
            if (trans_b) launch_gemm_tile<bf16, true>(d, tile_m, tile_n, (int)ntasks, grid, st);
            else launch_gemm_tile<bf16, false>(d, tile_m, tile_n, (int)ntasks, grid, st);
        }
        ARKMI_HIP(hipGetLastError());
    });
}

// ---- skinny matmul ---------------------------------------------------------------
namespace arkmi {

template <typename T>
__global__ __launch_bounds__(kBlock) void gemv_kernel(GemvDesc d, int ntasks) {
    Slot s = block_slot(dyn_lds(), kGemvLdsBytes);
    gemv_tasks<T>(d, blockIdx.x, gridDim.x, ntasks, s);
}

}  // namespace arkmi

extern "C" int arkmi_gemv_plan(int m, int n, int k, int num_tasks, int *num_tasks_out,
                               size_t *workspace_bytes) {
    return guard([&] {
        if (m < 1 || m > 16 || n < 1 || k < 1)
            ARKMI_FAIL(ARKMI_INVALID_USAGE, "the skinny matmul takes 1..16 rows and positive N, K");
        if (num_tasks < 0) ARKMI_FAIL(ARKMI_INVALID_USAGE, "negative task count");
        if (num_tasks == 0) num_tasks = device_facts(current_device()).num_cu;
        GemvDesc d{};
        d.m = m; d.n = n; d.k = k;
        const size_t bytes = gemv_partition(d, num_tasks);
        if (num_tasks_out) *num_tasks_out = d.num_tasks;
        if (workspace_bytes) *workspace_bytes = bytes;
    });
}

namespace arkmi {

constexpr int kMaxDevices = 64;

// What a skinny matmul asks of its operands; checked before anything is launched or written.
static void check_gemv_operands(const void *x, const void *w, const void *y, int n, int k, int64_t ldx, int64_t ldw,
                                int64_t ldy) {
    if (!x || !w || !y) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null tensor pointer");
    if (ldx < k || ldw < n || ldy < n) ARKMI_FAIL(ARKMI_INVALID_USAGE, "leading dimension too small");
    if ((n % 8) || (ldx % 8) || (ldw % 8) || ((uintptr_t)x & 15) || ((uintptr_t)w & 15))
        ARKMI_FAIL(ARKMI_UNSUPPORTED, "operands must be 16-byte aligned with N and leading dimensions % 8 == 0");
}

// Fills the descriptor of a skinny matmul whose operands passed check_gemv_operands and launches
// it with `workspace` (counters first, then partials) of at least the planned size.
static void launch_gemv(int dtype, const void *x, const void *w, void *y, int m, int n, int k, int64_t ldx,
                        int64_t ldw, int64_t ldy, int num_tasks, void *workspace, hipStream_t st) {
    GemvDesc d{};
    d.x = x; d.w = w; d.y = y;
    d.m = m; d.n = n; d.k = k;
    d.ldx = (int)ldx; d.ldw = (int)ldw; d.ldy = (int)ldy;
    d.dtype = dtype;
    gemv_partition(d, num_tasks);
    d.counters = static_cast<unsigned int *>(workspace);
    d.partial = reinterpret_cast<float *>(static_cast<char *>(workspace) + gemv_counter_bytes(d.n_blocks));
    // (set once per type and device; two threads that both find it unset both set it, which is harmless)
    static std::atomic<bool> attr_set[2][kMaxDevices];
    const int ti = dtype == ARKMI_FP16 ? 0 : 1;
    const int dev = current_device();
    if (dev < 0 || dev >= kMaxDevices) ARKMI_FAIL(ARKMI_UNSUPPORTED, "device index ", dev, " out of range");
    const void *kern = ti == 0 ? (const void *)gemv_kernel<f16> : (const void *)gemv_kernel<bf16>;
    if (!attr_set[ti][dev].load(std::memory_order_acquire)) {
        ARKMI_HIP(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, kGemvLdsBytes));
        attr_set[ti][dev].store(true, std::memory_order_release);
    }
    int ntasks = d.num_tasks;
    void *args[] = {&d, &ntasks};
    ARKMI_HIP(hipLaunchKernel(kern, dim3(ntasks), dim3(kBlock), args, kGemvLdsBytes, st));
}

// ---- the skinny matmul with its workspace inside the library ------------------------
// Device memory that belongs to the code object: every GPU the library runs on holds its
// own copy at its own address until the process ends.  In host code the array's name is a
// stand-in, not a device address; the address of a device's copy comes from
// hipGetSymbolAddress with that device current, once per device.
constexpr size_t kGemvStaticBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char g_gemv_scratch[kGemvStaticBytes];

// per device, null until resolved (threads that race to resolve a device store the same address)
static std::atomic<void *> g_gemv_scratch_ptr[kMaxDevices];

static void *gemv_static_workspace() {
    const int dev = current_device();
    if (dev < 0 || dev >= kMaxDevices) ARKMI_FAIL(ARKMI_UNSUPPORTED, "device index ", dev, " out of range");
    void *p = g_gemv_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        ARKMI_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(g_gemv_scratch)));
        if (!p) ARKMI_FAIL(ARKMI_GPU_ERROR, "the library's static workspace has no address on device ", dev);
        g_gemv_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    return p;
}

// Zero fill by a kernel: callers may be under stream capture, where memset nodes are avoided.
__global__ void zero_words_kernel(unsigned int *p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

}  // namespace arkmi

extern "C" int arkmi_gemv(int dtype, const void *x, const void *w, void *y, int m, int n, int k,
                          int64_t ldx, int64_t ldw, int64_t ldy, int num_tasks, void *workspace,
                          size_t workspace_bytes, void *stream) {
    return guard([&] {
        if (dtype != ARKMI_FP16 && dtype != ARKMI_BF16)
            ARKMI_FAIL(ARKMI_UNSUPPORTED, "the skinny matmul supports fp16/bf16, got dtype ", dtype);
        size_t need = 0;
        if (int rc = arkmi_gemv_plan(m, n, k, num_tasks, &num_tasks, &need))
            throw Error(rc, arkmi_last_error());
        if (!workspace || workspace_bytes < need)
            ARKMI_FAIL(ARKMI_INVALID_USAGE, "workspace of ", need, " bytes needed, got ", workspace_bytes);
        check_gemv_operands(x, w, y, n, k, ldx, ldw, ldy);
        launch_gemv(dtype, x, w, y, m, n, k, ldx, ldw, ldy, num_tasks, workspace, (hipStream_t)stream);
    });
}

extern "C" size_t arkmi_gemv_static_limit(void) { return arkmi::kGemvStaticBytes; }

extern "C" int arkmi_gemv_static(int dtype, const void *x, const void *w, void *y, int m, int n, int k,
                                 int64_t ldx, int64_t ldw, int64_t ldy, int num_tasks, void *stream) {
    return guard([&] {
        if (dtype != ARKMI_FP16 && dtype != ARKMI_BF16)
            ARKMI_FAIL(ARKMI_UNSUPPORTED, "the skinny matmul supports fp16/bf16, got dtype ", dtype);
        size_t need = 0;
        if (int rc = arkmi_gemv_plan(m, n, k, num_tasks, &num_tasks, &need))
            throw Error(rc, arkmi_last_error());
        if (need > kGemvStaticBytes)
            ARKMI_FAIL(ARKMI_UNSUPPORTED, "this shape needs ", need, " bytes of workspace; the library's static workspace holds ",
                       kGemvStaticBytes, " (use arkmi_gemv with a workspace of your own)");
        // a call that is going to be refused leaves the shared workspace alone
        check_gemv_operands(x, w, y, n, k, ldx, ldw, ldy);
        void *ws = gemv_static_workspace();
        hipStream_t st = (hipStream_t)stream;
        // the array keeps whatever the last call left: the arrival counters must start at zero
        const int n_blocks = (n + kGemvCols - 1) / kGemvCols;
        const int words = (int)(gemv_counter_bytes(n_blocks) / 4);
        hipLaunchKernelGGL(zero_words_kernel, dim3((words + 255) / 256), dim3(256), 0, st, static_cast<unsigned int *>(ws), words);
        ARKMI_HIP(hipGetLastError());
        launch_gemv(dtype, x, w, y, m, n, k, ldx, ldw, ldy, num_tasks, ws, st);
    });
}

// ---- measurement probes: what the machine sustains, beside the datasheet peaks ------
namespace arkmi {

// Every wave runs `iters` rounds of 16 independent v_mfma_f32_16x16x32_f16 on operand registers
// loaded from `operands` (random data draws more power than zeros, and the chip clocks down).
__global__ __launch_bounds__(kBlock) void probe_mfma_kernel(const u32x4 *operands, int iters, float *sink) {
    u32x4 a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a[i] = operands[(threadIdx.x + i * kBlock) & 65535];
        b[i] = operands[(threadIdx.x + i * kBlock + 7777) & 65535];
    }
    f32x4 acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = mfma16x32<f16>(a[i & 3], b[i >> 2], acc[i]);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    if (s == 1234567.f) sink[0] = s;  // keeps the loop alive
}

// Streams `bytes` from src as 16-byte vectors, 4 in flight per thread; writes them to dst when
// given (a copy), else folds them into a value that is (practically never) stored.
__global__ __launch_bounds__(256) void probe_stream_kernel(const u32x4 *src, u32x4 *dst, size_t n_vec, uint32_t *sink) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    u32x4 acc = {0, 0, 0, 0};
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec; i += 4 * stride) {
        u32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (i + u * stride < n_vec) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (i + u * stride < n_vec) {
                if (dst) __builtin_nontemporal_store(v[u], dst + i + u * stride);
                else acc ^= v[u];
            }
    }
    if (!dst && (acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = acc.x;
}

}  // namespace arkmi

extern "C" int arkmi_probe_mfma(const void *operands, size_t operand_bytes, int iters, void *sink, double *flops,
                                void *stream) {
    return guard([&] {
        if (!operands || !sink || operand_bytes < (size_t)65536 * 16)
            ARKMI_FAIL(ARKMI_INVALID_USAGE, "the MFMA probe reads 1 MiB of operand data and needs a 4-byte sink");
        if (iters < 1) ARKMI_FAIL(ARKMI_INVALID_USAGE, "iters must be positive");
        const int grid = device_facts(current_device()).num_cu;
        hipLaunchKernelGGL(probe_mfma_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream,
                           static_cast<const u32x4 *>(operands), iters, static_cast<float *>(sink));
        ARKMI_HIP(hipGetLastError());
        if (flops) *flops = (double)grid * (kBlock / 64) * (double)iters * 16.0 * (2.0 * 16 * 16 * 32);
    });
}

extern "C" int arkmi_probe_stream(const void *src, void *dst, size_t bytes, void *sink, void *stream) {
    return guard([&] {
        if (!src || !sink || (bytes % 16) || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15))
            ARKMI_FAIL(ARKMI_INVALID_USAGE, "the stream probe takes 16-byte aligned buffers of whole 16-byte vectors");
        const int grid = device_facts(current_device()).num_cu * 8;
        hipLaunchKernelGGL(probe_stream_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream,
                           static_cast<const u32x4 *>(src), static_cast<u32x4 *>(dst), bytes / 16,
                           static_cast<uint32_t *>(sink));
        ARKMI_HIP(hipGetLastError());
    });
}
