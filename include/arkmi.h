/*
 * arkmi — C ABI of the MI355X (gfx950) execution backend for the ARK model API.
 *
 * Everything the C++ `ark::` facade (the headers under include/ark) and any foreign-language
 * binding need crosses this boundary: plain pointers, sizes and NUL-terminated
 * strings, `int` status returns, no exceptions, no framework types.
 *
 * Status codes mirror the reference's error classes (ark/include/ark/error.hpp:
 * 13-43).  After a non-zero return, arkmi_last_error() gives the message for
 * the calling thread.
 *
 * Device pointers are raw HIP device addresses.  `stream` is a hipStream_t
 * passed as void* (NULL = the default stream).  Handles are not thread-safe;
 * distinct handles are independent.
 */
#ifndef ARKMI_H_
#define ARKMI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum arkmi_status {
    ARKMI_OK = 0,
    ARKMI_INTERNAL_ERROR = 1,      /* ark::InternalError */
    ARKMI_INVALID_USAGE = 2,       /* ark::InvalidUsageError */
    ARKMI_MODEL_ERROR = 3,         /* ark::ModelError */
    ARKMI_PLAN_ERROR = 4,          /* ark::PlanError */
    ARKMI_UNSUPPORTED = 5,         /* ark::UnsupportedError */
    ARKMI_SYSTEM_ERROR = 6,        /* ark::SystemError */
    ARKMI_GPU_ERROR = 7            /* ark::GpuError */
};

/* Element types; numbering is this library's own.  Names follow
 * ark/include/ark/data_type.hpp:14-22. */
enum arkmi_dtype {
    ARKMI_FP32 = 0,
    ARKMI_FP16 = 1,
    ARKMI_BF16 = 2,
    ARKMI_INT32 = 3,
    ARKMI_UINT32 = 4,
    ARKMI_INT8 = 5,
    ARKMI_UINT8 = 6,
    ARKMI_BYTE = 7
};

const char *arkmi_last_error(void);
const char *arkmi_version(void);

/* ark::init() (ark/api/init.cpp:15-19): reads the ARK_* environment variables again
 * (ARK_LOG_LEVEL, ARK_ENFORCE_PLAN_PATH, ...); they are otherwise read once, on first use.
 * This backend keeps no temporary directory, so there is nothing else to set up. */
int arkmi_init(void);

/* Device facts the planner reads (ark/gpu/gpu_manager.cpp:29-75: num_sm, arch
 * name, max threads/LDS).  arch is written as "ROCM_950" style text. */
typedef struct arkmi_device_info {
    int device_id;
    int num_cu;
    int wave_size;
    int max_threads_per_block;
    int lds_bytes_per_cu;
    int l2_bytes;
    size_t hbm_bytes;
    int clock_khz;
    char arch[32];
    char gcn_arch[64];
} arkmi_device_info;

int arkmi_device_info_get(int device_id, arkmi_device_info *out);

/* ------------------------------------------------------------------------
 * Stand-alone op launchers: one kernel launch per op on `stream`.  They run
 * the same device op bodies the persistent loop kernel runs, and serve (i) the
 * "same ops as separate kernels" comparison and (ii) per-op parity tests, the
 * role ark/ops/ops_test_common.cpp:34-224 (op_test) plays in the reference.
 * ---------------------------------------------------------------------- */

/* Row ops over the last axis of a dense-last-axis 4-D view.
 * kind: 0 reduce_sum, 1 reduce_max, 2 reduce_mean   (ark/ops/ops_reduce.cpp:11-127,
 *                                                    ark/include/kernels/reduce.h:341-498)
 *       3 softmax        (python/ark/ops.py:491-500)
 *       4 layernorm      (python/ark/ops.py:503-513; eps, no affine)
 *       5 rmsnorm        (examples/llama/model.py:92-99; weight optional)
 * rows = N*C*H positions; for reductions `out` receives one element per row at
 * out_ld spacing, otherwise a full row.  in_ld / out_ld are row pitches in
 * elements.  weight: length `cols`, fp32 if weight_fp32 else `dtype`. */
int arkmi_row_op(int kind, int dtype, const void *in, void *out,
                 const void *weight, int weight_fp32, int64_t rows,
                 int64_t cols, int64_t in_ld, int64_t out_ld, float eps,
                 void *stream);

/* Batched matmul C[b] = A[b] . B[b] on the MFMA units, fp16/bf16 operands, fp32
 * accumulate, result rounded once to `dtype`
 * (ark/ops/ops_matmul.cpp:13-252, ark/include/kernels/matmul.h:36-115).
 *   A: [m,k] row-major (lda); B: [k,n] row-major, or [n,k] when trans_b
 *   (the reference's transpose_other); a batch stride of 0 broadcasts the
 *   operand over the batch (matmul.h:80-101).
 *   tile_m/tile_n: output tile of one task (TileShapeMNK[0:2] of the plan
 *   config); 0 picks one.  m, n must be multiples of the tile and k of 64 —
 *   the reference's rule that padded shapes divide the tile
 *   (ops_matmul.cpp:139-144). */
int arkmi_gemm(int dtype, const void *a, const void *b, void *c, int batch,
               int m, int n, int k, int64_t lda, int64_t ldb, int64_t ldc,
               int64_t batch_stride_a, int64_t batch_stride_b,
               int64_t batch_stride_c, int trans_a, int trans_b, int tile_m,
               int tile_n, void *stream);

/* Skinny matmul ("decode GEMV"): Y[m,n] = X[m,k] . W[k,n], 1 <= m <= 16, W row-major
 * [k,n], fp32 accumulate, one rounding to `dtype`.  The shape the reference
 * sends through its general GEMM tile (ark/ops/ops_matmul.cpp:100-174,
 * ark/include/kernels/matmul.h:36-115); here W is streamed once at HBM rate.
 *   W is cut into units of 256 columns x 128 rows, numbered column block by
 *   column block, and dealt in contiguous ranges to `num_tasks` workgroups
 *   (0 = one per CU; clamped to the number of units), so every workgroup
 *   streams the same number of bytes.  Workgroups that share a column block
 *   meet through fp32 partial sums and arrival counters in `workspace`;
 *   arkmi_gemv_plan reports its size.  Its first 256*ceil(ceil(n/256)*4/256)
 *   bytes are the counters: zero them once; every call leaves them zero.
 *   Calls that share a workspace must not overlap in time. */
int arkmi_gemv_plan(int m, int n, int k, int num_tasks, int *num_tasks_out,
                    size_t *workspace_bytes);
int arkmi_gemv(int dtype, const void *x, const void *w, void *y, int m, int n,
               int k, int64_t ldx, int64_t ldw, int64_t ldy, int num_tasks,
               void *workspace, size_t workspace_bytes, void *stream);

/* arkmi_gemv for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments and results as arkmi_gemv, bit for
 * bit, without the workspace: the split-K partial sums and arrival counters live in
 * a fixed array inside the library (arkmi_gemv_static_limit() bytes, 16 MiB, held by
 * every GPU the library runs on until the process ends).  The call allocates and
 * frees nothing; it launches one small kernel that zeroes the counters and then the
 * matmul, both on `stream`.  A shape whose workspace (arkmi_gemv_plan) exceeds the
 * array is refused with ARKMI_UNSUPPORTED.  All calls on one GPU share the array:
 * calls that overlap in time on one GPU race. */
size_t arkmi_gemv_static_limit(void);
int arkmi_gemv_static(int dtype, const void *x, const void *w, void *y, int m, int n,
                      int k, int64_t ldx, int64_t ldw, int64_t ldy, int num_tasks,
                      void *stream);

/* Measurement probes (no counterpart in the reference): what this machine sustains, to print
 * beside the datasheet peaks.  Each call launches one kernel on `stream`; the caller times it.
 *   arkmi_probe_mfma: every CU's 8 waves run `iters` rounds of 16 independent
 *     v_mfma_f32_16x16x32_f16 on operands read from `operands` (>= 1 MiB; random values draw more
 *     power than zeros and lower the clock); *flops receives the flops of the launch.
 *   arkmi_probe_stream: reads `bytes` from src with 16-byte loads and writes them to dst (a copy)
 *     or, with dst == NULL, only reads.  `sink` is 4 bytes of device memory the kernels may write. */
int arkmi_probe_mfma(const void *operands, size_t operand_bytes, int iters, void *sink,
                     double *flops, void *stream);
int arkmi_probe_stream(const void *src, void *dst, size_t bytes, void *sink, void *stream);

/* ------------------------------------------------------------------------
 * Model building and planning for bindings that cannot use the C++ classes
 * directly.  Every call maps onto one member of ark::Model / PlannerContext /
 * Planner (ark/include/ark/model.hpp, planner.hpp); tensors are named by their
 * model-wide tensor id.  Returned strings are malloc'ed: release with
 * arkmi_free().
 * ---------------------------------------------------------------------- */
typedef struct arkmi_model arkmi_model;

typedef struct arkmi_tensor_info {
    int64_t id;
    int64_t buffer_id;
    int dtype;        /* arkmi_dtype */
    int ndims;
    int64_t shape[4], strides[4], offsets[4], padded_shape[4];
} arkmi_tensor_info;

/* A config rule: gets the op's JSON and the architecture name, returns a
 * config JSON string owned by the callee until the next call, or NULL / ""
 * to decline (ark::Planner::ConfigRule, planner.hpp:35-38). */
typedef const char *(*arkmi_config_rule)(const char *op_json, const char *arch,
                                         void *user);

void arkmi_free(void *p);
/* Tensor and buffer ids are process-global counters (model_tensor.cpp:135-138,
 * model_buffer.cpp:10-13); resetting them makes emitted ids reproducible. */
void arkmi_reset_ids(void);

int arkmi_model_create(int rank, int world_size, arkmi_model **out);
/* A model rebuilt from its serialized form: the text ark::Model::serialize()
 * writes (schema ark/model/model_json.cpp:24-101, docs/model_file.md; written by
 * ark/model/model_graph_impl.cpp:318-345).  This is how a caller that keeps the
 * reference's own ark::Model hands a finished graph to this library's planner:
 * arkmi_model_from_json(model.serialize()) -> arkmi_model_plan().  Tensors keep the
 * ids of the file; a malformed file is ARKMI_MODEL_ERROR. */
int arkmi_model_from_json(const char *model_json, arkmi_model **out);
int arkmi_model_destroy(arkmi_model *m);
/* Model::tensor.  Optional arrays may be NULL. */
int arkmi_model_tensor(arkmi_model *m, int ndims, const int64_t *shape,
                       int dtype, const int64_t *strides,
                       const int64_t *offsets, const int64_t *padded_shape,
                       int rank, const char *name, int64_t *tensor_out);
/* Any other Model member, by its C++ name ("matmul", "reduce_sum", "add",
 * "reshape", ...).  `inputs` are tensor ids in the member's argument order,
 * `output` the output tensor id or -1, `args_json` the remaining arguments by
 * parameter name, e.g. {"trans_other":true}, {"axis":-1,"keepdims":false},
 * {"value":0.5}, {"shape":[2,-1]}, {"permutation":[0,2,1,3]},
 * {"data_type":"FP16"}.  Result tensor ids are written to `results`. */
int arkmi_model_op(arkmi_model *m, const char *op, const int64_t *inputs,
                   int n_inputs, int64_t output, const char *args_json,
                   const char *name, int64_t *results, int max_results,
                   int *n_results);
int arkmi_model_tensor_info(arkmi_model *m, int64_t tensor,
                            arkmi_tensor_info *out);
int arkmi_model_serialize(arkmi_model *m, int pretty, char **out);
/* JSON of the model or of a compressed copy of it (Model::compress()); with
 * `with_context` every node also carries its context snapshot under
 * "Context" (ModelNode::context, ark/model/model_node.hpp). */
int arkmi_model_dump(arkmi_model *m, int compressed, int with_context,
                     int pretty, char **out);
/* Compresses the model in place (ModelGraph::compress_nodes). */
int arkmi_model_compress(arkmi_model *m);
int arkmi_model_verify(arkmi_model *m, int *ok);
/* PlannerContext scope: enter creates one, call invokes a member
 * ("processor_range" [b,e(,s)], "warp_range", "sram_range", "sync" true|false,
 * "config" {...}) on the innermost one, exit destroys it (LIFO). */
int arkmi_model_context_enter(arkmi_model *m);
int arkmi_model_context_call(arkmi_model *m, const char *member,
                             const char *args_json);
int arkmi_model_context_exit(arkmi_model *m);
/* Context::get on the innermost context: JSON text, "" if unset. */
int arkmi_model_context_get(arkmi_model *m, const char *key, char **out);
/* Planner::plan.  arch == NULL plans for device `device_id`; otherwise for the
 * named architecture with `num_processors` processors (no GPU needed). */
int arkmi_model_plan(arkmi_model *m, int device_id, const char *arch,
                     int num_processors, const arkmi_config_rule *rules,
                     void *const *rule_users, int n_rules, int pretty,
                     char **plan_out);

/* ------------------------------------------------------------------------
 * Executor: runs a plan JSON inside one persistent loop kernel.  One function
 * per member of ark::Executor (ark/include/ark/executor.hpp:19-90,
 * ark/api/executor.cpp:141-886); the C++ facade forwards to these.
 *   create  : parses the plan (or the file named by ARK_ENFORCE_PLAN_PATH),
 *             lays out and zero-fills the buffer arena.  stream == NULL makes
 *             the executor create its own non-blocking stream.
 *   compile : lowers the plan to the loop kernel's tables.
 *   launch  : starts the loop kernel (loop_mode) and the stop() timer.
 *   run(n)  : n iterations of the plan; returns at once.  wait: until done.
 *   stop    : waits, ends the kernel, returns milliseconds since launch.
 * ---------------------------------------------------------------------- */
typedef struct arkmi_exec arkmi_exec;

typedef struct arkmi_exec_info_t {
    int device_id;
    void *stream;
    int num_processors;        /* grid size of the loop kernel */
    int threads_per_processor; /* workgroup size */
    int lds_bytes;             /* dynamic LDS per workgroup (after compile) */
    size_t arena_bytes;
    int num_steps;             /* barriers + task sequences in the schedule */
    int num_barriers;          /* distinct barrier objects */
    int barriers_elided;       /* schedule barriers dropped at compile(): no data hazard */
    int kernel_families;       /* op families of the loop-kernel variant in use: 1 rows, 2 elementwise, 4 GEMM */
    int compiled, launched, destroyed, loop_mode;
    int iterations_done;
    int barriers_local;   /* grid barriers replaced by a workgroup-local sync */
    int iteration_sync;   /* between iterations of one run(n): 2 grid barrier, 1 workgroup-local sync, 0 nothing */
    int barriers_counted; /* grid barriers replaced by waits on per-row-block dependency counters */
    int gemv_chains;      /* runs of consecutive skinny matmuls that the loop kernel streams as one sequence */
    int gemv_claimed;     /* skinny matmuls (or runs) whose stretches the workgroups claim at run time */
} arkmi_exec_info_t;

int arkmi_exec_create(int device_id, void *stream, const char *name,
                      const char *plan_json, int loop_mode, arkmi_exec **out);
int arkmi_exec_destroy(arkmi_exec *h);   /* frees the handle */
int arkmi_exec_release(arkmi_exec *h);   /* Executor::destroy(): frees device state, keeps the handle */
int arkmi_exec_compile(arkmi_exec *h);
int arkmi_exec_launch(arkmi_exec *h);
int arkmi_exec_run(arkmi_exec *h, int iter);
/* The compiled plan's ops as separate kernels, for comparison with the loop
 * kernel: `iter` passes, one launch per task group in plan order on the
 * executor's stream, kernel boundaries in place of the barriers
 * (the reference's non-loop mode launches its one kernel per iteration,
 * ark/api/executor.cpp:705-711; this splits further, per op).  Asynchronous:
 * synchronise the stream to wait.  The loop kernel must not be launched. */
int arkmi_exec_run_separate(arkmi_exec *h, int iter);
int arkmi_exec_wait(arkmi_exec *h, int64_t max_spin_count);
int arkmi_exec_stop(arkmi_exec *h, int64_t max_spin_count, float *elapsed_ms);
int arkmi_exec_plan(arkmi_exec *h, char **plan_out);
int arkmi_exec_info(arkmi_exec *h, arkmi_exec_info_t *out);
/* Device address of a buffer (Executor::tensor_address, executor.cpp:774-781). */
int arkmi_exec_buffer_address(arkmi_exec *h, uint64_t buffer_id, uintptr_t *out);
/* tensor_read / tensor_write (executor.cpp:783-886): copies between the view
 * (shape, strides, offsets: `ndims` entries each) of a buffer and a dense
 * array `data` of `bytes` = nelems * elem_bytes.  stream NULL = a private one. */
int arkmi_exec_copy(arkmi_exec *h, uint64_t buffer_id, int ndims,
                    const int64_t *shape, const int64_t *strides,
                    const int64_t *offsets, int elem_bytes, void *data,
                    size_t bytes, void *stream, int to_device, int is_d2d);
/* Task placement evidence: with tracing enabled before compile(), every task
 * records (block, slot, order-within-slot).  records: 3 int32 per task of
 * the task group, indexed by position in its TaskRange. */
int arkmi_exec_enable_trace(arkmi_exec *h);
int arkmi_exec_read_trace(arkmi_exec *h, int task_group, int32_t *records,
                          int max_tasks, int *n_tasks);

/* With tracing enabled: microseconds block 0 spent in each schedule step
 * (task sequence or barrier) of the most recent iteration, read from the
 * GPU's constant-rate wall clock inside the loop kernel. */
int arkmi_exec_read_step_times(arkmi_exec *h, double *step_us, int max_steps,
                               int *n_steps);

/* Raw form of the above for every workgroup: ticks[block][step] is the wall
 * clock at which `block` entered `step` in the most recent iteration, with
 * one extra entry per block for the end of the body (n_steps + 1 per block);
 * ticks_per_ms is the clock rate. */
int arkmi_exec_read_step_clocks(arkmi_exec *h, uint64_t *ticks,
                                size_t max_entries, int *n_blocks,
                                int *n_steps, int *ticks_per_ms);

/* What compile() decides for a plan, without a GPU: the device steps (grid barriers kept, workgroup
 * syncs, task groups), the barrier statistics of arkmi_exec_info_t, and -- with dep_counters 1 (0: off,
 * -1: as ARKMI_DEP_COUNTERS says) -- the dependency counters: per consumer group the producer group, the
 * expected count per iteration and the counter span [lo, hi] each task waits for; per producer group
 * the row block each task signals.  Counterpart of reading the generated kernel source of the reference
 * (ark/codegen.cpp:109-158 places its sync_gpu calls there).  Free the text with arkmi_free. */
int arkmi_plan_analysis(const char *plan_json, int dep_counters, char **analysis_json);

/* The schedule a plan compiles to, as JSON: the ordered barriers and
 * task_seq<> argument lists the reference's code generator would emit
 * (ark/codegen.cpp:109-158,272-400).  No GPU needed. */
int arkmi_plan_schedule(const char *plan_json, char **schedule_json);
/* Task ids that (block, slot) runs in schedule step `step`, in order
 * (ark/include/kernels/kernel_template.in:11-27).  No GPU needed. */
int arkmi_schedule_tasks(const char *plan_json, int step, int block, int slot,
                         int64_t *tasks, int max_tasks, int *n_tasks);

#ifdef __cplusplus
}
#endif
#endif /* ARKMI_H_ */
