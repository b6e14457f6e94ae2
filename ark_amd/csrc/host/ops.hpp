// Per-op-type host behaviour that is not part of the op record itself:
// default plan configs, shape helpers and the lowering to device descriptors.
#pragma once
#include <ark/model.hpp>

#include "ir.hpp"

namespace ark {

// Access to ModelGraph internals for the host library's own translation units.
struct ModelGraphAccess {
    static std::shared_ptr<ContextStack> context(Model &model);
    static ModelGraph::Impl &impl(const ModelGraph &g);
    // Replaces the graph of `g` (a model rebuilt from its serialized form).
    static void adopt(ModelGraph &g, std::unique_ptr<ModelGraph::Impl> impl);
};

Dims broadcast_shape(const Dims &a, const Dims &b);
Dims matmul_problem_size(const Dims &in, const Dims &other, bool trans_in, bool trans_other);

// Default plan config of a non-virtual op for an architecture: at least
// NumWarps, SramBytes, NumTasks (ark/ops/ops_*.cpp default_config()).  For
// CUDA_* / ROCM_90A / ROCM_942 the reference's rules are reproduced; ROCM_950
// has this backend's own (one 8-wave slot per CU), sized for the `num_processors`
// the plan is made for.
Json default_config(const ModelOp &op, const Arch &arch, int num_processors);

// Config of an elementwise op that joins the task of `task_info` (an op fused
// behind its producer by a PlannerContext with sync(false)) on ROCM_950: when
// its output has the shape of the task's first op's output, it takes that
// op's tiling (the GEMM's output tile, or the elementwise tile), so task t of
// the follower covers exactly what task t of the producer wrote.  Empty when
// the op cannot follow.
//
// A follower whose output is a reshape of the producer's (same elements,
// e.g. [1, S, heads, head_dim] behind a GEMM that writes [1, S, heads * head_dim])
// also follows when each of its operands can be addressed over the producer's
// [rows, cols]: the config then carries "ViewAs": the producer's 4-D output
// shape, and the device descriptor is built over that shape.
Json follower_config(const ModelOp &op, const Json &task_info);

// An operand with element strides `s` over the dimensions `d` (0 where it
// broadcasts), re-addressed over [rows, cols] with cols the product of a
// suffix of d: offset(r, c) = r * row_stride + (c mod col_period) * col_stride
// (col_period 0: no wrap).  ok is false when no such form exists.
struct Collapsed2D {
    bool ok = false;
    int64_t row_stride = 0, col_stride = 0, col_period = 0;
};
Collapsed2D collapse_to_2d(const int64_t d[4], const int64_t s[4], int64_t cols);

// LDS bytes the MFMA GEMM body needs for an output tile.
int gemm_lds_bytes(int tile_m, int tile_n);

// The skinny matmul body (at most 16 rows times W[K,N]): LDS it needs, and the
// number of tasks its 256 x 128 units are dealt to on `num_cu` CUs.
int gemv_lds_bytes();
int64_t gemv_default_tasks(int64_t n, int64_t k, int num_cu);

}  // namespace ark
