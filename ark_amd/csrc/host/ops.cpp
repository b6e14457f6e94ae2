#include "ops.hpp"

namespace ark {

int gemm_lds_bytes(int tm, int tn) {
    // A ring of stages, each an A tile [tm][bk] and a B tile [tn][bk] (or
    // [bk][tn]) of 2-byte elements, unpadded; must match GemmShape / GemmLds in
    // kernels/gemm.h.
    const int bk = (tm + tn >= 512) ? 32 : 64;
    const int stages = (tm + tn >= 512) ? 4 : ((tm + tn >= 384) ? 3 : 4);
    return stages * (tm + tn) * bk * 2;
}

int gemv_lds_bytes() {
    // a flag line + per wave the larger of a staged 16 x 256 slab (row pitch
    // 512 + 32 bytes) and a 16 x (256 + 4) fp32 tile; must match kernels/gemv.h
    return 64 + 8 * std::max(16 * (256 * 2 + 32), 16 * (256 + 4) * 4);
}

int64_t gemv_default_tasks(int64_t n, int64_t k, int num_cu) {
    // units of 256 columns x 128 rows, one contiguous range per CU
    return std::min<int64_t>(num_cu, div_up(n, 256) * div_up(k, 128));
}

static Json tile_config(int num_warps, const Dims &shape4, int64_t th, int64_t tw) {
    Json c = Json::object();
    c["NumWarps"] = num_warps;
    c["SramBytes"] = 0;
    Json tile = Json::array();
    tile.push_back((long long)th);
    tile.push_back((long long)tw);
    c["Tile"] = tile;
    c["NumTasks"] = (long long)(shape4[0] * shape4[1] * div_up(shape4[2], th) * div_up(shape4[3], tw));
    return c;
}

static bool is_elementwise(const std::string &t) {
    static const char *types[] = {"Add", "Sub", "Mul", "Div", "Exp", "Gelu", "Relu", "Rsqrt",
                                  "Sigmoid", "Sqrt", "Copy", "Cast", "Rope", "SiluMul", "ScalarAdd",
                                  "ScalarMul", "ScalarAssign"};
    for (const char *x : types)
        if (t == x) return true;
    return false;
}

// ---- reference rules (other architectures) -------------------------------------------
static Json reference_config(const ModelOp &op, const Arch &arch) {
    const std::string &t = op.type();
    if (t == "Matmul") {
        // ark/ops/ops_matmul.cpp:181-243
        auto dt = op.result_tensors()[0]->data_type();
        if (dt != FP32.ref() && dt != FP16.ref() && dt != BF16.ref())
            ARK_ERR(PlanError, "Unsupported data type: ", dt->type_name());
        Dims mnk = matmul_problem_size(op.read_tensors()[0]->padded_shape(),
                                       op.read_tensors()[1]->padded_shape(),
                                       op.args().at("TransposeInput").i, op.args().at("TransposeOther").i);
        int64_t tm = (mnk[0] > mnk[1]) ? 256 : 128, tn = (mnk[0] > mnk[1]) ? 128 : 256, tk;
        int warps, sram;
        if (arch.belongs_to("CUDA_80")) {
            warps = 8; sram = 147456; tk = (dt == FP32.ref()) ? 32 : 64;
        } else if (arch.belongs_to("ROCM_942")) {
            warps = 4; sram = (dt == BF16.ref()) ? 24624 : 24672; tk = (dt == FP32.ref()) ? 16 : 32;
        } else {
            ARK_ERR(PlanError, "no default matmul config for architecture ", arch.name());
        }
        if (mnk[0] % tm != 0 || mnk[1] % tn != 0)
            ARK_ERR(PlanError, "output padded shape MNK ", mnk, " should be divisible by tile shape MNK <",
                    tm, ", ", tn, ", ", tk, ">");
        Json c = Json::object();
        c["NumWarps"] = warps;
        c["SramBytes"] = sram;
        Json tile = Json::array();
        tile.push_back((long long)tm); tile.push_back((long long)tn); tile.push_back((long long)tk);
        c["TileShapeMNK"] = tile;
        Dims rs = op.result_tensors()[0]->shape().dims4();
        c["NumTasks"] = (long long)(rs[0] * rs[1] * (mnk[0] / tm) * (mnk[1] / tn));
        return c;
    }
    if (t == "ReduceSum" || t == "ReduceMax" || t == "ReduceMean") {
        // ark/ops/ops_reduce.cpp:114-127
        Json c = Json::object();
        c["NumWarps"] = 1;
        int axis = (int)op.args().at("Axis").i;
        bool last = axis == op.read_tensors()[0]->shape().ndims() - 1 || axis == -1;
        c["ImplType"] = last ? "WarpWise" : "ElementWise";
        c["SramBytes"] = last ? 256 : 0;
        c["NumTasks"] = (long long)op.result_tensors()[0]->shape().nelems();
        return c;
    }
    if (is_elementwise(t)) {
        // ark/ops/ops_broadcast.cpp:45-66, ops_scalar.cpp:46-66
        Dims s = op.result_tensors()[0]->shape().dims4();
        return (s[2] > s[3]) ? tile_config(1, s, 64, 1) : tile_config(1, s, 1, 64);
    }
    if (t == "Transpose") {
        // ark/ops/ops_transpose.cpp:110-124
        return tile_config(1, op.result_tensors()[0]->shape().dims4(), 8, 8);
    }
    if (t == "Embedding") {
        // ark/ops/ops_embedding.cpp:58-66: one warp per output row
        Json c = Json::object();
        c["NumWarps"] = 1; c["SramBytes"] = 0;
        const Dims s = op.result_tensors()[0]->shape().dims4();
        c["NumTasks"] = (long long)(s[0] * s[1] * s[2]);
        return c;
    }
    if (t == "Noop") {
        Json c = Json::object();
        c["NumWarps"] = 1; c["SramBytes"] = 0; c["NumTasks"] = 0;
        return c;
    }
    ARK_ERR(PlanError, "no default config for op type ", t, " on architecture ", arch.name());
}

// ---- gfx950 rules ------------------------------------------------------------------------
// One slot of 8 waves (512 threads) per CU for every op, so a task always owns
// the whole workgroup and s_barrier is the only intra-task barrier.
constexpr int kWarps950 = 8;

// Rows a wave takes per row-op task: one while that still gives every CU a task,
// then more (up to 8), so a wave keeps the next row's loads in flight while it
// reduces and stores the current one.
static int64_t rows_per_wave950(int64_t rows, int num_cu) {
    return std::max<int64_t>(1, std::min<int64_t>(8, rows / ((int64_t)kWarps950 * num_cu)));
}

// `num_cu`: the processor count the plan is made for (the planner's NumProcessors
// argument), which decides tile sizes, rows per wave and skinny-matmul task counts.
static Json rocm950_config(const ModelOp &op, int num_cu) {
    const std::string &t = op.type();
    if (t == "Matmul") {
        auto dt = op.result_tensors()[0]->data_type();
        if (dt != FP16.ref() && dt != BF16.ref() && dt != FP32.ref())
            ARK_ERR(PlanError, "Unsupported data type for the MFMA GEMM: ", dt->type_name());
        const bool f32 = (dt == FP32.ref());
        Dims mnk = matmul_problem_size(op.read_tensors()[0]->padded_shape(),
                                       op.read_tensors()[1]->padded_shape(),
                                       op.args().at("TransposeInput").i, op.args().at("TransposeOther").i);
        Dims rs = op.result_tensors()[0]->shape().dims4();
        const int64_t batch = rs[0] * rs[1];
        const bool trans_in = op.args().at("TransposeInput").i, trans_other = op.args().at("TransposeOther").i;
        if (batch == 1 && rs[2] <= 16 && !trans_in && !trans_other && rs[3] % 8 == 0 && !f32) {
            // at most 16 rows: the skinny body streams W[K,N] once, dealt evenly to the CUs
            const int64_t k = op.read_tensors()[0]->shape()[-1];
            Json c = Json::object();
            c["NumWarps"] = kWarps950;
            c["SramBytes"] = gemv_lds_bytes();
            Json tile = Json::array();
            tile.push_back(16); tile.push_back(256); tile.push_back(128);
            c["TileShapeMNK"] = tile;
            c["NumTasks"] = (long long)gemv_default_tasks(rs[3], k, num_cu);
            return c;
        }
        // Largest tile that divides the padded problem and still gives every CU
        // a task; otherwise the dividing tile with the most tasks.
        // (of the two half-size tiles the 256-row one first: measured faster than 128x256 on
        // the same problem, 161 against 171 us on 4096^3 and 9 us per decoder layer)
        const int64_t cand[4][2] = {{256, 256}, {256, 128}, {128, 256}, {128, 128}};
        int64_t tm = 0, tn = 0;
        for (const auto &c : cand) {
            // the one tile shape of a transposed input and of FP32 operands
            if ((trans_in || f32) && (c[0] != 128 || c[1] != 128)) continue;
            if (mnk[0] % c[0] || mnk[1] % c[1]) continue;
            tm = c[0]; tn = c[1];
            if (batch * (mnk[0] / c[0]) * (mnk[1] / c[1]) >= num_cu) break;
        }
        if (tm == 0 || mnk[2] % 64 != 0)
            ARK_ERR(PlanError, "output padded shape MNK ", mnk,
                    " should be divisible by a tile shape of 128x128x64 or larger");
        // An output that gives 256x256 tiles to between half and all of the CUs, with a long K:
        // keep the large tile (two thirds of the operand traffic per flop of a 128x256 tile) and
        // split K in two, so the tiles' halves fill the chip: one task sends its partial sums,
        // the other adds them to its own and finishes the tile.  The exchange costs the finisher
        // about 9 us, which a 256x128 tiling loses from K = 4096 on (2048 x 4096 x 4096: 69
        // against 75 us; x 11008: 154 against 185 us).
        int64_t split = 1;
        if (!trans_in && !f32 && mnk[0] % 256 == 0 && mnk[1] % 256 == 0 && mnk[2] % 128 == 0 && mnk[2] >= 4096) {
            const int64_t tiles256 = batch * (mnk[0] / 256) * (mnk[1] / 256);
            if (tiles256 < num_cu && 2 * tiles256 >= num_cu) {
                tm = tn = 256;
                split = 2;
            }
        }
        Json c = Json::object();
        c["NumWarps"] = kWarps950;
        c["SramBytes"] = gemm_lds_bytes((int)tm, (int)tn);
        Json tile = Json::array();
        tile.push_back((long long)tm); tile.push_back((long long)tn); tile.push_back(64);
        c["TileShapeMNK"] = tile;
        if (split > 1) c["SplitK"] = (long long)split;
        c["NumTasks"] = (long long)(split * batch * (mnk[0] / tm) * (mnk[1] / tn));
        return c;
    }
    if (t == "MatmulSwiglu") {
        // one task = a 256- (or 128-) row by 128-column tile of the result, computed as a
        // 256-wide GEMM tile over the interleaved gate/up columns
        auto dt = op.result_tensors()[0]->data_type();
        if (dt != FP16.ref() && dt != BF16.ref())
            ARK_ERR(PlanError, "Unsupported data type for MatmulSwiglu: ", dt->type_name());
        const Dims rs = op.result_tensors()[0]->shape().dims4();
        const int64_t k = op.read_tensors()[0]->shape()[-1];
        if (rs[2] % 128 || rs[3] % 128 || k % 64)
            ARK_ERR(PlanError, "MatmulSwiglu needs rows and hidden size in multiples of 128 and dim in multiples of "
                               "64; got ", rs, ", dim ", k);
        const int64_t batch = rs[0] * rs[1];
        int64_t tm = 256;
        if (rs[2] % 256 || batch * (rs[2] / 256) * (rs[3] / 128) < num_cu) tm = 128;
        Json c = Json::object();
        c["NumWarps"] = kWarps950;
        c["SramBytes"] = gemm_lds_bytes((int)tm, 256);
        Json tile = Json::array();
        tile.push_back((long long)tm); tile.push_back(256); tile.push_back(64);
        c["TileShapeMNK"] = tile;
        c["NumTasks"] = (long long)(batch * (rs[2] / tm) * (rs[3] / 128));
        return c;
    }
    if (t == "ReduceSum" || t == "ReduceMax" || t == "ReduceMean") {
        Json c = Json::object();
        c["NumWarps"] = kWarps950;
        int axis = (int)op.args().at("Axis").i;
        const Dims &ish = op.read_tensors()[0]->shape();
        bool last = axis == ish.ndims() - 1 || axis == -1;
        c["ImplType"] = last ? "WarpWise" : "ElementWise";
        c["SramBytes"] = 0;
        int64_t outs = op.result_tensors()[0]->shape().nelems();
        // WarpWise: RowsPerWave output rows per wave; ElementWise: one output per thread
        if (last) {
            const int64_t rpw = rows_per_wave950(outs, num_cu);
            c["RowsPerWave"] = (long long)rpw;
            c["NumTasks"] = (long long)div_up(outs, kWarps950 * rpw);
        } else {
            c["NumTasks"] = (long long)div_up(outs, kWarps950 * 64);
        }
        return c;
    }
    if (t == "Attention") {
        // one task = 128 query positions of one (batch, head); steps of 128 keys, K and V
        // tiles of 32 KB each, double-buffered in LDS (must match kernels/attn.h)
        const Dims &qs = op.read_tensors()[0]->shape();
        if (qs[3] != 128) ARK_ERR(PlanError, "the attention body supports head_dim 128, got ", qs[3]);
        Json c = Json::object();
        c["NumWarps"] = kWarps950;
        c["SramBytes"] = 2 * 2 * 128 * (128 * 2);
        c["NumTasks"] = (long long)(qs[0] * qs[2] * div_up(qs[1], 128));
        return c;
    }
    if (t == "Softmax" || t == "Layernorm" || t == "Rmsnorm") {
        Json c = Json::object();
        c["NumWarps"] = kWarps950;
        c["SramBytes"] = 0;
        const Dims &s = op.result_tensors()[0]->shape();
        const int64_t rows = s.nelems() / s[-1];
        const int64_t rpw = rows_per_wave950(rows, num_cu);
        // RMSNorm keeps its fp32 weights in LDS for the rows of a task
        if (t == "Rmsnorm" && op.read_tensors().size() > 1 &&
            op.read_tensors()[1]->data_type() == FP32.ref() && s[-1] * 4 <= 65536)
            c["SramBytes"] = (long long)(s[-1] * 4);
        c["RowsPerWave"] = (long long)rpw;
        c["NumTasks"] = (long long)div_up(rows, kWarps950 * rpw);
        return c;
    }
    if (is_elementwise(t) || t == "Transpose") {
        // Row-major tiles of about 32 Ki elements: full-width rows of up to
        // 4096 elements, so every thread streams 16-byte vectors.
        Dims s = op.result_tensors()[0]->shape().dims4();
        int64_t tw = std::min<int64_t>(s[3], 4096);
        int64_t th = std::max<int64_t>(1, std::min<int64_t>(s[2], 32768 / tw));
        return tile_config(kWarps950, s, th, tw);
    }
    if (t == "Embedding") {
        // one wave per output row, eight rows per task
        Json c = Json::object();
        c["NumWarps"] = kWarps950; c["SramBytes"] = 0;
        const Dims s = op.result_tensors()[0]->shape().dims4();
        c["NumTasks"] = (long long)div_up(s[0] * s[1] * s[2], kWarps950);
        return c;
    }
    if (t == "Noop") {
        Json c = Json::object();
        c["NumWarps"] = 1; c["SramBytes"] = 0; c["NumTasks"] = 0;
        return c;
    }
    ARK_ERR(PlanError, "no default config for op type ", t, " on ROCM_950");
}

// Folds the dimensions [b, e) (extents d, strides s) into one axis: true with its
// stride when they are laid out as one dense run or all broadcast.
static bool fold_axis(const int64_t d[4], const int64_t s[4], int b, int e, int64_t *stride) {
    int64_t inner = -1;  // stride of the innermost folded dimension with extent > 1
    int64_t expect = 0;
    for (int i = e - 1; i >= b; --i) {
        if (d[i] == 1) continue;
        if (inner < 0) {
            inner = s[i];
            expect = s[i] * d[i];
        } else {
            if (s[i] != expect) return false;
            expect = s[i] * d[i];
        }
    }
    *stride = inner < 0 ? 0 : inner;
    return true;
}

Collapsed2D collapse_to_2d(const int64_t d[4], const int64_t s[4], int64_t cols) {
    Collapsed2D r;
    int k = 4;
    int64_t prod = 1;
    while (k > 0 && prod < cols) prod *= d[--k];
    if (prod != cols) return r;
    // leading extent-1 dimensions may sit on either side of the cut
    if (!fold_axis(d, s, 0, k, &r.row_stride)) return r;
    if (fold_axis(d, s, k, 4, &r.col_stride)) {
        r.ok = true;
        return r;
    }
    // outer part of the columns broadcast, inner part dense: the address wraps
    for (int j = k + 1; j < 4; ++j) {
        int64_t outer = 0, inner = 0;
        if (!fold_axis(d, s, k, j, &outer) || outer != 0) continue;
        if (!fold_axis(d, s, j, 4, &inner)) continue;
        int64_t period = 1;
        for (int i = j; i < 4; ++i) period *= d[i];
        r.ok = true;
        r.col_stride = inner;
        r.col_period = period;
        return r;
    }
    return r;
}

static void element_strides(const ModelTensorRef &t, const Dims &out4, int64_t d[4], int64_t s[4]) {
    const Dims sh = t->shape().dims4(), st = t->strides().dims4();
    int64_t acc = 1;
    for (int i = 3; i >= 0; --i) {
        d[i] = out4[i];
        s[i] = (sh[i] == 1 && out4[i] > 1) ? 0 : acc;
        acc *= st[i];
    }
}

Json follower_config(const ModelOp &op, const Json &task_info) {
    if (!is_elementwise(op.type())) return Json();
    const Json &lead = task_info.at("Ops").at((size_t)0);
    const Json &lc = lead.at("Config");
    const Dims out = op.result_tensors()[0]->shape().dims4();
    const Dims lead_out = Dims(lead.at("WriteTensors").at((size_t)0).at("Shape").as_int_vector()).dims4();
    std::vector<int64_t> tile;
    if (lead.at("Type").as_string() == "MatmulSwiglu") return Json();  // its output tiles are half its GEMM tiles
    if (lc.contains("TileShapeMNK")) {
        tile = lc.at("TileShapeMNK").as_int_vector();
        if (tile.at(0) < 32) return Json();  // the skinny matmul has no output tiles
    } else if (lc.contains("Tile")) {
        tile = lc.at("Tile").as_int_vector();
    } else {
        return Json();
    }
    if (tile.at(0) <= 0 || tile.at(1) <= 0 || tile.at(1) % 8) return Json();
    if (out == lead_out) return tile_config(kWarps950, out, tile.at(0), tile.at(1));

    // a reshape of the producer's output: every operand must be addressable over
    // the producer's [rows, cols]; only the second input may wrap along the columns
    if (lead_out[0] != 1 || lead_out[1] != 1 || out.nelems() != lead_out.nelems()) return Json();
    auto fits = [&](const ModelTensorRef &t, bool may_wrap) {
        int64_t d[4], s[4];
        element_strides(t, out, d, s);
        const Collapsed2D c = collapse_to_2d(d, s, lead_out[3]);
        return c.ok && (c.col_period == 0 || (may_wrap && c.col_period % 8 == 0));
    };
    if (!fits(op.result_tensors()[0], false)) return Json();
    const auto &reads = op.read_tensors();
    for (size_t i = 0; i < reads.size(); ++i)
        if (!fits(reads[i], i == 1)) return Json();
    Json c = tile_config(kWarps950, lead_out, tile.at(0), tile.at(1));
    Json view = Json::array();
    for (int i = 0; i < 4; ++i) view.push_back((long long)lead_out[i]);
    c["ViewAs"] = view;
    return c;
}

Json default_config(const ModelOp &op, const Arch &arch, int num_processors) {
    if (arch.belongs_to("ROCM_950")) return rocm950_config(op, std::max(1, num_processors));
    const std::string &t = op.type();
    if (t == "Softmax" || t == "Layernorm" || t == "Rmsnorm" || t == "Attention")
        ARK_ERR(PlanError, "op type ", t, " exists only on ROCM_950");
    if (t == "MatmulSwiglu") ARK_ERR(PlanError, "op type ", t, " exists only on ROCM_950");
    return reference_config(op, arch);
}

}  // namespace ark
