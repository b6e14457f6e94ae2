// Executor runtime behind arkmi_exec_* : compiles a plan JSON into the loop
// kernel's tables, owns the buffer arena and the host mailbox, and drives the
// launch / run / wait / stop life cycle.
//
// Behavioural reference: ark/api/executor.cpp:141-886 (single-GPU parts) and
// ark/codegen.cpp:79-429 (barrier placement and task_seq parameters).
#include <ark/error.hpp>

#include <algorithm>
#include <chrono>
#include <cstring>
#include <fstream>
#include <functional>
#include <list>
#include <map>
#include <thread>

#include "host/ir.hpp"
#include "host/ops.hpp"
#include "host_common.h"
#include "kernels/loop.h"
#include "loop_launch.h"
#include "schedule.hpp"

using ark::Json;

namespace arkmi {

// ---------------------------------------------------------------------------
// plan -> schedule (host only, no device addresses)
// ---------------------------------------------------------------------------
namespace {

struct Range2 {
    int64_t b, e;
    int64_t size() const { return e > b ? e - b : 0; }
    bool operator<(const Range2 &o) const { return b != o.b ? b < o.b : e < o.e; }
    bool operator==(const Range2 &o) const { return b == o.b && e == o.e; }
};

// The reference builds its ranges from the first two array elements only
// (codegen.cpp:111-112,275-281,289), so an optional third "step" element is
// ignored there; this is kept for identical task placement.
Range2 range_of(const Json &j) { return Range2{j.at((size_t)0).as_int(), j.at((size_t)1).as_int()}; }

Range2 intersect(const Range2 &a, const Range2 &b) {
    Range2 r{std::max(a.b, b.b), std::min(a.e, b.e)};
    if (r.e < r.b) r.e = r.b;
    return r;
}

}  // namespace

Schedule build_schedule(const Json &plan) {
    ark::verify_plan_json(plan);
    Schedule sch;
    sch.num_processors = (int)plan.at("NumProcessors").as_int();
    sch.num_warps_per_processor = (int)plan.at("NumWarpsPerProcessor").as_int();
    const Json &task_infos = plan.at("TaskInfos");

    std::map<Range2, int> barrier_ids;
    auto barrier_for = [&](const Range2 &r) {
        auto it = barrier_ids.find(r);
        if (it != barrier_ids.end()) return it->second;
        int id = (int)barrier_ids.size();
        barrier_ids[r] = id;
        return id;
    };
    auto emit_barrier = [&](const Range2 &r) {
        ScheduleStep st{};
        st.is_barrier = true;
        st.barrier_id = barrier_for(r);
        st.b = (int)r.b;
        st.e = (int)r.e;
        st.s = 1;
        sch.steps.push_back(st);
    };

    // Barrier placement (codegen.cpp:109-158): before a processor group runs,
    // every earlier not-yet-synchronised range that overlaps it is synchronised
    // — on its own barrier if it sticks out of the new range, otherwise
    // together with the new range.
    std::list<Range2> unsynced;
    size_t pg_idx = 0;
    for (const auto &pg : plan.at("ProcessorGroups").elements()) {
        Range2 pr = range_of(pg.at("ProcessorRange"));
        if (pr.e == pr.b) continue;
        if (pg_idx > 0) {
            bool need_sync = false;
            for (auto it = unsynced.begin(); it != unsynced.end();) {
                Range2 inter = intersect(pr, *it);
                if (inter.size() == 0) {
                    ++it;
                    continue;
                }
                if (inter.size() < it->size()) {
                    emit_barrier(*it);
                    if (inter.size() < pr.size()) need_sync = true;
                } else {
                    need_sync = true;
                }
                it = unsynced.erase(it);
            }
            if (need_sync) emit_barrier(pr);
        }
        for (const auto &rg : pg.at("ResourceGroups").elements()) {
            // codegen.cpp:272-400
            Range2 rpr = range_of(rg.at("ProcessorRange"));
            if (rpr.b < pr.b || rpr.e > pr.e)
                ARK_ERR(PlanError, "invalid processor range of resource group");
            const int64_t total_warps = range_of(rg.at("WarpRange")).size();
            const int64_t total_sram = range_of(rg.at("SramRange")).size();
            int64_t proc_cur = rpr.b;
            const int64_t proc_b = rpr.b, proc_e = rpr.e, proc_s = 1;
            for (const auto &tg : rg.at("TaskGroups").elements()) {
                const int64_t task_id = tg.at("TaskId").as_int();
                if (task_id < 0 || (size_t)task_id >= task_infos.size())
                    ARK_ERR(PlanError, "TaskId ", task_id, " out of range");
                const Json &ti = task_infos.at((size_t)task_id);
                Range2 tr = range_of(tg.at("TaskRange"));
                const int64_t gran = tg.at("Granularity").as_int();
                const int64_t warps_per_task = ti.at("NumWarps").as_int();
                const int64_t sram_per_task = ti.at("SramBytes").as_int();
                if (warps_per_task <= 0 || gran <= 0)
                    ARK_ERR(PlanError, "NumWarps and Granularity must be positive");
                int64_t n_slots = total_warps / warps_per_task;
                if (sram_per_task > 0) n_slots = std::min(n_slots, total_sram / sram_per_task);
                if (n_slots == 0) ARK_ERR(PlanError, "not enough resources for task group");
                ScheduleStep st{};
                st.is_barrier = false;
                st.proc_b = (int)proc_b; st.proc_e = (int)proc_e; st.proc_s = (int)proc_s;
                st.proc_cur = (int)proc_cur;
                st.task_b = (int)tr.b; st.task_e = (int)tr.e; st.task_s = 1;
                st.gran = (int)gran;
                st.n_slots = (int)n_slots;
                st.slot_warps = (int)warps_per_task;
                st.slot_sram = (int)(total_sram / n_slots);
                st.task_info = (int)task_id;
                sch.steps.push_back(st);
                // the next task group starts where this one stopped dealing
                const int64_t n_procs = rpr.size();
                if (n_procs > 0) {
                    int64_t idx = (proc_cur - proc_b) / proc_s;
                    idx = (idx + ark::div_up(tr.size(), gran)) % n_procs;
                    proc_cur = proc_b + idx * proc_s;
                }
            }
        }
        unsynced.push_back(pr);
        ++pg_idx;
    }
    sch.num_barriers = (int)barrier_ids.size();
    return sch;
}

// Cutting a run of skinny matmuls into stretches that the workgroups claim at run time: the
// first `coarse_share` of the run's units goes into long stretches (two of them are about that
// share of a workgroup's average load: every workgroup starts with two), the rest into short ones
// of `fine` units, so that the spread at the end of the run is a short stretch or two.
// ARKMI_GEMV_FINE / ARKMI_GEMV_COARSE_PERCENT override the defaults (for measurements).
constexpr int kGemvMinStretch = 3;  // the claim protocol's look-ahead needs 3 units per stretch
int gemv_fine_units() {
    const char *e = getenv("ARKMI_GEMV_FINE");
    const int v = e ? atoi(e) : 0;
    return v >= kGemvMinStretch && v <= 1024 ? v : 3;
}
double gemv_coarse_share() {
    const char *e = getenv("ARKMI_GEMV_COARSE_PERCENT");
    const int v = e ? atoi(e) : -1;
    return (v >= 0 && v <= 100 ? v : 85) / 100.0;
}

std::vector<int64_t> schedule_tasks_of(const Schedule &sch, const ScheduleStep &st, int block, int slot) {
    // kernel_template.in:11-27
    std::vector<int64_t> out;
    if (st.is_barrier) return out;
    if (!(block >= st.proc_b && block < st.proc_e && ((block - st.proc_b) % st.proc_s) == 0)) return out;
    if (slot >= st.n_slots) return out;
    const int64_t grid = sch.num_processors;
    const int64_t n_procs = (st.proc_e - st.proc_b + st.proc_s - 1) / st.proc_s;
    const int64_t p = ((block + grid - st.proc_cur) % grid) / st.proc_s;
    const int64_t base = st.task_b + p * st.task_s * st.gran;
    for (int64_t t = slot;; t += st.n_slots) {
        int64_t id = base + st.task_s * (t % st.gran + t / st.gran * st.gran * n_procs);
        if (id >= st.task_e) break;
        out.push_back(id);
    }
    return out;
}

Json schedule_to_json(const Schedule &sch) {
    Json j = Json::object();
    j["NumProcessors"] = sch.num_processors;
    j["NumWarpsPerProcessor"] = sch.num_warps_per_processor;
    j["NumBarriers"] = sch.num_barriers;
    Json steps = Json::array();
    for (const auto &st : sch.steps) {
        Json s = Json::object();
        if (st.is_barrier) {
            s["Kind"] = "Barrier";
            s["BarrierId"] = st.barrier_id;
            Json r = Json::array();
            r.push_back(st.b); r.push_back(st.e);
            s["ProcessorRange"] = r;
        } else {
            s["Kind"] = "TaskSeq";
            // template arguments of task_seq<> in the reference's order
            Json a = Json::array();
            for (int v : {st.proc_b, st.proc_e, st.proc_s, st.proc_cur, st.task_b, st.task_e, st.task_s,
                          st.gran, st.n_slots, st.slot_warps, st.slot_sram, st.task_info})
                a.push_back(v);
            s["Args"] = a;
        }
        steps.push_back(s);
    }
    j["Steps"] = steps;
    return j;
}

// ---------------------------------------------------------------------------
// op lowering: plan op JSON -> device descriptor
// ---------------------------------------------------------------------------
namespace {

struct View4 {
    char *ptr;
    int64_t shape[4], padded[4];
    int64_t es[4];  // element strides
    int dtype;
    size_t elem;
};

struct Lowering {
    char *arena;
    const std::map<size_t, size_t> &buffer_offset;
    // zero-filled device scratch that lives as long as the compiled plan
    std::function<void *(size_t)> scratch;

    View4 view(const ark::ModelTensorRef &t) const {
        View4 v{};
        auto it = buffer_offset.find(t->buffer()->id());
        if (it == buffer_offset.end()) ARK_ERR(PlanError, "tensor ", t->id(), " names an unknown buffer");
        v.ptr = arena + it->second + t->byte_offset();
        ark::Dims sh = t->shape().dims4(), st = t->strides().dims4(), pd = t->padded_shape().dims4();
        int64_t acc = 1;
        for (int i = 3; i >= 0; --i) {
            v.shape[i] = sh[i];
            v.padded[i] = pd[i];
            v.es[i] = acc;
            acc *= st[i];
        }
        v.dtype = t->data_type()->code();
        v.elem = t->data_type()->bytes();
        return v;
    }
};

int float_code(const View4 &v, const std::string &op) {
    if (v.dtype < 0 || v.dtype > 2)
        ARK_ERR(UnsupportedError, "op ", op, " supports FP32/FP16/BF16 tensors only");
    return v.dtype;
}

EwTensor ew_operand(const View4 &v, const int64_t out_shape[4], const int perm[4]) {
    EwTensor t{};
    t.ptr = v.ptr;
    for (int i = 0; i < 4; ++i) {
        const int src = perm ? perm[i] : i;
        // a dimension of extent 1 broadcasts along a longer output dimension
        t.s[i] = (v.shape[src] == 1 && out_shape[i] > 1) ? 0 : v.es[src];
    }
    return t;
}

DevOp lower_op(const Json &op_json, const Lowering &L, int slot_warps, int block_warps, int n_slots,
               int slot_sram) {
    auto op = ark::ModelOp::deserialize(op_json);
    const Json &cfg = op_json.at("Config");
    const std::string &type = op->type();
    DevOp d{};
    d.kind = DEV_NOOP;
    auto i_arg = [&](const char *k) -> int64_t {
        auto it = op->args().find(k);
        if (it == op->args().end()) ARK_ERR(PlanError, type, ": missing argument ", k);
        return it->second.i;
    };
    auto f_arg = [&](const char *k) -> float {
        auto it = op->args().find(k);
        if (it == op->args().end()) ARK_ERR(PlanError, type, ": missing argument ", k);
        return it->second.f;
    };

    if (type == "Noop") return d;

    if (type == "MatmulSwiglu") {
        if (n_slots != 1 || slot_warps != block_warps || slot_warps * 64 != kGemmThreads)
            ARK_ERR(UnsupportedError, "MatmulSwiglu tasks need one slot of ", kGemmThreads / 64,
                    " waves spanning the whole workgroup");
        View4 a = L.view(op->read_tensors()[0]), b = L.view(op->read_tensors()[1]), b2 = L.view(op->read_tensors()[2]);
        View4 c = L.view(op->write_tensors()[0]);
        if ((a.dtype != 1 && a.dtype != 2) || b.dtype != a.dtype || b2.dtype != a.dtype || c.dtype != a.dtype)
            ARK_ERR(UnsupportedError, "MatmulSwiglu supports FP16/BF16 operands of one type");
        if (!cfg.contains("TileShapeMNK")) ARK_ERR(PlanError, "MatmulSwiglu config needs TileShapeMNK");
        auto tile = cfg.at("TileShapeMNK").as_int_vector();
        const int tm = (int)tile.at(0), tn = (int)tile.at(1);
        if ((tm != 256 && tm != 128) || tn != 256)
            ARK_ERR(UnsupportedError, "MatmulSwiglu runs on 256x256 or 128x256 GEMM tiles, got ", tm, "x", tn);
        const int64_t M = c.shape[2], H = c.shape[3], K = a.shape[3];
        if (b.shape[0] * b.shape[1] != 1 || b.shape[2] != H || b.shape[3] != K || b2.shape[2] != H || b2.shape[3] != K ||
            a.shape[2] != M)
            ARK_ERR(PlanError, "MatmulSwiglu: operand shapes do not agree");
        if (M % tm || H % 128 || K % kGemmMinK)
            ARK_ERR(PlanError, "MatmulSwiglu: rows ", M, ", hidden ", H, ", dim ", K, " must be multiples of ", tm,
                    ", 128, ", kGemmMinK);
        if (b.es[2] != b2.es[2]) ARK_ERR(UnsupportedError, "MatmulSwiglu: the two weights must have the same row pitch");
        if (slot_sram < ark::gemm_lds_bytes(tm, tn))
            ARK_ERR(PlanError, "MatmulSwiglu tile ", tm, "x", tn, " needs ", ark::gemm_lds_bytes(tm, tn),
                    " bytes of SRAM, the slot has ", slot_sram);
        GemmDesc &g = d.gemm;
        g.a = a.ptr; g.b = b.ptr; g.b2 = b2.ptr; g.c = c.ptr;
        g.m = (int)M; g.n = (int)(2 * H); g.k = (int)K;
        g.lda = (int)a.es[2]; g.ldb = (int)b.es[2]; g.ldc = (int)c.es[2];
        if ((g.lda % 8) || (g.ldb % 8) || ((uintptr_t)a.ptr & 15) || ((uintptr_t)b.ptr & 15) || ((uintptr_t)b2.ptr & 15))
            ARK_ERR(UnsupportedError, "MatmulSwiglu operands must start 16-byte aligned with row pitches % 8 == 0");
        g.batch_c = (int)c.shape[1];
        for (int i = 0; i < 2; ++i) {
            g.a_bs[i] = (a.shape[i] == 1) ? 0 : a.es[i];
            g.b_bs[i] = 0;
            g.c_bs[i] = c.es[i];
        }
        g.trans_b = 1;
        g.dtype = a.dtype;
        g.split_k = 1;
        g.batch_total = (int)(c.shape[0] * c.shape[1]);
        g.tiles_m = (int)(M / tm); g.tiles_n = (int)(H / 128);
        g.store_m = (int)M; g.store_n = (int)H;
        if ((int64_t)cfg.at("NumTasks").as_int() != c.shape[0] * c.shape[1] * g.tiles_m * g.tiles_n)
            ARK_ERR(PlanError, "MatmulSwiglu: NumTasks must be batch * (rows / ", tm, ") * (hidden / 128)");
        d.kind = DEV_GEMM;
        d.gemm_tile_m = tm; d.gemm_tile_n = tn;
        return d;
    }

    if (type == "Matmul") {
        if (n_slots != 1 || slot_warps != block_warps || slot_warps * 64 != kGemmThreads)
            ARK_ERR(UnsupportedError, "Matmul tasks need one slot of ", kGemmThreads / 64,
                    " waves spanning the whole workgroup (NumWarps ", slot_warps,
                    ", NumWarpsPerProcessor ", block_warps, ", slots ", n_slots, ")");
        View4 a = L.view(op->read_tensors()[0]), b = L.view(op->read_tensors()[1]);
        View4 c = L.view(op->write_tensors()[0]);
        if (a.dtype != 0 && a.dtype != 1 && a.dtype != 2)
            ARK_ERR(UnsupportedError, "Matmul supports FP32/FP16/BF16 operands only");
        const bool f32 = (a.dtype == 0);
        const bool ta = i_arg("TransposeInput"), tb = i_arg("TransposeOther");
        ark::Dims mnk = ark::matmul_problem_size(op->read_tensors()[0]->padded_shape(),
                                                 op->read_tensors()[1]->padded_shape(), ta, tb);
        if (!cfg.contains("TileShapeMNK")) ARK_ERR(PlanError, "Matmul config needs TileShapeMNK");
        auto tile = cfg.at("TileShapeMNK").as_int_vector();
        const int tm = (int)tile.at(0), tn = (int)tile.at(1);
        if (tm == 16) {
            // skinny matmul: up to 16 rows against W[K,N], cut into 256 x 128 units
            if (tn != kGemvCols || (int)tile.at(2) != kGemvUnitK)
                ARK_ERR(PlanError, "a 16-row Matmul tile must be 16x", kGemvCols, "x", kGemvUnitK);
            if (tb) ARK_ERR(UnsupportedError, "the skinny Matmul body needs the other operand stored [K,N]");
            if (c.shape[0] * c.shape[1] != 1 || c.shape[2] > 16)
                ARK_ERR(PlanError, "the skinny Matmul body takes one batch of at most 16 rows");
            if (slot_sram < kGemvLdsBytes)
                ARK_ERR(PlanError, "the skinny Matmul body needs ", kGemvLdsBytes,
                        " bytes of SRAM, the slot has ", slot_sram);
            GemvDesc &g = d.gemv;
            g.x = a.ptr; g.w = b.ptr; g.y = c.ptr;
            g.m = (int)c.shape[2]; g.n = (int)c.shape[3]; g.k = (int)a.shape[3];
            g.ldx = (int)a.es[2]; g.ldw = (int)b.es[2]; g.ldy = (int)c.es[2];
            if ((g.n % 8) || (g.ldx % 8) || (g.ldw % 8) || ((uintptr_t)a.ptr & 15) || ((uintptr_t)b.ptr & 15))
                ARK_ERR(UnsupportedError,
                        "skinny Matmul operands must start 16-byte aligned with N and row pitches % 8 == 0");
            g.dtype = a.dtype;
            const int tasks = (int)cfg.at("NumTasks").as_int();
            (void)gemv_partition(g, tasks);
            if (g.num_tasks != tasks)
                ARK_ERR(PlanError, "a skinny Matmul of ", (int64_t)g.n_blocks * g.k_units,
                        " units cannot be dealt to ", tasks, " tasks");
            // room for the partial tiles of the finest cut the executor may choose for the block
            g.max_parts = std::max(g.max_parts, std::max(1, g.k_units / kGemvMinStretch));
            const size_t ws_bytes = gemv_counter_bytes(g.n_blocks) +
                                    (size_t)g.n_blocks * g.max_parts * g.m * kGemvCols * sizeof(float);
            char *ws = static_cast<char *>(L.scratch(ws_bytes));
            g.counters = reinterpret_cast<unsigned int *>(ws);
            g.partial = reinterpret_cast<float *>(ws + gemv_counter_bytes(g.n_blocks));
            d.kind = DEV_GEMV;
            return d;
        }
        const bool known = (tm == 256 || tm == 128) && (tn == 256 || tn == 128);
        if (!known) ARK_ERR(UnsupportedError, "no GEMM body for tile ", tm, "x", tn);
        if ((ta || f32) && (tm != 128 || tn != 128))
            ARK_ERR(UnsupportedError, "Matmul with TransposeInput or FP32 operands runs on 128x128 tiles only, got ",
                    tm, "x", tn);
        if (mnk[0] % tm || mnk[1] % tn || mnk[2] % kGemmMinK)
            ARK_ERR(PlanError, "output padded shape MNK ", mnk, " should be divisible by tile shape <",
                    tm, ", ", tn, ", ", kGemmMinK, ">");
        const int lds_need = f32 ? kGemmF32LdsBytes : ark::gemm_lds_bytes(tm, tn);
        if (slot_sram < lds_need)
            ARK_ERR(PlanError, "Matmul tile ", tm, "x", tn, " needs ", lds_need,
                    " bytes of SRAM, the slot has ", slot_sram);
        GemmDesc &g = d.gemm;
        g.a = a.ptr; g.b = b.ptr; g.c = c.ptr;
        g.m = (int)mnk[0]; g.n = (int)mnk[1]; g.k = (int)mnk[2];
        g.lda = (int)a.es[2]; g.ldb = (int)b.es[2]; g.ldc = (int)c.es[2];
        const int vec = f32 ? 4 : 8;  // elements per 16-byte vector
        if ((g.lda % vec) || (g.ldb % vec) || ((uintptr_t)a.ptr & 15) || ((uintptr_t)b.ptr & 15))
            ARK_ERR(UnsupportedError, "Matmul operands must start 16-byte aligned with row pitches of whole 16-byte vectors");
        g.batch_c = (int)c.shape[1];
        for (int i = 0; i < 2; ++i) {
            g.a_bs[i] = (a.shape[i] == 1) ? 0 : a.es[i];
            g.b_bs[i] = (b.shape[i] == 1) ? 0 : b.es[i];
            g.c_bs[i] = c.es[i];
        }
        g.trans_b = tb;
        g.trans_a = ta ? 1 : 0;
        g.dtype = a.dtype;
        g.tiles_m = g.m / tm; g.tiles_n = g.n / tn;
        g.store_m = (int)c.shape[2]; g.store_n = (int)c.shape[3];
        g.batch_total = (int)(c.shape[0] * c.shape[1]);
        g.split_k = cfg.contains("SplitK") ? (int)cfg.at("SplitK").as_int() : 1;
        const int64_t tiles = (int64_t)g.batch_total * g.tiles_m * g.tiles_n;
        if (g.split_k != 1 && g.split_k != 2) ARK_ERR(PlanError, "Matmul: SplitK must be 1 or 2, got ", g.split_k);
        if ((int64_t)cfg.at("NumTasks").as_int() != tiles * g.split_k)
            ARK_ERR(PlanError, "Matmul: NumTasks must be SplitK * batch * (M / ", tm, ") * (N / ", tn, ") = ",
                    tiles * g.split_k, ", got ", cfg.at("NumTasks").as_int());
        if (g.split_k == 2) {
            if (tm != 256 || tn != 256 || ta || f32 || (g.k % (2 * kGemmMinK)) || g.k < 8 * kGemmMinK)
                ARK_ERR(UnsupportedError, "Matmul: SplitK 2 runs on 256x256 tiles of FP16/BF16 operands with K % ",
                        2 * kGemmMinK, " == 0, K >= ", 8 * kGemmMinK, " and no TransposeInput");
            // The sender's part of K is shorter by twice the skew: its partial sums are then
            // written while the finisher still multiplies, and the finisher finds them there.
            // (2048 x 4096 x 4096, finisher's time: 70.6 us with equal parts, 67.5 with 192, 72.2
            // with 384; writing and announcing a tile's partial sums takes the time of ~6 K tiles.)
            int64_t skew = 192;
            if (const char *e = std::getenv("ARKMI_SPLITK_SKEW")) skew = std::atoll(e);
            skew = std::max<int64_t>(0, skew) / kGemmMinK * kGemmMinK;
            const int64_t min_part = 4 * kGemmMinK;  // a part of K fills the stage ring at least once
            int64_t at = (int64_t)g.k / 2 + skew;
            at = std::min<int64_t>(at, g.k - min_part);
            at = std::max<int64_t>(at, min_part);
            g.split_at = (int)at;
            // the sender's partial accumulators + one full/empty word per tile
            const size_t counter_bytes = ((size_t)tiles * 4 + 255) / 256 * 256;
            const size_t tile_bytes = (size_t)kGemmThreads * (256 / 2 / 16) * (256 / 4 / 16) * 16;
            char *ws = static_cast<char *>(L.scratch(counter_bytes + (size_t)tiles * tile_bytes));
            g.arrivals = reinterpret_cast<unsigned int *>(ws);
            g.partial = reinterpret_cast<float *>(ws + counter_bytes);
        }
        d.kind = DEV_GEMM;
        d.gemm_tile_m = tm; d.gemm_tile_n = tn;
        return d;
    }

    const bool is_reduce = (type == "ReduceSum" || type == "ReduceMax" || type == "ReduceMean");
    if (is_reduce || type == "Softmax" || type == "Layernorm" || type == "Rmsnorm") {
        View4 in = L.view(op->read_tensors()[0]);
        ark::ModelTensorRef out_t = op->write_tensors()[0];
        RowOpDesc &r = d.row;
        r.dtype = float_code(in, type);
        r.in = in.ptr;
        r.rows = in.shape[0] * in.shape[1] * in.shape[2];
        r.cols = (int)in.shape[3];
        r.dim_c = (int)in.shape[1];
        r.dim_h = (int)in.shape[2];
        for (int i = 0; i < 3; ++i) r.in_s[i] = in.es[i];
        if (is_reduce) {
            int axis = (int)i_arg("Axis");
            const int nd = op->read_tensors()[0]->shape().ndims();
            if (axis < 0) axis += nd;
            r.kind = type == "ReduceSum" ? ROW_SUM : type == "ReduceMax" ? ROW_MAX : ROW_MEAN;
            // the output with the reduced axis kept as extent 1
            ark::Dims osh = out_t->shape(), ost = out_t->strides(), oof = out_t->offsets();
            if (!i_arg("KeepDim")) {
                osh.insert(axis, 1); ost.insert(axis, 1); oof.insert(axis, 0);
            }
            ark::ModelTensor kept(out_t->data_type(), out_t->buffer(), osh, ost, oof, ark::Dims{});
            auto kept_ref = std::make_shared<ark::ModelTensor>(kept);
            View4 out = L.view(kept_ref);
            r.out = out.ptr;
            for (int i = 0; i < 3; ++i) r.out_s[i] = out.es[i];
            if (axis != nd - 1) {
                // one output per thread; the descriptor's row fields describe the output
                const int axis4 = axis + (4 - nd);
                r.red_len = (int)in.shape[axis4];
                r.red_stride = in.es[axis4];
                r.rows = out.shape[0] * out.shape[1] * out.shape[2];
                r.cols = (int)out.shape[3];
                r.dim_c = (int)out.shape[1];
                r.dim_h = (int)out.shape[2];
                if (r.red_len < 1) ARK_ERR(PlanError, type, ": empty reduction axis");
                if ((int64_t)cfg.at("NumTasks").as_int() * slot_warps * 64 < r.rows * r.cols)
                    ARK_ERR(PlanError, type, ": ", cfg.at("NumTasks").as_int(), " tasks of ", slot_warps * 64,
                            " threads do not cover ", r.rows * r.cols, " outputs");
                d.kind = DEV_ROW;
                return d;
            }
        } else {
            View4 out = L.view(out_t);
            r.out = out.ptr;
            for (int i = 0; i < 3; ++i) r.out_s[i] = out.es[i];
            r.kind = type == "Softmax" ? ROW_SOFTMAX : type == "Layernorm" ? ROW_LAYERNORM : ROW_RMSNORM;
            if (type != "Softmax") r.eps = f_arg("Eps");
            if (type == "Softmax") {
                r.scale = op->args().count("Scale") ? f_arg("Scale") : 1.0f;
                if (op->read_tensors().size() > 1) {
                    View4 mk = L.view(op->read_tensors()[1]);
                    if (mk.dtype != in.dtype) ARK_ERR(PlanError, "Softmax: the mask must have the input's type");
                    if (mk.shape[3] != in.shape[3] || mk.es[3] != 1)
                        ARK_ERR(PlanError, "Softmax: the mask must span the last axis densely");
                    r.weight = mk.ptr;
                    for (int i = 0; i < 3; ++i) {
                        if (mk.shape[i] != in.shape[i] && mk.shape[i] != 1)
                            ARK_ERR(PlanError, "Softmax: the mask does not broadcast to the input");
                        r.w_s[i] = (mk.shape[i] == 1 && in.shape[i] > 1) ? 0 : mk.es[i];
                    }
                }
                r.prescale = (r.weight || r.scale != 1.0f) ? 1 : 0;
            }
            if (type == "Rmsnorm" && op->read_tensors().size() > 1) {
                View4 w = L.view(op->read_tensors()[1]);
                r.weight = w.ptr;
                r.weight_fp32 = (w.dtype == 0);
            }
        }
        const int64_t rpw = cfg.contains("RowsPerWave") ? cfg.at("RowsPerWave").as_int() : 1;
        if (rpw < 1 || rpw > 64) ARK_ERR(PlanError, type, ": RowsPerWave must be in [1, 64]");
        r.rows_per_wave = (int)rpw;
        // the rows of a task share the weights: stage them in LDS when the slot has room
        r.weight_lds = (r.kind == ROW_RMSNORM && r.weight && r.weight_fp32 && (r.cols % 4) == 0 &&
                        ((uintptr_t)r.weight % 16) == 0 && (int64_t)r.cols * 4 <= slot_sram) ? 1 : 0;
        if ((int64_t)cfg.at("NumTasks").as_int() * slot_warps * rpw < r.rows)
            ARK_ERR(PlanError, type, ": ", cfg.at("NumTasks").as_int(), " tasks of ", slot_warps, " waves x ", rpw,
                    " rows do not cover ", r.rows, " rows");
        d.kind = DEV_ROW;
        return d;
    }

    if (type == "Embedding") {
        View4 in = L.view(op->read_tensors()[0]), w = L.view(op->read_tensors()[1]);
        View4 out = L.view(op->write_tensors()[0]);
        if (in.dtype != 3) ARK_ERR(PlanError, "Embedding: the index tensor must be INT32");
        if (w.dtype != out.dtype || w.dtype < 0 || w.dtype > 2)
            ARK_ERR(UnsupportedError, "Embedding supports FP32/FP16/BF16 tables and outputs of one type");
        if (w.shape[0] * w.shape[1] != 1 || w.es[3] != 1 || out.es[3] != 1 || out.shape[3] != w.shape[3])
            ARK_ERR(PlanError, "Embedding: the table must be [num_embeddings, dim] and the output [..., dim], both dense along dim");
        EmbedDesc &e = d.emb;
        e.idx = reinterpret_cast<const int32_t *>(in.ptr);
        e.weight = w.ptr; e.out = out.ptr;
        e.rows = out.shape[0] * out.shape[1] * out.shape[2];
        e.dim_c = (int)out.shape[1]; e.dim_h = (int)out.shape[2];
        // the indices' [.., a, b, c] line up with the output's [a, b, c, dim]
        if (in.shape[1] * in.shape[2] * in.shape[3] != e.rows || in.shape[0] != 1)
            ARK_ERR(PlanError, "Embedding: one index per output row expected");
        for (int i = 0; i < 3; ++i) {
            e.idx_s[i] = in.es[i + 1];
            e.out_s[i] = out.es[i];
        }
        e.w_pitch = w.es[2];
        e.emb_dim = (int)w.shape[3]; e.num_emb = (int)w.shape[2];
        e.elem = (int)w.elem;
        if ((int64_t)cfg.at("NumTasks").as_int() * slot_warps < e.rows)
            ARK_ERR(PlanError, "Embedding: ", cfg.at("NumTasks").as_int(), " tasks of ", slot_warps,
                    " waves do not cover ", e.rows, " rows");
        d.kind = DEV_EMBED;
        return d;
    }

    if (type == "Attention") {
        View4 q = L.view(op->read_tensors()[0]), k = L.view(op->read_tensors()[1]), v = L.view(op->read_tensors()[2]);
        View4 o = L.view(op->write_tensors()[0]);
        AttnDesc &a = d.attn;
        a.dtype = float_code(q, type);
        if (a.dtype == 0) ARK_ERR(UnsupportedError, "Attention supports FP16/BF16 tensors");
        if (q.shape[3] != kAttnD) ARK_ERR(UnsupportedError, "Attention supports head_dim ", kAttnD);
        if (slot_sram < kAttnLdsBytes)
            ARK_ERR(PlanError, "Attention needs ", kAttnLdsBytes, " bytes of SRAM, the slot has ", slot_sram);
        auto fill = [&](const View4 &t, const void *&ptr, int64_t (&st)[3], const char *what) {
            if (t.es[3] != 1 || ((uintptr_t)t.ptr & 15) || (t.es[0] % 8) || (t.es[1] % 8) || (t.es[2] % 8))
                ARK_ERR(UnsupportedError, "Attention: ", what,
                        " must be dense along head_dim, 16-byte aligned, with strides that are multiples of 8");
            ptr = t.ptr;
            st[0] = t.es[0]; st[1] = t.es[1]; st[2] = t.es[2];
        };
        const void *op_ptr = nullptr;
        fill(q, a.q, a.q_s, "q");
        fill(k, a.k, a.k_s, "k");
        fill(v, a.v, a.v_s, "v");
        fill(o, op_ptr, a.o_s, "the output");
        a.o = const_cast<void *>(op_ptr);
        a.batch = (int)q.shape[0]; a.seq_q = (int)q.shape[1]; a.heads = (int)q.shape[2];
        a.seq_k = (int)k.shape[1];
        a.scale = f_arg("Scale");
        a.causal = (int)i_arg("Causal");
        a.q_blocks = (a.seq_q + kAttnQBlock - 1) / kAttnQBlock;
        if ((int64_t)cfg.at("NumTasks").as_int() != (int64_t)attn_num_tasks(a.batch, a.heads, a.seq_q))
            ARK_ERR(PlanError, "Attention: NumTasks must be batch * heads * ceil(seq / ", kAttnQBlock, ")");
        d.kind = DEV_ATTN;
        return d;
    }

    // elementwise family
    struct Ew { const char *type; int op; int inputs; };
    static const Ew table[] = {
        {"Add", EW_ADD, 2}, {"Sub", EW_SUB, 2}, {"Mul", EW_MUL, 2}, {"Div", EW_DIV, 2}, {"SiluMul", EW_SILU_MUL, 2},
        {"Rope", EW_ROPE, 2}, {"Exp", EW_EXP, 1}, {"Gelu", EW_GELU, 1}, {"Relu", EW_RELU, 1},
        {"Rsqrt", EW_RSQRT, 1}, {"Sigmoid", EW_SIGMOID, 1}, {"Sqrt", EW_SQRT, 1},
        {"Copy", EW_COPY, 1}, {"Cast", EW_CAST, 1}, {"Transpose", EW_COPY, 1},
        {"ScalarAssign", EW_SCALAR_ASSIGN, 0}, {"ScalarAdd", EW_SCALAR_ADD, 1},
        {"ScalarMul", EW_SCALAR_MUL, 1}};
    for (const auto &e : table) {
        if (type != e.type) continue;
        View4 out = L.view(op->write_tensors()[0]);
        EwiseDesc &w = d.ew;
        int perm4[4] = {0, 1, 2, 3};
        const int *perm = nullptr;
        if (type == "Transpose") {
            auto it = op->args().find("Permutation");
            if (it == op->args().end()) ARK_ERR(PlanError, "Transpose: missing Permutation");
            const ark::Dims &p = it->second.dims;
            const int x = 4 - p.ndims();
            for (int i = 0; i < p.ndims(); ++i) perm4[i + x] = (int)p[i] + x;
            perm = perm4;
        }
        // "ViewAs": the op runs over a reshape of its output (the [rows, cols] of the
        // producer whose task it shares); every operand is re-addressed over it
        int64_t as2d[4] = {0, 0, 0, 0};
        const bool viewed = cfg.contains("ViewAs");
        if (viewed) {
            auto v = cfg.at("ViewAs").as_int_vector();
            int64_t n_view = 1, n_out = 1;
            for (int i = 0; i < 4; ++i) n_out *= out.shape[i];
            for (auto x : v) n_view *= x;
            if (v.size() != 4 || v[0] != 1 || v[1] != 1 || v[2] <= 0 || v[3] <= 0 || n_view != n_out || perm)
                ARK_ERR(PlanError, type, ": ViewAs must be [1, 1, rows, cols] with the output's element count");
            for (int i = 0; i < 4; ++i) as2d[i] = v[i];
        }
        const int64_t out_shape4[4] = {out.shape[0], out.shape[1], out.shape[2], out.shape[3]};
        auto re_address = [&](EwTensor t, bool may_wrap, int32_t *period) {
            if (!viewed) return t;
            const ark::Collapsed2D c = ark::collapse_to_2d(out_shape4, t.s, as2d[3]);
            if (!c.ok || (c.col_period != 0 && (!may_wrap || c.col_period % kEwGroup)))
                ARK_ERR(PlanError, type, ": an operand cannot be addressed over the ViewAs shape");
            t.s[0] = 0; t.s[1] = 0; t.s[2] = c.row_stride; t.s[3] = c.col_stride;
            if (period) *period = (int32_t)c.col_period;
            return t;
        };
        w.in1_period = 0;
        w.out = re_address(ew_operand(out, out.shape, nullptr), false, nullptr);
        auto code = [&](const View4 &v) {
            if (v.dtype > 3) ARK_ERR(UnsupportedError, "op ", type, ": unsupported tensor type");
            return v.dtype;
        };
        w.dt_out = code(out);
        w.dt_in = w.dt_out;
        if (e.inputs >= 1) {
            View4 in0 = L.view(op->read_tensors()[0]);
            w.in0 = re_address(ew_operand(in0, out.shape, perm), false, nullptr);
            w.dt_in = code(in0);
        }
        if (e.inputs >= 2) {
            View4 in1 = L.view(op->read_tensors()[1]);
            w.in1 = re_address(ew_operand(in1, out.shape, nullptr), true, &w.in1_period);
        }
        if (viewed) {
            for (int i = 0; i < 4; ++i) {
                out.shape[i] = as2d[i];
                w.shape[i] = (int)as2d[i];
            }
        } else {
            for (int i = 0; i < 4; ++i) w.shape[i] = (int)out.shape[i];
        }
        if (w.dt_in != w.dt_out && e.op != EW_CAST)
            ARK_ERR(PlanError, "op ", type, ": input and output types differ");
        {
            const bool int_ok = e.op == EW_CAST || e.op == EW_COPY || e.op == EW_ADD || e.op == EW_SUB ||
                                e.op == EW_MUL || e.op == EW_DIV || e.op == EW_SCALAR_ASSIGN ||
                                e.op == EW_SCALAR_ADD || e.op == EW_SCALAR_MUL;
            if ((w.dt_in == 3 || w.dt_out == 3) && !int_ok)
                ARK_ERR(UnsupportedError, "op ", type, " is not implemented for INT32");
        }
        if (e.op == EW_ROPE && (out.shape[3] % 2) != 0)
            ARK_ERR(PlanError, "Rope needs an even innermost dimension");
        w.op = e.op;
        if (e.op == EW_SCALAR_ASSIGN) w.param = f_arg("Value");
        if (e.op == EW_SCALAR_ADD || e.op == EW_SCALAR_MUL) w.param = f_arg("Factor");
        if (w.dt_out == 3 && (e.op == EW_SCALAR_ASSIGN || e.op == EW_SCALAR_ADD || e.op == EW_SCALAR_MUL)) {
            // The scalar travels as a float (as in the plan file) and the body
            // converts it to int32 by truncation.  That conversion is defined
            // only inside the int32 range; a value beyond 2^24 in magnitude is
            // already rounded to float precision when it gets here.
            const float v = w.param;
            if (!(v >= -2147483648.0f && v < 2147483648.0f))
                ARK_ERR(UnsupportedError, "op ", type, ": INT32 scalar ", v, " is outside the int32 range");
        }
        if (!cfg.contains("Tile")) ARK_ERR(PlanError, type, " config needs Tile");
        auto tile = cfg.at("Tile").as_int_vector();
        int64_t th = tile.at(0), tw = tile.at(1);
        if (th < 0) th = out.shape[2];
        if (tw < 0) tw = out.shape[3];
        if (th == 0 || tw == 0) ARK_ERR(PlanError, type, ": tile extents must be non-zero");
        if (e.op == EW_ROPE && (tw % 2) != 0) ARK_ERR(PlanError, "Rope needs an even tile width");
        w.tile_h = (int)th; w.tile_w = (int)tw;
        w.tiles_h = (int)ark::div_up(out.shape[2], th);
        w.tiles_w = (int)ark::div_up(out.shape[3], tw);
        {
            // the vector walk: dense or broadcast innermost axis, whole aligned
            // groups of 8, (n, c) slices addressable with 32-bit byte offsets
            auto fits = [&](const EwTensor &t, size_t es, bool is_out) {
                if (t.s[3] != 1 && !(t.s[3] == 0 && !is_out)) return false;
                if (t.s[3] == 1 && ((uintptr_t)t.ptr % 16)) return false;
                for (int i = 0; i < 3; ++i)
                    if (t.s[3] == 1 && (t.s[i] * (int64_t)es) % 16) return false;
                const int64_t extent = (out.shape[2] * std::abs(t.s[2]) + out.shape[3] * std::abs(t.s[3])) * (int64_t)es;
                return extent < ((int64_t)1 << 31);
            };
            const size_t es_in = (w.dt_in == 1 || w.dt_in == 2) ? 2 : 4, es_out = (w.dt_out == 1 || w.dt_out == 2) ? 2 : 4;
            bool fast = (out.shape[3] % kEwGroup) == 0 && (tw % kEwGroup) == 0 && fits(w.out, es_out, true);
            if (e.inputs >= 1) fast = fast && fits(w.in0, es_in, false);
            if (e.inputs >= 2) fast = fast && fits(w.in1, es_in, false);
            // a wrapping second input: the vector walk exists for Rope with a power-of-two period
            if (w.in1_period > 0)
                fast = fast && e.op == EW_ROPE && (w.in1_period & (w.in1_period - 1)) == 0;
            w.fast = fast ? 1 : 0;
        }
        d.kind = DEV_EWISE;
        return d;
    }
    ARK_ERR(UnsupportedError, "op type ", type, " has no device implementation in this backend");
}

}  // namespace

// ---------------------------------------------------------------------------
// data hazards between task groups (for eliding barriers nobody needs)
// ---------------------------------------------------------------------------
namespace {

// A matmul with one elementwise op behind it (Add, Sub, Mul, Div with the matmul's result as
// either input; Rope with it as the first): where every tile of C leaves through the staged
// store of gemm_tile and the op's operands are dense rows aligned to 16 bytes, the op is
// folded into that store (GemmDesc::fuse_*) instead of reading the tile back.  The values are
// the same bits either way: the store rounds C to the tensor type first, as the op would read
// it.  ARKMI_GEMM_FOLD_STORE=0 keeps the op a pass of its own.
static bool fold_into_store(DevOp &lead, const DevOp &next) {
    if (const char *e = getenv("ARKMI_GEMM_FOLD_STORE"))
        if (atoi(e) == 0) return false;
    if (lead.kind != DEV_GEMM || next.kind != DEV_EWISE) return false;
    GemmDesc &g = lead.gemm;
    const EwiseDesc &w = next.ew;
    const int tm = lead.gemm_tile_m, tn = lead.gemm_tile_n;
    // the staged store: fp16/bf16 tiles 128 or 256 columns wide, whole tiles, aligned rows
    if ((g.dtype != 1 && g.dtype != 2) || g.trans_a || g.b2 || g.batch_total != 1) return false;
    if ((tn != 128 && tn != 256) || (tm != 128 && tm != 256)) return false;
    if (g.store_m % tm || g.store_n % tn || (g.ldc % 8) || ((uintptr_t)g.c % 16)) return false;
    const bool arith = w.op == EW_ADD || w.op == EW_SUB || w.op == EW_MUL || w.op == EW_DIV;
    if (!arith && w.op != EW_ROPE) return false;
    if (w.dt_in != g.dtype || w.dt_out != g.dtype || !w.fast) return false;
    if (w.shape[0] != 1 || w.shape[1] != 1 || w.shape[2] != g.store_m || w.shape[3] != g.store_n) return false;
    if (w.tile_h != tm || w.tile_w != tn) return false;
    auto is_c = [&](const EwTensor &t) { return t.ptr == g.c && t.s[2] == g.ldc && t.s[3] == 1; };
    auto dense_rows = [](const EwTensor &t) {
        return t.s[3] == 1 && ((uintptr_t)t.ptr % 16) == 0 && (t.s[2] % 8) == 0 && t.s[2] >= 0 &&
               t.s[2] < ((int64_t)1 << 31);
    };
    const EwTensor *other = nullptr;
    int c_second = 0, period = 0;
    if (is_c(w.in0)) {
        other = &w.in1;
        period = w.in1_period;
    } else if (arith && is_c(w.in1) && w.in1_period == 0) {
        other = &w.in0;
        c_second = 1;
    } else {
        return false;
    }
    if (!dense_rows(*other) || !dense_rows(w.out) || w.out.s[2] == 0 || period < 0 || (period % 8)) return false;
    g.fuse_other = other->ptr;
    g.fuse_out = w.out.ptr;
    g.fuse_kind = 1 + w.op;
    g.fuse_c_second = c_second;
    g.fuse_ld_other = (int)other->s[2];
    g.fuse_ld_out = (int)w.out.s[2];
    g.fuse_period = period;
    return true;
}

struct Access {
    size_t buffer;
    size_t begin, end;  // byte range inside the buffer
    bool write;
    std::string view;   // type, shape, strides, offsets, padded shape: equal views address alike
    ark::Dims shape;
    int step = -1;      // schedule step of the task group that makes the access
    // True when task t of the op touches only tile t of this tensor: every access of a
    // tiled elementwise op, and the *result* of a matmul.  A matmul task reads a whole
    // row panel of its first operand and a column panel of its second, whoever wrote them.
    bool tile_local = false;
    // A read that spans more than the reading task's own part of the tensor (the
    // operands of a matmul or of attention): never a workgroup-local matter.
    bool panel_read = false;
};

bool tiled_elementwise(const std::string &type);

void add_access(std::vector<Access> &out, const Json &tensor_json, bool write, const std::string &op_type,
                bool split_k) {
    auto t = ark::ModelTensor::deserialize(tensor_json);
    ark::Dims st = t->strides(), pd = t->padded_shape();
    size_t last = 0, pitch = 1;
    for (int i = st.ndims() - 1; i >= 0; --i) {
        last += (size_t)(pd[i] - 1) * pitch;
        pitch *= (size_t)st[i];
    }
    const size_t elem = t->data_type()->bytes();
    Access a{t->buffer()->id(), t->byte_offset(), t->byte_offset() + (last + 1) * elem, write, "", t->shape(), -1};
    // (a matmul that splits K is finished by whichever half arrives last: no fixed workgroup)
    a.tile_local = tiled_elementwise(op_type) || (write && op_type == "Matmul" && !split_k);
    a.panel_read = !write && (op_type == "Matmul" || op_type == "MatmulSwiglu" || op_type == "Attention");
    a.view = tensor_json.at("DataType").dump() + tensor_json.at("Shape").dump() + tensor_json.at("Strides").dump() +
             tensor_json.at("Offsets").dump() + tensor_json.at("PaddedShape").dump();
    out.push_back(a);
}

std::vector<Access> accesses_of(const Json &task_info) {
    std::vector<Access> v;
    for (const auto &op : task_info.at("Ops").elements()) {
        const std::string type = op.at("Type").as_string();
        const Json &cfg = op.at("Config");
        const bool split = cfg.contains("SplitK") && cfg.at("SplitK").as_int() > 1;
        for (const auto &t : op.at("ReadTensors").elements()) add_access(v, t, false, type, split);
        for (const auto &t : op.at("WriteTensors").elements()) add_access(v, t, true, type, split);
        for (const auto &t : op.at("ResultTensors").elements()) add_access(v, t, true, type, split);
    }
    return v;
}

bool overlap(const Access &x, const Access &y) {
    return x.buffer == y.buffer && (x.write || y.write) && x.begin < y.end && y.begin < x.end;
}

// The elementwise ops whose task t covers exactly tile t of the output, for
// every operand that has the output's shape.
bool tiled_elementwise(const std::string &type) {
    static const char *names[] = {"Add", "Sub", "Mul", "Div", "SiluMul", "Rope", "Exp", "Gelu", "Relu", "Rsqrt", "Sigmoid",
                                  "Sqrt", "Copy", "Cast", "ScalarAssign", "ScalarAdd", "ScalarMul"};
    for (const char *n : names)
        if (type == n) return true;
    return false;
}

std::string dims4_key(const ark::Dims &d) {
    const ark::Dims d4 = d.dims4();
    std::string k;
    for (int i = 0; i < d4.ndims(); ++i) k += std::to_string((long long)d4[i]) + ",";
    return k;
}

// How a task group cuts its output: every op of the task writes a tensor of
// `shape` in tiles of th x tw, tile index row-major with the W tile fastest (the
// order of both the elementwise body and the GEMM body).  Not every task has one.
struct Tiling {
    bool ok = false;
    std::string shape;  // the outputs' common 4-D shape
    int64_t th = 0, tw = 0;
};

Tiling tiling_of(const Json &task_info) {
    Tiling t;
    for (const auto &op : task_info.at("Ops").elements()) {
        const std::string type = op.at("Type").as_string();
        const Json &cfg = op.at("Config");
        int64_t th, tw;
        if (type == "Matmul" && cfg.contains("TileShapeMNK")) {
            auto tile = cfg.at("TileShapeMNK").as_int_vector();
            th = tile.at(0); tw = tile.at(1);
            if (th < 32) return Tiling();  // the skinny matmul deals units of W, not output tiles
            if (cfg.contains("SplitK") && cfg.at("SplitK").as_int() > 1) return Tiling();  // no fixed workgroup per tile
        } else if (tiled_elementwise(type) && cfg.contains("Tile")) {
            auto tile = cfg.at("Tile").as_int_vector();
            th = tile.at(0); tw = tile.at(1);
        } else {
            return Tiling();
        }
        const std::string shape = dims4_key(ark::Dims(op.at("WriteTensors").at((size_t)0).at("Shape").as_int_vector()));
        if (t.ok && (shape != t.shape || th != t.th || tw != t.tw)) return Tiling();
        t.ok = true; t.shape = shape; t.th = th; t.tw = tw;
    }
    return t;
}

// True when the two task groups cut equal output shapes into the same tiles and
// deal them to the workgroups alike: task t of one and task t of the other run
// on the same workgroup and cover the same elements of any tensor of that shape.
bool same_decomposition(const Json &ti_a, const ScheduleStep &sa, const Json &ti_b, const ScheduleStep &sb,
                        std::string *shape) {
    const Tiling a = tiling_of(ti_a), b = tiling_of(ti_b);
    if (!a.ok || !b.ok || a.shape != b.shape || a.th != b.th || a.tw != b.tw) return false;
    if (shape) *shape = a.shape;
    return sa.proc_b == sb.proc_b && sa.proc_e == sb.proc_e && sa.proc_s == sb.proc_s && sa.proc_cur == sb.proc_cur &&
           sa.task_b == sb.task_b && sa.task_e == sb.task_e && sa.task_s == sb.task_s && sa.gran == sb.gran &&
           sa.n_slots == sb.n_slots && sa.slot_warps == sb.slot_warps;
}

}  // namespace

// ---------------------------------------------------------------------------
// per-task dependency counters (host side)
// ---------------------------------------------------------------------------
// A grid barrier orders every workgroup after every other.  Where everything that crosses it
// is a read of rows that tasks of an earlier group wrote, and both ops are of a kind whose
// tasks map to row ranges of one 2-D row space, the barrier is replaced by counters in device
// memory: a producer task adds one to the counter of the row block it completed (after a
// write-back of its L2), a consumer task waits until the counters of the blocks it reads have
// reached what one iteration contributes times the iteration number.
namespace {

using RowSpan = std::function<void(int, int64_t &, int64_t &)>;  // task index -> rows [r0, r1)

// One operand of an op as rows of a 2-D row space.
struct RowAccess {
    const char *ptr = nullptr;  // address of row 0
    int64_t pitch = 0;          // bytes between rows
    int64_t width = 0;          // bytes of a row the op touches (<= pitch)
    int64_t rows = 0;
    bool write = false;
    RowSpan span;
};

// Row accesses of one lowered op; an operand whose tasks do not map to row ranges is left out.
std::vector<RowAccess> row_accesses(const DevOp &op, int slot_warps) {
    std::vector<RowAccess> v;
    auto add = [&](const void *p, int64_t pitch, int64_t width, int64_t rows, bool write, RowSpan span) {
        if (!p || pitch <= 0 || rows <= 0 || width <= 0 || (width > pitch && rows > 1)) return;
        RowAccess a;
        a.ptr = static_cast<const char *>(p); a.pitch = pitch; a.width = std::min(width, pitch); a.rows = rows;
        a.write = write; a.span = std::move(span);
        v.push_back(std::move(a));
    };
    if (op.kind == DEV_ROW && op.row.red_len == 0) {
        const RowOpDesc &r = op.row;
        const int64_t elem = r.dtype == 0 ? 4 : 2;
        // rows r = (n, c, h) are equally spaced when the outer strides nest
        auto nested = [&](const int64_t s[3]) {
            const int64_t n = r.rows / std::max<int64_t>(1, (int64_t)r.dim_c * r.dim_h);
            if (r.dim_h > 1 && s[2] <= 0) return false;
            if (r.dim_c > 1 && s[1] != (int64_t)r.dim_h * s[2]) return false;
            if (n > 1 && s[0] != (int64_t)r.dim_c * r.dim_h * s[2]) return false;
            return s[2] > 0;
        };
        const int64_t per_task = (int64_t)slot_warps * std::max(1, r.rows_per_wave);
        const int64_t rows = r.rows;
        RowSpan span = [per_task, rows](int t, int64_t &r0, int64_t &r1) {
            r0 = std::min<int64_t>(rows, (int64_t)t * per_task);
            r1 = std::min<int64_t>(rows, r0 + per_task);
        };
        const bool reduce = r.kind == ROW_SUM || r.kind == ROW_MAX || r.kind == ROW_MEAN;
        if (nested(r.in_s)) add(r.in, r.in_s[2] * elem, (int64_t)r.cols * elem, rows, false, span);
        if (nested(r.out_s)) add(r.out, r.out_s[2] * elem, (reduce ? 1 : (int64_t)r.cols) * elem, rows, true, span);
    } else if (op.kind == DEV_GEMM && op.gemm.dtype != 0 && !op.gemm.trans_a && op.gemm.batch_total == 1) {
        const GemmDesc &g = op.gemm;
        const int bm = op.gemm_tile_m, tiles_n = g.tiles_n, tiles = g.tiles_m * g.tiles_n;
        auto rows_of = [bm, tiles_n, tiles](int64_t limit) -> RowSpan {
            return [bm, tiles_n, tiles, limit](int t, int64_t &r0, int64_t &r1) {
                const int tm = (t % tiles) / tiles_n;
                r0 = std::min<int64_t>(limit, (int64_t)tm * bm);
                r1 = std::min<int64_t>(limit, r0 + bm);
            };
        };
        const int64_t n_out = g.b2 ? g.n / 2 : g.n;
        add(g.a, (int64_t)g.lda * 2, (int64_t)g.k * 2, g.m, false, rows_of(g.m));
        add(g.c, (int64_t)g.ldc * 2, n_out * 2, g.store_m, true, rows_of(g.store_m));
        const int64_t k = g.k;
        if (!g.trans_b) {  // [K, N]: every task reads every row
            add(g.b, (int64_t)g.ldb * 2, (int64_t)g.n * 2, k, false, [k](int, int64_t &r0, int64_t &r1) { r0 = 0; r1 = k; });
        } else {           // [N, K]: the task's columns are rows of the operand
            const int bn = g.b2 ? op.gemm_tile_n / 2 : op.gemm_tile_n;
            RowSpan cols = [bn, tiles_n, tiles, n_out](int t, int64_t &r0, int64_t &r1) {
                const int tn = (t % tiles) % tiles_n;
                r0 = std::min<int64_t>(n_out, (int64_t)tn * bn);
                r1 = std::min<int64_t>(n_out, r0 + bn);
            };
            add(g.b, (int64_t)g.ldb * 2, k * 2, n_out, false, cols);
            if (g.b2) add(g.b2, (int64_t)g.ldb * 2, k * 2, n_out, false, cols);
        }
    } else if (op.kind == DEV_EWISE && op.ew.shape[0] * op.ew.shape[1] == 1) {
        const EwiseDesc &e = op.ew;
        const int64_t rows = e.shape[2], cols = e.shape[3];
        const int th = e.tile_h, tiles_h = e.tiles_h, tiles_w = e.tiles_w;
        RowSpan span = [rows, th, tiles_h, tiles_w](int t, int64_t &r0, int64_t &r1) {
            const int i = (t / tiles_w) % tiles_h;
            r0 = std::min<int64_t>(rows, (int64_t)i * th);
            r1 = std::min<int64_t>(rows, r0 + th);
        };
        RowSpan whole = [](int, int64_t &r0, int64_t &r1) { r0 = 0; r1 = 1; };
        const int64_t es_in = (e.dt_in == 1 || e.dt_in == 2) ? 2 : 4, es_out = (e.dt_out == 1 || e.dt_out == 2) ? 2 : 4;
        auto operand = [&](const EwTensor &t, int64_t es, bool write, int64_t period) {
            if (!t.ptr || (t.s[3] != 0 && t.s[3] != 1)) return;
            const int64_t w = (t.s[3] == 0 ? 1 : period > 0 ? period : cols) * es;
            if (t.s[2] == 0) add(t.ptr, w, w, 1, write, whole);  // one row every task reads
            else if (t.s[2] > 0) add(t.ptr, t.s[2] * es, w, rows, write, span);
        };
        operand(e.out, es_out, true, 0);
        if (e.op != EW_SCALAR_ASSIGN) operand(e.in0, es_in, false, 0);
        operand(e.in1, es_in, false, e.in1_period);
    } else if (op.kind == DEV_ATTN) {
        const AttnDesc &a = op.attn;
        const int QB = a.q_blocks, heads = a.heads, batch = a.batch, causal = a.causal;
        const int64_t sq = a.seq_q, sk = a.seq_k;
        auto decode = [QB, heads, batch, causal](int t, int &b, int &qb) {
            const int bh = t / QB;
            qb = t - bh * QB;
            if (causal && bh >= (batch * heads + 1) / 2) qb = QB - 1 - qb;
            b = bh / heads;
        };
        RowSpan q_span = [decode, sq](int t, int64_t &r0, int64_t &r1) {
            int b, qb;
            decode(t, b, qb);
            r0 = (int64_t)b * sq + std::min<int64_t>(sq, (int64_t)qb * kAttnQBlock);
            r1 = (int64_t)b * sq + std::min<int64_t>(sq, (int64_t)(qb + 1) * kAttnQBlock);
        };
        // keys are fetched in whole blocks of kAttnKBlock up to the task's last visible one
        RowSpan kv_span = [decode, sq, sk, causal](int t, int64_t &r0, int64_t &r1) {
            int b, qb;
            decode(t, b, qb);
            int64_t end = sk;
            if (causal) {
                end = std::min<int64_t>(sk, std::min<int64_t>((int64_t)(qb + 1) * kAttnQBlock, sq) + (sk - sq));
                end = std::min<int64_t>(sk, (std::max<int64_t>(0, end) + kAttnKBlock - 1) / kAttnKBlock * kAttnKBlock);
            }
            r0 = (int64_t)b * sk;
            r1 = r0 + end;
        };
        auto rows_ok = [&](const int64_t s[3], int64_t seq) { return s[1] > 0 && (batch == 1 || s[0] == seq * s[1]); };
        const int64_t w = (int64_t)heads * kAttnD * 2;  // all heads of a position, when they are adjacent
        auto width = [&](const int64_t s[3]) { return s[2] == kAttnD ? w : (int64_t)0; };
        if (rows_ok(a.q_s, sq)) add(a.q, a.q_s[1] * 2, width(a.q_s), (int64_t)batch * sq, false, q_span);
        if (rows_ok(a.k_s, sk)) add(a.k, a.k_s[1] * 2, width(a.k_s), (int64_t)batch * sk, false, kv_span);
        if (rows_ok(a.v_s, sk)) add(a.v, a.v_s[1] * 2, width(a.v_s), (int64_t)batch * sk, false, kv_span);
        if (rows_ok(a.o_s, sq)) add(a.o, a.o_s[1] * 2, width(a.o_s), (int64_t)batch * sq, true, q_span);
    }
    return v;
}

// A task group as the dependency analysis sees it.
struct DepGroup {
    int sched_step = -1;   // index into the schedule
    int segment = 0;       // schedule barriers ahead of it
    int group = -1;        // index into the device task groups
    int n_tasks = 0;       // tasks of the group
    int n_signal = 0;      // tasks that finish something (the tiles of a matmul that splits K)
    bool whole_block = false;
    std::vector<Access> acc;      // every operand (byte ranges inside buffers)
    std::vector<RowAccess> rows;  // the operands with a row structure (device addresses)
    // as a producer: the row block each task completes, set on first use
    std::vector<int> signal_map;
    int n_blocks = 0, per_block = 0;
    int counter_base = -1;
    // as a consumer: blocks [lo, hi] of each producer it waits for, per task
    struct Wait {
        int producer;  // index into the DepGroup list
        std::vector<std::pair<int, int>> span;
    };
    std::vector<Wait> waits;
};

const RowAccess *row_of(const DepGroup &g, const char *ptr, bool write) {
    for (const auto &r : g.rows)
        if (r.ptr == ptr && r.write == write) return &r;
    return nullptr;
}

// The row blocks of producer `x` as its write `w` cuts them: every task writes exactly one block
// of `br` rows, the blocks tile the rows, and every block gets the same number of tasks.
bool establish_blocks(DepGroup &x, const RowAccess &w, int64_t *br_out) {
    if (x.n_signal <= 0) return false;
    int64_t r0, r1, br = 0;
    w.span(0, r0, r1);
    br = r1 - r0;
    if (br <= 0) return false;
    std::vector<int> map((size_t)x.n_signal);
    for (int t = 0; t < x.n_signal; ++t) {
        w.span(t, r0, r1);
        if (r1 <= r0 || r0 % br != 0 || r1 != std::min(w.rows, r0 + br)) return false;
        map[(size_t)t] = (int)(r0 / br);
    }
    const int n_blocks = (int)((w.rows + br - 1) / br);
    std::vector<int> count((size_t)n_blocks, 0);
    for (int b : map) {
        if (b >= n_blocks) return false;
        ++count[(size_t)b];
    }
    for (int c : count)
        if (c != count[0] || c == 0) return false;
    if (x.signal_map.empty()) {
        x.signal_map = map;
        x.n_blocks = n_blocks;
        x.per_block = count[0];
    } else if (x.signal_map != map || x.n_blocks != n_blocks) {
        return false;
    }
    *br_out = br;
    return true;
}

constexpr int64_t kLine = 128;  // bytes of an L2 cache line

// Can the read `ay` of group y wait on counters for the write `ax` of group x?  On success the
// blocks each task of y waits for are merged into y.waits.
bool cover_with_counters(std::vector<DepGroup> &groups, int xi, const Access &ax, int yi, const Access &ay,
                         const char *arena, const std::map<size_t, size_t> &buffer_offset) {
    DepGroup &x = groups[(size_t)xi], &y = groups[(size_t)yi];
    if (!ax.write || ay.write || !x.whole_block || !y.whole_block) return false;
    const RowAccess *w = row_of(x, arena + buffer_offset.at(ax.buffer) + ax.begin, true);
    const RowAccess *r = row_of(y, arena + buffer_offset.at(ay.buffer) + ay.begin, false);
    if (!w || !r) return false;
    // A consumer reads through its L2 without invalidating it: lines it fetched for finished
    // rows must hold nothing another task still has to write, so rows own whole lines.
    if ((uintptr_t)w->ptr % kLine || w->pitch % kLine || w->width % kLine) return false;
    if (w->pitch != r->pitch) return false;
    const int64_t delta = r->ptr - w->ptr;
    int64_t shift = delta / w->pitch;
    if (delta < 0 && shift * w->pitch != delta) --shift;
    const int64_t col = delta - shift * w->pitch;
    if (col + r->width > w->pitch) return false;
    int64_t br = 0;
    if (!establish_blocks(x, *w, &br)) return false;
    DepGroup::Wait *wt = nullptr;
    for (auto &q : y.waits)
        if (q.producer == xi) wt = &q;
    if (!wt) {
        y.waits.push_back({xi, std::vector<std::pair<int, int>>((size_t)y.n_tasks, {0, -1})});
        wt = &y.waits.back();
    }
    for (int t = 0; t < y.n_tasks; ++t) {
        int64_t r0, r1;
        r->span(t, r0, r1);
        r0 = std::max<int64_t>(0, r0 + shift);
        r1 = std::min<int64_t>(w->rows, r1 + shift);
        if (r1 <= r0) continue;
        auto &s = wt->span[(size_t)t];
        const int lo = (int)(r0 / br), hi = (int)((r1 - 1) / br);
        if (s.second < s.first) s = {lo, hi};
        else s = {std::min(s.first, lo), std::max(s.second, hi)};
    }
    return true;
}

}  // namespace

// ---------------------------------------------------------------------------
// executor object
// ---------------------------------------------------------------------------
struct Executor {
    int device = 0;
    hipStream_t stream = nullptr;
    bool own_stream = false;
    std::string name;
    std::string plan_text;
    Json plan;
    bool loop_mode = true;

    Schedule sched;
    std::map<size_t, size_t> buffer_offset, buffer_bytes;
    size_t total_bytes = 0;

    char *arena = nullptr;
    LoopControl *ctl = nullptr;
    HostMailbox *mb = nullptr;      // host view
    HostMailbox *mb_dev = nullptr;  // device view
    DevOp *d_ops = nullptr;
    DevTaskGroup *d_groups = nullptr;
    DevStep *d_steps = nullptr;
    TraceRecord *d_trace = nullptr;
    unsigned long long *d_clock = nullptr;
    int wall_khz = 100000;
    std::vector<DevTaskGroup> h_groups;
    size_t trace_len = 0;
    bool trace_enabled = false;
    LoopProgram prog{};

    int grid = 1, threads = 64, lds_bytes = 0;
    int barriers_elided = 0;
    int barriers_local = 0;       // grid barriers replaced by a workgroup-local sync
    int barriers_counted = 0;     // grid barriers replaced by waits on dependency counters
    int gemv_chains = 0;          // runs of skinny matmuls streamed as one sequence
    // Analysis only (no device): compile() stops before anything touches the GPU and keeps the
    // tables it built.  force_deps: -1 take ARKMI_DEP_COUNTERS, 0 / 1 override it.
    bool dry = false;
    int force_deps = -1;
    std::vector<DevStep> dry_steps;
    std::vector<DevWait> dry_waits;
    std::vector<int32_t> dry_spans, dry_signal;
    std::vector<DevOp> dry_ops;
    size_t dry_counters = 0;
    DevWait *d_waits = nullptr;
    int32_t *d_spans = nullptr, *d_signal = nullptr;
    GemvSeqEntry *d_gemv_seq = nullptr;
    unsigned int *d_gemv_claims = nullptr;
    size_t gemv_claim_bytes = 0;
    int attn_xcd_ordered = 0;               // attention ops whose tasks run in the XCD-aware order
    int gemm_xcd_ordered = 0;               // matmuls whose tiles run in the XCD-aware order
    int barriers_widened = 0;               // barriers over part of the grid made full-grid for claimed stretches
    int gemv_claimed = 0;                   // skinny matmuls (or runs of them) whose stretches are claimed at run time
    std::vector<GemvSeqEntry> h_gemv_seq;  // the skinny matmuls' task sequences, per workgroup
    std::vector<int> group_sched_step;      // schedule step of every task group
    unsigned int *d_dep_counters = nullptr;
    size_t dep_counter_bytes = 0;
    bool iteration_local_across_groups = false;  // the local sync between iterations pairs two different groups
    int iteration_sync = 2;       // between iterations of one command: 2 grid barrier, 1 local sync, 0 nothing
    int families = 0;             // OpFamily bits of the compiled ops
    int kernel_families = 0;      // the loop-kernel variant in use
    const void *kernel = nullptr;
    std::vector<void *> scratch_allocs;  // per-op device scratch (split-K partials, counters)
    std::vector<char> group_fused;       // per task group: its elementwise follower rides in the matmul's store
    std::vector<int> h_group_fam;        // OpFamily bits of each task group
    std::vector<const void *> step_kernels_ready;  // step kernels whose LDS limit is set
    std::vector<int> dev_step_of;  // schedule step -> device step, -1 if elided
    int num_dev_steps = 0;
    uint64_t idle_ticks = 0, wait_ticks = 0;
    hipEvent_t ev_begin = nullptr, ev_end = nullptr;
    bool compiled = false, launched = false, destroyed = false;
    int pending_one_shot = 0;

    ~Executor() { release(); }

    void set_device() const { ARKMI_HIP(hipSetDevice(device)); }

    void init(int device_id, void *stream_, const std::string &name_, const std::string &plan_str,
              bool loop) {
        int n = 0;
        ARKMI_HIP(hipGetDeviceCount(&n));
        if (device_id < 0 || device_id >= n)
            ARK_ERR(InvalidUsageError, "Invalid device ID ", device_id);
        device = device_id;
        name = name_;
        loop_mode = loop;
        set_device();
        // ARK_ENFORCE_PLAN_PATH substitutes a plan file (executor.cpp:892-895)
        const std::string &forced = ark::get_env().enforce_plan_path;
        std::string text = plan_str;
        if (!forced.empty()) {
            std::ifstream f(forced);
            if (!f) ARK_ERR(SystemError, "cannot read ARK_ENFORCE_PLAN_PATH file ", forced);
            text.assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
            ARK_LOG(INFO, "Enforce executor plan path: ", forced);
        }
        try {
            plan = Json::parse(text);
        } catch (const std::exception &e) {
            ARK_ERR(PlanError, "failed to parse the plan: ", e.what());
        }
        plan_text = text;
        sched = build_schedule(plan);
        if (plan.at("WorldSize").as_int() != 1 || plan.at("Rank").as_int() != 0)
            ARK_ERR(UnsupportedError, "this backend runs single-GPU plans only (Rank 0, WorldSize 1)");
        if (sched.num_barriers > kMaxBarriers)
            ARK_ERR(UnsupportedError, "plan needs ", sched.num_barriers, " distinct barrier ranges; at most ",
                    kMaxBarriers, " are supported");
        layout_buffers();
        if (stream_) {
            stream = (hipStream_t)stream_;
        } else {
            ARKMI_HIP(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
            own_stream = true;
        }
        // 64 KiB-aligned, zero-filled once: padded regions rely on it
        ARKMI_HIP(hipMalloc((void **)&arena, std::max<size_t>(total_bytes, 256)));
        ARKMI_HIP(hipMemset(arena, 0, std::max<size_t>(total_bytes, 256)));
        ARKMI_HIP(hipMalloc((void **)&ctl, sizeof(LoopControl)));
        ARKMI_HIP(hipHostMalloc((void **)&mb, sizeof(HostMailbox), hipHostMallocMapped));
        std::memset((void *)mb, 0, sizeof(HostMailbox));
        ARKMI_HIP(hipHostGetDevicePointer((void **)&mb_dev, (void *)mb, 0));
        ARKMI_HIP(hipEventCreate(&ev_begin));
        ARKMI_HIP(hipEventCreate(&ev_end));
        ARKMI_HIP(hipDeviceSynchronize());
    }

    // Buffers in ascending id order; size = the largest view of the buffer
    // (executor.cpp:135-139,344-345,375-408).  Each buffer starts 256-byte
    // aligned so that 16-byte vector access never straddles a buffer start.
    void layout_buffers() {
        for (const auto &ti : plan.at("TaskInfos").elements())
            for (const auto &op : ti.at("Ops").elements())
                for (const char *k : {"ReadTensors", "WriteTensors", "ResultTensors"})
                    for (const auto &tj : op.at(k).elements()) {
                        auto t = ark::ModelTensor::deserialize(tj);
                        if (t->buffer()->rank() != -1 && t->buffer()->rank() != 0)
                            ARK_ERR(UnsupportedError, "remote buffers are not supported");
                        size_t &b = buffer_bytes[t->buffer()->id()];
                        b = std::max(b, t->buffer_bytes());
                    }
        size_t off = 0;
        for (const auto &kv : buffer_bytes) {
            buffer_offset[kv.first] = off;
            off += (kv.second + 255) / 256 * 256;
        }
        total_bytes = off;
    }

    void compile() {
        if (destroyed) ARK_ERR(InvalidUsageError, "executor is destroyed");
        if (compiled) return;
        if (!dry) set_device();
        const int block_warps = sched.num_warps_per_processor;
        threads = block_warps * 64;
        grid = sched.num_processors;
        if (threads > kLoopMaxThreads)
            ARK_ERR(UnsupportedError, "NumWarpsPerProcessor ", block_warps, " exceeds the loop kernel's ",
                    kLoopMaxThreads / 64, " waves per workgroup");
        Lowering L{arena, buffer_offset, [this](size_t bytes) {
                       void *p = nullptr;
                       if (dry) {  // addresses are only computed with, never followed
                           static uintptr_t next = (uintptr_t)1 << 46;
                           p = (void *)next;
                           next += (bytes + 255) / 256 * 256;
                           return p;
                       }
                       ARKMI_HIP(hipMalloc(&p, bytes));
                       ARKMI_HIP(hipMemset(p, 0, bytes));
                       scratch_allocs.push_back(p);
                       return p;
                   }};
        std::vector<DevOp> ops;
        std::vector<DevStep> steps;
        h_groups.clear();
        group_fused.clear();
        h_group_fam.clear();
        group_sched_step.clear();
        int max_slot_lds = 0;
        trace_len = 0;
        const Json &task_infos = plan.at("TaskInfos");
        // A barrier of the reference's schedule orders *processors*, whether
        // or not the groups around it touch the same data.  Here a barrier is
        // dropped when the task groups it releases share no buffer range (with
        // at least one writer) with anything run since the last full barrier;
        // ARKMI_KEEP_ALL_BARRIERS=1 keeps the reference's placement.
        const char *keep_env = getenv("ARKMI_KEEP_ALL_BARRIERS");
        const bool elide = !(keep_env && atoi(keep_env) != 0);
        std::vector<Access> pending;
        barriers_elided = 0;
        barriers_local = 0;
        families = 0;
        dev_step_of.assign(sched.steps.size(), -1);
        auto step_accesses = [&](size_t sj) {
            auto a = accesses_of(task_infos.at((size_t)sched.steps[sj].task_info));
            for (auto &x : a) x.step = (int)sj;
            return a;
        };
        // A dependency is local to a workgroup when both ops cut equal output shapes
        // into the same tiles on the same workgroups, both touch the shared tensor
        // tile by tile (an elementwise op, or a matmul as the writer: never a matmul's
        // operand reads, which span whole panels), and both see it through the same
        // view with the output's shape: the elements task t reads are the ones task t
        // of the other op wrote, on the same workgroup.  Such a dependency needs no
        // grid barrier.
        auto local_pair = [&](const Access &x, const Access &y) {
            if (!x.tile_local || !y.tile_local) return false;
            const auto &sx = sched.steps[(size_t)x.step];
            const auto &sy = sched.steps[(size_t)y.step];
            const Json &tx = task_infos.at((size_t)sx.task_info), &ty = task_infos.at((size_t)sy.task_info);
            std::string shape;
            if (!same_decomposition(tx, sx, ty, sy, &shape)) return false;
            if (x.view != y.view || x.begin != y.begin) return false;
            return dims4_key(x.shape) == shape && dims4_key(y.shape) == shape;
        };
        for (size_t si = 0; si < sched.steps.size(); ++si) {
            const auto &st = sched.steps[si];
            DevStep ds{};
            bool local_sync = false;
            if (st.is_barrier && elide) {
                std::vector<Access> next;
                for (size_t sj = si + 1; sj < sched.steps.size() && !sched.steps[sj].is_barrier; ++sj) {
                    auto a = step_accesses(sj);
                    next.insert(next.end(), a.begin(), a.end());
                }
                bool any = false, all_local = true;
                for (const auto &x : pending)
                    for (const auto &y : next)
                        if (overlap(x, y)) {
                            any = true;
                            if (!local_pair(x, y)) {
                                if (getenv("ARKMI_DEBUG_BARRIERS") && all_local)
                                    fprintf(stderr, "barrier %zu stays: steps %d -> %d, views '%s' vs '%s', begin %zu/%zu\n",
                                            si, x.step, y.step, x.view.c_str(), y.view.c_str(), x.begin, y.begin);
                                all_local = false;
                            }
                        }
                if (!any) {
                    ++barriers_elided;
                    continue;
                }
                if (all_local && st.b == 0 && st.e >= grid) {
                    local_sync = true;
                    ++barriers_local;
                } else if (st.b == 0 && st.e >= grid) {
                    pending.clear();
                }
            }
            if (!st.is_barrier) {
                auto a = step_accesses(si);
                pending.insert(pending.end(), a.begin(), a.end());
            }
            if (st.is_barrier && local_sync) {
                ds.kind = STEP_LOCAL_SYNC;
                dev_step_of[si] = (int)steps.size();
                steps.push_back(ds);
                continue;
            }
            if (st.is_barrier) {
                ds.kind = STEP_BARRIER;
                ds.index = st.barrier_id;
                ds.b = st.b; ds.e = st.e; ds.s = st.s;
                ds.count = (st.e - st.b + st.s - 1) / st.s;
                if (st.e > grid) ARK_ERR(PlanError, "barrier range exceeds NumProcessors");
            } else {
                if (st.slot_warps * st.n_slots > block_warps)
                    ARK_ERR(PlanError, "task group needs ", st.slot_warps * st.n_slots,
                            " warps but NumWarpsPerProcessor is ", block_warps);
                if (st.proc_e > grid) ARK_ERR(PlanError, "ProcessorRange exceeds NumProcessors");
                DevTaskGroup g{};
                g.proc_b = st.proc_b; g.proc_e = st.proc_e; g.proc_s = st.proc_s; g.proc_cur = st.proc_cur;
                g.task_b = st.task_b; g.task_e = st.task_e; g.task_s = st.task_s; g.gran = st.gran;
                g.n_slots = st.n_slots; g.slot_warps = st.slot_warps; g.slot_sram = st.slot_sram;
                g.op_begin = (int)ops.size();
                g.signal_begin = -1;
                const Json &ti = task_infos.at((size_t)st.task_info);
                const Json &ops_json = ti.at("Ops");
                if (ops_json.size() > 16)
                    ARK_ERR(UnsupportedError, "a task may hold at most 16 ops, got ", ops_json.size());
                // the ops of one task run for the same task ids: their task counts must agree
                // (an op with no tasks, such as Noop, aside)
                int64_t common_tasks = -1;
                for (const auto &oj : ops_json.elements()) {
                    int64_t nt = oj.at("Config").at("NumTasks").as_int();
                    if (nt == 0) continue;
                    // a matmul that splits K runs SplitK tasks per tile; its followers one per tile
                    if (oj.at("Config").contains("SplitK")) nt /= std::max<int64_t>(1, oj.at("Config").at("SplitK").as_int());
                    if (common_tasks < 0) common_tasks = nt;
                    if (nt != common_tasks)
                        ARK_ERR(PlanError, "the ops fused into task ", st.task_info, " have different NumTasks (", common_tasks,
                                " and ", nt, "): op ", oj.at("Type").as_string(), " cannot ride on the first op's tiles");
                }
                for (const auto &oj : ops_json.elements())
                    ops.push_back(lower_op(oj, L, st.slot_warps, block_warps, st.n_slots, st.slot_sram));
                g.op_count = (int)ops.size() - g.op_begin;
                // the loop kernel runs one task loop per kind of the first op; behind a matmul
                // come elementwise ops only, behind a small op any small op
                if (g.op_count > 1) {
                    const int k0 = ops[(size_t)g.op_begin].kind;
                    if (k0 == DEV_GEMV || k0 == DEV_ATTN)
                        ARK_ERR(UnsupportedError, "task ", st.task_info, ": no op can be fused behind a skinny matmul or "
                                "an attention op");
                    for (int o = g.op_begin + 1; o < (int)ops.size(); ++o) {
                        const int ko = ops[(size_t)o].kind;
                        if (ko == DEV_GEMM || ko == DEV_GEMV || ko == DEV_ATTN)
                            ARK_ERR(UnsupportedError, "task ", st.task_info, ": a matmul or attention op must be the "
                                    "first op of its task");
                        if (k0 == DEV_GEMM && ko != DEV_EWISE)
                            ARK_ERR(UnsupportedError, "task ", st.task_info, ": only elementwise ops can be fused "
                                    "behind a matmul");
                    }
                }
                group_fused.push_back(g.op_count == 2 && fold_into_store(ops[(size_t)g.op_begin],
                                                                          ops[(size_t)g.op_begin + 1]) ? 1 : 0);
                int group_fam = 0;
                // (an elementwise op folded into its matmul's store needs no body of its own)
                for (int o = g.op_begin; o < (group_fused.back() ? g.op_begin + 1 : (int)ops.size()); ++o)
                    group_fam |= ops[o].kind == DEV_ROW ? (ops[o].row.red_len > 0 ? FAM_EXT : FAM_ROW)
                               : ops[o].kind == DEV_GEMM
                                   ? ((ops[o].gemm.dtype == 0 || ops[o].gemm.trans_a) ? FAM_EXT
                                      : ops[o].gemm.split_k == 2 ? (FAM_GEMM | FAM_SPLITK) : FAM_GEMM)
                               : ops[o].kind == DEV_EWISE ? FAM_EWISE
                               : ops[o].kind == DEV_GEMV ? FAM_GEMV
                               : ops[o].kind == DEV_ATTN ? FAM_ATTN
                               : ops[o].kind == DEV_EMBED ? FAM_EXT : 0;
                families |= group_fam;
                h_group_fam.push_back(group_fam);
                g.trace_offset = (int)trace_len;
                trace_len += (size_t)std::max(0, (st.task_e - st.task_b + st.task_s - 1) / st.task_s);
                max_slot_lds = std::max(max_slot_lds, st.n_slots * st.slot_sram);
                ds.kind = STEP_TASKS;
                ds.index = (int)h_groups.size();
                h_groups.push_back(g);
                group_sched_step.push_back((int)si);
            }
            dev_step_of[si] = (int)steps.size();
            steps.push_back(ds);
        }
        num_dev_steps = (int)steps.size();

        // ---- row ops whose input another op reads afterwards: fetch it through the caches ---------
        // (RowOpDesc::in_read_again; ARKMI_ROW_CACHED_INPUT=0: every row op streams its input)
        {
            const char *env = getenv("ARKMI_ROW_CACHED_INPUT");
            const bool on = !(env && atoi(env) == 0);
            auto input_of = [&](const Json &op_json, Access &out) {
                std::vector<Access> v;
                const Json &reads = op_json.at("ReadTensors");
                if (reads.size() == 0) return false;
                add_access(v, reads.at((size_t)0), false, op_json.at("Type").as_string(), false);
                if (v.empty()) return false;
                out = v[0];
                return true;
            };
            auto same_bytes = [](const Access &x, const Access &y) {
                return x.buffer == y.buffer && x.begin < y.end && y.begin < x.end;
            };
            for (size_t si = 0; on && si < sched.steps.size(); ++si) {
                if (sched.steps[si].is_barrier || dev_step_of[si] < 0) continue;
                const DevTaskGroup &g = h_groups[(size_t)steps[(size_t)dev_step_of[si]].index];
                const Json &task_ops = task_infos.at((size_t)sched.steps[si].task_info).at("Ops");
                for (int o = 0; o < g.op_count; ++o) {
                    DevOp &op = ops[(size_t)(g.op_begin + o)];
                    Access in;
                    if (op.kind != DEV_ROW || op.row.red_len > 0 || !input_of(task_ops.at((size_t)o), in)) continue;
                    // the accesses that follow this op: the later ops of its task, then the later steps
                    std::vector<Access> later;
                    for (size_t o2 = (size_t)o + 1; o2 < task_ops.size(); ++o2) {
                        Json one = Json::object();
                        Json arr = Json::array();
                        arr.push_back(task_ops.at(o2));
                        one["Ops"] = arr;
                        auto a = accesses_of(one);
                        later.insert(later.end(), a.begin(), a.end());
                    }
                    for (size_t sj = si + 1; sj < sched.steps.size(); ++sj)
                        if (!sched.steps[sj].is_barrier) {
                            auto a = step_accesses(sj);
                            later.insert(later.end(), a.begin(), a.end());
                        }
                    for (const Access &y : later) {
                        if (!same_bytes(in, y)) continue;
                        op.row.in_read_again = y.write ? 0 : 1;  // (overwritten first: nobody reads these values again)
                        break;
                    }
                }
            }
        }

        // ---- dependency counters in place of full-grid barriers --------------------------------
        // Task groups since the last barrier that stays form a window.  A full-grid barrier inside
        // the window is replaced by a workgroup sync when every hazard between a group behind it
        // and a group of the window ahead of it is either local to a workgroup (as above) or a
        // read of rows whose writers signal counters the reader waits on.  A hazard that is
        // neither keeps the last barrier ahead of the reader.  ARKMI_DEP_COUNTERS=1 turns this on.
        barriers_counted = 0;
        // a hazard across a candidate barrier was accepted as workgroup-local: task t of both
        // groups must then keep computing tile t (no permuted tile order below)
        bool counted_relies_on_local = false;
        std::vector<DevWait> h_waits;
        std::vector<int32_t> h_spans, h_signal;
        size_t n_counters = 0;
        {
            // Off unless asked for: on the Llama layer the counters cost what the barriers cost
            // (each signal is an L2 write-back, the wait for the slowest producer stays, and the
            // iteration boundary needs its barrier back), measured 1169 against 1144 us.
            const char *dep_env = getenv("ARKMI_DEP_COUNTERS");
            bool use_deps = elide && (force_deps >= 0 ? force_deps != 0 : (dep_env && atoi(dep_env) != 0));
            for (const auto &st : sched.steps)
                if (st.is_barrier && !(st.b == 0 && st.e >= grid)) use_deps = false;
            std::vector<DepGroup> dg;
            std::vector<int> dg_of_step(sched.steps.size(), -1);
            if (use_deps) {
                int segment = 0;
                for (size_t si = 0; si < sched.steps.size(); ++si) {
                    if (sched.steps[si].is_barrier) {
                        ++segment;
                        continue;
                    }
                    DepGroup d;
                    d.sched_step = (int)si;
                    d.segment = segment;
                    d.group = steps[(size_t)dev_step_of[si]].index;
                    const DevTaskGroup &g = h_groups[(size_t)d.group];
                    d.n_tasks = std::max(0, (g.task_e - g.task_b + g.task_s - 1) / g.task_s);
                    d.n_signal = d.n_tasks;
                    const DevOp &first = ops[(size_t)g.op_begin];
                    if (first.kind == DEV_GEMM && first.gemm.split_k == 2)
                        d.n_signal = first.gemm.tiles_m * first.gemm.tiles_n * first.gemm.batch_total;
                    d.whole_block = g.n_slots == 1 && g.slot_warps == block_warps && g.task_b == 0 && g.task_s == 1;
                    d.acc = step_accesses(si);
                    for (int o = g.op_begin; o < g.op_begin + g.op_count; ++o) {
                        auto r = row_accesses(ops[(size_t)o], g.slot_warps);
                        d.rows.insert(d.rows.end(), r.begin(), r.end());
                    }
                    dg_of_step[si] = (int)dg.size();
                    dg.push_back(std::move(d));
                }
                std::vector<int> window;         // groups since the last barrier that stays
                std::vector<size_t> candidates;  // full-grid barriers inside the window
                std::vector<size_t> dropped;
                for (size_t si = 0; si < sched.steps.size(); ++si) {
                    if (sched.steps[si].is_barrier) {
                        if (dev_step_of[si] >= 0 && steps[(size_t)dev_step_of[si]].kind == STEP_BARRIER)
                            candidates.push_back(si);
                        continue;
                    }
                    const int yi = dg_of_step[si];
                    int uncovered_after = -1;
                    for (int xi : window) {
                        if (dg[(size_t)xi].segment == dg[(size_t)yi].segment) continue;
                        // (copies: cover_with_counters grows dg[yi].waits, not the access lists)
                        for (size_t ia = 0; ia < dg[(size_t)xi].acc.size(); ++ia)
                            for (size_t ib = 0; ib < dg[(size_t)yi].acc.size(); ++ib) {
                                const Access &ax = dg[(size_t)xi].acc[ia], &ay = dg[(size_t)yi].acc[ib];
                                if (!overlap(ax, ay)) continue;
                                if (local_pair(ax, ay)) {
                                    counted_relies_on_local = true;
                                    continue;
                                }
                                if (cover_with_counters(dg, xi, ax, yi, ay, arena, buffer_offset)) continue;
                                if (getenv("ARKMI_DEBUG_BARRIERS"))
                                    fprintf(stderr, "no counters for steps %d -> %d: views '%s' (%s) vs '%s' (%s)\n",
                                            ax.step, ay.step, ax.view.c_str(), ax.write ? "write" : "read",
                                            ay.view.c_str(), ay.write ? "write" : "read");
                                uncovered_after = std::max(uncovered_after, dg[(size_t)xi].sched_step);
                            }
                    }
                    if (uncovered_after >= 0) {
                        // the last barrier ahead of this group stays; what lies between it and the
                        // group is local to the group's workgroups (judged above), so it waits
                        // for nothing
                        if (candidates.empty() || (int)candidates.back() < uncovered_after)
                            ARK_ERR(InternalError, "no barrier left between steps ", uncovered_after, " and ", si);
                        const size_t keep = candidates.back();
                        candidates.pop_back();
                        dropped.insert(dropped.end(), candidates.begin(), candidates.end());
                        candidates.clear();
                        dg[(size_t)yi].waits.clear();
                        std::vector<int> rest;
                        for (int xi : window)
                            if ((size_t)dg[(size_t)xi].sched_step > keep) {
                                rest.push_back(xi);
                                // the barrier now orders these groups after everything ahead of it
                                auto &ws = dg[(size_t)xi].waits;
                                ws.erase(std::remove_if(ws.begin(), ws.end(),
                                                        [&](const DepGroup::Wait &w) {
                                                            return (size_t)dg[(size_t)w.producer].sched_step < keep;
                                                        }),
                                         ws.end());
                            }
                        window.swap(rest);
                    }
                    window.push_back(yi);
                }
                dropped.insert(dropped.end(), candidates.begin(), candidates.end());
                // a barrier behind the last group orders nothing inside the body: it is not counted
                for (size_t si : dropped) {
                    steps[(size_t)dev_step_of[si]].kind = STEP_LOCAL_SYNC;
                    ++barriers_counted;
                }
            }
            if (barriers_counted > 0) {
                for (auto &y : dg)
                    for (auto &w : y.waits) {
                        DepGroup &x = dg[(size_t)w.producer];
                        if (x.counter_base < 0) {
                            x.counter_base = (int)n_counters;
                            n_counters += (size_t)x.n_blocks;
                        }
                    }
                for (auto &d : dg) {
                    DevTaskGroup &g = h_groups[(size_t)d.group];
                    if (d.counter_base >= 0) {
                        g.signal_begin = (int)h_signal.size();
                        g.signal_base = d.counter_base;
                        h_signal.insert(h_signal.end(), d.signal_map.begin(), d.signal_map.end());
                    }
                    if (!d.waits.empty()) {
                        g.n_waits = (int)d.waits.size();
                        g.wait_begin = (int)h_waits.size();
                        g.span_begin = (int)h_spans.size();
                        for (const auto &w : d.waits)
                            h_waits.push_back(DevWait{dg[(size_t)w.producer].counter_base, dg[(size_t)w.producer].per_block});
                        for (int t = 0; t < d.n_tasks; ++t)
                            for (const auto &w : d.waits) {
                                h_spans.push_back(w.span[(size_t)t].first);
                                h_spans.push_back(w.span[(size_t)t].second);
                            }
                    }
                }
            }
        }

        // The boundary between two iterations of one command is one more barrier
        // candidate: what runs after the body's last full barrier meets what runs
        // before its first one (the whole body meets itself when it has none, and
        // workgroups may then drift several iterations apart, which the same
        // pairwise comparison covers).  A task group meets itself on the same
        // workgroups, task by task, so its own tensors are a local matter unless an
        // op keeps partial results in scratch memory that other workgroups finish.
        iteration_sync = 2;
        iteration_local_across_groups = false;
        if (elide) {
            bool whole_grid_only = true;
            int first_full = -1, last_full = -1;
            for (size_t si = 0; si < sched.steps.size(); ++si) {
                const auto &st = sched.steps[si];
                if (!st.is_barrier) continue;
                if (!(st.b == 0 && st.e >= grid)) whole_grid_only = false;
                if (dev_step_of[si] >= 0 && steps[(size_t)dev_step_of[si]].kind == STEP_BARRIER) {
                    if (first_full < 0) first_full = (int)si;
                    last_full = (int)si;
                }
            }
            if (whole_grid_only) {
                auto has_scratch = [&](int sj) {
                    const DevStep &dst = steps[(size_t)dev_step_of[(size_t)sj]];
                    return (h_group_fam[(size_t)dst.index] & (FAM_GEMV | FAM_SPLITK)) != 0;
                };
                std::vector<Access> tail, head;
                for (size_t sj = (size_t)(last_full + 1); sj < sched.steps.size(); ++sj)
                    if (!sched.steps[sj].is_barrier) {
                        auto a = step_accesses(sj);
                        tail.insert(tail.end(), a.begin(), a.end());
                    }
                const size_t head_end = first_full < 0 ? sched.steps.size() : (size_t)first_full;
                for (size_t sj = 0; sj < head_end; ++sj)
                    if (!sched.steps[sj].is_barrier) {
                        auto a = step_accesses(sj);
                        head.insert(head.end(), a.begin(), a.end());
                    }
                bool any = false, all_local = true;
                for (const auto &x : tail)
                    for (const auto &y : head) {
                        if (!overlap(x, y)) continue;
                        any = true;
                        bool local;
                        if (has_scratch(x.step) || has_scratch(y.step))
                            local = false;
                        else if (x.step == y.step)
                            local = !x.panel_read && !y.panel_read && x.view == y.view && x.begin == y.begin;
                        else {
                            local = local_pair(x, y);
                            if (local) iteration_local_across_groups = true;
                        }
                        if (!local) all_local = false;
                    }
                iteration_sync = !any ? 0 : all_local ? 1 : 2;
            }
            // (Without the barrier a GEMM body gains 6 % and the row-op workload 3 %: workgroups
            // that finish an iteration early start the next one instead of waiting.)
            // ARKMI_ITERATION_BARRIER=1 always keeps the barrier.
            const char *it_env = getenv("ARKMI_ITERATION_BARRIER");
            if (it_env && atoi(it_env) != 0) iteration_sync = 2;
        }
        // the counters count per iteration, and a reader relies on the caches having been
        // invalidated since the previous one
        if (barriers_counted > 0) iteration_sync = 2;

        // ---- matmul tiles in an XCD-aware order ---------------------------------------------------
        // Workgroups go to the eight XCDs round robin, and each XCD has an L2 of its own: with the
        // tiles in row-major task order, the tiles an XCD works on at a time lie strewn over the
        // output, and its L2 fetches nearly all of A (C1: 345 MB fetched for 67 MB of operands).
        // Where task t runs on workgroup t mod R, the matmul's tile index is permuted so that they
        // form a compact block (gemm_tile).  The tasks stay on their workgroups; the tile a task
        // computes changes, and the ops fused behind the matmul follow it.  ARKMI_GEMM_XCD=0: off.
        gemm_xcd_ordered = 0;
        attn_xcd_ordered = 0;
        {
            const char *xe = getenv("ARKMI_GEMM_XCD");
            // (a workgroup-local sync in place of a barrier rests on task t of both ops running on
            // the same workgroup for the same tile: plans that have one, inside the body or between
            // two groups across the iteration boundary, keep the plain order; a group that meets
            // only itself across iterations still computes the same tile on the same workgroup)
            const bool on = !(xe && atoi(xe) == 0) && !trace_enabled && barriers_local == 0 &&
                            !(barriers_counted > 0 && counted_relies_on_local) &&
                            !(iteration_sync == 1 && iteration_local_across_groups);
            // (the attention op likewise: the query blocks an XCD works on at a time then belong to
            // the same few heads)
            for (DevTaskGroup &g : h_groups) {
                DevOp &op0 = ops[(size_t)g.op_begin];
                if (!on || op0.kind != DEV_ATTN || g.n_waits > 0 || g.signal_begin >= 0) continue;
                // (task t on the (t mod n_procs)-th processor of a range that starts at a multiple of 8)
                if (g.proc_b % 8 != 0 || g.proc_s != 1 || g.proc_cur != g.proc_b || g.task_b != 0 || g.task_s != 1 ||
                    g.gran != 1)
                    continue;
                AttnDesc &d = op0.attn;
                const int n_procs = g.proc_e - g.proc_b;
                const int total = d.batch * d.heads * d.q_blocks, round = std::min(total, n_procs);
                if (g.task_e != total || n_procs % 8 != 0 || round % 8 != 0 || round < 16) continue;
                d.xcd_round = round;
                ++attn_xcd_ordered;
            }
            for (DevTaskGroup &g : h_groups) {
                DevOp &op0 = ops[(size_t)g.op_begin];
                if (!on || op0.kind != DEV_GEMM || op0.gemm.dtype == 0) continue;
                GemmDesc &d = op0.gemm;
                if (d.batch_total != 1 || g.n_waits > 0 || g.signal_begin >= 0) continue;  // (waits go by task index)
                if (g.proc_b % 8 != 0 || g.proc_s != 1 || g.proc_cur != g.proc_b || g.task_b != 0 || g.task_s != 1 ||
                    g.gran != 1)
                    continue;
                const int n_procs = g.proc_e - g.proc_b, tiles = d.tiles_m * d.tiles_n;
                const int round = std::min(tiles, n_procs);  // tiles in flight at once
                if (n_procs % 8 != 0 || tiles % 8 != 0 || round % 8 != 0 || round < 16) continue;
                if (g.task_e != tiles * (d.split_k == 2 ? 2 : 1)) continue;
                const int per = round / 8, cols_cost = op0.gemm_tile_n * (d.b2 ? 2 : 1);
                int best = 0;
                long best_cost = 0;
                for (int bm = 1; bm <= per; bm *= 2) {
                    if (d.tiles_m % bm != 0 || per % bm != 0) continue;
                    const long cost = (long)bm * op0.gemm_tile_m + (long)(per / bm) * cols_cost;
                    if (best == 0 || cost < best_cost) { best = bm; best_cost = cost; }
                }
                if (best == 0) continue;
                d.xcd_round = round;
                d.xcd_band = best;
                ++gemm_xcd_ordered;
            }
        }

        // ---- skinny matmuls: stretches, who streams which, runs of matmuls as one stream ----------
        // A workgroup streams stretches of consecutive units of one column block and folds at the
        // end of each (across the waves, then with the block's other stretches through partial
        // tiles in the order of the parts, so the result does not depend on who streamed what).
        // The one-op kernels run the plan's tasks on the plan's workgroups: a task's contiguous
        // range of units, cut at the column-block boundaries.  The loop kernel
        //  * runs matmuls that follow one another with no barrier or sync in between as one
        //    sequence: the next one's first loads are in flight while the current one folds
        //    (ARKMI_GEMV_CHAIN=0: every matmul by itself);
        //  * lets the workgroups claim stretches as they get free: a workgroup's share of the HBM bandwidth varies by tens of percent
        //    over a step, and with fixed shares the slowest one sets the time.  The run is then
        //    cut into long stretches first and short ones at the end (gemv_coarse_share)
        //    (ARKMI_GEMV_CLAIM=0: the tasks' fixed shares).
        gemv_chains = 0;
        gemv_claimed = 0;
        barriers_widened = 0;
        h_gemv_seq.clear();
        {
            const char *chain_env = getenv("ARKMI_GEMV_CHAIN"), *claim_env = getenv("ARKMI_GEMV_CLAIM");
            const bool chain_on = !(chain_env && atoi(chain_env) == 0) && !trace_enabled;
            const bool claim_on = !(claim_env && atoi(claim_env) == 0) && !trace_enabled;
            auto is_gemv = [&](const DevTaskGroup &g) {
                return g.op_count == 1 && ops[(size_t)g.op_begin].kind == DEV_GEMV;
            };
            auto chainable = [&](const DevStep &st) {
                if (st.kind != STEP_TASKS) return false;
                const DevTaskGroup &g = h_groups[(size_t)st.index];
                return is_gemv(g) && g.n_waits == 0 && g.signal_begin < 0;
            };
            // fixed shares: the tasks of the groups [first, first + n) on the plan's workgroups,
            // per workgroup in group order
            auto lay_out = [&](size_t first, size_t n, int32_t &begin, int32_t &stride) {
                std::vector<std::vector<GemvSeqEntry>> rows((size_t)grid);
                for (size_t gi = first; gi < first + n; ++gi) {
                    const DevTaskGroup &g = h_groups[gi];
                    const GemvDesc &d = ops[(size_t)g.op_begin].gemv;
                    const auto &st = sched.steps[(size_t)group_sched_step[gi]];
                    const int64_t U = (int64_t)d.n_blocks * d.k_units, T = d.num_tasks;
                    for (int block = 0; block < grid; ++block) {
                        int order = 0;
                        for (int64_t id : schedule_tasks_of(sched, st, block, 0)) {
                            const int this_order = order++;
                            if (id < 0 || id >= T) continue;  // (a task beyond the partition has no units)
                            const int64_t u1 = gemv_task_begin(id + 1, U, T);
                            for (int64_t u = gemv_task_begin(id, U, T); u < u1;) {
                                const int64_t nb = u / d.k_units, ku = u % d.k_units;
                                const int64_t t_first = gemv_task_of(nb * d.k_units, U, T);
                                const int64_t t_last = gemv_task_of((nb + 1) * d.k_units - 1, U, T);
                                GemvSeqEntry e{};
                                e.op = g.op_begin;
                                e.nb = (int32_t)nb;
                                e.ku = (int32_t)ku;
                                e.units = (int32_t)std::min<int64_t>(u1 - u, d.k_units - ku);
                                e.part = (int32_t)(id - t_first);
                                e.parts = (int32_t)(t_last - t_first + 1);
                                e.trace_index = trace_enabled ? g.trace_offset + (int)((id - g.task_b) / g.task_s) : -1;
                                e.order = this_order;
                                rows[(size_t)block].push_back(e);
                                u += e.units;
                            }
                        }
                    }
                }
                size_t longest = 0;
                for (const auto &r : rows) longest = std::max(longest, r.size());
                begin = (int32_t)h_gemv_seq.size();
                stride = (int32_t)longest + 1;
                GemvSeqEntry end{};
                end.op = -1;
                for (const auto &r : rows) {
                    h_gemv_seq.insert(h_gemv_seq.end(), r.begin(), r.end());
                    h_gemv_seq.insert(h_gemv_seq.end(), (size_t)stride - r.size(), end);
                }
            };
            // claimed at run time: possible when every column block has the 3 units a stretch needs
            // (the claim protocol's look-ahead).  Every workgroup of the grid then streams for the
            // matmul, whatever processors the plan names for it, and a barrier over part of the grid
            // would not wait for all of them: a plan that has such a matmul gets its remaining
            // barriers over part of the grid widened to the whole grid (a stronger order, reached
            // by every workgroup in the same place).
            bool any_claimable = false;
            for (const DevTaskGroup &g : h_groups)
                if (claim_on && is_gemv(g) && g.n_waits == 0 && g.signal_begin < 0 &&
                    ops[(size_t)g.op_begin].gemv.k_units >= kGemvMinStretch)
                    any_claimable = true;
            if (any_claimable)
                for (DevStep &st : steps)
                    if (st.kind == STEP_BARRIER && st.count != grid) {
                        st.b = 0; st.e = grid; st.s = 1; st.count = grid;
                        ++barriers_widened;
                    }
            auto claimable = [&](size_t first, size_t n) {
                if (!claim_on) return false;
                for (size_t gi = first; gi < first + n; ++gi)
                    if (ops[(size_t)h_groups[gi].op_begin].gemv.k_units < kGemvMinStretch) return false;
                return true;
            };
            auto lay_out_shared = [&](size_t first, size_t n, DevTaskGroup &head) {
                int64_t total = 0, done = 0;
                for (size_t gi = first; gi < first + n; ++gi) {
                    const GemvDesc &d = ops[(size_t)h_groups[gi].op_begin].gemv;
                    total += (int64_t)d.n_blocks * d.k_units;
                }
                const int fine = gemv_fine_units();
                const double share = gemv_coarse_share();
                const int coarse = std::max(fine, (int)std::llround(share * (double)total / (2.0 * grid)));
                head.run_begin = (int32_t)h_gemv_seq.size();
                for (size_t gi = first; gi < first + n; ++gi) {
                    const DevTaskGroup &g = h_groups[gi];
                    const GemvDesc &d = ops[(size_t)g.op_begin].gemv;
                    for (int nb = 0; nb < d.n_blocks; ++nb, done += d.k_units) {
                        const int want = (double)done < share * (double)total ? coarse : fine;
                        const int parts = std::max(1, std::min((d.k_units + want / 2) / want, d.k_units / kGemvMinStretch));
                        for (int p = 0; p < parts; ++p) {
                            GemvSeqEntry e{};
                            e.op = g.op_begin;
                            e.nb = nb;
                            e.ku = (int32_t)((int64_t)p * d.k_units / parts);
                            e.units = (int32_t)((int64_t)(p + 1) * d.k_units / parts) - e.ku;
                            e.part = p;
                            e.parts = parts;
                            e.trace_index = -1;
                            h_gemv_seq.push_back(e);
                        }
                    }
                }
                head.run_stride = (int32_t)h_gemv_seq.size() - head.run_begin;
                head.claim = gemv_claimed++;
            };
            for (size_t gi = 0; gi < h_groups.size(); ++gi) {
                DevTaskGroup &g = h_groups[gi];
                g.claim = -1;
                if (!is_gemv(g)) continue;
                lay_out(gi, 1, g.seq_begin, g.seq_stride);
                g.run_begin = g.seq_begin;
                g.run_stride = g.seq_stride;
            }
            std::vector<char> in_run(h_groups.size(), 0);
            for (size_t i = 0; chain_on && i < steps.size();) {
                size_t j = i;
                if (chainable(steps[i])) {
                    const int dtype = ops[(size_t)h_groups[(size_t)steps[i].index].op_begin].gemv.dtype;
                    for (j = i + 1; j < steps.size() && chainable(steps[j]) &&
                                    steps[j].index == steps[j - 1].index + 1 &&
                                    ops[(size_t)h_groups[(size_t)steps[j].index].op_begin].gemv.dtype == dtype;
                         ++j) {
                    }
                    if (j - i > 1) {
                        const size_t first = (size_t)steps[i].index, n = j - i;
                        DevTaskGroup &head = h_groups[first];
                        head.chain = (int)n;
                        for (size_t m = 1; m < n; ++m) h_groups[first + m].chain = -1;
                        for (size_t m = 0; m < n; ++m) in_run[first + m] = 1;
                        if (claimable(first, n)) lay_out_shared(first, n, head);
                        else lay_out(first, n, head.run_begin, head.run_stride);
                        ++gemv_chains;
                    }
                }
                i = std::max(j, i + 1);
            }
            for (size_t gi = 0; gi < h_groups.size(); ++gi)
                if (is_gemv(h_groups[gi]) && !in_run[gi] && claimable(gi, 1)) lay_out_shared(gi, 1, h_groups[gi]);
        }
        // claimed stretches are counted per iteration: iterations must not overlap
        if (gemv_claimed > 0) iteration_sync = 2;
        // ---- a row op touches the first rows of the row op that follows it ------------------------
        // A task's first loads overlap nothing: a workgroup that goes from one row op to the next
        // (no grid barrier between them) starts the next one with an empty pipeline.  Where the
        // next task step is a row op with the same dealing of rows to waves, every wave touches
        // the lines of its first row there while it finishes its last row here
        // (RowOpDesc::pf_*; a hint only: the values are discarded).  ARKMI_ROW_PREFETCH=0: off.
        {
            const char *env = getenv("ARKMI_ROW_PREFETCH");
            const bool on = !(env && atoi(env) == 0);
            const int n = (int)steps.size();
            auto row_op_of = [&](const DevStep &st) -> DevOp * {
                if (st.kind != STEP_TASKS) return nullptr;
                DevOp &op = ops[(size_t)h_groups[(size_t)st.index].op_begin];
                return (op.kind == DEV_ROW && op.row.red_len == 0) ? &op : nullptr;
            };
            for (int i = 0; on && i < n; ++i) {
                DevOp *cur = row_op_of(steps[(size_t)i]);
                if (!cur || h_groups[(size_t)steps[(size_t)i].index].op_count != 1) continue;
                int j = i;
                bool found = false;
                for (int hop = 0; hop < n; ++hop) {
                    if (++j == n) {
                        if (iteration_sync == 2) break;  // a grid barrier separates the iterations
                        j = 0;
                    }
                    if (steps[(size_t)j].kind == STEP_BARRIER) break;
                    if (steps[(size_t)j].kind == STEP_TASKS) { found = true; break; }
                }
                if (!found) continue;
                DevOp *nx = row_op_of(steps[(size_t)j]);
                if (!nx) continue;
                const DevTaskGroup &a = h_groups[(size_t)steps[(size_t)i].index], &b = h_groups[(size_t)steps[(size_t)j].index];
                const RowOpDesc &r = nx->row;
                const bool same_deal = a.proc_b == b.proc_b && a.proc_e == b.proc_e && a.proc_s == b.proc_s &&
                                       a.proc_cur == b.proc_cur && a.task_b == b.task_b && a.task_e == b.task_e &&
                                       a.task_s == b.task_s && a.gran == b.gran && a.n_slots == b.n_slots &&
                                       a.slot_warps == b.slot_warps && cur->row.rows == r.rows &&
                                       std::max(1, cur->row.rows_per_wave) == std::max(1, r.rows_per_wave);
                // rows of the next op's input one stride apart from first to last
                const int64_t n_outer = r.rows / std::max<int64_t>(1, (int64_t)r.dim_c * r.dim_h);
                const bool uniform = (r.dim_c == 1 || r.in_s[1] == (int64_t)r.dim_h * r.in_s[2]) &&
                                     (n_outer <= 1 || r.in_s[0] == (int64_t)r.dim_c * r.dim_h * r.in_s[2]);
                const int64_t elem = r.dtype == 0 ? 4 : 2;
                const int64_t len = (int64_t)r.cols * elem;
                if (!same_deal || !uniform || r.in_s[2] <= 0 || len > 2 * 64 * 128) continue;
                // the same rows this op has just fetched through the caches for that very reader
                if (r.in == cur->row.in && cur->row.in_read_again) continue;
                // a reader that fetches through the caches for the ops behind it: measured 1.3 % slower
                // with its first rows touched (three row ops over each of four X: 0.818 against 0.829
                // of 8 TB/s), where streaming readers gain 3-6 %
                if (r.in_read_again) continue;
                cur->row.pf_base = r.in;
                cur->row.pf_row_bytes = r.in_s[2] * elem;
                cur->row.pf_len = (int)len;
            }
        }
        lds_bytes = loop_kernel_lds_reserved() + max_slot_lds;
        if (dry) {
            (void)loop_kernel_select(families, &kernel_families);
            dry_steps = steps;
            dry_ops = ops;
            dry_waits = h_waits;
            dry_spans = h_spans;
            dry_signal = h_signal;
            dry_counters = n_counters;
            return;
        }
        const auto &facts = device_facts(device);
        if (lds_bytes > facts.lds_bytes)
            ARK_ERR(PlanError, "plan needs ", lds_bytes, " bytes of LDS per workgroup; the CU has ",
                    facts.lds_bytes);
        // ARKMI_LOOP_FAMILIES adds op families to the ones the plan needs (a larger kernel
        // variant than necessary: for measuring what a variant costs the bodies it holds)
        const char *fam_env = getenv("ARKMI_LOOP_FAMILIES");
        kernel = loop_kernel_select(families | (fam_env ? (atoi(fam_env) & FAM_ALL) : 0), &kernel_families);
        loop_kernel_prepare(kernel, lds_bytes);
        // every workgroup must be resident at once or the grid barriers cannot complete
        const int per_cu = loop_kernel_max_blocks_per_cu(kernel, threads, lds_bytes);
        if (per_cu < 1 || grid > per_cu * facts.num_cu)
            ARK_ERR(PlanError, "NumProcessors ", grid, " cannot be co-resident: ", per_cu,
                    " workgroup(s) per CU x ", facts.num_cu, " CUs");

        auto upload = [&](const void *src, size_t bytes, void **dst) {
            ARKMI_HIP(hipMalloc(dst, std::max<size_t>(bytes, 16)));
            if (bytes) ARKMI_HIP(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
        };
        upload(ops.data(), ops.size() * sizeof(DevOp), (void **)&d_ops);
        {
            // a follower folded into its matmul's store does not run as an op of its own
            std::vector<DevTaskGroup> dev_groups = h_groups;
            for (size_t gi = 0; gi < dev_groups.size(); ++gi)
                if (group_fused[gi]) dev_groups[gi].op_count = 1;
            upload(dev_groups.data(), dev_groups.size() * sizeof(DevTaskGroup), (void **)&d_groups);
        }
        upload(steps.data(), steps.size() * sizeof(DevStep), (void **)&d_steps);
        if (trace_enabled && trace_len) {
            ARKMI_HIP(hipMalloc((void **)&d_trace, trace_len * sizeof(TraceRecord)));
            ARKMI_HIP(hipMemset(d_trace, 0xff, trace_len * sizeof(TraceRecord)));
        }
        if (barriers_counted > 0) {
            upload(h_waits.data(), h_waits.size() * sizeof(DevWait), (void **)&d_waits);
            upload(h_spans.data(), h_spans.size() * sizeof(int32_t), (void **)&d_spans);
            upload(h_signal.data(), h_signal.size() * sizeof(int32_t), (void **)&d_signal);
            dep_counter_bytes = n_counters * kDepStride * sizeof(unsigned int);
            ARKMI_HIP(hipMalloc((void **)&d_dep_counters, dep_counter_bytes));
            ARKMI_HIP(hipMemset(d_dep_counters, 0, dep_counter_bytes));
        }
        if (!h_gemv_seq.empty())
            upload(h_gemv_seq.data(), h_gemv_seq.size() * sizeof(GemvSeqEntry), (void **)&d_gemv_seq);
        prog.gemv_seq = d_gemv_seq;
        if (gemv_claimed > 0) {
            gemv_claim_bytes = (size_t)gemv_claimed * 2 * kDepStride * sizeof(unsigned int);
            ARKMI_HIP(hipMalloc((void **)&d_gemv_claims, gemv_claim_bytes));
            ARKMI_HIP(hipMemset(d_gemv_claims, 0, gemv_claim_bytes));
        }
        prog.gemv_claims = d_gemv_claims;
        prog.waits = d_waits;
        prog.wait_spans = d_spans;
        prog.signal_map = d_signal;
        prog.dep_counters = d_dep_counters;
        prog.steps = d_steps;
        prog.groups = d_groups;
        prog.ops = d_ops;
        prog.trace = d_trace;
        if (trace_enabled) {
            const size_t n = (steps.size() + 1) * (size_t)grid * sizeof(unsigned long long);
            ARKMI_HIP(hipMalloc((void **)&d_clock, n));
            ARKMI_HIP(hipMemset(d_clock, 0, n));
        }
        prog.step_clock = d_clock;
        prog.num_steps = (int)steps.size();
        prog.num_blocks = grid;
        prog.iter_sync = iteration_sync;

        (void)hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, device);
        if (wall_khz <= 0) wall_khz = 100000;
        auto env_ms = [](const char *n, long dflt) {
            const char *v = getenv(n);
            return v ? atol(v) : dflt;
        };
        idle_ticks = (uint64_t)env_ms("ARKMI_IDLE_EXIT_MS", 2000) * (uint64_t)wall_khz;
        wait_ticks = (uint64_t)env_ms("ARKMI_BARRIER_LIMIT_MS", 20000) * (uint64_t)wall_khz;
        compiled = true;
    }

    bool kernel_resident() const { return launched && hipEventQuery(ev_end) == hipErrorNotReady; }

    void start_kernel() {
        // control block and mailbox start from zero on every kernel launch
        ARKMI_HIP(hipMemsetAsync(ctl, 0, sizeof(LoopControl), stream));
        if (d_dep_counters) ARKMI_HIP(hipMemsetAsync(d_dep_counters, 0, dep_counter_bytes, stream));
        if (d_gemv_claims) ARKMI_HIP(hipMemsetAsync(d_gemv_claims, 0, gemv_claim_bytes, stream));
        mb->status = MB_OK;
        mb->alive = 1;
        loop_kernel_launch(kernel, prog, ctl, mb_dev, grid, threads, lds_bytes, 0, idle_ticks, wait_ticks, stream);
        ARKMI_HIP(hipEventRecord(ev_end, stream));
    }

    void launch() {
        if (destroyed) ARK_ERR(InvalidUsageError, "executor is destroyed");
        if (!compiled) ARK_ERR(InvalidUsageError, "Need to compile first before initialization.");
        if (launched) {
            ARK_LOG(WARN, "Ignore launching twice.");
            return;
        }
        set_device();
        ARKMI_HIP(hipEventRecord(ev_begin, stream));
        mb->cmd = 0;
        mb->done = 0;
        launched = true;
        if (loop_mode) start_kernel();
    }

    void check_status() {
        if (mb->status == MB_ABORTED)
            ARK_ERR(GpuError, "the loop kernel gave up waiting at a grid barrier (limit ",
                    "ARKMI_BARRIER_LIMIT_MS); the plan's workgroups did not all arrive");
    }

    void run(int iter) {
        if (iter <= 0) return;
        if (!launched) ARK_ERR(InvalidUsageError, "Need to launch before running.");
        set_device();
        if (loop_mode) {
            wait(-1);  // a previous run may still be in flight
            if (!kernel_resident()) {
                check_status();
                start_kernel();  // it left after the idle limit; bring it back
            }
            __atomic_store_n(&mb->cmd, iter, __ATOMIC_RELEASE);
        } else {
            ARKMI_HIP(hipMemsetAsync(ctl, 0, sizeof(LoopControl), stream));
            if (d_dep_counters) ARKMI_HIP(hipMemsetAsync(d_dep_counters, 0, dep_counter_bytes, stream));
            if (d_gemv_claims) ARKMI_HIP(hipMemsetAsync(d_gemv_claims, 0, gemv_claim_bytes, stream));
            loop_kernel_launch(kernel, prog, ctl, mb_dev, grid, threads, lds_bytes, iter, idle_ticks, wait_ticks,
                               stream);
        }
    }

    // The plan's ops as separate kernels: `iter` passes, one launch per task group
    // in plan order on the executor's stream (kernel boundaries stand in for the
    // barriers).  Asynchronous; the loop kernel must not be resident.
    void run_separate(int iter) {
        if (destroyed) ARK_ERR(InvalidUsageError, "executor is destroyed");
        if (!compiled) ARK_ERR(InvalidUsageError, "Need to compile first.");
        if (launched && loop_mode) ARK_ERR(InvalidUsageError, "stop the loop kernel before running its ops as separate kernels");
        set_device();
        // the bodies' bounded waits (the split of K) use the control block's abort word
        ARKMI_HIP(hipMemsetAsync(ctl, 0, sizeof(LoopControl), stream));
        for (int it = 0; it < iter; ++it) {
            for (size_t gi = 0; gi < h_groups.size(); ++gi) {
                const void *k = step_kernel_select(h_group_fam[gi]);
                if (std::find(step_kernels_ready.begin(), step_kernels_ready.end(), k) == step_kernels_ready.end()) {
                    loop_kernel_prepare(k, lds_bytes);
                    step_kernels_ready.push_back(k);
                }
                const DevTaskGroup &g = h_groups[gi];
                step_kernel_launch(k, prog, ctl, mb_dev, (int)gi, grid, threads,
                                   loop_kernel_lds_reserved() + g.n_slots * g.slot_sram, wait_ticks, stream);
            }
        }
    }

    void wait(int64_t max_spin) {
        if (!launched) return;
        set_device();
        if (!loop_mode) {
            ARKMI_HIP(hipStreamSynchronize(stream));
            check_status();
            return;
        }
        int64_t spins = 0;
        while (__atomic_load_n(&mb->cmd, __ATOMIC_ACQUIRE) > 0) {
            if (++spins >= (max_spin > 0 ? max_spin : 4096)) {
                spins = 0;
                check_status();  // a barrier that gave up is reported even if the kernel lingers
                hipError_t q = hipEventQuery(ev_end);
                if (q == hipSuccess) {
                    // the kernel is gone while a command is pending
                    check_status();
                    if (__atomic_load_n(&mb->cmd, __ATOMIC_ACQUIRE) > 0) {
                        if (max_spin > 0) {
                            ARK_LOG(WARN, "Stream is finished but the loop flag is still set.");
                            return;
                        }
                        start_kernel();  // raced with its idle exit: resume the pending command
                    }
                } else if (q != hipErrorNotReady) {
                    ARK_ERR(GpuError, "loop kernel failed: ", hipGetErrorString(q));
                } else if (max_spin > 0) {
                    return;  // bounded wait requested
                }
                std::this_thread::yield();
            }
        }
        check_status();
    }

    float stop(int64_t max_spin) {
        if (!launched) return 0.f;
        set_device();
        wait(max_spin);
        if (loop_mode) {
            __atomic_store_n(&mb->cmd, -1, __ATOMIC_RELEASE);
            ARKMI_HIP(hipStreamSynchronize(stream));
            mb->cmd = 0;
        } else {
            ARKMI_HIP(hipStreamSynchronize(stream));
        }
        hipEvent_t ev_stop;
        ARKMI_HIP(hipEventCreate(&ev_stop));
        ARKMI_HIP(hipEventRecord(ev_stop, stream));
        ARKMI_HIP(hipEventSynchronize(ev_stop));
        float ms = 0.f;
        ARKMI_HIP(hipEventElapsedTime(&ms, ev_begin, ev_stop));
        (void)hipEventDestroy(ev_stop);
        launched = false;
        check_status();
        return ms;
    }

    void release() {
        if (destroyed) return;
        try {
            if (launched) stop(-1);
        } catch (...) {
        }
        (void)hipSetDevice(device);
        for (void *p : {(void *)arena, (void *)ctl, (void *)d_ops, (void *)d_groups, (void *)d_steps,
                        (void *)d_trace, (void *)d_clock, (void *)d_waits, (void *)d_spans, (void *)d_signal,
                        (void *)d_dep_counters, (void *)d_gemv_seq, (void *)d_gemv_claims})
            if (p) (void)hipFree(p);
        for (void *p : scratch_allocs) (void)hipFree(p);
        scratch_allocs.clear();
        if (mb) (void)hipHostFree((void *)mb);
        if (ev_begin) (void)hipEventDestroy(ev_begin);
        if (ev_end) (void)hipEventDestroy(ev_end);
        if (own_stream && stream) (void)hipStreamDestroy(stream);
        arena = nullptr; ctl = nullptr; d_ops = nullptr; d_groups = nullptr; d_steps = nullptr;
        d_trace = nullptr; d_clock = nullptr; d_waits = nullptr; d_spans = nullptr; d_signal = nullptr;
        d_dep_counters = nullptr; d_gemv_seq = nullptr; d_gemv_claims = nullptr; mb = nullptr; ev_begin = ev_end = nullptr; stream = nullptr;
        destroyed = true;
    }

    // Copies between a (possibly strided) tensor view and a dense user buffer
    // (executor.cpp:783-886).
    void copy(size_t buffer_id, int ndims, const int64_t *shape, const int64_t *strides,
              const int64_t *offsets, size_t elem, void *data, size_t bytes, hipStream_t user_stream,
              bool to_device, bool is_d2d) {
        if (destroyed) ARK_ERR(InvalidUsageError, "executor is destroyed");
        set_device();
        auto it = buffer_offset.find(buffer_id);
        if (it == buffer_offset.end()) ARK_ERR(InvalidUsageError, "unknown buffer id ", buffer_id);
        if (ndims < 1 || ndims > 4) ARK_ERR(InvalidUsageError, "ndims must be 1..4");
        int64_t sh[4] = {1, 1, 1, 1}, st[4] = {1, 1, 1, 1}, of[4] = {0, 0, 0, 0};
        for (int i = 0; i < ndims; ++i) {
            sh[4 - ndims + i] = shape[i];
            st[4 - ndims + i] = strides[i];
            of[4 - ndims + i] = offsets[i];
        }
        size_t nelems = (size_t)(sh[0] * sh[1] * sh[2] * sh[3]);
        if (bytes != nelems * elem)
            ARK_ERR(InvalidUsageError, "Destination bytes (", bytes, ") mismatches the tensor data bytes (",
                    nelems * elem, ").");
        int64_t es[4];
        int64_t acc = 1;
        for (int i = 3; i >= 0; --i) {
            es[i] = acc;
            acc *= st[i];
        }
        for (int i = 0; i < 4; ++i)
            if (sh[i] < 0 || of[i] < 0 || st[i] < 1 || of[i] + sh[i] > st[i])
                ARK_ERR(InvalidUsageError, "tensor view: offset + shape exceeds the stride in dimension ", i - (4 - ndims));
        if ((size_t)acc * elem > buffer_bytes.at(buffer_id))
            ARK_ERR(InvalidUsageError, "tensor view exceeds its buffer");
        char *base = arena + it->second +
                     (size_t)(of[0] * es[0] + of[1] * es[1] + of[2] * es[2] + of[3]) * elem;
        hipStream_t cs = user_stream;
        bool own = false;
        if (!cs) {
            ARKMI_HIP(hipStreamCreateWithFlags(&cs, hipStreamNonBlocking));
            own = true;
        } else if (cs == stream && launched && loop_mode) {
            ARK_LOG(WARN, "copying on the loop kernel's stream while it is launched will deadlock");
        }
        hipMemcpyKind kind = is_d2d ? hipMemcpyDeviceToDevice
                                    : (to_device ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost);
        const size_t row_bytes = (size_t)sh[3] * elem;
        char *user = static_cast<char *>(data);
        // collapse to 2-D copies: rows of sh[3] elements at pitch st[3]
        for (int64_t n = 0; n < sh[0]; ++n)
            for (int64_t c = 0; c < sh[1]; ++c) {
                char *dev = base + (size_t)(n * es[0] + c * es[1]) * elem;
                char *usr = user + (size_t)((n * sh[1] + c) * sh[2]) * row_bytes;
                if (to_device)
                    ARKMI_HIP(hipMemcpy2DAsync(dev, (size_t)st[3] * elem, usr, row_bytes, row_bytes,
                                               (size_t)sh[2], kind, cs));
                else
                    ARKMI_HIP(hipMemcpy2DAsync(usr, row_bytes, dev, (size_t)st[3] * elem, row_bytes,
                                               (size_t)sh[2], kind, cs));
            }
        ARKMI_HIP(hipStreamSynchronize(cs));
        if (own) (void)hipStreamDestroy(cs);
    }
};

}  // namespace arkmi

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------
using arkmi::Executor;

struct arkmi_exec {
    Executor ex;
};

namespace {

template <typename F>
int guard_exec(F &&f) {
    try {
        f();
        return ARKMI_OK;
    } catch (const ark::InvalidUsageError &e) { arkmi::set_last_error(e.what()); return ARKMI_INVALID_USAGE;
    } catch (const ark::ModelError &e) { arkmi::set_last_error(e.what()); return ARKMI_MODEL_ERROR;
    } catch (const ark::PlanError &e) { arkmi::set_last_error(e.what()); return ARKMI_PLAN_ERROR;
    } catch (const ark::UnsupportedError &e) { arkmi::set_last_error(e.what()); return ARKMI_UNSUPPORTED;
    } catch (const ark::SystemError &e) { arkmi::set_last_error(e.what()); return ARKMI_SYSTEM_ERROR;
    } catch (const ark::GpuError &e) { arkmi::set_last_error(e.what()); return ARKMI_GPU_ERROR;
    } catch (const ark::BaseError &e) { arkmi::set_last_error(e.what()); return ARKMI_INTERNAL_ERROR;
    } catch (const arkmi::Error &e) { arkmi::set_last_error(e.what()); return e.code;
    } catch (const std::exception &e) { arkmi::set_last_error(e.what()); return ARKMI_INTERNAL_ERROR;
    } catch (...) { arkmi::set_last_error("unknown exception"); return ARKMI_INTERNAL_ERROR; }
}

char *dup_text(const std::string &s) {
    char *p = (char *)std::malloc(s.size() + 1);
    if (!p) ARK_ERR(SystemError, "out of memory");
    std::memcpy(p, s.c_str(), s.size() + 1);
    return p;
}

}  // namespace

extern "C" {

int arkmi_exec_create(int device_id, void *stream, const char *name, const char *plan_json,
                      int loop_mode, arkmi_exec **out) {
    return guard_exec([&] {
        if (!out || !plan_json) ARK_ERR(InvalidUsageError, "null argument");
        auto h = std::make_unique<arkmi_exec>();
        h->ex.init(device_id, stream, name ? name : "", plan_json, loop_mode != 0);
        *out = h.release();
    });
}

int arkmi_exec_destroy(arkmi_exec *h) {
    return guard_exec([&] {
        if (!h) return;
        h->ex.release();
        delete h;
    });
}

int arkmi_exec_release(arkmi_exec *h) {
    return guard_exec([&] {
        if (!h) ARK_ERR(InvalidUsageError, "null argument");
        h->ex.release();
    });
}

int arkmi_exec_enable_trace(arkmi_exec *h) {
    return guard_exec([&] {
        if (!h) ARK_ERR(InvalidUsageError, "null argument");
        if (h->ex.compiled) ARK_ERR(InvalidUsageError, "enable tracing before compile()");
        h->ex.trace_enabled = true;
    });
}

int arkmi_exec_compile(arkmi_exec *h) {
    return guard_exec([&] {
        if (!h) ARK_ERR(InvalidUsageError, "null argument");
        h->ex.compile();
    });
}

int arkmi_exec_launch(arkmi_exec *h) {
    return guard_exec([&] {
        if (!h) ARK_ERR(InvalidUsageError, "null argument");
        h->ex.launch();
    });
}

int arkmi_exec_run(arkmi_exec *h, int iter) {
    return guard_exec([&] {
        if (!h) ARK_ERR(InvalidUsageError, "null argument");
        h->ex.run(iter);
    });
}

int arkmi_exec_run_separate(arkmi_exec *h, int iter) {
    return guard_exec([&] {
        if (!h) ARK_ERR(InvalidUsageError, "null argument");
        h->ex.run_separate(iter);
    });
}

int arkmi_exec_wait(arkmi_exec *h, int64_t max_spin_count) {
    return guard_exec([&] {
        if (!h) ARK_ERR(InvalidUsageError, "null argument");
        h->ex.wait(max_spin_count);
    });
}

int arkmi_exec_stop(arkmi_exec *h, int64_t max_spin_count, float *elapsed_ms) {
    return guard_exec([&] {
        if (!h) ARK_ERR(InvalidUsageError, "null argument");
        float ms = h->ex.stop(max_spin_count);
        if (elapsed_ms) *elapsed_ms = ms;
    });
}

int arkmi_exec_plan(arkmi_exec *h, char **out) {
    return guard_exec([&] {
        if (!h || !out) ARK_ERR(InvalidUsageError, "null argument");
        *out = dup_text(h->ex.plan_text);
    });
}

int arkmi_exec_info(arkmi_exec *h, arkmi_exec_info_t *out) {
    return guard_exec([&] {
        if (!h || !out) ARK_ERR(InvalidUsageError, "null argument");
        std::memset(out, 0, sizeof(*out));
        out->device_id = h->ex.device;
        out->stream = (void *)h->ex.stream;
        out->num_processors = h->ex.sched.num_processors;
        out->threads_per_processor = h->ex.sched.num_warps_per_processor * 64;
        out->lds_bytes = h->ex.lds_bytes;
        out->arena_bytes = h->ex.total_bytes;
        out->num_steps = (int)h->ex.sched.steps.size();
        out->num_barriers = h->ex.sched.num_barriers;
        out->barriers_elided = h->ex.barriers_elided;
        out->kernel_families = h->ex.kernel_families;
        out->compiled = h->ex.compiled;
        out->launched = h->ex.launched;
        out->destroyed = h->ex.destroyed;
        out->loop_mode = h->ex.loop_mode;
        out->iterations_done = h->ex.mb ? h->ex.mb->done : 0;
        out->barriers_local = h->ex.barriers_local;
        out->iteration_sync = h->ex.iteration_sync;
        out->barriers_counted = h->ex.barriers_counted;
        out->gemv_chains = h->ex.gemv_chains;
        out->gemv_claimed = h->ex.gemv_claimed;
    });
}

int arkmi_exec_buffer_address(arkmi_exec *h, uint64_t buffer_id, uintptr_t *out) {
    return guard_exec([&] {
        if (!h || !out) ARK_ERR(InvalidUsageError, "null argument");
        auto it = h->ex.buffer_offset.find((size_t)buffer_id);
        if (it == h->ex.buffer_offset.end())
            ARK_ERR(InvalidUsageError, "Tensor has an unknown buffer ID ", buffer_id);
        *out = (uintptr_t)(h->ex.arena + it->second);
    });
}

int arkmi_exec_copy(arkmi_exec *h, uint64_t buffer_id, int ndims, const int64_t *shape,
                    const int64_t *strides, const int64_t *offsets, int elem_bytes, void *data,
                    size_t bytes, void *stream, int to_device, int is_d2d) {
    return guard_exec([&] {
        if (!h || !shape || !strides || !offsets || !data) ARK_ERR(InvalidUsageError, "null argument");
        h->ex.copy((size_t)buffer_id, ndims, shape, strides, offsets, (size_t)elem_bytes, data, bytes,
                   (hipStream_t)stream, to_device != 0, is_d2d != 0);
    });
}

int arkmi_exec_read_trace(arkmi_exec *h, int task_group, int32_t *records, int max_tasks, int *n_tasks) {
    return guard_exec([&] {
        if (!h || !n_tasks) ARK_ERR(InvalidUsageError, "null argument");
        auto &ex = h->ex;
        if (!ex.trace_enabled || !ex.d_trace) ARK_ERR(InvalidUsageError, "tracing is not enabled");
        if (task_group < 0 || (size_t)task_group >= ex.h_groups.size())
            ARK_ERR(InvalidUsageError, "task group index out of range");
        const auto &g = ex.h_groups[(size_t)task_group];
        int n = std::max(0, (g.task_e - g.task_b + g.task_s - 1) / g.task_s);
        *n_tasks = n;
        if (!records) return;
        n = std::min(n, max_tasks);
        ex.set_device();
        ARKMI_HIP(hipMemcpy(records, ex.d_trace + g.trace_offset, (size_t)n * sizeof(arkmi::TraceRecord),
                            hipMemcpyDeviceToHost));
    });
}

// Entry time of every schedule step per block: an elided barrier takes the
// entry time of the step after it (zero duration).
static std::vector<uint64_t> schedule_clocks(arkmi::Executor &ex) {
    const size_t nd = (size_t)ex.num_dev_steps + 1, ns = ex.sched.steps.size() + 1;
    std::vector<uint64_t> dev((size_t)ex.grid * nd), out((size_t)ex.grid * ns);
    ex.set_device();
    ARKMI_HIP(hipMemcpy(dev.data(), ex.d_clock, dev.size() * sizeof(uint64_t), hipMemcpyDeviceToHost));
    for (int b = 0; b < ex.grid; ++b) {
        uint64_t next = dev[(size_t)b * nd + nd - 1];
        out[(size_t)b * ns + ns - 1] = next;
        for (int i = (int)ns - 2; i >= 0; --i) {
            const int d = ex.dev_step_of[(size_t)i];
            if (d >= 0) next = dev[(size_t)b * nd + (size_t)d];
            out[(size_t)b * ns + (size_t)i] = next;
        }
    }
    return out;
}

int arkmi_exec_read_step_times(arkmi_exec *h, double *step_us, int max_steps, int *n_steps) {
    return guard_exec([&] {
        if (!h || !n_steps) ARK_ERR(InvalidUsageError, "null argument");
        auto &ex = h->ex;
        if (!ex.trace_enabled || !ex.d_clock) ARK_ERR(InvalidUsageError, "tracing is not enabled");
        const int n = (int)ex.sched.steps.size();
        *n_steps = n;
        if (!step_us) return;
        auto clk = schedule_clocks(ex);  // block 0 comes first
        for (int i = 0; i < n && i < max_steps; ++i)
            step_us[i] = (double)(clk[(size_t)i + 1] - clk[(size_t)i]) * 1000.0 / (double)ex.wall_khz;
    });
}

int arkmi_exec_read_step_clocks(arkmi_exec *h, uint64_t *ticks, size_t max_entries, int *n_blocks,
                                int *n_steps, int *ticks_per_ms) {
    return guard_exec([&] {
        if (!h || !n_blocks || !n_steps) ARK_ERR(InvalidUsageError, "null argument");
        auto &ex = h->ex;
        if (!ex.trace_enabled || !ex.d_clock) ARK_ERR(InvalidUsageError, "tracing is not enabled");
        *n_blocks = ex.grid;
        *n_steps = (int)ex.sched.steps.size();
        if (ticks_per_ms) *ticks_per_ms = ex.wall_khz;
        if (!ticks) return;
        auto clk = schedule_clocks(ex);
        std::memcpy(ticks, clk.data(), std::min(max_entries, clk.size()) * sizeof(uint64_t));
    });
}

int arkmi_plan_analysis(const char *plan_json, int dep_counters, char **analysis_json) {
    return guard_exec([&] {
        if (!plan_json || !analysis_json) ARK_ERR(InvalidUsageError, "null argument");
        arkmi::Executor ex;
        ex.dry = true;
        ex.force_deps = dep_counters;
        try {
            ex.plan = Json::parse(plan_json);
        } catch (const std::exception &e) {
            ARK_ERR(PlanError, "failed to parse the plan: ", e.what());
        }
        ex.plan_text = plan_json;
        ex.sched = arkmi::build_schedule(ex.plan);
        ex.layout_buffers();
        ex.arena = (char *)((uintptr_t)1 << 45);  // a stand-in base address: nothing is read through it
        try {
            ex.compile();
        } catch (...) {
            ex.arena = nullptr;
            ex.destroyed = true;
            throw;
        }
        ex.arena = nullptr;
        ex.destroyed = true;  // nothing to release
        Json out = Json::object();
        out["NumProcessors"] = (long long)ex.grid;
        out["KernelFamilies"] = (long long)ex.kernel_families;
        out["BarriersElided"] = (long long)ex.barriers_elided;
        out["BarriersLocal"] = (long long)ex.barriers_local;
        out["BarriersCounted"] = (long long)ex.barriers_counted;
        out["GemvChains"] = (long long)ex.gemv_chains;
        out["GemvClaimed"] = (long long)ex.gemv_claimed;
        out["GemmXcdOrdered"] = (long long)ex.gemm_xcd_ordered;
        out["AttnXcdOrdered"] = (long long)ex.attn_xcd_ordered;
        out["BarriersWidened"] = (long long)ex.barriers_widened;
        out["IterationSync"] = (long long)ex.iteration_sync;
        out["NumCounters"] = (long long)ex.dry_counters;
        Json steps = Json::array();
        for (const auto &st : ex.dry_steps) {
            Json j = Json::object();
            if (st.kind == arkmi::STEP_BARRIER) {
                j["Kind"] = "Barrier";
                j["Count"] = (long long)st.count;
            } else if (st.kind == arkmi::STEP_LOCAL_SYNC) {
                j["Kind"] = "LocalSync";
            } else {
                const arkmi::DevTaskGroup &g = ex.h_groups[(size_t)st.index];
                const int n_tasks = std::max(0, (g.task_e - g.task_b + g.task_s - 1) / g.task_s);
                j["Kind"] = "Tasks";
                j["Group"] = (long long)st.index;
                j["NumTasks"] = (long long)n_tasks;
                j["Chain"] = (long long)g.chain;
                if (ex.dry_ops.size() >= (size_t)(g.op_begin + g.op_count)) {
                    Json again = Json::array();
                    bool any_row = false;
                    for (int o = 0; o < g.op_count; ++o) {
                        const arkmi::DevOp &op = ex.dry_ops[(size_t)(g.op_begin + o)];
                        any_row = any_row || op.kind == arkmi::DEV_ROW;
                        again.push_back((long long)(op.kind == arkmi::DEV_ROW ? op.row.in_read_again : 0));
                    }
                    if (any_row) j["InputReadAgain"] = again;
                    const arkmi::DevOp &first = ex.dry_ops[(size_t)g.op_begin];
                    if (first.kind == arkmi::DEV_ROW) j["TouchesNextRows"] = first.row.pf_base != nullptr;
                }
                if (ex.dry_ops.size() > (size_t)g.op_begin && ex.dry_ops[(size_t)g.op_begin].kind == arkmi::DEV_GEMM) {
                    j["XcdRound"] = (long long)ex.dry_ops[(size_t)g.op_begin].gemm.xcd_round;
                    j["XcdBand"] = (long long)ex.dry_ops[(size_t)g.op_begin].gemm.xcd_band;
                    if (ex.dry_ops[(size_t)g.op_begin].gemm.split_k == 2) {
                        j["SplitAt"] = (long long)ex.dry_ops[(size_t)g.op_begin].gemm.split_at;
                    }
                }
                j["Claimed"] = g.claim >= 0;
                j["FoldedIntoStore"] = (size_t)st.index < ex.group_fused.size() && ex.group_fused[(size_t)st.index] != 0;
                Json waits = Json::array();
                for (int w = 0; w < g.n_waits; ++w) {
                    const arkmi::DevWait &dw = ex.dry_waits[(size_t)(g.wait_begin + w)];
                    Json jw = Json::object();
                    long long producer = -1;
                    for (size_t gi = 0; gi < ex.h_groups.size(); ++gi)
                        if (ex.h_groups[gi].signal_begin >= 0 && ex.h_groups[gi].signal_base == dw.counter_base)
                            producer = (long long)gi;
                    jw["ProducerGroup"] = producer;
                    jw["Expect"] = (long long)dw.expect;
                    Json spans = Json::array();
                    for (int t = 0; t < n_tasks; ++t) {
                        Json sp = Json::array();
                        sp.push_back((long long)ex.dry_spans[(size_t)(g.span_begin + 2 * (t * g.n_waits + w))]);
                        sp.push_back((long long)ex.dry_spans[(size_t)(g.span_begin + 2 * (t * g.n_waits + w) + 1)]);
                        spans.push_back(sp);
                    }
                    jw["Spans"] = spans;
                    waits.push_back(jw);
                }
                j["Waits"] = waits;
                if (g.signal_begin >= 0 && ex.barriers_counted > 0) {
                    Json map = Json::array();
                    int n_signal = n_tasks;
                    // (a matmul that splits K signals once per tile)
                    size_t end = ex.dry_signal.size();
                    for (const auto &g2 : ex.h_groups)
                        if (g2.signal_begin > g.signal_begin) end = std::min(end, (size_t)g2.signal_begin);
                    n_signal = (int)(end - (size_t)g.signal_begin);
                    for (int t = 0; t < n_signal; ++t) map.push_back((long long)ex.dry_signal[(size_t)(g.signal_begin + t)]);
                    j["SignalMap"] = map;
                }
            }
            steps.push_back(j);
        }
        out["Steps"] = steps;
        *analysis_json = dup_text(out.dump());
    });
}

int arkmi_plan_schedule(const char *plan_json, char **schedule_json) {
    return guard_exec([&] {
        if (!plan_json || !schedule_json) ARK_ERR(InvalidUsageError, "null argument");
        Json plan;
        try {
            plan = Json::parse(plan_json);
        } catch (const std::exception &e) {
            ARK_ERR(PlanError, "failed to parse the plan: ", e.what());
        }
        *schedule_json = dup_text(arkmi::schedule_to_json(arkmi::build_schedule(plan)).dump());
    });
}

int arkmi_schedule_tasks(const char *plan_json, int step, int block, int slot, int64_t *tasks,
                         int max_tasks, int *n_tasks) {
    return guard_exec([&] {
        if (!plan_json || !n_tasks) ARK_ERR(InvalidUsageError, "null argument");
        arkmi::Schedule sch = arkmi::build_schedule(Json::parse(plan_json));
        if (step < 0 || (size_t)step >= sch.steps.size()) ARK_ERR(InvalidUsageError, "step out of range");
        auto v = arkmi::schedule_tasks_of(sch, sch.steps[(size_t)step], block, slot);
        *n_tasks = (int)v.size();
        for (size_t i = 0; i < v.size() && (int)i < max_tasks && tasks; ++i) tasks[i] = v[i];
    });
}

}  // extern "C"
