// Planner: compressed model -> plan JSON.
//
// Restates ark/api/planner.cpp:127-262.  The plan is a pure function of
// (model, number of processors, architecture name): the device is queried for
// those two facts only, and a constructor that takes them directly makes the
// planner usable (and testable) without a GPU.
#include <ark/model.hpp>
#include <ark/planner.hpp>
#include <sys/stat.h>

#include <fstream>

#include "../../../include/arkmi.h"
#include "ir.hpp"
#include "ops.hpp"

namespace ark {

class Planner::Impl {
   public:
    Impl(const Model &model, const std::string &arch, int num_processors, int device_id)
        : model_(model.compress()), arch_(Arch::from_name(arch)), num_processors_(num_processors),
          device_id_(device_id) {}

    std::string plan(bool pretty) const;

    Model model_;
    Arch arch_;
    int num_processors_;
    int device_id_;
    std::vector<Planner::ConfigRule> rules_;
};

static void write_text(const std::string &dir, const std::string &file, const std::string &text) {
    ::mkdir(dir.c_str(), 0777);
    std::ofstream f(dir + "/" + file);
    if (f) f << text;
}

static Json node_ctx(const ModelNodeRef &node, const std::string &key) {
    auto it = node->context.find(key);
    return it == node->context.end() ? Json() : it->second;
}

static int64_t need_field(const ModelOp &op, const Json &config, const char *field) {
    if (!config.contains(field))
        ARK_ERR(PlanError, "Config field not found: ", field, " in ", op.name());
    return config.at(field).as_int();
}

static Json range2(int64_t b, int64_t e) {
    Json r = Json::array();
    r.push_back((long long)b);
    r.push_back((long long)e);
    return r;
}

std::string Planner::Impl::plan(bool pretty) const {
    const int64_t num_sm = num_processors_;
    Json task_infos = Json::array();
    Json processor_groups = Json::array();
    int64_t max_processor_id = 1, max_warp_id = 1, next_task_id = 0;
    int prev_ctx_id = -1;
    bool first_op = true;

    for (const auto &node : model_.nodes()) {
        const auto &op = node->op;
        if (op->is_virtual()) continue;

        // config: context > first rule that answers > op default
        Json config;
        Json ctx_config = node_ctx(node, "Config");
        if (!ctx_config.empty()) {
            config = ctx_config;
        } else if (!rules_.empty()) {
            const std::string op_str = op->serialize().dump();
            for (const auto &rule : rules_) {
                std::string answer = rule(op_str, arch_.name());
                if (!answer.empty()) {
                    config = Json::parse(answer);
                    break;
                }
            }
        }
        const bool config_given = !config.empty();
        if (config.empty()) config = default_config(*op, arch_, num_processors_);

        Json ctx_id = node_ctx(node, "Id");
        Json ctx_sync = node_ctx(node, "Sync");
        const int id = ctx_id.empty() ? -1 : (int)ctx_id.as_int();
        const bool sync = ctx_sync.empty() ? true : ctx_sync.as_bool();
        const bool fuse = (id == prev_ctx_id && !sync);
        if (fuse && !config_given && arch_.belongs_to("ROCM_950")) {
            // an elementwise op fused behind its producer takes the producer's tiling
            Json follower = follower_config(*op, task_infos.back());
            if (!follower.empty()) config = follower;
        }
        const int64_t num_warps = need_field(*op, config, "NumWarps");
        const int64_t num_tasks = need_field(*op, config, "NumTasks");
        const int64_t sram_bytes = need_field(*op, config, "SramBytes");
        const int64_t granularity = config.value_or<int64_t>("Granularity", 1);

        Json op_json = op->serialize();
        op_json["Config"] = config;

        if (fuse) {
            // same planner context, no sync requested: fuse into the previous task
            Json &ti = task_infos.back();
            ti["NumWarps"] = (long long)std::max(ti["NumWarps"].as_int(), num_warps);
            ti["SramBytes"] = (long long)std::max(ti["SramBytes"].as_int(), sram_bytes);
            ti["Ops"].push_back(op_json);
        } else {
            Json ti = Json::object();
            // ids start at 0 and pre-increment afterwards (planner.cpp:190)
            ti["Id"] = (long long)(first_op ? next_task_id : ++next_task_id);
            ti["NumWarps"] = (long long)num_warps;
            ti["SramBytes"] = (long long)sram_bytes;
            Json ops = Json::array();
            ops.push_back(op_json);
            ti["Ops"] = ops;
            task_infos.push_back(ti);

            Json ctx_pr = node_ctx(node, "ProcessorRange");
            Json ctx_wr = node_ctx(node, "WarpRange");
            Json ctx_sr = node_ctx(node, "SramRange");

            Json pg = Json::object();
            if (!ctx_pr.empty()) {
                pg["ProcessorRange"] = ctx_pr;
                max_processor_id = std::max(max_processor_id, ctx_pr.at((size_t)1).as_int());
            } else {
                int64_t n = std::min(num_sm, num_tasks);
                pg["ProcessorRange"] = range2(0, n);
                max_processor_id = std::max(max_processor_id, n);
            }
            Json rg = Json::object();
            rg["ProcessorRange"] = pg["ProcessorRange"];
            if (!ctx_wr.empty()) {
                rg["WarpRange"] = ctx_wr;
                max_warp_id = std::max(max_warp_id, ctx_wr.at((size_t)1).as_int());
            } else {
                rg["WarpRange"] = range2(0, num_warps);
                max_warp_id = std::max(max_warp_id, num_warps);
            }
            rg["SramRange"] = ctx_sr.empty() ? range2(0, sram_bytes) : ctx_sr;
            Json tg = Json::object();
            tg["TaskId"] = ti["Id"];
            tg["TaskRange"] = range2(0, num_tasks);
            tg["Granularity"] = (long long)granularity;
            Json tgs = Json::array();
            tgs.push_back(tg);
            rg["TaskGroups"] = tgs;
            Json rgs = Json::array();
            rgs.push_back(rg);
            pg["ResourceGroups"] = rgs;
            processor_groups.push_back(pg);
        }
        prev_ctx_id = id;
        first_op = false;
    }

    Json plan = Json::object();
    plan["Rank"] = model_.rank();
    plan["WorldSize"] = model_.world_size();
    plan["Architecture"] = arch_.name();
    plan["NumProcessors"] = (long long)max_processor_id;
    plan["NumWarpsPerProcessor"] = (long long)max_warp_id;
    plan["TaskInfos"] = task_infos;
    plan["ProcessorGroups"] = processor_groups;

    std::string text = pretty ? ::arkmi::dump_pretty_plan(plan) : plan.dump();
    const std::string &tmp = get_env().path_tmp_dir;
    const std::string tag = std::to_string(device_id_ < 0 ? 0 : device_id_);
    write_text(tmp, "model_gpu" + tag + ".json", model_.serialize());
    write_text(tmp, "plan_gpu" + tag + ".json", text);
    return text;
}

static std::shared_ptr<Planner::Impl> impl_for_device(const Model &model, int device_id) {
    arkmi_device_info info;
    if (arkmi_device_info_get(device_id, &info) != ARKMI_OK)
        ARK_ERR(GpuError, "cannot query device ", device_id, ": ", arkmi_last_error());
    return std::make_shared<Planner::Impl>(model, info.arch, info.num_cu, device_id);
}

Planner::Planner(const Model &model, int device_id) : impl_(impl_for_device(model, device_id)) {}
Planner::Planner(const Model &model, const std::string &arch_name, int num_processors)
    : impl_(std::make_shared<Impl>(model, arch_name, num_processors, -1)) {}
Planner::~Planner() = default;

void Planner::install_config_rule(ConfigRule rule) {
    // an exception inside a rule skips the rule (planner.cpp:108-118)
    impl_->rules_.push_back([rule](const std::string &op, const std::string &arch) -> std::string {
        try {
            return rule(op, arch);
        } catch (const std::exception &e) {
            ARK_LOG(WARN, "Skipping a config rule due to an error: ", e.what());
            return "";
        }
    });
}

std::string Planner::plan(bool pretty) const { return impl_->plan(pretty); }

}  // namespace ark
