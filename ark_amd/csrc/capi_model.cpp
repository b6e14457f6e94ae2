// C ABI over ark::Model / PlannerContext / Planner.
#include <ark/ark.hpp>

#include <cstdlib>
#include <cstring>
#include <map>

#include "host/ir.hpp"
#include "host/ops.hpp"
#include "host_common.h"

using ark::Json;

struct arkmi_model {
    ark::Model model;
    std::map<int64_t, ark::Tensor> tensors;
    std::vector<std::unique_ptr<ark::PlannerContext>> contexts;
    arkmi_model(int rank, int ws) : model(rank, ws) {}
    int64_t keep(const ark::Tensor &t) {
        tensors[(int64_t)t.id()] = t;
        return (int64_t)t.id();
    }
    ark::Tensor get(int64_t id) const {
        if (id < 0) return ark::NullTensor;
        auto it = tensors.find(id);
        if (it == tensors.end()) ARKMI_FAIL(ARKMI_INVALID_USAGE, "unknown tensor id ", id);
        return it->second;
    }
};

namespace {

// ark:: exceptions -> status codes
template <typename F>
int guard_ark(F &&f) {
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

char *dup_string(const std::string &s) {
    char *p = (char *)std::malloc(s.size() + 1);
    if (!p) ARKMI_FAIL(ARKMI_SYSTEM_ERROR, "out of memory");
    std::memcpy(p, s.c_str(), s.size() + 1);
    return p;
}

ark::Dims dims_of(const int64_t *v, int n) {
    if (!v) return ark::Dims();
    return ark::Dims(std::vector<ark::DimType>(v, v + n));
}

ark::Dims dims_arg(const Json &args, const char *key) {
    if (!args.contains(key)) return ark::Dims();
    return ark::Dims(args.at(key).as_int_vector());
}

const ark::DataType &dtype_of(int code) {
    static const ark::DataType *all[] = {&ark::FP32, &ark::FP16, &ark::BF16, &ark::INT32,
                                         &ark::UINT32, &ark::INT8, &ark::UINT8, &ark::BYTE};
    if (code < 0 || code > 7) ARKMI_FAIL(ARKMI_INVALID_USAGE, "unknown dtype code ", code);
    return *all[code];
}

float float_arg(const Json &args, const char *key, float dflt) {
    return args.contains(key) ? (float)args.at(key).as_double() : dflt;
}

}  // namespace

extern "C" {

void arkmi_free(void *p) { std::free(p); }

void arkmi_reset_ids(void) {
    ark::ModelTensor::reset_ids(0);
    ark::ModelBuffer::reset_ids(0);
}

int arkmi_model_create(int rank, int world_size, arkmi_model **out) {
    return guard_ark([&] {
        if (!out) ARKMI_FAIL(ARKMI_INVALID_USAGE, "out is null");
        *out = new arkmi_model(rank, world_size);
    });
}

int arkmi_model_from_json(const char *model_json, arkmi_model **out) {
    return guard_ark([&] {
        if (!model_json || !out) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null argument");
        Json j;
        try {
            j = Json::parse(model_json);
        } catch (const std::exception &e) {
            ARK_ERR(ModelError, "failed to parse the model: ", e.what());
        }
        auto graph = ark::ModelGraph::Impl::deserialize(j);  // verifies the format first
        auto m = std::make_unique<arkmi_model>(graph->rank_, graph->world_size_);
        // every tensor of the file becomes addressable by its id, and ids handed out
        // later (ops added to the rebuilt model) stay clear of the file's
        for (const auto &node : graph->nodes_)
            for (const auto *vec : {&node->op->read_tensors(), &node->op->write_tensors(), &node->op->result_tensors()})
                for (const auto &t : *vec) {
                    m->tensors[(int64_t)t->id()] = ark::Tensor(t);
                    ark::ModelTensor::reserve_id(t->id());
                    ark::ModelBuffer::reserve_id(t->buffer()->id());
                }
        ark::ModelGraphAccess::adopt(m->model, std::move(graph));
        *out = m.release();
    });
}

int arkmi_model_destroy(arkmi_model *m) {
    return guard_ark([&] {
        if (!m) return;
        while (!m->contexts.empty()) m->contexts.pop_back();
        delete m;
    });
}

int arkmi_model_tensor(arkmi_model *m, int ndims, const int64_t *shape, int dtype,
                       const int64_t *strides, const int64_t *offsets,
                       const int64_t *padded_shape, int rank, const char *name,
                       int64_t *tensor_out) {
    return guard_ark([&] {
        if (!m || !shape || !tensor_out) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null argument");
        if (ndims < 0 || ndims > 4) ARKMI_FAIL(ARKMI_INVALID_USAGE, "ndims must be 0..4");
        ark::Tensor t = m->model.tensor(dims_of(shape, ndims), dtype_of(dtype), dims_of(strides, ndims),
                                        dims_of(offsets, ndims), dims_of(padded_shape, ndims), rank,
                                        name ? name : "");
        *tensor_out = m->keep(t);
    });
}

int arkmi_model_op(arkmi_model *m, const char *op_c, const int64_t *inputs, int n_inputs,
                   int64_t output, const char *args_json, const char *name_c, int64_t *results,
                   int max_results, int *n_results) {
    return guard_ark([&] {
        if (!m || !op_c) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null argument");
        const std::string op(op_c), name(name_c ? name_c : "");
        Json args = (args_json && *args_json) ? Json::parse(args_json) : Json::object();
        auto in = [&](int i) -> ark::Tensor {
            if (i >= n_inputs) return ark::NullTensor;
            return m->get(inputs[i]);
        };
        auto need_inputs = [&](int n) {
            if (n_inputs < n) ARKMI_FAIL(ARKMI_INVALID_USAGE, op, " needs ", n, " input tensor(s)");
        };
        ark::Tensor out = m->get(output);
        ark::Model &M = m->model;
        std::vector<ark::Tensor> res;
        const bool scalar = args.contains("value");
        if (op == "matmul") {
            need_inputs(2);
            res = {M.matmul(in(0), in(1), out, args.value_or<bool>("trans_input", false),
                            args.value_or<bool>("trans_other", false), name)};
        } else if (op == "reduce_sum" || op == "reduce_mean" || op == "reduce_max") {
            need_inputs(1);
            int axis = (int)args.value_or<int64_t>("axis", -1);
            bool keep = args.value_or<bool>("keepdims", true);
            res = {op == "reduce_sum"    ? M.reduce_sum(in(0), axis, keep, out, name)
                   : op == "reduce_mean" ? M.reduce_mean(in(0), axis, keep, out, name)
                                         : M.reduce_max(in(0), axis, keep, out, name)};
        } else if (op == "softmax") {
            need_inputs(1);
            res = {M.softmax(in(0), n_inputs > 1 ? in(1) : ark::NullTensor, float_arg(args, "scale", 1.f), out, name)};
        } else if (op == "layernorm") {
            need_inputs(1);
            res = {M.layernorm(in(0), float_arg(args, "eps", 1e-6f), out, name)};
        } else if (op == "rmsnorm") {
            need_inputs(1);
            res = {M.rmsnorm(in(0), in(1), float_arg(args, "eps", 0.f), out, name)};
        } else if (op == "add" || op == "sub" || op == "mul" || op == "div") {
            need_inputs(1);
            if (scalar) {
                float v = (float)args.at("value").as_double();
                res = {op == "add"   ? M.add(in(0), v, out, name)
                       : op == "sub" ? M.sub(in(0), v, out, name)
                       : op == "mul" ? M.mul(in(0), v, out, name)
                                     : M.div(in(0), v, out, name)};
            } else {
                need_inputs(2);
                res = {op == "add"   ? M.add(in(0), in(1), out, name)
                       : op == "sub" ? M.sub(in(0), in(1), out, name)
                       : op == "mul" ? M.mul(in(0), in(1), out, name)
                                     : M.div(in(0), in(1), out, name)};
            }
        } else if (op == "rope") {
            need_inputs(2);
            res = {M.rope(in(0), in(1), out, name)};
        } else if (op == "embedding") {
            need_inputs(2);
            res = {M.embedding(in(0), in(1), out, name)};
        } else if (op == "swiglu") {
            need_inputs(3);
            res = {M.swiglu(in(0), in(1), in(2), out, name)};
        } else if (op == "attention") {
            need_inputs(3);
            res = {M.attention(in(0), in(1), in(2), float_arg(args, "scale", 1.f),
                               args.value_or<bool>("causal", false), out, name)};
        } else if (op == "silu_mul") {
            need_inputs(2);
            res = {M.silu_mul(in(0), in(1), out, name)};
        } else if (op == "exp" || op == "sqrt" || op == "rsqrt" || op == "relu" || op == "gelu" ||
                   op == "sigmoid") {
            need_inputs(1);
            res = {op == "exp"     ? M.exp(in(0), out, name)
                   : op == "sqrt"  ? M.sqrt(in(0), out, name)
                   : op == "rsqrt" ? M.rsqrt(in(0), out, name)
                   : op == "relu"  ? M.relu(in(0), out, name)
                   : op == "gelu"  ? M.gelu(in(0), out, name)
                                   : M.sigmoid(in(0), out, name)};
        } else if (op == "copy") {
            if (scalar) res = {M.copy((float)args.at("value").as_double(), out, name)};
            else { need_inputs(1); res = {M.copy(in(0), out, name)}; }
        } else if (op == "constant") {
            res = {M.constant((float)args.at("value").as_double(), dims_arg(args, "shape"),
                              ark::DataType::from_name(args.at("data_type").as_string()), name)};
        } else if (op == "cast") {
            need_inputs(1);
            res = {M.cast(in(0), ark::DataType::from_name(args.at("data_type").as_string()), out, name)};
        } else if (op == "transpose") {
            need_inputs(1);
            res = {M.transpose(in(0), args.at("permutation").as_int_vector(), out, name)};
        } else if (op == "reshape") {
            need_inputs(1);
            res = {M.reshape(in(0), dims_arg(args, "shape"), args.value_or<bool>("allowzero", false), name)};
        } else if (op == "refer") {
            need_inputs(1);
            res = {M.refer(in(0), dims_arg(args, "shape"), dims_arg(args, "strides"),
                           dims_arg(args, "offsets"), dims_arg(args, "padded_shape"), name)};
        } else if (op == "identity") {
            need_inputs(1);
            std::vector<ark::Tensor> deps;
            for (int i = 1; i < n_inputs; ++i) deps.push_back(in(i));
            res = {M.identity(in(0), deps, name)};
        } else if (op == "sharding") {
            need_inputs(1);
            res = M.sharding(in(0), args.at("axis").as_int(), args.at("dim_per_shard").as_int(), name);
        } else if (op == "noop") {
            need_inputs(1);
            M.noop(in(0), name);
        } else {
            ARKMI_FAIL(ARKMI_UNSUPPORTED, "unknown Model member: ", op);
        }
        if (n_results) *n_results = (int)res.size();
        for (size_t i = 0; i < res.size(); ++i) {
            int64_t id = m->keep(res[i]);
            if (results && (int)i < max_results) results[i] = id;
        }
    });
}

int arkmi_model_tensor_info(arkmi_model *m, int64_t tensor, arkmi_tensor_info *out) {
    return guard_ark([&] {
        if (!m || !out) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null argument");
        ark::Tensor t = m->get(tensor);
        if (t.is_null()) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null tensor");
        std::memset(out, 0, sizeof(*out));
        out->id = (int64_t)t.id();
        out->buffer_id = (int64_t)t.ref()->buffer()->id();
        out->dtype = t.ref()->data_type()->code();
        out->ndims = t.shape().ndims();
        for (int i = 0; i < out->ndims; ++i) {
            out->shape[i] = t.shape()[i];
            out->strides[i] = t.strides()[i];
            out->offsets[i] = t.offsets()[i];
            out->padded_shape[i] = t.padded_shape()[i];
        }
    });
}

int arkmi_model_serialize(arkmi_model *m, int pretty, char **out) {
    return guard_ark([&] {
        if (!m || !out) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null argument");
        *out = dup_string(m->model.serialize(pretty != 0));
    });
}

int arkmi_model_dump(arkmi_model *m, int compressed, int with_context, int pretty, char **out) {
    return guard_ark([&] {
        if (!m || !out) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null argument");
        ark::Model copy = compressed ? m->model.compress() : ark::Model(m->model);
        Json j = ark::ModelGraphAccess::impl(copy).to_json(with_context != 0);
        *out = dup_string(pretty ? ::arkmi::dump_pretty_model(j) : j.dump());
    });
}

int arkmi_model_context_get(arkmi_model *m, const char *key, char **out) {
    return guard_ark([&] {
        if (!m || !key || !out) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null argument");
        if (m->contexts.empty()) ARKMI_FAIL(ARKMI_INVALID_USAGE, "no planner context is open");
        *out = dup_string(m->contexts.back()->get(key));
    });
}

int arkmi_model_compress(arkmi_model *m) {
    return guard_ark([&] {
        if (!m) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null argument");
        m->model.compress_nodes();
    });
}

int arkmi_model_verify(arkmi_model *m, int *ok) {
    return guard_ark([&] {
        if (!m || !ok) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null argument");
        *ok = m->model.verify() ? 1 : 0;
    });
}

int arkmi_model_context_enter(arkmi_model *m) {
    return guard_ark([&] {
        if (!m) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null argument");
        m->contexts.push_back(std::make_unique<ark::PlannerContext>(m->model));
    });
}

int arkmi_model_context_call(arkmi_model *m, const char *member, const char *args_json) {
    return guard_ark([&] {
        if (!m || !member || !args_json) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null argument");
        if (m->contexts.empty()) ARKMI_FAIL(ARKMI_INVALID_USAGE, "no planner context is open");
        ark::PlannerContext &ctx = *m->contexts.back();
        const std::string f(member);
        Json a = Json::parse(args_json);
        auto range = [&](void (ark::PlannerContext::*fn)(int, int, int)) {
            auto v = a.as_int_vector();
            if (v.size() < 2 || v.size() > 3) ARKMI_FAIL(ARKMI_INVALID_USAGE, "range needs [b,e] or [b,e,s]");
            (ctx.*fn)((int)v[0], (int)v[1], v.size() == 3 ? (int)v[2] : 1);
        };
        if (f == "processor_range") range(&ark::PlannerContext::processor_range);
        else if (f == "warp_range") range(&ark::PlannerContext::warp_range);
        else if (f == "sram_range") range(&ark::PlannerContext::sram_range);
        else if (f == "sync") ctx.sync(a.as_bool());
        else if (f == "config") ctx.config(a.dump());
        else ARKMI_FAIL(ARKMI_UNSUPPORTED, "unknown PlannerContext member: ", f);
    });
}

int arkmi_model_context_exit(arkmi_model *m) {
    return guard_ark([&] {
        if (!m) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null argument");
        if (m->contexts.empty()) ARKMI_FAIL(ARKMI_INVALID_USAGE, "no planner context is open");
        m->contexts.pop_back();
    });
}

int arkmi_model_plan(arkmi_model *m, int device_id, const char *arch, int num_processors,
                     const arkmi_config_rule *rules, void *const *rule_users, int n_rules,
                     int pretty, char **plan_out) {
    return guard_ark([&] {
        if (!m || !plan_out) ARKMI_FAIL(ARKMI_INVALID_USAGE, "null argument");
        std::unique_ptr<ark::Planner> planner;
        if (arch) planner = std::make_unique<ark::Planner>(m->model, std::string(arch), num_processors);
        else planner = std::make_unique<ark::Planner>(m->model, device_id);
        for (int i = 0; i < n_rules; ++i) {
            arkmi_config_rule fn = rules[i];
            void *user = rule_users ? rule_users[i] : nullptr;
            planner->install_config_rule([fn, user](const std::string &op, const std::string &a) {
                const char *r = fn(op.c_str(), a.c_str(), user);
                return std::string(r ? r : "");
            });
        }
        *plan_out = dup_string(planner->plan(pretty != 0));
    });
}

}  // extern "C"
