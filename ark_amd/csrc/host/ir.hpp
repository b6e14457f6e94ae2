// Internal model IR behind the public ark:: handles: data types, buffers,
// tensor views, ops, graph nodes, plus error/log helpers.
//
// Behavioural reference: ark/model/{model_tensor,model_buffer,model_offset,
// model_op,model_op_arg,model_graph_impl}.cpp.  Unlike the reference, which has
// one C++ class per op type, an op here is a plain record (type name, tensors,
// args); per-type behaviour lives in function tables (host/ops.cpp).
#pragma once
#include <ark/log.hpp>
#include <unistd.h>

#include <ark/dims.hpp>
#include <ark/data_type.hpp>
#include <ark/error.hpp>
#include <ark/model_graph.hpp>
#include <ark/tensor.hpp>
#include <iostream>
#include <map>
#include <memory>
#include <set>
#include <sstream>
#include <string>
#include <vector>

#include "json.hpp"

namespace ark {

using Json = ::arkmi::Json;

// ---- errors and logging: "ARK <pid> <LEVEL> file:line message" -----------------
LogLevel log_level();

template <typename... Args>
std::string format_message(const char *level, const char *file, int line, Args &&...args) {
    std::ostringstream ss;
    std::string f(file);
    size_t pos = f.rfind("csrc/");
    if (pos != std::string::npos) f = f.substr(pos + 5);
    ss << "ARK " << ::getpid() << ' ' << level << ' ' << f << ':' << line << ' ';
    (ss << ... << args);
    return ss.str();
}

#define ARK_ERR(Type, ...) \
    throw ::ark::Type(::ark::format_message("ERROR", __FILE__, __LINE__, __VA_ARGS__))

#define ARK_LOG(level, ...)                                                                  \
    do {                                                                                     \
        if (::ark::level >= ::ark::log_level())                                              \
            std::clog << ::ark::format_message(#level, __FILE__, __LINE__, __VA_ARGS__) << '\n'; \
    } while (0)

// ---- environment (ark/env.cpp:10-66) -----------------------------------------------
struct Env {
    std::string log_level;          // ARK_LOG_LEVEL (INFO)
    std::string path_root_dir;      // ARK_ROOT
    std::string path_tmp_dir;       // ARK_TMP (/tmp/ark)
    bool keep_tmp;                  // ARK_KEEP_TMP (1)
    int num_ranks_per_host;         // ARK_NUM_RANKS_PER_HOST (8)
    bool ignore_binary_cache;       // ARK_IGNORE_BINARY_CACHE (1)
    std::string enforce_plan_path;  // ARK_ENFORCE_PLAN_PATH ("")
};
const Env &get_env();
void reload_env();

// ---- architectures (ark/arch.cpp:12-91) ---------------------------------------------
class Arch {
   public:
    explicit Arch(const std::string &name);
    const std::string &name() const { return name_; }
    // "ROCM_950" belongs to "ROCM" and "ANY"; every arch belongs to "ANY".
    bool belongs_to(const std::string &family) const;
    // Throws UnsupportedError for names outside the known list.
    static Arch from_name(const std::string &name);

   private:
    std::string name_;
    std::vector<std::string> parts_;
};

// ---- data types ----------------------------------------------------------------------
class ModelDataT {
   public:
    ModelDataT(const std::string &name, size_t bytes, int code)
        : name_(name), bytes_(bytes), code_(code) {}
    const std::string &type_name() const { return name_; }
    size_t bytes() const { return bytes_; }
    int code() const { return code_; }  // arkmi_dtype, -1 for NONE

   private:
    std::string name_;
    size_t bytes_;
    int code_;
};

// ---- buffers / tensors -----------------------------------------------------------------
class ModelBuffer {
   public:
    explicit ModelBuffer(int rank = -1);
    ModelBuffer(size_t id, int rank) : id_(id), rank_(rank) {}
    size_t id() const { return id_; }
    int rank() const { return rank_; }
    Json serialize() const;
    static std::shared_ptr<ModelBuffer> deserialize(const Json &j);
    // Process-global id counter; tests reset it to reproduce golden files.
    static void reset_ids(size_t next = 0);
    // Moves the counter past `id` (ids read from a file must not be handed out again).
    static void reserve_id(size_t id);

   private:
    size_t id_;
    int rank_;
};
using ModelBufferRef = std::shared_ptr<ModelBuffer>;

class ModelTensor {
   public:
    ModelTensor(ModelDataType data_type, ModelBufferRef buffer, const Dims &shape,
                const Dims &strides = {}, const Dims &offsets = {}, const Dims &padded_shape = {});
    ModelTensor(const ModelTensor &other);  // fresh id, same view of the same buffer

    size_t id() const { return id_; }
    ModelDataType data_type() const { return data_type_; }
    ModelBufferRef buffer() const { return buffer_; }
    const Dims &shape() const { return shape_; }
    const Dims &strides() const { return strides_; }
    const Dims &offsets() const { return offsets_; }
    const Dims &padded_shape() const { return padded_shape_; }
    size_t shape_bytes() const;
    // Byte offset of the view's first element inside its buffer
    // (ark/model/model_offset.cpp:13-27).
    size_t byte_offset() const;
    // Bytes the buffer must have to hold this view: prod(strides) * elem.
    size_t buffer_bytes() const;

    Json serialize() const;
    static std::shared_ptr<ModelTensor> deserialize(const Json &j);
    static void reset_ids(size_t next = 0);
    static void reserve_id(size_t id);

   private:
    size_t id_;
    ModelDataType data_type_;
    ModelBufferRef buffer_;
    Dims shape_, strides_, offsets_, padded_shape_;
};

// ---- op arguments ------------------------------------------------------------------------
struct ModelOpArg {
    enum Kind { INT, UINT32, INT64, UINT64, BOOL, FLOAT, DIMS } kind = INT;
    int64_t i = 0;
    float f = 0.f;
    Dims dims;
    ModelOpArg() = default;
    ModelOpArg(int v) : kind(INT), i(v) {}
    ModelOpArg(bool v) : kind(BOOL), i(v) {}
    ModelOpArg(float v) : kind(FLOAT), f(v) {}
    ModelOpArg(const Dims &d) : kind(DIMS), dims(d) {}
    Json serialize() const;  // {"BOOL":false} style
    static ModelOpArg deserialize(const Json &j);
};

// ---- ops --------------------------------------------------------------------------------------
class ModelOp {
   public:
    ModelOp(const std::string &type, bool is_virtual = false) : type_(type), virtual_(is_virtual) {}
    const std::string &type() const { return type_; }
    const std::string &name() const { return name_; }
    void set_name(const std::string &n) { name_ = n; }
    bool is_virtual() const { return virtual_; }
    const std::vector<ModelTensorRef> &read_tensors() const { return read_; }
    const std::vector<ModelTensorRef> &write_tensors() const { return write_; }
    const std::vector<ModelTensorRef> &result_tensors() const { return result_; }
    // read + write tensors, deduplicated, ordered by tensor id
    std::vector<ModelTensorRef> input_tensors() const;
    const std::map<std::string, ModelOpArg> &args() const { return args_; }
    // inputs and results must not overlap
    void verify() const;

    Json serialize() const;
    static std::shared_ptr<ModelOp> deserialize(const Json &j);
    static bool known_type(const std::string &type);

    std::vector<ModelTensorRef> read_, write_, result_;
    std::map<std::string, ModelOpArg> args_;

   private:
    std::string type_, name_;
    bool virtual_;
};
using ModelOpRef = std::shared_ptr<ModelOp>;

// ---- graph --------------------------------------------------------------------------------------
// Insertion-ordered set (ark/unique_list.hpp).
template <typename T>
class UniqueList {
   public:
    void push_back(const T &v) {
        if (!contains(v)) items_.push_back(v);
    }
    void erase(const T &v) {
        for (auto it = items_.begin(); it != items_.end(); ++it)
            if (*it == v) {
                items_.erase(it);
                return;
            }
    }
    bool contains(const T &v) const {
        for (const auto &x : items_)
            if (x == v) return true;
        return false;
    }
    size_t index(const T &v) const {
        for (size_t i = 0; i < items_.size(); ++i)
            if (items_[i] == v) return i;
        return (size_t)-1;
    }
    bool empty() const { return items_.empty(); }
    size_t size() const { return items_.size(); }
    auto begin() const { return items_.begin(); }
    auto end() const { return items_.end(); }
    const T &operator[](size_t i) const { return items_[i]; }

   private:
    std::vector<T> items_;
};

class ModelNode {
   public:
    ModelOpRef op;
    UniqueList<ModelNodeRef> consumers;
    UniqueList<ModelNodeRef> producers;
    std::map<std::string, Json> context;  // snapshot of the context stack
};

class ContextStack {
   public:
    void push(const std::string &key, const Json &value) { store_[key].push_back(value); }
    void pop(const std::string &key);
    bool has(const std::string &key) const { return store_.count(key) > 0; }
    Json get(const std::string &key) const;
    std::map<std::string, Json> snapshot() const;

   private:
    std::map<std::string, std::vector<Json>> store_;
};

class ModelGraph::Impl {
   public:
    Impl(int rank, int world_size)
        : rank_(rank), world_size_(world_size), context_(std::make_shared<ContextStack>()) {}
    Impl(const Impl &other) { *this = other; }
    Impl &operator=(const Impl &other);

    // Names the op (snake_case of its type when `name` is empty, "_<n>" suffix
    // on repeats) and adds it to the graph.
    ModelOpRef add_named_op(ModelOpRef op, const std::string &name);
    void compress_nodes();
    bool verify() const;
    std::string serialize(bool pretty) const;
    // with_context adds each node's context snapshot as a "Context" object
    Json to_json(bool with_context = false) const;
    // Rebuilds a graph from serialize()'s output (optionally carrying the
    // per-node "Context" objects this backend adds).
    static std::unique_ptr<Impl> deserialize(const Json &j);

    int rank_, world_size_;
    bool compressed_ = false;
    UniqueList<ModelNodeRef> nodes_;
    std::multiset<std::string> op_names_;
    std::map<ModelTensorRef, ModelOpRef> producer_of_;
    std::map<ModelOpRef, ModelNodeRef> node_of_;
    std::shared_ptr<ContextStack> context_;

   private:
    ModelNodeRef add_op(ModelOpRef op);
    void remove_node(ModelNodeRef node);
    void remove_virtual(UniqueList<ModelNodeRef> &seen, const std::vector<ModelNodeRef> &boundary);
    Json node_json(const ModelNodeRef &node, bool with_context) const;
};

// ---- small utilities (ark/utils/utils_string.cpp, utils_math.cpp) -----------------------------
bool is_pascal(const std::string &s);
std::string pascal_to_snake(const std::string &s);
inline int64_t div_up(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Verifies the shape of a plan / model JSON (ark/model/model_json.cpp:24-101,222-284);
// throws PlanError / ModelError.
void verify_plan_json(const Json &plan);
void verify_model_json(const Json &model);

}  // namespace ark
