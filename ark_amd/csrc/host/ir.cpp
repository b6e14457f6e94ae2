#include "ir.hpp"

#include <algorithm>
#include <cctype>
#include <cstdlib>

namespace ark {

// ---------------------------------------------------------------------------
// environment / logging
// ---------------------------------------------------------------------------
static std::string env_str(const char *name, const std::string &dflt) {
    const char *v = std::getenv(name);
    return v ? std::string(v) : dflt;
}
static bool env_flag(const char *name, bool dflt) {
    const char *v = std::getenv(name);
    return v ? std::string(v) == "1" : dflt;
}

static std::unique_ptr<Env> g_env;

void reload_env() {
    auto e = std::make_unique<Env>();
    e->log_level = env_str("ARK_LOG_LEVEL", "INFO");
    e->path_root_dir = env_str("ARK_ROOT", "/usr/local/ark");
    e->path_tmp_dir = env_str("ARK_TMP", "/tmp/ark");
    e->keep_tmp = env_flag("ARK_KEEP_TMP", true);
    const char *n = std::getenv("ARK_NUM_RANKS_PER_HOST");
    e->num_ranks_per_host = n ? std::atoi(n) : 8;
    e->ignore_binary_cache = env_flag("ARK_IGNORE_BINARY_CACHE", true);
    e->enforce_plan_path = env_str("ARK_ENFORCE_PLAN_PATH", "");
    g_env = std::move(e);
}

const Env &get_env() {
    if (!g_env) reload_env();
    return *g_env;
}

LogLevel log_level() {
    const std::string &l = get_env().log_level;
    if (l == "DEBUG") return DEBUG;
    if (l == "WARN") return WARN;
    if (l == "ERROR") return ERROR;
    return INFO;
}

// ---------------------------------------------------------------------------
// strings
// ---------------------------------------------------------------------------
bool is_pascal(const std::string &s) {
    if (s.empty() || !std::isupper((unsigned char)s[0])) return false;
    return std::all_of(s.begin() + 1, s.end(), [](unsigned char c) { return std::isalnum(c); });
}

std::string pascal_to_snake(const std::string &s) {
    if (!is_pascal(s)) ARK_ERR(InvalidUsageError, "given string (", s, ") is not in Pascal case");
    std::string out;
    for (size_t i = 0; i < s.size(); ++i) {
        if (i > 0 && std::isupper((unsigned char)s[i])) out += '_';
        out += (char)std::tolower((unsigned char)s[i]);
    }
    return out;
}

// ---------------------------------------------------------------------------
// Arch
// ---------------------------------------------------------------------------
Arch::Arch(const std::string &name) : name_(name) {
    if (name == "ANY") return;
    size_t s = 0;
    while (s <= name.size()) {
        size_t u = name.find('_', s);
        if (u == std::string::npos) u = name.size();
        parts_.push_back(name.substr(s, u - s));
        s = u + 1;
    }
}

bool Arch::belongs_to(const std::string &family) const {
    Arch f(family);
    if (parts_.size() < f.parts_.size()) return false;
    for (size_t i = 0; i < f.parts_.size(); ++i)
        if (parts_[i] != f.parts_[i]) return false;
    return true;
}

Arch Arch::from_name(const std::string &name) {
    // The reference's list (arch.cpp:77-88) plus this backend's target.
    static const char *known[] = {"ANY",  "CUDA",     "CUDA_70",  "CUDA_80", "CUDA_90",
                                  "ROCM", "ROCM_90A", "ROCM_942", "ROCM_950"};
    for (const char *k : known)
        if (name == k) return Arch(name);
    ARK_ERR(UnsupportedError, "Unknown architecture type: ", name);
}

// ---------------------------------------------------------------------------
// Dims
// ---------------------------------------------------------------------------
Dims::Dims() {}
Dims::Dims(DimType d0) : data_{d0} {}
Dims::Dims(DimType d0, DimType d1) : data_{d0, d1} {}
Dims::Dims(DimType d0, DimType d1, DimType d2) : data_{d0, d1, d2} {}
Dims::Dims(DimType d0, DimType d1, DimType d2, DimType d3) : data_{d0, d1, d2, d3} {}
Dims::Dims(const Dims &other) {
    if (other.is_invalid()) ARK_ERR(InvalidUsageError, "invalid dims given");
    data_ = other.data_;
}
Dims::Dims(const std::vector<DimType> &vec) {
    if ((DimType)vec.size() > DIMS_LEN)
        ARK_ERR(InvalidUsageError, "only support dims with size <= ", DIMS_LEN, ". Given size ",
                vec.size());
    data_ = vec;
}
DimType Dims::nelems() const {
    if (has_negative()) return -1;
    if (data_.empty()) return 0;
    DimType n = 1;
    for (auto d : data_) n *= d;
    return n;
}
int Dims::ndims() const { return (int)data_.size(); }
Dims Dims::dims4() const {
    std::vector<DimType> v(DIMS_LEN - data_.size(), 1);
    v.insert(v.end(), data_.begin(), data_.end());
    return Dims(v);
}
bool Dims::is_zeros() const {
    if (is_invalid()) return false;
    return std::all_of(data_.begin(), data_.end(), [](DimType d) { return d == 0; });
}
bool Dims::is_no_dim() const { return data_.empty(); }
bool Dims::has_negative() const {
    return std::any_of(data_.begin(), data_.end(), [](DimType d) { return d < 0; });
}
bool Dims::is_invalid() const { return (DimType)data_.size() > DIMS_LEN; }
const std::vector<DimType> &Dims::vector() const { return data_; }
void Dims::insert(int idx, DimType dim) {
    int nd = ndims();
    if (nd >= DIMS_LEN) ARK_ERR(InvalidUsageError, "too many dimensions: ", *this);
    if (idx > nd || -idx > nd + 1)
        ARK_ERR(InvalidUsageError, "invalid index given: ", idx, " for ", *this);
    if (idx < 0) idx += nd + 1;
    data_.insert(data_.begin() + idx, dim);
}
DimType Dims::erase(int idx) {
    int nd = ndims();
    if (idx >= nd || -idx > nd) ARK_ERR(InvalidUsageError, "invalid index given: ", idx, " for ", *this);
    if (idx < 0) idx += nd;
    DimType v = data_[idx];
    data_.erase(data_.begin() + idx);
    return v;
}
DimType &Dims::operator[](int idx) {
    int nd = ndims();
    if (idx >= nd || -idx > nd) ARK_ERR(InvalidUsageError, "invalid index given: ", idx, " for ", *this);
    return data_[idx < 0 ? idx + nd : idx];
}
const DimType &Dims::operator[](int idx) const {
    int nd = ndims();
    if (idx >= nd || -idx > nd) ARK_ERR(InvalidUsageError, "invalid index given: ", idx, " for ", *this);
    return data_[idx < 0 ? idx + nd : idx];
}
bool operator==(const Dims &a, const Dims &b) { return a.data_ == b.data_; }
bool operator!=(const Dims &a, const Dims &b) { return !(a == b); }
std::ostream &operator<<(std::ostream &os, const Dims &dims) {
    if (dims.is_invalid()) ARK_ERR(InvalidUsageError, "invalid dims given");
    os << '<';
    for (int i = 0; i < dims.ndims(); ++i) os << (i ? ", " : "") << dims[i];
    return os << '>';
}

// ---------------------------------------------------------------------------
// DataType
// ---------------------------------------------------------------------------
const DataType NONE(std::make_shared<ModelDataT>("NONE", 0, -1));
const DataType FP32(std::make_shared<ModelDataT>("FP32", 4, 0));
const DataType FP16(std::make_shared<ModelDataT>("FP16", 2, 1));
const DataType BF16(std::make_shared<ModelDataT>("BF16", 2, 2));
const DataType INT32(std::make_shared<ModelDataT>("INT32", 4, 3));
const DataType UINT32(std::make_shared<ModelDataT>("UINT32", 4, 4));
const DataType INT8(std::make_shared<ModelDataT>("INT8", 1, 5));
const DataType UINT8(std::make_shared<ModelDataT>("UINT8", 1, 6));
const DataType BYTE(std::make_shared<ModelDataT>("BYTE", 1, 7));

size_t DataType::bytes() const { return ref_->bytes(); }
const std::string &DataType::name() const { return ref_->type_name(); }
const DataType &DataType::from_name(const std::string &type_name) {
    static const DataType *all[] = {&NONE, &FP32, &FP16, &BF16, &INT32, &UINT32, &INT8, &UINT8, &BYTE};
    for (auto *d : all)
        if (d->name() == type_name) return *d;
    ARK_ERR(ModelError, "Unknown data type: ", type_name);
}

// ---------------------------------------------------------------------------
// ModelBuffer / ModelTensor
// ---------------------------------------------------------------------------
static size_t g_next_buffer_id = 0;
static size_t g_next_tensor_id = 0;

ModelBuffer::ModelBuffer(int rank) : id_(g_next_buffer_id++), rank_(rank) {}
void ModelBuffer::reset_ids(size_t next) { g_next_buffer_id = next; }
void ModelBuffer::reserve_id(size_t id) { g_next_buffer_id = std::max(g_next_buffer_id, id + 1); }

Json ModelBuffer::serialize() const {
    Json j = Json::object();
    j["Id"] = (unsigned long)id_;
    j["Rank"] = rank_;
    j["SendTags"] = Json::array();
    j["RecvTags"] = Json::array();
    return j;
}

std::shared_ptr<ModelBuffer> ModelBuffer::deserialize(const Json &j) {
    for (const char *k : {"Id", "Rank", "SendTags", "RecvTags"})
        if (!j.contains(k)) ARK_ERR(ModelError, "ModelBuffer deserialization failed: missing ", k);
    return std::make_shared<ModelBuffer>((size_t)j.at("Id").as_int(), (int)j.at("Rank").as_int());
}

ModelTensor::ModelTensor(ModelDataType data_type, ModelBufferRef buffer, const Dims &shape,
                         const Dims &strides, const Dims &offsets, const Dims &padded_shape)
    : data_type_(data_type), buffer_(buffer) {
    if (shape.is_no_dim()) {
        shape_ = Dims(1);  // a single-element constant
    } else if (shape.has_negative() || shape.nelems() == 0) {
        ARK_ERR(ModelError, "Tensor shape should consist of only positive numbers. Given: ", shape);
    } else {
        shape_ = shape;
    }
    const int nd = shape_.ndims();
    if (padded_shape.is_no_dim()) {
        padded_shape_ = shape_;
    } else {
        if (padded_shape.ndims() != nd)
            ARK_ERR(ModelError,
                    "Tensor shape and padded shape should have the same number of dimensions. "
                    "Given: shape ", shape_, " padded_shape ", padded_shape);
        padded_shape_ = padded_shape;
    }
    for (int i = 0; i < nd; ++i)
        if (shape_[i] > padded_shape_[i])
            ARK_ERR(ModelError, "Tensor shape exceeds the padded shape. shape ", shape_,
                    " padded_shape ", padded_shape_);
    if (strides.is_no_dim()) {
        strides_ = padded_shape_;
    } else {
        if (strides.ndims() != nd)
            ARK_ERR(ModelError,
                    "Tensor shapes and strides should have the same number of dimensions. "
                    "Given: shape ", shape_, " strides ", strides);
        strides_ = strides;
    }
    if (offsets.is_no_dim()) {
        offsets_ = Dims(std::vector<DimType>(nd, 0));
    } else {
        if (offsets.ndims() != nd)
            ARK_ERR(ModelError,
                    "Tensor shape and offs should have the same number of dimensions. "
                    "Given: shape ", shape_, " offs ", offsets);
        offsets_ = offsets;
    }
    for (int i = 0; i < nd; ++i)
        if (offsets_[i] + padded_shape_[i] > strides_[i])
            ARK_ERR(ModelError, "Tensor exceeds the memory boundary. offs ", offsets_,
                    " padded_shape ", padded_shape_, " strides ", strides_);
    id_ = g_next_tensor_id++;
}

ModelTensor::ModelTensor(const ModelTensor &o)
    : id_(g_next_tensor_id++), data_type_(o.data_type_), buffer_(o.buffer_), shape_(o.shape_),
      strides_(o.strides_), offsets_(o.offsets_), padded_shape_(o.padded_shape_) {}

void ModelTensor::reset_ids(size_t next) { g_next_tensor_id = next; }
void ModelTensor::reserve_id(size_t id) { g_next_tensor_id = std::max(g_next_tensor_id, id + 1); }

size_t ModelTensor::shape_bytes() const { return shape_.nelems() * data_type_->bytes(); }

size_t ModelTensor::byte_offset() const {
    size_t off = 0, pitch = 1;
    for (int i = strides_.ndims() - 1; i >= 0; --i) {
        off += (size_t)offsets_[i] * pitch;
        pitch *= (size_t)strides_[i];
    }
    return off * data_type_->bytes();
}

size_t ModelTensor::buffer_bytes() const { return (size_t)strides_.nelems() * data_type_->bytes(); }

Json ModelTensor::serialize() const {
    Json j = Json::object();
    j["Id"] = (unsigned long)id_;
    j["DataType"] = data_type_->type_name();
    j["Shape"] = Json(shape_.vector());
    j["Strides"] = Json(strides_.vector());
    j["Offsets"] = Json(offsets_.vector());
    j["PaddedShape"] = Json(padded_shape_.vector());
    j["Buffer"] = buffer_->serialize();
    return j;
}

std::shared_ptr<ModelTensor> ModelTensor::deserialize(const Json &j) {
    for (const char *k : {"DataType", "Buffer", "Shape", "Strides", "Offsets", "PaddedShape", "Id"})
        if (!j.contains(k)) ARK_ERR(ModelError, "ModelTensor deserialization failed: missing ", k);
    auto t = std::make_shared<ModelTensor>(
        DataType::from_name(j.at("DataType").as_string()).ref(),
        ModelBuffer::deserialize(j.at("Buffer")), Dims(j.at("Shape").as_int_vector()),
        Dims(j.at("Strides").as_int_vector()), Dims(j.at("Offsets").as_int_vector()),
        Dims(j.at("PaddedShape").as_int_vector()));
    g_next_tensor_id--;  // deserialisation does not consume a fresh id
    t->id_ = (size_t)j.at("Id").as_int();
    return t;
}

size_t Tensor::id() const { return ref_ ? ref_->id() : (size_t)-1; }
Dims Tensor::shape() const { return ref_ ? ref_->shape() : Dims(); }
Dims Tensor::strides() const { return ref_ ? ref_->strides() : Dims(); }
Dims Tensor::offsets() const { return ref_ ? ref_->offsets() : Dims(); }
Dims Tensor::padded_shape() const { return ref_ ? ref_->padded_shape() : Dims(); }
const DataType &Tensor::data_type() const {
    if (!ref_) return NONE;
    return DataType::from_name(ref_->data_type()->type_name());
}
std::ostream &operator<<(std::ostream &os, const Tensor &tensor) {
    if (tensor.is_null()) return os << "null";
    return os << tensor.ref()->serialize().dump();
}

// ---------------------------------------------------------------------------
// ModelOpArg / ModelOp
// ---------------------------------------------------------------------------
Json ModelOpArg::serialize() const {
    Json j = Json::object();
    switch (kind) {
        case INT: j["INT"] = (long long)i; break;
        case UINT32: j["UINT32"] = (unsigned long long)i; break;
        case INT64: j["INT64"] = (long long)i; break;
        case UINT64: j["UINT64"] = (unsigned long long)i; break;
        case BOOL: j["BOOL"] = (bool)i; break;
        case FLOAT: j["FLOAT"] = f; break;  // widened to double, shortest round trip
        case DIMS: j["DIMS"] = Json(dims.vector()); break;
    }
    return j;
}

ModelOpArg ModelOpArg::deserialize(const Json &j) {
    if (!j.is_object() || j.size() != 1)
        ARK_ERR(ModelError, "Tried to deserialize an unknown type of argument: ", j.dump());
    const auto &m = j.items()[0];
    const std::string &t = m.first;
    ModelOpArg a;
    try {
        if (t == "INT") { a.kind = INT; a.i = m.second.as_int(); }
        else if (t == "UINT32") { a.kind = UINT32; a.i = m.second.as_int(); }
        else if (t == "INT64") { a.kind = INT64; a.i = m.second.as_int(); }
        else if (t == "UINT64") { a.kind = UINT64; a.i = m.second.as_int(); }
        else if (t == "BOOL") { a.kind = BOOL; a.i = m.second.as_bool(); }
        else if (t == "FLOAT") { a.kind = FLOAT; a.f = (float)m.second.as_double(); }
        else if (t == "DIMS") { a.kind = DIMS; a.dims = Dims(m.second.as_int_vector()); }
        else ARK_ERR(ModelError, "Tried to deserialize an unknown type of argument: ", j.dump());
    } catch (const BaseError &) {
        throw;
    } catch (const std::exception &e) {
        ARK_ERR(ModelError, "Failed to deserialize `", j.dump(), "`: ", e.what());
    }
    return a;
}

std::vector<ModelTensorRef> ModelOp::input_tensors() const {
    std::vector<ModelTensorRef> v(read_);
    v.insert(v.end(), write_.begin(), write_.end());
    std::sort(v.begin(), v.end(),
              [](const ModelTensorRef &a, const ModelTensorRef &b) { return a->id() < b->id(); });
    v.erase(std::unique(v.begin(), v.end()), v.end());
    return v;
}

void ModelOp::verify() const {
    for (const auto &t : input_tensors())
        if (!t->buffer()) ARK_ERR(InternalError, "input tensor buffer is null");
    for (const auto &t : result_) {
        if (!t->buffer()) ARK_ERR(InternalError, "output tensor buffer is null");
        for (const auto &i : input_tensors())
            if (i == t) ARK_ERR(InternalError, "cyclic dependency detected");
    }
}

bool ModelOp::known_type(const std::string &type) {
    // Registered types of the reference (ark/model/model_op.cpp:54-86) plus the
    // fused row ops and SiluMul of this backend.
    static const std::set<std::string> types = {
        "Add", "Cast", "Copy", "Div", "Embedding", "Exp", "Gelu", "Matmul", "Mul", "Noop", "Recv",
        "ReduceMax", "ReduceMean", "ReduceSum", "Relu", "Reshape", "Rope", "Rsqrt", "ScalarAdd",
        "ScalarAssign", "ScalarMul", "Send", "SendDone", "Sigmoid", "Sqrt", "Sub", "Tensor",
        "Transpose", "SendPacket", "RecvPacket", "RecvReduceSendPacket", "RecvReduceSend",
        "DeviceSync", "Softmax", "Layernorm", "Rmsnorm", "SiluMul", "Attention", "MatmulSwiglu"};
    return types.count(type) > 0;
}

Json ModelOp::serialize() const {
    Json j = Json::object();
    j["Type"] = type_;
    j["Name"] = name_;
    j["IsVirtual"] = virtual_;
    auto list = [](const std::vector<ModelTensorRef> &ts) {
        Json a = Json::array();
        for (const auto &t : ts) a.push_back(t->serialize());
        return a;
    };
    j["ReadTensors"] = list(read_);
    j["WriteTensors"] = list(write_);
    j["ResultTensors"] = list(result_);
    Json args = Json::object();
    for (const auto &kv : args_) args[kv.first] = kv.second.serialize();  // std::map: sorted names
    j["Args"] = args;
    return j;
}

std::shared_ptr<ModelOp> ModelOp::deserialize(const Json &j) {
    for (const char *k :
         {"Type", "Name", "IsVirtual", "ReadTensors", "WriteTensors", "ResultTensors", "Args"})
        if (!j.contains(k)) ARK_ERR(ModelError, "ModelOp deserialization failed: missing ", k);
    const std::string &type = j.at("Type").as_string();
    if (!known_type(type)) ARK_ERR(ModelError, "Unknown model op type: ", type);
    auto op = std::make_shared<ModelOp>(type, j.at("IsVirtual").as_bool());
    op->set_name(j.at("Name").as_string());
    // Tensors with equal ids inside one op are the same object.
    std::map<size_t, ModelTensorRef> seen;
    auto load = [&](const Json &arr, std::vector<ModelTensorRef> &dst) {
        for (const auto &t : arr.elements()) {
            auto ref = ModelTensor::deserialize(t);
            auto it = seen.find(ref->id());
            if (it != seen.end()) ref = it->second;
            else seen[ref->id()] = ref;
            dst.push_back(ref);
        }
    };
    load(j.at("ReadTensors"), op->read_);
    load(j.at("WriteTensors"), op->write_);
    load(j.at("ResultTensors"), op->result_);
    for (const auto &m : j.at("Args").items()) op->args_[m.first] = ModelOpArg::deserialize(m.second);
    return op;
}

// ---------------------------------------------------------------------------
// JSON shape verification
// ---------------------------------------------------------------------------
template <typename E>
static void need(const std::string &what, const Json &j, std::initializer_list<const char *> fields,
                 std::initializer_list<const char *> arrays) {
    for (const char *f : fields)
        if (!j.contains(f)) throw E(format_message("ERROR", __FILE__, __LINE__, what, ": ", f,
                                                   " not found. Given: ", j.dump()));
    for (const char *f : arrays)
        if (!j.at(f).is_array())
            throw E(format_message("ERROR", __FILE__, __LINE__, what, ": ", f,
                                   " is not an array. Given: ", j.dump()));
}

template <typename E>
static void verify_tensor_json(const Json &j) {
    need<E>("TensorJson", j, {"Id", "DataType", "Shape", "Strides", "Offsets", "PaddedShape", "Buffer"},
            {"Shape", "Strides", "Offsets", "PaddedShape"});
    need<E>("BufferJson", j.at("Buffer"), {"Id", "Rank", "SendTags", "RecvTags"},
            {"SendTags", "RecvTags"});
}

template <typename E>
static void verify_op_json(const Json &j, bool need_config) {
    need<E>("OpJson", j,
            {"Type", "Name", "IsVirtual", "ReadTensors", "WriteTensors", "ResultTensors", "Args"},
            {"ReadTensors", "WriteTensors", "ResultTensors"});
    if (need_config) need<E>("OpJson", j, {"Config"}, {});
    for (const char *k : {"ReadTensors", "WriteTensors", "ResultTensors"})
        for (const auto &t : j.at(k).elements()) verify_tensor_json<E>(t);
}

void verify_model_json(const Json &j) {
    need<ModelError>("ModelJson", j, {"Rank", "WorldSize", "Nodes"}, {"Nodes"});
    for (const auto &n : j.at("Nodes").elements()) {
        need<ModelError>("NodeJson", n, {"Id", "ProducerNodeIds", "ConsumerNodeIds", "Op"},
                         {"ProducerNodeIds", "ConsumerNodeIds"});
        verify_op_json<ModelError>(n.at("Op"), false);
    }
}

void verify_plan_json(const Json &j) {
    for (const char *f : {"Rank", "WorldSize", "Architecture", "NumProcessors",
                          "NumWarpsPerProcessor", "TaskInfos", "ProcessorGroups"})
        if (!j.contains(f)) ARK_ERR(PlanError, f, " not found");
    if (!j.at("TaskInfos").is_array()) ARK_ERR(PlanError, "TaskInfos is not an array");
    if (!j.at("ProcessorGroups").is_array()) ARK_ERR(PlanError, "ProcessorGroups is not an array");
    for (const auto &ti : j.at("TaskInfos").elements()) {
        need<PlanError>("TaskInfoJson", ti, {"Id", "NumWarps", "SramBytes", "Ops"}, {"Ops"});
        for (const auto &op : ti.at("Ops").elements()) verify_op_json<PlanError>(op, true);
    }
    for (const auto &pg : j.at("ProcessorGroups").elements()) {
        need<PlanError>("ProcessorGroupJson", pg, {"ProcessorRange", "ResourceGroups"},
                        {"ProcessorRange", "ResourceGroups"});
        for (const auto &rg : pg.at("ResourceGroups").elements()) {
            need<PlanError>("ResourceGroupJson", rg,
                            {"ProcessorRange", "WarpRange", "SramRange", "TaskGroups"},
                            {"ProcessorRange", "WarpRange", "SramRange", "TaskGroups"});
            for (const auto &tg : rg.at("TaskGroups").elements())
                need<PlanError>("TaskGroupJson", tg, {"TaskId", "TaskRange", "Granularity"},
                                {"TaskRange"});
        }
    }
}

// ---------------------------------------------------------------------------
// graph
// ---------------------------------------------------------------------------
void ContextStack::pop(const std::string &key) {
    auto it = store_.find(key);
    if (it == store_.end() || it->second.empty()) ARK_ERR(InternalError, "context stack is empty");
    it->second.pop_back();
    if (it->second.empty()) store_.erase(it);
}

Json ContextStack::get(const std::string &key) const {
    auto it = store_.find(key);
    return (it == store_.end() || it->second.empty()) ? Json() : it->second.back();
}

std::map<std::string, Json> ContextStack::snapshot() const {
    std::map<std::string, Json> cur;
    for (const auto &kv : store_)
        if (!kv.second.empty()) cur[kv.first] = kv.second.back();
    return cur;
}

ModelGraph::Impl &ModelGraph::Impl::operator=(const Impl &other) {
    std::map<ModelNodeRef, ModelNodeRef> twin;
    nodes_ = UniqueList<ModelNodeRef>();
    for (const auto &n : other.nodes_) {
        auto c = std::make_shared<ModelNode>();
        c->op = n->op;
        c->context = n->context;
        twin[n] = c;
        nodes_.push_back(c);
    }
    for (const auto &n : other.nodes_) {
        auto c = twin.at(n);
        for (const auto &p : n->producers) c->producers.push_back(twin.at(p));
        for (const auto &q : n->consumers) c->consumers.push_back(twin.at(q));
    }
    node_of_.clear();
    for (const auto &kv : other.node_of_) node_of_[kv.first] = twin.at(kv.second);
    producer_of_ = other.producer_of_;
    op_names_ = other.op_names_;
    rank_ = other.rank_;
    world_size_ = other.world_size_;
    compressed_ = other.compressed_;
    context_ = std::make_shared<ContextStack>(*other.context_);
    return *this;
}

ModelOpRef ModelGraph::Impl::add_named_op(ModelOpRef op, const std::string &name) {
    std::string n = name.empty() ? pascal_to_snake(op->type()) : name;
    size_t count = op_names_.count(n);
    op_names_.insert(n);
    if (count > 0) n += "_" + std::to_string(count);
    op->set_name(n);
    add_op(op);
    return op;
}

ModelNodeRef ModelGraph::Impl::add_op(ModelOpRef op) {
    for (const auto &t : op->input_tensors()) {
        if (producer_of_.find(t) == producer_of_.end()) {
            // An input nobody produced yet is declared by an implicit virtual
            // "Tensor" op (model_graph_impl.cpp:181-190).
            auto decl = std::make_shared<ModelOp>("Tensor", true);
            decl->result_ = {t};
            add_op(decl);
        }
    }
    for (const auto &t : op->result_tensors()) {
        if (producer_of_.find(t) != producer_of_.end())
            ARK_ERR(InternalError, "Tensor has already been produced by an op. ",
                    t->serialize().dump());
        producer_of_[t] = op;
    }
    auto node = std::make_shared<ModelNode>();
    node->op = op;
    node_of_[op] = node;
    for (const auto &t : op->input_tensors()) {
        auto producer = node_of_.at(producer_of_.at(t));
        node->producers.push_back(producer);
        producer->consumers.push_back(node);
    }
    node->context = context_->snapshot();
    nodes_.push_back(node);
    return node;
}

void ModelGraph::Impl::remove_node(ModelNodeRef node) {
    if (!nodes_.contains(node))
        ARK_ERR(InternalError, "attempted to remove a node that is not in the graph");
    for (const auto &c : node->consumers) c->producers.erase(node);
    for (const auto &p : node->producers) p->consumers.erase(node);
    for (const auto &c : node->consumers)
        for (const auto &p : node->producers) {
            c->producers.push_back(p);
            p->consumers.push_back(c);
        }
    auto it = node_of_.find(node->op);
    if (it != node_of_.end() && it->second == node) node_of_.erase(it);
    nodes_.erase(node);
}

void ModelGraph::Impl::compress_nodes() {
    if (compressed_) return;
    std::vector<ModelNodeRef> leaves;
    for (const auto &n : nodes_)
        if (n->consumers.empty()) leaves.push_back(n);
    UniqueList<ModelNodeRef> seen;
    remove_virtual(seen, leaves);
    compressed_ = true;
}

// Breadth-first from the leaves towards the producers: a producer joins the
// next frontier only when all of its other consumers were already visited, so
// each node is handled once; virtual nodes are spliced out on the way
// (model_graph_impl.cpp:255-316).
void ModelGraph::Impl::remove_virtual(UniqueList<ModelNodeRef> &seen,
                                      const std::vector<ModelNodeRef> &boundary) {
    std::vector<ModelNodeRef> frontier = boundary;
    while (!frontier.empty()) {
        std::vector<ModelNodeRef> next;
        for (const auto &node : frontier) {
            if (!node->op) ARK_ERR(InternalError, "unexpected error: empty node");
            std::vector<ModelNodeRef> producers(node->producers.begin(), node->producers.end());
            for (const auto &p : producers) {
                bool ready = true;
                for (const auto &c : p->consumers)
                    if (c != node && !seen.contains(c)) {
                        ready = false;
                        break;
                    }
                if (!ready) continue;
                if (seen.contains(p)) ARK_ERR(InternalError, "circular dependency detected");
                next.push_back(p);
            }
            if (node->op->is_virtual())
                remove_node(node);
            else
                seen.push_back(node);
        }
        frontier = std::move(next);
    }
}

bool ModelGraph::Impl::verify() const {
    try {
        for (const auto &n : nodes_) {
            if (!n->op) return false;
            auto it = node_of_.find(n->op);
            if (it == node_of_.end() || it->second != n) return false;
            n->op->verify();
            for (const auto &t : n->op->result_tensors()) {
                auto p = producer_of_.find(t);
                if (p == producer_of_.end() || p->second != n->op) return false;
            }
            for (const auto &t : n->op->input_tensors())
                if (producer_of_.find(t) == producer_of_.end()) return false;
            for (const auto &p : n->producers)
                if (!p->consumers.contains(n)) return false;
            for (const auto &c : n->consumers)
                if (!c->producers.contains(n)) return false;
        }
        verify_model_json(Json::parse(serialize(false)));
    } catch (const BaseError &) {
        return false;
    }
    return true;
}

Json ModelGraph::Impl::node_json(const ModelNodeRef &node, bool with_context) const {
    Json j = Json::object();
    j["Id"] = (unsigned long)nodes_.index(node);
    Json prod = Json::array(), cons = Json::array();
    for (const auto &p : node->producers) prod.push_back((unsigned long)nodes_.index(p));
    for (const auto &c : node->consumers) cons.push_back((unsigned long)nodes_.index(c));
    j["ProducerNodeIds"] = prod;
    j["ConsumerNodeIds"] = cons;
    j["Op"] = node->op->serialize();
    if (with_context) {
        Json ctx = Json::object();
        for (const auto &kv : node->context) ctx[kv.first] = kv.second;
        j["Context"] = ctx;
    }
    return j;
}

Json ModelGraph::Impl::to_json(bool with_context) const {
    Json j = Json::object();
    j["Rank"] = rank_;
    j["WorldSize"] = world_size_;
    Json nodes = Json::array();
    for (const auto &n : nodes_) nodes.push_back(node_json(n, with_context));
    j["Nodes"] = nodes;
    return j;
}

std::string ModelGraph::Impl::serialize(bool pretty) const {
    Json j = to_json();
    return pretty ? ::arkmi::dump_pretty_model(j) : j.dump();
}

std::unique_ptr<ModelGraph::Impl> ModelGraph::Impl::deserialize(const Json &j) {
    verify_model_json(j);
    auto g = std::make_unique<Impl>((int)j.at("Rank").as_int(), (int)j.at("WorldSize").as_int());
    // Tensors are shared between ops by id.
    std::map<size_t, ModelTensorRef> tensors;
    std::vector<ModelNodeRef> nodes;
    for (const auto &nj : j.at("Nodes").elements()) {
        auto op = ModelOp::deserialize(nj.at("Op"));
        for (auto *vec : {&op->read_, &op->write_, &op->result_})
            for (auto &t : *vec) {
                auto it = tensors.find(t->id());
                if (it != tensors.end()) t = it->second;
                else tensors[t->id()] = t;
            }
        auto node = std::make_shared<ModelNode>();
        node->op = op;
        if (nj.contains("Context"))
            for (const auto &m : nj.at("Context").items()) node->context[m.first] = m.second;
        g->node_of_[op] = node;
        for (const auto &t : op->result_tensors()) g->producer_of_[t] = op;
        g->op_names_.insert(op->name());
        g->nodes_.push_back(node);
        nodes.push_back(node);
    }
    size_t idx = 0;
    for (const auto &nj : j.at("Nodes").elements()) {
        auto &node = nodes[idx++];
        for (const auto &p : nj.at("ProducerNodeIds").elements())
            node->producers.push_back(nodes.at((size_t)p.as_int()));
        for (const auto &c : nj.at("ConsumerNodeIds").elements())
            node->consumers.push_back(nodes.at((size_t)c.as_int()));
    }
    return g;
}

}  // namespace ark
