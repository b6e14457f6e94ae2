// ark::Model op builders: shape inference, validation and graph insertion.
//
// Each builder restates the rules of the matching reference op class
// (file:line cited per function); ops are plain ModelOp records here.
#include <ark/context.hpp>
#include <ark/model.hpp>
#include <ark/planner.hpp>

#include "ir.hpp"
#include "ops.hpp"

namespace ark {

// ---------------------------------------------------------------------------
// checks shared by the builders (ark/ops/ops_common.cpp:13-93)
// ---------------------------------------------------------------------------
namespace {

void check_null(const ModelTensorRef &t) {
    if (!t) ARK_ERR(ModelError, "tensor is null");
}
void check_same_dtype(const ModelTensorRef &a, const ModelTensorRef &b) {
    if (a->data_type() != b->data_type())
        ARK_ERR(ModelError, "data types mismatch: ", a->data_type()->type_name(),
                " != ", b->data_type()->type_name());
}
void check_dtype(const ModelTensorRef &a, const ModelDataType &dt) {
    if (a->data_type() != dt)
        ARK_ERR(ModelError, "data types mismatch: ", a->data_type()->type_name(),
                " != ", dt->type_name());
}
void check_shape(const ModelTensorRef &t, const Dims &shape) {
    if (t->shape() != shape) ARK_ERR(ModelError, "shape mismatch: ", t->shape(), " != ", shape);
}
void check_padded_shape(const ModelTensorRef &t, const Dims &shape) {
    if (t->padded_shape() != shape)
        ARK_ERR(ModelError, "padded shape mismatch: ", t->padded_shape(), " != ", shape);
}

ModelTensorRef fresh(const ModelDataType &dt, const Dims &shape, const Dims &padded = {}) {
    return std::make_shared<ModelTensor>(dt, std::make_shared<ModelBuffer>(), shape, Dims{}, Dims{},
                                         padded);
}

// An op with one output view: reads `reads`, writes `output`, and yields a
// new tensor object (fresh id) that aliases the output view.
ModelOpRef compute_op(const std::string &type, std::vector<ModelTensorRef> reads,
                      ModelTensorRef output) {
    auto op = std::make_shared<ModelOp>(type);
    op->read_ = std::move(reads);
    op->write_ = {output};
    op->result_ = {std::make_shared<ModelTensor>(*output)};
    return op;
}

// Virtual "Tensor" op: a view on `buffer` (ark/ops/ops_tensor.cpp:11-25).
ModelOpRef view_op(ModelBufferRef buffer, const Dims &shape, const ModelDataType &dt,
                   const Dims &strides, const Dims &offsets, const Dims &padded,
                   std::vector<ModelTensorRef> reads) {
    auto op = std::make_shared<ModelOp>("Tensor", true);
    if (!buffer) buffer = std::make_shared<ModelBuffer>();
    op->result_ = {std::make_shared<ModelTensor>(dt, buffer, shape, strides, offsets, padded)};
    op->read_ = std::move(reads);
    op->verify();
    return op;
}

}  // namespace

Dims broadcast_shape(const Dims &a, const Dims &b) {
    std::vector<DimType> rev;
    int nd = std::max(a.ndims(), b.ndims());
    for (int i = 1; i <= nd; ++i) {
        DimType d1 = (i - 1 < a.ndims()) ? a[-i] : 1;
        DimType d2 = (i - 1 < b.ndims()) ? b[-i] : 1;
        if (d1 == d2 || d2 == 1) rev.push_back(d1);
        else if (d1 == 1) rev.push_back(d2);
        else ARK_ERR(ModelError, "input and other cannot be broadcasted: ", a, ", ", b);
    }
    return Dims(std::vector<DimType>(rev.rbegin(), rev.rend()));
}

// M, N, K of a matmul from operand shapes (ark/ops/ops_matmul.cpp:13-42).
Dims matmul_problem_size(const Dims &in, const Dims &other, bool trans_in, bool trans_other) {
    if (in.ndims() < 1 || other.ndims() < 1) ARK_ERR(InternalError, "unexpected");
    DimType m = (in.ndims() == 1) ? 1 : in[-2];
    DimType n = (other.ndims() == 1) ? 1 : other[-1];
    DimType k = in[-1];
    DimType k2 = (other.ndims() == 1) ? other[0] : other[-2];
    if (trans_in) std::swap(m, k);
    if (trans_other) std::swap(n, k2);
    if (k != k2) ARK_ERR(ModelError, "padded inner dimensions mismatch: ", k, " and ", k2);
    return Dims(m, n, k);
}

// Output shape with NumPy broadcasting of the batch dims (ops_matmul.cpp:44-70).
static Dims matmul_output_shape(const Dims &in, const Dims &other, bool ti, bool to) {
    Dims mnk = matmul_problem_size(in, other, ti, to);
    int nd = std::max(in.ndims(), other.ndims());
    if (nd < 3) return Dims(mnk[0], mnk[1]);
    Dims i4 = in.dims4(), o4 = other.dims4();
    Dims nc = broadcast_shape(Dims(i4[0], i4[1]), Dims(o4[0], o4[1]));
    if (nd == 4) return Dims(nc[0], nc[1], mnk[0], mnk[1]);
    return Dims(nc[1], mnk[0], mnk[1]);
}

// ---------------------------------------------------------------------------
// ModelGraph / Model plumbing
// ---------------------------------------------------------------------------
ModelGraph::ModelGraph(int rank, int world_size) : impl_(std::make_unique<Impl>(rank, world_size)) {}
ModelGraph::ModelGraph(const ModelGraph &other) : impl_(std::make_unique<Impl>(*other.impl_)) {}
ModelGraph::~ModelGraph() = default;
ModelGraph &ModelGraph::operator=(const ModelGraph &other) {
    *impl_ = *other.impl_;
    return *this;
}
int ModelGraph::rank() const { return impl_->rank_; }
int ModelGraph::world_size() const { return impl_->world_size_; }
void ModelGraph::compress_nodes() { impl_->compress_nodes(); }
bool ModelGraph::compressed() const { return impl_->compressed_; }
bool ModelGraph::verify() const { return impl_->verify(); }
std::string ModelGraph::serialize(bool pretty) const { return impl_->serialize(pretty); }
std::vector<ModelNodeRef> ModelGraph::nodes() const {
    return std::vector<ModelNodeRef>(impl_->nodes_.begin(), impl_->nodes_.end());
}

static size_t next_model_id() {
    static size_t id = 0;
    return id++;
}

Model::Model(int rank, int world_size) : ModelGraph(rank, world_size), id_(next_model_id()) {
    if (rank < 0 || world_size < 1 || rank >= world_size)
        ARK_ERR(ModelError, "Invalid rank ", rank, " for world size ", world_size);
}
Model::Model(const Model &other) : ModelGraph(other), id_(next_model_id()), next_tag_(other.next_tag_) {}
size_t Model::id() const { return id_; }
Model Model::compress() const {
    Model m(*this);
    m.compress_nodes();
    return m;
}
int Model::unique_tag() { return next_tag_++; }

#define ADD_OP(op, name) impl_->add_named_op((op), (name))->result_tensors()[0]

// ---------------------------------------------------------------------------
// views
// ---------------------------------------------------------------------------
Tensor Model::tensor(const Dims &shape, const DataType &data_type, const Dims &strides,
                     const Dims &offsets, const Dims &padded_shape, int rank,
                     const std::string &name) {
    if (rank != -1) {
        if (rank == this->rank()) rank = -1;
        else if (rank < 0 || rank >= this->world_size()) ARK_ERR(ModelError, "Invalid rank ", rank);
    }
    return ADD_OP(view_op(std::make_shared<ModelBuffer>(rank), shape, data_type.ref(), strides,
                          offsets, padded_shape, {}),
                  name);
}

// ark/ops/ops_refer.cpp:10-26
Tensor Model::refer(Tensor input, const Dims &shape, const Dims &strides, const Dims &offsets,
                    const Dims &padded_shape, const std::string &name) {
    check_null(input.ref());
    auto in = input.ref();
    return ADD_OP(view_op(in->buffer(), shape, in->data_type(), strides, offsets, padded_shape, {in}),
                  name);
}

// ark/ops/ops_identity.cpp:12-36
Tensor Model::identity(Tensor input, const std::vector<Tensor> &deps, const std::string &name) {
    check_null(input.ref());
    auto in = input.ref();
    std::vector<ModelTensorRef> reads{in};
    for (const auto &d : deps) {
        bool dup = false;
        for (const auto &r : reads) dup |= (r == d.ref());
        if (!dup) reads.push_back(d.ref());
    }
    return ADD_OP(view_op(in->buffer(), in->shape(), in->data_type(), in->strides(), in->offsets(),
                          in->padded_shape(), reads),
                  name);
}

// ark/ops/ops_sharding.cpp:9-34
std::vector<Tensor> Model::sharding(Tensor input, DimType axis, DimType dim_per_shard,
                                    const std::string &name) {
    check_null(input.ref());
    if (axis >= DIMS_LEN || axis < 0 || axis >= input.shape().ndims())
        ARK_ERR(ModelError, "invlaid axis value: ", axis);
    if (dim_per_shard <= 0 || (input.shape()[(int)axis] % dim_per_shard) != 0)
        ARK_ERR(ModelError, "dimension length of axis ", axis, " (", input.shape()[(int)axis],
                ") is not divided by the dimension per shard (", dim_per_shard, ").");
    std::vector<Tensor> shards;
    DimType n = input.shape()[(int)axis] / dim_per_shard;
    Dims shape = input.shape(), offs = input.offsets();
    shape[(int)axis] = dim_per_shard;
    for (DimType i = 0; i < n; ++i) {
        shards.push_back(refer(input, shape, input.strides(), offs, {},
                               name + "/shard_" + std::to_string(i)));
        offs[(int)axis] += dim_per_shard;
    }
    return shards;
}

void Model::noop(Tensor input, const std::string &name) {
    check_null(input.ref());
    auto op = std::make_shared<ModelOp>("Noop");
    op->read_ = {input.ref()};
    op->verify();
    impl_->add_named_op(op, name);
}

// Stride/offset inference of a reshaped view (results as ark/ops/ops_reshape.cpp:16-132).
//
// The rule: read innermost-first, the old and the new shape fall into runs of
// dimensions with equal element counts (a run closes as soon as the two counts
// agree).  Inside a run
//   * every old dimension but the outermost must be dense (stride == extent,
//     offset 0): only then do the run's old dimensions address one contiguous
//     axis of G = product of their strides positions;
//   * every new dimension but the outermost is dense too (stride = its extent);
//   * the outermost new dimension takes what is left of G, G / (inner new extents),
//     which must divide, and the outermost old dimension's offset, counted in
//     steps of the inner new extents (which must divide as well).
// New dimensions of extent 1 left over in front get stride 1; old ones left over
// in front must be dense.
namespace {
struct ReshapeRun {
    int old_outer, old_inner;  // old dimensions [old_outer, old_inner]
    int new_outer, new_inner;  // new dimensions [new_outer, new_inner]
};
}  // namespace

static void reshape_view(const ModelTensorRef &in, const Dims &target, bool allowzero, Dims &shape,
                         Dims &strides, Dims &offsets) {
    const Dims &old_shape = in->shape(), &old_strides = in->strides(), &old_offsets = in->offsets();
    std::vector<DimType> want;
    for (int i = 0; i < target.ndims(); ++i)
        want.push_back((target[i] == 0 && !allowzero) ? old_shape[i] : target[i]);
    if (want.empty()) want.push_back(1);  // a scalar is a one-element vector
    shape = Dims(want);
    if (shape.nelems() != old_shape.nelems())
        ARK_ERR(ModelError, "reshape from ", old_shape, " to ", target, " changes the number of elements");
    auto refuse = [&]() {
        ARK_ERR(ModelError, "reshape of a tensor with shape ", old_shape, " and strides ", old_strides, " to ", shape,
                " is not a view of the same memory (a dimension that would be merged is padded or offset); "
                "copy the tensor into a dense one first");
    };
    auto dense = [&](int i) { return old_strides[i] == old_shape[i] && old_offsets[i] == 0; };

    // cut both shapes into runs, innermost first
    std::vector<ReshapeRun> runs;
    int oi = old_shape.ndims() - 1, ni = shape.ndims() - 1;
    while (oi >= 0 && ni >= 0) {
        ReshapeRun r{oi, oi, ni, ni};
        DimType old_count = old_shape[oi], new_count = shape[ni];
        bool open = true;
        while (open) {
            if (old_count == new_count) {
                open = false;
            } else if (old_count > new_count) {
                if (r.new_outer == 0) break;
                new_count *= shape[--r.new_outer];
            } else {
                if (r.old_outer == 0) break;
                old_count *= old_shape[--r.old_outer];
            }
        }
        if (open) refuse();  // cannot happen when the element counts agree
        runs.push_back(r);
        oi = r.old_outer - 1;
        ni = r.new_outer - 1;
    }
    std::vector<DimType> new_strides((size_t)shape.ndims(), 1), new_offsets((size_t)shape.ndims(), 0);
    for (const ReshapeRun &r : runs) {
        DimType positions = 1, merged_inner = 1;  // G, and the extents of the old dimensions inside the outermost
        for (int i = r.old_inner; i >= r.old_outer; --i) {
            if (i > r.old_outer) {
                if (!dense(i)) refuse();
                merged_inner *= old_shape[i];
            }
            positions *= old_strides[i];
        }
        DimType split_inner = 1;
        for (int j = r.new_inner; j > r.new_outer; --j) {
            new_strides[(size_t)j] = shape[j];
            split_inner *= shape[j];
        }
        if (split_inner == 0 || positions % split_inner != 0) refuse();
        new_strides[(size_t)r.new_outer] = positions / split_inner;
        // The outermost old dimension's offset, in elements of the run, must be a whole
        // number of steps of the inner new extents: otherwise the view starts inside an
        // inner new dimension and no (stride, offset) pair addresses it.  (The reference
        // rounds down here and returns a view of the wrong elements.)
        const DimType lead = old_offsets[r.old_outer] * merged_inner;
        if (lead % split_inner != 0) refuse();
        new_offsets[(size_t)r.new_outer] = lead / split_inner;
    }
    for (; ni >= 0; --ni)
        if (shape[ni] != 1) refuse();
    for (; oi >= 0; --oi)
        if (old_shape[oi] != 1 || !dense(oi)) refuse();
    strides = Dims(new_strides);
    offsets = Dims(new_offsets);
}

// ark/ops/ops_reshape.cpp:153-204
Tensor Model::reshape(Tensor input, const Dims &shape, bool allowzero, const std::string &name) {
    check_null(input.ref());
    std::vector<DimType> inferred;
    int neg = -1;
    bool has_zero = false;
    DimType total = 1;
    for (int i = 0; i < shape.ndims(); ++i) {
        if (shape[i] == -1) {
            if (neg != -1) ARK_ERR(ModelError, "multiple -1 in shape: ", shape);
            neg = i;
        } else if (shape[i] < 0) {
            ARK_ERR(ModelError, "shape cannot include negative values except -1. Given: ", shape);
        } else {
            has_zero |= (shape[i] == 0);
            total *= shape[i];
        }
        inferred.push_back(shape[i]);
    }
    DimType n = input.shape().nelems();
    if (neg != -1) {
        if (has_zero)
            ARK_ERR(ModelError, "shape cannot include both 0 and -1 at the same time. Given: ", shape);
        if (n % total != 0)
            ARK_ERR(ModelError, "number of elements mismatch: reshape from ", input.shape(), " to ",
                    shape);
        inferred[neg] = n / total;
    } else if (!has_zero && n != total) {
        ARK_ERR(ModelError, "number of elements mismatch: reshape from ", input.shape(), " to ",
                shape);
    }
    Dims ns, nst, nof;
    reshape_view(input.ref(), Dims(inferred), allowzero, ns, nst, nof);
    auto in = input.ref();
    return ADD_OP(view_op(in->buffer(), ns, in->data_type(), nst, nof, {}, {in}), name);
}

// ---------------------------------------------------------------------------
// matmul (ark/ops/ops_matmul.cpp:72-98)
// ---------------------------------------------------------------------------
Tensor Model::matmul(Tensor input, Tensor other, Tensor output, bool trans_input, bool trans_other,
                     const std::string &name) {
    check_null(input.ref());
    check_null(other.ref());
    auto in = input.ref(), ot = other.ref(), out = output.ref();
    check_same_dtype(in, ot);
    Dims oshape = matmul_output_shape(in->shape(), ot->shape(), trans_input, trans_other);
    Dims opadded = matmul_output_shape(in->padded_shape(), ot->padded_shape(), trans_input, trans_other);
    if (out) {
        check_shape(out, oshape);
        check_padded_shape(out, opadded);
    } else {
        out = fresh(in->data_type(), oshape, opadded);
    }
    auto op = compute_op("Matmul", {in, ot}, out);
    op->args_["TransposeInput"] = ModelOpArg(trans_input);
    op->args_["TransposeOther"] = ModelOpArg(trans_other);
    op->verify();
    return ADD_OP(op, name);
}

// ---------------------------------------------------------------------------
// reductions (ark/ops/ops_reduce.cpp:11-49)
// ---------------------------------------------------------------------------
static ModelOpRef make_reduce(const std::string &type, ModelTensorRef in, int axis, bool keepdims,
                              ModelTensorRef out) {
    check_null(in);
    Dims reduced(in->shape());
    if (axis < 0) axis += reduced.ndims();
    if (axis < 0 || axis >= reduced.ndims()) ARK_ERR(ModelError, "invalid reduction axis ", axis);
    if (keepdims) reduced[axis] = 1;
    else reduced.erase(axis);
    if (out) {
        check_same_dtype(in, out);
        if (out->shape() != reduced)
            ARK_ERR(ModelError, "invalid output shape ", out->shape(), " with input shape ",
                    in->shape(), ", reduction axis ", axis, ", and keepdims ", keepdims);
        if (out == in)
            ARK_ERR(ModelError, "output tensor cannot be the same as input tensor for reduce_sum op");
    } else {
        out = fresh(in->data_type(), reduced);
    }
    auto op = compute_op(type, {in}, out);
    op->args_["Axis"] = ModelOpArg(axis);
    op->args_["KeepDim"] = ModelOpArg(keepdims);
    op->verify();
    return op;
}

Tensor Model::reduce_sum(Tensor input, int axis, bool keepdims, Tensor output, const std::string &name) {
    return ADD_OP(make_reduce("ReduceSum", input.ref(), axis, keepdims, output.ref()), name);
}
Tensor Model::reduce_mean(Tensor input, int axis, bool keepdims, Tensor output, const std::string &name) {
    return ADD_OP(make_reduce("ReduceMean", input.ref(), axis, keepdims, output.ref()), name);
}
Tensor Model::reduce_max(Tensor input, int axis, bool keepdims, Tensor output, const std::string &name) {
    return ADD_OP(make_reduce("ReduceMax", input.ref(), axis, keepdims, output.ref()), name);
}

// ---------------------------------------------------------------------------
// fused row ops (no reference op class; semantics from python/ark/ops.py:491-513
// and examples/llama/model.py:92-99)
// ---------------------------------------------------------------------------
static ModelOpRef make_row_op(const std::string &type, ModelTensorRef in, ModelTensorRef weight,
                              ModelTensorRef out) {
    check_null(in);
    if (out) {
        check_same_dtype(in, out);
        check_shape(out, in->shape());
    } else {
        out = fresh(in->data_type(), in->shape());
    }
    std::vector<ModelTensorRef> reads{in};
    if (weight) {
        if (weight->shape().nelems() != in->shape()[-1] || weight->shape()[-1] != in->shape()[-1])
            ARK_ERR(ModelError, "weight shape ", weight->shape(),
                    " does not match the last dimension of the input ", in->shape());
        if (weight->data_type() != FP32.ref()) check_same_dtype(in, weight);
        reads.push_back(weight);
    }
    return compute_op(type, reads, out);
}

Tensor Model::softmax(Tensor input, Tensor output, const std::string &name) {
    auto op = make_row_op("Softmax", input.ref(), nullptr, output.ref());
    op->verify();
    return ADD_OP(op, name);
}
// softmax(input * scale + mask) over the last axis: the scores -> scale -> add mask
// -> softmax chain of the reference's attention (examples/llama/model.py:426-433)
// as one op.  The mask broadcasts against the input NumPy-style.
Tensor Model::softmax(Tensor input, Tensor mask, float scale, Tensor output, const std::string &name) {
    if (mask.is_null() && scale == 1.0f) return softmax(input, output, name);
    auto op = make_row_op("Softmax", input.ref(), nullptr, output.ref());
    if (!mask.is_null()) {
        check_same_dtype(input.ref(), mask.ref());
        if (broadcast_shape(input.ref()->shape(), mask.ref()->shape()) != input.ref()->shape())
            ARK_ERR(ModelError, "mask shape ", mask.ref()->shape(), " does not broadcast to the input shape ",
                    input.ref()->shape());
        if (mask.ref()->shape()[-1] != input.ref()->shape()[-1])
            ARK_ERR(ModelError, "the mask must span the last axis of the input");
        op->read_.push_back(mask.ref());
    }
    op->args_["Scale"] = ModelOpArg(scale);
    op->verify();
    return ADD_OP(op, name);
}
Tensor Model::layernorm(Tensor input, float eps, Tensor output, const std::string &name) {
    auto op = make_row_op("Layernorm", input.ref(), nullptr, output.ref());
    op->args_["Eps"] = ModelOpArg(eps);
    op->verify();
    return ADD_OP(op, name);
}
Tensor Model::rmsnorm(Tensor input, Tensor weight, float eps, Tensor output, const std::string &name) {
    auto op = make_row_op("Rmsnorm", input.ref(), weight.ref(), output.ref());
    op->args_["Eps"] = ModelOpArg(eps);
    op->verify();
    return ADD_OP(op, name);
}

// ---------------------------------------------------------------------------
// elementwise (ark/ops/ops_broadcast.cpp:11-23,68-91)
// ---------------------------------------------------------------------------
static ModelOpRef make_unary(const std::string &type, ModelTensorRef in, ModelTensorRef out,
                             ModelDataType out_dtype = nullptr) {
    check_null(in);
    if (!out_dtype) out_dtype = in->data_type();
    if (out) check_dtype(out, out_dtype);
    else out = fresh(out_dtype, in->shape());
    check_shape(out, broadcast_shape(in->shape(), out->shape()));
    auto op = compute_op(type, {in}, out);
    op->verify();
    return op;
}

static ModelOpRef make_binary(const std::string &type, ModelTensorRef in, ModelTensorRef other,
                              ModelTensorRef out) {
    check_null(in);
    check_null(other);
    check_same_dtype(in, other);
    if (out) check_same_dtype(in, out);
    Dims oshape = broadcast_shape(in->shape(), other->shape());
    if (out) check_shape(out, oshape);
    else out = fresh(in->data_type(), oshape);
    auto op = compute_op(type, {in, other}, out);
    op->verify();
    return op;
}

Tensor Model::add(Tensor input, Tensor other, Tensor output, const std::string &name) {
    return ADD_OP(make_binary("Add", input.ref(), other.ref(), output.ref()), name);
}
Tensor Model::sub(Tensor input, Tensor other, Tensor output, const std::string &name) {
    return ADD_OP(make_binary("Sub", input.ref(), other.ref(), output.ref()), name);
}
Tensor Model::mul(Tensor input, Tensor other, Tensor output, const std::string &name) {
    return ADD_OP(make_binary("Mul", input.ref(), other.ref(), output.ref()), name);
}
Tensor Model::div(Tensor input, Tensor other, Tensor output, const std::string &name) {
    return ADD_OP(make_binary("Div", input.ref(), other.ref(), output.ref()), name);
}
// Attention over [batch, seq, heads, head_dim] tensors: per (batch, head),
// softmax(q k^T * scale + mask) v with mask = -inf where key > query + (seq_k -
// seq_q) if `causal`.  The chain of examples/llama/model.py:421-443 as one op.
Tensor Model::attention(Tensor q, Tensor k, Tensor v, float scale, bool causal, Tensor output,
                        const std::string &name) {
    check_null(q.ref());
    check_null(k.ref());
    check_null(v.ref());
    check_same_dtype(q.ref(), k.ref());
    check_same_dtype(q.ref(), v.ref());
    const Dims qs = q.ref()->shape(), ks = k.ref()->shape(), vs = v.ref()->shape();
    if (qs.ndims() != 4 || ks.ndims() != 4 || vs.ndims() != 4)
        ARK_ERR(ModelError, "attention takes [batch, seq, heads, head_dim] tensors");
    if (ks != vs || qs[0] != ks[0] || qs[2] != ks[2] || qs[3] != ks[3])
        ARK_ERR(ModelError, "attention shapes do not agree: q ", qs, ", k ", ks, ", v ", vs);
    if (!(scale > 0.f)) ARK_ERR(ModelError, "attention scale must be positive");
    ModelTensorRef out = output.ref();
    if (out) {
        check_same_dtype(q.ref(), out);
        check_shape(out, qs);
    } else {
        out = fresh(q.ref()->data_type(), qs);
    }
    auto op = compute_op("Attention", {q.ref(), k.ref(), v.ref()}, out);
    op->args_["Scale"] = ModelOpArg(scale);
    op->args_["Causal"] = ModelOpArg(causal);
    op->verify();
    return ADD_OP(op, name);
}

// silu(input . gate^T) * (input . up^T): both projections of the reference's
// feed-forward (examples/llama/model.py:326-331) and its gate in one GEMM pass; the
// products stay in fp32 until the one rounding of the result.
Tensor Model::swiglu(Tensor input, Tensor gate, Tensor up, Tensor output, const std::string &name) {
    check_null(input.ref());
    check_null(gate.ref());
    check_null(up.ref());
    check_same_dtype(input.ref(), gate.ref());
    check_same_dtype(input.ref(), up.ref());
    const Dims is = input.ref()->shape(), gs = gate.ref()->shape(), us = up.ref()->shape();
    if (is.ndims() < 2 || gs.ndims() != 2 || gs != us)
        ARK_ERR(ModelError, "swiglu takes input [..., m, dim] and two weights [hidden, dim]; got ", is, ", ", gs,
                ", ", us);
    if (is[-1] != gs[1]) ARK_ERR(ModelError, "swiglu: inner dimensions differ: ", is, " x ", gs);
    std::vector<DimType> od;
    for (int i = 0; i < is.ndims() - 1; ++i) od.push_back(is[i]);
    od.push_back(gs[0]);
    const Dims os(od);
    ModelTensorRef out = output.ref();
    if (out) {
        check_same_dtype(input.ref(), out);
        check_shape(out, os);
    } else {
        out = fresh(input.ref()->data_type(), os);
    }
    auto op = compute_op("MatmulSwiglu", {input.ref(), gate.ref(), up.ref()}, out);
    op->verify();
    return ADD_OP(op, name);
}

// silu(input) * other = input * sigmoid(input) * other in one pass: the SwiGLU
// gate of the reference's feed-forward (examples/llama/model.py:281-293, 329-331)
// without its two intermediate tensors
Tensor Model::silu_mul(Tensor input, Tensor other, Tensor output, const std::string &name) {
    return ADD_OP(make_binary("SiluMul", input.ref(), other.ref(), output.ref()), name);
}
// ark/ops/ops_rope.cpp:10-19
Tensor Model::rope(Tensor input, Tensor other, Tensor output, const std::string &name) {
    return ADD_OP(make_binary("Rope", input.ref(), other.ref(), output.ref()), name);
}

Tensor Model::exp(Tensor input, Tensor output, const std::string &name) {
    return ADD_OP(make_unary("Exp", input.ref(), output.ref()), name);
}
Tensor Model::sqrt(Tensor input, Tensor output, const std::string &name) {
    return ADD_OP(make_unary("Sqrt", input.ref(), output.ref()), name);
}
Tensor Model::rsqrt(Tensor input, Tensor output, const std::string &name) {
    return ADD_OP(make_unary("Rsqrt", input.ref(), output.ref()), name);
}
Tensor Model::relu(Tensor input, Tensor output, const std::string &name) {
    return ADD_OP(make_unary("Relu", input.ref(), output.ref()), name);
}
Tensor Model::gelu(Tensor input, Tensor output, const std::string &name) {
    return ADD_OP(make_unary("Gelu", input.ref(), output.ref()), name);
}
Tensor Model::sigmoid(Tensor input, Tensor output, const std::string &name) {
    return ADD_OP(make_unary("Sigmoid", input.ref(), output.ref()), name);
}
Tensor Model::copy(Tensor input, Tensor output, const std::string &name) {
    return ADD_OP(make_unary("Copy", input.ref(), output.ref()), name);
}

// scalar ops (ark/ops/ops_scalar.cpp:10-165)
static ModelOpRef make_scalar_assign(float val, const Dims &shape, ModelDataType dt, ModelTensorRef out) {
    if (out) {
        check_shape(out, shape);
        check_dtype(out, dt);
    } else {
        out = fresh(dt, shape);
    }
    auto op = compute_op("ScalarAssign", {}, out);
    op->args_["Value"] = ModelOpArg(val);
    op->verify();
    return op;
}
static ModelOpRef make_scalar(const std::string &type, ModelTensorRef in, float factor, ModelTensorRef out) {
    auto op = make_unary(type, in, out);
    op->args_["Factor"] = ModelOpArg(factor);
    return op;
}
Tensor Model::constant(float val, const Dims &shape, DataType data_type, const std::string &name) {
    return ADD_OP(make_scalar_assign(val, shape, data_type.ref(), nullptr), name);
}
Tensor Model::copy(float val, Tensor output, const std::string &name) {
    if (output.is_null()) return ADD_OP(make_scalar_assign(val, Dims(1), FP32.ref(), nullptr), name);
    return ADD_OP(make_scalar_assign(val, output.shape(), output.data_type().ref(), output.ref()), name);
}
Tensor Model::add(Tensor input, float value, Tensor output, const std::string &name) {
    return ADD_OP(make_scalar("ScalarAdd", input.ref(), value, output.ref()), name);
}
Tensor Model::sub(Tensor input, float value, Tensor output, const std::string &name) {
    return ADD_OP(make_scalar("ScalarAdd", input.ref(), -value, output.ref()), name);
}
Tensor Model::mul(Tensor input, float value, Tensor output, const std::string &name) {
    return ADD_OP(make_scalar("ScalarMul", input.ref(), value, output.ref()), name);
}
Tensor Model::div(Tensor input, float value, Tensor output, const std::string &name) {
    return ADD_OP(make_scalar("ScalarMul", input.ref(), 1 / value, output.ref()), name);
}

// cast (ark/ops/ops_cast.cpp:11-132): same-type cast without an output is an
// identity; casts to/from BYTE without an output reinterpret the buffer.
Tensor Model::cast(Tensor input, const DataType &data_type, Tensor output, const std::string &name) {
    check_null(input.ref());
    auto in = input.ref();
    if (output.is_null()) {
        if (input.data_type() == data_type) return identity(input, {}, name);
        if (data_type == BYTE || input.data_type() == BYTE) {
            Dims sh = in->shape(), st = in->strides(), of = in->offsets(), pd = in->padded_shape();
            if (input.data_type() == BYTE) {
                DimType eb = (DimType)data_type.bytes();
                if (in->shape_bytes() < (size_t)eb)
                    ARK_ERR(ModelError, "input tensor is too small to be casted to ", data_type.name());
                int last = sh.ndims() - 1;
                for (; last >= 0; --last)
                    if (last == 0 || st[last] > 1) break;
                for (const Dims *d : {&sh, &st, &of, &pd})
                    if (((*d)[last] % eb) != 0)
                        ARK_ERR(ModelError, "the last greater-than-1 dimension of the input tensor (",
                                (*d)[last], ") is not divisible by the size of the output tensor type (",
                                eb, ")");
                sh[last] /= eb; st[last] /= eb; of[last] /= eb; pd[last] /= eb;
            } else {
                DimType eb = (DimType)input.data_type().bytes();
                sh[-1] *= eb; st[-1] *= eb; of[-1] *= eb; pd[-1] *= eb;
            }
            return ADD_OP(view_op(in->buffer(), sh, data_type.ref(), st, of, pd, {in}), name);
        }
    }
    return ADD_OP(make_unary("Cast", in, output.ref(), data_type.ref()), name);
}

// embedding (ark/ops/ops_embedding.cpp:10-36): the output takes the indices' shape with the
// table's row length appended
Tensor Model::embedding(Tensor input, Tensor weight, Tensor output, const std::string &name) {
    check_null(input.ref());
    check_null(weight.ref());
    auto in = input.ref(), w = weight.ref(), out = output.ref();
    if (in->shape().ndims() > 3) ARK_ERR(ModelError, "input shape ndims > 3: ", in->shape());
    if (w->shape().ndims() != 2) ARK_ERR(ModelError, "weight shape ndims != 2: ", w->shape());
    if (out) {
        check_same_dtype(w, out);
    } else {
        const Dims i4 = in->shape().dims4();
        out = fresh(w->data_type(), Dims(i4[1], i4[2], i4[3], w->shape()[-1]));
    }
    auto op = compute_op("Embedding", {in, w}, out);
    op->verify();
    return ADD_OP(op, name);
}

// transpose (ark/ops/ops_transpose.cpp:37-79)
Tensor Model::transpose(Tensor input, const std::vector<int64_t> &permutation, Tensor output,
                        const std::string &name) {
    check_null(input.ref());
    auto in = input.ref(), out = output.ref();
    Dims perm(permutation);
    int nd = in->shape().ndims();
    if (nd != perm.ndims())
        ARK_ERR(ModelError,
                "The number of dimensions of permutation should be the same as the number of "
                "dimensions of input. Given input shape: ", in->shape(), ", permutation: ", perm);
    std::vector<int> count(nd, 0);
    std::vector<DimType> pshape;
    for (int i = 0; i < nd; ++i) {
        if (perm[i] >= nd || perm[i] < 0)
            ARK_ERR(ModelError,
                    "Each value in permutation should be less than the number of input dimensions. "
                    "Given permutation: ", perm);
        if (count[perm[i]]++ > 0)
            ARK_ERR(ModelError, "Each value in permutation should be unique. Given permutation: ", perm);
        pshape.push_back(in->shape()[(int)perm[i]]);
    }
    if (out) {
        check_same_dtype(in, out);
        check_shape(out, Dims(pshape));
    } else {
        out = fresh(in->data_type(), Dims(pshape));
    }
    auto op = compute_op("Transpose", {in}, out);
    op->args_["Permutation"] = ModelOpArg(perm);
    op->verify();
    return ADD_OP(op, name);
}

// ---------------------------------------------------------------------------
// Context / PlannerContext (ark/context_impl.cpp:22-49, ark/api/planner.cpp:18-87)
// ---------------------------------------------------------------------------
class Context::Impl {
   public:
    explicit Impl(Model &model) : stack_(ModelGraphAccess::context(model)) {
        static int next_id = 0;
        id_ = next_id++;
    }
    ~Impl() {
        for (auto it = keys_.rbegin(); it != keys_.rend(); ++it) stack_->pop(*it);
    }
    void set(const std::string &key, const Json &value, ContextType type) {
        if (type == ContextType::Overwrite) {
            push(key, value);
        } else if (type == ContextType::Extend) {
            Json cur = stack_->get(key);
            if (cur.empty()) {
                push(key, value);
            } else if (!cur.is_object() || !value.is_object()) {
                ARK_ERR(InvalidUsageError,
                        "Context value must be a JSON object when type is ContextTypeExtend. Key: ",
                        key, ", old value: ", cur.dump(), ", new value: ", value.dump());
            } else {
                for (const auto &m : value.items()) cur[m.first] = m.second;
                push(key, cur);
            }
        } else if (type == ContextType::Immutable) {
            if (!stack_->has(key)) push(key, value);
        } else {
            ARK_ERR(InvalidUsageError, "Unknown context type");
        }
    }
    void push(const std::string &key, const Json &value) {
        stack_->push(key, value);
        keys_.push_back(key);
    }
    std::shared_ptr<ContextStack> stack_;
    std::vector<std::string> keys_;
    int id_;
};

std::shared_ptr<ContextStack> ModelGraphAccess::context(Model &model) { return model.impl_->context_; }
ModelGraph::Impl &ModelGraphAccess::impl(const ModelGraph &g) { return *g.impl_; }
void ModelGraphAccess::adopt(ModelGraph &g, std::unique_ptr<ModelGraph::Impl> impl) { g.impl_ = std::move(impl); }

Context::Context(Model &model) : impl_(std::make_shared<Impl>(model)) {}
int Context::id() const { return impl_->id_; }
std::string Context::get(const std::string &key) const {
    return impl_->stack_->has(key) ? impl_->stack_->get(key).dump() : "";
}
void Context::set(const std::string &key, const std::string &value, ContextType type) {
    Json v;
    try {
        v = Json::parse(value);
    } catch (const std::exception &) {
        ARK_ERR(InvalidUsageError, "Failed to parse context value as JSON: `", value, "`");
    }
    impl_->set(key, v, type);
}

PlannerContext::PlannerContext(Model &model) : Context(model) {
    impl_->set("Id", Json(id()), ContextType::Immutable);
}

static bool range_subset(int b, int e, int s, int pb, int pe, int ps) {
    // every element of [b,e) step s lies in [pb,pe) step ps
    // (ark/range.hpp:12-107, is_subset_of)
    if (b >= e) return true;
    if (b < pb || e > pe) return false;
    if ((b - pb) % ps != 0) return false;
    int count = (e - b + s - 1) / s;
    return count <= 1 || s % ps == 0;
}

void PlannerContext::check_range(const std::string &key, int start, int end, int step) {
    Json prev = impl_->stack_->get(key);
    if (prev.empty()) return;
    auto v = prev.as_int_vector();
    if (v.size() < 2 || v.size() > 3) ARK_ERR(InternalError, "unexpected");
    int ps = v.size() == 3 ? (int)v[2] : 1;
    if (!range_subset(start, end, step, (int)v[0], (int)v[1], ps))
        ARK_ERR(PlanError, "New ", key, " [", start, ", ", end, ", ", step,
                "] is not a subset of the previous range ", prev.dump());
}

static Json range_json(int start, int end, int step) {
    Json r = Json::array();
    r.push_back(start);
    r.push_back(end);
    if (step != 1) r.push_back(step);
    return r;
}

void PlannerContext::processor_range(int start, int end, int step) {
    check_range("ProcessorRange", start, end, step);
    impl_->set("ProcessorRange", range_json(start, end, step), ContextType::Overwrite);
}
void PlannerContext::warp_range(int start, int end, int step) {
    check_range("WarpRange", start, end, step);
    impl_->set("WarpRange", range_json(start, end, step), ContextType::Overwrite);
}
void PlannerContext::sram_range(int start, int end, int step) {
    check_range("SramRange", start, end, step);
    impl_->set("SramRange", range_json(start, end, step), ContextType::Overwrite);
}
void PlannerContext::sync(bool sync) {
    if (sync) {
        // `true` never overrides an enclosing `false`
        if (impl_->stack_->get("Sync") == Json(false)) {
            ARK_LOG(WARN, "Ignoring sync(true) while sync(false) is already set");
            return;
        }
        impl_->set("Sync", Json(true), ContextType::Immutable);
    } else {
        impl_->set("Sync", Json(false), ContextType::Overwrite);
    }
}
void PlannerContext::config(const std::string &config) {
    Json v;
    try {
        v = Json::parse(config);
    } catch (const std::exception &) {
        ARK_ERR(InvalidUsageError, "Failed to parse config as JSON: `", config, "`");
    }
    impl_->set("Config", v, ContextType::Extend);
}

}  // namespace ark
