// ark::Model — the op-builder API.  Signatures follow the reference
// (ark/include/ark/model.hpp:18-258) so existing single-GPU model code
// compiles unchanged; communication ops are not part of this backend.
#ifndef ARK_MODEL_HPP
#define ARK_MODEL_HPP

#include <ark/data_type.hpp>
#include <ark/dims.hpp>
#include <ark/model_graph.hpp>
#include <ark/tensor.hpp>
#include <string>
#include <vector>

namespace ark {

class Model : public ModelGraph {
   public:
    Model(int rank = 0, int world_size = 1);
    Model(const Model &other);
    ~Model() {}
    Model &operator=(const Model &other) = default;

    size_t id() const;
    // A copy of this model with virtual ops removed.
    Model compress() const;
    int unique_tag();

    // ---- tensors and views (no kernel) -----------------------------------
    // `strides` is the extent of the underlying buffer per dimension,
    // `offsets` where the view starts, `padded_shape` the region kernels may
    // touch (>= shape, <= strides - offsets).  Padding is zero-filled once.
    Tensor tensor(const Dims &shape, const DataType &data_type, const Dims &strides = {},
                  const Dims &offsets = {}, const Dims &padded_shape = {}, int rank = -1,
                  const std::string &name = "");
    Tensor refer(Tensor input, const Dims &shape = {}, const Dims &strides = {},
                 const Dims &offsets = {}, const Dims &padded_shape = {},
                 const std::string &name = "");
    // One -1 is inferred; 0 keeps the input's dimension unless `allowzero`.
    Tensor reshape(Tensor input, const Dims &shape, bool allowzero = false,
                   const std::string &name = "");
    // Same tensor, additionally ordered after the producers of `deps`.
    Tensor identity(Tensor input, const std::vector<Tensor> &deps = {},
                    const std::string &name = "");
    std::vector<Tensor> sharding(Tensor input, DimType axis, DimType dim_per_shard,
                                 const std::string &name = "");
    void noop(Tensor input, const std::string &name = "");
    Tensor constant(float val, const Dims &shape, DataType data_type,
                    const std::string &name = "");

    // ---- contraction ------------------------------------------------------
    Tensor matmul(Tensor input, Tensor other, Tensor output = NullTensor, bool trans_input = false,
                  bool trans_other = false, const std::string &name = "");

    // ---- reductions ---------------------------------------------------------
    Tensor reduce_sum(Tensor input, int axis, bool keepdims = true, Tensor output = NullTensor,
                      const std::string &name = "");
    Tensor reduce_mean(Tensor input, int axis, bool keepdims = true, Tensor output = NullTensor,
                       const std::string &name = "");
    Tensor reduce_max(Tensor input, int axis, bool keepdims = true, Tensor output = NullTensor,
                      const std::string &name = "");

    // ---- fused row ops (extensions of this backend) ------------------------
    // One kernel each for what the reference composes from 5-7 ops
    // (python/ark/ops.py:491-513, examples/llama/model.py:92-99).
    Tensor softmax(Tensor input, Tensor output = NullTensor, const std::string &name = "");
    // softmax(input * scale + mask): the attention chain scale -> add mask ->
    // softmax (examples/llama/model.py:426-433) as one op; mask may be NullTensor
    Tensor softmax(Tensor input, Tensor mask, float scale, Tensor output = NullTensor,
                   const std::string &name = "");
    Tensor layernorm(Tensor input, float eps = 1e-6f, Tensor output = NullTensor,
                     const std::string &name = "");
    // weight: NullTensor, or [.., dim] in FP32 or the input's type.
    Tensor rmsnorm(Tensor input, Tensor weight = NullTensor, float eps = 0.f,
                   Tensor output = NullTensor, const std::string &name = "");

    // ---- elementwise --------------------------------------------------------
    Tensor add(Tensor input, Tensor other, Tensor output = NullTensor,
               const std::string &name = "");
    Tensor add(Tensor input, float value, Tensor output = NullTensor,
               const std::string &name = "");
    Tensor sub(Tensor input, Tensor other, Tensor output = NullTensor,
               const std::string &name = "");
    Tensor sub(Tensor input, float value, Tensor output = NullTensor,
               const std::string &name = "");
    Tensor mul(Tensor input, Tensor other, Tensor output = NullTensor,
               const std::string &name = "");
    Tensor mul(Tensor input, float value, Tensor output = NullTensor,
               const std::string &name = "");
    Tensor div(Tensor input, Tensor other, Tensor output = NullTensor,
               const std::string &name = "");
    Tensor div(Tensor input, float value, Tensor output = NullTensor,
               const std::string &name = "");
    Tensor exp(Tensor input, Tensor output = NullTensor, const std::string &name = "");
    Tensor sqrt(Tensor input, Tensor output = NullTensor, const std::string &name = "");
    Tensor rsqrt(Tensor input, Tensor output = NullTensor, const std::string &name = "");
    Tensor relu(Tensor input, Tensor output = NullTensor, const std::string &name = "");
    Tensor gelu(Tensor input, Tensor output = NullTensor, const std::string &name = "");
    Tensor sigmoid(Tensor input, Tensor output = NullTensor, const std::string &name = "");
    Tensor copy(Tensor input, Tensor output = NullTensor, const std::string &name = "");
    Tensor copy(float val, Tensor output = NullTensor, const std::string &name = "");
    Tensor cast(Tensor input, const DataType &data_type, Tensor output = NullTensor,
                const std::string &name = "");
    // Rotary embedding: complex multiply of adjacent (even, odd) pairs.
    // softmax(q k^T * scale [+ causal mask]) v over [batch, seq, heads, head_dim]
    // tensors, as one op (extension: the reference composes transposes, two
    // matmuls, a scalar multiply, a mask add and a five-op softmax)
    Tensor attention(Tensor q, Tensor k, Tensor v, float scale, bool causal, Tensor output = NullTensor,
                     const std::string &name = "");
    // silu(input . gate^T) * (input . up^T) with gate, up stored [hidden, dim] as the reference's
    // Linear stores its weights: the SwiGLU front half of a feed-forward as one op (extension:
    // the reference runs two matmuls, sigmoid, mul, mul; examples/llama/model.py:296-333)
    Tensor swiglu(Tensor input, Tensor gate, Tensor up, Tensor output = NullTensor, const std::string &name = "");
    // silu(input) * other in one op (extension: the reference composes sigmoid, mul, mul)
    Tensor silu_mul(Tensor input, Tensor other, Tensor output = NullTensor, const std::string &name = "");
    Tensor rope(Tensor input, Tensor other, Tensor output = NullTensor,
                const std::string &name = "");
    // Rows of `weight` [num_embeddings, dim] picked by the INT32 indices of `input` (at
    // most 3-D); negative indices count from the end of the table.
    Tensor embedding(Tensor input, Tensor weight, Tensor output = NullTensor, const std::string &name = "");
    // 4-D permutation copy.
    Tensor transpose(Tensor input, const std::vector<int64_t> &permutation,
                     Tensor output = NullTensor, const std::string &name = "");

   private:
    size_t id_;
    int next_tag_ = 0;
};

}  // namespace ark

#endif  // ARK_MODEL_HPP
