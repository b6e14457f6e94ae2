"""CPU tests of the Model op API: shape inference, validation, graph
compression.  Cases restate ark/api/model_test.cpp, ark/ops/ops_*_test.cpp
(*_invalid and shape checks) and python/unittest/test_ops.py (output shapes)."""
import json

import pytest

from ark_amd import Model, ArkmiError


def raises_model_error(fn):
    with pytest.raises(ArkmiError) as e:
        fn()
    assert e.value.kind == "ModelError", e.value
    return e.value


def nodes_of(m):
    return m.dump(compressed=True)["Nodes"]


# ---------------------------------------------------------------- graph (api/model_test.cpp:13-120)
def test_model_basics_compress():
    m = Model()
    t0, t1 = m.tensor([1], "fp32"), m.tensor([1], "fp32")
    t2 = m.add(t0, t1)
    assert m.verify()
    n = nodes_of(m)
    assert len(n) == 1 and n[0]["Op"]["Type"] == "Add"
    assert n[0]["Op"]["ResultTensors"][0]["Id"] == t2.id
    assert [t["Id"] for t in n[0]["Op"]["ReadTensors"]] == [t0.id, t1.id]
    assert n[0]["ProducerNodeIds"] == [] and n[0]["ConsumerNodeIds"] == []
    t3 = m.add(t2, t1)
    n = nodes_of(m)
    assert len(n) == 2
    assert n[0]["ConsumerNodeIds"] == [1] and n[1]["ProducerNodeIds"] == [0]
    t4 = m.relu(t3)
    n = nodes_of(m)
    assert [x["Op"]["Type"] for x in n] == ["Add", "Add", "Relu"]
    assert n[2]["ProducerNodeIds"] == [1] and n[1]["ConsumerNodeIds"] == [2]
    # an op with two consumers
    t5 = m.exp(t3)
    m.add(t4, t5)
    n = nodes_of(m)
    assert len(n) == 5
    assert sorted(n[1]["ConsumerNodeIds"]) == [2, 3]
    assert sorted(n[4]["ProducerNodeIds"]) == [2, 3]
    # the uncompressed model keeps its virtual Tensor ops
    full = m.dump()["Nodes"]
    assert sum(x["Op"]["IsVirtual"] for x in full) >= 2 and len(full) > len(n)


def test_identity_and_dependencies():
    """ops_identity_test.cpp:9-46: identity adds execution dependencies."""
    m = Model()
    t0, t1, t2 = (m.tensor([1], "fp32") for _ in range(3))
    a = m.relu(t0)
    b = m.relu(t1)
    i = m.identity(t2, deps=[a, b])
    assert i.buffer_id == t2.buffer_id and i.shape == t2.shape
    m.relu(i)
    n = nodes_of(m)
    assert len(n) == 3
    assert sorted(n[2]["ProducerNodeIds"]) == [0, 1]   # the virtual identity is spliced out


def test_sharding():
    """ops_sharding_test.cpp:10-60."""
    m = Model()
    t = m.tensor([3, 9, 2], "fp32")
    shards = m.sharding(t, axis=1, dim_per_shard=3)
    assert len(shards) == 3
    for i, s in enumerate(shards):
        assert s.shape == [3, 3, 2] and s.strides == [3, 9, 2] and s.offsets == [0, 3 * i, 0]
        assert s.buffer_id == t.buffer_id
    raises_model_error(lambda: m.sharding(t, axis=1, dim_per_shard=4))


def test_op_auto_names():
    m = Model()
    t = m.tensor([64], "fp32")
    m.relu(t)
    m.relu(t)
    m.relu(t, name="mine")
    m.reduce_sum(t, 0)
    names = [x["Op"]["Name"] for x in nodes_of(m)]
    assert names == ["relu", "relu_1", "mine", "reduce_sum"]


# ---------------------------------------------------------------- tensors
def test_tensor_validation():
    m = Model()
    t = m.tensor([2, 3], "fp16", strides=[4, 8], offsets=[1, 2], padded_shape=[3, 6])
    assert (t.shape, t.strides, t.offsets, t.padded_shape) == ([2, 3], [4, 8], [1, 2], [3, 6])
    d = m.tensor([5, 7], "fp32")
    assert d.strides == [5, 7] and d.offsets == [0, 0] and d.padded_shape == [5, 7]
    raises_model_error(lambda: m.tensor([0, 3], "fp32"))
    raises_model_error(lambda: m.tensor([2, -3], "fp32"))
    raises_model_error(lambda: m.tensor([2, 3], "fp32", padded_shape=[2, 2]))      # shape > padded
    raises_model_error(lambda: m.tensor([2, 3], "fp32", strides=[2, 3], offsets=[0, 1]))  # out of bounds
    raises_model_error(lambda: m.tensor([2, 3], "fp32", strides=[2]))
    with pytest.raises(ArkmiError) as e:
        m.tensor([1, 2, 3, 4, 5], "fp32")
    assert e.value.kind == "InvalidUsageError"


def test_reshape_stride_inference():
    """ops_reshape_test.cpp:76-212."""
    m = Model()
    cases = [
        (([32, 64], [32, 100], None), [32, 64], [32, 64], [32, 100], None),
        (([32, 64], [32, 100], None), [32, 32, 2], [32, 32, 2], [32, 50, 2], None),
        (([3, 8, 4, 64], [3, 16, 4, 64], None), [3, 32, 64], [3, 32, 64], [3, 64, 64], None),
        (([2, 3, 4, 5], [3, 3, 4, 5], None), [120], [120], [180], None),
        (([2, 3, 4, 5], [3, 3, 8, 5], None), [6, 20], [6, 20], [9, 40], None),
        (([4, 3], [4, 9], [0, 5]), [4, 3, 1], [4, 3, 1], [4, 9, 1], [0, 5, 0]),
        (([2, 6, 2], [3, 6, 2], [1, 0, 0]), [8, 3], [8, 3], [12, 3], [4, 0]),
        (([64, 256], [512, 512], [128, 128]), [1, 64, 256], [1, 64, 256], [1, 512, 512], [0, 128, 128]),
        (([1, 64, 256], [1, 512, 512], [0, 128, 128]), [64, 256], [64, 256], [512, 512], [128, 128]),
    ]
    for (shape, strides, offs), target, want_shape, want_strides, want_offs in cases:
        t = m.tensor(shape, "fp32", strides=strides, offsets=offs)
        r = m.reshape(t, target)
        assert r.shape == want_shape and r.strides == want_strides, (shape, target, r.strides)
        if want_offs is not None:
            assert r.offsets == want_offs
        assert r.buffer_id == t.buffer_id
    t = m.tensor([4, 6], "fp32")
    assert m.reshape(t, [-1, 3]).shape == [8, 3]
    assert m.reshape(t, [0, 2, 3]).shape == [4, 2, 3]          # 0 keeps the input dimension
    raises_model_error(lambda: m.reshape(t, [-1, -1]))
    raises_model_error(lambda: m.reshape(t, [5, 5]))
    raises_model_error(lambda: m.reshape(t, [-1, 0]))
    # merging across a padded (non-dense) dimension cannot be expressed as a view
    p = m.tensor([4, 6], "fp32", strides=[4, 8])
    raises_model_error(lambda: m.reshape(p, [24]))


def _addresses(shape, strides, offsets):
    """Element offsets of a view inside its buffer, in row-major order of `shape`."""
    import itertools
    import numpy as np
    pitch = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        pitch[i] = pitch[i + 1] * strides[i + 1]
    out = []
    for idx in itertools.product(*[range(s) for s in shape]):
        out.append(sum((o + i) * p for i, o, p in zip(idx, offsets, pitch)))
    return np.array(out, dtype=np.int64)


def test_reshape_addresses_the_same_elements_brute_force():
    """Whatever strides/offsets reshape infers, element i (row-major) of the result must
    sit where element i of the input sits: brute force over random padded and offset
    views and every factorisation of their element count into up to four extents.  A
    refusal is allowed only when a merged dimension is padded or offset."""
    import itertools
    import numpy as np
    rng = np.random.default_rng(7)

    def factorisations(n, k):
        if k == 1:
            yield [n]
            return
        for d in range(1, n + 1):
            if n % d == 0:
                for rest in factorisations(n // d, k - 1):
                    yield [d] + rest

    m = Model()
    accepted = refused = 0
    for trial in range(60):
        nd = int(rng.integers(1, 5))
        shape = [int(rng.choice([1, 2, 3, 4, 6])) for _ in range(nd)]
        pad = [int(rng.choice([0, 0, 1, 2])) for _ in range(nd)]
        offs = [int(rng.integers(0, p + 1)) for p in pad]
        strides = [s + p for s, p in zip(shape, pad)]
        t = m.tensor(shape, "fp32", strides=strides, offsets=offs)
        src = _addresses(shape, strides, offs)
        n = int(np.prod(shape))
        dense_all = all(p == 0 for p in pad)
        for k in range(1, 5):
            for target in itertools.islice(factorisations(n, k), 12):
                try:
                    r = m.reshape(t, target)
                except ArkmiError as e:
                    assert e.kind == "ModelError"
                    assert not dense_all, (shape, strides, offs, target)  # a dense tensor reshapes to anything
                    refused += 1
                    continue
                accepted += 1
                assert r.shape == target
                for sh, st, of in zip(r.shape, r.strides, r.offsets):
                    assert of + sh <= st
                dst = _addresses(r.shape, r.strides, r.offsets)
                assert np.array_equal(src, dst), (shape, strides, offs, target, r.strides, r.offsets)
    assert accepted > 300 and refused > 50, (accepted, refused)


def test_refer_and_cast_views():
    m = Model()
    t = m.tensor([4, 8], "fp16")
    r = m.refer(t, shape=[2, 4], strides=[4, 8], offsets=[1, 2])
    assert r.buffer_id == t.buffer_id and r.offsets == [1, 2]
    same = m.cast(t, "fp16")
    assert same.buffer_id == t.buffer_id and same.shape == t.shape       # identity
    as_bytes = m.cast(t, "byte")
    assert as_bytes.shape == [4, 16] and as_bytes.buffer_id == t.buffer_id
    back = m.cast(as_bytes, "fp32")
    assert back.shape == [4, 4] and back.buffer_id == t.buffer_id
    real = m.cast(t, "fp32")
    assert real.buffer_id != t.buffer_id and real.dtype == "fp32" and real.shape == [4, 8]
    odd = m.tensor([3, 5], "byte")
    raises_model_error(lambda: m.cast(odd, "fp16"))


# ---------------------------------------------------------------- op shape rules
def test_matmul_shapes_and_invalid():
    m = Model()
    a, b = m.tensor([128, 64], "fp16"), m.tensor([64, 256], "fp16")
    assert m.matmul(a, b).shape == [128, 256]
    bt = m.tensor([256, 64], "fp16")
    assert m.matmul(a, bt, trans_other=True).shape == [128, 256]
    at = m.tensor([64, 128], "fp16")
    assert m.matmul(at, b, trans_input=True).shape == [128, 256]
    b3 = m.tensor([3, 7, 64, 32], "fp16")
    a3 = m.tensor([3, 1, 128, 64], "fp16")
    assert m.matmul(a3, b3).shape == [3, 7, 128, 32]                      # batch broadcast
    assert m.matmul(m.tensor([5, 128, 64], "fp16"), b).shape == [5, 128, 256]
    # ops_matmul_test.cpp:563-573
    raises_model_error(lambda: m.matmul(a, m.tensor([128, 256], "fp16")))
    raises_model_error(lambda: m.matmul(m.tensor([3, 3, 128, 128], "fp16"), m.tensor([2, 3, 128, 128], "fp16")))
    raises_model_error(lambda: m.matmul(a, m.tensor([64, 256], "bf16")))
    raises_model_error(lambda: m.matmul(a, b, output=m.tensor([128, 128], "fp16")))
    # padded operands give a padded result (ops_matmul.cpp:72-88)
    pa = m.tensor([2, 64], "fp16", padded_shape=[128, 64])
    pb = m.tensor([64, 9], "fp16", padded_shape=[64, 128])
    c = m.matmul(pa, pb)
    assert c.shape == [2, 9] and c.padded_shape == [128, 128]


def test_reduce_shapes_and_invalid():
    """ops_reduce_test.cpp:379-455."""
    m = Model()
    t = m.tensor([7, 2, 4, 1024], "bf16")
    assert m.reduce_sum(t, 0).shape == [1, 2, 4, 1024]
    assert m.reduce_max(t, -1).shape == [7, 2, 4, 1]
    assert m.reduce_mean(t, 2, keepdims=False).shape == [7, 2, 1024]
    raises_model_error(lambda: m.reduce_sum(t, 0, True, m.tensor([1, 2, 4, 1024], "fp32")))
    raises_model_error(lambda: m.reduce_sum(t, 3, True, m.tensor([7, 2, 4, 1], "fp32")))
    raises_model_error(lambda: m.reduce_sum(t, 0, True, m.tensor([1, 2, 4, 512], "bf16")))
    raises_model_error(lambda: m.reduce_sum(t, 4))
    raises_model_error(lambda: m.reduce_sum(t, -5))


def test_elementwise_shapes_and_invalid():
    m = Model()
    a = m.tensor([4, 1, 1024], "fp16")
    b = m.tensor([1, 2, 1], "fp16")
    assert m.add(a, b).shape == [4, 2, 1024]
    assert m.mul(a, 2.0).shape == a.shape
    raises_model_error(lambda: m.add(a, m.tensor([3, 1, 1024], "fp16")))       # not broadcastable
    raises_model_error(lambda: m.add(a, m.tensor([4, 1, 1024], "fp32")))       # dtype mismatch
    raises_model_error(lambda: m.exp(a, m.tensor([4, 1, 1024], "fp32")))       # ops_math_test.cpp:120-134
    raises_model_error(lambda: m.exp(a, m.tensor([4, 1, 512], "fp16")))
    raises_model_error(lambda: m.rope(a, m.tensor([4, 1, 1024], "bf16")))      # ops_rope_test.cpp:72-94
    out = m.tensor([4, 1, 1024], "fp16")
    assert m.relu(a, out).buffer_id == out.buffer_id
    c = m.constant(1.5, [2, 3], "fp32")
    assert c.shape == [2, 3] and c.dtype == "fp32"
    assert m.transpose(m.tensor([5, 3, 32, 128], "fp16"), [0, 2, 1, 3]).shape == [5, 32, 3, 128]
    raises_model_error(lambda: m.transpose(a, [0, 1]))
    raises_model_error(lambda: m.transpose(a, [0, 0, 1]))
    raises_model_error(lambda: m.transpose(a, [0, 1, 3]))


def test_fused_row_ops_shapes():
    m = Model()
    x = m.tensor([8, 2048, 4096], "bf16")
    assert m.softmax(x).shape == x.shape
    assert m.layernorm(x, 1e-5).shape == x.shape
    assert m.rmsnorm(x, m.tensor([1, 1, 4096], "fp32"), 1e-6).shape == x.shape
    assert m.rmsnorm(x, m.tensor([4096], "bf16")).shape == x.shape
    raises_model_error(lambda: m.rmsnorm(x, m.tensor([2048], "fp32")))
    raises_model_error(lambda: m.rmsnorm(x, m.tensor([4096], "fp16")))
    raises_model_error(lambda: m.softmax(x, m.tensor([8, 2048, 4096], "fp16")))


# ---------------------------------------------------------------- fused ops of this backend
def test_attention_and_swiglu_shape_rules():
    m = Model()
    q = m.tensor([2, 256, 4, 128], "bf16")
    k = m.tensor([2, 384, 4, 128], "bf16")
    v = m.tensor([2, 384, 4, 128], "bf16")
    o = m.attention(q, k, v, 0.0884, causal=True)
    assert o.shape == [2, 256, 4, 128] and o.dtype == "bf16"
    raises_model_error(lambda: m.attention(q, k, m.tensor([2, 256, 4, 128], "bf16"), 0.1))    # k, v differ
    raises_model_error(lambda: m.attention(q, m.tensor([2, 384, 8, 128], "bf16"), v, 0.1))    # heads differ
    raises_model_error(lambda: m.attention(q, k, v, 0.0))                                     # scale
    raises_model_error(lambda: m.attention(m.tensor([256, 4, 128], "bf16"), k, v, 0.1))      # rank
    raises_model_error(lambda: m.attention(q, k, m.tensor([2, 384, 4, 128], "fp16"), 0.1))    # types

    x = m.tensor([3, 256, 512], "fp16")
    w1, w3 = m.tensor([1024, 512], "fp16"), m.tensor([1024, 512], "fp16")
    h = m.swiglu(x, w1, w3)
    assert h.shape == [3, 256, 1024]
    raises_model_error(lambda: m.swiglu(x, w1, m.tensor([512, 512], "fp16")))                # weights differ
    raises_model_error(lambda: m.swiglu(x, m.tensor([1024, 256], "fp16"), m.tensor([1024, 256], "fp16")))  # inner dim
    raises_model_error(lambda: m.swiglu(x, w1, m.tensor([1024, 512], "bf16")))               # types
    ops = [n["Op"]["Type"] for n in nodes_of(m)]
    assert ops == ["Attention", "MatmulSwiglu"]


def test_fused_op_plans_exist_only_on_rocm950():
    m = Model()
    x = m.tensor([1, 2048, 4096], "bf16")
    m.swiglu(x, m.tensor([11008, 4096], "bf16"), m.tensor([11008, 4096], "bf16"))
    q = m.tensor([1, 2048, 32, 128], "bf16")
    m.attention(q, q, q, 0.0884, causal=True)
    plan = json.loads(m.plan(arch="ROCM_950", num_processors=256))
    sw, at = (ti["Ops"][0]["Config"] for ti in plan["TaskInfos"])
    assert sw["TileShapeMNK"] == [256, 256, 64] and sw["NumTasks"] == 8 * 86   # 256 rows x 128 result columns per task
    assert at["NumTasks"] == 32 * 16 and at["SramBytes"] == 131072              # 128 query positions of one head per task
    with pytest.raises(ArkmiError) as e:
        m.plan(arch="CUDA_80", num_processors=108)
    assert e.value.kind == "PlanError"


def test_embedding_shapes_and_invalid():
    """ops_embedding.cpp:10-36, ops_embedding_test.cpp:98-112."""
    m = Model()
    ti = m.tensor([8, 3, 64], "int32")
    tw = m.tensor([100, 4096], "fp16")
    out = m.embedding(ti, tw)
    assert out.shape == [8, 3, 64, 4096] and out.dtype == "fp16"
    assert m.embedding(m.tensor([7], "int32"), tw).shape == [1, 1, 7, 4096]
    raises_model_error(lambda: m.embedding(m.tensor([4, 8, 3, 64], "int32"), m.tensor([100, 1024], "fp32")))
    raises_model_error(lambda: m.embedding(ti, m.tensor([2, 100, 1024], "fp32")))
    raises_model_error(lambda: m.embedding(ti, tw, m.tensor([8, 3, 64, 4096], "fp32")))  # output type != table type
    # default configs: one warp per row on the reference's architectures, one wave per row here
    import json
    p = json.loads(m.plan(arch="CUDA_80", num_processors=108))
    cfg = p["TaskInfos"][0]["Ops"][0]["Config"]
    assert cfg["NumWarps"] == 1 and cfg["NumTasks"] == 8 * 3 * 64
    p = json.loads(m.plan(arch="ROCM_950", num_processors=256))
    cfg = p["TaskInfos"][0]["Ops"][0]["Config"]
    assert cfg["NumWarps"] == 8 and cfg["NumTasks"] == 8 * 3 * 64 // 8


def test_int32_scalars_outside_the_int32_range_are_refused():
    """A scalar operand travels as a float, in the plan file and to the kernel
    (ark/ops/ops_scalar.cpp:82-111 keeps "Factor" as a float too), and the INT32 body
    truncates it to the element type like ark/include/kernels/scalar.h:13-41.  That
    conversion is defined inside the int32 range only: compile() refuses the rest, and
    a scalar that JSON cannot spell is refused when the op is made."""
    from ark_amd import Model, plan_analysis, ArkmiError

    def compile_with(v):
        m = Model()
        t = m.tensor([64, 256], "int32")
        m.mul(t, v)
        plan_analysis(m.plan(arch="ROCM_950", num_processors=256), 0)

    for v in (0.0, 3.5, -7.9, 16777218.0, 2147483520.0, -2147483648.0):
        compile_with(v)
    for v in (2147483648.0, 3e9, -2147483904.0, -3e9, 1e30):
        with pytest.raises(ArkmiError) as e:
            compile_with(v)
        assert e.value.kind == "UnsupportedError" and "INT32 scalar" in str(e.value)
    for v in (float("inf"), float("nan")):
        with pytest.raises(ArkmiError) as e:
            compile_with(v)
        assert e.value.kind == "InvalidUsageError" and "not finite" in str(e.value)
    m = Model()
    m.mul(m.tensor([64, 256], "fp32"), 1e30)   # float tensors take any finite scalar
    plan_analysis(m.plan(arch="ROCM_950", num_processors=256), 0)
