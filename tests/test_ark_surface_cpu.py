"""The `ark`-named Python surface without a GPU: shapes every op function returns
(restating python/unittest/test_ops.py:7-218), data type tags (test_data_type.py:9-77), the error
classes (test_error.py:7-13), the global model (test_model.py:8-29), planner and module plumbing,
and the runtime's refusals before launch."""
import json

import numpy as np
import pytest

import ark_amd.ark as ark


@pytest.fixture(autouse=True)
def fresh_model():
    ark.init()
    yield
    ark.init()


def t64(dtype=None):
    return ark.tensor([64, 64], dtype or ark.fp16)


def test_arithmetic_shapes_and_number_operands():
    a, b = t64(), t64()
    for f in (ark.add, ark.sub, ark.mul, ark.div):
        assert f(a, b).shape() == [64, 64]
        assert f(a, 1.0).shape() == [64, 64]
    assert ark.add(1.0, a).shape() == [64, 64]
    assert ark.mul(2.0, a).shape() == [64, 64]
    assert ark.add(1.0, 1.0) == 2.0
    assert ark.sub(3.0, 1.0) == 2.0
    with pytest.raises(ark.InvalidUsageError):
        ark.sub(1.0, a)
    out = t64()
    filled = ark.add(1.0, 2.0, output=out)  # two numbers and an output: a constant fill
    assert filled.shape() == [64, 64]


def test_cast_constant_copy():
    a = t64()
    b = ark.cast(a, ark.fp32)
    assert b.shape() == [64, 64] and b.dtype() == ark.fp32
    assert ark.constant(1.0, [64, 64]).shape() == [64, 64]
    assert ark.ones([4, 8], ark.fp16).dtype() == ark.fp16
    assert ark.zeros([4, 8]).shape() == [4, 8]
    assert ark.copy(a).shape() == [64, 64]


def test_embedding_shape():
    idx = ark.tensor([64, 64], ark.int32)
    table = ark.tensor([100, 4096], ark.fp16)
    assert ark.embedding(idx, table).shape() == [1, 64, 64, 4096]


@pytest.mark.parametrize("name", ["exp", "gelu", "relu", "rsqrt", "sigmoid", "sqrt", "identity",
                                  "softmax", "layernorm"])
def test_unary_shapes(name):
    assert getattr(ark, name)(t64()).shape() == [64, 64]


def test_matmul_rope_shapes():
    assert ark.matmul(t64(), t64()).shape() == [64, 64]
    a = ark.tensor([128, 64], ark.fp16)
    b = ark.tensor([256, 64], ark.fp16)
    assert ark.matmul(a, b, transpose_other=True).shape() == [128, 256]
    assert ark.rope(t64(), t64()).shape() == [64, 64]


@pytest.mark.parametrize("name", ["reduce_max", "reduce_mean", "reduce_sum", "mean"])
def test_reduce_shapes(name):
    f = getattr(ark, name)
    a = ark.tensor([64, 32], ark.fp16)
    assert f(a, axis=0, keepdims=True).shape() == [1, 32]
    assert f(a, axis=1, keepdims=True).shape() == [64, 1]
    assert f(a, axis=0, keepdims=False).shape() == [32]
    assert f(a, axis=1, keepdims=False).shape() == [64]


def test_reshape_sharding_transpose():
    a = t64()
    assert ark.reshape(a, [64, 64, 1]).shape() == [64, 64, 1]
    assert ark.reshape(a, [-1, 16]).shape() == [256, 16]
    shards = ark.sharding(a, axis=0, dim_per_shard=2)
    assert len(shards) == 32 and shards[0].shape() == [2, 64]
    assert ark.transpose(ark.tensor([64, 32], ark.fp16), [1, 0]).shape() == [32, 64]
    with pytest.raises(ark.InvalidUsageError):
        ark.reshape(a, 64)
    with pytest.raises(ark.InvalidUsageError):
        ark.reshape(a, [1, 1, 1, 64, 64])
    with pytest.raises(ark.InvalidUsageError):
        ark.transpose(a, 1)
    with pytest.raises(ark.InvalidUsageError):
        ark.tensor([1, 2, 3, 4, 5], ark.fp16)
    with pytest.raises(ark.InvalidUsageError):
        ark.tensor(64, ark.fp16)
    with pytest.raises(ark.InvalidUsageError):
        ark.identity(a, deps=[1])


def test_tensor_handle():
    a = ark.tensor([8, 16], ark.fp16, strides=[8, 32], offsets=[0, 4])
    assert a.shape() == [8, 16] and a.strides() == [8, 32] and a.nelems() == 128
    assert a.dtype() == ark.fp16
    # before launch: to_numpy gives an array of the right shape and type, from_numpy refuses
    arr = a.to_numpy()
    assert arr.shape == (8, 16) and arr.dtype == np.float16
    with pytest.raises(RuntimeError, match="not allocated yet"):
        a.from_numpy(np.zeros((8, 16), np.float16))


def test_data_types():
    pairs = [(ark.fp32, np.float32, 4, "FP32"), (ark.fp16, np.float16, 2, "FP16"),
             (ark.int32, np.int32, 4, "INT32"), (ark.uint32, np.uint32, 4, "UINT32"),
             (ark.int8, np.int8, 1, "INT8"), (ark.uint8, np.uint8, 1, "UINT8")]
    for tag, npt, size, cname in pairs:
        assert ark.DataType.from_numpy(np.dtype(npt)) == tag
        assert ark.DataType.from_name(tag.__name__) == tag
        assert ark.DataType.from_ctype(getattr(ark.core, cname)) == tag
        assert tag.to_numpy() == npt
        assert tag.ctype() == getattr(ark.core, cname)
        assert tag.element_size() == size
    assert ark.bf16.element_size() == 2 and ark.bf16.to_numpy() == np.uint16
    assert ark.byte.element_size() == 1
    with pytest.raises(ark.error.InvalidUsageError):
        ark.DataType.from_numpy(None)
    with pytest.raises(ark.error.InvalidUsageError):
        ark.DataType.from_name("unknown")
    with pytest.raises(ark.error.InvalidUsageError):
        ark.DataType.from_ctype(None)


def test_error_classes():
    try:
        raise ark.InternalError("test")
    except ark.BaseError as e:
        assert isinstance(e, ark.InternalError)
        assert str(e) == "test"
    # errors from the native side arrive as the class of the same name
    with pytest.raises(ark.ModelError):
        ark.matmul(ark.tensor([64, 32], ark.fp16), ark.tensor([64, 32], ark.fp16))
    with pytest.raises(ark.UnsupportedError):
        ark.Planner(arch="NO_SUCH_ARCH", num_processors=4).plan()
    for cls in (ark.InternalError, ark.InvalidUsageError, ark.ModelError, ark.PlanError,
                ark.UnsupportedError, ark.SystemError, ark.GpuError):
        assert issubclass(cls, ark.BaseError)


def test_global_model_and_reset():
    ark.add(t64(), t64())
    m = json.loads(ark.Model.get_model().compress().serialize())
    assert len(m["Nodes"]) == 1 and m["Nodes"][0]["Op"]["Type"] == "Add"
    ark.Model.reset()
    m = json.loads(ark.Model.get_model().compress().serialize())
    assert m["Nodes"] == []
    ark.set_rank(0)
    ark.set_world_size(1)
    assert ark.Model.get_rank() == 0 and ark.Model.get_world_size() == 1
    assert isinstance(ark.version(), str)


def test_planner_plan_and_context():
    a, b = ark.tensor([256, 256], ark.fp16), ark.tensor([256, 256], ark.fp16)
    with ark.PlannerContext(processor_range=[0, 8], sync=False,
                            config={"NumWarps": 8, "SramBytes": 0, "Tile": [64, 256], "NumTasks": 4}):
        c = ark.add(a, b)
    ark.relu(c)          # no context config: the installed rule is asked about this one only
    seen = []

    def rule(op_json, arch):
        seen.append((json.loads(op_json)["Type"], arch))
        return ""

    pl = ark.Planner(arch="ROCM_950", num_processors=256)
    pl.install_config_rule(rule)
    plan = pl.plan()
    assert seen == [("Relu", "ROCM_950")]
    # NumProcessors of a plan is the highest processor any task uses, not the device's count
    assert plan.architecture == "ROCM_950" and plan.num_processors == 8
    assert plan.rank == 0 and plan.world_size == 1 and plan.num_warps_per_processor == 8
    assert len(plan.task_infos) == 2 and plan.task_infos[0]["NumWarps"] == 8
    assert plan.task_infos[0]["Ops"][0]["Config"]["Tile"] == [64, 256]
    assert plan.processor_groups[0]["ProcessorRange"] == [0, 8]
    again = ark.Plan.from_str(str(plan))
    assert again.plan == plan.plan
    empty = ark.Plan(None)
    assert empty.task_infos == [] and empty.architecture == "ANY"


def test_plan_from_file(tmp_path):
    ark.relu(t64())
    plan = ark.Planner(arch="ROCM_950", num_processors=256).plan()
    f = tmp_path / "plan.json"
    f.write_text(str(plan))
    assert ark.Plan.from_file(str(f)).plan == plan.plan


class _Linear(ark.Module):
    def __init__(self, k, n):
        super().__init__()
        self.weight = ark.parameter([k, n], ark.fp16)
        self.scratch = ark.tensor([k, n], ark.fp16)  # a plain tensor is not a parameter

    def forward(self, x):
        return ark.matmul(x, self.weight)


class _Mlp(ark.Module):
    def __init__(self):
        super().__init__()
        self.up = _Linear(64, 128)
        self.down = _Linear(128, 64)
        self.bias = ark.parameter([1, 64], ark.fp16)

    def forward(self, x):
        return ark.add(self.down(ark.relu(self.up(x))), self.bias)


def test_module_tree_and_params_dict():
    mlp = _Mlp()
    assert list(mlp.sub_modules) == ["up", "down"]
    assert sorted(mlp.params_dict()) == ["bias", "down.weight", "up.weight"]
    assert sorted(mlp.params_dict("mlp.")) == ["mlp.bias", "mlp.down.weight", "mlp.up.weight"]
    y = mlp(ark.tensor([32, 64], ark.fp16))
    assert y.shape() == [32, 64]
    with pytest.raises(TypeError):
        mlp.register_module("x", 3)
    with pytest.raises(TypeError):
        mlp.register_parameter("x", ark.tensor([1], ark.fp16))
    # before launch a state dict has shapes and types but no data; loading refuses
    sd = mlp.state_dict()
    assert sd["up.weight"].shape == (64, 128) and sd["up.weight"].dtype == np.float16
    with pytest.raises(RuntimeError):
        mlp.load_state_dict({k: np.zeros(v.shape, v.dtype) for k, v in sd.items()})


def test_save_load_round_trip(tmp_path):
    sd = {"w": np.arange(12, dtype=np.float16).reshape(3, 4)}
    f = str(tmp_path / "sd.pkl")
    ark.save(sd, f)
    back = ark.load(f)
    assert list(back) == ["w"] and np.array_equal(back["w"], sd["w"])


def test_runtime_refuses_before_launch():
    rt = ark.Runtime.get_runtime()
    assert rt is ark.Runtime.get_runtime()
    assert rt.state == ark.Runtime.State.Init and not rt.launched() and not rt.running()
    with pytest.raises(RuntimeError, match="not launched"):
        rt.run()
    with pytest.raises(RuntimeError, match="not launched"):
        rt.barrier()
    rt.wait()           # a warning, not an error
    assert rt.stop() is None
    rt.reset()
    assert rt.state == ark.Runtime.State.Init


def test_load_refuses_a_pickle_that_names_other_globals(tmp_path):
    import pickle

    class _Payload:
        def __reduce__(self):
            return (print, ("code from the file ran",))

    f = tmp_path / "bad.pkl"
    f.write_bytes(pickle.dumps({"w": _Payload()}))
    with pytest.raises(pickle.UnpicklingError, match="refusing"):
        ark.load(str(f))
    # arrays of every storage type the tensors use, nested containers and numpy scalars pass
    sd = {"a": np.ones((2, 3), np.float32), "b": np.arange(4, dtype=np.int32),
          "c": {"d": [np.float16(1.5), (1, 2.0, "s", None, True)]}}
    g = str(tmp_path / "good.pkl")
    ark.save(sd, g)
    back = ark.load(g)
    assert np.array_equal(back["a"], sd["a"]) and back["c"]["d"][0] == np.float16(1.5)
    assert back["c"]["d"][1] == (1, 2.0, "s", None, True)


def test_runtime_transition_table_is_total_and_matches_the_reference_life_cycle():
    """Every (state, call) pair has an entry; the end states are the ones
    python/ark/runtime.py:60-168 reaches (stop leaves LaunchedNotRunning, run refuses unless
    launched and idle, wait/stop/launch in the wrong state are skipped)."""
    S, T = ark.Runtime.State, ark.Runtime._TABLE
    calls = ["launch", "run", "wait", "barrier", "stop"]
    assert sorted(T, key=str) == sorted(((s, c) for s in S for c in calls), key=str)
    ends = {(s, c): T[(s, c)][1] for s in S for c in calls}
    assert ends[(S.Init, "launch")] == S.LaunchedNotRunning
    assert ends[(S.LaunchedNotRunning, "run")] == S.Running
    assert ends[(S.Running, "wait")] == S.LaunchedNotRunning
    assert ends[(S.Running, "stop")] == ends[(S.LaunchedNotRunning, "stop")] == S.LaunchedNotRunning
    refused = {k for k, (a, _) in T.items() if a is ark.Runtime._refuse}
    assert refused == {(S.Init, "run"), (S.Init, "barrier"), (S.Running, "run"), (S.Running, "barrier")}
    skipped = {k for k, (a, _) in T.items() if a is None}
    assert skipped == {(S.LaunchedNotRunning, "launch"), (S.Running, "launch"), (S.Init, "wait"),
                       (S.LaunchedNotRunning, "wait"), (S.Init, "stop")}
    assert all(ends[k] == k[0] for k in refused | skipped)


def test_module_reassignment_and_a_module_without_forward():
    m = _Mlp()
    first = m.up
    m.up = _Linear(64, 32)                       # replaces the entry, keeps its position
    assert list(m.sub_modules) == ["up", "down"] and m.sub_modules["up"] is not first
    assert list(m.params_dict()) == ["up.weight", "down.weight", "bias"]   # sub-modules first
    assert ark.Module()() is None
