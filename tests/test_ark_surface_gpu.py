"""The `ark`-named Python surface on the GPU: the runtime's life cycle
(python/ark/runtime.py:33-168, python/unittest/test_runtime.py:7-12), tensor I/O through numpy
and a Module's state dict, with the results checked against the CPU oracle."""
import numpy as np
import pytest

import ark_amd.ark as ark
from helpers import make

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def fresh():
    ark.init()
    yield
    ark.Runtime.get_runtime().reset()
    ark.init()


def test_runtime_empty_model():
    with ark.Runtime.get_runtime() as rt:
        rt.launch()
        rt.run()
        rt.stop()


class Mlp(ark.Module):
    def __init__(self, d, h):
        super().__init__()
        self.up = ark.parameter([d, h], ark.fp16)
        self.down = ark.parameter([h, d], ark.fp16)

    def forward(self, x):
        return ark.matmul(ark.relu(ark.matmul(x, self.up)), self.down)


def test_runtime_states_module_state_dict_and_numpy_io(oracle):
    m, d, h = 256, 512, 1024
    x = ark.tensor([m, d], ark.fp16)
    mlp = Mlp(d, h)
    y = mlp(x)
    rt = ark.Runtime.get_runtime()
    assert rt.state == ark.Runtime.State.Init
    rt.launch()
    assert rt.state == ark.Runtime.State.LaunchedNotRunning and rt.launched() and not rt.running()
    rt.launch()  # second launch: a warning and no change
    assert rt.state == ark.Runtime.State.LaunchedNotRunning

    sd = {"up": make(oracle, (d, h), "fp16", 11, scale=0.05),
          "down": make(oracle, (h, d), "fp16", 12, scale=0.05)}
    mlp.load_state_dict(sd)
    xs = make(oracle, (m, d), "fp16", 13)
    assert x.from_numpy(xs) is x
    back = mlp.state_dict()
    assert sorted(back) == ["down", "up"]
    assert np.array_equal(back["up"], sd["up"]) and np.array_equal(back["down"], sd["down"])
    assert np.array_equal(x.to_numpy(), xs)
    # from_numpy converts other element types to the tensor's
    x.from_numpy(xs.astype(np.float32))
    assert np.array_equal(x.to_numpy(), xs)

    rt.run(non_blocking=True)
    assert rt.running()
    with pytest.raises(RuntimeError, match="not launched"):
        rt.run()       # already running
    rt.wait()
    assert rt.state == ark.Runtime.State.LaunchedNotRunning
    got = y.to_numpy()
    hid = oracle.unary(oracle.matmul(xs, sd["up"], "fp16"), "relu", "fp16")
    ref = oracle.matmul(hid, sd["down"], "fp16")
    # Two chained matmuls: the second one sums 1024 products of rounded activations in another
    # order than the oracle, so small outputs differ by more than their own rounding; judged
    # against the largest output (a wrong operand, transposition or missing relu is O(1) there)
    diff = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    assert diff.max() <= 2e-3 * np.abs(ref.astype(np.float64)).max(), diff.max()

    # to_numpy into a caller's array, and its refusals
    dst = np.zeros((m, d), np.float16)
    assert y.to_numpy(dst) is dst and np.array_equal(dst, got)
    with pytest.raises(ValueError, match="shape"):
        y.to_numpy(np.zeros((d, m), np.float16))
    with pytest.raises(ValueError, match="dtype"):
        y.to_numpy(np.zeros((m, d), np.float32))
    with pytest.raises(ValueError, match="contiguous"):
        y.to_numpy(np.zeros((d, m), np.float16).T)
    with pytest.raises(ValueError, match="size"):
        x.from_numpy(np.zeros((m, d + 1), np.float16))

    ms = rt.stop()
    assert ms is not None and ms >= 0.0
    assert rt.launched()          # stop keeps the executor for another launch
    rt.launch()                   # already "launched": skipped, as in the reference
    rt.reset()
    assert rt.state == ark.Runtime.State.Init and rt.executor is None


def test_launch_with_a_given_plan_and_a_second_model_after_init(oracle):
    a = ark.tensor([128, 256], ark.fp16)
    b = ark.add(a, 1.0)
    plan = ark.Planner().plan()
    assert plan.architecture == "ROCM_950"
    with ark.Runtime() as rt:
        rt.launch(plan=plan)
        xs = make(oracle, (128, 256), "fp16", 5)
        a.from_numpy(xs)
        rt.run(iter=3)
        assert np.array_equal(b.to_numpy(), oracle.scalar(xs, 1.0, "add", "fp16"))
    ark.init()
    c = ark.tensor([64, 64], ark.fp32)
    d = ark.mul(c, 2.0)
    with ark.Runtime() as rt:
        rt.launch()
        cs = make(oracle, (64, 64), "fp32", 6)
        c.from_numpy(cs)
        rt.run()
        assert np.array_equal(d.to_numpy(), oracle.scalar(cs, 2.0, "mul", "fp32"))
