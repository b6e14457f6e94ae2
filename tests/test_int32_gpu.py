"""INT32 arithmetic on the GPU (Add, Sub, Mul, Div, ScalarAssign/Add/Mul on INT32 tensors; the
reference instantiates its broadcast kernels with the generic `a + b` ... `a / b` functors for this
type, ark/include/kernels/common/type_intrinsics.h:174-252, and casts a scalar op's float value to
the element type, ark/include/kernels/scalar.h:13-41; it has no test of its own for INT32).  Bit for
bit against the oracle, which tests/test_oracle_cpu.py pins by Python's integers."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _run(model, feeds, outs):
    from ark_amd import Executor
    ex = Executor(model.plan(device_id=0)).compile()
    for t, a in feeds:
        ex.tensor_write(t, a)
    ex.launch()
    ex.run(1)
    ex.wait()
    got = [ex.tensor_read(t) for t in outs]
    ex.stop()
    return got


@pytest.mark.parametrize("shape,bshape", [((4, 300), (4, 300)), ((2, 3, 64, 1024), (2, 3, 64, 1024)),
                                          ((8, 2048), (1, 2048)), ((8, 2048), (8, 1)), ((5, 7), (1,))])
def test_int32_binary_ops(oracle, shape, bshape):
    """Values over the whole 32-bit range (sums and products wrap around, quotients truncate toward
    zero), dense and broadcast operands, a vectorised and a ragged shape."""
    from ark_amd import Model
    rng = np.random.default_rng(11)
    a = rng.integers(-2 ** 31, 2 ** 31, shape, dtype=np.int64).astype(np.int32)
    b = rng.integers(-2 ** 31, 2 ** 31, bshape, dtype=np.int64).astype(np.int32)
    small = rng.integers(1, 1000, bshape).astype(np.int32) * rng.choice([-1, 1], bshape).astype(np.int32)
    m = Model()
    ta, tb, ts = m.tensor(list(shape), "int32"), m.tensor(list(bshape), "int32"), m.tensor(list(bshape), "int32")
    outs = [m.add(ta, tb), m.sub(ta, tb), m.mul(ta, tb), m.div(ta, ts), m.div(ta, tb)]
    got = _run(m, [(ta, a), (tb, b), (ts, small)], outs)
    want = [oracle.binary(a, b, "add", "int32"), oracle.binary(a, b, "sub", "int32"),
            oracle.binary(a, b, "mul", "int32"), oracle.binary(a, small, "div", "int32"),
            oracle.binary(a, b, "div", "int32")]
    for g, w, name in zip(got, want, ("add", "sub", "mul", "div small", "div")):
        assert g.dtype == np.int32 and np.array_equal(g.reshape(w.shape), w), name


def test_int32_scalar_ops_and_division_corner_cases(oracle):
    from ark_amd import Model
    rng = np.random.default_rng(12)
    x = rng.integers(-2 ** 31, 2 ** 31, (16, 520), dtype=np.int64).astype(np.int32)
    m = Model()
    tx = m.tensor([16, 520], "int32")
    outs = [m.add(tx, -7.9), m.mul(tx, 3.5), m.mul(tx, -100000)]
    # x / 0 and INT_MIN / -1 (undefined in C) give 0; 7 / 2, -7 / 2, 7 / -2, -7 / -2 truncate
    num = np.array([[7, -7, 7, -7, 5, -2 ** 31, 2 ** 31 - 1, 0]], np.int32)
    den = np.array([[2, 2, -2, -2, 0, -1, -1, 0]], np.int32)
    tn, td = m.tensor([1, 8], "int32"), m.tensor([1, 8], "int32")
    outs.append(m.div(tn, td))
    got = _run(m, [(tx, x), (tn, num), (td, den)], outs)
    assert np.array_equal(got[0], oracle.scalar(x, -7.9, "add", "int32"))
    assert np.array_equal(got[1], oracle.scalar(x, 3.5, "mul", "int32"))
    assert np.array_equal(got[2], oracle.scalar(x, -100000, "mul", "int32"))
    assert list(got[3].reshape(-1)) == [3, -3, -3, 3, 0, 0, -(2 ** 31 - 1), 0]
    assert np.array_equal(got[3], oracle.binary(num, den, "div", "int32"))


def test_int32_transcendental_ops_are_refused(oracle):
    from ark_amd import Model, Executor
    m = Model()
    try:
        m.exp(m.tensor([4, 64], "int32"))
        plan = m.plan(device_id=0)
    except Exception:
        return  # refused at model or plan time
    with pytest.raises(Exception):
        Executor(plan).compile()
