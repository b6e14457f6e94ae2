"""The XCD-aware order of matmul tiles in the loop kernel: the tile a task computes is permuted so
that the tiles one XCD works on at a time form a compact block; the arithmetic of a tile does not
change, so every result must equal, bit for bit, the one of the plain order (ARKMI_GEMM_XCD=0),
which tests/test_gemm_gpu.py and tests/test_executor_gpu.py hold against the oracle.  The reference
deals tiles in task order only (ark/codegen.cpp:318-385)."""
import json

import numpy as np
import pytest

from helpers import make

pytestmark = pytest.mark.gpu


def _run(plan, feeds, outs, iters=2):
    from ark_amd import Executor
    ex = Executor(plan, device_id=0).compile()
    for t, a in feeds:
        ex.tensor_write(t, a)
    ex.launch()
    ex.run(iters)
    ex.wait()
    got = [ex.tensor_read(t) for t in outs]
    ex.stop()
    return got


def _both_orders(monkeypatch, plan, feeds, outs):
    from ark_amd import plan_analysis
    ordered = plan_analysis(plan)["GemmXcdOrdered"]
    a = _run(plan, feeds, outs)
    monkeypatch.setenv("ARKMI_GEMM_XCD", "0")
    assert plan_analysis(plan)["GemmXcdOrdered"] == 0
    b = _run(plan, feeds, outs)
    monkeypatch.delenv("ARKMI_GEMM_XCD")
    for x, y in zip(a, b):
        assert np.array_equal(x, y)
    return ordered, a


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("m,n,k,trans_b", [
    (4096, 4096, 512, False),    # 256 tiles of 256x256: one full round
    (2048, 4096, 256, True),     # 256 tiles of 128x256
    (4096, 6144, 256, False),    # 384 tiles: one full round and half of one
    (8192, 4096, 128, True),     # 512 tiles: two full rounds
    (2048, 2048, 256, False),    # fewer tiles than workgroups
    (2304, 4096, 128, False),    # 9 tile rows: the band height must divide them
])
def test_matmul_same_bits_in_both_tile_orders(oracle, monkeypatch, dtype, m, n, k, trans_b):
    from ark_amd import Model
    a = make(oracle, (m, k), dtype, seed=1, dist="normal")
    b = make(oracle, (n, k) if trans_b else (k, n), dtype, seed=2, dist="normal", scale=0.1)
    mod = Model()
    ta, tb = mod.tensor([m, k], dtype), mod.tensor(list(b.shape), dtype)
    tc = mod.matmul(ta, tb, trans_other=trans_b)
    ordered, (c,) = _both_orders(monkeypatch, mod.plan(device_id=0), [(ta, a), (tb, b)], [tc])
    assert ordered == 1
    # and the tiles are where they belong: sampled rows against the oracle
    rows = np.sort(np.random.default_rng(0).choice(m, 24, replace=False))
    rows[0], rows[-1] = 0, m - 1
    ref = oracle.matmul(np.ascontiguousarray(a[rows]), b, dtype, trans_b=trans_b)
    rel, _, _ = oracle.max_rel_error(ref, np.ascontiguousarray(c[rows]), dtype)
    assert rel <= 1e-2


def test_split_k_swiglu_and_fused_followers_in_both_tile_orders(oracle, monkeypatch):
    """A SwiGLU front half (gate/up pair in one pass: 688 tiles, two full rounds and a part) and a
    matmul that splits K with the residual add fused behind it: the op behind a matmul goes by the
    tile the task computed, and both halves of a split meet on that tile."""
    from ark_amd import Model, llama
    dtype = "bf16"
    mod = Model()
    ff = llama.FeedForward(mod, 4096, 11008, dtype)
    tx = mod.tensor([2048, 4096], dtype)
    ty = ff.forward(tx, fused=True, residual=tx)
    feeds = [(tx, make(oracle, (2048, 4096), dtype, seed=3, dist="normal"))]
    for i, (name, t) in enumerate(ff.params().items()):
        feeds.append((t, make(oracle, tuple(t.shape), dtype, seed=10 + i, dist="normal", scale=0.03)))
    plan = mod.plan(device_id=0)
    cfgs = [o["Config"] for ti in json.loads(plan)["TaskInfos"] for o in ti["Ops"]]
    assert any(c.get("SplitK") == 2 for c in cfgs)
    ordered, _ = _both_orders(monkeypatch, plan, feeds, [ty])
    assert ordered >= 2
