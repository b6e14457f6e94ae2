"""GPU parity of the fused attention op (softmax(q k^T * scale [+ causal mask]) v
over [batch, seq, heads, head_dim] tensors) against the chain the reference's
attention builds (examples/llama/model.py:421-443: transposes, Matmul, ScalarMul,
Add(mask), the five-op softmax of python/ark/ops.py:491-500, Matmul, transpose)
evaluated op by op on the CPU oracle.

The reference has no numeric test for this chain; each oracle op is pinned
separately by the reference's op-test baselines.  The chain rounds the scores to
the storage type four times before the second product (in bf16 that alone moves
a probability by up to ~2 %), the fused op keeps them in fp32 and rounds only
the probabilities.  Two bounds, on max|diff| / max|ref| and rms(diff) / rms(ref):
  against the chain:                         1e-2 (fp16), 3e-2 (bf16);
  against the same formula in float64 numpy: 2e-3 (fp16), 1e-2 (bf16),
and the fused op must be at least as close to float64 as the chain is (x1.25).
"""
import numpy as np
import pytest

import llama_ref as R
from helpers import make

pytestmark = pytest.mark.gpu


def ref_attention(O, q, k, v, scale, causal, dtype):
    b, sq, h, d = q.shape
    sk = k.shape[1]
    qt = np.ascontiguousarray(q.transpose(0, 2, 1, 3))
    kt = np.ascontiguousarray(k.transpose(0, 2, 3, 1))
    vt = np.ascontiguousarray(v.transpose(0, 2, 1, 3))
    scores = O.scalar(O.matmul(qt, kt, dtype), scale, "mul", dtype)
    if causal:
        mask = np.zeros((1, 1, sq, sk), np.float32)
        qi, ki = np.meshgrid(np.arange(sq), np.arange(sk), indexing="ij")
        mask[0, 0][ki > qi + (sk - sq)] = -np.inf
        scores = O.binary(scores, O.to_storage(mask, dtype), "add", dtype)
    out = O.matmul(R.softmax(O, scores, dtype), vt, dtype)
    return np.ascontiguousarray(out.transpose(0, 2, 1, 3))


def exact_attention(O, q, k, v, scale, causal, dtype):
    qf, kf, vf = (O.to_f32(a, dtype).astype(np.float64) for a in (q, k, v))
    s = np.einsum("bqhd,bkhd->bhqk", qf, kf) * scale
    sq, sk = s.shape[2:]
    if causal:
        qi, ki = np.meshgrid(np.arange(sq), np.arange(sk), indexing="ij")
        s[:, :, ki > qi + (sk - sq)] = -np.inf
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    return np.einsum("bhqk,bkhd->bqhd", p, vf)


def errors(O, ref_f, got, dtype):
    g = O.to_f32(got, dtype).astype(np.float64)
    d = g - ref_f
    return np.abs(d).max() / np.abs(ref_f).max(), np.sqrt((d * d).mean() / (ref_f * ref_f).mean())


def run_attention(q, k, v, scale, causal, dtype, loop_mode=True):
    from ark_amd import Model, Executor
    m = Model()
    tq, tk, tv = m.tensor(q.shape, dtype), m.tensor(k.shape, dtype), m.tensor(v.shape, dtype)
    out = m.attention(tq, tk, tv, scale, causal=causal)
    ex = Executor(m.plan(device_id=0), device_id=0, loop_mode=loop_mode).compile()
    for t, a in ((tq, q), (tk, k), (tv, v)):
        ex.tensor_write(t, a)
    ex.launch()
    ex.run(2)  # twice: the second pass must not depend on what the first left in LDS
    ex.wait()
    got = ex.tensor_read(out)
    ex.stop()
    return got


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(1, 256, 256, 2), (2, 200, 200, 3), (1, 128, 384, 1), (1, 64, 70, 2),
                                   (1, 1024, 1024, 4)])
def test_attention_matches_chain(oracle, dtype, causal, shape):
    b, sq, sk, h = shape
    q = make(oracle, (b, sq, h, 128), dtype, 81)
    k = make(oracle, (b, sk, h, 128), dtype, 82)
    v = make(oracle, (b, sk, h, 128), dtype, 83)
    scale = 1.0 / np.sqrt(128.0)
    got = run_attention(q, k, v, scale, causal, dtype)
    ref = ref_attention(oracle, q, k, v, scale, causal, dtype)
    mx, rms = R.composite_error(oracle, ref, got, dtype)
    tol = {"fp16": 1e-2, "bf16": 3e-2}[dtype]
    assert mx <= tol and rms <= tol, (mx, rms)
    exact = exact_attention(oracle, q, k, v, scale, causal, dtype)
    emx, erms = errors(oracle, exact, got, dtype)
    cmx, crms = errors(oracle, exact, ref, dtype)
    etol = {"fp16": 2e-3, "bf16": 1e-2}[dtype]
    assert emx <= etol and erms <= etol, (emx, erms)
    assert erms <= 1.25 * crms, (erms, crms)


def test_attention_one_hot_value_pick(oracle):
    """With keys that make one score dominate (q = 30 * k_j), the output row is the
    matching row of V to within the softmax tail: pins the key <-> value pairing
    of the second product, whose contraction order is permuted."""
    dtype = "bf16"
    sk = 192
    rng = np.random.default_rng(5)
    kf = rng.standard_normal((1, sk, 1, 128)).astype(np.float32)
    kf /= np.linalg.norm(kf, axis=-1, keepdims=True)
    pick = rng.permutation(sk)[:128]
    qf = 60.0 * kf[:, pick]
    v = make(oracle, (1, sk, 1, 128), dtype, 91)
    got = run_attention(oracle.to_storage(qf, dtype), oracle.to_storage(kf, dtype), v, 1.0, False, dtype)
    want = oracle.to_f32(v, dtype)[0, pick, 0]
    assert np.abs(oracle.to_f32(got, dtype)[0, :, 0] - want).max() <= 2e-2 * np.abs(want).max()


def test_attention_causal_first_row_is_first_value(oracle):
    """Query 0 sees key 0 only."""
    dtype = "fp16"
    q = make(oracle, (1, 256, 2, 128), dtype, 95)
    k = make(oracle, (1, 256, 2, 128), dtype, 96)
    v = make(oracle, (1, 256, 2, 128), dtype, 97)
    got = run_attention(q, k, v, 0.0883883, True, dtype)
    assert np.array_equal(got[0, 0], v[0, 0])


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(1, 2048, 2048, 32), (2, 1024, 1024, 12), (1, 640, 640, 8)])
def test_attention_same_bits_in_both_task_orders(oracle, monkeypatch, causal, shape):
    """The XCD-aware order of the attention tasks (the query blocks an XCD works on at a time belong
    to the same few heads) changes which workgroup computes a (head, query block), not how: the same
    bits as in plain task order (ARKMI_GEMM_XCD=0), on the decoder layer's shape (two full rounds of
    256 tasks), with a partial last round (192 tasks in a round of 192; 40 tasks), and a sampled
    head against float64."""
    from ark_amd import Model, plan_analysis
    b, sq, sk, h = shape
    dtype = "bf16"
    q = make(oracle, (b, sq, h, 128), dtype, 91)
    k = make(oracle, (b, sk, h, 128), dtype, 92)
    v = make(oracle, (b, sk, h, 128), dtype, 93)
    scale = 1.0 / np.sqrt(128.0)
    m = Model()
    tq, tk, tv = m.tensor(q.shape, dtype), m.tensor(k.shape, dtype), m.tensor(v.shape, dtype)
    m.attention(tq, tk, tv, scale, causal=causal)
    assert plan_analysis(m.plan(arch="ROCM_950", num_processors=256))["AttnXcdOrdered"] == 1
    got = run_attention(q, k, v, scale, causal, dtype)
    monkeypatch.setenv("ARKMI_GEMM_XCD", "0")
    plain = run_attention(q, k, v, scale, causal, dtype)
    assert np.array_equal(got, plain)
    hs = [0, h - 1]
    exact = exact_attention(oracle, q[:, :, hs], k[:, :, hs], v[:, :, hs], scale, causal, dtype)
    emx, erms = errors(oracle, exact, np.ascontiguousarray(got[:, :, hs]), dtype)
    assert emx <= 1e-2 and erms <= 1e-2, (emx, erms)
