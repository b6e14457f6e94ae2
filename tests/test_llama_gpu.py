"""GPU parity of the Llama-shaped compositions (SwiGLU feed-forward, attention,
decoder layer) run as ONE plan in the persistent loop kernel, against the CPU
oracle evaluating the same compositions op by op.

The reference has no numeric test for these (examples/llama/model_test.py
compares against a PyTorch checkpoint that is not available and prints the
differences); parity here is pinned by the oracle's per-op functions, each of
which is pinned separately by the reference's op-test baselines.

Metric for a whole composition: outputs are sums of thousands of rounded
terms, so single elements near zero carry no relative meaning.  The tests
bound max|diff| / max|ref| and rms(diff) / rms(ref) by 1e-2 (the tolerance
the per-op GEMM tests use per element).
"""
import numpy as np
import pytest

import llama_ref as R
from helpers import make

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _run(m, feeds, fetch, loop_mode=True):
    from ark_amd import Executor
    ex = Executor(m.plan(device_id=0), device_id=0, loop_mode=loop_mode).compile()
    for t, a in feeds.items():
        ex.tensor_write(t, a)
    ex.launch()
    ex.run(1)
    ex.wait()
    out = ex.tensor_read(fetch)
    info = ex.info()
    ex.stop()
    return out, info


def _ffn_case(oracle, rows, dim, hidden, dtype, seed):
    x = make(oracle, (rows, dim), dtype, seed, "normal")
    w1 = make(oracle, (hidden, dim), dtype, seed + 1, "normal", scale=0.02)
    w2 = make(oracle, (dim, hidden), dtype, seed + 2, "normal", scale=0.02)
    w3 = make(oracle, (hidden, dim), dtype, seed + 3, "normal", scale=0.02)
    return x, w1, w2, w3


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_ffn_small(oracle, dtype):
    from ark_amd import Model, llama
    rows, dim, hidden = 256, 512, 768
    x, w1, w2, w3 = _ffn_case(oracle, rows, dim, hidden, dtype, 100)
    m = Model()
    tx = m.tensor([rows, dim], dtype)
    ff = llama.FeedForward(m, dim, hidden, dtype)
    out = ff.forward(tx)
    got, info = _run(m, {tx: x, ff.w1: w1, ff.w2: w2, ff.w3: w3}, out)
    ref = R.feed_forward(oracle, x, w1, w2, w3, dtype)
    mx, rms = R.composite_error(oracle, ref, got, dtype)
    assert mx <= TOL and rms <= TOL, (mx, rms)


@pytest.mark.parametrize("fused", [False, True])
def test_ffn_full_size_sampled_rows(oracle, fused):
    """x[8192,4096] bf16 -> 11008 -> 4096 in one loop kernel, as the reference's
    composition and as the fused path the benchmark times (SwiGLU as one GEMM pass);
    the oracle evaluates 256 sampled rows (every output column of those rows)."""
    from ark_amd import Model, llama
    dtype, rows, dim, hidden = "bf16", 8192, 4096, 11008
    x, w1, w2, w3 = _ffn_case(oracle, rows, dim, hidden, dtype, 200)
    m = Model()
    tx = m.tensor([rows, dim], dtype)
    ff = llama.FeedForward(m, dim, hidden, dtype)
    out = ff.forward(tx, fused=fused)
    got, info = _run(m, {tx: x, ff.w1: w1, ff.w2: w2, ff.w3: w3}, out)
    pick = np.sort(np.random.default_rng(7).choice(rows, 256, replace=False))
    pick[0], pick[-1] = 0, rows - 1
    ref = R.feed_forward(oracle, np.ascontiguousarray(x[pick]), w1, w2, w3, dtype)
    mx, rms = R.composite_error(oracle, ref, got[pick], dtype)
    assert mx <= TOL and rms <= TOL, (mx, rms)


def _layer_case(oracle, m, seq, dim, heads, hidden, dtype, seed):
    from ark_amd import llama
    blk = llama.TransformerBlock(m, dim, heads, hidden, dtype)
    vals = {}
    for i, (name, t) in enumerate(sorted(blk.params().items())):
        if name.endswith("_norm"):
            vals[name] = np.random.default_rng(seed + i).uniform(0.5, 1.5, t.shape).astype(np.float32)
        else:
            vals[name] = make(oracle, tuple(t.shape), dtype, seed + i, "normal", scale=0.02)
    x = make(oracle, (1, seq, dim), dtype, seed + 50, "normal")
    freqs = llama.precompute_freqs_cis(dim // heads, seq)
    mask = llama.causal_mask(seq, -np.inf)
    return blk, vals, x, freqs, mask


@pytest.mark.parametrize("fused", [False, True, "attention"])
@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_decoder_layer_small(oracle, dtype, fused):
    from ark_amd import Model
    seq, dim, heads, hidden = 256, 512, 4, 768
    m = Model()
    blk, vals, x, freqs, mask = _layer_case(oracle, m, seq, dim, heads, hidden, dtype, 300)
    tx = m.tensor([1, seq, dim], dtype)
    tf = m.tensor([1, seq, 1, dim // heads], dtype)
    tm = m.tensor([1, 1, seq, seq], dtype)
    out = blk.forward(tx, tf, tm, fused=fused, causal=(fused == "attention"))
    feeds = {tx: x, tf: oracle.to_storage(freqs, dtype), tm: oracle.to_storage(mask, dtype)}
    if fused == "attention":
        del feeds[tm]  # the attention op applies the causal mask itself: no mask tensor in the plan
    feeds.update({t: vals[name] for name, t in blk.params().items()})
    got, info = _run(m, feeds, out)
    ref = R.transformer_block(oracle, x, vals, freqs, mask, heads, dtype)
    mx, rms = R.composite_error(oracle, ref, got, dtype)
    assert mx <= TOL and rms <= TOL, (mx, rms)


@pytest.mark.parametrize("fused", [False, True, "attention", "side_by_side"])
def test_decoder_layer_full_size_sampled_rows(oracle, fused):
    """Llama-2-7B layer shape: seq 2048, d 4096, 32 heads x 128, SwiGLU 11008,
    bf16, RoPE base 10000, causal mask.  The oracle evaluates 256 sampled query
    positions against the whole sequence's keys and values.  "side_by_side": the attention-op
    plan with the query and key projections on 256x256 tiles on the two halves of the processors
    at the same time (no barrier between them)."""
    from ark_amd import Model
    pair_on = None
    if fused == "side_by_side":
        fused, pair_on = "attention", 256
    dtype, seq, dim, heads, hidden = "bf16", 2048, 4096, 32, 11008
    m = Model()
    blk, vals, x, freqs, mask = _layer_case(oracle, m, seq, dim, heads, hidden, dtype, 400)
    tx = m.tensor([1, seq, dim], dtype)
    tf = m.tensor([1, seq, 1, dim // heads], dtype)
    tm = m.tensor([1, 1, seq, seq], dtype)
    out = blk.forward(tx, tf, tm, fused=fused, causal=(fused == "attention"), pair_on=pair_on)
    feeds = {tx: x, tf: oracle.to_storage(freqs, dtype), tm: oracle.to_storage(mask, dtype)}
    if fused == "attention":
        del feeds[tm]  # the attention op applies the causal mask itself: no mask tensor in the plan
    feeds.update({t: vals[name] for name, t in blk.params().items()})
    got, info = _run(m, feeds, out)
    if pair_on:
        import json
        from ark_amd import plan_schedule
        groups = json.loads(m.plan(device_id=0))["ProcessorGroups"]
        assert [g["ProcessorRange"] for g in groups[1:3]] == [[0, 128], [128, 256]]
    pick = np.sort(np.random.default_rng(9).choice(seq, 256, replace=False))
    pick[0], pick[-1] = 0, seq - 1
    ref = R.transformer_block(oracle, x, vals, freqs, mask, heads, dtype, q_rows=pick)
    mx, rms = R.composite_error(oracle, ref, got[:, pick], dtype)
    assert mx <= TOL and rms <= TOL, (mx, rms)


@pytest.mark.parametrize("fused", [False, True, "attention"])
def test_separate_kernels_match_loop_kernel(oracle, fused):
    """The plan's ops launched one kernel per op give the loop kernel's result
    bit for bit (same bodies, same task order inside each op)."""
    import torch
    from ark_amd import Model, Executor
    dtype = "bf16"
    seq, dim, heads, hidden = 256, 512, 4, 768
    m = Model()
    blk, vals, x, freqs, mask = _layer_case(oracle, m, seq, dim, heads, hidden, dtype, 500)
    tx = m.tensor([1, seq, dim], dtype)
    tf = m.tensor([1, seq, 1, dim // heads], dtype)
    tm = m.tensor([1, 1, seq, seq], dtype)
    out = blk.forward(tx, tf, tm, fused=fused, causal=(fused == "attention"))
    feeds = {tx: x, tf: oracle.to_storage(freqs, dtype), tm: oracle.to_storage(mask, dtype)}
    if fused == "attention":
        del feeds[tm]  # the attention op applies the causal mask itself: no mask tensor in the plan
    feeds.update({t: vals[name] for name, t in blk.params().items()})
    plan = m.plan(device_id=0)
    got_loop, _ = _run(m, feeds, out)
    ex = Executor(plan, device_id=0, loop_mode=False).compile()
    for t, a in feeds.items():
        ex.tensor_write(t, a)
    ex.run_separate(1)
    torch.cuda.synchronize()
    got_sep = ex.tensor_read(out)
    assert np.array_equal(got_loop, got_sep)
