"""Llama-style building blocks expressed with the Model op API.

These are the callers of the hot path: the op-by-op compositions the reference
defines in Python (softmax: python/ark/ops.py:491-500; RMSNorm, SiLU, SwiGLU
feed-forward, attention and the decoder block: examples/llama/model.py:79-99,
281-333, 336-444, 447-485; rotary table: examples/llama/generator.py:20-27).

Every builder takes `fused`:
  fused=False  the reference's composition, one op per step (RMSNorm = 7 ops,
               softmax = 5 ops, SiLU = 2 ops, scale and mask as separate ops);
  fused=True   this backend's fused ops in place of those chains: rmsnorm as one
               op; attention as one op when the mask is causal (or absent), else
               softmax(scores * scale + mask) as one op with the keys consumed
               as the transposed GEMM operand; silu(w1 x) * (w3 x) as one GEMM pass;
               the rotation and the residual adds on the tiles of the GEMMs that
               produce their inputs.
Weights are stored [out, in] and used with trans_other=True, as the
reference's Linear does (examples/llama/model.py:275-278).
"""
import math

import numpy as np


def softmax(m, x, output=None, fused=False):
    """Softmax over the last axis (python/ark/ops.py:491-500)."""
    if fused:
        return m.softmax(x, output)
    mx = m.reduce_max(x, axis=-1)
    shifted = m.sub(x, mx, output)
    e = m.exp(shifted, shifted)
    s = m.reduce_sum(e, axis=-1)
    return m.div(e, s, e)


def rmsnorm(m, x, weight, dtype, eps=0.0, fused=False):
    """x * rsqrt(mean(x^2)) * weight with weight fp32 [1, 1, dim]
    (examples/llama/model.py:92-99; the reference adds no eps)."""
    if fused:
        return m.rmsnorm(x, weight, eps)
    if eps != 0.0:
        raise ValueError("the op-by-op RMSNorm of the reference has no eps")
    xf = m.cast(x, "fp32")
    x2 = m.mul(xf, xf)
    mean = m.reduce_mean(x2, axis=-1)
    rrms = m.rsqrt(mean)
    y = m.mul(xf, rrms)
    y = m.mul(y, weight, y)
    return m.cast(y, dtype)


def silu(m, x):
    """x * sigmoid(x), the sigmoid written to a tensor of its own
    (examples/llama/model.py:281-293)."""
    out = m.tensor(x.shape, x.dtype)
    return m.mul(x, m.sigmoid(x, out))


def linear(m, x, weight):
    return m.matmul(x, weight, trans_other=True)


class FeedForward:
    """w2(silu(w1 x) * w3 x) (examples/llama/model.py:296-333)."""

    def __init__(self, m, dim, hidden_dim, dtype):
        self.m, self.dtype = m, dtype
        self.w1 = m.tensor([hidden_dim, dim], dtype)
        self.w2 = m.tensor([dim, hidden_dim], dtype)
        self.w3 = m.tensor([hidden_dim, dim], dtype)

    def params(self):
        return {"w1": self.w1, "w2": self.w2, "w3": self.w3}

    def forward(self, x, fused=False, residual=None):
        m = self.m
        if fused == "follower":
            # Both projections back to back, and silu(g) * u as one op fused behind the
            # second one: in a context with sync(False) an elementwise op takes the GEMM's
            # output tiling and runs on each tile right after it is written, by the
            # workgroup that wrote it.
            g = linear(m, x, self.w1)
            with m.planner_context(sync=False):
                u = linear(m, x, self.w3)
                h = m.silu_mul(g, u)
        elif fused:
            # both projections and the gate in one GEMM pass: g and u never reach memory
            h = m.swiglu(x, self.w1, self.w3)
        if fused:
            if residual is None:
                return linear(m, h, self.w2)
            with m.planner_context(sync=False):
                return m.add(residual, linear(m, h, self.w2))
        x1 = silu(m, linear(m, x, self.w1))
        x2 = linear(m, x, self.w3)
        return linear(m, m.mul(x1, x2), self.w2)


class Attention:
    """Multi-head self-attention over a whole sequence, no KV cache
    (examples/llama/model.py:336-444)."""

    def __init__(self, m, dim, n_heads, dtype):
        self.m, self.dtype, self.dim, self.n_heads = m, dtype, dim, n_heads
        self.head_dim = dim // n_heads
        self.wq = m.tensor([dim, dim], dtype)
        self.wk = m.tensor([dim, dim], dtype)
        self.wv = m.tensor([dim, dim], dtype)
        self.wo = m.tensor([dim, dim], dtype)

    def params(self):
        return {"wq": self.wq, "wk": self.wk, "wv": self.wv, "wo": self.wo}

    def forward(self, x, freqs_cis, mask, fused=False, residual=None, causal=False, pair_on=None):
        """causal=True (fused path only) states that `mask` is the causal mask: the
        attention then runs as one op that applies it arithmetically, skips the key
        blocks above the diagonal and needs no transposes.  pair_on=P (fused path only): the
        number of processors the plan is made for; see below."""
        m = self.m
        bsz, seqlen, _ = x.shape
        h, hd = self.n_heads, self.head_dim
        # With 256x256 tiles one projection of this size may fill exactly half of the processors:
        # the query and key projections, which do not depend on each other, are then placed side by
        # side (ProcessorRange, the reference's planner-context mechanism,
        # python/ark/planner.py:110-170), and the loop kernel, which drops the barrier between
        # independent ops, runs them at the same time on full-size tiles instead of one after the
        # other on half-size ones.
        rows = bsz * seqlen
        side_by_side = (fused and freqs_cis is not None and pair_on is not None and pair_on % 2 == 0
                        and rows % 256 == 0 and self.dim % 256 == 0
                        and (rows // 256) * (self.dim // 256) == pair_on // 2)
        if side_by_side:
            big = {"NumWarps": 8, "SramBytes": 131072, "TileShapeMNK": [256, 256, 64], "NumTasks": pair_on // 2}
            half = pair_on // 2
            with m.planner_context(processor_range=[0, half], sync=False):
                with m.planner_context(config=big):
                    yq = linear(m, x, self.wq)
                xq = m.rope(m.reshape(yq, [bsz, seqlen, h, hd]), freqs_cis)
            with m.planner_context(processor_range=[half, pair_on], sync=False):
                with m.planner_context(config=big):
                    yk = linear(m, x, self.wk)
                xk = m.rope(m.reshape(yk, [bsz, seqlen, h, hd]), freqs_cis)
        elif fused and freqs_cis is not None:
            # the rotation rides on the projections' tiles (a tile spans whole heads)
            with m.planner_context(sync=False):
                xq = m.rope(m.reshape(linear(m, x, self.wq), [bsz, seqlen, h, hd]), freqs_cis)
            with m.planner_context(sync=False):
                xk = m.rope(m.reshape(linear(m, x, self.wk), [bsz, seqlen, h, hd]), freqs_cis)
        else:
            xq = m.reshape(linear(m, x, self.wq), [bsz, seqlen, h, hd])
            xk = m.reshape(linear(m, x, self.wk), [bsz, seqlen, h, hd])
            if freqs_cis is not None:
                xq = m.rope(xq, freqs_cis)
                xk = m.rope(xk, freqs_cis)
        xv = m.reshape(linear(m, x, self.wv), [bsz, seqlen, h, hd])
        if fused and (causal or mask is None):
            out = m.attention(xq, xk, xv, 1.0 / math.sqrt(hd), causal=causal)
            out = m.reshape(out, [bsz, seqlen, h * hd])
            if residual is None:
                return linear(m, out, self.wo)
            with m.planner_context(sync=False):
                return m.add(residual, linear(m, out, self.wo))
        xq = m.transpose(xq, [0, 2, 1, 3])
        values = m.transpose(xv, [0, 2, 1, 3])
        if fused:
            # keys stay [b, h, s, hd]: the GEMM reads them as the transposed operand, and
            # scale, mask and softmax are one pass over the scores
            keys = m.transpose(xk, [0, 2, 1, 3])
            scores = m.matmul(xq, keys, trans_other=True)
            scores = m.softmax(scores, output=scores, mask=mask, scale=1.0 / math.sqrt(hd))
        else:
            keys = m.transpose(xk, [0, 2, 3, 1])
            scores = m.matmul(xq, keys)
            scores = m.mul(scores, 1.0 / math.sqrt(hd))
            if mask is not None:
                scores = m.add(scores, mask)
            scores = softmax(m, scores, output=scores, fused=False)
        out = m.matmul(scores, values)
        out = m.transpose(out, [0, 2, 1, 3])
        out = m.reshape(out, [bsz, seqlen, h * hd])
        if residual is None:
            return linear(m, out, self.wo)
        with m.planner_context(sync=False):
            return m.add(residual, linear(m, out, self.wo))


class TransformerBlock:
    """x + attention(norm(x)), then h + ffn(norm(h))
    (examples/llama/model.py:447-485)."""

    def __init__(self, m, dim, n_heads, hidden_dim, dtype, norm_eps=0.0):
        self.m, self.dtype, self.norm_eps = m, dtype, norm_eps
        self.attention = Attention(m, dim, n_heads, dtype)
        self.feed_forward = FeedForward(m, dim, hidden_dim, dtype)
        self.attention_norm = m.tensor([1, 1, dim], "fp32")
        self.ffn_norm = m.tensor([1, 1, dim], "fp32")

    def params(self):
        p = {"attention_norm": self.attention_norm, "ffn_norm": self.ffn_norm}
        p.update({"attention." + k: v for k, v in self.attention.params().items()})
        p.update({"feed_forward." + k: v for k, v in self.feed_forward.params().items()})
        return p

    def forward(self, x, freqs_cis, mask, fused=False, causal=False, pair_on=None):
        """pair_on=P (fused path): the plan is made for P processors; projections that fill half of
        them on full-size tiles are placed side by side (Attention.forward)."""
        m = self.m
        nx = rmsnorm(m, x, self.attention_norm, self.dtype, self.norm_eps, fused)
        if not fused:
            h = m.add(x, self.attention.forward(nx, freqs_cis, mask, fused))
            nh = rmsnorm(m, h, self.ffn_norm, self.dtype, self.norm_eps, fused)
            return m.add(h, self.feed_forward.forward(nh, fused))
        # the residual adds ride on the output projections' tiles
        h = self.attention.forward(nx, freqs_cis, mask, fused, residual=x, causal=causal, pair_on=pair_on)
        nh = rmsnorm(m, h, self.ffn_norm, self.dtype, self.norm_eps, fused)
        return self.feed_forward.forward(nh, fused, residual=h)


def precompute_freqs_cis(head_dim, seqlen, theta=10000.0):
    """Rotary table [1, seqlen, 1, head_dim] fp32 with (cos, sin) interleaved:
    element 2j is cos(t * theta^(-2j/d)), element 2j+1 its sin
    (examples/llama/generator.py:20-27, layout model_test.py:379-384)."""
    j = np.arange(0, head_dim, 2, dtype=np.float64)[: head_dim // 2]
    freqs = 1.0 / (theta ** (j / head_dim))
    ang = np.outer(np.arange(seqlen, dtype=np.float64), freqs)
    out = np.empty((seqlen, head_dim), np.float32)
    out[:, 0::2] = np.cos(ang)
    out[:, 1::2] = np.sin(ang)
    return out.reshape(1, seqlen, 1, head_dim)


def causal_mask(seqlen, dtype_min):
    """[1, 1, seqlen, seqlen]: `dtype_min` above the diagonal, 0 elsewhere.  The
    reference fills -inf (model_test.py:507-511); a finite minimum keeps rows
    NaN-free when the mask is added in the storage type."""
    mask = np.zeros((seqlen, seqlen), np.float32)
    mask[np.triu_indices(seqlen, k=1)] = dtype_min
    return mask.reshape(1, 1, seqlen, seqlen)
