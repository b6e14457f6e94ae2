"""Shared helpers of the GPU parity tests: seeded inputs in storage dtypes and
the torch <-> numpy bridges (bf16 travels as uint16 bit patterns)."""
import numpy as np
import torch

TORCH_DT = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}


def make(oracle, shape, dtype, seed, dist="normal", lo=-1.0, hi=1.0, scale=1.0):
    """Seeded values from the counter-based generator the benchmark draws from too
    (ark_amd/prng.py), rounded once to the storage dtype; CPU oracle and GPU read the
    same bits.  Returns the numpy storage array."""
    from ark_amd import prng
    if dist == "normal":
        x = prng.normal(seed, tuple(shape), 0.0, scale)
    else:
        x = prng.uniform(seed, tuple(shape), lo, hi)
    return oracle.to_storage(x, dtype)


def to_gpu(a, dtype):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype == "bf16":
        t = t.view(torch.bfloat16)
    return t.cuda()


def to_np(t, dtype):
    t = t.detach().cpu().contiguous()
    if dtype == "bf16":
        return t.view(torch.uint16).numpy()
    return t.numpy()
