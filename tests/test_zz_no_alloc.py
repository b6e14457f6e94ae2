"""The skinny matmul through the entry point that allocates nothing (arkmi_gemv_static: its
split-K partial sums and arrival counters live in a fixed array inside the library) against
arkmi_gemv with a caller-provided workspace: bit for bit, on two calls in a row, the second
with a smaller input, and a shape beyond the array's size is refused."""
import numpy as np
import pytest
import torch

from helpers import make, to_gpu

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_static_workspace_matches_caller_workspace(oracle, dtype):
    from ark_amd import ops
    shapes = [(8, 4096, 11008, 0), (3, 1024, 1536, 37)]  # (m, n, k, tasks): the second call is smaller
    for m, n, k, tasks in shapes:
        x = to_gpu(make(oracle, (m, k), dtype, seed=61, dist="normal"), dtype)
        w = to_gpu(make(oracle, (k, n), dtype, seed=62, dist="normal", scale=0.02), dtype)
        want = ops.gemv(x, w, num_tasks=tasks)
        out = torch.full_like(want, float("nan"))
        got = ops.gemv_static(x, w, out, num_tasks=tasks)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (m, n, k)
    # and once more with the first shape: the array now holds the smaller call's leftovers
    m, n, k, tasks = shapes[0]
    x = to_gpu(make(oracle, (m, k), dtype, seed=63, dist="normal"), dtype)
    w = to_gpu(make(oracle, (k, n), dtype, seed=64, dist="normal", scale=0.02), dtype)
    want = ops.gemv(x, w, num_tasks=tasks)
    got = ops.gemv_static(x, w, torch.empty_like(want), num_tasks=tasks)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_static_workspace_rejects_oversized_shapes(oracle):
    from ark_amd import ops, ArkmiError
    limit = ops.gemv_static_limit()
    assert limit == 16 << 20
    # 16 rows x 262144 columns split over many tasks needs more partial-sum space than the array holds
    m, n, k = 16, 262144, 256
    x = torch.zeros(m, k, device="cuda", dtype=torch.bfloat16)
    w = torch.zeros(k, n, device="cuda", dtype=torch.bfloat16)
    out = torch.empty(m, n, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ArkmiError) as e:
        ops.gemv_static(x, w, out, num_tasks=1537)
    assert e.value.kind == "UnsupportedError" and "static workspace" in str(e.value)
