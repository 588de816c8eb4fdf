"""Each kernel alone against a plain float32 formula, at sizes other than the engine's."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _ops():
    from sharpinference_amd import ops

    return ops


def _rand(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


@pytest.mark.parametrize("M", [1, 5, 16, 17, 40, 64])
@pytest.mark.parametrize("N,K", [(132, 128), (1000, 256), (5120, 1024), (20, 384)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_gemm_skinny(M, N, K, out_dtype):
    ops = _ops()
    x = _rand(M, K, dtype=torch.bfloat16, seed=M)
    w = _rand(N, K, dtype=torch.bfloat16, scale=0.1, seed=N)
    ref = x.float() @ w.float().T
    for R in (1, 2, 4):
        for NW in (4, 8, 16):
            got = ops.gemm_skinny(x, w, out_dtype, R=R, NW=NW).float()
            tol = 2e-2 if out_dtype == torch.bfloat16 else 1e-3
            assert float((got - ref).abs().max()) <= tol * float(ref.abs().max()), (M, N, K, R, NW)


def test_gemm_skinny_rows_do_not_depend_on_the_batch():
    ops = _ops()
    x = _rand(64, 512, dtype=torch.bfloat16, seed=3)
    w = _rand(516, 512, dtype=torch.bfloat16, scale=0.1, seed=4)
    full = ops.gemm_skinny(x, w, torch.float32)
    for m in (1, 7, 16, 33):
        part = ops.gemm_skinny(x[:m].contiguous(), w, torch.float32)
        assert torch.equal(part, full[:m]), m


@pytest.mark.parametrize("rows,E", [(8, 4), (64, 16), (33, 5), (1, 3)])
def test_gemm_skinny_grouped(rows, E):
    ops = _ops()
    N, K, T = 264, 256, 40
    g = torch.Generator().manual_seed(rows)
    x = _rand(T, K, dtype=torch.bfloat16, seed=1)
    w = _rand(E, N, K, dtype=torch.bfloat16, scale=0.1, seed=2)
    expert = torch.sort(torch.randint(0, E, (rows,), generator=g)).values
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    for e in range(E):
        offsets[e + 1] = offsets[e] + int((expert == e).sum())
    a_rows = torch.randint(0, T, (rows,), generator=g, dtype=torch.int32)
    ref = torch.stack([x[int(a_rows[i])].float() @ w[int(expert[i])].float().T for i in range(rows)])
    for R, NW in ((1, 16), (2, 8), (4, 4)):
        got = ops.gemm_skinny(x, w, torch.float32, a_rows=a_rows.to(DEV), offsets=offsets.to(DEV), n_rows=rows, R=R, NW=NW)
        assert float((got - ref).abs().max()) <= 1e-3 * float(ref.abs().max()), (R, NW)
