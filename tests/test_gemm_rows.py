"""Few-rows GEMM (`ksa_gemm_rows`) against an fp64 product of the same 16-bit inputs.

The kernel accumulates in fp32 and rounds once; the reference's `F.linear` does the same up to
summation order, so the check is: |y - y64| <= one unit in the last place of the 16-bit result
(plus a small absolute term where the result cancels to near zero).
"""
import pytest
import torch


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(1, 16, 32), (8, 6144, 2560), (8, 2560, 4096), (8, 19456, 2560),
                                   (8, 2560, 9728), (16, 1000, 640), (3, 40, 96), (5, 151936, 2560)])
def test_gpu_linear_rows(dtype, M, N, K):
    from ksa_amd.gemm import linear_rows
    g = torch.Generator().manual_seed(M * 7 + N + K)
    x = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.05).to(dtype)
    y = linear_rows(x.cuda(), w.cuda()).cpu()
    ref = x.double() @ w.double().T
    mant = 7 if dtype == torch.bfloat16 else 10
    ulp = torch.exp2(torch.floor(torch.log2(ref.abs().clamp_min(1e-30))) - mant)
    err = (y.double() - ref).abs()
    assert (err <= ulp * 1.01 + 1e-3 * ref.abs().max() * 2.0 ** -mant).all(), float((err / ulp).max())


@pytest.mark.gpu
def test_gpu_linear_rows_views_and_errors():
    from ksa_amd import KsaError
    from ksa_amd.gemm import linear_rows
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 4, 256, generator=g).bfloat16().cuda()        # [b, q, K] -> 8 rows
    w = torch.randn(3 * 64, 256, generator=g).bfloat16().cuda()
    y = linear_rows(x, w[64:128])                                    # a row slice of a fused weight
    ref = (x.double() @ w[64:128].double().T)
    assert y.shape == (2, 4, 64) and (y.double() - ref).abs().max() <= 0.02 * ref.abs().max()
    with pytest.raises(AssertionError):
        linear_rows(torch.zeros(17, 64, dtype=torch.bfloat16, device="cuda"), w[:, :64].contiguous())
    with pytest.raises(KsaError):
        linear_rows(torch.zeros(2, 48, dtype=torch.bfloat16, device="cuda"),
                    torch.zeros(8, 48, dtype=torch.bfloat16, device="cuda"))   # K not a multiple of 32
