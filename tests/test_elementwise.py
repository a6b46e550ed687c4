"""Fused residual-add + RMSNorm and SiLU-mul kernels against the reference's op sequence.

Oracle: `oracle/cpu_path.add_rmsnorm` / `silu_mul` = the reference's torch ops
(examples/pretrain/hf_template/modeling_qwen3sa.py:64-79, :507-514, :946, :952) on the CPU in the
input dtype.  Pins of the oracle (CPU tests): an fp64 closed form, scale invariance of the norm,
SiLU special values.  GPU tests: bit-identical to the oracle except where the fp32 summation
order / the exponential differ in the last place: at most 0.5 % of the elements, each by one
unit in the last place of the rounded intermediate (at most two of the result).
"""
import pytest
import torch

from oracle import cpu_path


def test_oracle_rmsnorm_closed_form():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 96, generator=g, dtype=torch.float64)
    r = torch.randn(5, 96, generator=g, dtype=torch.float64)
    w = torch.randn(96, generator=g, dtype=torch.float64)
    s, y = cpu_path.add_rmsnorm(x.float(), r.float(), w.float(), 1e-6)
    t = x + r
    exp = w * t / torch.sqrt((t * t).mean(-1, keepdim=True) + 1e-6)
    assert torch.allclose(s.double(), t, atol=1e-6)
    assert torch.allclose(y.double(), exp, atol=1e-5, rtol=1e-5)
    # scale invariance (eps aside): norm(4 x) == norm(x)
    _, y4 = cpu_path.add_rmsnorm(4 * x.float(), None, w.float(), 0.0)
    _, y1 = cpu_path.add_rmsnorm(x.float(), None, w.float(), 0.0)
    assert torch.allclose(y4, y1, atol=1e-5, rtol=1e-5)


def test_oracle_silu_values():
    gate = torch.tensor([0.0, 1.0, -1.0, 20.0, -20.0])
    up = torch.tensor([3.0, 2.0, 2.0, 1.0, 1.0])
    out = cpu_path.silu_mul(gate, up)
    e = torch.tensor(1.0).exp()
    exp = torch.tensor([0.0, 2.0 / (1 + 1 / e), -2.0 / (1 + e), 20.0, -20.0 * torch.tensor(-20.0).exp()])
    assert torch.allclose(out, exp, atol=1e-6, rtol=1e-5)


def _ulp_check(got, exp, max_frac):
    got, exp = got.cpu(), exp.cpu()
    diff = got != exp
    frac = diff.float().mean().item()
    if diff.any():
        a, b = got[diff].float(), exp[diff].float()
        mag = torch.maximum(a.abs(), b.abs())
        emin, mant = (-126, 7) if got.dtype == torch.bfloat16 else (-14, 10)   # subnormals share one spacing
        ulp = torch.exp2(torch.floor(torch.log2(mag.clamp_min(1e-38))).clamp_min(emin) - mant)
        # one unit in the last place of the normalised value can be two of the product with the
        # weight when the product falls into the binade below
        assert ((a - b).abs() <= 2 * ulp * 1.001).all(), "a mismatch larger than two units in the last place"
    assert frac <= max_frac, f"{frac:.4%} of the elements differ"
    return frac


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,H", [(1, 64), (7, 2560), (33, 4096), (5, 8192), (300, 520)])
@pytest.mark.parametrize("with_res", [True, False])
def test_gpu_add_rmsnorm(dtype, rows, H, with_res):
    from ksa_amd.elementwise import add_rmsnorm
    g = torch.Generator().manual_seed(rows * 31 + H)
    x = (torch.randn(2, rows, H, generator=g) * 1.5).to(dtype)
    r = torch.randn(2, rows, H, generator=g).to(dtype) if with_res else None
    w = (1 + 0.1 * torch.randn(H, generator=g)).to(dtype)
    s_exp, y_exp = cpu_path.add_rmsnorm(x, r, w, 1e-6)
    s, y = add_rmsnorm(x.cuda(), r.cuda() if with_res else None, w.cuda(), 1e-6)
    assert torch.equal(s.cpu(), s_exp), "the residual sum must be bit-exact"
    _ulp_check(y, y_exp, 5e-3)


@pytest.mark.gpu
def test_gpu_add_rmsnorm_strided_rows_and_errors():
    from ksa_amd import KsaError
    from ksa_amd.elementwise import add_rmsnorm
    big = torch.randn(6, 3 * 256, generator=torch.Generator().manual_seed(1)).bfloat16().cuda()
    x = big[:, 256:512]                       # row stride 768
    w = torch.ones(256, dtype=torch.bfloat16, device="cuda")
    _, y = add_rmsnorm(x, None, w)
    _, y_exp = cpu_path.add_rmsnorm(x.cpu(), None, w.cpu())
    _ulp_check(y, y_exp, 5e-3)
    with pytest.raises(KsaError):
        add_rmsnorm(torch.zeros(2, 12, dtype=torch.bfloat16, device="cuda"), None,
                    torch.ones(12, dtype=torch.bfloat16, device="cuda"))      # H not a multiple of 8
    with pytest.raises(KsaError):
        add_rmsnorm(torch.zeros(2, 16384, dtype=torch.bfloat16, device="cuda"), None,
                    torch.ones(16384, dtype=torch.bfloat16, device="cuda"))   # H above the supported size


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,I", [(1, 8), (9, 9728), (130, 2056)])
def test_gpu_silu_mul(dtype, rows, I):
    from ksa_amd.elementwise import silu_mul
    g = torch.Generator().manual_seed(rows + I)
    gu = (torch.randn(rows, 2 * I, generator=g) * 3).to(dtype)
    gate, up = gu[:, :I], gu[:, I:]            # halves of one fused projection output
    exp = cpu_path.silu_mul(gate, up)
    gug = gu.cuda()
    got = silu_mul(gug[:, :I], gug[:, I:])
    _ulp_check(got, exp, 5e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,N", [(8, 151936), (1, 8), (3, 1000), (5, 8192 + 3), (16, 5)])
def test_gpu_argmax_rows(dtype, rows, N):
    """The greedy token choice against torch.argmax on the CPU (first index among equal values:
    16-bit logits tie often), with the row maximum planted at both ends, inside a tail that is
    shorter than one 16-byte item, and doubled."""
    from ksa_amd.elementwise import argmax_rows
    g = torch.Generator().manual_seed(rows * 1000 + N)
    Np = (N + 7) // 8 * 8
    x = torch.randn(rows, Np, generator=g).to(dtype)[:, :N]   # rows start 16-byte aligned
    x[0, N - 1] = 30.0
    if rows > 1:
        x[1, 0] = 30.0
    if rows > 2:
        x[2, N // 2] = 30.0
        x[2, N - 1] = 30.0                                    # the first of two equal maxima wins
    def dev(t):  # same padded row stride on the GPU (a plain .cuda() would pack the rows)
        buf = torch.zeros(rows, Np, dtype=dtype, device="cuda")
        buf[:, :N] = t
        return buf[:, :N]

    got = argmax_rows(dev(x)).cpu()
    want = x.float().argmax(-1)
    assert got.dtype == torch.long and torch.equal(got, want), (got, want)
    if rows > 3 and N > 20:
        x[3, 17] = float("nan")                               # a NaN counts as the largest value
        assert int(argmax_rows(dev(x))[3]) == 17 == int(x.float().argmax(-1)[3])
