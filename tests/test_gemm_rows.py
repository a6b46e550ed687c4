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
                                   (8, 2560, 9728), (16, 1000, 640), (3, 40, 96), (5, 151936, 2560),
                                   # 17 to 128 rows: the wide form (row blocks of 16; K with a short last chunk;
                                   # column tiles that end inside a wave's 16 columns)
                                   (17, 16, 32), (72, 6144, 2560), (72, 2560, 4096), (72, 19456, 2560),
                                   (72, 2560, 9728), (64, 1000, 640), (33, 40, 96), (128, 300, 1120),
                                   (100, 2050, 544), (80, 151936, 2560), (112, 130, 1024)])
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
        linear_rows(torch.zeros(129, 64, dtype=torch.bfloat16, device="cuda"), w[:, :64].contiguous())
    with pytest.raises(KsaError):
        linear_rows(torch.zeros(2, 48, dtype=torch.bfloat16, device="cuda"),
                    torch.zeros(8, 48, dtype=torch.bfloat16, device="cuda"))   # K not a multiple of 32


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(8, 2560, 4096), (8, 2560, 9728), (1, 2560, 4096), (16, 1024, 1024), (3, 64, 512),
                                   (2, 8192, 1024), (72, 2560, 4096), (72, 2560, 9728), (40, 1024, 2048),
                                   (128, 512, 4096)])
def test_gpu_deferred_product_into_add_rmsnorm(dtype, M, N, K):
    """A product left as K-split partial sums and added inside `add_rmsnorm`: the sum with the
    residual is bit for bit what the reduced product followed by `add_rmsnorm` gives (same
    summation order over the splits, same rounding points); the normalised output may differ by
    one unit in the last place of the rounded normalised value in a few elements (two of the product
    with the weight when that falls into the binade below), because the mean square is summed over a
    workgroup instead of a wave.  A product that is not split comes back as a plain tensor."""
    from ksa_amd import add_rmsnorm
    from ksa_amd.gemm import SplitKPartials, linear_rows
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(1, M, K, generator=g).to(dtype).cuda()
    w = (torch.randn(N, K, generator=g) * 0.05).to(dtype).cuda()
    res = torch.randn(1, M, N, generator=g).to(dtype).cuda()
    nw = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype).cuda()
    s0, h0 = add_rmsnorm(linear_rows(x, w), res, nw, 1e-6)
    d = linear_rows(x, w, defer=True)
    if N * K >= 2560 * 4096:
        assert isinstance(d, SplitKPartials) and d.shape == (1, M, N)
    s1, h1 = add_rmsnorm(d, res, nw, 1e-6)
    assert s1.shape == s0.shape and torch.equal(s0, s1)
    a, b = h0.float().flatten(), h1.float().flatten()
    mant = 7 if dtype == torch.bfloat16 else 10
    ulp = torch.exp2(torch.floor(torch.log2(a.abs().clamp_min(2.0 ** -14))) - mant)
    assert ((a - b).abs() <= 2 * ulp * 1.001).all()
    assert ((a - b).abs() > ulp * 1.01).float().mean() <= 1e-4
    assert (a != b).float().mean() <= 0.01


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,I,K", [(8, 9728, 2560), (1, 9728, 2560), (16, 520, 1024), (5, 64, 512), (72, 1024, 4096),
                                   (30, 520, 2048)])
def test_gpu_deferred_gate_up_into_silu_mul(dtype, M, I, K):
    """gate | up left as K-split partial sums and added inside `silu_mul`: bit for bit the
    two-kernel result (the halves are summed in split order and rounded before the activation)."""
    from ksa_amd import silu_mul
    from ksa_amd.gemm import SplitKPartials, linear_rows
    g = torch.Generator().manual_seed(M + I + K)
    x = torch.randn(1, M, K, generator=g).to(dtype).cuda()
    w = (torch.randn(2 * I, K, generator=g) * 0.05).to(dtype).cuda()
    gu = linear_rows(x, w)
    want = silu_mul(gu[..., :I], gu[..., I:])
    assert torch.equal(silu_mul(gu), want)                     # whole projection as one tensor
    d = linear_rows(x, w, defer=True)
    if I >= 9728:
        assert isinstance(d, SplitKPartials)
    got = silu_mul(d)
    assert got.shape == want.shape and torch.equal(got, want)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,I,K", [(8, 9728, 2560), (1, 9728, 2560), (16, 520, 1024), (5, 64, 512), (3, 40, 96),
                                   (8, 1000, 1056), (2, 48, 8192), (16, 32, 5088),
                                   # 17 to 128 rows: x in chunks through LDS, gate and up waves meet behind the walk
                                   (72, 9728, 2560), (17, 40, 96), (64, 1000, 1056), (128, 200, 512), (100, 72, 1600)])
def test_gpu_gate_up_silu_one_launch(dtype, M, I, K):
    """The gate | up projection with the activation folded in (one launch, K not split) against the
    fp64 statement of the same rounding points - out = round(SiLU(round(g))) * round(u) - and against
    the two-kernel path.  The fp32 sums over K run in a different order than the split-K path's, so
    a gate or up value that lies next to a rounding boundary may round the other way: the result
    may then differ from the exact-sum statement by one unit in the last place of an intermediate
    (relative 2^-7 in bf16, 2^-10 in fp16), which SiLU passes on multiplied by |1 + g (1 - sigmoid(g))|
    <= 1 + |g|, in a small share of the elements.  Where a gate or up sum cancels to almost nothing the
    fp32 sum itself is off by more than such a unit (about 1e-6 absolute at these magnitudes; the
    two-kernel path shows the same): an absolute term of 2e-6 on either sum, passed on through the
    other factor."""
    from ksa_amd import silu_mul
    from ksa_amd.gemm import gate_up_silu_rows, linear_rows
    g = torch.Generator().manual_seed(M + I + K)
    x = torch.randn(1, M, K, generator=g).to(dtype)
    w = (torch.randn(2 * I, K, generator=g) * 0.05).to(dtype)
    got = gate_up_silu_rows(x.cuda(), w.cuda())
    assert got.shape == (1, M, I) and got.dtype == dtype
    y = (x.double()[0] @ w.double().T)
    gate, up = y[:, :I].to(dtype).double(), y[:, I:].to(dtype).double()
    want = ((gate / (1 + torch.exp(-gate))).to(dtype).double() * up).to(dtype)
    a, b = got[0].float().cpu(), want.float()
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    act64 = gate / (1 + torch.exp(-gate))
    tol = ulp * (3 + gate.abs().float()) * b.abs() + 1e-6 + 2e-6 * (1.1 * up.abs() + act64.abs()).float()
    assert ((a - b).abs() <= tol).all(), ((a - b).abs() / tol).max()
    assert (a != b).float().mean() <= 0.02
    two = silu_mul(linear_rows(x.cuda(), w.cuda()))
    assert (two[0].float().cpu() != a).float().mean() <= 0.02


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,H,I", [(8, 2560, 9728), (1, 2560, 9728), (16, 1024, 768), (3, 256, 256), (5, 4096, 512),
                                   (8, 768, 2304), (16, 2560, 1024)])
def test_gpu_mlp_rows_one_launch(dtype, M, H, I):
    """The MLP of a layer in one launch of resident workgroups (gate | up + SiLU -> grid barrier ->
    down) against the two separate launches it stands for: the down projection, added up from its
    partial sums, equal to the separate path's to within the few 16-bit units that a different
    split of K allows, and close to the fp64 product of the 16-bit activation the separate path
    makes (the activation itself is computed in the same order in both).  Run three times on one
    workspace (the barrier words count on), the last time after another shape has used a workspace
    of its own."""
    from ksa_amd import silu_mul
    from ksa_amd.gemm import MlpRowsWorkspace, gate_up_silu_rows, linear_rows, mlp_rows
    g = torch.Generator().manual_seed(M * 7 + H + I)
    dev = torch.device("cuda")
    h = torch.randn(1, M, H, generator=g).to(dtype).to(dev)
    w_gu = (torch.randn(2 * I, H, generator=g) * 0.04).to(dtype).to(dev)
    w_dn = (torch.randn(H, I, generator=g) * 0.03).to(dtype).to(dev)
    act = gate_up_silu_rows(h, w_gu) if M * (H + 8) * 2 <= 160 * 1024 else silu_mul(linear_rows(h, w_gu))
    d_ref = linear_rows(act, w_dn)
    want = (act[0].double() @ w_dn.double().T)
    ws = MlpRowsWorkspace(H, I, dev)
    for rep in range(3):
        if rep == 2:
            ws_other = MlpRowsWorkspace(256, 512, dev)
            mlp_rows(torch.ones(1, 2, 256, dtype=dtype, device=dev), torch.ones(1024, 256, dtype=dtype, device=dev),
                     torch.ones(256, 512, dtype=dtype, device=dev), ws_other)
            assert not ws_other.failed()
        d_part = mlp_rows(h, w_gu, w_dn, ws)
        torch.cuda.synchronize()
        assert not ws.failed(), "a workgroup gave up at the grid barrier"
        parts = d_part.workspace.view(torch.float32).view(d_part.ksplit, 16, H)[:, :M]
        d_new = parts.sum(0).to(dtype)
        err = (parts.double().sum(0) - want).abs().max().item()
        assert err <= 2e-3 * want.abs().max().item() + 1e-4, err
        ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
        diff = (d_new.float() - d_ref[0].float()).abs()
        assert (diff <= 2 * ulp * d_ref[0].float().abs() + 4 * ulp * want.abs().max().item() * 2.0 ** -6).all(), diff.max()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,H,I", [(8, 2560, 9728), (1, 2560, 9728), (16, 1024, 768), (3, 128, 64), (5, 4096, 512),
                                   (16, 2560, 1024)])
def test_gpu_add_rmsnorm_mlp_rows_one_launch(dtype, M, H, I):
    """Residual add + norm + MLP in one launch against ksa_add_rmsnorm_partials followed by ksa_mlp_rows:
    the sum with the residual bit-identical; the down projection (added up from its partial sums) to
    within what a last-place difference of a few normalised values can move it.  Three launches on one
    workspace, mixed with launches of the form without the norm stage."""
    from ksa_amd import add_rmsnorm
    from ksa_amd.gemm import MlpRowsWorkspace, SplitKPartials, add_rmsnorm_mlp_rows, linear_rows, mlp_rows
    g = torch.Generator().manual_seed(M * 7 + H + I)
    dev = torch.device("cuda")
    Ko = 512 if H <= 1024 else 4096
    attn = torch.randn(1, M, Ko, generator=g).to(dtype).to(dev)
    w_o = (torch.randn(H, Ko, generator=g) * 0.03).to(dtype).to(dev)
    res = torch.randn(1, M, H, generator=g).to(dtype).to(dev)
    nw = (1 + 0.1 * torch.randn(H, generator=g)).to(dtype).to(dev)
    w_gu = (torch.randn(2 * I, H, generator=g) * 0.04).to(dtype).to(dev)
    w_dn = (torch.randn(H, I, generator=g) * 0.03).to(dtype).to(dev)
    o = linear_rows(attn, w_o, defer=True)
    if not isinstance(o, SplitKPartials):  # K too short to be split: present the product as one slice
        ws1 = torch.zeros(16, H, dtype=torch.float32, device=dev)
        ws1[:M] = o[0].float()
        o = SplitKPartials(ws1.view(-1).view(torch.uint8), 1, M, (1, M, H), dtype)
    ws = MlpRowsWorkspace(H, I, dev)
    x_ref, h_ref = add_rmsnorm(o, res, nw, 1e-6)
    d_ref = mlp_rows(h_ref, w_gu, w_dn, ws)
    sum_ref = d_ref.workspace.view(torch.float32).view(d_ref.ksplit, 16, H)[:, :M].sum(0)
    for rep in range(3):
        x_new, d_new = add_rmsnorm_mlp_rows(o, res, nw, 1e-6, w_gu, w_dn, ws)
        torch.cuda.synchronize()
        assert not ws.failed(), "a workgroup gave up waiting"
        assert torch.equal(x_new, x_ref)
        sum_new = d_new.workspace.view(torch.float32).view(d_new.ksplit, 16, H)[:, :M].sum(0)
        assert (sum_new - sum_ref).abs().max().item() <= 4e-3 * sum_ref.abs().max().item() + 1e-5
        if rep == 1:
            mlp_rows(h_ref, w_gu, w_dn, ws)


def _o_partials(M, H, dtype, dev, g):
    """The K-split partial sums of an o projection for M rows, as `linear_rows(..., defer=True)` leaves them."""
    from ksa_amd.gemm import SplitKPartials, linear_rows
    attn = torch.randn(1, M, 4096, generator=g).to(dtype).to(dev)
    w_o = (torch.randn(H, 4096, generator=g) * 0.03).to(dtype).to(dev)
    o = linear_rows(attn, w_o, defer=True)
    assert isinstance(o, SplitKPartials)
    return o


@pytest.mark.gpu
def test_gpu_mlp_rows_row_count_changes_on_one_workspace():
    """Launches with 8, then 2, then 8, then 1, then 16 rows on ONE workspace, with and without the norm
    stage: the words that the waits compare against must not depend on the row counts of earlier
    launches.  (With a target of "launches x rows of this launch" a 2-row launch behind 8-row ones would
    not wait for its norm stage at all and read the rows of an earlier launch.)  Every result is compared
    with the same call on a fresh workspace, bit for bit, and the norm stage's input differs from launch
    to launch so that stale rows cannot pass."""
    from ksa_amd.gemm import MlpRowsWorkspace, add_rmsnorm_mlp_rows, mlp_rows
    dtype, dev = torch.bfloat16, torch.device("cuda")
    H, I = 2560, 9728
    g = torch.Generator().manual_seed(5)
    nw = (1 + 0.1 * torch.randn(H, generator=g)).to(dtype).to(dev)
    w_gu = (torch.randn(2 * I, H, generator=g) * 0.04).to(dtype).to(dev)
    w_dn = (torch.randn(H, I, generator=g) * 0.03).to(dtype).to(dev)
    shared = MlpRowsWorkspace(H, I, dev)
    for step, (M, with_norm) in enumerate([(8, True), (8, True), (2, True), (8, True), (1, False), (1, True),
                                           (16, True), (3, False), (2, True), (2, True), (16, True)]):
        res = torch.randn(1, M, H, generator=g).to(dtype).to(dev)
        if with_norm:
            o = _o_partials(M, H, dtype, dev, g)
            run = lambda ws: add_rmsnorm_mlp_rows(o, res, nw, 1e-6, w_gu, w_dn, ws)
        else:
            run = lambda ws: (None, mlp_rows(res, w_gu, w_dn, ws))
        x_a, d_a = run(shared)
        fresh = MlpRowsWorkspace(H, I, dev)
        x_b, d_b = run(fresh)
        torch.cuda.synchronize()
        assert not shared.failed() and not fresh.failed(), (step, M)
        if with_norm:
            assert torch.equal(x_a, x_b), (step, M)
        pa = d_a.workspace.view(torch.float32).view(d_a.ksplit, 16, H)[:, :M]
        pb = d_b.workspace.view(torch.float32).view(d_b.ksplit, 16, H)[:, :M]
        assert torch.equal(pa, pb), (step, M, (pa - pb).abs().max().item())


@pytest.mark.gpu
def test_gpu_mlp_rows_bounded_wait_gives_up_and_recovers():
    """The give-up path, forced from the host: the word that holds the number of past launches is set
    far ahead, so the count that the down workgroups wait for cannot be reached.  The first of them to
    exhaust its bounded wait (about a second) sets the status word, the others see it and leave, the
    launch ends normally.  `failed()` then reports it and zeroes the workspace, and the next launch on
    it equals a launch on a fresh workspace bit for bit."""
    from ksa_amd import _lib
    from ksa_amd.gemm import MlpRowsWorkspace, mlp_rows
    dtype, dev = torch.bfloat16, torch.device("cuda")
    M, H, I = 8, 2560, 9728
    g = torch.Generator().manual_seed(9)
    h = torch.randn(1, M, H, generator=g).to(dtype).to(dev)
    w_gu = (torch.randn(2 * I, H, generator=g) * 0.04).to(dtype).to(dev)
    w_dn = (torch.randn(H, I, generator=g) * 0.03).to(dtype).to(dev)
    ws = MlpRowsWorkspace(H, I, dev)
    assert _lib.lib().ksa_mlp_rows_status_offset() == 2 * 512
    ws.buf[:8].view(torch.int64).fill_(1 << 40)   # word 0: launches so far
    torch.cuda.synchronize()
    mlp_rows(h, w_gu, w_dn, ws)
    torch.cuda.synchronize()                       # every workgroup has left
    assert int(ws._status.item()) == 1
    assert ws.failed()
    assert int(ws.buf.view(torch.int64).abs().sum().item()) == 0
    assert not ws.failed()
    got = mlp_rows(h, w_gu, w_dn, ws)
    want = mlp_rows(h, w_gu, w_dn, MlpRowsWorkspace(H, I, dev))
    torch.cuda.synchronize()
    assert not ws.failed()
    assert torch.equal(got.workspace.view(torch.float32).view(got.ksplit, 16, H)[:, :M],
                       want.workspace.view(torch.float32).view(want.ksplit, 16, H)[:, :M])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gpu_streaming_weight_layout(dtype):
    """`TiledWeight` (`ksa_tile_weights`): [ceil(N / 16)][K / 32][16][32] with zero rows past N, from a
    matrix and from a row slice of a larger one; and every few-rows kernel gives bit for bit the result
    of the row-major call on it (same products in the same order, only the addresses differ)."""
    from ksa_amd.gemm import (MlpRowsWorkspace, TiledWeight, add_rmsnorm_mlp_rows, gate_up_silu_rows, linear_rows,
                              mlp_rows)
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(11)

    def sums(d):  # the rows of the partial sums that exist (a slice holds whole 16-row blocks)
        return d.workspace.view(torch.float32).view(d.ksplit, -1, d.shape[-1])[:, :d.rows]
    for N, K in ((40, 96), (2560, 4096), (1000, 640)):
        big = (torch.randn(N + 8, K + 64, generator=g) * 0.05).to(dtype).to(dev)
        w = big[8:, :K]                                   # rows 8.., a row stride above K
        t = TiledWeight(w)
        Np = (N + 15) // 16 * 16
        ref = torch.zeros(Np, K, dtype=dtype, device=dev)
        ref[:N] = w
        ref = ref.view(Np // 16, 16, K // 32, 32).permute(0, 2, 1, 3).contiguous().view(-1)
        assert torch.equal(t.data, ref)
        for M in (1, 8, 16, 17, 72, 128):
            x = torch.randn(M, K, generator=g).to(dtype).to(dev)
            assert torch.equal(linear_rows(x, t), linear_rows(x, w)), (N, K, M)
    # deferred partial sums as well
    w = (torch.randn(2560, 4096, generator=g) * 0.05).to(dtype).to(dev)
    t = TiledWeight(w)
    for M in (8, 72):
        x = torch.randn(M, 4096, generator=g).to(dtype).to(dev)
        a, b = linear_rows(x, t, defer=True), linear_rows(x, w, defer=True)
        assert a.ksplit == b.ksplit and torch.equal(sums(a), sums(b))
    # gate | up with the activation, the one-launch MLP, and the MLP with the norm in front
    H, I = 1024, 768
    w_gu = (torch.randn(2 * I, H, generator=g) * 0.04).to(dtype).to(dev)
    w_dn = (torch.randn(H, I, generator=g) * 0.03).to(dtype).to(dev)
    t_gu, t_dn = TiledWeight(w_gu), TiledWeight(w_dn)
    for M in (3, 16, 40, 128):
        x = torch.randn(1, M, H, generator=g).to(dtype).to(dev)
        assert torch.equal(gate_up_silu_rows(x, t_gu), gate_up_silu_rows(x, w_gu)), M
    ws = MlpRowsWorkspace(H, I, dev)
    for M in (1, 8, 16):
        x = torch.randn(1, M, H, generator=g).to(dtype).to(dev)
        a, b = mlp_rows(x, t_gu, t_dn, ws), mlp_rows(x, w_gu, w_dn, ws)
        assert torch.equal(sums(a), sums(b)), M
        w_o = (torch.randn(H, 512, generator=g) * 0.05).to(dtype).to(dev)
        attn = torch.randn(1, M, 512, generator=g).to(dtype).to(dev)
        res = torch.randn(1, M, H, generator=g).to(dtype).to(dev)
        nw = (1 + 0.1 * torch.randn(H, generator=g)).to(dtype).to(dev)
        o = linear_rows(attn, TiledWeight(w_o), defer=True)
        if isinstance(o, type(a)):
            s1, d1 = add_rmsnorm_mlp_rows(o, res, nw, 1e-6, t_gu, t_dn, ws)
            s0, d0 = add_rmsnorm_mlp_rows(o, res, nw, 1e-6, w_gu, w_dn, ws)
            assert torch.equal(s0, s1) and torch.equal(sums(d0), sums(d1)), M
    assert not ws.failed()
