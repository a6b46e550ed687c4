"""Pre-attention step (q/k RMSNorm + rotary embedding + layout write).

CPU part: the oracle restatement (`oracle.cpu_path.pre_attention`, the reference's sequence of
16-bit tensor ops) is pinned by what the mathematics fixes, computed independently in float64:
unit RMS after the norm, the rotation as a complex multiplication that preserves pair norms,
the relative-position property of rotary scores, the identity at position 0 and pass-through of v.
GPU part: the HIP kernel against that oracle, bit for bit up to one unit in the last place of
the 16-bit type on a small fraction of elements (fp32 rsqrt and summation order differ).
"""
import numpy as np
import pytest
import torch

from oracle import cpu_path


def _rope_tables(S, D, base=10000.0, pos=None, dtype=torch.float32):
    pos = torch.arange(S, dtype=torch.float64) if pos is None else torch.as_tensor(pos, dtype=torch.float64)
    inv = 1.0 / (base ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
    ang = pos[:, None] * inv[None, :]
    emb = torch.cat((ang, ang), dim=-1)            # HF layout: the two halves repeat the angles
    return emb.cos().to(dtype)[None], emb.sin().to(dtype)[None], ang


def _inputs(b, S, Hq, Hkv, D, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, S, Hq, D, generator=g).to(dtype)
    k = torch.randn(b, S, Hkv, D, generator=g).to(dtype)
    v = torch.randn(b, S, Hkv, D, generator=g).to(dtype)
    qw = (1.0 + 0.1 * torch.randn(D, generator=g)).to(dtype)
    kw = (1.0 + 0.1 * torch.randn(D, generator=g)).to(dtype)
    return q, k, v, qw, kw


def test_oracle_fp32_matches_float64_closed_form():
    b, S, Hq, Hkv, D = 2, 37, 4, 2, 128
    q, k, v, qw, kw = _inputs(b, S, Hq, Hkv, D, 0, torch.float32)
    cos, sin, ang = _rope_tables(S, D)
    qo, ko, vo = cpu_path.pre_attention(q, k, v, qw, kw, cos, sin, eps=1e-6)
    assert torch.equal(vo, v)
    # independent float64 computation: RMSNorm, then complex rotation of the pairs (j, j + D/2)
    for x, w, got in ((q, qw, qo), (k, kw, ko)):
        xd = x.double()
        n = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-6) * w.double()
        z = torch.complex(n[..., : D // 2], n[..., D // 2:])
        rot = z * torch.polar(torch.ones_like(ang), ang)[None, :, None, :]
        want = torch.cat((rot.real, rot.imag), dim=-1)
        assert (got.double() - want).abs().max() < 2e-5


def test_oracle_invariants():
    b, S, H, D = 1, 64, 2, 64
    q, k, v, _, _ = _inputs(b, S, H, H, D, 1, torch.float32)
    ones = torch.ones(D)
    cos, sin, _ = _rope_tables(S, D)
    qo, ko, _ = cpu_path.pre_attention(q, k, v, ones, ones, cos, sin, eps=0.0)
    # unit RMS per head row survives the rotation (it preserves the norm of every pair)
    assert ((qo * qo).mean(-1) - 1).abs().max() < 1e-5
    # position 0 is the identity rotation
    q0 = q[:, 0] / torch.sqrt((q[:, 0] ** 2).mean(-1, keepdim=True))
    assert (qo[:, 0] - q0).abs().max() < 1e-6
    # relative-position property: <rope(q, m), rope(k, n)> depends on m - n only
    qc = q[:, :1].expand(b, S, H, D).contiguous()
    kc = k[:, :1].expand(b, S, H, D).contiguous()
    qr, kr, _ = cpu_path.pre_attention(qc, kc, v, ones, ones, cos, sin, eps=0.0)
    s1 = (qr[0, 10, 0] * kr[0, 3, 0]).sum()
    s2 = (qr[0, 40, 0] * kr[0, 33, 0]).sum()
    assert abs(s1 - s2) < 1e-3


def test_oracle_rounding_points_bf16():
    """In bf16 every tensor op of the reference rounds; the restatement must show exactly the
    roundings of the chain norm -> weight -> (z cos) + (rot(z) sin), checked element by element
    with explicit float32 arithmetic and round-to-nearest-even to bf16."""
    b, S, H, D = 1, 5, 1, 64
    q, k, v, qw, kw = _inputs(b, S, H, H, D, 2, torch.bfloat16)
    cos, sin, _ = _rope_tables(S, D, dtype=torch.bfloat16)
    qo, _, _ = cpu_path.pre_attention(q, k, v, qw, kw, cos, sin, eps=1e-6)

    def r(x):  # float32 -> bf16 -> float32
        return x.to(torch.bfloat16).to(torch.float32)
    x = q.float()
    inv = torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6)
    z = r(qw.float() * r(x * inv))
    rot = torch.cat((-z[..., D // 2:], z[..., : D // 2]), dim=-1)
    want = r(r(z * cos.float()[:, :, None]) + r(rot * sin.float()[:, :, None]))
    assert torch.equal(qo.float(), want)


def _ulp_report(got, want):
    """(largest difference in units of the last place of the largest magnitude, fraction of
    elements that differ at all).  The output is a sum of two rounded products, so a one-ulp
    difference in a product shows up as one ulp of that product, not of the (possibly much
    smaller) sum."""
    ulp = 2.0 ** (-7 if want.dtype == torch.bfloat16 else -10) * float(want.float().abs().max())
    d = (got.float() - want.float()).abs()
    return float(d.max()) / ulp, float((d != 0).float().mean())


@pytest.mark.gpu
@pytest.mark.parametrize("case", [
    (1, 1000, 32, 8, 128, torch.bfloat16),
    (2, 333, 16, 8, 128, torch.bfloat16),
    (1, 257, 6, 2, 64, torch.bfloat16),     # head_dim 64, head count not a multiple of the wave's rows
    (2, 130, 4, 4, 128, torch.float16),
])
def test_pre_attention_gpu(case):
    import ksa_amd
    b, S, Hq, Hkv, D, dtype = case
    q, k, v, qw, kw = _inputs(b, S, Hq, Hkv, D, 3, dtype)
    pos = torch.arange(S) * 3 + 5                      # any positions
    cos, sin, _ = _rope_tables(S, D, pos=pos, dtype=dtype)
    want = cpu_path.pre_attention(q, k, v, qw, kw, cos, sin, eps=1e-6)
    dev = torch.device("cuda")
    got = ksa_amd.pre_attention(q.to(dev), k.to(dev), v.to(dev), qw.to(dev), kw.to(dev), cos.to(dev),
                                sin.to(dev), eps=1e-6)
    torch.cuda.synchronize()
    for name, g, w in zip("qkv", got, want):
        mx, frac = _ulp_report(g.cpu(), w)
        assert mx <= 1 and frac < 2e-3, (name, mx, frac)
    assert torch.equal(got[2].cpu(), v)


@pytest.mark.gpu
def test_pre_attention_gpu_writes_into_cache_layout_and_in_place():
    """k and v go straight into rows of a [b, Hkv, capacity, D] cache tensor (the reference:
    transpose + `past_key_values.update` copies), q is normalised and rotated in place."""
    import ksa_amd
    b, S, Hq, Hkv, D, dtype = 2, 200, 8, 2, 128, torch.bfloat16
    q, k, v, qw, kw = _inputs(b, S, Hq, Hkv, D, 4, dtype)
    cos, sin, _ = _rope_tables(S, D, dtype=dtype)
    want = cpu_path.pre_attention(q, k, v, qw, kw, cos, sin, eps=1e-6)
    dev = torch.device("cuda")
    cap, start = 512, 40
    kc = torch.zeros(b, Hkv, cap, D, dtype=dtype, device=dev)
    vc = torch.zeros_like(kc)
    # projections as the model holds them: one [b, S, (Hq + 2 Hkv) D] buffer, sliced
    qkv = torch.cat((q.reshape(b, S, -1), k.reshape(b, S, -1), v.reshape(b, S, -1)), dim=-1).to(dev)
    qv = qkv[..., : Hq * D].view(b, S, Hq, D)
    kv = qkv[..., Hq * D: (Hq + Hkv) * D].view(b, S, Hkv, D)
    vv = qkv[..., (Hq + Hkv) * D:].view(b, S, Hkv, D)
    ksa_amd.pre_attention(qv, kv, vv, qw.to(dev), kw.to(dev), cos.to(dev), sin.to(dev), eps=1e-6, q_out=qv,
                          k_out=kc[:, :, start:start + S].transpose(1, 2),
                          v_out=vc[:, :, start:start + S].transpose(1, 2))
    torch.cuda.synchronize()
    assert _ulp_report(qv.cpu(), want[0])[0] <= 1
    assert _ulp_report(kc[:, :, start:start + S].transpose(1, 2).cpu().contiguous(), want[1])[0] <= 1
    assert torch.equal(vc[:, :, start:start + S].transpose(1, 2).cpu(), v)
    assert kc[:, :, :start].abs().max() == 0 and kc[:, :, start + S:].abs().max() == 0


@pytest.mark.gpu
@pytest.mark.parametrize("S", [1, 3])
def test_pre_attention_gpu_cache_row_from_device_memory(S):
    """`kv_out_row`: each sequence's k and v land at the cache row a device-side int32 names
    (the cursor of a recorded decode step), with the values of a call that was given the row on
    the host; q and the rest of the cache are untouched by it."""
    import ksa_amd
    b, Hq, Hkv, D, dtype = 3, 8, 2, 128, torch.bfloat16
    q, k, v, qw, kw = _inputs(b, S, Hq, Hkv, D, 9, dtype)
    cos, sin, _ = _rope_tables(S, D, dtype=dtype)
    dev = torch.device("cuda")
    cap = 64
    rows = [5, 40, 17]
    args = [t.to(dev) for t in (q, k, v, qw, kw, cos, sin)]
    kc = torch.zeros(b, Hkv, cap, D, dtype=dtype, device=dev)
    vc = torch.zeros_like(kc)
    cursor = torch.tensor(rows, dtype=torch.int32, device=dev)
    q1, _, _ = ksa_amd.pre_attention(*args, eps=1e-6, k_out=kc[:, :, :S].transpose(1, 2),
                                     v_out=vc[:, :, :S].transpose(1, 2), kv_out_row=cursor)
    q0, k0, v0 = ksa_amd.pre_attention(*args, eps=1e-6)
    torch.cuda.synchronize()
    assert torch.equal(q0, q1)
    for i, r in enumerate(rows):
        assert torch.equal(kc[i, :, r:r + S].transpose(0, 1), k0[i])
        assert torch.equal(vc[i, :, r:r + S].transpose(0, 1), v0[i])
        kc[i, :, r:r + S] = 0
        vc[i, :, r:r + S] = 0
    assert kc.abs().max() == 0 and vc.abs().max() == 0
    with pytest.raises(AssertionError):
        ksa_amd.pre_attention(*args, eps=1e-6, kv_out_row=cursor)          # needs k_out / v_out
    with pytest.raises(AssertionError):
        ksa_amd.pre_attention(*args, eps=1e-6, k_out=kc[:, :, :S].transpose(1, 2),
                              v_out=vc[:, :, :S].transpose(1, 2), kv_out_row=cursor.long())


@pytest.mark.gpu
def test_pre_attention_rejects_bad_inputs():
    import ksa_amd
    dev = torch.device("cuda")
    q = torch.zeros(1, 8, 2, 96, dtype=torch.bfloat16, device=dev)
    w = torch.ones(96, dtype=torch.bfloat16, device=dev)
    c = torch.ones(1, 8, 96, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ksa_amd.KsaError):
        ksa_amd.pre_attention(q, q, q, w, w, c, c)
    with pytest.raises(AssertionError):
        ksa_amd.pre_attention(q.float(), q.float(), q.float(), w, w, c, c)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("b,S,Hq,Hkv,D", [(8, 1, 32, 8, 128), (1, 1, 32, 8, 128), (2, 3, 6, 2, 64), (16, 1, 4, 4, 128),
                                          (8, 9, 32, 8, 128), (64, 1, 32, 8, 128), (14, 9, 6, 2, 64)])
def test_pre_attention_gpu_from_split_k_partials(dtype, b, S, Hq, Hkv, D):
    """q | k | v still as the K-split partial sums of the fused projection: the kernel adds them
    itself and returns bit for bit what the reduced projection followed by `pre_attention` gives,
    including the write to a cache row named in device memory."""
    import ksa_amd
    from ksa_amd.gemm import SplitKPartials, linear_rows
    from ksa_amd.pre import pre_attention_partials
    dev = torch.device("cuda")
    K = 2560
    g = torch.Generator().manual_seed(b * 100 + S * 10 + Hq)
    x = torch.randn(b, S, K, generator=g).to(dtype).to(dev)
    w = (torch.randn((Hq + 2 * Hkv) * D, K, generator=g) * 0.05).to(dtype).to(dev)
    qw = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype).to(dev)
    kw = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype).to(dev)
    cos, sin, _ = _rope_tables(S, D, dtype=dtype)
    cos, sin = cos.to(dev), sin.to(dev)
    qkv = linear_rows(x, w)
    q = qkv[..., : Hq * D].view(b, S, Hq, D)
    k = qkv[..., Hq * D: (Hq + Hkv) * D].view(b, S, Hkv, D)
    v = qkv[..., (Hq + Hkv) * D:].view(b, S, Hkv, D)
    q0, k0, v0 = ksa_amd.pre_attention(q, k, v, qw, kw, cos, sin, eps=1e-6)
    d = linear_rows(x, w, defer=True)
    if not isinstance(d, SplitKPartials):
        pytest.skip("this shape is not split over K")
    cap = 32
    kc = torch.zeros(b, Hkv, cap, D, dtype=dtype, device=dev)
    vc = torch.zeros_like(kc)
    cursor = (torch.arange(b, device=dev, dtype=torch.int32) * 3) % (cap - S)
    q1, _, _ = pre_attention_partials(d, Hq, Hkv, D, qw, kw, cos, sin, eps=1e-6,
                                      k_out=kc[:, :, :S].transpose(1, 2), v_out=vc[:, :, :S].transpose(1, 2),
                                      kv_out_row=cursor)
    torch.cuda.synchronize()
    assert torch.equal(q0, q1)
    for i in range(b):
        r = int(cursor[i])
        assert torch.equal(kc[i, :, r:r + S].transpose(0, 1), k0[i])
        assert torch.equal(vc[i, :, r:r + S].transpose(0, 1), v0[i])


@pytest.mark.gpu
@pytest.mark.parametrize("from_partials", [False, True])
@pytest.mark.parametrize("b,S,Hq,Hkv,D", [(8, 9, 32, 8, 128), (3, 5, 6, 2, 64)])
def test_pre_attention_gpu_row_per_token(from_partials, b, S, Hq, Hkv, D):
    """`kv_out_row` as a table [b, S]: every token's k and v land in the cache row the table names (a
    chunk-boundary step: the text token at the cache cursor, the summary tokens in rows of their own),
    bit for bit the values of the plain call; q is unchanged; no other cache row is touched."""
    import ksa_amd
    from ksa_amd.gemm import SplitKPartials, linear_rows
    from ksa_amd.pre import pre_attention_partials
    dev = torch.device("cuda")
    dtype = torch.bfloat16
    K = 2560
    g = torch.Generator().manual_seed(b * 100 + S * 10 + Hq + 7)
    x = torch.randn(b, S, K, generator=g).to(dtype).to(dev)
    w = (torch.randn((Hq + 2 * Hkv) * D, K, generator=g) * 0.05).to(dtype).to(dev)
    qw = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype).to(dev)
    kw = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype).to(dev)
    cos, sin, _ = _rope_tables(S, D, dtype=dtype)
    cos, sin = cos.to(dev), sin.to(dev)
    qkv = linear_rows(x, w)
    q = qkv[..., : Hq * D].view(b, S, Hq, D)
    k = qkv[..., Hq * D: (Hq + Hkv) * D].view(b, S, Hkv, D)
    v = qkv[..., (Hq + Hkv) * D:].view(b, S, Hkv, D)
    q0, k0, v0 = ksa_amd.pre_attention(q, k, v, qw, kw, cos, sin, eps=1e-6)
    cap = 64
    kc = torch.full((b, Hkv, cap, D), 7.0, dtype=dtype, device=dev)
    vc = torch.full((b, Hkv, cap, D), -3.0, dtype=dtype, device=dev)
    # token 0 at a per-sequence cursor, the others in a run of rows elsewhere (also per sequence)
    table = torch.empty(b, S, dtype=torch.int32)
    for i in range(b):
        table[i, 0] = 40 + (i * 5) % 20
        table[i, 1:] = torch.arange(S - 1) + (i % 3) * 10
    table = table.to(dev)
    slots = dict(k_out=kc[:, :, :S].transpose(1, 2), v_out=vc[:, :, :S].transpose(1, 2), kv_out_row=table)
    if from_partials:
        d = linear_rows(x, w, defer=True)
        if not isinstance(d, SplitKPartials):
            pytest.skip("this shape is not split over K")
        q1, _, _ = pre_attention_partials(d, Hq, Hkv, D, qw, kw, cos, sin, eps=1e-6, **slots)
    else:
        q1, _, _ = ksa_amd.pre_attention(q, k, v, qw, kw, cos, sin, eps=1e-6, **slots)
    torch.cuda.synchronize()
    assert torch.equal(q0, q1)
    touched = torch.zeros(b, cap, dtype=torch.bool)
    for i in range(b):
        for t in range(S):
            r = int(table[i, t])
            touched[i, r] = True
            assert torch.equal(kc[i, :, r], k0[i, t]) and torch.equal(vc[i, :, r], v0[i, t])
    untouched = ~touched.to(dev)
    assert (kc.transpose(1, 2)[untouched] == 7.0).all() and (vc.transpose(1, 2)[untouched] == -3.0).all()
