"""GPU parity of decode attention and the cache row mover against the CPU oracle."""
import numpy as np
import pytest
import torch

from conftest import to_np
from oracle import c_oracle

pytestmark = pytest.mark.gpu

ATOL = 2e-2   # bf16 GPU vs fp32 oracle, stated bar
RTOL_INF = 2e-2


def _mk(Bz, Hq, Hkv, Q, D, rows, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(Bz, Hq, Q, D, generator=g).to(dtype)
    k = torch.randn(Bz, Hkv, rows, D, generator=g).to(dtype)
    v = torch.randn(Bz, Hkv, rows, D, generator=g).to(dtype)
    return q, k, v


def _check(q, k, v, start, end, nsplit, scale=None):
    import ksa_amd
    dev = torch.device("cuda")
    Bz = q.shape[0]
    st = torch.as_tensor(start, dtype=torch.int32, device=dev) if np.ndim(start) else int(start)
    en = torch.as_tensor(end, dtype=torch.int32, device=dev) if np.ndim(end) else int(end)
    out = ksa_amd.ksa_decode(q.to(dev), k.to(dev), v.to(dev), st, en, scale=scale, nsplit=nsplit)
    torch.cuda.synchronize()
    want = c_oracle.decode(to_np(q), to_np(k), to_np(v), np.broadcast_to(start, (Bz,)),
                           np.broadcast_to(end, (Bz,)), scale=scale)
    got = to_np(out)
    err = np.abs(got - want).max()
    assert np.isfinite(got).all()
    assert err <= ATOL and err <= RTOL_INF * np.abs(want).max(), (err, np.abs(want).max())


@pytest.mark.parametrize("nsplit", [1, 2, 5, None])
def test_decode_small(nsplit):
    q, k, v = _mk(3, 8, 2, 1, 128, 700, seed=0)
    _check(q, k, v, 0, 700, nsplit)


@pytest.mark.parametrize("nsplit", [1, 3])
def test_decode_per_sequence_ranges(nsplit):
    """ragged [start, end) per sequence, including one-row and sub-tile slices"""
    q, k, v = _mk(6, 8, 4, 1, 128, 1000, seed=1)
    start = np.array([0, 5, 136, 999, 100, 17], np.int32)
    end = np.array([1000, 6, 900, 1000, 131, 530], np.int32)
    _check(q, k, v, start, end, nsplit)


def test_decode_strided_view_like_hf():
    """HF hands in cache[:, :, start:end, :] views (non-contiguous batch/head strides)."""
    import ksa_amd
    dev = torch.device("cuda")
    q, k, v = _mk(2, 32, 8, 1, 128, 2000, seed=2)
    kd, vd = k.to(dev), v.to(dev)
    kview, vview = kd[:, :, 37:1500, :], vd[:, :, 37:1500, :]

    class M:
        num_key_value_groups = 4
    out, w = ksa_amd.decode_attention_forward(M(), q.to(dev), kview, vview, None, scaling=128 ** -0.5)
    assert w is None and out.shape == (2, 1, 32, 128)
    want = c_oracle.decode(to_np(q), to_np(k), to_np(v), 37, 1500)
    assert np.abs(to_np(out) - want).max() <= ATOL


def test_decode_boundary_queries():
    """chunk-boundary step: S = 8 summary queries x g = 4 heads fill one 32-column tile;
    Q = 9 needs two column blocks."""
    for Q in (8, 9):
        q, k, v = _mk(2, 8, 2, Q, 128, 136, seed=3)
        _check(q, k, v, 0, 136, 1)
        _check(q, k, v, 0, 136, 2)


def test_decode_head_dim_64_and_fp16():
    q, k, v = _mk(2, 4, 2, 1, 64, 555, seed=4)
    _check(q, k, v, 3, 555, 2)
    q, k, v = _mk(2, 4, 2, 1, 128, 555, seed=5, dtype=torch.float16)
    _check(q, k, v, 3, 555, 1)


@pytest.mark.parametrize("D", [256, 96, 192, 40])
def test_decode_other_head_dims(D):
    """Head dimension 256 (kernels of its own) and multiples of 8 without one (zero-padded copies of the
    attended rows at the next kernel size): scalar and per-sequence ranges, splits, the boundary step's
    9 query tokens, fp16."""
    q, k, v = _mk(3, 8, 2, 1, D, 900, seed=30 + D)
    _check(q, k, v, 5, 900, 1)
    _check(q, k, v, np.array([0, 100, 640], np.int32), np.array([900, 777, 641], np.int32), 3)
    q, k, v = _mk(2, 4, 2, 9, D, 300, seed=31 + D, dtype=torch.float16)
    _check(q, k, v, 0, 136, 2)


def test_decode_peaked_softmax():
    """large scale -> near one-hot attention: exercises the running-max rescale"""
    q, k, v = _mk(2, 8, 2, 1, 128, 3000, seed=6)
    _check(q, k, v, 0, 3000, 1, scale=1.0)
    _check(q, k, v, 0, 3000, 4, scale=1.0)


def test_decode_cfg3_shape_subset():
    """cfg 3 geometry (cap 17288, S=8, C=128, ring 512, 8192 summaries) on 4 of the 64
    sequences: slice [136 - cbl, 8808)."""
    Bz, cap = 4, 17288
    q, k, v = _mk(Bz, 32, 8, 1, 128, cap, seed=7)
    cbl = np.array([1, 128, 57, 100], np.int32)
    _check(q, k, v, 136 - cbl, np.full(Bz, 8808, np.int32), None)


def test_decode_cfg3_full_batch():
    """cfg 3 itself: batch 64, 32/8 heads, cap 17288, per-sequence slice [136 - cbl, 8808) with
    cbl uniform in [1, 128]: all 64 x 32 output rows against the oracle (one sequence at a
    time on the host), and the split-K identity (1 split == 4 splits up to rounding)."""
    import ksa_amd
    dev = torch.device("cuda")
    Bz, Hq, Hkv, D, cap = 64, 32, 8, 128, 17288
    g = torch.Generator(device=dev).manual_seed(11)
    k = torch.randn(Bz, Hkv, cap, D, generator=g, device=dev).to(torch.bfloat16)
    v = torch.randn(Bz, Hkv, cap, D, generator=g, device=dev).to(torch.bfloat16)
    q = torch.randn(Bz, Hq, 1, D, generator=g, device=dev).to(torch.bfloat16)
    cbl = torch.randint(1, 129, (Bz,), generator=g, device=dev, dtype=torch.int32)
    start = (136 - cbl).to(torch.int32)
    end = torch.full((Bz,), 8808, dtype=torch.int32, device=dev)
    out1 = ksa_amd.ksa_decode(q, k, v, start, end, nsplit=1)
    out4 = ksa_amd.ksa_decode(q, k, v, start, end, nsplit=4)
    outa = ksa_amd.ksa_decode(q, k, v, start, end)
    torch.cuda.synchronize()
    assert (out1.float() - out4.float()).abs().max().item() <= 2e-3
    assert (out1.float() - outa.float()).abs().max().item() <= 2e-3
    got = to_np(out1)
    st, en = start.cpu().numpy(), end.cpu().numpy()
    worst = 0.0
    for b in range(Bz):
        want = c_oracle.decode(to_np(q[b:b + 1]), to_np(k[b:b + 1]), to_np(v[b:b + 1]), st[b:b + 1], en[b:b + 1])
        err = np.abs(got[b:b + 1] - want).max()
        worst = max(worst, err)
        assert err <= ATOL and err <= RTOL_INF * np.abs(want).max(), (b, err)
    assert np.isfinite(got).all()


def test_copy_rows():
    import ksa_amd
    from ksa_amd.cache import _move_rows
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(0)
    src = torch.randn(2, 3, 50, 128, generator=g).bfloat16().to(dev)
    dst = torch.zeros(2, 3, 80, 128, dtype=torch.bfloat16, device=dev)
    _move_rows(src, dst, 20, 5, 33)
    assert torch.equal(dst[:, :, 33:53], src[:, :, 5:25]) and float(dst[:, :, :33].abs().sum()) == 0
    idx = torch.tensor([7, 3, 49, 0], dtype=torch.int32, device=dev)
    _move_rows(src, dst, 4, dst_start=60, src_index=idx)
    assert torch.equal(dst[:, :, 60:64], src[:, :, idx.long()])


def test_decode_empty_and_single_row_ranges():
    """Ragged extremes: a sequence whose row range is empty (the reference never produces one; this
    build defines its output as zeros, not NaN), one with a single row (output = that row of V) and
    ordinary ones in the same launch, with one and with several splits."""
    import ksa_amd
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(31)
    b, Hq, Hkv, D, rows = 4, 8, 2, 128, 900
    q = torch.randn(b, Hq, 1, D, generator=g).bfloat16()
    kc = torch.randn(b, Hkv, rows, D, generator=g).bfloat16()
    vc = torch.randn(b, Hkv, rows, D, generator=g).bfloat16()
    start = np.array([100, 500, 0, 37], np.int32)
    end = np.array([100, 501, 900, 300], np.int32)
    for nsplit in (1, 4):
        got = ksa_amd.ksa_decode(q.to(dev), kc.to(dev), vc.to(dev), torch.as_tensor(start, device=dev),
                                 torch.as_tensor(end, device=dev), nsplit=nsplit).float().cpu().numpy()
        assert np.isfinite(got).all()
        assert np.abs(got[0]).max() == 0.0
        want1 = vc[1, :, 500].float().numpy()                     # [Hkv, D]; head h reads kv head h // g
        assert np.array_equal(got[1, 0], np.repeat(want1, Hq // Hkv, axis=0))
        ref = c_oracle.decode(q[2:].float().numpy(), kc[2:].float().numpy(), vc[2:].float().numpy(), start[2:], end[2:])
        assert np.abs(got[2:] - ref).max() <= 2e-2


def _weights_oracle(q, k, start, end, scale, mask=None):
    """softmax(q K^T * scale + mask) in float64 per (sequence, head, query token) over rows [start, end)."""
    Bz, Hq, Q, D = q.shape
    g = Hq // k.shape[1]
    L = int(np.max(end - start))
    out = np.zeros((Bz, Hq, Q, L))
    for b in range(Bz):
        n = int(end[b] - start[b])
        for h in range(Hq):
            s = q[b, h].astype(np.float64) @ k[b, h // g, start[b]:end[b]].astype(np.float64).T * scale
            if mask is not None:
                s = s + np.broadcast_to(mask, (Bz, Hq, Q, L))[b, h, :, :n]
            s -= s.max(axis=-1, keepdims=True)
            e = np.exp(s)
            out[b, h, :, :n] = e / e.sum(axis=-1, keepdims=True)
    return out


@pytest.mark.parametrize("D,dtype", [(128, torch.bfloat16), (64, torch.float16), (256, torch.bfloat16), (96, torch.bfloat16)])
def test_decode_weights_match_softmax(D, dtype):
    """The probabilities of the eager decode variant (modeling_qwen3sa.py:569-588) against a float64
    soft-max of the same scores: per-sequence ranges of different lengths (zeros behind the shorter
    ones), one query token and the boundary step's nine, GQA, an additive mask; each row sums to 1.
    Tolerance: the rounding of a probability to the 16-bit type (relative 2^-8 for bf16, 2^-11 for
    fp16) plus an absolute 1e-6."""
    import ksa_amd
    dev = torch.device("cuda")
    rel = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    for Q, rows, start, end in ((1, 900, np.array([0, 100, 640]), np.array([900, 777, 641])),
                                (9, 300, np.array([3, 3, 3]), np.array([139, 139, 139]))):
        q, k, v = _mk(3, 8, 2, Q, D, rows, seed=90 + Q + D, dtype=dtype)
        scale = D ** -0.5
        st, en = (torch.as_tensor(x, dtype=torch.int32, device=dev) for x in (start, end))
        w = ksa_amd.ksa_decode_weights(q.to(dev), k.to(dev), st, en)
        L = int((end - start).max())
        assert w.shape == (3, 8, Q, L) and w.dtype == dtype
        want = _weights_oracle(to_np(q), to_np(k), start, end, scale)
        got = to_np(w).astype(np.float64)
        assert (np.abs(got - want) <= rel * want + 1e-6).all(), np.abs(got - want).max()
        assert np.abs(got.sum(-1) - 1).max() <= 2e-2
        for b in range(3):
            assert (got[b, :, :, end[b] - start[b]:] == 0).all()
    # scalar range + additive mask that removes every third position and biases the rest
    q, k, v = _mk(2, 4, 4, 2, D, 200, seed=99, dtype=dtype)
    mask = torch.zeros(2, 1, 2, 150, dtype=dtype)
    mask[..., ::3] = float("-inf")
    mask[..., 1::3] = 0.5
    w = ksa_amd.ksa_decode_weights(q.to(dev), k.to(dev), 20, 170, mask=mask.to(dev))
    want = _weights_oracle(to_np(q), to_np(k), np.full(2, 20), np.full(2, 170), D ** -0.5, mask=to_np(mask).astype(np.float64))
    got = to_np(w).astype(np.float64)
    assert (np.abs(got - want) <= rel * want + 1e-6).all() and (got[..., ::3] == 0).all()


def test_eager_attention_forward_signature():
    """The reference's eager decode attention function (modeling_qwen3sa.py:569-588), as its cache call
    sites use it (:816-870: a slice of the cache, mask None): output equal to the SDPA variant's,
    probabilities consistent with it (weights @ V reproduces the output)."""
    import ksa_amd
    dev = torch.device("cuda")
    q, k, v = _mk(2, 8, 2, 1, 128, 500, seed=123)
    q, k, v = q.to(dev), k.to(dev), v.to(dev)

    class M:
        num_key_value_groups = 4
    out, w = ksa_amd.eager_attention_forward(M(), q, k[:, :, 7:444], v[:, :, 7:444], None, scaling=128 ** -0.5)
    ref, none = ksa_amd.decode_attention_forward(M(), q, k[:, :, 7:444], v[:, :, 7:444], None, scaling=128 ** -0.5)
    assert none is None and torch.equal(out, ref)
    assert w.shape == (2, 8, 1, 437)
    vv = v[:, :, 7:444].float().repeat_interleave(4, dim=1)           # [b, Hq, L, D]
    recon = torch.matmul(w.float(), vv).transpose(1, 2)                # [b, 1, Hq, D]
    assert (recon - out.float()).abs().max().item() <= 2e-2
    with pytest.raises(NotImplementedError):
        ksa_amd.eager_attention_forward(M(), q, k, v, torch.zeros(1, device=dev), scaling=1.0)


@pytest.mark.parametrize("D,dtype,g", [(128, torch.bfloat16, 4), (128, torch.float16, 1), (64, torch.bfloat16, 2),
                                       (256, torch.bfloat16, 4)])
@pytest.mark.parametrize("nsplit", [1, 3, None])
def test_decode_boundary_equals_two_decodes(D, dtype, g, nsplit):
    """The chunk-boundary form (text token over its range, the S summary tokens over theirs, one launch)
    against the two separate launches it stands for - bit for bit at the same split count - and
    against the oracle; per-sequence text ranges as device tensors with a scalar summary range (the
    small-window layer of a replayed step), per-sequence ranges for both (large window), and scalars."""
    import ksa_amd
    dev = torch.device("cuda")
    Bz, Hkv, S, C, rows = 3, 2, 8, 128, 1200
    q, k, v = _mk(Bz, Hkv * g, Hkv, 1 + S, D, rows, seed=17 + D + g, dtype=dtype)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    t0, t1 = np.array([136 - 5, 136 - 128, 136 - 77], np.int32), np.array([1100, 1100, 900], np.int32)
    cases = [((torch.as_tensor(t0, device=dev), torch.as_tensor(t1, device=dev)), (0, S + C), t0, t1, np.zeros(3, np.int32), np.full(3, S + C, np.int32))]
    s0, s1 = np.array([700, 650, 820], np.int32), np.array([836, 786, 956], np.int32)
    cases.append(((torch.as_tensor(np.zeros(3, np.int32), device=dev), torch.as_tensor(s1 - S, device=dev)),
                  (torch.as_tensor(s0, device=dev), torch.as_tensor(s1, device=dev)), np.zeros(3, np.int32), s1 - S, s0, s1))
    cases.append(((10, 1111), (0, 136), np.full(3, 10, np.int32), np.full(3, 1111, np.int32), np.zeros(3, np.int32), np.full(3, 136, np.int32)))
    for (ta, tb), (sa, sb), ta_n, tb_n, sa_n, sb_n in cases:
        got = ksa_amd.ksa_decode_boundary(qd, kd, vd, ta, tb, sa, sb, nsplit=nsplit)
        assert got.shape == (Bz, 1 + S, Hkv * g, D)
        want_t = c_oracle.decode(to_np(q[:, :, :1]), to_np(k), to_np(v), ta_n, tb_n)
        want_s = c_oracle.decode(to_np(q[:, :, 1:]), to_np(k), to_np(v), sa_n, sb_n)
        want = np.concatenate([want_t, want_s], axis=1)
        err = np.abs(to_np(got) - want).max()
        assert err <= ATOL and err <= RTOL_INF * np.abs(want).max(), err
        if nsplit is not None:
            two = torch.cat([ksa_amd.ksa_decode(qd[:, :, :1], kd, vd, ta, tb, nsplit=nsplit),
                             ksa_amd.ksa_decode(qd[:, :, 1:], kd, vd, sa, sb, nsplit=nsplit)], dim=1)
            assert torch.equal(got, two)
