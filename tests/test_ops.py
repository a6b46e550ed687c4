"""The helper operators as `torch.ops.ksa_amd.*` (`ksa_amd/ops.py`): registration and shape-only (fake)
kernels on the CPU; on the GPU each operator against the direct call (bit-identical: same kernel),
`torch.library.opcheck`, and a traced layer body (`torch.compile`, graph capture without code
generation) against the same body run eagerly.
"""
import pytest
import torch

H, I, HQ, HKV, D = 256, 512, 4, 2, 64


def _layer_weights(dev, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)

    def r(*shape, s=0.05):
        return (torch.randn(*shape, generator=g) * s).to(dtype).to(dev)

    return {"norm1": 1 + r(H), "norm2": 1 + r(H), "qkv": r((HQ + 2 * HKV) * D, H), "o": r(H, HQ * D),
            "gate_up": r(2 * I, H), "down": r(H, I), "qn": 1 + r(D), "kn": 1 + r(D)}


def _rope(rows, dev, dtype):
    pos = torch.arange(rows, dtype=torch.float32)
    inv = 1.0 / (10000 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    f = torch.outer(pos, inv)
    e = torch.cat((f, f), -1)
    return e.cos().to(dtype).to(dev)[None], e.sin().to(dtype).to(dev)[None]


def test_operators_registered_with_fake_kernels():
    import ksa_amd
    from torch._subclasses.fake_tensor import FakeTensorMode
    ns = torch.ops.ksa_amd
    for name in ksa_amd.ops.OPERATORS:
        assert hasattr(ns, name), name
    ks = ksa_amd.ops.mlp_rows_down_splits(H, I)
    with FakeTensorMode():
        bf = dict(dtype=torch.bfloat16, device="cuda")
        x = torch.empty(2, 4, H, **bf)
        w = torch.empty(H, **bf)
        s, y = ns.add_rmsnorm(x, x, w, 1e-6)
        assert s.shape == x.shape and y.shape == x.shape and y.dtype == torch.bfloat16 and y.device.type == "cuda"
        assert ns.rmsnorm(x, w, 1e-6).shape == x.shape
        qkv = ns.linear_rows(x, torch.empty((HQ + 2 * HKV) * D, H, **bf))
        assert qkv.shape == (2, 4, (HQ + 2 * HKV) * D)
        q = qkv[..., :HQ * D].view(2, 4, HQ, D)
        k = qkv[..., HQ * D:(HQ + HKV) * D].view(2, 4, HKV, D)
        cs = torch.empty(1, 4, D, **bf)
        qo, ko, vo = ns.pre_attention(q, k, k, torch.empty(D, **bf), torch.empty(D, **bf), cs, cs, 1e-6)
        assert qo.shape == q.shape and ko.shape == k.shape and vo.shape == k.shape
        assert ns.gate_up_silu_rows(x, torch.empty(2 * I, H, **bf)).shape == (2, 4, I)
        g = torch.empty(2, 4, I, **bf)
        assert ns.silu_mul(g, g).shape == g.shape
        part = ns.mlp_rows(x, torch.empty(2 * I, H, **bf), torch.empty(H, I, **bf),
                           torch.empty(64, dtype=torch.uint8, device="cuda"))
        assert part.shape == (ks, 16, H) and part.dtype == torch.float32
        s2, y2 = ns.add_rmsnorm_partials(part, x, w, 1e-6)
        assert s2.shape == x.shape and y2.dtype == torch.bfloat16
        am = ns.argmax_rows(torch.empty(2, 4, 1000, **bf))
        assert am.shape == (2, 4) and am.dtype == torch.long


def _layer_body(ka, x, res, W, cos, sin):
    """The element-wise and few-rows steps of one decoder layer around the attention call (which is left
    out: q stands in for its output), through the package-level functions."""
    res, h = ka.add_rmsnorm(x, res, W["norm1"], 1e-6)
    qkv = ka.linear_rows(h, W["qkv"])
    b, S = x.shape[:2]
    q = qkv[..., :HQ * D].view(b, S, HQ, D)
    k = qkv[..., HQ * D:(HQ + HKV) * D].view(b, S, HKV, D)
    v = qkv[..., (HQ + HKV) * D:].view(b, S, HKV, D)
    q, k, v = ka.pre_attention(q, k, v, W["qn"], W["kn"], cos, sin, 1e-6)
    o = ka.linear_rows(q.reshape(b, S, HQ * D), W["o"])
    res, h = ka.add_rmsnorm(o, res, W["norm2"], 1e-6)
    a = ka.silu_mul(ka.linear_rows(h, W["gate_up"]))
    return res, ka.linear_rows(a, W["down"]), k, v


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gpu_traced_layer_body_equals_eager(dtype):
    import ksa_amd
    dev = torch.device("cuda", 0)
    W = _layer_weights(dev, dtype)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 4, H, generator=g).to(dtype).to(dev)
    res = torch.randn(2, 4, H, generator=g).to(dtype).to(dev)
    cos, sin = _rope(4, dev, dtype)
    exp = _layer_body(ksa_amd, x, res, W, cos, sin)
    torch._dynamo.reset()
    seen = []

    def backend(gm, example_inputs):  # graph capture only: the captured graph is run as it is
        seen.extend(str(n.target) for n in gm.graph.nodes if n.op == "call_function")
        return gm.forward

    fn = torch.compile(lambda x, res, cos, sin: _layer_body(ksa_amd, x, res, W, cos, sin), backend=backend,
                       fullgraph=True)
    got = fn(x, res, cos, sin)
    for name in ("add_rmsnorm", "linear_rows", "pre_attention", "silu_mul"):
        assert any("ksa_amd." + name in t or "ksa_amd::" + name in t for t in seen), (name, seen)
    for a, b in zip(got, exp):
        assert torch.equal(a, b)


@pytest.mark.gpu
def test_gpu_operators_equal_direct_calls_and_opcheck():
    import ksa_amd
    from ksa_amd import elementwise, gemm, pre
    ns = torch.ops.ksa_amd
    dev = torch.device("cuda", 0)
    dtype = torch.bfloat16
    W = _layer_weights(dev, dtype, seed=2)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(8, H, generator=g).to(dtype).to(dev)
    res = torch.randn(8, H, generator=g).to(dtype).to(dev)
    cases = []
    # residual add + norm, norm alone
    s, y = ns.add_rmsnorm(x, res, W["norm1"], 1e-6)
    es, ey = elementwise.add_rmsnorm(x, res, W["norm1"], 1e-6)
    assert torch.equal(s, es) and torch.equal(y, ey)
    assert torch.equal(ns.rmsnorm(x, W["norm1"], 1e-6), elementwise.add_rmsnorm(x, None, W["norm1"], 1e-6)[1])
    cases.append((ns.add_rmsnorm, (x, res, W["norm1"], 1e-6)))
    cases.append((ns.rmsnorm, (x, W["norm1"], 1e-6)))
    # projections
    assert torch.equal(ns.linear_rows(x, W["qkv"]), gemm.linear_rows(x, W["qkv"]))
    assert torch.equal(ns.gate_up_silu_rows(x, W["gate_up"]), gemm.gate_up_silu_rows(x, W["gate_up"]))
    cases.append((ns.linear_rows, (x, W["qkv"])))
    cases.append((ns.gate_up_silu_rows, (x, W["gate_up"])))
    gu = gemm.linear_rows(x, W["gate_up"])
    assert torch.equal(ns.silu_mul(gu[:, :I], gu[:, I:]), elementwise.silu_mul(gu))
    cases.append((ns.silu_mul, (gu[:, :I], gu[:, I:])))
    # q/k norm + rotary
    qkv = gemm.linear_rows(x, W["qkv"]).view(2, 4, -1)
    q = qkv[..., :HQ * D].view(2, 4, HQ, D)
    k = qkv[..., HQ * D:(HQ + HKV) * D].view(2, 4, HKV, D)
    v = qkv[..., (HQ + HKV) * D:].view(2, 4, HKV, D)
    cos, sin = _rope(4, dev, dtype)
    for a, b in zip(ns.pre_attention(q, k, v, W["qn"], W["kn"], cos, sin, 1e-6),
                    pre.pre_attention(q, k, v, W["qn"], W["kn"], cos, sin, 1e-6)):
        assert torch.equal(a, b)
    cases.append((ns.pre_attention, (q, k, v, W["qn"], W["kn"], cos, sin, 1e-6)))
    # one-launch MLP and the norm that adds its partial sums: against the separate launches
    ws = ksa_amd.ops.mlp_rows_workspace(H, I, dev)
    part = ns.mlp_rows(x, W["gate_up"], W["down"], ws)
    s2, y2 = ns.add_rmsnorm_partials(part, res, W["norm2"], 1e-6)
    down = gemm.linear_rows(gemm.gate_up_silu_rows(x, W["gate_up"]), W["down"])
    es2, ey2 = elementwise.add_rmsnorm(down, res, W["norm2"], 1e-6)
    # (the partial sums are added in fp32 and rounded once, the separate launches round the product first)
    assert (s2.float() - es2.float()).abs().max() <= 2 ** -6 * es2.float().abs().max()
    assert (y2.float() - ey2.float()).abs().max() <= 2 ** -5 * ey2.float().abs().max()
    logits = torch.randn(8, 1000, generator=g).to(dtype).to(dev)
    assert torch.equal(ns.argmax_rows(logits), torch.argmax(logits, dim=-1))
    cases.append((ns.argmax_rows, (logits,)))
    for op, args in cases:
        torch.library.opcheck(op, args, test_utils=("test_schema", "test_faketensor"))
    # the workspace argument is declared as written to
    torch.library.opcheck(ns.mlp_rows, (x, W["gate_up"], W["down"], ws), test_utils=("test_schema", "test_faketensor"))
    assert int(ws[ksa_amd._lib.lib().ksa_mlp_rows_status_offset():][:8].view(torch.int64).item()) == 0
