"""The decode entry point that allocates nothing (`ksa_decode_fwd_noalloc`, split-K partials in
the library's own fixed device array) against `ksa_decode_fwd` with a caller-provided workspace:
bit-identical outputs (same kernels, same arithmetic), on two calls in a row, the second with
a smaller problem, so that stale partials of the first call would show.  Called through the C
ABI (ctypes), outputs and inputs preallocated by the test."""
import ctypes
import gc

import numpy as np
import pytest
import torch

from oracle import c_oracle

pytestmark = pytest.mark.gpu


def _call(lib_fn, q, kc, vc, out, start, end, nsplit, ws=None):
    from ksa_amd import _lib
    b, Hq, Q, D = q.shape
    args = [q.data_ptr(), kc.data_ptr(), vc.data_ptr(), out.data_ptr(), start.data_ptr(), end.data_ptr(), 0, 0,
            b, Hq, kc.shape[1], Q, D, 0,
            _lib.strides3(q, (0, 1, 2)), _lib.strides3(kc, (0, 1, 2)), _lib.strides3(vc, (0, 1, 2)),
            _lib.strides3(out, (0, 1, 2)), ctypes.c_float(D ** -0.5), nsplit]
    if ws is not None:
        args += [ws.data_ptr(), ctypes.c_size_t(ws.numel())]
    args.append(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return lib_fn(*args)


def _case(seed, b, Hq, Hkv, Q, rows, nsplit, dev):
    g = torch.Generator().manual_seed(seed)
    D = 128
    q = torch.randn(b, Hq, Q, D, generator=g).bfloat16().to(dev)
    kc = torch.randn(b, Hkv, rows, D, generator=g).bfloat16().to(dev)
    vc = torch.randn(b, Hkv, rows, D, generator=g).bfloat16().to(dev)
    start = torch.randint(0, rows // 4, (b,), generator=g).to(torch.int32)
    end = (start + torch.randint(1, rows - rows // 4, (b,), generator=g).to(torch.int32)).clamp(max=rows)
    return q, kc, vc, start.to(dev), end.to(dev)


def test_decode_noalloc_matches_workspace_entry_point():
    from ksa_amd import _lib
    L = _lib.lib()
    dev = torch.device("cuda")
    cap = L.ksa_decode_noalloc_max_workspace_bytes()
    assert cap == 32 << 20
    # first call: a larger problem with many splits; second call: smaller in every dimension
    for seed, (b, Hq, Hkv, Q, rows, nsplit) in enumerate([(6, 16, 4, 1, 3000, 8), (2, 8, 2, 1, 700, 3),
                                                          (3, 8, 2, 9, 900, 4), (1, 8, 8, 1, 300, 2)]):
        q, kc, vc, start, end = _case(seed, b, Hq, Hkv, Q, rows, nsplit, dev)
        need = L.ksa_decode_workspace_bytes(b, Hq, Hkv, Q, 128, nsplit)
        assert 0 < need <= cap
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        want = torch.full((b, Q, Hq, 128), float("nan"), dtype=torch.bfloat16, device=dev)
        got = torch.full_like(want, float("nan"))
        assert _call(L.ksa_decode_fwd, q, kc, vc, want, start, end, nsplit, ws) == 0
        # nothing may be allocated or freed, neither through torch's allocator nor below it
        # (a hipMalloc inside the library shows in the device's free bytes, not in torch's count)
        # (garbage of earlier tests collected in the middle of the window would show as a change that
        # the call did not make: collect it first and keep the collector off for the window)
        gc.collect()
        torch.cuda.synchronize()
        gc.disable()
        try:
            before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
            assert _call(L.ksa_decode_fwd_noalloc, q, kc, vc, got, start, end, nsplit) == 0
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated() == before
            if seed > 0:   # (the first call on a device may load the library's code object)
                assert torch.cuda.mem_get_info()[0] == free_before
        finally:
            gc.enable()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (seed, b, Hq, Hkv, Q, rows, nsplit)
        ref = c_oracle.decode(q.float().cpu().numpy(), kc.float().cpu().numpy(), vc.float().cpu().numpy(),
                              start.cpu().numpy(), end.cpu().numpy())
        assert np.abs(got.float().cpu().numpy() - ref).max() <= 2e-2
    # one split needs no scratch at all and takes the same path
    q, kc, vc, start, end = _case(9, 2, 8, 2, 1, 500, 1, dev)
    want = torch.empty(2, 1, 8, 128, dtype=torch.bfloat16, device=dev)
    got = torch.empty_like(want)
    assert _call(L.ksa_decode_fwd, q, kc, vc, want, start, end, 1, torch.empty(16, dtype=torch.uint8, device=dev)) == 0
    assert _call(L.ksa_decode_fwd_noalloc, q, kc, vc, got, start, end, 1) == 0
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_decode_noalloc_rejects_oversized_problem():
    """A problem whose partials do not fit the fixed array is refused before any launch."""
    from ksa_amd import _lib
    L = _lib.lib()
    dev = torch.device("cuda")
    b, Hq, Hkv, Q, rows, nsplit = 64, 32, 8, 1, 64, 16
    assert L.ksa_decode_workspace_bytes(b, Hq, Hkv, Q, 128, nsplit) > L.ksa_decode_noalloc_max_workspace_bytes()
    q, kc, vc, start, end = _case(1, b, Hq, Hkv, Q, rows, nsplit, dev)
    out = torch.zeros(b, Q, Hq, 128, dtype=torch.bfloat16, device=dev)
    rc = _call(L.ksa_decode_fwd_noalloc, q, kc, vc, out, start, end, nsplit)
    assert rc == -4 and b"workspace" in L.ksa_error_string(rc)
    torch.cuda.synchronize()
    assert int(out.abs().sum()) == 0
