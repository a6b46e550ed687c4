"""CPU fp32 stand-ins for the attention-side and element-wise operators of `ksa_amd.model`, built from
the oracle's restatements.  TEST INFRASTRUCTURE ONLY: with these the build's own end-to-end
module runs on the host in fp32, which is the run its GPU results are compared with.

Follows examples/pretrain/hf_template/modeling_qwen3sa.py: :64-79, :516-554, :660-666
(pre-attention, via cpu_path.pre_attention), whl-sa summary_attn/interface.py:271-289 (the
summary rows form the key prefix; dense masked soft-max via ksa_oracle.masked_attention),
:557-566, :591-612 (decode: un-masked soft-max over the cache slice), :85-505 (the cache,
product bookkeeping with a host row mover), :64-79, :507-514, :946, :952 (residual add + RMSNorm,
SiLU-mul, via cpu_path).
"""
from __future__ import annotations

import numpy as np
import torch

from . import cpu_path
from . import ksa_oracle as O


def _host_mover(src, dst, nrows, src_start=0, dst_start=0, src_index=None):
    if nrows <= 0:
        return
    rows = src_index.long() if src_index is not None else torch.arange(src_start, src_start + nrows)
    dst[:, :, dst_start:dst_start + nrows, :] = src[:, :, rows[:nrows], :].clone()


class OracleOps:
    def __init__(self):
        from ksa_amd.cache import Qwen3RingBufferCache

        class HostCache(Qwen3RingBufferCache):
            _move_rows = staticmethod(_host_mover)
        self.cache_cls = HostCache

    @staticmethod
    def pre_attention(q, k, v, qw, kw, cos, sin, eps, q_out=None, k_out=None, v_out=None, kv_out_row=None):
        assert kv_out_row is None, "device-side cache cursors belong to the GPU operators"
        qo, ko, vo = cpu_path.pre_attention(q, k, v, qw, kw, cos, sin, eps)
        res = []
        for given, val in ((q_out, qo), (k_out, ko), (v_out, vo)):
            if given is not None:
                given.copy_(val)
                val = given
            res.append(val)
        return tuple(res)

    @staticmethod
    def linear(x, weight, defer=False):  # `defer` is a launch-count hint of the GPU operators
        return torch.nn.functional.linear(x, weight)
    add_rmsnorm = staticmethod(cpu_path.add_rmsnorm)
    @staticmethod
    def silu_mul(gate, up=None):
        if up is None:  # the whole gate | up projection
            I = gate.shape[-1] // 2
            gate, up = gate[..., :I], gate[..., I:]
        return cpu_path.silu_mul(gate, up)

    @staticmethod
    def summary_attn_func(q, k, v, C, S, W, summary_pos=None):
        sp = None if summary_pos is None else summary_pos.numpy()
        outs = []
        for b in range(q.shape[0]):
            o, _ = O.masked_attention(q[b].numpy(), k[b].numpy(), v[b].numpy(), C, S, W,
                                      summary_pos=sp, dtype=np.float64)
            outs.append(torch.from_numpy(o).to(q.dtype))
        return torch.stack(outs), None

    @staticmethod
    def decode(q, kbuf, vbuf, start, end, scale):
        # only the attended rows are converted (the rest of a cache buffer is uninitialised)
        o = O.decode_attention(q.numpy(), kbuf[:, :, start:end].numpy(), vbuf[:, :, start:end].numpy(),
                               scale=scale)
        return torch.from_numpy(o).to(q.dtype)
