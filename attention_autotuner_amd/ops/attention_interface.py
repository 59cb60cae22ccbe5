"""``flash_attn_func(q, k, v, device_type[, causal[, softmax_scale]])`` -- fused attention forward.

Drop-in for reference python/ops/attention_interface.py:8-60: same tensor layout ([B, H, S, D] fp16 on
the GPU), same positional arguments, same asserts on the head sizes, same tune-then-launch flow.
Additions: ``causal`` is honoured (the reference accepts and ignores it) and ``softmax_scale``
defaults to 1/sqrt(d_qk) (the reference hard-codes 0.125, available as REFERENCE_SOFTMAX_SCALE).
"""
import math

import torch

from ..arch import Arch
from ..autotuner import gfx950_space
from ..autotuner.runtime import Runtime
from ..autotuner.tunner import AttnTunner
from ._resolve import resolve

REFERENCE_SOFTMAX_SCALE = 0.125


class MultiHeadAttnFunc(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, device_type: Arch, causal=False, softmax_scale=None):
        """q: (batch, nheads, seqlen_q, key_dim); k: (batch, nheads, seqlen_k, key_dim);
        v: (batch, nheads, seqlen_k, head_dim); returns (batch, nheads, seqlen_q, head_dim)."""
        if not (q.is_cuda and k.is_cuda and v.is_cuda):
            raise RuntimeError("flash_attn_func runs on the GPU only (HIP kernels); move q, k, v to a cuda device")
        assert q.dtype == torch.float16 and k.dtype == torch.float16 and v.dtype == torch.float16
        q, k, v = [x.contiguous() for x in (q, k, v)]
        batch_size, nheads, seqlen_q, key_dim = q.shape
        seqlen_k = k.shape[2]
        head_dim = v.shape[-1]
        assert k.shape == (batch_size, nheads, seqlen_k, key_dim) and v.shape[:3] == k.shape[:3]
        assert head_dim % 64 == 0 and head_dim <= 512
        assert key_dim % 64 == 0 and key_dim <= 256
        if softmax_scale is None:
            softmax_scale = 1.0 / math.sqrt(key_dim)

        o = torch.empty(batch_size, nheads, seqlen_q, head_dim, device=q.device, dtype=q.dtype)
        tuner = AttnTunner(arch=device_type, torch_array=[q, k, v, o], causal=causal, softmax_scale=softmax_scale)
        cc = resolve(tuner, lambda: gfx950_space.default_forward_config("attn", key_dim, head_dim, device_type, seqlen_q, seqlen_k))
        Runtime(device_type, cc).apply([q, k, v, o], softmax_scale=softmax_scale, causal=causal)
        ctx.save_for_backward(q, k, v)
        ctx.device_type = device_type
        return o

    @staticmethod
    def backward(ctx, do):
        raise NotImplementedError("attention backward is not part of this operator (the reference leaves it empty as well)")


flash_attn_func = MultiHeadAttnFunc.apply
