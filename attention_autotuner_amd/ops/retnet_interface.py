"""``RetNetAttnFunc(q, k, v, mask, device_type[, causal])`` -- RetNet parallel retention, fwd + bwd.

Drop-in for reference python/ops/retnet_interface.py:8-57:
``S = (q k^T) * mask``, ``r = clamp(sum_j |S|, min=1)`` (treated as a constant in the gradient),
``o = (S / r) v``.  mask is [H, S_q, S_kv] fp16.  ``causal=True`` promises the mask is zero above the
diagonal, which lets the kernels skip those tiles (the reference accepts and ignores the flag).
backward returns one gradient per forward input (the reference returns one too few).
"""
import torch

from ..arch import Arch
from ..autotuner import gfx950_space
from ..autotuner.runtime import Runtime
from ..autotuner.tunner import RetTunner, RetBwdTunner
from ._resolve import resolve


class RetNetAttn(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, mask, device_type: Arch, causal=False):
        if not (q.is_cuda and k.is_cuda and v.is_cuda and mask.is_cuda):
            raise RuntimeError("RetNetAttnFunc runs on the GPU only (HIP kernels); move the tensors to a cuda device")
        assert q.dtype == torch.float16 and k.dtype == torch.float16 and v.dtype == torch.float16 and mask.dtype == torch.float16
        q, k, v = [x.contiguous() for x in (q, k, v)]
        maskr = mask.detach().contiguous()
        batch_size, nheads, seqlen_q, key_dim = q.shape
        seqlen_k = k.shape[2]
        head_dim = v.shape[-1]
        assert maskr.shape == (nheads, seqlen_q, seqlen_k)
        assert head_dim % 64 == 0 and head_dim <= 512
        assert key_dim % 64 == 0 and key_dim <= 256

        o = torch.empty(batch_size, nheads, seqlen_q, head_dim, device=q.device, dtype=torch.float16)
        r = torch.empty(batch_size, nheads, seqlen_q, device=q.device, dtype=torch.float32)
        arrays = [q, k, v, maskr, o, r]
        tuner = RetTunner(arch=device_type, torch_array=arrays, causal=causal)
        cc = resolve(tuner, lambda: gfx950_space.default_forward_config("ret", key_dim, head_dim, device_type, seqlen_q, seqlen_k))
        Runtime(device_type, cc).apply(arrays, causal=causal)
        ctx.save_for_backward(q, k, v, maskr, r)
        ctx.device_type = device_type
        ctx.causal = causal
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, mask, r = ctx.saved_tensors
        device_type = ctx.device_type
        batch_size, nheads, seqlen_q, key_dim = q.shape
        head_dim = v.shape[-1]
        seqlen_k = k.shape[2]
        do = do.contiguous()
        dq = torch.empty_like(q)
        dk = torch.empty_like(k)
        dv = torch.empty_like(v)
        dq_accum = torch.zeros([batch_size, nheads, seqlen_q, key_dim], device=q.device, dtype=torch.float32)
        arrays = [q, k, v, mask, do, r, dq, dk, dv, dq_accum]
        tuner = RetBwdTunner(arch=device_type, torch_array=arrays, causal=ctx.causal)
        tuned_now = tuner.check_cache() is None
        cc = resolve(tuner, lambda: gfx950_space.default_backward_config(key_dim, head_dim, device_type, seqlen_q, seqlen_k))
        if tuned_now:
            dq_accum.zero_()                      # tuning launches accumulated into the scratch
        Runtime(device_type, cc).apply(arrays, causal=ctx.causal)
        return dq, dk, dv, None, None, None


RetNetAttnFunc = RetNetAttn.apply
