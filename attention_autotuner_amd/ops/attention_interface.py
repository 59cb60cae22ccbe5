"""``flash_attn_func(q, k, v, device_type[, causal[, softmax_scale]])`` -- fused attention forward.

Drop-in for reference python/ops/attention_interface.py:8-60: same tensor layout ([B, H, S, D] fp16 on
the GPU), same positional arguments, same asserts on the head sizes, same tune-then-launch flow.
Additions: ``causal`` is honoured (the reference accepts and ignores it), ``softmax_scale``
defaults to 1/sqrt(d_qk) (the reference hard-codes 0.125, available as REFERENCE_SOFTMAX_SCALE), and
``backward`` is implemented (the reference's is an empty stub, python/ops/attention_interface.py:37-58):
when any input requires a gradient the forward also stores the log-sum-exp of every row, and the
backward launches the attention-backward library (dq, dk, dv in fp16, no atomics).
"""
import math

import torch

from ..arch import Arch
from ..autotuner import gfx950_space
from ..autotuner.tunner import AttnBwdTunner, AttnTunner
from ._resolve import NoGraph, planned, wants_graph

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
        causal = bool(causal)
        _, rt = planned(("attn", device_type.name, batch_size, nheads, seqlen_q, seqlen_k, key_dim, head_dim, causal),
                        lambda: AttnTunner(arch=device_type, torch_array=[q, k, v, o], causal=causal, softmax_scale=softmax_scale),
                        lambda: gfx950_space.default_forward_config("attn", key_dim, head_dim, device_type, seqlen_q, seqlen_k))
        needs_grad = any(ctx.needs_input_grad[:3])
        lse = torch.empty(batch_size, nheads, seqlen_q, device=q.device, dtype=torch.float32) if needs_grad else None
        rt.apply([q, k, v, o], softmax_scale=softmax_scale, causal=causal, lse=lse)
        if needs_grad:
            ctx.save_for_backward(q, k, v, o, lse)
        ctx.device_type = device_type
        ctx.causal = bool(causal)
        ctx.softmax_scale = float(softmax_scale)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse = ctx.saved_tensors
        device_type = ctx.device_type
        key_dim, head_dim = q.shape[-1], v.shape[-1]
        seqlen_q, seqlen_k = q.shape[2], k.shape[2]
        do = do.contiguous()
        assert do.dtype == torch.float16 and do.shape == o.shape
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        arrays = [q, k, v, o, do, lse, dq, dk, dv]
        try:
            _, rt = planned(("attn_bwd", device_type.name, q.shape[0], q.shape[1], seqlen_q, seqlen_k, key_dim, head_dim, ctx.causal),
                            lambda: AttnBwdTunner(arch=device_type, torch_array=arrays, causal=ctx.causal, softmax_scale=ctx.softmax_scale),
                            lambda: gfx950_space.default_attn_backward_config(key_dim, head_dim, device_type, seqlen_q, seqlen_k))
        except gfx950_space.NoValidConfigError as e:      # e.g. d_v = 512: dK and dV do not fit one wave's registers
            raise NotImplementedError(f"attention backward: {e}") from e
        rt.apply(arrays, softmax_scale=ctx.softmax_scale, causal=ctx.causal)
        return dq, dk, dv, None, None, None


def flash_attn_func(q, k, v, device_type: Arch, causal=False, softmax_scale=None):
    """``MultiHeadAttnFunc.apply`` (the reference's ``flash_attn_func``, python/ops/attention_interface.py:60) when a
    gradient may be asked for; the same forward without the autograd machinery otherwise."""
    if wants_graph(q, k, v):
        return MultiHeadAttnFunc.apply(q, k, v, device_type, causal, softmax_scale)
    return MultiHeadAttnFunc.forward(NoGraph(), q, k, v, device_type, causal, softmax_scale)
