"""``RetNetAttnFunc(q, k, v, mask, device_type[, causal])`` -- RetNet parallel retention, fwd + bwd.

Drop-in for reference python/ops/retnet_interface.py:8-57:
``S = (q k^T) * mask``, ``r = clamp(sum_j |S|, min=1)`` (treated as a constant in the gradient),
``o = (S / r) v``.  mask is [H, S_q, S_kv] fp16.  Tiles in which the mask is zero contribute exactly
nothing, and RetNet's own masks are zero above the diagonal, so by default (``causal=None``) the forward
scans the mask once (one read of it, on the GPU, no host synchronisation) and forward and backward then
skip the all-zero tiles at the start and end of every band of rows; the result has the same bits as the
dense walk.  ``causal=True`` promises zeros above the diagonal instead of scanning, ``causal=False`` walks
every tile as the reference does (it accepts the flag and ignores it).
backward returns one gradient per forward input (the reference returns one too few).
A model applies one mask in every layer and step: ``scan = retnet_mask_scan(mask, device_type)`` takes the scan once
and ``RetNetAttnFunc(q, k, v, mask, device_type, scan)`` reuses it (the caller vouches that ``mask`` has not changed
since; 18 us per forward at H 8, S 2048).

``RetNetDecayAttnFunc(q, k, v, gamma, device_type)`` is the same operator for RetNet's own mask,
``mask[h, i, j] = gamma_h^(i + S_kv - S_q - j)`` on and below that diagonal and 0 above it: the mask is
built in registers from ``gamma`` ([H], 0.5 <= gamma_h <= 1) instead of being streamed from a
[H, S_q, S_kv] tensor, and tiles above the diagonal are skipped.  The reference has no such entry (it
always streams the tensor, python/ops/retnet_interface.py:26-31).
"""
import torch

from ..arch import Arch
from ..autotuner import gfx950_space
from ..autotuner.runtime import Runtime
from ..autotuner.tunner import RetTunner, RetBwdTunner
from ._resolve import NoGraph, planned, wants_graph


def retnet_mask_scan(mask, device_type: Arch):
    """The scan of ``mask`` ([H, S_q, S_kv] fp16 on the GPU) that ``RetNetAttnFunc(..., causal=None)`` would take in its
    forward: pass the result as ``causal`` to every call that uses this same, unchanged mask.  The bytes have the layout
    every RetNet library reads (``AAT_MASK_SCANNED``)."""
    assert mask.is_cuda and mask.dtype == torch.float16 and mask.dim() == 3
    maskr = mask.detach().contiguous()
    nheads, seqlen_q, seqlen_k = maskr.shape
    # the scan is part of a forward launch: a one-batch launch of the smallest library on zeros
    rt = Runtime(device_type, gfx950_space.default_forward_config("ret", 64, 64, device_type, seqlen_q, seqlen_k))
    z = torch.zeros(1, nheads, max(seqlen_q, seqlen_k), 64, device=mask.device, dtype=torch.float16)
    o = torch.empty(1, nheads, seqlen_q, 64, device=mask.device, dtype=torch.float16)
    r = torch.empty(1, nheads, seqlen_q, device=mask.device, dtype=torch.float32)
    scan = torch.empty(rt.workspace_size(1, nheads, seqlen_q, seqlen_k), dtype=torch.uint8, device=mask.device)
    rt.apply([z[:, :, :seqlen_q].contiguous(), z[:, :, :seqlen_k].contiguous(), z[:, :, :seqlen_k].contiguous(), maskr, o, r],
             causal="scan", workspace=scan)
    return scan


class RetNetAttn(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, mask, device_type: Arch, causal=None):
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
        # the scanning walk is tuned as the causal one: masks that have zero tiles to skip are of that kind
        reused = causal if torch.is_tensor(causal) else None      # a scan taken earlier (retnet_mask_scan)
        if reused is not None:
            causal = None
        # ... but a tuning run on a cache miss times and verifies its candidates in the mode launched here, on this mask
        walk, mode = causal is None or bool(causal), "scan" if causal is None else None
        _, rt = planned(("ret", device_type.name, batch_size, nheads, seqlen_q, seqlen_k, key_dim, head_dim, walk, mode),
                        lambda: RetTunner(arch=device_type, torch_array=arrays, causal=walk, mask_mode=mode),
                        lambda: gfx950_space.default_forward_config("ret", key_dim, head_dim, device_type, seqlen_q, seqlen_k))
        scan = None
        if reused is not None:
            scan = reused
            assert scan.is_cuda and scan.dtype == torch.uint8 and scan.numel() >= rt.workspace_size(batch_size, nheads, seqlen_q, seqlen_k), \
                "causal: a scan from retnet_mask_scan(mask, device_type) of a mask of this shape"
            rt.apply(arrays, causal="scanned", workspace=scan)
        elif causal is None:                   # the scan lands in `scan`; the backward reads it from there
            scan = torch.empty(rt.workspace_size(batch_size, nheads, seqlen_q, seqlen_k), dtype=torch.uint8, device=q.device)
            rt.apply(arrays, causal="scan", workspace=scan)
        else:
            rt.apply(arrays, causal=bool(causal))
        ctx.save_for_backward(q, k, v, maskr, r)
        ctx.device_type = device_type
        ctx.causal = causal
        ctx.mask_scan = scan
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
        # The reference's kernel accumulates dQ into this fp32 scratch with atomics; the kernels here never
        # touch it (dQ is produced directly), so a token buffer stands in for the [B,H,S_q,d_qk] tensor -- uninitialised:
        # zeroing it would put a fill kernel between the forward's and the backward's launches for nothing.
        dq_accum = torch.empty(1, device=q.device, dtype=torch.float32)
        arrays = [q, k, v, mask, do, r, dq, dk, dv, dq_accum]
        walk, mode = ctx.causal is None or bool(ctx.causal), "scan" if ctx.mask_scan is not None else None
        _, rt = planned(("ret_bwd", device_type.name, batch_size, nheads, seqlen_q, seqlen_k, key_dim, head_dim, walk, mode),
                        lambda: RetBwdTunner(arch=device_type, torch_array=arrays, causal=walk, mask_mode=mode),
                        lambda: gfx950_space.default_backward_config(key_dim, head_dim, device_type, seqlen_q, seqlen_k))
        if ctx.mask_scan is not None:
            rt.apply(arrays, causal="scanned", workspace=ctx.mask_scan)
        else:
            rt.apply(arrays, causal=bool(ctx.causal))
        return dq, dk, dv, None, None, None


_LOG2_GAMMA = {}          # (rates, device) -> log2(gamma) on the device: the rates of a model never change between calls


def _log2_gamma(gamma, nheads, device):
    """fp32 [H] tensor of log2(gamma_h) on ``device``.  Checking the rates and copying them to the GPU takes a
    host round trip, so the result is kept per set of rates."""
    values = tuple(float(g) for g in (gamma.detach().cpu().reshape(-1).tolist() if torch.is_tensor(gamma) else gamma))
    key = (values, str(device))
    lg = _LOG2_GAMMA.get(key)
    if lg is None:
        g64 = torch.tensor(values, dtype=torch.float64)
        assert g64.numel() == nheads and bool(((g64 >= 0.5) & (g64 <= 1.0)).all()), "one decay rate in [0.5, 1] per head"
        lg = torch.log2(g64).to(device=device, dtype=torch.float32).contiguous()
        if len(_LOG2_GAMMA) >= 64:
            _LOG2_GAMMA.clear()
        _LOG2_GAMMA[key] = lg
    assert lg.numel() == nheads, "one decay rate in [0.5, 1] per head"
    return lg


class RetNetDecayAttn(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, gamma, device_type: Arch):
        if not (q.is_cuda and k.is_cuda and v.is_cuda):
            raise RuntimeError("RetNetDecayAttnFunc runs on the GPU only (HIP kernels); move the tensors to a cuda device")
        assert q.dtype == torch.float16 and k.dtype == torch.float16 and v.dtype == torch.float16
        q, k, v = [x.contiguous() for x in (q, k, v)]
        batch_size, nheads, seqlen_q, key_dim = q.shape
        seqlen_k = k.shape[2]
        head_dim = v.shape[-1]
        assert head_dim % 64 == 0 and head_dim <= 512
        assert key_dim % 64 == 0 and key_dim <= 256
        lg = _log2_gamma(gamma, nheads, q.device)

        o = torch.empty(batch_size, nheads, seqlen_q, head_dim, device=q.device, dtype=torch.float16)
        r = torch.empty(batch_size, nheads, seqlen_q, device=q.device, dtype=torch.float32)
        arrays = [q, k, v, lg, o, r]
        _, rt = planned(("ret_decay", device_type.name, batch_size, nheads, seqlen_q, seqlen_k, key_dim, head_dim),
                        lambda: RetTunner(arch=device_type, torch_array=arrays, decay=True),
                        lambda: gfx950_space.default_forward_config("ret", key_dim, head_dim, device_type, seqlen_q, seqlen_k))
        rt.apply(arrays, decay=True)
        ctx.save_for_backward(q, k, v, lg, r)
        ctx.device_type = device_type
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, lg, r = ctx.saved_tensors
        device_type = ctx.device_type
        key_dim, head_dim = q.shape[-1], v.shape[-1]
        seqlen_q, seqlen_k = q.shape[2], k.shape[2]
        do = do.contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        arrays = [q, k, v, lg, do, r, dq, dk, dv]
        _, rt = planned(("ret_bwd_decay", device_type.name, q.shape[0], q.shape[1], seqlen_q, seqlen_k, key_dim, head_dim),
                        lambda: RetBwdTunner(arch=device_type, torch_array=arrays, decay=True),
                        lambda: gfx950_space.default_backward_config(key_dim, head_dim, device_type, seqlen_q, seqlen_k))
        rt.apply(arrays, decay=True)
        return dq, dk, dv, None, None


def RetNetAttnFunc(q, k, v, mask, device_type: Arch, causal=None):
    """``RetNetAttn.apply`` (the reference's ``RetNetAttnFunc``, python/ops/retnet_interface.py:57) when a gradient may
    be asked for; the same forward without the autograd machinery otherwise."""
    if wants_graph(q, k, v):
        return RetNetAttn.apply(q, k, v, mask, device_type, causal)
    return RetNetAttn.forward(NoGraph(), q, k, v, mask, device_type, causal)


def RetNetDecayAttnFunc(q, k, v, gamma, device_type: Arch):
    if wants_graph(q, k, v):
        return RetNetDecayAttn.apply(q, k, v, gamma, device_type)
    return RetNetDecayAttn.forward(NoGraph(), q, k, v, gamma, device_type)
