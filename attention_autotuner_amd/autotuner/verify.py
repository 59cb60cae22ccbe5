"""Guard used by the tuning loop: before a configuration is written to the cache, its library is run
once on the tuner's own tensors and its outputs are compared with plain fp32 torch math on the GPU.

The reference's tuner ranks candidates by time alone (python/autotuner/base_tunner.py:157-168).  Here a
candidate is a separately compiled kernel with its own register allocation, so a wrong-but-fast library
must not be able to win.  This is a sanity bound (``atol + rtol * |ref|``), not the parity test: parity
against the CPU oracle lives in tests/.
"""
import math

import torch

ATOL, RTOL = 4e-3, 4e-3
_CHUNK_ELEMS = 1 << 29            # cap on the fp32 score matrix of one chunk (2 GiB)


def _heads_per_chunk(sq, sk):
    return max(1, _CHUNK_ELEMS // max(1, sq * sk))


def _causal_keep(sq, sk, device):
    i = torch.arange(sq, device=device).unsqueeze(1)
    j = torch.arange(sk, device=device).unsqueeze(0)
    return j <= i + (sk - sq)


def _flat(t, last=2):
    """[B, H, ...] -> [B*H, ...] view."""
    return t.reshape(t.shape[0] * t.shape[1], *t.shape[2:])


def _chunks(n, step):
    return [(a, min(n, a + step)) for a in range(0, n, step)]


def attention_forward(q, k, v, scale, causal):
    qf, kf, vf = _flat(q), _flat(k), _flat(v)
    sq, sk = q.shape[2], k.shape[2]
    out = torch.empty(qf.shape[0], sq, v.shape[-1], dtype=torch.float32, device=q.device)
    keep = _causal_keep(sq, sk, q.device) if causal else None
    for a, b in _chunks(qf.shape[0], _heads_per_chunk(sq, sk)):
        s = torch.matmul(qf[a:b].float(), kf[a:b].float().transpose(-1, -2)) * scale
        if causal:
            s = s.masked_fill(~keep, float("-inf"))
        p = torch.nan_to_num(torch.softmax(s, dim=-1), nan=0.0)
        out[a:b] = torch.matmul(p, vf[a:b].float())
    return {3: out.view(*q.shape[:3], v.shape[-1])}


def attention_backward(q, k, v, o, do, lse, scale, causal):
    """Gradients for the o / lse as given (the tuner feeds synthetic ones)."""
    qf, kf, vf, of, gf, lf = _flat(q), _flat(k), _flat(v), _flat(o), _flat(do), _flat(lse)
    sq, sk = q.shape[2], k.shape[2]
    dq, dk, dv = (torch.empty(t.shape, dtype=torch.float32, device=q.device) for t in (qf, kf, vf))
    keep = _causal_keep(sq, sk, q.device) if causal else None
    for a, b in _chunks(qf.shape[0], max(1, _heads_per_chunk(sq, sk) // 2)):
        s = torch.matmul(qf[a:b].float(), kf[a:b].float().transpose(-1, -2)) * scale
        p = torch.exp(s - lf[a:b].unsqueeze(-1))
        if causal:
            p = p.masked_fill(~keep, 0.0)
        p = p.half().float()                              # the kernels round P and dS to fp16
        delta = (gf[a:b].float() * of[a:b].float()).sum(-1, keepdim=True)
        dv[a:b] = torch.matmul(p.transpose(-1, -2), gf[a:b].float())
        ds = (p * (torch.matmul(gf[a:b].float(), vf[a:b].float().transpose(-1, -2)) - delta)).half().float()
        dk[a:b] = torch.matmul(ds.transpose(-1, -2), qf[a:b].float()) * scale
        dq[a:b] = torch.matmul(ds, kf[a:b].float()) * scale
    return {6: dq.view(q.shape), 7: dk.view(k.shape), 8: dv.view(v.shape)}


def retnet_forward(q, k, v, mask):
    b, h = q.shape[:2]
    o = torch.empty(*q.shape[:3], v.shape[-1], dtype=torch.float32, device=q.device)
    r = torch.empty(*q.shape[:3], dtype=torch.float32, device=q.device)
    for i in range(b):
        s = torch.matmul(q[i].float(), k[i].float().transpose(-1, -2)) * mask.float()
        ri = s.abs().sum(-1, keepdim=True).clamp(min=1.0)
        o[i] = torch.matmul(s / ri, v[i].float())
        r[i] = ri.squeeze(-1)
    return {4: o, 5: r}


def retnet_backward(q, k, v, mask, do, r):
    dq, dk, dv = (torch.empty(t.shape, dtype=torch.float32, device=q.device) for t in (q, k, v))
    for i in range(q.shape[0]):
        ri = r[i].float().unsqueeze(-1)
        p = ((torch.matmul(q[i].float(), k[i].float().transpose(-1, -2)) * mask.float()) / ri).half().float()
        dv[i] = torch.matmul(p.transpose(-1, -2), do[i].float())
        ds = ((torch.matmul(do[i].float(), v[i].float().transpose(-1, -2)) / ri) * mask.float()).half().float()
        dk[i] = torch.matmul(ds.transpose(-1, -2), q[i].float())
        dq[i] = torch.matmul(ds, k[i].float())
    return {6: dq, 7: dk, 8: dv}


def decay_mask(lg2gamma, sq, sk):
    """[H, sq, sk] fp32: gamma_h^(i + sk - sq - j) on and below that diagonal, zero above it."""
    e = (torch.arange(sq, device=lg2gamma.device).view(1, sq, 1) + (sk - sq)
         - torch.arange(sk, device=lg2gamma.device).view(1, 1, sk)).float()
    d = torch.exp2(lg2gamma.float().view(-1, 1, 1) * e.clamp(min=0))
    return torch.where(e >= 0, d, torch.zeros((), device=d.device))


def reference_outputs(op, arrays, scale=None, causal=False, decay=False):
    """{index into ``arrays``: fp32 reference tensor} for the output tensors of operator ``op``."""
    if decay:                     # arrays[3] is log2(gamma); the backward's list has no dqaccum at the end
        arrays = list(arrays)
        arrays[3] = decay_mask(arrays[3], arrays[0].shape[2], arrays[1].shape[2])
    if op == "attn":
        q, k, v = arrays[:3]
        return attention_forward(q, k, v, scale if scale is not None else 1.0 / math.sqrt(q.shape[-1]), causal)
    if op == "attn_bwd":
        q, k, v, o, do, lse = arrays[:6]
        return attention_backward(q, k, v, o, do, lse, scale if scale is not None else 1.0 / math.sqrt(q.shape[-1]), causal)
    if op == "ret":
        return retnet_forward(*arrays[:4])
    if op == "ret_bwd":
        return retnet_backward(*arrays[:6])
    raise KeyError(op)


def outputs_match(arrays, reference):
    """True when every output tensor is within ``ATOL + RTOL * |ref|`` of its reference."""
    for idx, ref in reference.items():
        got = arrays[idx].float()
        if not torch.isfinite(got).all():
            return False
        if not bool(((got - ref).abs() <= ATOL + RTOL * ref.abs()).all()):
            return False
    return True
