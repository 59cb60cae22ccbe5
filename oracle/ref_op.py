"""fp32 restatement of the reference's torch math for attention and RetNet parallel retention.

TEST INFRASTRUCTURE ONLY -- the product path never imports this file.

Every function upcasts its (fp16) inputs to fp32 on the CPU and evaluates the closed form the
reference uses as its own correctness check:

* ``attention_ref``   follows reference python/utils/ref_op.py:2-6  (``softmax(q k^T * scale) v``); the
  reference hard-codes scale = 0.125, here it is an argument (``None`` -> 1/sqrt(d_qk)) and a causal
  lower-triangular mask (aligned to the bottom-right corner when S_q != S_kv) can be applied.
* ``attention_bwd_ref`` is the closed form of the attention gradients (the reference declares the
  operator, python/ops/attention_interface.py:37-58, and leaves it empty): with ``P = softmax(S)``,
  ``delta = rowsum(dO * O)``: ``dV = P^T dO``, ``dS = P * (dO V^T - delta)``, ``dK = scale dS^T Q``,
  ``dQ = scale dS K``; pinned by autograd through ``attention_ref`` and fp64 gradcheck.  With
  ``operand_dtype=torch.float16`` P and dS are rounded before the contraction that consumes them, as the kernels
  do; ``attention_bwd_rounding_bound`` is the worst case that rounding can move each gradient entry by.
* ``retnet_ref``      follows reference python/utils/ref_op.py:8-13 (``S = q k^T * mask``,
  ``r = clamp(sum|S|, min=1)`` detached, ``o = (S / r) v``) and also returns ``r``.
* ``retnet_bwd_ref``  is the closed form the backward kernel evaluates, reference
  csrc/kernels/retnet/bwd/bwd_colblock.h:522-576: with r constant, ``P = S / r``,
  ``dV = P^T dO``, ``dS = (dO V^T / r) * mask``, ``dK = dS^T Q``, ``dQ = dS K``; with
  ``operand_dtype=torch.float16`` P and dS are rounded where the reference kernel rounds them (:509, :551);
  ``retnet_bwd_rounding_bound`` is the worst case that rounding can move each gradient entry by.
* ``retnet_decay_mask`` is the decay matrix of the benchmark configuration:
  ``D[h, n, m] = gamma_h^(n-m)`` for n >= m else 0, ``gamma_h = 1 - 2^(-5-h)``.
* ``retnet_recurrent_ref`` is the closed form of the recurrent scan of reference
  csrc/kernels/retnet/recurrent/recurrent.h:110-114,303-330 (``S_n = a_n S_{n-1} + k_n^T v_n``,
  ``out_n = q_n S_n`` over the first ``block_kdim`` key dims, fp32 tensors laid out [B, H, dim, L]):
  ``out = V (K^T Q * D)`` with ``D[m, n] = prod_{m<j<=n} a_j`` for m <= n, else 0, in fp64.  The products
  are taken literally (no logarithms), so zero and negative decays mean what they mean in the scan.
* ``attention_online_ref`` / ``retnet_online_ref`` restate the tile-by-tile recurrences sketched in
  reference README.md:81-99 and python/tests/attntuner_demo.py:59-97,122-161; they exist so a test
  can show the online form equals the one-shot form.

Pinned by tests/test_oracle.py against torch's scaled_dot_product_attention, fp64 brute force
(oracle/brute.c), closed-form special cases, autograd and gradcheck.  No function here is
"parity unpinned".
"""
import math

import torch

REFERENCE_SOFTMAX_SCALE = 0.125  # reference python/utils/ref_op.py:3


def _f32(x):
    return x.detach().to(device="cpu", dtype=torch.float32)


def causal_allowed(seq_q, seq_k):
    """Boolean [seq_q, seq_k]: query i sees kv j iff j <= i + (seq_k - seq_q)."""
    i = torch.arange(seq_q).unsqueeze(1)
    j = torch.arange(seq_k).unsqueeze(0)
    return j <= i + (seq_k - seq_q)


def attention_ref(q, k, v, softmax_scale=None, causal=False, return_lse=False):
    q, k, v = _f32(q), _f32(k), _f32(v)
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(q.shape[-1])
    s = (q @ k.transpose(-1, -2)) * softmax_scale
    if causal:
        s = s.masked_fill(~causal_allowed(q.shape[-2], k.shape[-2]), float("-inf"))
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse.unsqueeze(-1))
    p = torch.nan_to_num(p, nan=0.0)  # rows with no visible kv produce 0, not NaN
    o = p @ v
    return (o, lse) if return_lse else o


def _attention_bwd_parts(q, k, v, do, softmax_scale, causal, o, lse, operand_dtype=None):
    q, k, v, do = _f32(q), _f32(k), _f32(v), _f32(do)
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(q.shape[-1])
    s = (q @ k.transpose(-1, -2)) * softmax_scale
    if causal:
        s = s.masked_fill(~causal_allowed(q.shape[-2], k.shape[-2]), float("-inf"))
    lse = torch.logsumexp(s, dim=-1) if lse is None else _f32(lse)
    p = torch.nan_to_num(torch.exp(s - lse.unsqueeze(-1)), nan=0.0, posinf=0.0)
    o = p @ v if o is None else _f32(o)
    if operand_dtype is not None:
        o = o.to(operand_dtype).float()                     # delta is taken from the output as the forward stored it
    delta = (do * o).sum(dim=-1, keepdim=True)
    ds = p * (do @ v.transpose(-1, -2) - delta)
    return q, k, v, do, softmax_scale, p, ds, o


def attention_bwd_ref(q, k, v, do, softmax_scale=None, causal=False, o=None, lse=None, operand_dtype=None):
    """Gradients of ``attention_ref`` w.r.t. q, k, v.  ``o`` / ``lse`` (as a forward kernel stored them) are
    used for delta and P when given, otherwise recomputed.  ``operand_dtype=torch.float16`` restates the
    kernels' arithmetic: delta from the fp16 output, P and dS rounded before the contraction that consumes
    them (the roundings of the reference's RetNet backward, csrc/kernels/retnet/bwd/bwd_colblock.h:509,551;
    the reference has no attention backward)."""
    q, k, v, do, softmax_scale, p, ds, _ = _attention_bwd_parts(q, k, v, do, softmax_scale, causal, o, lse, operand_dtype)
    if operand_dtype is not None:
        p, ds = p.to(operand_dtype).float(), ds.to(operand_dtype).float()
    dv = p.transpose(-1, -2) @ do
    dk = (ds.transpose(-1, -2) @ q) * softmax_scale
    dq = (ds @ k) * softmax_scale
    return dq, dk, dv


def attention_bwd_rounding_bound(q, k, v, do, softmax_scale=None, causal=False, o_stored=None):
    """Per-entry sums of term magnitudes for dq, dk, dv: the fp16 roundings of the kernels' arithmetic (P, dS,
    and the output that delta is taken from) move a gradient entry by at most 2^-11 times its sum.  An error e_i
    in delta_i moves every dS_ij of the row by P_ij e_i; with the exact output rounded to fp16 e_i is at most
    2^-11 sum_d |dO_id O_id|, with ``o_stored`` (the output a forward kernel actually wrote) it is the actual
    difference |sum_d dO_id (o_stored - O)_id|, entered here divided by 2^-11."""
    q, k, v, do, softmax_scale, p, ds, o = _attention_bwd_parts(q, k, v, do, softmax_scale, causal, None, None)
    p = p.abs()
    if o_stored is None:
        delta_dev = (do * o).abs().sum(dim=-1, keepdim=True)
    else:
        delta_dev = (do * (_f32(o_stored) - o)).sum(dim=-1, keepdim=True).abs() * 2.0 ** 11
    ds = ds.abs() + p * delta_dev
    return (ds @ k.abs()) * softmax_scale, (ds.transpose(-1, -2) @ q.abs()) * softmax_scale, p.transpose(-1, -2) @ do.abs()


def retnet_ref(q, k, v, mask, return_r=False):
    q, k, v, mask = _f32(q), _f32(k), _f32(v), _f32(mask)
    s = (q @ k.transpose(-1, -2)) * mask
    r = s.abs().sum(dim=-1, keepdim=True).clamp(min=1.0)
    o = (s / r) @ v
    return (o, r.squeeze(-1)) if return_r else o


def retnet_bwd_ref(q, k, v, mask, do, r=None, operand_dtype=None):
    """Gradients of ``retnet_ref`` w.r.t. q, k, v with r treated as a constant.

    ``operand_dtype=torch.float16`` restates the reference kernel's arithmetic instead of the exact closed
    form: P and dS are rounded to fp16 before the contraction that consumes them (reference
    csrc/kernels/retnet/bwd/bwd_colblock.h:509 and :551), everything else stays fp32.  The two differ by at
    most 2^-11 * sum_j |term_j| per gradient entry (tests/test_oracle.py pins that bound)."""
    q, k, v, mask, do = _f32(q), _f32(k), _f32(v), _f32(mask), _f32(do)
    s = (q @ k.transpose(-1, -2)) * mask
    if r is None:
        r = s.abs().sum(dim=-1).clamp(min=1.0)
    r = _f32(r).unsqueeze(-1)
    p = s / r
    ds = ((do @ v.transpose(-1, -2)) / r) * mask
    if operand_dtype is not None:
        p, ds = p.to(operand_dtype).float(), ds.to(operand_dtype).float()
    dv = p.transpose(-1, -2) @ do
    dk = ds.transpose(-1, -2) @ q
    dq = ds @ k
    return dq, dk, dv


def retnet_bwd_rounding_bound(q, k, v, mask, do, r=None):
    """Per-entry bound on |rounded-operand form - exact form| of ``retnet_bwd_ref``: rounding P or dS to fp16
    moves each entry by at most 2^-11 of its magnitude, so a gradient entry moves by at most
    2^-11 * sum_j |operand_j| |other factor_j|.  Returns that sum (without the 2^-11) for dq, dk, dv."""
    q, k, v, mask, do = _f32(q), _f32(k), _f32(v), _f32(mask), _f32(do)
    s = (q @ k.transpose(-1, -2)) * mask
    if r is None:
        r = s.abs().sum(dim=-1).clamp(min=1.0)
    r = _f32(r).unsqueeze(-1)
    p = (s / r).abs()
    ds = (((do @ v.transpose(-1, -2)) / r) * mask).abs()
    return ds @ k.abs(), ds.transpose(-1, -2) @ q.abs(), p.transpose(-1, -2) @ do.abs()


def retnet_decay_mask(nheads, seq_q, seq_k, dtype=torch.float16):
    n = torch.arange(seq_q, dtype=torch.float64).view(1, seq_q, 1)
    m = torch.arange(seq_k, dtype=torch.float64).view(1, 1, seq_k)
    gamma = 1.0 - torch.pow(2.0, -5.0 - torch.arange(nheads, dtype=torch.float64)).view(nheads, 1, 1)
    d = torch.where(n >= m, gamma ** (n - m).clamp(min=0), torch.zeros((), dtype=torch.float64))
    return d.to(dtype) if dtype == torch.float64 else d.to(torch.float32).to(dtype)


def retnet_recurrent_decay_matrix(decay):
    """decay [H, L] -> D [H, L(m), L(n)] fp64, D[h, m, n] = prod_{m<j<=n} decay[h, j] for m <= n, 0 below."""
    a = decay.detach().to(device="cpu", dtype=torch.float64)
    nheads, seqlen = a.shape
    d = torch.zeros(nheads, seqlen, seqlen, dtype=torch.float64)
    for m in range(seqlen):
        d[:, m, m] = 1.0
        if m + 1 < seqlen:
            d[:, m, m + 1:] = torch.cumprod(a[:, m + 1:], dim=-1)
    return d


def retnet_recurrent_ref(q, k, v, decay, block_kdim=None):
    """q, k [B, H, kdim, L], v [B, H, vdim, L], decay [H, L] -> out [B, H, vdim, L] (fp64 math, fp32 result)."""
    q, k, v = (x.detach().to(device="cpu", dtype=torch.float64) for x in (q, k, v))
    kd = block_kdim or q.shape[2]
    s = k[:, :, :kd].transpose(-1, -2) @ q[:, :, :kd]            # [B, H, L(m), L(n)]
    p = s * retnet_recurrent_decay_matrix(decay).unsqueeze(0)
    return (v @ p).to(torch.float32)


def attention_online_ref(q, k, v, softmax_scale=None, causal=False, block_kv=64):
    """Tile-by-tile recurrence with an unscaled running max, as the kernels evaluate it."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(q.shape[-1])
    sq, sk = q.shape[-2], k.shape[-2]
    allowed = causal_allowed(sq, sk) if causal else None
    m = torch.full(q.shape[:-1], float("-inf"))
    l = torch.zeros(q.shape[:-1])
    o = torch.zeros(*q.shape[:-1], v.shape[-1])
    for j0 in range(0, sk, block_kv):
        s = q @ k[..., j0:j0 + block_kv, :].transpose(-1, -2)
        if causal:
            s = s.masked_fill(~allowed[:, j0:j0 + block_kv], float("-inf"))
        m_new = torch.maximum(m, s.amax(dim=-1))
        m_use = torch.where(torch.isinf(m_new), torch.zeros_like(m_new), m_new)
        alpha = torch.exp((m - m_use) * softmax_scale)
        p = torch.exp((s - m_use.unsqueeze(-1)) * softmax_scale)
        l = l * alpha + p.sum(dim=-1)
        o = o * alpha.unsqueeze(-1) + p.half().float() @ v[..., j0:j0 + block_kv, :]
        m = m_new
    return o / l.unsqueeze(-1)


def retnet_online_ref(q, k, v, mask, block_kv=64):
    """Running abs-sum recurrence: R += sum|S|, r = max(R, 1), O = O r_old/r_new + half(S/r_new) V."""
    q, k, v, mask = _f32(q), _f32(k), _f32(v), _f32(mask)
    sk = k.shape[-2]
    big_r = torch.zeros(q.shape[:-1])
    r_old = torch.ones(q.shape[:-1])
    o = torch.zeros(*q.shape[:-1], v.shape[-1])
    for j0 in range(0, sk, block_kv):
        s = (q @ k[..., j0:j0 + block_kv, :].transpose(-1, -2)) * mask[..., j0:j0 + block_kv]
        big_r = big_r + s.abs().sum(dim=-1)
        r_new = big_r.clamp(min=1.0)
        o = o * (r_old / r_new).unsqueeze(-1) + (s / r_new.unsqueeze(-1)).half().float() @ v[..., j0:j0 + block_kv, :]
        r_old = r_new
    return o, r_old


def attention_split_merge_ref(q, k, v, softmax_scale=None, n_splits=2):
    """Split the kv range, run each part independently, merge with the log-sum-exp weights."""
    sk = k.shape[-2]
    step = sk // n_splits
    outs, lses = [], []
    for i in range(n_splits):
        o_i, lse_i = attention_ref(q, k[..., i * step:(i + 1) * step, :], v[..., i * step:(i + 1) * step, :],
                                   softmax_scale, False, return_lse=True)
        outs.append(o_i)
        lses.append(lse_i)
    lse = torch.logsumexp(torch.stack(lses), dim=0)
    o = sum(o_i * torch.exp(l_i - lse).unsqueeze(-1) for o_i, l_i in zip(outs, lses))
    return o
