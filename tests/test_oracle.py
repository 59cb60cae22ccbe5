"""Pins oracle/ref_op.py: library routines, fp64 brute force, closed forms, autograd, gradcheck.

Each check is chosen so that a plausible slip in the restatement (dropped scale, mask applied after
the abs-sum, missing clamp, transposed operand, r not detached) fails at least one of them.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import brute, ref_op


def _rand(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).half()


# ---------------------------------------------------------------------------------- attention
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("sq,sk", [(32, 32), (16, 48)])
def test_attention_matches_torch_sdpa(causal, sq, sk):
    if causal and sq != sk:
        pytest.skip("torch's is_causal aligns top-left; bottom-right alignment is checked by brute force")
    q, k, v = _rand(2, 3, sq, 64, seed=1), _rand(2, 3, sk, 64, seed=2), _rand(2, 3, sk, 128, seed=3)
    for scale in (0.125, 1 / math.sqrt(64), 0.3):
        want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), scale=scale, is_causal=causal)
        got = ref_op.attention_ref(q, k, v, softmax_scale=scale, causal=causal)
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("sq,sk", [(8, 8), (4, 12), (12, 4)])
def test_attention_matches_fp64_brute_force(causal, sq, sk):
    q, k, v = _rand(1, 2, sq, 64, seed=4), _rand(1, 2, sk, 64, seed=5), _rand(1, 2, sk, 64, seed=6)
    want = brute.attention_fwd(q.float().numpy(), k.float().numpy(), v.float().numpy(), 0.2, causal)
    got = ref_op.attention_ref(q, k, v, softmax_scale=0.2, causal=causal).numpy()
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-5)


def test_attention_closed_forms():
    q, k, v = _rand(1, 2, 16, 64, seed=7), _rand(1, 2, 16, 64, seed=8), _rand(1, 2, 16, 64, seed=9)
    ones = torch.ones_like(v)
    torch.testing.assert_close(ref_op.attention_ref(q, k, ones), ones.float())                      # rows of P sum to 1
    mean_v = v.float().mean(dim=-2, keepdim=True).expand(-1, -1, 16, -1)
    torch.testing.assert_close(ref_op.attention_ref(q, k, v, softmax_scale=0.0), mean_v)            # scale 0 -> mean
    same_k = k[..., :1, :].expand_as(k)
    torch.testing.assert_close(ref_op.attention_ref(q, same_k, v), mean_v, rtol=1e-5, atol=1e-5)    # identical keys -> mean
    prefix = torch.cumsum(v.float(), dim=-2) / torch.arange(1, 17).view(1, 1, 16, 1)
    torch.testing.assert_close(ref_op.attention_ref(q, k, v, softmax_scale=0.0, causal=True), prefix)
    torch.testing.assert_close(ref_op.attention_ref(q, k, v, causal=True)[..., 0, :], v.float()[..., 0, :])
    perm = torch.randperm(16, generator=torch.Generator().manual_seed(0))                           # kv order is irrelevant
    torch.testing.assert_close(ref_op.attention_ref(q, k[..., perm, :], v[..., perm, :]), ref_op.attention_ref(q, k, v))
    eye = torch.eye(16).expand(1, 2, 16, 16).half()                                                 # one-hot V returns P
    p = ref_op.attention_ref(q, k, eye, softmax_scale=0.125)
    want = torch.softmax(q.float() @ k.float().transpose(-1, -2) * 0.125, dim=-1)
    torch.testing.assert_close(p, want)
    assert ref_op.REFERENCE_SOFTMAX_SCALE == 0.125
    torch.testing.assert_close(ref_op.attention_ref(q, k, v), ref_op.attention_ref(q, k, v, softmax_scale=0.125))  # d=64


@pytest.mark.parametrize("causal", [False, True])
def test_attention_online_and_split_forms_agree(causal):
    q, k, v = _rand(1, 2, 64, 64, seed=10), _rand(1, 2, 128, 64, seed=11), _rand(1, 2, 128, 64, seed=12)
    full = ref_op.attention_ref(q, k, v, causal=causal)
    online = ref_op.attention_online_ref(q, k, v, causal=causal, block_kv=32)
    assert (full - online).abs().max() < 2e-3       # only P's fp16 rounding separates them
    if not causal:
        torch.testing.assert_close(ref_op.attention_split_merge_ref(q, k, v, n_splits=4), full, rtol=1e-5, atol=1e-5)


def test_attention_lse():
    q, k, v = _rand(1, 1, 8, 64, seed=13), _rand(1, 1, 8, 64, seed=14), _rand(1, 1, 8, 64, seed=15)
    _, lse = ref_op.attention_ref(q, k, v, softmax_scale=0.125, return_lse=True)
    want = torch.log(torch.exp(q.float() @ k.float().transpose(-1, -2) * 0.125).sum(-1))
    torch.testing.assert_close(lse, want)


# ---------------------------------------------------------------------------------- RetNet forward
def test_decay_mask_closed_form():
    m = ref_op.retnet_decay_mask(3, 8, 8, dtype=torch.float32)
    for h in range(3):
        g = 1 - 2.0 ** (-5 - h)
        for n in range(8):
            for j in range(8):
                want = g ** (n - j) if n >= j else 0.0
                assert abs(m[h, n, j].item() - want) < 1e-6
    m16 = ref_op.retnet_decay_mask(2, 2048, 2048)
    assert m16.dtype == torch.float16 and m16[0, 2047, 0] == 0 and m16[0, 5, 5] == 1       # fp16 underflow far from the diagonal


def test_retnet_matches_fp64_brute_force():
    q, k, v = _rand(2, 2, 8, 64, seed=20), _rand(2, 2, 12, 64, seed=21), _rand(2, 2, 12, 128, seed=22)
    mask = _rand(2, 8, 12, seed=23)
    o, r = ref_op.retnet_ref(q, k, v, mask, return_r=True)
    bo, br = brute.retnet_fwd(q.float().numpy(), k.float().numpy(), v.float().numpy(), mask.float().numpy())
    np.testing.assert_allclose(o.numpy(), bo, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(r.numpy(), br, rtol=2e-5, atol=2e-5)


def test_retnet_closed_forms():
    q, k, v = _rand(1, 2, 16, 64, seed=24), _rand(1, 2, 16, 64, seed=25), _rand(1, 2, 16, 64, seed=26)
    zero = torch.zeros(2, 16, 16).half()
    o, r = ref_op.retnet_ref(q, k, v, zero, return_r=True)
    assert o.abs().max() == 0 and (r == 1).all()                                       # M = 0
    tiny_q = (q.float() * 1e-3).half()
    ones = torch.ones(2, 16, 16).half()
    o, r = ref_op.retnet_ref(tiny_q, k, v, ones, return_r=True)
    assert (r == 1).all()                                                              # clamp active -> plain matmuls
    torch.testing.assert_close(o, (tiny_q.float() @ k.float().transpose(-1, -2)) @ v.float())
    mask = ref_op.retnet_decay_mask(2, 16, 16)
    o1, r1 = ref_op.retnet_ref(q, k, v, mask, return_r=True)
    assert (r1 > 1).all()
    o2 = ref_op.retnet_ref((q.float() * 2).half(), k, v, mask)                          # r > 1: scale invariance in q
    torch.testing.assert_close(o1, o2, rtol=1e-5, atol=1e-5)
    s = (q.float() @ k.float().transpose(-1, -2)) * mask.float()
    torch.testing.assert_close(r1, s.abs().sum(-1).clamp(min=1.0))
    torch.testing.assert_close((s / r1.unsqueeze(-1)).abs().sum(-1), torch.ones_like(r1))
    # numerator equals the recurrent form  S_n = gamma S_{n-1} + k_n^T v_n,  num_n = q_n S_n
    # (unrounded decay mask here: the recurrence uses the exact gamma)
    s = (q.double() @ k.double().transpose(-1, -2)) * ref_op.retnet_decay_mask(2, 16, 16, dtype=torch.float64)
    for h in range(2):
        g = 1 - 2.0 ** (-5 - h)
        state = torch.zeros(64, 64, dtype=torch.float64)
        for n in range(16):
            state = g * state + k[0, h, n].double().unsqueeze(1) * v[0, h, n].double().unsqueeze(0)
            num = q[0, h, n].double() @ state
            want = (s[0, h, n].double() @ v[0, h].double())
            torch.testing.assert_close(num, want, rtol=1e-6, atol=1e-6)


def test_retnet_online_form_agrees():
    q, k, v = _rand(1, 2, 32, 64, seed=27), _rand(1, 2, 128, 64, seed=28), _rand(1, 2, 128, 64, seed=29)
    mask = _rand(2, 32, 128, seed=30, scale=0.5)
    o, r = ref_op.retnet_ref(q, k, v, mask, return_r=True)
    oo, ro = ref_op.retnet_online_ref(q, k, v, mask, block_kv=32)
    torch.testing.assert_close(ro, r, rtol=1e-5, atol=1e-5)
    assert (o - oo).abs().max() < 2e-3


# ---------------------------------------------------------------------------------- RetNet backward
def _autograd_grads(q, k, v, mask, do, dtype=torch.float32):
    qq, kk, vv = (t.detach().to(dtype).requires_grad_(True) for t in (q, k, v))
    s = (qq @ kk.transpose(-1, -2)) * mask.to(dtype)
    r = s.detach().abs().sum(dim=-1, keepdim=True).clamp(min=1.0)
    o = (s / r) @ vv
    o.backward(do.to(dtype))
    return qq.grad, kk.grad, vv.grad


def test_retnet_bwd_matches_autograd_and_brute_force():
    q, k, v = _rand(2, 2, 8, 64, seed=31), _rand(2, 2, 12, 64, seed=32), _rand(2, 2, 12, 128, seed=33)
    mask, do = _rand(2, 8, 12, seed=34), _rand(2, 2, 8, 128, seed=35)
    got = ref_op.retnet_bwd_ref(q, k, v, mask, do)
    want = _autograd_grads(q, k, v, mask, do)
    for g, w in zip(got, want):
        torch.testing.assert_close(g, w, rtol=1e-4, atol=1e-4)
    b = brute.retnet_bwd(*(t.float().numpy() for t in (q, k, v, mask, do)))
    for g, w in zip(got, b):
        np.testing.assert_allclose(g.numpy(), w, rtol=1e-4, atol=1e-4)


def test_retnet_bwd_gradcheck_fp64():
    g = torch.Generator().manual_seed(36)
    q, k, v = (torch.randn(1, 1, 4, 6, generator=g, dtype=torch.float64) for _ in range(3))
    mask = torch.randn(1, 4, 4, generator=g, dtype=torch.float64)
    do = torch.randn(1, 1, 4, 6, generator=g, dtype=torch.float64)
    r = ((q @ k.transpose(-1, -2)) * mask).abs().sum(-1, keepdim=True).clamp(min=1.0)

    def f(qq, kk, vv):                         # r frozen, as the reference detaches it
        return (((qq @ kk.transpose(-1, -2)) * mask) / r) @ vv

    assert torch.autograd.gradcheck(f, tuple(t.clone().requires_grad_(True) for t in (q, k, v)), eps=1e-6, atol=1e-6)
    want = torch.autograd.grad(f(*(t.requires_grad_(True) for t in (q, k, v))), (q, k, v), do)
    got = ref_op.retnet_bwd_ref(q, k, v, mask, do)
    for a, b in zip(got, want):
        torch.testing.assert_close(a, b.float(), rtol=1e-4, atol=1e-4)


def test_retnet_bwd_linearity_and_zero_mask():
    q, k, v = _rand(1, 2, 8, 64, seed=37), _rand(1, 2, 8, 64, seed=38), _rand(1, 2, 8, 64, seed=39)
    mask = _rand(2, 8, 8, seed=40)
    d1, d2 = _rand(1, 2, 8, 64, seed=41), _rand(1, 2, 8, 64, seed=42)
    g1 = ref_op.retnet_bwd_ref(q, k, v, mask, d1.float())
    g2 = ref_op.retnet_bwd_ref(q, k, v, mask, d2.float())
    g12 = ref_op.retnet_bwd_ref(q, k, v, mask, 2 * d1.float() - 3 * d2.float())
    for a, b, c in zip(g1, g2, g12):
        torch.testing.assert_close(2 * a - 3 * b, c, rtol=1e-4, atol=1e-4)
    for g in ref_op.retnet_bwd_ref(q, k, v, torch.zeros_like(mask), d1):
        assert g.abs().max() == 0


def test_retnet_bwd_rounded_operands_stay_within_the_rounding_bound():
    """The variant that rounds P and dS to fp16 where the reference kernel does differs from the exact closed
    form by at most half an fp16 ulp per rounded entry: |delta| <= 2^-11 * sum_j |operand_j| |other_j|, and it is
    the exact form again once P and dS are representable (a one-hot mask row with power-of-two data)."""
    q, k, v = _rand(1, 2, 16, 64, seed=43), _rand(1, 2, 16, 64, seed=44), _rand(1, 2, 16, 128, seed=45)
    mask, do = ref_op.retnet_decay_mask(2, 16, 16), _rand(1, 2, 16, 128, seed=46)
    exact = ref_op.retnet_bwd_ref(q, k, v, mask, do)
    rounded = ref_op.retnet_bwd_ref(q, k, v, mask, do, operand_dtype=torch.float16)
    bounds = ref_op.retnet_bwd_rounding_bound(q, k, v, mask, do)
    differs = False
    for e, g, b in zip(exact, rounded, bounds):
        assert ((e - g).abs() <= 2.0 ** -11 * b * 1.001 + 1e-7).all()
        differs |= bool((e != g).any())
    assert differs                                      # the rounding is really applied
    eye = torch.eye(16).expand(2, 16, 16)                # P = +-1 and dS = (dO v) / |q k| on the diagonal only
    q2 = torch.zeros(1, 2, 16, 64); q2[..., 0] = 2.0
    k2 = torch.zeros(1, 2, 16, 64); k2[..., 0] = 4.0    # S_ii = 8, r = 8
    v2 = torch.zeros(1, 2, 16, 128); v2[..., 1] = 0.5
    d2 = torch.zeros(1, 2, 16, 128); d2[..., 1] = 16.0  # dO v = 8 -> dS = 1
    for e, g in zip(ref_op.retnet_bwd_ref(q2, k2, v2, eye, d2),
                    ref_op.retnet_bwd_ref(q2, k2, v2, eye, d2, operand_dtype=torch.float16)):
        assert torch.equal(e, g)
    dq, dk, dv = ref_op.retnet_bwd_ref(q2, k2, v2, eye, d2, operand_dtype=torch.float16)
    assert dq[0, 0, 3, 0] == 4.0 and dk[0, 0, 3, 0] == 2.0 and dv[0, 0, 3, 1] == 16.0


def test_attention_bwd_rounded_operands_stay_within_the_rounding_bound():
    q, k, v, do = _rand(1, 2, 24, 64, seed=61), _rand(1, 2, 40, 64, seed=62), _rand(1, 2, 40, 128, seed=63), _rand(1, 2, 24, 128, seed=64)
    for causal in (False, True):
        exact = ref_op.attention_bwd_ref(q, k, v, do, 0.2, causal)
        rounded = ref_op.attention_bwd_ref(q, k, v, do, 0.2, causal, operand_dtype=torch.float16)
        bounds = ref_op.attention_bwd_rounding_bound(q, k, v, do, 0.2, causal)
        stored = ref_op.attention_ref(q, k, v, 0.2, causal).half()           # the same bound from the actual difference in delta
        tight = ref_op.attention_bwd_rounding_bound(q, k, v, do, 0.2, causal, o_stored=stored)
        assert all((t <= b * 1.001 + 1e-6).all() for t, b in zip(tight, bounds))
        differs = False
        for e, g, b in zip(exact, rounded, bounds):
            assert ((e - g).abs() <= 2.0 ** -11 * b * 1.001 + 1e-7).all()
            differs |= bool((e != g).any())
        assert differs
    # one visible key per query: P = 1 exactly, so dV = dO; dS = dO.v - dO.o vanishes up to the rounding of o
    one = [t[..., :1, :] for t in (q, k, v, do)]
    dq, dk, dv = ref_op.attention_bwd_ref(*one, 0.2, True)
    assert torch.equal(dv, one[3].float()) and dq.abs().max() <= 1e-5 and dk.abs().max() <= 1e-5
    dq16, _, dv16 = ref_op.attention_bwd_ref(*one, 0.2, True, operand_dtype=torch.float16)
    assert torch.equal(dv16, one[3].float()) and dq16.abs().max() <= 2.0 ** -11 * (one[3].float().abs() * one[2].float().abs()).sum() * 0.2 * one[1].abs().max() * 1.01


# ------------------------------------------------------------------------------------ the parity bound
def test_tolerance_rule_accepts_and_rejects_what_it_says():
    from oracle import tolerance
    ref = torch.tensor([0.5, 1.5, 3.0, 5.0, 100.0])
    assert torch.equal(tolerance.fp16_ulp(ref), torch.tensor([2.0 ** -11, 2.0 ** -10, 2.0 ** -9, 2.0 ** -8, 2.0 ** -4]))
    ok, small, large, n = tolerance.check(ref + torch.tensor([1.9e-3, -1.9e-3, 1.9e-3, 3.9e-3, -0.06]), ref)
    assert ok and n == 2 and abs(small - 1.9e-3) < 1e-6 and 0.9 < large <= 1.0
    assert not tolerance.check(ref + torch.tensor([0.0, 0.0, 2.1e-3, 0.0, 0.0]), ref)[0]          # 2e-3 is literal below 4
    assert not tolerance.check(ref + torch.tensor([0.0, 0.0, 0.0, 4.0e-3, 0.0]), ref)[0]          # one ulp at 5 is 3.9e-3
    assert not tolerance.check(ref + torch.tensor([0.0, 0.0, 0.0, 0.0, 0.07]), ref)[0]
    assert not tolerance.check(torch.tensor([float("nan")]), torch.tensor([0.0]))[0]
    # the rounded-operand rule: half an ulp of the result plus 2^-11 of the given sum of term magnitudes
    terms = torch.tensor([1.0, 2.0, 4.0, 8.0, 100.0])
    edge = 0.5 * tolerance.fp16_ulp(ref) + 2.0 ** -11 * terms
    assert tolerance.check_rounded_operand(ref + edge, ref, terms)[0]
    for i in range(5):
        bad = ref.clone()
        bad[i] -= 1.1 * edge[i] + 1e-4
        assert not tolerance.check_rounded_operand(bad, ref, terms)[0]
    with pytest.raises(AssertionError):
        tolerance.assert_close(ref + 0.01, ref, "rejects")


# ---------------------------------------------------------------------------------- attention backward
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("sq,sk", [(8, 8), (6, 10)])
def test_attention_bwd_matches_autograd_through_sdpa(causal, sq, sk):
    """Independent route: autograd through torch's own scaled_dot_product_attention in fp64."""
    q, k, v = _rand(2, 2, sq, 64, seed=51), _rand(2, 2, sk, 64, seed=52), _rand(2, 2, sk, 128, seed=53)
    do = _rand(2, 2, sq, 128, seed=54)
    scale = 0.2
    qq, kk, vv = (t.double().clone().requires_grad_(True) for t in (q, k, v))
    allowed = ref_op.causal_allowed(sq, sk) if causal else None
    out = F.scaled_dot_product_attention(qq, kk, vv, attn_mask=allowed, scale=scale)
    out.backward(do.double())
    got = ref_op.attention_bwd_ref(q, k, v, do, scale, causal)
    for g, w in zip(got, (qq.grad, kk.grad, vv.grad)):
        torch.testing.assert_close(g, w.float(), rtol=1e-4, atol=1e-4)


def test_attention_bwd_gradcheck_fp64_and_stored_forward():
    g = torch.Generator().manual_seed(55)
    q, k, v = (torch.randn(1, 1, 4, 6, generator=g, dtype=torch.float64) for _ in range(3))
    do = torch.randn(1, 1, 4, 6, generator=g, dtype=torch.float64)

    def f(qq, kk, vv):
        return torch.softmax((qq @ kk.transpose(-1, -2)) * 0.3, dim=-1) @ vv

    assert torch.autograd.gradcheck(f, tuple(t.clone().requires_grad_(True) for t in (q, k, v)), eps=1e-6, atol=1e-6)
    want = torch.autograd.grad(f(*(t.requires_grad_(True) for t in (q, k, v))), (q, k, v), do)
    got = ref_op.attention_bwd_ref(q, k, v, do, 0.3)
    for a, b in zip(got, want):
        torch.testing.assert_close(a, b.float(), rtol=1e-4, atol=1e-4)
    # the o / lse a forward kernel stored reproduce the same gradients as the recomputed ones
    o, lse = ref_op.attention_ref(q, k, v, 0.3, return_lse=True)
    again = ref_op.attention_bwd_ref(q, k, v, do, 0.3, o=o, lse=lse)
    for a, b in zip(got, again):
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-5)


def test_attention_bwd_closed_forms():
    q, k, v = _rand(1, 2, 8, 64, seed=56), _rand(1, 2, 8, 64, seed=57), _rand(1, 2, 8, 64, seed=58)
    d1, d2 = _rand(1, 2, 8, 64, seed=59), _rand(1, 2, 8, 64, seed=60)
    # linear in dO
    g1, g2 = ref_op.attention_bwd_ref(q, k, v, d1.float()), ref_op.attention_bwd_ref(q, k, v, d2.float())
    g12 = ref_op.attention_bwd_ref(q, k, v, 2 * d1.float() - 3 * d2.float())
    for a, b, c in zip(g1, g2, g12):
        torch.testing.assert_close(2 * a - 3 * b, c, rtol=1e-4, atol=1e-4)
    # scale 0: P is uniform, so dQ = dK = 0 and every dV row is the mean of dO
    dq, dk, dv = ref_op.attention_bwd_ref(q, k, v, d1, 0.0)
    assert dq.abs().max() == 0 and dk.abs().max() == 0
    torch.testing.assert_close(dv, d1.float().mean(dim=-2, keepdim=True).expand_as(dv), rtol=1e-5, atol=1e-5)
    # softmax rows sum to one, so dS rows sum to zero: a shift of every key by one vector leaves dQ's
    # projection on that vector unchanged -> sum over kv of dS is 0  <=>  dQ computed with K := 1 vanishes
    dq1, _, _ = ref_op.attention_bwd_ref(q, torch.ones_like(k), v, d1)
    assert dq1.abs().max() < 1e-5
    # causal, first query row sees one key: P = 1 there, so dS = P (dP - delta) = 0 and dQ[0] = 0
    dqc, _, dvc = ref_op.attention_bwd_ref(q, k, v, d1, None, True)
    assert dqc[..., 0, :].abs().max() < 1e-6


# ---------------------------------------------------------------------------------------------------
# RetNet recurrent form: two independent statements (a sequential fp64 recurrence in C, the parallel
# closed form in torch) pinned against each other and against what the mathematics fixes.
def _recurrent_inputs(seed, b=2, h=3, kdim=8, vdim=5, seqlen=37, lo=-1.0, hi=1.0):
    g = torch.Generator().manual_seed(seed)
    q = torch.rand(b, h, kdim, seqlen, generator=g) * 2 - 1
    k = torch.rand(b, h, kdim, seqlen, generator=g) * 2 - 1
    v = torch.rand(b, h, vdim, seqlen, generator=g) * 2 - 1
    decay = torch.rand(h, seqlen, generator=g) * (hi - lo) + lo
    return q, k, v, decay


def test_recurrent_closed_form_matches_the_sequential_recurrence():
    q, k, v, decay = _recurrent_inputs(0)
    decay[0, 5] = 0.0                      # a zero cuts the history, negative values flip signs
    decay[1, 9] = -0.75
    closed = ref_op.retnet_recurrent_ref(q, k, v, decay)
    scan = torch.from_numpy(brute.retnet_recurrent(q.numpy(), k.numpy(), v.numpy(), decay.numpy()))
    assert torch.allclose(closed, scan, atol=2e-6, rtol=1e-5)
    # only the first block_kdim key dims take part
    part = ref_op.retnet_recurrent_ref(q, k, v, decay, block_kdim=3)
    scan3 = torch.from_numpy(brute.retnet_recurrent(q.numpy(), k.numpy(), v.numpy(), decay.numpy(), block_kdim=3))
    assert torch.allclose(part, scan3, atol=2e-6, rtol=1e-5)
    assert torch.allclose(part, ref_op.retnet_recurrent_ref(q[:, :, :3], k[:, :, :3], v, decay), atol=1e-6)
    assert not torch.allclose(part, closed, atol=1e-3)


def test_recurrent_special_cases():
    q, k, v, decay = _recurrent_inputs(1, seqlen=24)
    h, seqlen = decay.shape
    # decay 1: causal linear attention, out = V tril(K^T Q)
    ones = torch.ones(h, seqlen)
    s = k.transpose(-1, -2).double() @ q.double()
    expect = (v.double() @ torch.triu(s)).float()            # [m, n] kept for m <= n
    assert torch.allclose(ref_op.retnet_recurrent_ref(q, k, v, ones), expect, atol=1e-5)
    assert torch.allclose(torch.from_numpy(brute.retnet_recurrent(q.numpy(), k.numpy(), v.numpy(), ones.numpy())), expect, atol=1e-5)
    # decay 0: no history, out_n = (q_n . k_n) v_n
    zeros = torch.zeros(h, seqlen)
    expect0 = (q * k).sum(dim=2, keepdim=True) * v
    assert torch.allclose(ref_op.retnet_recurrent_ref(q, k, v, zeros), expect0, atol=1e-6)
    assert torch.allclose(torch.from_numpy(brute.retnet_recurrent(q.numpy(), k.numpy(), v.numpy(), zeros.numpy())), expect0, atol=1e-6)
    # decay matrix entries: diagonal 1, first superdiagonal a_n, zero below the diagonal
    d = ref_op.retnet_recurrent_decay_matrix(decay)
    assert torch.equal(torch.diagonal(d, dim1=1, dim2=2), torch.ones(h, seqlen, dtype=torch.float64))
    assert torch.allclose(torch.diagonal(d, offset=1, dim1=1, dim2=2), decay[:, 1:].double())
    assert torch.equal(torch.tril(d, diagonal=-1), torch.zeros_like(d))
    assert torch.allclose(d[:, 2, 7], decay[:, 3:8].double().prod(dim=-1))
    # linear in v and in q
    q2, _, v2, _ = _recurrent_inputs(2, seqlen=24)
    lhs = ref_op.retnet_recurrent_ref(q, k, v + 2 * v2, decay)
    assert torch.allclose(lhs, ref_op.retnet_recurrent_ref(q, k, v, decay) + 2 * ref_op.retnet_recurrent_ref(q, k, v2, decay), atol=1e-5)
    lhs = ref_op.retnet_recurrent_ref(q - q2, k, v, decay)
    assert torch.allclose(lhs, ref_op.retnet_recurrent_ref(q, k, v, decay) - ref_op.retnet_recurrent_ref(q2, k, v, decay), atol=1e-5)


def test_recurrent_form_equals_parallel_retention_for_a_constant_decay():
    """With decay[h, n] = gamma_h the scan is the numerator of parallel retention under the decay mask."""
    b, h, seqlen, kdim, vdim = 1, 2, 32, 16, 8
    g = torch.Generator().manual_seed(3)
    q = torch.randn(b, h, seqlen, kdim, generator=g)
    k = torch.randn(b, h, seqlen, kdim, generator=g)
    v = torch.randn(b, h, seqlen, vdim, generator=g)
    mask = ref_op.retnet_decay_mask(h, seqlen, seqlen, dtype=torch.float32)
    o, r = ref_op.retnet_ref(q, k, v, mask, return_r=True)
    numerator = o * r.unsqueeze(-1)                              # undo the normalisation: (q k^T * mask) v
    gamma = 1.0 - 2.0 ** (-5.0 - torch.arange(h, dtype=torch.float32))
    decay = gamma.unsqueeze(1).expand(h, seqlen).contiguous()
    out = ref_op.retnet_recurrent_ref(q.transpose(-1, -2), k.transpose(-1, -2), v.transpose(-1, -2), decay)
    assert torch.allclose(out.transpose(-1, -2), numerator, atol=2e-4, rtol=1e-4)
