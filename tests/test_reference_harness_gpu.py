"""The full-size cases of the reference's own harness, through the public operators, every (batch, head) slice against
the oracle: reference python/tests/test_runtime.py:12-88,97-161 (B4 H8 S2048 at d_qk/d_v 256/256, 256/128 and 128/128 for
the attention forward; 256/256 with a dense N(0,1) mask for the RetNet forward and backward) and the head sizes of
python/benchmarks/bench_retnet.py:99-104 (64, 128, 192, 256 at S2048).  Inputs are torch.randn under seed 0 as there;
the reference compares with rtol = atol = 1e-3 on the GPU, these tests hold the kernels to the bound of
oracle/tolerance.py against the fp32 oracle on the host."""
import pytest
import torch

import attention_autotuner_amd as aat
from attention_autotuner_amd.arch import MI355X
from oracle import ref_op, tolerance

pytestmark = pytest.mark.gpu
ARCH = MI355X()
B, H, S = 4, 8, 2048


def _randn(g, *shape):
    return torch.randn(*shape, generator=g).half()


@pytest.mark.parametrize("dqk,dv", [(256, 256), (256, 128), (128, 128)])
def test_attention_forward_at_the_reference_harness_sizes(dqk, dv):
    g = torch.Generator().manual_seed(0)
    q, k, v = _randn(g, B, H, S, dqk), _randn(g, B, H, S, dqk), _randn(g, B, H, S, dv)
    o = aat.flash_attn_func(q.cuda(), k.cuda(), v.cuda(), ARCH).float().cpu()
    for b in range(B):
        tolerance.assert_close(o[b], ref_op.attention_ref(q[b], k[b], v[b]), f"attention {dqk}/{dv} batch {b}")
    # the reference's kernels hard-code scale 0.125 whatever the head size (csrc/kernels/attention/regfuse/regfuse.h:50): that call too
    o = aat.flash_attn_func(q.cuda(), k.cuda(), v.cuda(), ARCH, False, aat.REFERENCE_SOFTMAX_SCALE).float().cpu()
    tolerance.assert_close(o[B - 1], ref_op.attention_ref(q[B - 1], k[B - 1], v[B - 1], 0.125), f"attention {dqk}/{dv} at the literal scale")


@pytest.mark.parametrize("d", [64, 128, 192, 256])
def test_retnet_forward_and_backward_with_a_dense_mask_at_the_reference_harness_sizes(d):
    g = torch.Generator().manual_seed(0)
    q, k, v, do = (_randn(g, B, H, S, d) for _ in range(4))
    mask = _randn(g, H, S, S)                                  # dense N(0,1): nothing to skip
    qc, kc, vc = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = aat.RetNetAttnFunc(qc, kc, vc, mask.cuda(), ARCH)      # as the reference calls it: five arguments
    o.backward(do.cuda())
    torch.cuda.synchronize()
    grads = (qc.grad, kc.grad, vc.grad)
    for b in range(B):
        sl = slice(b, b + 1)
        tolerance.assert_close(o[sl].detach(), ref_op.retnet_ref(q[sl], k[sl], v[sl], mask), f"retnet {d}/{d} dense mask batch {b} o")
        as_kernel = ref_op.retnet_bwd_ref(q[sl], k[sl], v[sl], mask, do[sl], operand_dtype=torch.float16)
        exact = ref_op.retnet_bwd_ref(q[sl], k[sl], v[sl], mask, do[sl])
        terms = ref_op.retnet_bwd_rounding_bound(q[sl], k[sl], v[sl], mask, do[sl])
        for name, got, wk, we, t in zip(("dq", "dk", "dv"), grads, as_kernel, exact, terms):
            tolerance.assert_close(got[sl], wk, f"retnet {d}/{d} dense mask batch {b} {name} vs fp16-operand form")
            tolerance.assert_close_rounded_operand(got[sl], we, t, f"retnet {d}/{d} dense mask batch {b} {name} vs exact fp32 form")
