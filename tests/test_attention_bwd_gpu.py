"""GPU parity of the attention backward (dq, dk, dv) against the CPU oracle, through the operator and
through the C ABI.

Tolerance (oracle/tolerance.py; gradients are checked twice, see _grads_close): max |err| <= 2e-3 on fp16 gradients versus the fp32 oracle on the same
seeded inputs wherever |ref| < 4, one fp16 unit in the last place of the reference above; the forward's
log-sum-exp is compared at 1e-3 absolute.
"""
import ctypes
import os
import math

import pytest
import torch

import attention_autotuner_amd as aat
from attention_autotuner_amd.arch import MI355X
from attention_autotuner_amd.autotuner import Runtime, codegen, gfx950_space, library, prebuilt
from attention_autotuner_amd.autotuner.configs import AttnBwdConfig
from attention_autotuner_amd.autotuner import prebuilt_extra as parity_matrix
from oracle import ref_op, tolerance

pytestmark = pytest.mark.gpu
ARCH = MI355X()


def _inputs(b, h, sq, sk, dqk, dv, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, h, sq, dqk, generator=g).half()
    k = torch.randn(b, h, sk, dqk, generator=g).half()
    v = torch.randn(b, h, sk, dv, generator=g).half()
    do = torch.randn(b, h, sq, dv, generator=g).half()
    return q, k, v, do


def _close(got, ref):
    ok, worst_small, worst_large, n_large = tolerance.check(got, ref)
    print(f"  max |err| {worst_small:.3e} (|ref| < 4), {worst_large:.2f} ulp over {n_large} entries with |ref| >= 4")
    return ok, (worst_small, worst_large)


def _grads_close(what, grads, q, k, v, do, scale, causal, o=None):
    """dq, dk, dv held to the literal rule against the kernels' arithmetic (delta from the fp16 output the
    forward stored -- ``o`` when the operator's own forward wrote it -- and P, dS rounded to fp16 before the
    dependent contraction) and, against the exact fp32 form, to what those roundings can do in the worst case."""
    as_kernel = ref_op.attention_bwd_ref(q, k, v, do, scale, causal, o=o, operand_dtype=torch.float16)
    exact = ref_op.attention_bwd_ref(q, k, v, do, scale, causal)
    terms = ref_op.attention_bwd_rounding_bound(q, k, v, do, scale, causal, o_stored=o)
    for name, g, wk, we, t in zip(("dq", "dk", "dv"), grads, as_kernel, exact, terms):
        tolerance.assert_close(g, wk, f"{what} {name} vs fp16-operand form")
        tolerance.assert_close_rounded_operand(g, we, t, f"{what} {name} vs exact fp32 form")


def _op_grads(q, k, v, do, causal, scale=None):
    qc, kc, vc = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = aat.flash_attn_func(qc, kc, vc, ARCH, causal, scale)
    o.backward(do.cuda())
    return o, qc.grad, kc.grad, vc.grad


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dqk,dv", parity_matrix.ATTN_BWD_DIMS)
@pytest.mark.parametrize("sq,sk", [(256, 256), (128, 384), (384, 128)])
def test_operator_backward_matches_oracle(dqk, dv, sq, sk, causal):
    q, k, v, do = _inputs(2, 3, sq, sk, dqk, dv, seed=sq + dqk)
    o, dq, dk, dv_ = _op_grads(q, k, v, do, causal)
    _grads_close(f"{dqk}/{dv} {sq}x{sk} causal={causal}", (dq, dk, dv_), q, k, v, do, None, causal, o=o.detach())


def test_forward_lse_entry_matches_oracle():
    q, k, v, _ = _inputs(1, 4, 256, 512, 128, 128, seed=3)
    for causal in (False, True):
        cfg = gfx950_space.default_forward_config("attn", 128, 128, ARCH, 256, 512)
        o = torch.empty(1, 4, 256, 128, dtype=torch.float16, device="cuda")
        lse = torch.empty(1, 4, 256, dtype=torch.float32, device="cuda")
        Runtime(ARCH, cfg).apply([q.cuda(), k.cuda(), v.cuda(), o], causal=causal, lse=lse)
        ref_o, ref_lse = ref_op.attention_ref(q, k, v, None, causal, return_lse=True)
        assert (lse.cpu() - ref_lse).abs().max().item() <= 1e-3
        assert (o.float().cpu() - ref_o).abs().max().item() <= 2e-3


@pytest.mark.parametrize("causal", [False, True])
def test_config2_backward_b4_h32_s2048_d128(causal):
    q, k, v, do = _inputs(4, 32, 2048, 2048, 128, 128, seed=1)
    o, dq, dk, dv_ = _op_grads(q, k, v, do, causal)
    for b, h in ((0, 0), (2, 17), (3, 31)):          # (batch, head) slices are independent
        sl = (slice(b, b + 1), slice(h, h + 1))
        _grads_close(f"config 2 ({b},{h}) causal={causal}", (dq[sl], dk[sl], dv_[sl]), q[sl], k[sl], v[sl], do[sl], None, causal, o=o[sl].detach())
    # size-independent properties on the whole problem: rows of dS sum to zero, so with K := 1 dQ vanishes;
    # and the gradients are linear in dO
    ones = torch.ones_like(k)
    _, dq1, _, _ = _op_grads(q, ones, v, do, causal)
    assert dq1.float().abs().max().item() <= 2e-3
    _, dq2, dk2, dv2 = _op_grads(q, k, v, (2 * do.float()).half(), causal)
    for g1, g2 in ((dq, dq2), (dk, dk2), (dv_, dv2)):
        assert (2 * g1.float() - g2.float()).abs().max().item() <= 4e-3 + 2e-3 * g2.float().abs().max().item()


# every tile shape of the parity set with the row kernel at one wave per SIMD, and at two where two blocks fit a CU's LDS
TILE_CASES = [(br, bc, nt, st, wpe) for br, bc, nt, st in parity_matrix.ATTN_BWD_TILES for wpe in (1, 2)
              if gfx950_space.attn_backward_valid(AttnBwdConfig(br, bc, 128, 128, nt, st, row_waves_per_eu=wpe), ARCH)]
assert len(TILE_CASES) > len(parity_matrix.ATTN_BWD_TILES)


@pytest.mark.parametrize("br,bc,nt,st,row_wpe", TILE_CASES)
def test_tile_variants_agree(br, bc, nt, st, row_wpe):
    """Tile shapes of the parity set, the row kernel compiled for one and for two waves per SIMD."""
    q, k, v, do = _inputs(1, 2, 256, 256, 128, 128, seed=5)
    o_ref, lse_ref = ref_op.attention_ref(q, k, v, 0.11, True, return_lse=True)
    cfg = AttnBwdConfig(br, bc, 128, 128, nt, st, row_waves_per_eu=row_wpe)
    arrays = [t.cuda() for t in (q, k, v, o_ref.half(), do, lse_ref)]
    grads = [torch.empty_like(arrays[0]), torch.empty_like(arrays[1]), torch.empty_like(arrays[2])]
    Runtime(ARCH, cfg).apply(arrays + grads, softmax_scale=0.11, causal=True)
    _grads_close(str(cfg), grads, q, k, v, do, 0.11, True)


def test_row_kernel_with_its_own_tile_height():
    """Column kernel on 64-row streamed tiles, row kernel (two waves per SIMD) on 32-row ones."""
    q, k, v, do = _inputs(1, 2, 256, 384, 128, 128, seed=6)
    o_ref, lse_ref = ref_op.attention_ref(q, k, v, 0.11, True, return_lse=True)
    cfg = AttnBwdConfig(64, 64, 128, 128, 128, 2, row_waves_per_eu=2, row_Bc=32)
    assert str(cfg) == "attn_bwd_64_64_128_128_128_2_rw2_rb32" and gfx950_space.attn_backward_valid(cfg, ARCH)
    arrays = [t.cuda() for t in (q, k, v, o_ref.half(), do, lse_ref)]
    grads = [torch.empty_like(arrays[0]), torch.empty_like(arrays[1]), torch.empty_like(arrays[2])]
    Runtime(ARCH, cfg).apply(arrays + grads, softmax_scale=0.11, causal=True)
    _grads_close(str(cfg), grads, q, k, v, do, 0.11, True)


def test_abi_error_paths_and_stream():
    cfg = gfx950_space.default_attn_backward_config(128, 128, ARCH, 128, 128)
    lib = library.load(codegen.compile_config(cfg, ARCH), "attn_bwd")
    q, k, v, do = (t.cuda() for t in _inputs(1, 1, 256, 256, 128, 128, seed=7))
    o = torch.zeros_like(do)
    lse = torch.zeros(1, 1, 256, device="cuda")
    dq, dk, dv_ = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    ptrs = [ctypes.c_void_p(t.data_ptr()) for t in (q, k, v, o, do, lse, dq, dk, dv_)]
    null = ctypes.c_void_p(0)
    # no workspace -> AAT_ERR_WORKSPACE; indivisible length -> AAT_ERR_SHAPE; nothing is launched in either case
    assert lib.kernel_entry_ex(*ptrs, 1, 1, 256, 256, ctypes.c_float(0.1), 0, null, ctypes.c_size_t(0), null) == -3
    ws = torch.empty(lib.workspace_size(1, 1, 256, 256), dtype=torch.uint8, device="cuda")
    wsp, wsn = ctypes.c_void_p(ws.data_ptr()), ctypes.c_size_t(ws.numel())
    assert lib.kernel_entry_ex(*ptrs, 1, 1, 200, 256, ctypes.c_float(0.1), 0, wsp, wsn, null) == -2
    assert lib.profile_ex(*ptrs, 1, 1, 256, 256, ctypes.c_float(0.1), 0, null, ctypes.c_size_t(0), null) == -1.0
    # launches on the stream it is given
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        rc = lib.kernel_entry_ex(*ptrs, 1, 1, 256, 256, ctypes.c_float(0.1), 0, wsp, wsn, ctypes.c_void_p(side.cuda_stream))
    side.synchronize()
    assert rc == 0 and torch.isfinite(dq.float()).all()


def test_a_problem_without_a_backward_configuration_says_so(monkeypatch):
    """The forward runs; the backward reports what the search space cannot cover as NotImplementedError."""
    from attention_autotuner_amd.autotuner import base_tunner, gfx950_space

    def none_fits(*a, **kw):
        raise gfx950_space.NoValidConfigError("no default attn_bwd configuration fits")
    q, k, v, do = _inputs(1, 1, 128, 128, 64, 64, seed=9)
    qc, kc, vc = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = aat.flash_attn_func(qc, kc, vc, ARCH)
    monkeypatch.setattr(gfx950_space, "default_attn_backward_config", none_fits)
    for key in [key for key in base_tunner._memo if key[0] == "plan" and key[3] == "attn_bwd"]:
        del base_tunner._memo[key]
    with pytest.raises(NotImplementedError):
        o.backward(do.cuda())


@pytest.mark.parametrize("tile", parity_matrix.ATTN_BWD_SPLIT_TILES)
def test_one_column_kernel_per_output_agrees(tile):
    """dV and dK from separate column kernels (each on its own register budget), against the oracle and, bit for
    bit, against the two-output kernel of the same tile shape (same arithmetic in the same order)."""
    q, k, v, do = _inputs(1, 2, 256, 384, 128, 128, seed=15)
    cfg = parity_matrix.attn_bwd_split_config(*tile)
    assert gfx950_space.attn_backward_valid(cfg, ARCH), cfg
    for causal in (False, True):
        o_ref, lse_ref = ref_op.attention_ref(q, k, v, 0.09, causal, return_lse=True)
        arrays = [t.cuda() for t in (q, k, v, o_ref.half(), do, lse_ref)]
        grads = [torch.empty_like(arrays[0]), torch.empty_like(arrays[1]), torch.empty_like(arrays[2])]
        Runtime(ARCH, cfg).apply(arrays + grads, softmax_scale=0.09, causal=causal)
        _grads_close(f"{cfg} causal={causal}", grads, q, k, v, do, 0.09, causal)
        whole = AttnBwdConfig(cfg.Br, cfg.Bc, 128, 128, cfg.Nthreads, cfg.num_stages_qk)
        if gfx950_space.attn_backward_valid(whole, ARCH) and os.path.exists(codegen.library_path(whole)):
            both = [torch.empty_like(g) for g in grads]
            Runtime(ARCH, whole).apply(arrays + both, softmax_scale=0.09, causal=causal)
            assert torch.equal(both[1], grads[1]) and torch.equal(both[2], grads[2]), (cfg, causal)
