"""GPU parity of the attention forward kernels against the CPU oracle, through the C ABI.

Tolerance: max-abs error <= 2e-3 on fp16 outputs versus the fp32 oracle on the same seeded inputs.
"""
import ctypes
import math
import os

import pytest
import torch

import attention_autotuner_amd as aat
from attention_autotuner_amd.arch import MI355X
from attention_autotuner_amd.autotuner import AttnConfig, Runtime, codegen, gfx950_space, library
from attention_autotuner_amd.autotuner.runtime import KernelLaunchError
from oracle import ref_op

pytestmark = pytest.mark.gpu
ARCH = MI355X()
TOL = 2e-3


def _inputs(b, h, sq, sk, dqk, dv, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, h, sq, dqk, generator=g).half()
    k = torch.randn(b, h, sk, dqk, generator=g).half()
    v = torch.randn(b, h, sk, dv, generator=g).half()
    return q, k, v


def _err(o, ref):
    return (o.float().cpu() - ref).abs().max().item()


@pytest.mark.parametrize("causal", [False, True])
def test_config1_plumbing_b2_h8_s512_d64(causal):
    q, k, v = _inputs(2, 8, 512, 512, 64, 64)
    o = aat.flash_attn_func(q.cuda(), k.cuda(), v.cuda(), ARCH, causal)
    assert o.shape == (2, 8, 512, 64) and o.dtype == torch.float16
    assert _err(o, ref_op.attention_ref(q, k, v, 1 / math.sqrt(64), causal)) <= TOL


@pytest.mark.parametrize("causal", [False, True])
def test_config2_headline_b4_h32_s2048_d128(causal):
    q, k, v = _inputs(4, 32, 2048, 2048, 128, 128, seed=1)
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    o = aat.flash_attn_func(qc, kc, vc, ARCH, causal)
    # the oracle on every (batch, head) slice, one batch element (32 heads) at a time
    oc = o.float().cpu()
    worst = max(((oc[b] - ref_op.attention_ref(q[b], k[b], v[b], None, causal)).abs().amax(dim=(-1, -2)).max().item(), b) for b in range(4))
    print(f"config 2 causal={causal}: max |err| over all 128 slices {worst[0]:.3e} (batch {worst[1]})")
    assert worst[0] <= TOL, worst
    # size-independent properties on the whole problem
    ones = torch.ones_like(vc)
    o1 = aat.flash_attn_func(qc, kc, ones, ARCH, causal)
    err1 = (o1.float() - 1).abs().max().item()
    assert err1 <= 1e-3            # rows of P sum to one
    o0 = aat.flash_attn_func(qc, kc, vc, ARCH, causal, 0.0)        # scale 0: (prefix) mean of V
    if causal:
        want = torch.cumsum(vc.float(), dim=2) / torch.arange(1, 2049, device="cuda").view(1, 1, -1, 1)
    else:
        want = vc.float().mean(dim=2, keepdim=True).expand_as(o0)
    err0 = (o0.float() - want).abs().max().item()
    assert err0 <= TOL
    again = aat.flash_attn_func(qc, kc, vc, ARCH, causal)
    assert torch.equal(o, again)                                    # deterministic
    # one batch element at a time (the tuner may pick another tiling for that problem)
    alone = aat.flash_attn_func(qc[2:3], kc[2:3], vc[2:3], ARCH, causal)
    assert (alone[0].float() - o[2].float()).abs().max().item() <= 1e-3


def test_config5_long_kv_b1_h32_sq256_sk16384_d128():
    q, k, v = _inputs(1, 32, 256, 16384, 128, 128, seed=2)
    o = aat.flash_attn_func(q.cuda(), k.cuda(), v.cuda(), ARCH)
    assert _err(o, ref_op.attention_ref(q, k, v)) <= TOL


def test_reference_literal_scale_and_explicit_scale():
    q, k, v = _inputs(1, 4, 256, 256, 128, 128, seed=3)
    o = aat.flash_attn_func(q.cuda(), k.cuda(), v.cuda(), ARCH, False, aat.REFERENCE_SOFTMAX_SCALE)
    assert _err(o, ref_op.attention_ref(q, k, v, 0.125)) <= TOL
    o = aat.flash_attn_func(q.cuda(), k.cuda(), v.cuda(), ARCH, False, 0.05)
    assert _err(o, ref_op.attention_ref(q, k, v, 0.05)) <= TOL


def test_scaled_inputs_like_the_reference_tuner_demo():
    # the reference's tuner driver uses k, v = 3 * randn: sharper softmax
    q, k, v = _inputs(1, 4, 256, 512, 64, 64, seed=4)
    k, v = (3 * k.float()).half(), (3 * v.float()).half()
    o = aat.flash_attn_func(q.cuda(), k.cuda(), v.cuda(), ARCH)
    assert _err(o, ref_op.attention_ref(q, k, v)) <= 3 * TOL      # |v| is 3x larger


from attention_autotuner_amd.autotuner import prebuilt_extra as parity_matrix
from attention_autotuner_amd.autotuner.prebuilt_extra import PARITY_DIMS, PARITY_TILES as CONFIGS


@pytest.mark.parametrize("dqk,dv", PARITY_DIMS)
def test_every_configuration_agrees_with_the_oracle(dqk, dv):
    q, k, v = _inputs(1, 2, 256, 512, dqk, dv, seed=5)
    refs = {c: ref_op.attention_ref(q, k, v, None, c) for c in (False, True)}
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    ran = 0
    variants = [(t, 0) for t in CONFIGS] + [(t, 1) for t in CONFIGS if t[3:5] == (2, 2)]
    for (br, bc, nt, sq, sv, wpe), pipe in variants:
        cfg = AttnConfig(br, bc, dqk, dv, dqk, bc, sq, sv, nt, True, waves_per_eu=wpe, sw_pipeline=pipe).set_fuse_type("register")
        if not gfx950_space.forward_valid(cfg, ARCH):
            continue
        assert os.path.exists(codegen.library_path(cfg)), f"library for {cfg} was not built ahead of time"
        for causal in (False, True):
            o = torch.zeros(1, 2, 256, dv, dtype=torch.float16, device="cuda")
            Runtime(ARCH, cfg).apply([qc, kc, vc, o], causal=causal)
            assert _err(o, refs[causal]) <= TOL, (cfg, causal)
        ran += 1
    assert ran >= 3


@pytest.mark.parametrize("dqk,dv", parity_matrix.UNIT_DIMS)
def test_units_inside_a_kv_tile_agree_with_the_oracle(dqk, dv):
    """Configurations whose waves own two or more 32-row groups and work a kv tile through in 32- or 64-row units (where
    registers are scarce: operand addresses from one register, in-place operand rings, scalar-base tile copies), causal and
    not, S_q != S_kv, and a problem whose row blocks outnumber what the chip holds (persistent variant where one exists)."""
    q, k, v = _inputs(1, 3, 1024, 1280, dqk, dv, seed=21)
    refs = {c: ref_op.attention_ref(q, k, v, None, c) for c in (False, True)}
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    qm, km, vm = _inputs(2, 140, 1024, 256, dqk, dv, seed=22)           # 560 / 1120 / 2240 row blocks, four or two kv tiles
    ref_many = torch.cat([ref_op.attention_ref(qm[b:b + 1], km[b:b + 1], vm[b:b + 1]) for b in range(2)])
    qmc, kmc, vmc = qm.cuda(), km.cuda(), vm.cuda()
    ran = 0
    for t in parity_matrix.UNIT_TILES:
        cfg = parity_matrix.unit_config(*t, dqk, dv)
        if not gfx950_space.forward_valid(cfg, ARCH):
            continue
        assert os.path.exists(codegen.library_path(cfg)), f"library for {cfg} was not built ahead of time"
        for causal in (False, True):
            o = torch.full((1, 3, 1024, dv), float("nan"), dtype=torch.float16, device="cuda")
            Runtime(ARCH, cfg).apply([qc, kc, vc, o], causal=causal)
            assert _err(o, refs[causal]) <= TOL, (cfg, causal)
        o = torch.full((2, 140, 1024, dv), float("nan"), dtype=torch.float16, device="cuda")
        lse = torch.zeros(2, 140, 1024, dtype=torch.float32, device="cuda")
        Runtime(ARCH, cfg).apply([qmc, kmc, vmc, o], lse=lse)
        assert _err(o, ref_many) <= TOL, cfg
        ref_lse = torch.logsumexp(qm[1, 139].float() @ km[1, 139].float().t() / math.sqrt(dqk), dim=-1)
        assert (lse[1, 139].cpu() - ref_lse).abs().max().item() <= 1e-3, cfg
        ran += 1
    assert ran >= 2, (dqk, dv, ran)


def _persistent_ok(br, bc, nt, sq, sv, wpe, dqk, dv):
    """Mirror of AttnFwdRegfuse::Persist<WPE>::kOk (csrc/kernels/attention/regfuse/regfuse.h)."""
    nw = nt // 64
    stage = (br // nw) * (dv * 2 + 16)
    main = sq * bc * dqk * 2 + sv * bc * dv * 2
    budget = (160 * 1024 // max(1, wpe * 4 // nw)) & ~2047
    smem = max(min(main + nw * stage, budget), main)
    return (sq, sv) == (2, 2) and wpe >= 2 and (smem - main) // stage + bc * dqk * 2 // stage + bc * dv * 2 // stage >= nw


def _persistent_tiles(dqk, dv):
    out = []
    for br, bc, nt, sq, sv, wpe in CONFIGS:
        cfg = AttnConfig(br, bc, dqk, dv, dqk, bc, sq, sv, nt, True, waves_per_eu=wpe).set_fuse_type("register")
        if gfx950_space.forward_valid(cfg, ARCH) and _persistent_ok(br, bc, nt, sq, sv, wpe, dqk, dv):
            out.append(cfg)
    return out


# head sizes at which some configuration of the parity set has a persistent variant (the others leave no LDS for the staging)
PERSISTENT_DIMS = [d for d in PARITY_DIMS if _persistent_tiles(*d)]
assert (128, 128) in PERSISTENT_DIMS and (64, 64) in PERSISTENT_DIMS


@pytest.mark.parametrize("dqk,dv", PERSISTENT_DIMS)
def test_persistent_blocks_agree_with_the_oracle(dqk, dv):
    """More row blocks than the chip holds at once: non-causal launches of the configurations that have a
    persistent variant walk several row blocks per block (unevenly: 2080, 1040 or 520 row blocks)."""
    q, k, v = _inputs(2, 130, 512, 256, dqk, dv, seed=11)
    ref = ref_op.attention_ref(q, k, v, None, False)
    ref_lse = torch.logsumexp(q.float() @ k.float().transpose(-1, -2) / math.sqrt(dqk), dim=-1)
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    ran = 0
    for cfg in _persistent_tiles(dqk, dv):
        o = torch.zeros(2, 130, 512, dv, dtype=torch.float16, device="cuda")
        lse = torch.zeros(2, 130, 512, dtype=torch.float32, device="cuda")
        Runtime(ARCH, cfg).apply([qc, kc, vc, o], lse=lse)
        assert _err(o, ref) <= TOL, cfg
        assert (lse.cpu() - ref_lse).abs().max().item() <= 1e-3, cfg
        plain_entry = torch.zeros_like(o)
        Runtime(ARCH, cfg).apply([qc, kc, vc, plain_entry])            # without the log-sum-exp output
        assert torch.equal(plain_entry, o), cfg
        # one (batch, head) at a time the same library takes the one-row-block-per-block path: same bits
        single = torch.zeros(1, 1, 512, dv, dtype=torch.float16, device="cuda")
        for b, h in ((0, 0), (1, 77), (1, 129)):
            Runtime(ARCH, cfg).apply([qc[b:b + 1, h:h + 1].contiguous(), kc[b:b + 1, h:h + 1].contiguous(),
                                      vc[b:b + 1, h:h + 1].contiguous(), single])
            assert torch.equal(single[0, 0], o[b, h]), (cfg, b, h)
        ran += 1
    assert ran >= 1


@pytest.mark.parametrize("dqk,dv", [(64, 64), (128, 128), (256, 512)])
def test_lds_fused_variants_agree_with_the_oracle(dqk, dv):
    from attention_autotuner_amd.autotuner.prebuilt_extra import SHARED_TILES
    q, k, v = _inputs(1, 2, 128, 256, dqk, dv, seed=8)
    refs = {c: ref_op.attention_ref(q, k, v, None, c) for c in (False, True)}
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    ran = 0
    for br, bc, nt, sq, sv, w1n, w2n, wpe in SHARED_TILES:
        cfg = AttnConfig(br, bc, dqk, dv, dqk, bc, sq, sv, nt, True, w1n, w2n, waves_per_eu=wpe)
        cfg.fuse_type = "shared"
        if not gfx950_space.forward_valid(cfg, ARCH):
            continue
        assert os.path.exists(codegen.library_path(cfg)), f"library for {cfg} was not built ahead of time"
        for causal in (False, True):
            o = torch.zeros(1, 2, 128, dv, dtype=torch.float16, device="cuda")
            Runtime(ARCH, cfg).apply([qc, kc, vc, o], causal=causal)
            assert _err(o, refs[causal]) <= TOL, (cfg, causal)
        ran += 1
    assert ran >= 1


@pytest.mark.parametrize("dqk,ns,sk", [(128, 4, 1024), (128, 8, 16384), (64, 2, 512)])
def test_kv_split_matches_the_oracle_and_the_unsplit_kernel(dqk, ns, sk):
    q, k, v = _inputs(1, 4, 256, sk, dqk, dqk, seed=9)
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    cfg = AttnConfig(128, 64, dqk, dqk, dqk, 64, 2, 2, 256, True, waves_per_eu=2, kv_splits=ns).set_fuse_type("register")
    assert os.path.exists(codegen.library_path(cfg))
    rt = Runtime(ARCH, cfg)
    need = rt.workspace_size(1, 4, 256, sk)
    assert need == ns * 4 * 256 * (dqk + 1) * 4
    o = torch.zeros(1, 4, 256, dqk, dtype=torch.float16, device="cuda")
    rt.apply([qc, kc, vc, o])                                   # Runtime allocates the workspace it was asked for
    assert _err(o, ref_op.attention_ref(q, k, v)) <= TOL
    unsplit = AttnConfig(128, 64, dqk, dqk, dqk, 64, 2, 2, 256, True, waves_per_eu=2).set_fuse_type("register")
    o1 = torch.zeros_like(o)
    Runtime(ARCH, unsplit).apply([qc, kc, vc, o1])
    assert (o.float() - o1.float()).abs().max().item() <= 1e-3
    # a causal call on a splitting configuration runs the unsplit causal kernel
    if sk == 512:
        q2, k2, v2 = _inputs(1, 4, 512, 512, dqk, dqk, seed=10)
        o2 = torch.zeros(1, 4, 512, dqk, dtype=torch.float16, device="cuda")
        rt.apply([q2.cuda(), k2.cuda(), v2.cuda(), o2], causal=True)
        assert _err(o2, ref_op.attention_ref(q2, k2, v2, None, True)) <= TOL
    # without a workspace the extended entry point refuses; the reference-signature one runs unsplit
    lib = library.load(rt._path(), "attn")
    ptrs = [ctypes.c_void_p(t.data_ptr()) for t in (qc, kc, vc, o)]
    rc = lib.kernel_entry_ex(*ptrs, 1, 4, 256, sk, ctypes.c_float(0.1), 0, None, 0, None)
    assert rc == -3


def test_reference_signature_entry_points():
    """profile / kernel_entry keep the reference's argument order (kernel_entry swaps the lengths)
    and its literal behaviour: scale 0.125, non-causal, null stream."""
    q, k, v = _inputs(1, 2, 256, 512, 128, 128, seed=6)
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    o = torch.zeros(1, 2, 256, 128, dtype=torch.float16, device="cuda")
    cfg = gfx950_space.default_forward_config("attn", 128, 128, ARCH)
    lib = library.load(Runtime(ARCH, cfg)._path(), "attn")
    ptrs = [ctypes.c_void_p(t.data_ptr()) for t in (qc, kc, vc, o)]
    torch.cuda.synchronize()
    assert lib.kernel_entry(*ptrs, 1, 2, 512, 256) == 0          # (B, H, Seq_k, Seq_q)
    torch.cuda.synchronize()
    assert _err(o, ref_op.attention_ref(q, k, v, 0.125)) <= TOL
    ms = lib.profile(*ptrs, 1, 2, 256, 512)                       # (B, H, Seq_q, Seq_k)
    assert 0 < ms < 50
    assert lib.kernel_entry(*ptrs, 1, 2, 500, 256) == -2          # indivisible: refused, nothing launched
    assert lib.profile(*ptrs, 1, 2, 256, 500) == -1


def test_indivisible_shape_raises():
    q, k, v = _inputs(1, 1, 128, 80, 64, 64)
    with pytest.raises((KernelLaunchError, ValueError)):   # 80 is not a multiple of any kv tile
        aat.flash_attn_func(q.cuda(), k.cuda(), v.cuda(), ARCH)


def test_runs_on_the_current_stream():
    q, k, v = _inputs(1, 2, 256, 256, 64, 64, seed=7)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        o = aat.flash_attn_func(q.cuda(), k.cuda(), v.cuda(), ARCH)
    s.synchronize()
    assert _err(o, ref_op.attention_ref(q, k, v)) <= TOL


def test_offsets_beyond_int32_elements():
    """k and v hold 2^31 elements each: the last (batch, head) slice sits past every 32-bit element offset.
    The kernel must give that slice exactly what it gives the same data placed at offset zero."""
    b, h, sq, sk, d = 16, 32, 256, 32768, 128
    g = torch.Generator(device="cuda").manual_seed(11)
    k = torch.empty(b, h, sk, d, dtype=torch.float16, device="cuda")
    v = torch.empty(b, h, sk, d, dtype=torch.float16, device="cuda")
    assert k.numel() == 2 ** 31
    k[-1, -1].normal_(generator=g)
    v[-1, -1].normal_(generator=g)
    k[0, 0].normal_(generator=g)
    v[0, 0].normal_(generator=g)
    q = torch.randn(b, h, sq, d, generator=g, dtype=torch.float16, device="cuda")
    o = aat.flash_attn_func(q, k, v, ARCH)
    for bi, hi in ((b - 1, h - 1), (0, 0)):
        small = aat.flash_attn_func(q[bi:bi + 1, hi:hi + 1].contiguous(), k[bi:bi + 1, hi:hi + 1].contiguous(),
                                    v[bi:bi + 1, hi:hi + 1].contiguous(), ARCH)
        ref = ref_op.attention_ref(q[bi:bi + 1, hi:hi + 1].cpu(), k[bi:bi + 1, hi:hi + 1].cpu(), v[bi:bi + 1, hi:hi + 1].cpu())
        assert _err(o[bi:bi + 1, hi:hi + 1], ref) <= TOL
        assert _err(small, ref) <= TOL


def test_forward_replays_from_a_captured_graph():
    """A launch through the C ABI can be captured (it allocates nothing and uses the stream it is given);
    replays with new inputs match eager launches."""
    q, k, v = (t.cuda() for t in _inputs(2, 4, 512, 512, 128, 128, seed=21))
    cfg = gfx950_space.default_forward_config("attn", 128, 128, ARCH, 512, 512)
    rt = Runtime(ARCH, cfg)
    o = torch.empty_like(q)
    rt.apply([q, k, v, o], causal=True)                  # first call outside capture: one-time LDS opt-in
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rt.apply([q, k, v, o], causal=True)
    for seed in (22, 23, 24):
        q2, k2, v2 = (t.cuda() for t in _inputs(2, 4, 512, 512, 128, 128, seed=seed))
        q.copy_(q2), k.copy_(k2), v.copy_(v2)
        graph.replay()
        torch.cuda.synchronize()
        eager = torch.empty_like(o)
        rt.apply([q, k, v, eager], causal=True)
        torch.cuda.synchronize()
        assert torch.equal(o, eager)
        assert _err(o, ref_op.attention_ref(q2, k2, v2, None, True)) <= TOL


def test_persistent_forward_replays_from_a_captured_graph():
    """The same for a launch that takes the persistent-block kernel (more row blocks than the chip holds)."""
    cfg = parity_matrix.persistent_graph_config()
    assert _persistent_ok(256, 128, 512, 2, 2, 2, 128, 128)
    q, k, v = (t.cuda() for t in _inputs(2, 130, 512, 256, 128, 128, seed=31))
    rt = Runtime(ARCH, cfg)
    o = torch.empty_like(q)
    rt.apply([q, k, v, o])                               # first call outside capture: one-time set-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rt.apply([q, k, v, o])
    for seed in (32, 33):
        q2, k2, v2 = _inputs(2, 130, 512, 256, 128, 128, seed=seed)
        q.copy_(q2.cuda()), k.copy_(k2.cuda()), v.copy_(v2.cuda())
        graph.replay()
        torch.cuda.synchronize()
        eager = torch.empty_like(o)
        rt.apply([q, k, v, eager])
        torch.cuda.synchronize()
        assert torch.equal(o, eager)
        assert _err(o, ref_op.attention_ref(q2, k2, v2, None, False)) <= TOL


def test_calls_without_a_gradient_skip_autograd_and_repeated_calls_keep_one_plan():
    """``flash_attn_func`` on inputs that need no gradient runs the forward directly; with a gradient it goes through
    ``MultiHeadAttnFunc.apply``.  Same bits either way, and the (configuration, runtime) pair of a problem is resolved
    once per process."""
    from attention_autotuner_amd.autotuner import base_tunner
    q, k, v = (t.cuda() for t in _inputs(2, 4, 512, 512, 128, 128, seed=41))
    o0 = aat.flash_attn_func(q, k, v, ARCH, True)
    keys = [key for key in base_tunner._memo if key[0] == "plan" and key[3] == "attn" and key[5:] == (2, 4, 512, 512, 128, 128, True)]
    assert len(keys) == 1
    plan = base_tunner._memo[keys[0]]
    qg = q.clone().requires_grad_(True)
    o1 = aat.flash_attn_func(qg, k, v, ARCH, True)
    assert o1.requires_grad and o1.grad_fn is not None and not o0.requires_grad
    with torch.no_grad():
        o2 = aat.flash_attn_func(qg, k, v, ARCH, True)
    assert not o2.requires_grad and torch.equal(o0, o1) and torch.equal(o0, o2)
    assert base_tunner._memo[keys[0]] is plan
    o1.backward(torch.ones_like(o1))
    assert qg.grad is not None and bool(torch.isfinite(qg.grad).all())
    assert _err(o0, ref_op.attention_ref(*(t.cpu() for t in (q, k, v)), None, True)) <= TOL
