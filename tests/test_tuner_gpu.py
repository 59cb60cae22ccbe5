"""The tuning loop on the GPU: times prebuilt candidates, checks the winner against torch math before
caching it, and discards a candidate whose output is wrong (nothing is compiled inside these tests:
the candidate lists are restricted to libraries of the shipping set)."""
import json
import os

import pytest

from attention_autotuner_amd.autotuner import prebuilt_extra as parity_matrix
import torch

from attention_autotuner_amd.arch import MI355X
from attention_autotuner_amd.autotuner import AttnConfig, AttnTunner, RetBwdTunner, codegen, gfx950_space, prebuilt, verify
from attention_autotuner_amd.autotuner.tunner import AttnBwdTunner
from attention_autotuner_amd.benchmarks.tune import make_tensors

pytestmark = pytest.mark.gpu
ARCH = MI355X()


def _prebuilt_attention_candidates(dqk, dv):
    out = []
    for br, bc, nt, sq, sv, wpe in parity_matrix.PARITY_TILES[:4]:
        cfg = AttnConfig(br, bc, dqk, dv, dqk, bc, sq, sv, nt, True, waves_per_eu=wpe).set_fuse_type("register")
        if gfx950_space.forward_valid(cfg, ARCH) and os.path.exists(codegen.library_path(cfg)):
            out.append(cfg)
    return out


def test_tune_times_verifies_and_caches(tmp_path, monkeypatch):
    arrays = make_tensors("attn", 1, 4, 512, 512, 128, 128, "cuda")
    tuner = AttnTunner(ARCH, arrays, causal=True)
    tuner.cache_path = str(tmp_path / "cache")
    cands = _prebuilt_attention_candidates(128, 128)
    assert len(cands) >= 2
    monkeypatch.setattr(tuner, "get_tuned_configs", lambda: cands)
    best = tuner.tune(log_path=str(tmp_path / "logs"), use_cache=False)
    assert best in cands and tuner.last_timings[best] == min(tuner.last_timings.values())
    with open(tuner._cache_file()) as f:
        assert json.load(f)["Br"] == best.Br
    log = (tmp_path / "logs" / "profile_result_attn_128_128.txt").read_text()
    assert "best config:" in log and log.count("Config(") == len(cands) + 1
    # a second tuner for the same problem finds the cached entry without timing anything
    again = AttnTunner(ARCH, arrays, causal=True)
    again.cache_path = tuner.cache_path
    assert again.check_cache() == best


def test_a_fast_but_wrong_candidate_is_discarded(tmp_path, monkeypatch):
    arrays = make_tensors("attn", 1, 4, 512, 512, 128, 128, "cuda")
    tuner = AttnTunner(ARCH, arrays)
    tuner.cache_path = str(tmp_path / "cache")
    cands = _prebuilt_attention_candidates(128, 128)
    monkeypatch.setattr(tuner, "get_tuned_configs", lambda: cands)
    fastest = {}
    real = verify.outputs_match

    def first_call_fails(arrs, ref):
        if not fastest:
            fastest["seen"] = True
            return False
        return real(arrs, ref)

    monkeypatch.setattr(verify, "outputs_match", first_call_fails)
    best = tuner.tune(log_path=None, use_cache=False)
    ranked = sorted((c for c in tuner.last_timings), key=lambda c: tuner.last_timings[c])
    assert tuner.last_timings[ranked[-1]] == 1e8           # the discarded winner is recorded as failed
    assert best == ranked[0] and best != ranked[-1]


@pytest.mark.parametrize("op,cls,dims", [("ret_bwd", RetBwdTunner, (1, 2, 256, 256, 64, 64)),
                                         ("attn_bwd", AttnBwdTunner, (1, 2, 256, 256, 128, 128))])
def test_backward_libraries_pass_the_guard(op, cls, dims):
    arrays = make_tensors(op, *dims, "cuda")
    tuner = cls(ARCH, arrays, causal=False)
    cfg = (gfx950_space.default_backward_config(dims[4], dims[5], ARCH, 128, 128) if op == "ret_bwd"
           else gfx950_space.default_attn_backward_config(dims[4], dims[5], ARCH, 128, 128))
    assert tuner.verify(codegen.compile_config(cfg, ARCH))
    # and the guard does notice a wrong output
    idx = next(iter(tuner._reference))
    tuner._reference[idx] = tuner._reference[idx] + 1.0
    assert not tuner.verify(codegen.compile_config(cfg, ARCH))


def test_a_library_that_is_not_built_is_compiled_on_this_machine_and_runs(tmp_path, monkeypatch):
    """The path a first call takes without prebuilt libraries: hipcc on the GPU box itself (one small
    configuration, into a scratch build directory), then the launch, checked against the oracle; and with
    compiling switched off the same miss is an error that names the library."""
    from attention_autotuner_amd.autotuner import Runtime
    from attention_autotuner_amd.autotuner.runtime import KernelLaunchError
    from oracle import ref_op
    cfg = AttnConfig(64, 32, 64, 64, 64, 32, 1, 1, 128, True, waves_per_eu=1).set_fuse_type("register")
    assert gfx950_space.forward_valid(cfg, ARCH)
    build = str(tmp_path / "build")
    monkeypatch.setenv("AAT_NO_JIT", "1")
    with pytest.raises(codegen.MissingLibraryError, match="AAT_NO_JIT"):
        Runtime(ARCH, cfg, tmp_dir=build)
    monkeypatch.setenv("AAT_NO_JIT", "0")
    rt = Runtime(ARCH, cfg, tmp_dir=build)                     # compiles here
    assert rt._path().startswith(build) and os.path.exists(rt._path())
    usage = codegen.resource_usage(rt._path())
    assert usage and not codegen.spilling_kernels(usage)
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(1, 2, 128, 64, generator=g).half() for _ in range(3))
    o = torch.zeros(1, 2, 128, 64, dtype=torch.float16, device="cuda")
    for causal in (False, True):
        rt.apply([q.cuda(), k.cuda(), v.cuda(), o], causal=causal)
        assert (o.float().cpu() - ref_op.attention_ref(q, k, v, None, causal)).abs().max().item() <= 2e-3


def test_default_operator_call_on_a_dense_mask_tunes_in_the_mode_it_launches(tmp_path, monkeypatch):
    """``RetNetAttnFunc(q, k, v, mask, arch)`` as the reference calls it (reference python/tests/test_runtime.py:38-62:
    a dense N(0,1) mask), with an empty tuning cache and tuning on a miss: the operator launches the scanning walk,
    so the tuners it starts must time and verify their candidates in that mode on this mask -- under the causal
    promise every candidate would fail the guard on a mask that is not zero above the diagonal.  Candidates are
    restricted to libraries built ahead of time (nothing compiles here)."""
    import attention_autotuner_amd as aat
    from attention_autotuner_amd.autotuner import base_tunner
    from attention_autotuner_amd.autotuner.tunner import RetTunner
    from attention_autotuner_amd.ops import _resolve
    from oracle import ref_op, tolerance
    monkeypatch.setenv("AAT_TUNE_ON_MISS", "1")
    monkeypatch.setattr(base_tunner, "DEFAULT_CACHE_DIR", str(tmp_path / "cache"))
    monkeypatch.setattr(_resolve, "DEFAULT_LOG_DIR", str(tmp_path / "logs"))
    fwd = [c for c in parity_matrix.parity_configs(ARCH) if c.operation == "ret" and (c.Kd, c.D) == (128, 128)
           and os.path.exists(codegen.library_path(c))]
    bwd = []
    for seq in (None, 128, 64):
        c = gfx950_space.default_backward_config(128, 128, ARCH, seq, seq)
        if c not in bwd and os.path.exists(codegen.library_path(c)):
            bwd.append(c)
    assert len(fwd) >= 2 and bwd
    monkeypatch.setattr(RetTunner, "get_tuned_configs", lambda self: fwd)
    monkeypatch.setattr(RetBwdTunner, "get_tuned_configs", lambda self: bwd)
    g = torch.Generator().manual_seed(0)
    q, k, v, do = (torch.randn(1, 2, 256, 128, generator=g).half() for _ in range(4))
    mask = torch.randn(2, 256, 256, generator=g).half()                # dense: nothing to skip, nothing promised
    qc, kc, vc = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = aat.RetNetAttnFunc(qc, kc, vc, mask.cuda(), ARCH)
    o.backward(do.cuda())
    torch.cuda.synchronize()
    tolerance.assert_close(o.detach(), ref_op.retnet_ref(q, k, v, mask), "tuned on a miss, dense mask: o")
    for name, got, want in zip(("dq", "dk", "dv"), (qc.grad, kc.grad, vc.grad),
                               ref_op.retnet_bwd_ref(q, k, v, mask, do, operand_dtype=torch.float16)):
        tolerance.assert_close(got, want, f"tuned on a miss, dense mask: {name}")
    written = sorted(os.listdir(tmp_path / "cache"))
    assert written == ["best_config_retnet_MI355X_128_128_b1h2q256k256_c1.json",
                       "best_config_retnet_bwd_MI355X_128_128_b1h2q256k256_c1.json"], written
    logs = sorted(os.listdir(tmp_path / "logs"))
    assert logs == ["profile_result_ret_128_128.txt", "profile_result_ret_bwd_128_128.txt"], logs


def test_a_stored_ds_beyond_the_runtime_limit_is_timed_as_it_will_be_launched(monkeypatch):
    """The tuner grants a candidate the workspace the runtime would: above the runtime's dS limit the room for a stored dS
    is withheld in both, so such a candidate is timed on the chained passes it will actually run."""
    from attention_autotuner_amd.autotuner import library, runtime
    cfg = parity_matrix.ret_bwd_stored_ds_config(64, 128, 64, 32, 128, 128)
    lib_path = codegen.library_path(cfg)
    assert os.path.exists(lib_path)
    arrays = make_tensors("ret_bwd", 1, 2, 256, 256, 64, 128, "cuda")
    tuner = RetBwdTunner(ARCH, arrays, causal=True)
    lib = library.load(lib_path, "ret_bwd")
    full = int(lib.workspace_size(1, 2, 256, 256))
    ds_bytes = 2 * 1 * 2 * 256 * 256
    assert tuner._workspace(lib, cfg)[1] == full and full > ds_bytes
    monkeypatch.setattr(runtime, "MAX_DS_BYTES", ds_bytes - 1)
    assert tuner._workspace(lib, cfg)[1] == full - ds_bytes
    assert tuner.profile(lib_path, config=cfg) < base_tunner_failed() and tuner.verify(lib_path, config=cfg)


def base_tunner_failed():
    from attention_autotuner_amd.autotuner import base_tunner
    return base_tunner.FAILED
