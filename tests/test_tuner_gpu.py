"""The tuning loop on the GPU: times prebuilt candidates, checks the winner against torch math before
caching it, and discards a candidate whose output is wrong (nothing is compiled inside these tests:
the candidate lists are restricted to libraries of the shipping set)."""
import json
import os

import pytest

import parity_matrix
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
