"""Host-side checks that run without a GPU: wrapper text, hipcc compile for gfx950, exported symbols
versus include/aat_kernel_abi.h, failure handling of the compile driver and of the tuning cache."""
import ctypes
import json
import os
import re

import pytest
import torch

from attention_autotuner_amd.arch import MI355X
from attention_autotuner_amd.autotuner import AttnConfig, AttnTunner, Runtime, codegen, gfx950_space, library, prebuilt
from attention_autotuner_amd.autotuner import base_tunner

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "aat_kernel_abi.h")
ARCH = MI355X()


def _declared_symbols(op_macro):
    """Function names include/aat_kernel_abi.h declares for one operator."""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    common = text.split("#if defined(AAT_OP_ATTN)")[0]
    block = re.search(r"defined\(%s\)(.*?)(#elif|#endif)" % op_macro, text, flags=re.S).group(1)
    names = re.findall(r"\b([a-z_]+)\s*\(", common + block)
    return sorted(set(n for n in names if n not in ("defined",)))


def test_header_declares_the_reference_pair_for_every_operator():
    pair = ["abi_version", "config_string", "kernel_entry", "kernel_entry_ex", "profile", "profile_ex", "workspace_size"]
    assert _declared_symbols("AAT_OP_ATTN") == sorted(pair + ["kernel_entry_lse"])
    for macro in ("AAT_OP_RET", "AAT_OP_RET_BWD"):
        assert _declared_symbols(macro) == sorted(pair + ["kernel_entry_decay", "profile_decay"])
    # the attention backward has no reference signature to keep: only the extended entry points
    assert _declared_symbols("AAT_OP_ATTN_BWD") == ["abi_version", "config_string", "kernel_entry_ex", "profile_ex", "workspace_size"]
    # the recurrent form keeps the reference's own entry-point name (reference recurrent.h:427)
    assert _declared_symbols("AAT_OP_RET_RECURRENT") == ["abi_version", "config_string", "retnet_recurrent_fwd",
                                                         "retnet_recurrent_fwd_ex", "retnet_recurrent_fwd_noalloc",
                                                         "retnet_recurrent_profile", "retnet_recurrent_workspace_size",
                                                         "workspace_size"]


def test_wrapper_text_carries_the_configuration():
    cfg = gfx950_space.default_forward_config("attn", 128, 128, ARCH)
    src = codegen.render(cfg)
    for field in ("Br", "Bc", "Kd", "D", "Nthreads", "num_stages_qk", "num_stages_v"):
        assert f"constexpr int {field} = {getattr(cfg, field)};" in src
    assert 'extern "C" float profile(' in src and 'extern "C" int kernel_entry(' in src
    assert "int Seq_k, int Seq_q)" in src.split('extern "C" int kernel_entry(')[1].split("{")[0]   # reference order
    assert "int Seq_q, int Seq_k)" in src.split('extern "C" float profile(')[1].split("{")[0]
    cmd = codegen.hipcc_command("a.hip", "a.so", ARCH)
    assert "--offload-arch=gfx950" in cmd and "-packed-fp32-ops" in cmd


def test_shipping_set_is_built_and_exports_the_abi():
    cfgs = prebuilt.shipping_set(ARCH)
    assert cfgs
    macro = {"attn": "AAT_OP_ATTN", "ret": "AAT_OP_RET", "ret_bwd": "AAT_OP_RET_BWD", "attn_bwd": "AAT_OP_ATTN_BWD",
             "ret_recurrent": "AAT_OP_RET_RECURRENT"}
    assert {c.operation for c in cfgs} == set(macro)
    for cfg in cfgs:
        path = codegen.compile_config(cfg, ARCH, timeout=600)          # already built by build(); builds if not
        assert path and os.path.exists(path), cfg
        raw = ctypes.CDLL(path)
        for name in _declared_symbols(macro[cfg.operation]):
            assert hasattr(raw, name), (cfg, name)
        lib = library.load(path, cfg.operation)
        assert lib.abi_version() == 4
        assert lib.config_string().decode() == f"{cfg.operation}:{cfg}"
        if cfg.operation == "ret_recurrent":
            factors = 4 * (2048 // 32) * 5120                                         # one record per (head, chunk)
            assert lib.workspace_size(8, 4, 2048, 2048) == factors
            assert lib.retnet_recurrent_workspace_size(8, 4, 128, 64, 2048, 128) == factors
            # beyond 128 key dims: plus a second output-sized buffer for the passes that add
            assert lib.retnet_recurrent_workspace_size(8, 4, 256, 64, 2048, 256) == factors + 8 * 4 * 64 * 2048 * 4
            assert lib.retnet_recurrent_workspace_size(8, 4, 256, 64, 2000, 256) == 0     # unsupported shape
        elif cfg.operation == "attn_bwd":
            assert lib.workspace_size(2, 3, 256, 512) == 2 * 2 * 3 * 256 * 4      # lse2 + delta, fp32 per query row
        elif cfg.operation in ("ret", "ret_bwd"):       # the mask scan: 2 range ends per band of 32 query rows + a byte per 32 x 32 tile
            # a backward built with a stored dS adds the room for it: B*H*S_q*S_kv fp16
            ds = 2 if getattr(cfg, "ds_rows", 0) else 0
            assert lib.workspace_size(5, 3, 256, 512) == 768 + ds * 5 * 3 * 256 * 512      # 4 * 3 * 2 * 8 + 3 * 8 * 16 = 576, in units of 256
            assert lib.workspace_size(1, 1, 256, 256) == 256 + ds * 256 * 256              # rounded up to 256 bytes
            assert lib.workspace_size(1, 1, 256, 320) == 256                       # a length its dK kernel cannot tile: the scan alone
        elif getattr(cfg, "kv_splits", 1) == 1:
            assert lib.workspace_size(1, 1, 256, 256) == 0


def test_failed_compile_is_skipped_not_fatal(tmp_path):
    bad = AttnConfig(96, 64, 128, 128, 128, 64, 1, 1, 256, True).set_fuse_type("register")   # 96 rows / 4 waves: static_assert
    assert codegen.compile_config(bad, ARCH, str(tmp_path), timeout=120) is None
    logs = [f for f in os.listdir(tmp_path / "attn") if f.endswith(".log")]
    assert logs and "static assertion" in open(tmp_path / "attn" / logs[0]).read()
    with pytest.raises(Exception):
        Runtime(ARCH, bad, tmp_dir=str(tmp_path))
    good = gfx950_space.default_forward_config("attn", 64, 64, ARCH)
    # a configuration listed twice is built once (two compiles of one library in one process used to collide)
    res = codegen.compile_parallel([bad, good, good], ARCH, str(tmp_path), timeout=300)
    assert res[0] is None and res[1] and os.path.exists(res[1]) and res[2] == res[1]
    assert not [f for f in os.listdir(tmp_path / "attn") if ".tmp" in f]


def test_compile_timeout_yields_none(tmp_path):
    cfg = gfx950_space.default_forward_config("attn", 64, 64, ARCH)
    assert codegen.compile_config(cfg, ARCH, str(tmp_path), timeout=0.05) is None
    assert not [f for f in os.listdir(tmp_path / "attn") if f.endswith(".so")]


def _meta(dqk=128, dv=128, sq=2048, sk=2048):
    return [torch.empty(4, 32, sq, dqk, dtype=torch.float16, device="meta"),
            torch.empty(4, 32, sk, dqk, dtype=torch.float16, device="meta"),
            torch.empty(4, 32, sk, dv, dtype=torch.float16, device="meta")]


def test_cache_roundtrip_corruption_and_key(tmp_path, monkeypatch):
    base_tunner._memo.clear()
    t = AttnTunner(ARCH, _meta(), causal=True)
    t.cache_path = str(tmp_path)
    assert t.check_cache() is None
    cfg = gfx950_space.default_forward_config("attn", 128, 128, ARCH)
    t._write_cache(cfg)
    base_tunner._memo.clear()
    assert t.check_cache() == cfg
    name = os.path.basename(t._cache_file())
    assert name == "best_config_attention_MI355X_128_128_b4h32q2048k2048_c1.json"
    # a different problem (non-causal, other lengths) does not see that entry
    t2 = AttnTunner(ARCH, _meta(sq=256, sk=16384), causal=False)
    t2.cache_path = str(tmp_path)
    assert t2.check_cache() is None
    # the reference's file name is honoured as a fallback
    with open(tmp_path / "best_config_attention_128_128.json", "w") as f:
        json.dump(cfg.to_dict(), f)
    assert t2.check_cache() == cfg
    # corrupt files are ignored
    base_tunner._memo.clear()
    with open(t._cache_file(), "w") as f:
        f.write("{not json")
    os.remove(tmp_path / "best_config_attention_128_128.json")
    assert t.check_cache() is None
    # a cached tile that does not divide the problem is ignored
    t3 = AttnTunner(ARCH, _meta(sq=64, sk=2048), causal=True)
    t3.cache_path = str(tmp_path)
    with open(t3._cache_file(), "w") as f:
        json.dump(cfg.to_dict(), f)
    assert cfg.Br > 64 and t3.check_cache() is None


def test_validity_model_rejects_over_lds_and_over_register():
    over_lds = AttnConfig(128, 128, 256, 512, 256, 128, 2, 2, 256, True, waves_per_eu=1).set_fuse_type("register")
    assert gfx950_space.forward_lds_bytes(over_lds) > ARCH.smem_cap
    assert not gfx950_space.forward_valid(over_lds, ARCH)
    over_reg = AttnConfig(128, 64, 256, 512, 256, 64, 1, 1, 128, True, waves_per_eu=2).set_fuse_type("register")
    assert not gfx950_space.forward_valid(over_reg, ARCH)
    ok = gfx950_space.default_forward_config("attn", 128, 128, ARCH, 128, 128)
    assert gfx950_space.forward_valid(ok, ARCH) and ok.Br == 128
    assert gfx950_space.forward_lds_bytes(ok) == 2 * 64 * 128 * 2 * 2      # two K and two V buffers of 64 x 128 fp16
    big = gfx950_space.default_forward_config("attn", 128, 128, ARCH)
    assert gfx950_space.forward_lds_bytes(big) == 256 * (128 * 2 + 16)    # the output staging area dominates


def test_ops_refuse_cpu_tensors():
    import attention_autotuner_amd as aat
    q = torch.zeros(1, 1, 128, 64, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU only"):
        aat.flash_attn_func(q, q, q, ARCH)
    with pytest.raises(RuntimeError, match="GPU only"):
        aat.RetNetAttnFunc(q, q, q, torch.zeros(1, 128, 128, dtype=torch.float16), ARCH)
    x = torch.zeros(1, 1, 64, 32)
    with pytest.raises(RuntimeError, match="GPU only"):
        aat.retnet_recurrent_fwd(x, x, x, torch.ones(1, 32))


# ------------------------------------------------------------------------------ the tuning loop's guard
def test_verify_reference_math_matches_the_oracle_and_rejects_a_perturbed_output():
    """verify.py is torch math on whatever device its tensors live on: on the CPU its reference outputs agree
    with the oracle, an output equal to them passes, and one wrong element, a NaN or a scaled tensor fails."""
    from attention_autotuner_amd.autotuner import verify
    from oracle import ref_op
    g = torch.Generator().manual_seed(5)
    q, k = torch.randn(1, 2, 64, 64, generator=g).half(), torch.randn(1, 2, 96, 64, generator=g).half()
    v, do = torch.randn(1, 2, 96, 128, generator=g).half(), torch.randn(1, 2, 64, 128, generator=g).half()
    mask = torch.randn(2, 64, 96, generator=g).half()
    for causal in (False, True):
        want = ref_op.attention_ref(q, k, v, 0.2, causal)
        ref = verify.reference_outputs("attn", [q, k, v, None], scale=0.2, causal=causal)
        torch.testing.assert_close(ref[3], want, rtol=1e-5, atol=1e-5)
        arrays = [q, k, v, want.half()]
        assert verify.outputs_match(arrays, ref)
        for spoil in ("element", "nan", "scale"):
            bad = want.clone()
            if spoil == "element":
                bad[0, 1, 63, 5] += 0.05
            elif spoil == "nan":
                bad[0, 0, 0, 0] = float("nan")
            else:
                bad *= 1.05
            assert not verify.outputs_match([q, k, v, bad.half()], ref), (causal, spoil)
    o_ref, r_ref = ref_op.retnet_ref(q, k, v, mask, return_r=True)
    ref = verify.reference_outputs("ret", [q, k, v, mask, None, None])
    torch.testing.assert_close(ref[4], o_ref, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(ref[5], r_ref, rtol=1e-5, atol=1e-5)
    grads = ref_op.retnet_bwd_ref(q, k, v, mask, do, r_ref, operand_dtype=torch.float16)
    ref = verify.reference_outputs("ret_bwd", [q, k, v, mask, do, r_ref, None, None, None, None])
    for idx, gr in zip((6, 7, 8), grads):
        torch.testing.assert_close(ref[idx], gr, rtol=1e-5, atol=1e-5)
    outs = [q, k, v, mask, do, r_ref] + [t.half() for t in grads]
    assert verify.outputs_match(outs, ref)
    outs[7] = (grads[1] + 0.05 * (torch.arange(grads[1].numel()).view_as(grads[1]) == 77)).half()
    assert not verify.outputs_match(outs, ref)
    # the decay variant builds its mask from log2(gamma): gamma^(i + sk - sq - j) on and below the diagonal
    lg = torch.log2(torch.tensor([0.9, 0.5]))
    d = verify.decay_mask(lg, 4, 6)
    assert d.shape == (2, 4, 6) and d[0, 0, 2] == 1.0 and d[0, 0, 3] == 0.0 and abs(d[0, 3, 2].item() - 0.9 ** 3) < 1e-6
    assert abs(d[1, 2, 0].item() - 0.5 ** 4) < 1e-7


# ---------------------------------------------------------------------- the compiler's resource report
REMARKS = """
x.hip:2:1: remark: Function Name: _ZN3aat13ret_bwd_chainILi256ELi512ELi512ELi128ELi32ELi256ELi3ELi2ELNS_7BwdPassE0ELi1ELb1ELb0EEEvPKDF16_ [-Rpass-analysis=kernel-resource-usage]
x.hip:2:1: remark:     TotalSGPRs: 58 [-Rpass-analysis=kernel-resource-usage]
x.hip:2:1: remark:     VGPRs: 256 [-Rpass-analysis=kernel-resource-usage]
x.hip:2:1: remark:     AGPRs: 256 [-Rpass-analysis=kernel-resource-usage]
x.hip:2:1: remark:     ScratchSize [bytes/lane]: 2416 [-Rpass-analysis=kernel-resource-usage]
x.hip:2:1: remark:     Dynamic Stack: False [-Rpass-analysis=kernel-resource-usage]
x.hip:2:1: remark:     Occupancy [waves/SIMD]: 1 [-Rpass-analysis=kernel-resource-usage]
x.hip:2:1: remark:     SGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
x.hip:2:1: remark:     VGPRs Spill: 604 [-Rpass-analysis=kernel-resource-usage]
x.hip:2:1: remark:     LDS Size [bytes/block]: 0 [-Rpass-analysis=kernel-resource-usage]
x.hip:3:1: remark: Function Name: _ZN3aat13ret_bwd_chainILi256ELi512ELi512ELi128ELi32ELi256ELi3ELi2ELNS_7BwdPassE0ELi1ELb0ELb0EEEvPKDF16_ [-Rpass-analysis=kernel-resource-usage]
x.hip:3:1: remark:     VGPRs: 250 [-Rpass-analysis=kernel-resource-usage]
x.hip:3:1: remark:     ScratchSize [bytes/lane]: 16 [-Rpass-analysis=kernel-resource-usage]
"""


def test_resource_report_is_parsed_and_decides_what_the_tuner_times(tmp_path, monkeypatch):
    # a build that keeps its temporaries prints the same remarks with the source position behind "remark:"
    kept = codegen.parse_resource_usage("remark: a/b.h:83:0: Function Name: _Z1kv [-Rpass-analysis=kernel-resource-usage]\n"
                                        "remark: a/b.h:83:0:     VGPRs: 42 [-Rpass-analysis=kernel-resource-usage]\n"
                                        "remark: a/b.h:83:0:     ScratchSize [bytes/lane]: 16 [-Rpass-analysis=kernel-resource-usage]\n")
    assert kept == [{"kernel": "_Z1kv", "vgprs": 42, "scratch_bytes": 16}]
    usage = codegen.parse_resource_usage(REMARKS)
    assert [k["scratch_bytes"] for k in usage] == [2416, 16] and usage[0]["vgprs"] == 256 and usage[0]["vgpr_spills"] == 604
    assert usage[0]["occupancy"] == 1 and usage[0]["agprs"] == 256 and usage[0]["sgprs"] == 58
    assert codegen.template_bools(usage[0]["kernel"]) == [True, False] and codegen.template_bools(usage[1]["kernel"]) == [False, False]
    assert codegen.template_bools("_ZN3aat21flashattn_fwd_regfuseILi128ELi128ELi256ELi64ELi512ELi2ELi2ELi2ELb0ELb1ELb0ELb0EEEvPKDF16_") == [False, True, False, False]
    assert codegen.template_bools("_Z6kernelPf") == []
    assert [k["scratch_bytes"] for k in codegen.spilling_kernels(usage)] == [2416]          # 16 bytes are below the threshold
    assert codegen.spilling_kernels(usage, lambda name: not codegen.template_bools(name)[0]) == []
    assert codegen.spilling_kernels(None) == []
    # a decay tuner looks at the decay kernels of a library, a mask-tensor tuner at the others
    from attention_autotuner_amd.autotuner import RetBwdTunner
    from attention_autotuner_amd.benchmarks.tune import make_tensors
    arrays = make_tensors("ret_bwd", 1, 2, 256, 256, 256, 512, "meta")
    assert RetBwdTunner(ARCH, arrays, decay=True)._kernel_matters(usage[0]["kernel"])
    assert not RetBwdTunner(ARCH, arrays, causal=True)._kernel_matters(usage[0]["kernel"])
    assert RetBwdTunner(ARCH, arrays, causal=True)._kernel_matters("_ZN3aat18ret_bwd_dk_from_dsILi256ELi128ELi64ELi256ELi2ELi2EEEvPKDF16_S2_PDF16_iiiiPKiii")
    attn = AttnTunner(ARCH, make_tensors("attn", 1, 2, 256, 256, 128, 128, "meta"), causal=True)
    name = "_ZN3aat21flashattn_fwd_regfuseILi128ELi128ELi256ELi64ELi512ELi2ELi2ELi2ELi64ELb0ELb%dELb0ELb0ELb%dEEEvPKDF16_"
    assert attn._kernel_matters(name % (1, 0)) and not attn._kernel_matters(name % (0, 0))
    assert not attn._kernel_matters(name % (1, 1))            # the paired causal variant is launched only from a build that does not spill
    # every library of the shipping set carries its report, with one entry per kernel it holds
    cfg = gfx950_space.default_forward_config("attn", 128, 128, ARCH)
    report = codegen.resource_usage(codegen.library_path(cfg))
    assert report and all("vgprs" in k and "scratch_bytes" in k for k in report)
    assert any("flashattn_fwd_regfuse" in k["kernel"] for k in report)


def test_tune_skips_a_candidate_the_compiler_reports_as_spilling(tmp_path, monkeypatch):
    """The loop never times (here: never even loads) a library whose report shows a spilled working set."""
    from attention_autotuner_amd.benchmarks.tune import make_tensors
    tuner = AttnTunner(ARCH, make_tensors("attn", 1, 2, 256, 256, 128, 128, "meta"))
    tuner.cache_path = str(tmp_path / "cache")
    good = AttnConfig(128, 64, 128, 128, 128, 64, 2, 2, 256, True, waves_per_eu=2).set_fuse_type("register")
    bad = AttnConfig(128, 32, 128, 128, 128, 32, 2, 2, 256, True, waves_per_eu=2).set_fuse_type("register")
    monkeypatch.setattr(tuner, "get_tuned_configs", lambda: [good, bad])
    monkeypatch.setattr(tuner, "compile_parallel", lambda cfgs, timeout=None: [base_tunner.CompileResult(c, str(c)) for c in cfgs])
    reports = {str(good): [{"kernel": "_Z1aILb0ELb0ELb0ELb0EEvPf", "scratch_bytes": 0}],
               str(bad): [{"kernel": "_Z1aILb0ELb0ELb0ELb0EEvPf", "scratch_bytes": 900}]}
    monkeypatch.setattr(codegen, "resource_usage", lambda lib: reports[lib])
    timed = []
    monkeypatch.setattr(tuner, "profile", lambda lib, config=None: timed.append(lib) or 1.0)
    monkeypatch.setattr(tuner, "verify", lambda lib, config=None: True)
    best = tuner.tune(log_path=str(tmp_path / "logs"), use_cache=False)
    assert best == good and timed == [str(good)] and tuner.rejected_spills == {bad: 900}
    log = (tmp_path / "logs" / "profile_result_attn_128_128.txt").read_text()
    assert "not timed (compiler reports 900 bytes/lane of scratch): " + str(bad) in log


LISTING = """
_ZN3aat15ret_fwd_regfuseILi128ELi128EEEvPKDF16_:
	;;#ASMSTART
	; aat: accumulation registers addressed by number
	;;#ASMEND
	global_load_dwordx4 a[2:5], v[6:7], off
	;;#ASMSTART
	v_mfma_f32_32x32x16_f16 a[0:15], v[0:3], v[4:7], a[0:15]
	;;#ASMEND
	v_accvgpr_read_b32 v66, a14
	s_endpgm
_ZN3aat15ret_fwd_regfuseILi256ELi512EEEvPKDF16_:
	;;#ASMSTART
	; aat: accumulation registers addressed by number
	;;#ASMEND
	;;#ASMSTART
	v_accvgpr_write_b32 a[255], 0
	;;#ASMEND
	v_add_f32_e32 v1, v2, v3              ; a12 in a comment is no operand
	s_endpgm
_ZN3aat21flashattn_fwd_regfuseILi128EEEvPKDF16_:
	v_mfma_f32_32x32x16_f16 a[0:15], v[0:3], v[4:7], a[0:15]
	;;#ASMSTART
	v_accvgpr_read_b32 v5, a7
	;;#ASMEND
	v_accvgpr_read_b32 v1, a3
	s_endpgm
"""


def test_a_build_whose_compiler_uses_the_numbered_accumulation_registers_is_rejected(tmp_path):
    """Kernels that address accumulation registers by number (utils/acc_file.h) are only sound when the compiler keeps
    nothing of its own in that file.  The listing check: a kernel that names such registers inside its asm statements and
    also in compiler-emitted instructions is reported; one that does only the former, or one without the mark (ordinary
    MFMA code, accumulators handed to asm statements as operands), is not.  And a configuration known to provoke it (two row groups per wave: the fragments no longer fit
    the vector registers) fails to build, with the reason in its log."""
    assert codegen.foreign_accumulator_use(LISTING) == {"_ZN3aat15ret_fwd_regfuseILi128ELi128EEEvPKDF16_": 2}
    from attention_autotuner_amd.autotuner.configs import RetConfig
    tight = RetConfig(256, 128, 128, 128, 128, 128, 1, 1, 1, 256, True, waves_per_eu=1).set_fuse_type("register")
    assert codegen.may_hold_numbered_accumulators(tight)
    assert not codegen.may_hold_numbered_accumulators(gfx950_space.default_forward_config("attn", 128, 128, ARCH))
    assert codegen.compile_config(tight, ARCH, build_dir=str(tmp_path), force=True) is None
    log = open(codegen.library_path(tight, str(tmp_path))[:-3] + ".log").read()
    assert "accumulation registers" in log and "ret_fwd_regfuse" in log
    assert not [f for f in os.listdir(os.path.dirname(codegen.library_path(tight, str(tmp_path)))) if f.endswith((".so", ".d"))]
    # the shipped one-wave configuration of the same kernel passes the check
    fine = gfx950_space.default_forward_config("ret", 256, 512, ARCH)
    assert fine.waves_per_eu == 1 and fine.fuse_type == "register" and os.path.exists(codegen.library_path(fine))


def test_no_cached_winner_keeps_its_working_set_in_scratch():
    """Every configuration in the shipped tuning cache is built, carries the compiler's report, and none of the kernels a
    launch of it can take keeps more than the tolerated few dwords in scratch memory.  (The paired causal variant of the
    attention forward is the one exception the wrapper handles itself: it is only launched from a build in which the
    runtime reports no scratch for it.)"""
    import glob
    from attention_autotuner_amd.autotuner.configs import supported_configs
    entries = sorted(glob.glob(os.path.join(base_tunner.DEFAULT_CACHE_DIR, "best_config_*.json")))
    assert len(entries) >= 18
    for path in entries:
        with open(path) as f:
            dd = json.load(f)
        cfg = supported_configs[dd["operation"]].from_dict(dd)
        decay = "_decay_" in os.path.basename(path)           # the entry of a decay-mask problem launches the DECAY kernels
        usage = codegen.resource_usage(codegen.library_path(cfg))
        assert usage, cfg

        def launched(name):
            flags = codegen.template_bools(name)
            if "flashattn_fwd_regfuse" in name and len(flags) == 5:          # <..., PIPE, CAUSAL, SPLIT, PERSIST, PAIR>
                return not flags[4]
            if "ret_fwd" in name and flags:                                  # <..., DECAY>
                return flags[-1] == decay
            if "ret_bwd_chain" in name and len(flags) == 2:                  # <..., PASS, WPE, DECAY, DS_OUT>
                return flags[0] == decay
            return True
        assert codegen.spilling_kernels(usage, launched) == [], (os.path.basename(path), codegen.spilling_kernels(usage, launched))


def test_without_tuning_a_miss_launches_the_entry_of_the_nearest_problem(tmp_path, monkeypatch):
    """AAT_TUNE_ON_MISS=0: same operator, head sizes and mask walk; nearest lengths first; tiles must divide the problem."""
    from attention_autotuner_amd.ops import _resolve
    base_tunner._memo.clear()
    near = AttnConfig(Br=128, Bc=64, Kd=128, D=128, Nthreads=256)
    far = AttnConfig(Br=256, Bc=128, Kd=128, D=128, Nthreads=256)
    other_walk = AttnConfig(Br=64, Bc=64, Kd=128, D=128, Nthreads=128)

    def entry(name, cfg):
        with open(tmp_path / name, "w") as f:
            json.dump(cfg.to_dict(), f)
    entry("best_config_attention_MI355X_128_128_b4h32q2048k2048_c0.json", near)
    entry("best_config_attention_MI355X_128_128_b1h32q256k16384_c0.json", far)
    entry("best_config_attention_MI355X_128_128_b4h32q1024k1024_c1.json", other_walk)
    entry("best_config_attention_MI355X_64_64_b4h32q1024k1024_c0.json", other_walk)
    entry("best_config_attention_bwd_MI355X_128_128_b4h32q1024k1024_c0.json", other_walk)
    monkeypatch.setenv("AAT_TUNE_ON_MISS", "0")
    default = gfx950_space.default_forward_config("attn", 128, 128, ARCH)

    def resolved(**kw):
        t = AttnTunner(ARCH, _meta(**kw), causal=False)
        t.cache_path = str(tmp_path)
        assert t.check_cache() is None
        return _resolve.resolve(t, lambda: default), t

    cfg, t = resolved(sq=1024, sk=1024)
    assert cfg == near and t.check_cache() == near        # and the process remembers it for this problem
    assert resolved(sq=256, sk=8192)[0] == far
    assert resolved(sq=384, sk=8192)[0] == near           # 256-row blocks do not divide 384 rows: the next nearest
    assert resolved(sq=64, sk=2048)[0] == default         # the one entry within reach does not fit: the built-in default
    base_tunner._memo.clear()


def test_an_operator_resolves_a_problem_once_and_again_after_a_tuning_result_is_written(tmp_path, monkeypatch):
    from attention_autotuner_amd.ops import _resolve
    base_tunner._memo.clear()
    monkeypatch.setattr(_resolve, "Runtime", lambda arch, cc: ("runtime of", cc))      # no library is built or loaded here
    monkeypatch.setenv("AAT_TUNE_ON_MISS", "0")
    default = gfx950_space.default_forward_config("attn", 128, 128, ARCH)
    tuned = AttnConfig(Br=128, Bc=64, Kd=128, D=128, Nthreads=256)
    built = []

    def make():
        t = AttnTunner(ARCH, _meta(), causal=False)
        t.cache_path = str(tmp_path)
        built.append(t)
        return t
    key = ("attn", ARCH.name, 4, 32, 2048, 2048, 128, 128, False)
    cc, rt = _resolve.planned(key, make, lambda: default)
    assert cc == default and rt == ("runtime of", default) and len(built) == 1
    assert _resolve.planned(key, make, lambda: default)[0] is cc and len(built) == 1      # one dictionary lookup, no tuner
    built[0]._write_cache(tuned)
    assert _resolve.planned(key, make, lambda: default)[0] == tuned and len(built) == 2
    base_tunner._memo.clear()
