"""The restated reference search space must reproduce the reference's published tuning logs."""
import os
import re

import pytest
import torch

from attention_autotuner_amd.arch import MI355X
from reference_space import A100, RTX4090
from attention_autotuner_amd.autotuner import AttnTunner, RetTunner, RetBwdTunner, AttnConfig, RetConfig, RetBwdConfig, gfx950_space
from attention_autotuner_amd.autotuner.configs import balanced_wave_split, supported_configs

GOLD = os.path.join(os.path.dirname(__file__), "golden", "tuning_logs")


def _log_configs(path):
    """Config lines of a log, in order, up to the 'best config' trailer; plus the best line."""
    lines = open(path).read().splitlines()
    cut = lines.index("best config: ")
    cfgs = [l for l in lines[:cut] if l.startswith("Config(")]
    lat = [float(l) for l in lines[:cut] if re.fullmatch(r"[0-9.eE+-]+", l)]
    return cfgs, lat, lines[cut + 1], float(lines[cut + 2])


def _fake_arrays(dqk, dv):
    q = torch.empty(4, 8, 2048, dqk, dtype=torch.float16, device="meta")
    k = torch.empty(4, 8, 2048, dqk, dtype=torch.float16, device="meta")
    v = torch.empty(4, 8, 2048, dv, dtype=torch.float16, device="meta")
    return [q, k, v]


EXACT = [
    ("A100", A100, "attn", 256, 256, 84),
    ("RTX4090", RTX4090, "attn", 256, 128, 68),
    ("RTX4090", RTX4090, "attn", 256, 256, 48),
    ("RTX4090", RTX4090, "attn", 256, 64, 80),
    ("RTX4090", RTX4090, "attn", 64, 64, 84),
]


@pytest.mark.parametrize("name,arch_cls,op,dqk,dv,count", EXACT)
def test_enumeration_matches_published_log(name, arch_cls, op, dqk, dv, count):
    cfgs, lat, best, best_ms = _log_configs(os.path.join(GOLD, name, f"profile_result_{op}_{dqk}_{dv}.txt"))
    assert len(cfgs) == count == len(lat)
    mine = [repr(c) for c in AttnTunner(arch_cls(), _fake_arrays(dqk, dv)).get_tuned_configs()]
    assert mine == cfgs
    # the logged best is the argmin of the logged latencies
    assert best == cfgs[lat.index(min(lat))] and best_ms == min(lat)


def test_stale_attn_128_128_log_is_superset_minus_removed_rule():
    cfgs, _, _, _ = _log_configs(os.path.join(GOLD, "RTX4090", "profile_result_attn_128_128.txt"))
    mine = [repr(c) for c in AttnTunner(RTX4090(), _fake_arrays(128, 128)).get_tuned_configs()]
    extra = [c for c in cfgs if c not in mine]
    assert [c for c in cfgs if c in mine] == mine           # same order on the common part
    assert len(extra) == 4
    for c in extra:                                          # rows a later rule removed
        assert "Br=32" in c and "BlockKSmem=32," in c and "Nthreads=256" in c


def test_stale_retnet_log_format_and_membership():
    cfgs, lat, best, best_ms = _log_configs(os.path.join(GOLD, "A100", "profile_result_ret_256_256.txt"))
    assert len(cfgs) == 42 == len(lat)
    mine = [repr(c) for c in RetTunner(A100(), _fake_arrays(256, 256) + [None]).get_tuned_configs()]
    assert len(mine) == 76
    assert set(cfgs) <= set(mine)
    assert best in cfgs and best_ms == min(lat)


def test_reference_bwd_space_is_empty_at_benchmark_shape():
    # dqk=256, dv=512: every (Br, Bc >= 64) tile needs more shared memory than an A100 has
    t = RetBwdTunner(A100(), _fake_arrays(256, 512))
    assert t.get_tuned_configs() == []
    t2 = RetBwdTunner(A100(), _fake_arrays(256, 256))
    got = t2.get_tuned_configs()
    assert got and all(c.Br >= 64 and c.Bc >= 64 for c in got)
    # the 256-thread config the reference's runtime test hand-picks is a member of its own space
    assert any((c.Br, c.Bc, c.mmawarpsN, c.mmawarpsN_dk, c.mmawarpsN_dv, c.mmawarpsN_dq, c.Nthreads) == (64, 64, 2, 4, 4, 4, 256) for c in got)


def test_balanced_wave_split_known_values():
    assert balanced_wave_split(4, 32, 32) == (2, 2)
    assert balanced_wave_split(8, 32, 32) is None
    assert balanced_wave_split(4, 64, 256) == (1, 4)


def test_config_text_forms_and_roundtrip():
    c = AttnConfig(128, 128, 256, 256, 256, 32, 1, 2, 256, True).set_fuse_type("register")
    assert repr(c) == ("Config(fuse_type=register, Br=128, Bc=128, BlockKSmem=256, BlockKSmem2=32, num_stages_qk=1, "
                       "num_stages_v=2, Nthreads=256, unrollLastIter=1)")
    assert str(c) == "register_128_128_256_256_256_32_1_2_256_1"
    s = AttnConfig(32, 32, 256, 256, 256, 32, 1, 1, 128, True).set_fuse_type("shared")
    assert repr(s).endswith("unrollLastIter=1,warps_mma1_n=2,warp_mma_n=4)")
    r = RetConfig(128, 64, 256, 256, 256, 64, 1, 1, 1, 256, True).set_fuse_type("register")
    assert repr(r) == ("Config(fuse_type=register, Br=128, Bc=64, BlockKSmem=256, BlockKSmem2=64, num_stages_qk=1, "
                       "num_stages_mask=1, num_stages_v=1, Nthreads=256, unrollLastIter=1)")
    b = RetBwdConfig(64, 64, 256, 256, 2, 4, 4, 4)
    assert str(b).startswith("ret_bwd_64_64_256_256_2_4_4_4_256_1_256_1_1_1_1_1")
    for cfg in (c, s, r, b):
        back = supported_configs[cfg.operation].from_dict(cfg.to_dict())
        assert back == cfg and repr(back) == repr(cfg) and str(back) == str(cfg)
        assert back.template_dir and os.path.isdir(back.template_dir)
    w = AttnConfig(128, 64, 128, 128, 128, 64, 2, 2, 256, True, waves_per_eu=2).set_fuse_type("register")
    assert str(w).endswith("_w2") and "waves_per_eu=2" in repr(w)
    # attention backward: the row kernel's own register budget is part of the key and of the log line,
    # and records written before the knob existed read back with both kernels on the same budget
    from attention_autotuner_amd.autotuner.configs import AttnBwdConfig
    a = AttnBwdConfig(128, 64, 128, 128, 256, 2, row_waves_per_eu=2)
    assert str(a) == "attn_bwd_128_64_128_128_256_2_rw2" and repr(a).endswith("num_stages_qk=2, row_waves_per_eu=2)")
    back = AttnBwdConfig.from_dict(a.to_dict())
    assert back == a and str(back) == str(a) and back.row_waves_per_eu == 2
    mixed = AttnBwdConfig(128, 64, 128, 128, 256, 2, row_waves_per_eu=2, row_Bc=32)
    assert str(mixed) == "attn_bwd_128_64_128_128_256_2_rw2_rb32" and repr(mixed).endswith("row_waves_per_eu=2, row_Bc=32)")
    assert AttnBwdConfig.from_dict(mixed.to_dict()) == mixed and gfx950_space.attn_backward_valid(mixed, MI355X())
    assert not gfx950_space.attn_backward_valid(AttnBwdConfig(128, 64, 128, 128, 256, 2, row_Bc=32), MI355X())   # only with a budget of its own
    plain = AttnBwdConfig(128, 64, 128, 128, 256, 2)
    assert str(plain) == "attn_bwd_128_64_128_128_256_2" and plain.row_waves_per_eu == 1
    old = {k: v for k, v in plain.to_dict().items() if k not in ("row_waves_per_eu", "row_Bc")}
    assert AttnBwdConfig.from_dict(old) == plain
    arch = MI355X()
    assert gfx950_space.attn_backward_valid(a, arch)
    assert not gfx950_space.attn_backward_valid(AttnBwdConfig(128, 64, 128, 128, 256, 3, row_waves_per_eu=2), arch)   # two 99 KB blocks
    assert not gfx950_space.attn_backward_valid(AttnBwdConfig(128, 32, 256, 256, 256, 2, row_waves_per_eu=2), arch)  # registers


def test_mi355x_space_is_valid_and_nonempty():
    arch = MI355X()
    for dqk, dv in ((64, 64), (128, 128), (256, 256), (256, 512)):
        cfgs = AttnTunner(arch, _fake_arrays(dqk, dv)).get_tuned_configs()
        reg = [c for c in cfgs if c.fuse_type == "register"]
        shared = [c for c in cfgs if c.fuse_type == "shared"]
        assert shared, (dqk, dv)
        # d_v = 512 puts 256 accumulator registers on every lane of a register-fused wave: such candidates are
        # enumerated (the tuning loop rejects them from the compiler's resource report) but never a default
        assert reg, (dqk, dv)
        assert all(gfx950_space.forward_likely_spills(c) for c in reg) == (dv == 512), (dqk, dv)
        assert gfx950_space.default_forward_config("attn", dqk, dv, arch).fuse_type == ("shared" if dv == 512 else "register")
        for c in cfgs:
            if c.fuse_type == "register":
                assert c.Br % (32 * (c.Nthreads // 64)) == 0      # every wave owns whole 32-row groups
            else:
                nw = c.Nthreads // 64
                assert nw % c.warps_mma1_n == 0 and nw % c.warps_mma_n == 0
                assert c.Bc % (32 * c.warps_mma1_n) == 0 and dv % (32 * c.warps_mma_n) == 0
            assert c.BlockKSmem == dqk and c.Bc % c.BlockKSmem2 == 0
            if c.BlockKSmem2 != c.Bc:     # units inside a kv tile: plain register-fused schedule, two or more row groups per wave
                assert c.fuse_type == "register" and not c.sw_pipeline and (c.num_stages_qk, c.num_stages_v) == (2, 2)
                assert c.BlockKSmem2 % 32 == 0 and c.Br // (c.Nthreads // 64) >= 64
    with pytest.raises(RuntimeError):
        AttnTunner(A100(), _fake_arrays(64, 64)).tune()
