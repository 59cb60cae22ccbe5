"""The cost model that prunes the tuning search (the reference exports (configuration, cycles) pairs for such
a model, python/tests/export_costmodel_config.py:31-56, and never reads them back): fitted on one recorded
tuning run of an MI355X, it must keep the measured winner of runs it has not seen."""
import os

import numpy as np
import pytest
import torch

from attention_autotuner_amd.arch import MI355X
from attention_autotuner_amd.autotuner import AttnConfig, AttnTunner, costmodel

LOGS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tuning_logs", "MI355X")
RUNS = {                                                  # file -> (shape, causal)
    "attn_b4h32q2048k2048_c0_128_128.txt": ((4, 32, 2048, 2048), False),
    "attn_b4h32q2048k2048_c1_128_128.txt": ((4, 32, 2048, 2048), True),
    "attn_b8h16q1024k1024_c0_128_128.txt": ((8, 16, 1024, 1024), False),
    "attn_b2h32q4096k4096_c1_128_128.txt": ((2, 32, 4096, 4096), True),
    # the headline problems searched in full again after later kernel changes (walk order, wave priority): the model
    # fitted on the first run has seen neither the kernels nor the timings of these
    "attn_b4h32q2048k2048_c0_128_128_later.txt": ((4, 32, 2048, 2048), False),
    "attn_b4h32q2048k2048_c1_128_128_later.txt": ((4, 32, 2048, 2048), True),
}
# ... and again with the candidates that work a kv tile through in units (two 32-row groups per wave, Br up to 512) and,
# for the long-kv problem, the kv-splitting candidates: new kernels, new winners
RUNS_WITH_UNITS = {
    "attn_b4h32q2048k2048_c0_128_128_units.txt": ((4, 32, 2048, 2048), False),
    "attn_b4h32q2048k2048_c1_128_128_units.txt": ((4, 32, 2048, 2048), True),
    "attn_b1h32q256k16384_c0_128_128_units.txt": ((1, 32, 256, 16384), False),
    # searched in full once more after the operand rings changed their wait order: the causal winner moved to 512-row blocks
    "attn_b4h32q2048k2048_c0_128_128_units2.txt": ((4, 32, 2048, 2048), False),
    "attn_b4h32q2048k2048_c1_128_128_units2.txt": ((4, 32, 2048, 2048), True),
}
EXPORTS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "costmodel_export")


def _samples(name):
    shape, causal = {**RUNS, **RUNS_WITH_UNITS}[name]
    return costmodel.samples_from_tuning_log(os.path.join(LOGS, name), "attn", 128, 128, shape, causal)


def test_log_lines_parse_back_into_the_configurations_that_wrote_them():
    cfg = AttnConfig(128, 32, 128, 128, 128, 32, 2, 1, 256, True, waves_per_eu=3).set_fuse_type("register")
    back = costmodel.config_from_log_line(repr(cfg), "attn", 128, 128)
    assert str(back) == str(cfg) and back.waves_per_eu == 3 and back.fuse_type == "register"
    shared = AttnConfig(64, 64, 128, 128, 128, 64, 2, 2, 256, True, 2, 4, waves_per_eu=2)
    shared.fuse_type = "shared"
    back = costmodel.config_from_log_line(repr(shared), "attn", 128, 128)
    assert str(back) == str(shared) and (back.warps_mma1_n, back.warps_mma_n) == (2, 4)
    split = AttnConfig(256, 64, 128, 128, 128, 64, 2, 2, 512, True, waves_per_eu=2, kv_splits=8).set_fuse_type("register")
    assert costmodel.config_from_log_line(repr(split), "attn", 128, 128).kv_splits == 8
    runs = _samples("attn_b4h32q2048k2048_c0_128_128.txt")
    assert len(runs) > 150 and all(0.2 < ms < 5 for *_, ms in runs)
    assert min(runs, key=lambda s: s[3])[0].Br == 256          # the recorded winner of the headline problem


def test_fit_recovers_a_known_linear_law():
    rng = np.random.default_rng(0)
    truth = np.array([3e-7, 2e-7, 1e-6, 4e-7, 2e-4, 1e-2, 1e-6, 0.05])
    cfgs = [s[0] for s in _samples("attn_b4h32q2048k2048_c0_128_128.txt")]
    shape = (4, 32, 2048, 2048)
    data = [(c, shape, False, float(truth @ costmodel.features(c, shape)) * (1 + 0.002 * rng.standard_normal())) for c in cfgs]
    model = costmodel.CostModel().fit(data, ridge=1e-9)
    pred = np.array([model.predict(c, shape) for c in cfgs])
    want = np.array([d[3] for d in data])
    assert np.abs(pred - want).max() <= 0.02 * want.max()
    assert model.rank_of_best(data) <= 2
    again = costmodel.CostModel.from_dict(model.to_dict())
    assert again.predict(cfgs[0], shape) == model.predict(cfgs[0], shape)
    with pytest.raises(ValueError):
        costmodel.CostModel.from_dict({"features": ["other"], "weights": [1.0]})


def test_model_fitted_on_one_run_keeps_the_winner_of_the_others():
    model = costmodel.CostModel().fit(_samples("attn_b4h32q2048k2048_c0_128_128.txt"))
    for name in RUNS:
        runs = _samples(name)
        times = np.array([s[3] for s in runs])
        pred = np.array([model.predict(*s[:3]) for s in runs])
        keep = np.argsort(pred)[:max(AttnTunner.keep_min, int(len(runs) * AttnTunner.keep_fraction + 0.999))]
        assert model.rank_of_best(runs) < len(keep), name                  # the measured winner survives the cut
        assert times[keep].min() == times.min(), name
        assert np.corrcoef(pred, times)[0, 1] > 0.8, name                  # and the model follows the measurements overall


def test_shipped_model_is_the_fit_on_exported_cycles_and_keeps_every_recorded_winner():
    """The model next to the tuning cache is fitted on the cycle counts of benchmarks/export_costmodel_config.py (three
    problems: the headline, its causal variant, the long-kv shape with its kv-splitting candidates; candidates the
    compiler reports as spilling left out, as in the tuning loop).  Ranking by counted cycles must keep the measured
    winner of every recorded tuning run -- timed in milliseconds on other boxes, six of them with kernels older than the
    export."""
    exports = sorted(os.path.join(EXPORTS, f) for f in os.listdir(EXPORTS) if f.endswith(".json"))
    assert len(exports) == 3
    samples = [s for path in exports for s in costmodel.samples_from_export(path, max_scratch_bytes=64)]
    assert len(samples) > 700 and any(getattr(s[0], "kv_splits", 1) > 1 for s in samples) and any(s[2] for s in samples)
    model = costmodel.CostModel(unit="cycles").fit(samples)
    shipped = costmodel.CostModel.load(os.path.join(AttnTunner(MI355X(), _meta(4, 32, 2048)).cache_path, "costmodel_attn.json"))
    np.testing.assert_allclose(shipped.weights, model.weights, rtol=1e-6)
    assert shipped.unit == "cycles"
    for name in list(RUNS) + list(RUNS_WITH_UNITS):
        runs = _samples(name)
        times = np.array([s[3] for s in runs])
        pred = np.array([shipped.predict(*s[:3]) for s in runs])
        keep = np.argsort(pred)[:max(AttnTunner.keep_min, int(len(runs) * AttnTunner.keep_fraction + 0.999))]
        assert times[keep].min() == times.min(), (name, shipped.rank_of_best(runs))
        assert np.corrcoef(pred, times)[0, 1] > 0.8, name
    # the spilling candidates are in the export (ten times the cycles of the rest) and would be all a fit sees
    everything = [s for path in exports for s in costmodel.samples_from_export(path)]
    assert len(everything) > len(samples) + 100


def _meta(b, h, s, d=128):
    return [torch.empty(b, h, s, d, dtype=torch.float16, device="meta") for _ in range(4)]


def test_tuner_prunes_with_the_shipped_model_and_not_without(monkeypatch):
    tuner = AttnTunner(MI355X(), _meta(4, 32, 2048), causal=True)
    assert tuner.cost_model is not None
    cfgs = [c for c in tuner.get_tuned_configs() if tuner._fits_problem(c)]
    kept = tuner.prune(cfgs)
    assert len(kept) == max(tuner.keep_min, int(len(cfgs) * tuner.keep_fraction + 0.999)) and len(kept) + len(tuner.pruned) == len(cfgs)
    winner = min(_samples("attn_b4h32q2048k2048_c1_128_128.txt"), key=lambda s: s[3])[0]
    assert str(winner) in {str(c) for c in kept}
    few = cfgs[:tuner.keep_min]
    assert tuner.prune(few) == few                                          # nothing to gain on a handful
    monkeypatch.setenv("AAT_TUNE_PRUNE", "0")
    exhaustive = AttnTunner(MI355X(), _meta(4, 32, 2048), causal=True)
    assert exhaustive.cost_model is None and exhaustive.prune(cfgs) == cfgs


@pytest.mark.gpu
def test_cycle_exporter_counts_prebuilt_candidates_in_the_reference_tuple_layout(tmp_path):
    """benchmarks/export_costmodel_config.py end to end on a few libraries that are already built: one rocprofv3 counter
    run, one record per candidate in the tuple layout of reference python/tests/export_costmodel_config.py:31-56
    (``Nwarps`` there counts 32-lane warps, here 64-lane waves), cycles that a fit can read back."""
    import json
    import subprocess
    import sys
    out = tmp_path / "export.json"
    dims = (1, 8, 512, 512, 128, 128)
    env = dict(os.environ, AAT_NO_JIT="1", TMPDIR=str(tmp_path))
    done = subprocess.run([sys.executable, "-m", "attention_autotuner_amd.benchmarks.export_costmodel_config", "attn",
                           *map(str, dims), "--only-built", "--limit", "4", "--out", str(out)],
                          capture_output=True, text=True, timeout=300, env=env,
                          cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-2000:]
    records = json.loads(out.read_text())
    assert len(records) == 4
    b, h, sq, sk, dqk, dv = dims
    for r in records:
        c = r["config"]
        nw = c["Nthreads"] // 64
        w1n, w2n = (c["warps_mma1_n"], c["warps_mma_n"]) if c["fuse_type"] == "shared" else (1, 1)
        assert r["cost_model_config"] == [[sq, sk, dqk, dv], [c["Br"], c["Bc"], c["BlockKSmem"], c["D"]],
                                          [c["Br"] // (nw // w1n), c["Bc"] // w1n, 16], [c["Br"] // (nw // w2n), c["D"] // w2n, 16], b, h]
        # 1 x 8 x 512 x 512 x (128 + 128) x 2 flop at no more than 2.5 PFLOP/s and 2.4 GHz, and nowhere near a millisecond
        assert 1000 < r["cycles"] < 2_000_000 and r["causal"] is False
        assert r["lds_bytes"] > 0 and r["registers"] > 0
    samples = costmodel.samples_from_export(str(out))
    assert [s[1] for s in samples] == [(b, h, sq, sk)] * 4 and all(s[3] == r["cycles"] for s, r in zip(samples, records))
    assert np.isfinite(costmodel.CostModel(unit="cycles").fit(samples).weights).all()


# ---- RetNet forward and backward spaces -----------------------------------------------------------------
RET_RUNS = {                                              # file -> (operator, (B, H, Sq, Sk, d_qk, d_v), causal walk)
    "ret_b4h8q2048k2048_c0_256_512.txt": ("ret", (4, 8, 2048, 2048, 256, 512), False),
    "ret_b4h8q2048k2048_c1_256_512.txt": ("ret", (4, 8, 2048, 2048, 256, 512), True),
    "ret_decay_b4h8q2048k2048_c1_256_512.txt": ("ret", (4, 8, 2048, 2048, 256, 512), True),
    "ret_b4h8q2048k2048_c1_128_128.txt": ("ret", (4, 8, 2048, 2048, 128, 128), True),
    "ret_b4h8q2048k2048_c1_256_256.txt": ("ret", (4, 8, 2048, 2048, 256, 256), True),
    "ret_bwd_b4h8q2048k2048_c0_256_512.txt": ("ret_bwd", (4, 8, 2048, 2048, 256, 512), False),
    "ret_bwd_b4h8q2048k2048_c1_256_512.txt": ("ret_bwd", (4, 8, 2048, 2048, 256, 512), True),
    "ret_bwd_decay_b4h8q2048k2048_c1_256_512.txt": ("ret_bwd", (4, 8, 2048, 2048, 256, 512), True),
    "ret_bwd_b4h8q2048k2048_c1_128_128.txt": ("ret_bwd", (4, 8, 2048, 2048, 128, 128), True),
    "ret_bwd_b4h8q2048k2048_c1_256_256.txt": ("ret_bwd", (4, 8, 2048, 2048, 256, 256), True),
}


def _ret_samples(name):
    op, (b, h, sq, sk, dqk, dv), causal = RET_RUNS[name]
    return costmodel.samples_from_tuning_log(os.path.join(LOGS, name), op, dqk, dv, (b, h, sq, sk), causal)


def _survives(model, runs, tuner_cls):
    times = np.array([s[3] for s in runs])
    pred = np.array([model.predict(*s[:3]) for s in runs])
    keep = np.argsort(pred)[:max(tuner_cls.keep_min, int(len(runs) * tuner_cls.keep_fraction + 0.999))]
    return times[keep].min() == times.min()


@pytest.mark.parametrize("op", ["ret", "ret_bwd"])
def test_retnet_models_keep_the_winner_of_head_sizes_they_have_not_seen(op):
    """Recorded exhaustive runs of the RetNet forward and backward spaces (three head-size pairs, dense, causal and decay
    walks; the backward with its per-pass buffer counts and the stored-dS variants).  The shipped models are the fit on
    all of them; a model fitted WITHOUT the runs of one head-size pair must still rank that pair's measured winners
    inside the share the tuning loop keeps."""
    from attention_autotuner_amd.autotuner import RetBwdTunner, RetTunner
    from attention_autotuner_amd.benchmarks.tune import make_tensors
    cls = RetTunner if op == "ret" else RetBwdTunner
    names = [n for n, r in RET_RUNS.items() if r[0] == op]
    runs = {n: _ret_samples(n) for n in names}
    assert all(len(r) >= 27 for r in runs.values())
    if op == "ret_bwd":                                    # lines of the backward log parse back with every knob
        some = runs["ret_bwd_b4h8q2048k2048_c1_256_512.txt"]
        assert {c.ds_rows for c, *_ in some} == {0, 128, 256} and len({(c.num_stages_qk, c.num_stages_dv, c.num_stages_ds, c.num_stages_dq) for c, *_ in some}) > 4
    everything = [s for r in runs.values() for s in r]
    fitted = costmodel.CostModel(unit="ms", names=costmodel.RET_FEATURES).fit(everything)
    tuner = cls(MI355X(), make_tensors(op, 4, 8, 2048, 2048, 256, 512, "meta"), causal=True)
    assert tuner.cost_model is not None and tuner.cost_model.names == costmodel.RET_FEATURES
    np.testing.assert_allclose(tuner.cost_model.weights, fitted.weights, rtol=1e-6)
    for n in names:
        assert _survives(tuner.cost_model, runs[n], cls), (n, tuner.cost_model.rank_of_best(runs[n]))
    for dims in {RET_RUNS[n][1][4:] for n in names}:
        train = [s for n in names if RET_RUNS[n][1][4:] != dims for s in runs[n]]
        held_out = costmodel.CostModel(unit="ms", names=costmodel.RET_FEATURES).fit(train)
        for n in names:
            if RET_RUNS[n][1][4:] == dims:
                assert _survives(held_out, runs[n], cls), (dims, n, held_out.rank_of_best(runs[n]))
    # the tuner prunes with it, and AAT_TUNE_PRUNE=0 switches that off
    cfgs = [c for c in tuner.get_tuned_configs() if tuner._fits_problem(c)]
    kept = tuner.prune(cfgs)
    assert len(kept) == max(tuner.keep_min, int(len(cfgs) * tuner.keep_fraction + 0.999)) < len(cfgs)


ATTN_BWD_RUNS = {                                         # file -> ((B, H, Sq, Sk, d_qk, d_v), causal)
    "attn_bwd_b4h32q2048k2048_c0_128_128.txt": ((4, 32, 2048, 2048, 128, 128), False),
    "attn_bwd_b4h32q2048k2048_c1_128_128.txt": ((4, 32, 2048, 2048, 128, 128), True),
    "attn_bwd_b8h32q1024k1024_c1_128_128.txt": ((8, 32, 1024, 1024, 128, 128), True),
    "attn_bwd_b4h8q2048k2048_c0_64_64.txt": ((4, 8, 2048, 2048, 64, 64), False),
    "attn_bwd_b4h32q2048k2048_c1_64_64.txt": ((4, 32, 2048, 2048, 64, 64), True),
    "attn_bwd_b4h8q2048k2048_c1_192_192.txt": ((4, 8, 2048, 2048, 192, 192), True),
    "attn_bwd_b4h8q2048k2048_c0_256_256.txt": ((4, 8, 2048, 2048, 256, 256), False),
}


def test_attention_backward_model_keeps_the_winner_of_head_sizes_it_has_not_seen():
    """Seven recorded exhaustive runs of the attention backward space (four head sizes, three problem shapes, both walks;
    the row kernel's own occupancy and tile height and the one-kernel-per-output variants among the candidates).  The
    shipped model is the fit on all of them; fitted without one head size it still ranks that size's winners inside the
    share the tuning loop keeps."""
    from attention_autotuner_amd.autotuner.tunner import AttnBwdTunner
    from attention_autotuner_amd.benchmarks.tune import make_tensors
    runs = {n: costmodel.samples_from_tuning_log(os.path.join(LOGS, n), "attn_bwd", p[4], p[5], p[:4], c) for n, (p, c) in ATTN_BWD_RUNS.items()}
    assert [len(runs[n]) for n in ATTN_BWD_RUNS] == [50, 50, 50, 118, 118, 15, 6]
    some = runs["attn_bwd_b4h32q2048k2048_c0_128_128.txt"]       # the log lines parse back with every knob
    assert {c.col_split for c, *_ in some} == {0, 1} and {c.row_waves_per_eu for c, *_ in some} == {1, 2} and {c.row_Bc for c, *_ in some} == {32, 64}
    fitted = costmodel.CostModel(unit="ms", names=costmodel.RET_FEATURES).fit([s for r in runs.values() for s in r])
    tuner = AttnBwdTunner(MI355X(), make_tensors("attn_bwd", 4, 32, 2048, 2048, 128, 128, "meta"), causal=True)
    assert tuner.cost_model is not None and tuner.cost_model.names == costmodel.RET_FEATURES
    np.testing.assert_allclose(tuner.cost_model.weights, fitted.weights, rtol=1e-6)
    for n in runs:
        assert _survives(tuner.cost_model, runs[n], AttnBwdTunner), (n, tuner.cost_model.rank_of_best(runs[n]))
    for dims in {p[4:] for p, _ in ATTN_BWD_RUNS.values()}:
        train = [s for n, (p, _) in ATTN_BWD_RUNS.items() if p[4:] != dims for s in runs[n]]
        held_out = costmodel.CostModel(unit="ms", names=costmodel.RET_FEATURES).fit(train)
        for n, (p, _) in ATTN_BWD_RUNS.items():
            if p[4:] == dims:
                assert _survives(held_out, runs[n], AttnBwdTunner), (dims, n, held_out.rank_of_best(runs[n]))
    cfgs = [c for c in tuner.get_tuned_configs() if tuner._fits_problem(c)]
    kept = tuner.prune(cfgs)
    assert len(kept) == max(tuner.keep_min, int(len(cfgs) * tuner.keep_fraction + 0.999)) < len(cfgs)


def test_an_attention_model_file_still_loads_and_a_foreign_feature_set_does_not(tmp_path):
    m = costmodel.CostModel.load(os.path.join(AttnTunner(MI355X(), _meta(4, 32, 2048)).cache_path, "costmodel_attn.json"))
    assert m.names == costmodel.FEATURES
    with pytest.raises(ValueError):
        costmodel.CostModel.from_dict({"features": ["matrix", "moon_phase"], "weights": [1.0, 2.0]})
