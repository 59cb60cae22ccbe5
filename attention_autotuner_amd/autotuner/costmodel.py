"""A fitted cost model of a search space (forward kernels, RetNet backward), used to decide which candidates are worth timing.

The reference exports (configuration, measured cycles) pairs for such a model and stops there
(reference python/tests/export_costmodel_config.py:31-56; nothing in the reference reads the file back).
Here the pairs come from either source this package produces -- the cycle counts of
``benchmarks/export_costmodel_config.py`` or the per-candidate times in a tuner's
``profile_result_*.txt`` log -- and the model is what ``BaseTunner.prune`` ranks candidates with.

The model is deliberately small: a handful of per-launch quantities that can be computed from a
configuration and a problem shape alone, each an estimate of cycles spent on one resource,

    matrix    MFMA cycles per SIMD                       (the same for every configuration of a problem, up to
                                                          the tiles a causal walk cannot skip)
    lds       LDS bytes the waves read per CU            (falls with rows per wave and with the kv tile height)
    vector    score elements a lane processes            (falls when waves split the kv range, rises with recompute)
    exposed   the three above divided by the waves a SIMD interleaves (latency nobody hides)
    steps     kv steps per block times resident rounds   (per-step fixed costs: barriers, waits, DMA issue)
    blocks    blocks per CU                              (prologue / epilogue)
    tail      rounds the last, partly filled, wave of blocks adds

combined linearly with weights fitted by ridge regression on measured launches.  It only has to rank:
``BaseTunner.prune`` keeps the best third it predicts, and the test suite checks on recorded tuning logs that
the measured winner survives that cut on problems the model was not fitted on.
"""
import json
import math
import re

import numpy as np

from . import gfx950_space
from .configs import supported_configs

FEATURES = ("matrix", "lds", "vector", "exposed", "steps", "blocks", "tail", "one")
# ... and three more for the RetNet spaces, whose candidates differ mostly in what the first eight do not see:
#     stream    bytes a CU pulls from L2 into LDS (K/V/mask or Y/Z tiles), at 64 bytes per cycle
#     sync      block-wide barriers a block passes (two per step with single buffers, one with double, one more where
#               the LDS-fused kernel exchanges row statistics)
#     solo      matrix cycles of kernels that run one wave per SIMD (nothing to overlap with)
RET_FEATURES = FEATURES + ("stream", "sync", "solo")
ALL_FEATURES = RET_FEATURES
SIMDS, CUS = 1024, 256


def _rounds(n_blocks, per_cu):
    resident = CUS * per_cu
    return n_blocks / resident, math.ceil(n_blocks / resident)


def _chain_features(n_blocks, steps, rows, tile, kx, dz, nw, per_cu, wave_lds_share=1.0, barriers=2, mask_tiles=1):
    """The per-launch quantities of one chained-contraction kernel: ``rows`` resident rows per block, streamed tiles of
    ``tile`` rows, first contraction over ``kx`` columns, second into ``dz`` columns; every wave reads whole tiles."""
    waves_per_simd = max(1.0, per_cu * nw / 4.0)
    mfma_per_step = rows * tile * (kx + dz) / (32 * 32 * 16)
    matrix = n_blocks * steps * mfma_per_step * 32.0 / SIMDS
    lds = n_blocks * steps * nw * (tile * kx * 2 + tile * dz * 2) * wave_lds_share / 128.0 / CUS
    vector = n_blocks * steps * nw * (rows * tile / 64.0 / nw) * 6.0 / SIMDS
    exposed = (matrix + lds + vector) / waves_per_simd
    frac_rounds, whole_rounds = _rounds(n_blocks, per_cu)
    tail = (whole_rounds - frac_rounds) * steps * mfma_per_step * 32.0 / nw
    stream = n_blocks * steps * (tile * kx * 2 + tile * dz * 2 + rows * tile * 2 * mask_tiles) / 64.0 / CUS
    sync = steps * whole_rounds * barriers
    solo = matrix if waves_per_simd <= 1.0 else 0.0
    return np.array([matrix, lds, vector, exposed, steps * whole_rounds, float(whole_rounds), tail, 0.0, stream, sync, solo])


def backward_features(cfg, shape, causal=False):
    """The same quantities for a RetNet backward configuration, summed over the kernels one launch runs: the dV pass
    (resident kv rows, streamed query tiles), the dQ pass (resident query rows, streamed kv tiles) and either the chained
    dK pass or, with a stored dS, the dK kernel that reads it back (a third of a chained pass's matrix work, two waves per
    SIMD, ``ds_rows`` kv rows per block)."""
    b, h, sq, sk = shape
    nw = cfg.Nthreads // 64
    half = 0.5 if causal else 1.0                         # a causal walk visits about half the streamed tiles
    per_cu = gfx950_space.blocks_per_cu(cfg)
    dvb = gfx950_space.backward_dv_cols(cfg)
    total = np.zeros(len(ALL_FEATURES))
    bars_v = 2 if (cfg.num_stages_qk == 1 or cfg.num_stages_dv == 1) else 1
    sds, sdq = getattr(cfg, "num_stages_ds", cfg.num_stages_qk), getattr(cfg, "num_stages_dq", cfg.num_stages_dv)
    bars_q = 2 if (sds == 1 or sdq == 1) else 1
    # dV: grid over kv blocks (x column slices where the output is cut), streams Sq / Bc query tiles
    total += _chain_features(b * h * (sk // cfg.Br) * (cfg.D // dvb), half * sq / cfg.Bc + 0.5 * causal, cfg.Br, cfg.Bc, cfg.Kd, dvb, nw, per_cu, barriers=bars_v)
    # dQ: grid over query blocks, streams Sk / Bc kv tiles
    total += _chain_features(b * h * (sq // cfg.Br), half * sk / cfg.Bc + 0.5 * causal, cfg.Br, cfg.Bc, cfg.D, cfg.Kd, nw, per_cu, barriers=bars_q)
    ds_rows = getattr(cfg, "ds_rows", 0)
    if ds_rows:                                           # dK = dS^T Q only: 64-row query tiles, 2 * ds_rows threads
        total += _chain_features(b * h * (sk // ds_rows), half * sq / 64 + 0.5 * causal, ds_rows, 64, 0, cfg.Kd, ds_rows // 32, 2, barriers=1, mask_tiles=1)
        total[8] += b * h * sq * sk * 2 * 2 * half / 64.0 / CUS       # the dS round trip through memory (written once, read once)
    else:
        total += _chain_features(b * h * (sk // cfg.Br), half * sq / cfg.Bc + 0.5 * causal, cfg.Br, cfg.Bc, cfg.D, cfg.Kd, nw, per_cu, barriers=bars_q)
    total[7] = 1.0
    return total


def attn_backward_features(cfg, shape, causal=False):
    """The same quantities for an attention backward configuration, summed over its kernels: the column kernel (``Br`` kv
    rows resident, query tiles of ``Bc`` rows streamed; S, dP, dV and dK: contractions over d_qk + d_v and into
    d_v + d_qk columns) -- or, with ``col_split``, one column kernel for dV (S and dV) and one for dK (S, dP and dK), each
    at its own waves per SIMD -- and the row kernel (``Br`` query rows resident, kv tiles of ``row_Bc`` rows; S, dP, dQ)."""
    b, h, sq, sk = shape
    nw = cfg.Nthreads // 64
    half = 0.5 if causal else 1.0

    def per_cu(wpe):
        return max(1, wpe * 4 // nw)
    total = np.zeros(len(ALL_FEATURES))
    col_blocks, col_steps = b * h * (sk // cfg.Br), half * sq / cfg.Bc + 0.5 * causal
    if getattr(cfg, "col_split", 0):
        total += _chain_features(col_blocks, col_steps, cfg.Br, cfg.Bc, cfg.Kd, cfg.D, nw, per_cu(cfg.dv_waves_per_eu), barriers=1, mask_tiles=0)
        total += _chain_features(col_blocks, col_steps, cfg.Br, cfg.Bc, cfg.Kd + cfg.D, cfg.Kd, nw, per_cu(cfg.dk_waves_per_eu), barriers=1, mask_tiles=0)
    else:
        total += _chain_features(col_blocks, col_steps, cfg.Br, cfg.Bc, cfg.Kd + cfg.D, cfg.D + cfg.Kd, nw, per_cu(cfg.waves_per_eu), barriers=1, mask_tiles=0)
    row_bc = getattr(cfg, "row_Bc", cfg.Bc)
    row_wpe = getattr(cfg, "row_waves_per_eu", cfg.waves_per_eu)
    total += _chain_features(b * h * (sq // cfg.Br), half * sk / row_bc + 0.5 * causal, cfg.Br, row_bc, cfg.Kd + cfg.D, cfg.Kd, nw, per_cu(row_wpe), barriers=1, mask_tiles=0)
    total[7] = 1.0
    return total


def features(cfg, shape, causal=False, names=FEATURES):
    """The feature vector (in the order of ``names``) of configuration ``cfg`` on ``shape`` = (B, H, Sq, Sk): forward
    kernels in ``forward_features``, the backward operators in ``backward_features`` / ``attn_backward_features``."""
    op = getattr(cfg, "operation", "")
    full = (backward_features if op == "ret_bwd" else attn_backward_features if op == "attn_bwd" else forward_features)(cfg, shape, causal)
    return np.array([full[ALL_FEATURES.index(n)] for n in names])


def forward_features(cfg, shape, causal=False):
    b, h, sq, sk = shape
    nw = cfg.Nthreads // 64
    splits = max(1, getattr(cfg, "kv_splits", 1))
    n_blocks = b * h * (sq // cfg.Br) * splits
    steps = sk / cfg.Bc / splits
    if causal:                                            # a row block walks the tiles up to its own diagonal
        steps = (sk / cfg.Bc) * 0.5 + 0.5 * cfg.Br / cfg.Bc + 0.5
    per_cu = gfx950_space.blocks_per_cu(cfg)
    lds_room = max(1, 160 * 1024 // max(1, gfx950_space.forward_lds_bytes(cfg)))
    per_cu = max(1, min(per_cu, lds_room))
    waves_per_simd = max(1.0, per_cu * nw / 4.0)
    mfma_per_step = cfg.Br * cfg.Bc * (cfg.Kd + cfg.D) / (32 * 32 * 16)      # 32x32x16 MFMAs of one block step
    matrix = n_blocks * steps * mfma_per_step * 32.0 / SIMDS               # 32 cycles each
    if cfg.fuse_type == "shared":
        w1n, w2n = max(1, cfg.warps_mma1_n), max(1, cfg.warps_mma_n)
        k_reads = (nw // w1n) * cfg.Bc * cfg.Kd * 2 / w1n * w1n            # every row group reads the K tile slice of its column group
        v_reads = (nw // w2n) * cfg.Bc * cfg.D * 2
        p_traffic = 2 * cfg.Br * cfg.Bc * 2 * max(1, w2n // 2)             # P written once, read by every d slice
        lds_bytes = k_reads + v_reads + p_traffic
        vec = cfg.Br * cfg.Bc / 64.0 / nw
    else:
        lds_bytes = nw * (cfg.Bc * cfg.Kd * 2 + cfg.Bc * cfg.D * 2)         # every wave reads the whole K and V tile
        vec = cfg.Br * cfg.Bc / 64.0 / nw
    lds = n_blocks * steps * lds_bytes / 128.0 / CUS                       # 128 bytes per cycle per CU
    vector = n_blocks * steps * nw * vec * 6.0 / SIMDS                     # about six vector instructions per score element
    exposed = (matrix + lds + vector) / waves_per_simd
    frac_rounds, whole_rounds = _rounds(n_blocks, per_cu)
    step_count = steps * whole_rounds
    tail = (whole_rounds - frac_rounds) * steps * mfma_per_step * 32.0 / nw
    if getattr(cfg, "sw_pipeline", 0):
        exposed *= 0.8
    has_mask = getattr(cfg, "operation", "") == "ret"
    stream = n_blocks * steps * (cfg.Bc * (cfg.Kd + cfg.D) * 2 + (cfg.Br * cfg.Bc * 2 if has_mask else 0)) / 64.0 / CUS
    single = getattr(cfg, "num_stages_qk", 2) == 1 or getattr(cfg, "num_stages_v", 2) == 1
    barriers = (2 if single else 1) + (1 if cfg.fuse_type == "shared" and max(1, cfg.warps_mma1_n) > 1 else 0) + (1 if cfg.fuse_type == "shared" else 0)
    sync = step_count * barriers
    solo = matrix if waves_per_simd <= 1.0 else 0.0
    return np.array([matrix, lds, vector, exposed, step_count, float(whole_rounds), tail, 1.0, stream, sync, solo])


class CostModel:
    def __init__(self, weights=None, unit="ms", names=FEATURES):
        self.names = tuple(names)
        self.weights = np.zeros(len(self.names)) if weights is None else np.asarray(weights, dtype=float)
        self.unit = unit

    def predict(self, cfg, shape, causal=False):
        return float(self.weights @ features(cfg, shape, causal, self.names))

    def fit(self, samples, ridge=1e-3):
        """``samples``: iterable of (cfg, shape, causal, measured cost).  Ridge regression on features scaled to
        unit mean, so that one weight does not dominate because its feature is counted in larger units."""
        x = np.array([features(c, s, ca, self.names) for c, s, ca, _ in samples])
        y = np.array([t for *_, t in samples], dtype=float)
        scale = np.maximum(x.mean(axis=0), 1e-12)
        xs = x / scale
        a = xs.T @ xs + ridge * len(y) * np.eye(xs.shape[1])
        self.weights = np.linalg.solve(a, xs.T @ y) / scale
        return self

    def rank_of_best(self, samples):
        """Position (0 = first) that the measured-best sample has in the model's ranking of ``samples``."""
        samples = list(samples)
        best = min(range(len(samples)), key=lambda i: samples[i][3])
        order = sorted(range(len(samples)), key=lambda i: self.predict(*samples[i][:3]))
        return order.index(best)

    def to_dict(self):
        return {"features": list(self.names), "weights": [float(w) for w in self.weights], "unit": self.unit}

    @classmethod
    def from_dict(cls, d):
        if any(n not in ALL_FEATURES for n in d["features"]) or len(d["features"]) != len(d["weights"]):
            raise ValueError("cost model was fitted on a feature set this version does not compute")
        return cls(d["weights"], d.get("unit", "ms"), d["features"])

    def save(self, path):
        with open(path, "w") as f:
            json.dump(self.to_dict(), f, indent=1)

    @classmethod
    def load(cls, path):
        with open(path) as f:
            return cls.from_dict(json.load(f))


# ---- measured samples ---------------------------------------------------------------------------------
_FIELD = re.compile(r"(\w+)=([^,()\s]+)")


def config_from_log_line(text, op, dim_qk, dim_v):
    """The configuration behind a ``Config(field=value, ...)`` line of a tuner's log.  The line carries neither
    the operator nor the head sizes (the reference's layout: they are in the file name)."""
    fields = {}
    for key, raw in _FIELD.findall(text.partition("(")[2]):
        if raw in ("True", "False"):
            fields[key] = raw == "True"
        else:
            try:
                fields[key] = int(raw)
            except ValueError:
                fields[key] = raw
    if "warp_mma_n" in fields:                              # the reference's spelling in the log
        fields["warps_mma_n"] = fields.pop("warp_mma_n")
    nw = max(1, fields.get("Nthreads", 64) // 64)
    fields.setdefault("warps_mma1_n", nw)
    fields.setdefault("warps_mma_n", nw)
    fields.update(Kd=dim_qk, D=dim_v)
    return supported_configs[op].from_dict(fields)


def samples_from_tuning_log(path, op, dim_qk, dim_v, shape, causal=False, failed=1e7):
    """(cfg, shape, causal, ms) for every timed candidate in a ``profile_result_*.txt``."""
    out = []
    with open(path) as f:
        lines = [l.rstrip("\n") for l in f]
    for i in range(len(lines) - 1):
        if not re.match(r"\w*Config\(", lines[i]) or (i > 0 and lines[i - 1].startswith("best config")):
            continue
        try:
            ms = float(lines[i + 1])
        except ValueError:
            continue
        if ms < failed:
            out.append((config_from_log_line(lines[i], op, dim_qk, dim_v), tuple(shape), bool(causal), ms))
    return out


def samples_from_summary(path, op, only=None):
    """Samples of every recorded tuning run of ``op`` listed in a ``summary.jsonl`` (one JSON object per run with its
    problem, its causal flag and the path of its per-candidate log, as ``benchmarks/tune.py`` prints them).  Log paths are
    taken relative to the summary's directory when they do not exist as written.  ``only``: a predicate on the run record."""
    import os
    out = []
    with open(path) as f:
        runs = [json.loads(l) for l in f if l.strip()]
    for r in runs:
        if r.get("op") != op or (only is not None and not only(r)):
            continue
        log = r["log"]
        if not os.path.exists(log):
            log = os.path.join(os.path.dirname(os.path.abspath(path)), os.path.basename(log))
        b, h, sq, sk, dqk, dv = r["problem"]
        causal = bool(r.get("causal")) or "decay" in os.path.basename(log)
        out += samples_from_tuning_log(log, op, dqk, dv, (b, h, sq, sk), causal)
    return out


def samples_from_export(path, max_scratch_bytes=None):
    """(cfg, shape, causal, cycles) from the JSON of ``benchmarks/export_costmodel_config.py``.  ``max_scratch_bytes``:
    leave out the candidates whose library keeps more than that per lane in scratch memory -- the tuning loop does not
    time those either, and their cycle counts (ten times the rest) would be all a least-squares fit sees."""
    with open(path) as f:
        records = json.load(f)
    out = []
    for r in records:
        if max_scratch_bytes is not None and (r.get("scratch_bytes") or 0) > max_scratch_bytes:
            continue
        cfg = supported_configs[r["config"]["operation"]].from_dict(r["config"])
        (sq, sk, _, _), _, _, _, b, h = r["cost_model_config"]
        out.append((cfg, (b, h, sq, sk), bool(r.get("causal", False)), float(r["cycles"])))
    return out


def main(argv=None):
    """``python -m attention_autotuner_amd.autotuner.costmodel fit EXPORT.json [EXPORT.json ...] --out MODEL.json``:
    fit on the cycle counts of one or more exporter runs (candidates that spill left out) and write the model."""
    import argparse
    from . import codegen
    ap = argparse.ArgumentParser()
    ap.add_argument("command", choices=["fit", "fit-logs"])
    ap.add_argument("exports", nargs="+", help="fit: exporter JSON files; fit-logs: entries of a tuning summary.jsonl (see fit_from_summary)")
    ap.add_argument("--out", required=True)
    ap.add_argument("--op", default=None, help="fit-logs: the operator whose runs are used")
    args = ap.parse_args(argv)
    if args.command == "fit-logs":
        samples = [s for path in args.exports for s in samples_from_summary(path, args.op)]
        model = CostModel(unit="ms", names=RET_FEATURES if args.op in ("ret", "ret_bwd", "attn_bwd") else FEATURES).fit(samples)
        model.save(args.out)
        print(json.dumps({"samples": len(samples), "out": args.out}))
        return 0
    samples = [s for path in args.exports for s in samples_from_export(path, codegen.MAX_SCRATCH_BYTES)]
    model = CostModel(unit="cycles").fit(samples)
    model.save(args.out)
    print(json.dumps({"samples": len(samples), "out": args.out, "rank_of_best": model.rank_of_best(samples)}))
    return 0


if __name__ == "__main__":
    import sys
    sys.exit(main())

