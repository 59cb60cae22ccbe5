"""A fitted cost model of the forward search space, used to decide which candidates are worth timing.

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
SIMDS, CUS = 1024, 256


def _rounds(n_blocks, per_cu):
    resident = CUS * per_cu
    return n_blocks / resident, math.ceil(n_blocks / resident)


def features(cfg, shape, causal=False):
    """The feature vector (order of FEATURES) of forward configuration ``cfg`` on ``shape`` = (B, H, Sq, Sk)."""
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
    return np.array([matrix, lds, vector, exposed, step_count, float(whole_rounds), tail, 1.0])


class CostModel:
    def __init__(self, weights=None, unit="ms"):
        self.weights = np.zeros(len(FEATURES)) if weights is None else np.asarray(weights, dtype=float)
        self.unit = unit

    def predict(self, cfg, shape, causal=False):
        return float(self.weights @ features(cfg, shape, causal))

    def fit(self, samples, ridge=1e-3):
        """``samples``: iterable of (cfg, shape, causal, measured cost).  Ridge regression on features scaled to
        unit mean, so that one weight does not dominate because its feature is counted in larger units."""
        x = np.array([features(c, s, ca) for c, s, ca, _ in samples])
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
        return {"features": list(FEATURES), "weights": [float(w) for w in self.weights], "unit": self.unit}

    @classmethod
    def from_dict(cls, d):
        if list(d["features"]) != list(FEATURES):
            raise ValueError("cost model was fitted on a different feature set")
        return cls(d["weights"], d.get("unit", "ms"))

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
        if not lines[i].startswith("Config(") or (i > 0 and lines[i - 1].startswith("best config")):
            continue
        try:
            ms = float(lines[i + 1])
        except ValueError:
            continue
        if ms < failed:
            out.append((config_from_log_line(lines[i], op, dim_qk, dim_v), tuple(shape), bool(causal), ms))
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
    ap.add_argument("command", choices=["fit"])
    ap.add_argument("exports", nargs="+")
    ap.add_argument("--out", required=True)
    args = ap.parse_args(argv)
    samples = [s for path in args.exports for s in samples_from_export(path, codegen.MAX_SCRATCH_BYTES)]
    model = CostModel(unit="cycles").fit(samples)
    model.save(args.out)
    print(json.dumps({"samples": len(samples), "out": args.out, "rank_of_best": model.rank_of_best(samples)}))
    return 0


if __name__ == "__main__":
    import sys
    sys.exit(main())

