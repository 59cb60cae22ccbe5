"""Export (configuration features, measured cycles) pairs for fitting a cost model of the search space.

MI355X counterpart of reference python/tests/export_costmodel_config.py:1-62 and python/tests/ncu_profile.py:10-44:
the reference runs Nsight Compute once per candidate and reads "Elapsed Cycles"; here ONE rocprofv3
counter run (GRBM_GUI_ACTIVE, busy cycles summed over the 8 XCDs) covers every candidate, because the
candidates are separately built libraries that one process can launch back to back.

    python -m attention_autotuner_amd.benchmarks.export_costmodel_config attn 4 32 2048 2048 128 128 [--causal] [--limit N] [--only-built] [--out FILE]

The outer invocation builds the candidate libraries, starts itself under ``rocprofv3 --pmc`` with
``--run-candidates`` (that inner process launches every candidate twice: one warm-up, one counted),
matches the counter rows to the candidates by dispatch order and writes a JSON list of

    {"config": {...}, "cost_model_config": [[Sq, Sk, dqk, dv], [Br, Bc, BlockK, D], [wave tile of the first
     contraction], [wave tile of the second], B, H], "causal": bool, "cycles": int, "dispatches": int, "scratch_bytes": int,
     "lds_bytes": int, "registers": int}

in the tuple layout of the reference's exporter (wave tiles are (rows, columns, 16): the rows and
columns one wave computes per step and the MFMA k depth).
"""
import argparse
import csv
import glob
import json
import os
import subprocess
import sys
import tempfile

import torch

from ..arch import MI355X
from ..autotuner import codegen, gfx950_space, library
from .tune import make_tensors

TUNERS = {"attn": "AttnTunner", "ret": "RetTunner"}
XCDS = 8


def candidates(op, dims, causal, limit, only_built=False):
    """The tuner's candidates for the problem; ``only_built``: those whose
    library is already in the build directory (a machine without a compiler, or a process that must not start one)."""
    from ..autotuner import tunner
    b, h, sq, sk, dqk, dv = dims
    arrays = make_tensors(op, b, h, sq, sk, dqk, dv, "meta")
    t = getattr(tunner, TUNERS[op])(MI355X(), arrays, causal=causal)
    cfgs = [c for c in t.get_tuned_configs() if t._fits_problem(c)]
    if only_built:
        cfgs = [c for c in cfgs if os.path.exists(codegen.library_path(c))]
    return cfgs[:limit] if limit else cfgs


def cost_model_tuple(cfg, dims):
    b, h, sq, sk, dqk, dv = dims
    nw = cfg.Nthreads // 64
    if cfg.fuse_type == "shared":
        w1n, w2n = cfg.warps_mma1_n, cfg.warps_mma_n
    else:                                                 # register fuse: every wave owns whole rows of both contractions
        w1n = w2n = 1
    tile1 = (cfg.Br // (nw // w1n), cfg.Bc // w1n, 16)
    tile2 = (cfg.Br // (nw // w2n), cfg.D // w2n, 16)
    return [[sq, sk, dqk, dv], [cfg.Br, cfg.Bc, cfg.BlockKSmem, cfg.D], list(tile1), list(tile2), b, h]


def dispatches_per_launch(cfg, dims, causal):
    """Kernels one launch of ``cfg`` enqueues: a kv-splitting attention configuration runs its split kernel and the
    merge (csrc/kernels/attention/regfuse/profile_code.py: ``split_applies``), everything else one kernel."""
    ns = getattr(cfg, "kv_splits", 1)
    return 2 if (cfg.operation == "attn" and ns > 1 and not causal and (dims[3] // cfg.Bc) % ns == 0) else 1


def scratch_bytes(cfg):
    """Largest per-lane scratch of any kernel in the configuration's library (the compiler's report), or None."""
    usage = codegen.resource_usage(codegen.library_path(cfg))
    return max((k.get("scratch_bytes", 0) for k in usage), default=0) if usage else None


def run_candidates(op, dims, causal, limit, only_built=False):
    """Inner mode (under rocprofv3): launch every candidate library twice."""
    import ctypes
    b, h, sq, sk, dqk, dv = dims
    arrays = make_tensors(op, b, h, sq, sk, dqk, dv, "cuda")
    ptrs = [ctypes.c_void_p(t.data_ptr()) for t in arrays]
    extra = [ctypes.c_float(dqk ** -0.5), ctypes.c_int(int(causal))] if op == "attn" else [ctypes.c_int(int(causal))]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for cfg in candidates(op, dims, causal, limit, only_built):
        path = codegen.library_path(cfg)
        if not os.path.exists(path):
            continue
        lib = library.load(path, op)
        need = int(lib.workspace_size(b, h, sq, sk))
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
        for _ in range(2):
            rc = lib.kernel_entry_ex(*ptrs, b, h, sq, sk, *extra, ctypes.c_void_p(ws.data_ptr() if need else 0), ctypes.c_size_t(need), stream)
            if rc != 0:
                raise RuntimeError(f"{cfg}: kernel_entry_ex returned {rc}")
        torch.cuda.synchronize()
        print("LAUNCHED " + str(cfg), flush=True)


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("op", choices=sorted(TUNERS))
    ap.add_argument("dims", type=int, nargs=6, metavar="N", help="B H Sq Sk dqk dv")
    ap.add_argument("--causal", action="store_true")
    ap.add_argument("--limit", type=int, default=0, help="only the first N candidates")
    ap.add_argument("--only-built", action="store_true", help="only candidates whose library is already built (nothing is compiled)")
    ap.add_argument("--out", default=None)
    ap.add_argument("--run-candidates", action="store_true", help=argparse.SUPPRESS)
    args = ap.parse_args(argv)
    if args.run_candidates:
        run_candidates(args.op, args.dims, args.causal, args.limit, args.only_built)
        return 0

    arch = MI355X()
    cfgs = candidates(args.op, args.dims, args.causal, args.limit, args.only_built)
    if not cfgs:
        raise RuntimeError("no candidate library to count")
    if not args.only_built:
        libs = codegen.compile_parallel(cfgs, arch, timeout=300)
        cfgs = [c for c, l in zip(cfgs, libs) if l is not None]
    out_dir = tempfile.mkdtemp(prefix="aat_costmodel_", dir=os.environ.get("TMPDIR", "/tmp"))
    inner = [sys.executable, "-m", "attention_autotuner_amd.benchmarks.export_costmodel_config", args.op,
             *map(str, args.dims), "--run-candidates", "--limit", str(args.limit)] + (["--causal"] if args.causal else []) + \
            (["--only-built"] if args.only_built else [])
    cmd = ["rocprofv3", "--pmc", "GRBM_GUI_ACTIVE", "--output-format", "csv", "-d", out_dir, "-o", "cm", "--", *inner]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=1800)
    launched = [l.split(" ", 1)[1] for l in res.stdout.splitlines() if l.startswith("LAUNCHED ")]
    if res.returncode != 0 or not launched:
        sys.stderr.write(res.stdout[-2000:] + res.stderr[-2000:])
        raise RuntimeError("the counter run failed")
    rows = []
    for path in glob.glob(os.path.join(out_dir, "**", "*counter_collection.csv"), recursive=True):
        with open(path) as f:
            rows += [r for r in csv.DictReader(f) if r["Counter_Name"] == "GRBM_GUI_ACTIVE" and "aat" in r["Kernel_Name"]]
    rows.sort(key=lambda r: int(r["Dispatch_Id"]))
    # every candidate was launched twice (warm-up, counted): the cycles of a launch are those of its kernels together
    by_name = {str(c): c for c in cfgs}
    per_launch = [dispatches_per_launch(by_name[name], args.dims, args.causal) for name in launched]
    if len(rows) != 2 * sum(per_launch):
        raise RuntimeError(f"{len(rows)} counted dispatches for {len(launched)} candidates ({sum(per_launch)} kernels per round)")
    records, at = [], 0
    for name, k in zip(launched, per_launch):
        cfg = by_name[name]
        counted = rows[at + k:at + 2 * k]
        at += 2 * k
        records.append({"config": cfg.to_dict(), "cost_model_config": cost_model_tuple(cfg, args.dims), "causal": bool(args.causal),
                        "cycles": int(sum(float(r["Counter_Value"]) for r in counted) / XCDS), "dispatches": k,
                        "scratch_bytes": scratch_bytes(cfg),
                        "lds_bytes": gfx950_space.forward_lds_bytes(cfg), "registers": gfx950_space.forward_reg_estimate(cfg)})
    out = args.out or f"{args.op}_{args.dims[4]}_{args.dims[5]}_costmodel.json"
    with open(out, "w") as f:
        json.dump(records, f, indent=1)
    best = min(records, key=lambda r: r["cycles"])
    print(json.dumps({"candidates": len(records), "out": out, "fewest_cycles": best["cycles"],
                      "best": str(by_name[launched[records.index(best)]])}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
