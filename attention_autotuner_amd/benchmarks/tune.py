"""Tune one problem and record the result (counterpart of the reference's tuner drivers,
python/tests/attntuner_demo.py:186-192 and python/tests/test_retbwdtunner.py:88-92).

    python -m attention_autotuner_amd.benchmarks.tune attn    B H Sq Sk dqk dv [--causal] [--compile-only]
    python -m attention_autotuner_amd.benchmarks.tune ret     B H Sq Sk dqk dv [--causal]
    python -m attention_autotuner_amd.benchmarks.tune ret_bwd B H Sq Sk dqk dv [--causal]
    python -m attention_autotuner_amd.benchmarks.tune attn_bwd B H Sq Sk dqk dv [--causal]
    python -m attention_autotuner_amd.benchmarks.tune ret|ret_bwd ... --decay      (decay mask built in registers)
    python -m attention_autotuner_amd.benchmarks.tune ... --input-path DIR       (q.pt, k.pt, v.pt, mask.pt, do.pt instead of synthetic tensors)

Writes the best configuration into the tuning cache, the per-candidate log next to it, and prints a
one-line JSON summary.  ``--compile-only`` builds the candidate libraries a tuning run would time (no GPU
needed; all of them under AAT_TUNE_PRUNE=0) so that a later run on a machine without spare CPU time only
has to time them.
"""
import argparse
import json
import math
import os
import sys
import time

import torch

from ..arch import MI355X
from ..autotuner import AttnTunner, RetBwdTunner, RetTunner, codegen
from ..autotuner.tunner import AttnBwdTunner
from ..ops._resolve import DEFAULT_LOG_DIR


def make_tensors(op, b, h, sq, sk, dqk, dv, device, seed=0):
    g = torch.Generator().manual_seed(seed)

    def mk(*shape):
        t = torch.randn(*shape, generator=g).half()
        return t.to(device)

    if device == "meta":
        def mk(*shape):                                        # noqa: F811 - shapes only
            return torch.empty(*shape, dtype=torch.float16, device="meta")
    q, k, v = mk(b, h, sq, dqk), mk(b, h, sk, dqk), mk(b, h, sk, dv)
    if op == "attn":
        return [q, k, v, torch.empty(b, h, sq, dv, dtype=torch.float16, device=device)]
    if op == "attn_bwd":
        # timing only: any finite o and a log-sum-exp of the right magnitude (log S_kv) will do
        o, do = mk(b, h, sq, dv), mk(b, h, sq, dv)
        lse = torch.empty(b, h, sq, dtype=torch.float32, device=device)
        if device != "meta":
            lse.fill_(math.log(sk))
        return [q, k, v, o, do, lse, torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)]
    n = torch.arange(sq, dtype=torch.float64).view(1, sq, 1)
    m = torch.arange(sk, dtype=torch.float64).view(1, 1, sk)
    gamma = (1.0 - torch.pow(2.0, -5.0 - torch.arange(h, dtype=torch.float64))).view(h, 1, 1)
    mask = torch.where(n + (sk - sq) >= m, gamma ** (n + (sk - sq) - m).clamp(min=0), torch.zeros((), dtype=torch.float64))
    mask = mask.float().half().to(device) if device != "meta" else torch.empty(h, sq, sk, dtype=torch.float16, device="meta")
    o = torch.empty(b, h, sq, dv, dtype=torch.float16, device=device)
    r = torch.ones(b, h, sq, dtype=torch.float32, device=device) if device != "meta" else torch.empty(b, h, sq, device="meta")
    if op == "ret":
        return [q, k, v, mask, o, r]
    do = mk(b, h, sq, dv)
    if device != "meta":
        r.fill_(50.0)
    dq, dk, dv_ = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    acc = torch.zeros(1, dtype=torch.float32, device=device) if device != "meta" else torch.empty(1, device="meta")
    return [q, k, v, mask, do, r, dq, dk, dv_, acc]


def load_inputs(arrays, op, input_path, device):
    """Replace the synthetic q, k, v (and the RetNet mask, and dO where there is one) by tensors stored under ``input_path``
    as q.pt, k.pt, v.pt, mask.pt, do.pt -- the layout of the reference's tuner driver
    (reference python/tests/attntuner_demo.py:38-43: a singleton dimension 1 is dropped, the leading [B, H, S, d] corner is
    used).  Files are read with ``weights_only=True``: plain tensors only, nothing in them is executed.  A file that is
    absent keeps the synthetic tensor."""
    def corner(name, like):
        path = os.path.join(input_path, name)
        if not os.path.exists(path):
            return like
        t = torch.load(path, map_location="cpu", weights_only=True)
        if t.dim() == like.dim() + 1 and t.shape[1] == 1:
            t = t.squeeze(1)
        if t.dim() != like.dim() or any(a < b for a, b in zip(t.shape, like.shape)):
            raise ValueError(f"{path}: shape {tuple(t.shape)} does not cover the problem's {tuple(like.shape)}")
        t = t[tuple(slice(0, n) for n in like.shape)].to(like.dtype).contiguous()
        return t.to(device) if device != "meta" else like
    arrays[0], arrays[1], arrays[2] = corner("q.pt", arrays[0]), corner("k.pt", arrays[1]), corner("v.pt", arrays[2])
    if op in ("ret", "ret_bwd"):
        arrays[3] = corner("mask.pt", arrays[3])
    if op in ("ret_bwd", "attn_bwd"):
        arrays[4] = corner("do.pt", arrays[4])
    return arrays


def flops(op, b, h, sq, sk, dqk, dv, causal):
    f = 2.0 * b * h * sq * sk * ((dqk + dv) if op in ("attn", "ret") else (3 * dqk + 2 * dv))
    return f / 2 if (causal and op in ("attn", "attn_bwd")) else f      # RetNet rates are quoted on the dense count


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("op", choices=["attn", "ret", "ret_bwd", "attn_bwd"])
    ap.add_argument("dims", type=int, nargs=6, metavar="N", help="B H Sq Sk dqk dv")
    ap.add_argument("--causal", action="store_true")
    ap.add_argument("--decay", action="store_true", help="RetNet only: decay mask built in registers from one rate per head")
    ap.add_argument("--compile-only", action="store_true")
    ap.add_argument("--log-dir", default=DEFAULT_LOG_DIR)
    ap.add_argument("--cache-dir", default=None, help="where the best configuration is recorded (default: the package's tuning cache)")
    ap.add_argument("--cost-model", default=None, help="a fitted cost model (JSON): only the candidates it ranks best are built and timed")
    ap.add_argument("--input-path", default="", help="directory with q.pt, k.pt, v.pt (mask.pt, do.pt): tune on these tensors instead of synthetic ones")
    args = ap.parse_args(argv)
    b, h, sq, sk, dqk, dv = args.dims
    arch = MI355X()
    cls = {"attn": AttnTunner, "ret": RetTunner, "ret_bwd": RetBwdTunner, "attn_bwd": AttnBwdTunner}[args.op]
    device = "meta" if args.compile_only else "cuda"
    arrays = make_tensors(args.op, b, h, sq, sk, dqk, dv, device)
    if args.input_path:
        arrays = load_inputs(arrays, args.op, args.input_path, device)
    if args.decay:
        if args.op not in ("ret", "ret_bwd"):
            ap.error("--decay applies to ret and ret_bwd")
        gamma = 1.0 - torch.pow(2.0, -5.0 - torch.arange(h, dtype=torch.float64))
        arrays[3] = torch.log2(gamma).float().to(device) if device != "meta" else torch.empty(h, device="meta")
        if args.op == "ret_bwd":
            arrays = arrays[:9]                                # no dqaccum in the decay entry points
        tuner = cls(arch, arrays, decay=True)
    else:
        tuner = cls(arch, arrays, causal=args.causal)
    if args.cache_dir:
        tuner.cache_path = args.cache_dir
    if args.cost_model:
        from ..autotuner.costmodel import CostModel
        tuner.cost_model = CostModel.load(args.cost_model)
    if args.compile_only:
        cfgs = tuner.prune([c for c in tuner.get_tuned_configs() if tuner._fits_problem(c)])   # what a tuning run would time
        t0 = time.time()
        libs = codegen.compile_parallel(cfgs, arch, timeout=300)
        print(json.dumps({"op": args.op, "candidates": len(cfgs), "built": sum(l is not None for l in libs),
                          "seconds": round(time.time() - t0, 1)}))
        return 0
    log_dir = os.path.join(args.log_dir, f"{args.op}{'_decay' if args.decay else ''}_b{b}h{h}q{sq}k{sk}_c{int(args.causal or args.decay)}")
    best = tuner.tune(log_path=log_dir, use_cache=False)
    ms = tuner.last_timings[best]
    ok = [t for t in tuner.last_timings.values() if t < 1e7]
    print(json.dumps({"op": args.op, "problem": args.dims, "causal": args.causal, "best": str(best), "ms": round(ms, 5),
                      "tflops": round(flops(args.op, b, h, sq, sk, dqk, dv, args.causal) / ms / 1e9, 1),
                      "candidates": len(tuner.last_timings), "ran": len(ok), "worst_ms": round(max(ok), 4),
                      "spilling_not_timed": len(tuner.rejected_spills), "ranked_out": len(tuner.pruned),
                      "cache": tuner._cache_file(), "log": log_dir}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
