#!/usr/bin/env python3
"""Headline benchmark: flash-attention forward, B4 H32 S2048 D128 fp16, non-causal, on one MI355X.

A step is one launch of the fused forward kernel, through the C ABI of its config library, on inputs
already resident in HBM.  Prints one JSON line (throughput in TFLOP/s with the dominant kernel's MFMA
roofline fraction and a host-CPU baseline of the same math), preceded by human-readable lines on
stderr.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
os.environ.setdefault("AAT_TUNE_ON_MISS", "0")

PEAK_TFLOPS = 2500.0          # MI355X dense fp16 MFMA
B, H, S, D = 4, 32, 2048, 128


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def attn_flops(b, h, sq, sk, dqk, dv, causal=False):
    f = 2.0 * b * h * sq * sk * (dqk + dv)
    return f / 2 if causal else f


def resolve_config(aat, arch, tensors, causal):
    from attention_autotuner_amd.autotuner import AttnTunner, gfx950_space
    t = AttnTunner(arch, tensors, causal=causal)
    cfg = t.check_cache()
    if cfg is None:
        q, k, v = tensors[:3]
        cfg = gfx950_space.default_forward_config("attn", q.shape[-1], v.shape[-1], arch, q.shape[2], k.shape[2])
    return cfg


MIN_WARMUP_MS = 100.0         # wall time of back-to-back launches before anything is timed, whatever --warmup says


def time_launches(fn, steps, warmup, before_each=None, flush_l2=False):
    """Timing of `steps` calls after at least MIN_WARMUP_MS of back-to-back calls plus `warmup` more:
    the shader clock needs tens of milliseconds of load to settle, so a warm-up counted in launches
    measures the ramp (a 0.3 ms kernel timed after 5 launches runs 15-20 % below its settled rate)."""
    from attention_autotuner_amd.benchmarks.do_bench import LaunchTimer
    return LaunchTimer(MIN_WARMUP_MS).measure(fn, calls=steps, warmup_calls=warmup, before_each=before_each, flush_l2=flush_l2)


def cpu_baseline(chunk=32):
    """The oracle's fp32 torch attention on the host cores over the whole headline workload (all B*H slices, `chunk`
    of them at a time so the score matrices stay within a few GB), three passes."""
    import torch
    from oracle import ref_op
    torch.set_num_threads(os.cpu_count() or 1)
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, chunk, S, D, generator=g).half()
    k = torch.randn(1, chunk, S, D, generator=g).half()
    v = torch.randn(1, chunk, S, D, generator=g).half()
    ref_op.attention_ref(q[:, :1], k[:, :1], v[:, :1])                   # warm-up
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        for _ in range(B * H // chunk):                                  # the same values again: timing does not depend on them
            ref_op.attention_ref(q, k, v)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[1]
    tflops = attn_flops(B, H, S, S, D, D) / med / 1e12
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            model = next((l.split(":", 1)[1].strip() for l in f if l.startswith("model name")), "")
    except OSError:
        pass
    return {"value": round(tflops, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle attention_ref fp32, all {B * H} (batch,head) slices of S={S} D={D} ({chunk} at a time), median of 3 passes: {med * 1e3:.0f} ms",
            "cpu_model": model, "os_cpu_count": os.cpu_count()}


def measured_traffic(cfg, algorithmic_bytes):
    """(HBM bytes per launch, where the figure comes from).  Measured with rocprofv3 (FETCH_SIZE + WRITE_SIZE, each scaled
    by a plain copy of known size) for this kernel configuration when a profile of it has been recorded in
    profiles/traffic.json; a configuration without one (a re-tuned cache entry that nobody profiled yet) is reported with the
    algorithmic bytes, says so in the record, and is announced on stderr."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            got = json.load(f).get(str(cfg), {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        got = None
    if got is not None:
        return got, "rocprofv3 FETCH_SIZE + WRITE_SIZE (profiles/traffic.json)"
    log(f"WARNING: profiles/traffic.json holds no counter profile of {cfg}: roofline.traffic is the ALGORITHMIC byte count, not a measurement")
    return int(algorithmic_bytes), "algorithmic (no counter profile recorded for this kernel configuration)"


def cpu_baseline_retnet():
    """The oracle's fp32 torch RetNet forward (retnet_ref) and closed-form backward (retnet_bwd_ref) on the host cores at
    the RetNet backward shape of the reference's headline configurations (B4 H8 S2048, d_qk 256, d_v 512, decay mask), every (batch, head) slice once, one batch
    (8 heads) at a time."""
    import torch
    from oracle import ref_op
    b, h, s, dqk, dv = 4, 8, 2048, 256, 512
    torch.set_num_threads(os.cpu_count() or 1)
    g = torch.Generator().manual_seed(0)
    q, k = (torch.randn(1, h, s, dqk, generator=g).half() for _ in range(2))
    v, do = (torch.randn(1, h, s, dv, generator=g).half() for _ in range(2))
    mask = ref_op.retnet_decay_mask(h, s, s)
    ref_op.retnet_ref(q[:, :1], k[:, :1], v[:, :1], mask[:1])           # warm-up
    t0 = time.perf_counter()
    for _ in range(b):                                                  # the same values again: timing does not depend on them
        ref_op.retnet_ref(q, k, v, mask)
    t1 = time.perf_counter()
    for _ in range(b):
        ref_op.retnet_bwd_ref(q, k, v, mask, do)
    t2 = time.perf_counter()
    fwd = 2.0 * b * h * s * s * (dqk + dv)
    bwd = 2.0 * b * h * s * s * (3 * dqk + 2 * dv)
    return {"value": round((fwd + bwd) / (t2 - t0) / 1e12, 4), "unit": "TFLOP/s (dense-mask count)", "cores": torch.get_num_threads(), "kind": "port",
            "fwd_ms": round((t1 - t0) * 1e3, 1), "bwd_ms": round((t2 - t1) * 1e3, 1),
            "sample": f"oracle retnet_ref + retnet_bwd_ref fp32, all {b * h} (batch,head) slices of S={s} d_qk={dqk} d_v={dv}, one pass"}


def extra(ms_timing, flops, peak=PEAK_TFLOPS, issued_ratio=None, **more):
    """One side measurement: median per-call GPU time and its roofline fraction on the algorithmic count."""
    ms = ms_timing.median
    out = {"ms": round(ms, 5), "p20_ms": round(ms_timing.quantile(0.2), 5), "p80_ms": round(ms_timing.quantile(0.8), 5),
           "tflops": round(flops / ms / 1e9, 1),
           "roofline": {"bound": "mfma", "achieved": round(flops / ms / 1e9, 1), "peak": peak, "unit": "TFLOP/s",
                        "frac": round(flops / ms / 1e9 / peak, 4), "algorithmic_flops": flops}}
    if issued_ratio is not None:                  # matrix work the kernels issue / the algorithmic count
        out["roofline"]["issued_over_algorithmic"] = issued_ratio
    out.update(more)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=300)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the causal / long-kv / RetNet side measurements")
    ap.add_argument("--no-flush-pass", action="store_true", help="skip the second headline measurement (L2 flushed before each launch)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run plain 256 MiB device copies, so a profiler's HBM byte counters can be scaled by a known transfer")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py measures one GPU: the path has no cross-GPU component (batch x head slices are independent); run with --gpus 1")
        sys.exit(2)

    os.environ.setdefault("AAT_NO_JIT", "1")     # a missing library is an error here, never a compile inside a measurement
    import torch
    import attention_autotuner_amd as aat
    from attention_autotuner_amd.autotuner import Runtime

    if not torch.cuda.is_available():
        log("bench.py needs a GPU")
        sys.exit(1)
    arch = aat.MI355X()
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)

    def mk(*shape):
        return torch.randn(*shape, generator=g).half().to(dev)

    q, k, v = mk(B, H, S, D), mk(B, H, S, D), mk(B, H, S, D)
    o = torch.empty(B, H, S, D, dtype=torch.float16, device=dev)
    scale = 1.0 / math.sqrt(D)

    if args.copy_calibration:
        src = torch.empty(128 * 1024 * 1024, dtype=torch.float16, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)                      # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    cfg = resolve_config(aat, arch, [q, k, v, o], False)
    rt = Runtime(arch, cfg)
    log(f"config: {cfg!r}")

    step = rt.bind([q, k, v, o], softmax_scale=scale, causal=False)     # one kernel_entry_ex call per step

    hot = time_launches(step, args.steps, args.warmup)
    from attention_autotuner_amd.benchmarks.do_bench import gpu_state_under_load
    hot.sclk_mhz, hot.power_w = gpu_state_under_load(step)
    flops = attn_flops(B, H, S, S, D, D)
    value = flops / (hot.wall_ms_per_call * 1e-3) / 1e12
    achieved = flops / (hot.mean * 1e-3) / 1e12
    log(f"attention fwd non-causal: {hot.wall_ms_per_call:.4f} ms/step wall, {hot.mean:.4f} ms/launch mean "
        f"(median {hot.median:.4f}, p20 {hot.quantile(0.2):.4f}, p80 {hot.quantile(0.8):.4f}; warm-up {hot.warmup_calls} launches / {hot.warmup_ms:.0f} ms; "
        f"sclk {hot.sclk_mhz and round(hot.sclk_mhz)} MHz, {hot.power_w and round(hot.power_w)} W) -> {achieved:.1f} TFLOP/s = {100 * achieved / PEAK_TFLOPS:.1f}% of peak")
    timing = {"hot_l2": hot.summary()}
    if not args.no_flush_pass:
        cold = time_launches(step, args.steps, args.warmup, flush_l2=True)
        timing["l2_flushed"] = dict(cold.summary(), tflops_median=round(flops / cold.median / 1e9, 1))
        log(f"  with a 256 MB write before each launch: median {cold.median:.4f} ms (p20 {cold.quantile(0.2):.4f}, p80 {cold.quantile(0.8):.4f}) "
            f"-> {flops / cold.median / 1e9:.1f} TFLOP/s")

    extras = {}
    if not args.no_extras:
        try:
            extras.update(side_measurements(aat, arch, Runtime, mk, max(20, args.steps // 4), max(5, args.warmup // 4)))
        except Exception as e:                       # side numbers never invalidate the headline
            log(f"side measurements failed: {e!r}")

    traffic, traffic_source = measured_traffic(cfg, 2 * (q.numel() + k.numel() + v.numel() + o.numel()))
    out = {
        "metric": "attention fwd TFLOP/s (B4 H32 S2048 D128 fp16, non-causal)",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(hot.wall_ms_per_call, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16", "data": "synthetic",
        "config": {"workload": "configs[1]: flash-attention forward q,k,v [4,32,2048,128] fp16 N(0,1), scale 1/sqrt(128), non-causal",
                   "kernel_config": str(cfg), "pct_of_fp16_mfma_peak": round(100 * value / PEAK_TFLOPS, 2),
                   "min_warmup_ms": MIN_WARMUP_MS},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_TFLOPS, 4), "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": "flashattn_fwd_" + ("regfuse" if cfg.fuse_type == "register" else "smemfuse"),
                     "launch_ms": round(hot.mean, 5), "algorithmic_flops_per_launch": flops},
        "timing": timing,
        "extras": extras,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
        log(f"cpu baseline: {out['cpu_baseline']}")
        if not args.no_extras:
            try:
                extras["cpu_baseline_retnet_fwd_bwd_b4h8s2048_dqk256_dv512"] = cpu_baseline_retnet()
                log(f"cpu baseline, retnet fwd+bwd: {extras['cpu_baseline_retnet_fwd_bwd_b4h8s2048_dqk256_dv512']}")
            except Exception as e:                   # a side number: never invalidates the headline
                log(f"retnet cpu baseline failed: {e!r}")
    print(json.dumps(out), flush=True)


def side_measurements(aat, arch, Runtime, mk, steps, warmup):
    """Causal headline, the long-kv shape and RetNet forward/backward, when their kernels exist."""
    import torch
    res = {}
    q, k, v = mk(B, H, S, D), mk(B, H, S, D), mk(B, H, S, D)
    o = torch.empty_like(q)
    cfg = resolve_config(aat, arch, [q, k, v, o], True)
    rt = Runtime(arch, cfg)
    t = time_launches(lambda: rt.apply([q, k, v, o], causal=True), steps, warmup)
    res["attn_causal_b4h32s2048d128"] = extra(t, attn_flops(B, H, S, S, D, D, True), config=str(cfg))
    log(f"attention fwd causal: {t.median:.4f} ms -> {res['attn_causal_b4h32s2048d128']['tflops']} TFLOP/s")

    q5, k5, v5 = mk(1, 32, 256, D), mk(1, 32, 16384, D), mk(1, 32, 16384, D)
    o5 = torch.empty_like(q5)
    cfg5 = resolve_config(aat, arch, [q5, k5, v5, o5], False)
    rt5 = Runtime(arch, cfg5)
    t = time_launches(lambda: rt5.apply([q5, k5, v5, o5]), steps, warmup)
    bytes5 = 2 * (q5.numel() + k5.numel() + v5.numel() + o5.numel())
    e5 = extra(t, attn_flops(1, 32, 256, 16384, D, D), config=str(cfg5), gbps=round(bytes5 / t.median / 1e6, 1))
    e5["roofline"] = {"bound": "hbm", "achieved": round(bytes5 / t.median / 1e6, 1), "peak": 8000.0, "unit": "GB/s",
                      "frac": round(bytes5 / t.median / 1e6 / 8000.0, 4), "algorithmic_bytes": bytes5}
    res["attn_longkv_b1h32q256k16384d128"] = e5
    log(f"attention fwd long-kv: {t.median:.4f} ms -> {e5['tflops']} TFLOP/s, {e5['gbps']} GB/s")
    # shorter rows (the configuration this problem resolves to: the wrapper takes its persistent-block kernel there)
    qs, ks, vs = mk(16, H, 512, D), mk(16, H, 512, D), mk(16, H, 512, D)
    os_ = torch.empty_like(qs)
    rts = Runtime(arch, resolve_config(aat, arch, [qs, ks, vs, os_], False))
    t = time_launches(lambda: rts.apply([qs, ks, vs, os_]), steps, warmup)
    res["attn_short_rows_b16h32s512d128"] = extra(t, attn_flops(16, H, 512, 512, D, D), config=str(rts.config))
    log(f"attention fwd S=512 B=16: {t.median:.4f} ms -> {res['attn_short_rows_b16h32s512d128']['tflops']} TFLOP/s")
    res.update(attention_backward_measurement(aat, arch, mk, steps, warmup))
    res.update(retnet_measurements(aat, arch, mk, steps, warmup))
    res.update(retnet_recurrent_measurement(aat, steps, warmup))
    return res


def retnet_recurrent_measurement(aat, steps, warmup):
    """RetNet recurrent form at the shape of the reference's own bench (benchmarks/retnet/retnet.cu:236:
    B 8, H 32, L 2048, 128 key and value dims, fp32).  5 flops per (position, key dim, value dim): the
    recurrence's two multiply-adds and one multiply; fp32 MFMA peak 157.3 TFLOP/s."""
    import torch
    if not hasattr(aat, "retnet_recurrent_fwd"):
        return {}
    b, h, kd, vd, seqlen = 8, 32, 128, 128, 2048
    g = torch.Generator(device="cuda").manual_seed(11)
    q, k = (torch.rand(b, h, kd, seqlen, generator=g, device="cuda") * 2 - 1 for _ in range(2))
    v = torch.rand(b, h, vd, seqlen, generator=g, device="cuda") * 2 - 1
    decay = (1.0 - 2.0 ** (-5.0 - torch.arange(h, dtype=torch.float32, device="cuda"))).unsqueeze(1).expand(h, seqlen).contiguous()
    out = torch.empty_like(v)
    ws = torch.empty(h * (seqlen // 32) * 5120, dtype=torch.uint8, device="cuda")
    t = time_launches(lambda: aat.retnet_recurrent_fwd(q, k, v, decay, out=out, workspace=ws), steps, warmup)
    flops = 5.0 * b * h * seqlen * kd * vd
    nbytes = 4.0 * (q.numel() + k.numel() + v.numel() + out.numel())
    res = extra(t, flops, peak=157.3, gbps=round(nbytes / t.median / 1e6, 1))
    res["frac_of_fp32_mfma_peak"] = res["roofline"]["frac"]
    log(f"retnet recurrent fwd: {t.median:.4f} ms -> {res['tflops']} TFLOP/s ({res['gbps']} GB/s)")
    return {"retnet_recurrent_b8h32s2048_dqk128_dv128_f32": res}


def attention_backward_measurement(aat, arch, mk, steps, warmup):
    """Forward + backward of the headline problem through the operator (autograd), non-causal."""
    q, k, v, do = (mk(B, H, S, D) for _ in range(4))
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    fwd, bwd = attn_flops(B, H, S, S, D, D), 2.0 * B * H * S * S * (3 * D + 2 * D)

    def reset():
        q.grad = k.grad = v.grad = None

    t = time_launches(lambda: aat.flash_attn_func(q, k, v, arch).backward(do), steps, warmup, before_each=reset)
    log(f"attention fwd+bwd: {t.median:.4f} ms -> {(fwd + bwd) / t.median / 1e9:.1f} TFLOP/s")
    # the column and the row kernel both evaluate S and dP: 7 contractions issued for the 5 counted, plus the forward's 2
    return {"attn_fwd_bwd_b4h32s2048d128": extra(t, fwd + bwd, issued_ratio=round((2 + 7) / (2 + 5), 3))}


def retnet_decay_mask(heads, seq_q, seq_k, device):
    """D[h, n, m] = gamma_h^(n - m) for n >= m, else 0, gamma_h = 1 - 2^(-5-h); fp32 closed form rounded to fp16."""
    import torch
    gamma = 1.0 - torch.pow(2.0, -5.0 - torch.arange(heads, dtype=torch.float32, device=device))
    dist = (torch.arange(seq_q, device=device).unsqueeze(1) - torch.arange(seq_k, device=device).unsqueeze(0)).float()
    mask = torch.pow(gamma.view(-1, 1, 1), dist.clamp(min=0).unsqueeze(0)) * (dist >= 0).unsqueeze(0)
    return mask.half()


def retnet_measurements(aat, arch, mk, steps, warmup):
    import torch
    from attention_autotuner_amd.autotuner import gfx950_space
    res = {}
    if not hasattr(gfx950_space, "default_backward_config"):
        return res
    b, h, s, dqk, dv = 4, 8, 2048, 256, 512
    q, k, v, do = mk(b, h, s, dqk), mk(b, h, s, dqk), mk(b, h, s, dv), mk(b, h, s, dv)
    mask = retnet_decay_mask(h, s, s, "cuda")
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    fwd_flops = 2.0 * b * h * s * s * (dqk + dv)
    bwd_flops = 2.0 * b * h * s * s * (3 * dqk + 2 * dv)
    def reset():
        q.grad = k.grad = v.grad = None

    # Three chained backward passes evaluate dO V^T twice: 3 (d_qk + d_v) issued for the 3 d_qk + 2 d_v counted.  A
    # configuration that stores dS (ds_rows != 0 in the tuning cache entry the operator resolves to) issues the count.
    def issued_ratio(kind, c):
        name = f"best_config_{kind}_{arch.name}_{dqk}_{dv}_b{b}h{h}q{s}k{s}_c{c}.json"
        try:
            with open(os.path.join(os.path.dirname(os.path.abspath(aat.__file__)), "cache", name)) as f:
                stored = bool(json.load(f).get("ds_rows", 0))
        except (OSError, ValueError):
            stored = False
        bwd_issued = (3 * dqk + 2 * dv) if stored else 3 * (dqk + dv)
        return round(((dqk + dv) + bwd_issued) / ((dqk + dv) + 3 * dqk + 2 * dv), 3)
    half = "non-zero (lower-triangular) half of the dense-mask count"
    # The operator as the reference calls it: RetNetAttnFunc(q, k, v, mask, arch).  It scans the mask tensor for
    # all-zero tiles (one read of it, part of the timed call) and walks only the rest; the decay mask is zero above
    # the diagonal, so the roofline fraction is taken on half of the dense count.  The *_dense_walk entries
    # are the same operator told to walk every tile, as the reference's kernels do.
    with torch.no_grad():
        t = time_launches(lambda: aat.RetNetAttnFunc(q, k, v, mask, arch), steps, warmup)
    res["retnet_fwd_b4h8s2048_dqk256_dv512"] = extra(t, fwd_flops / 2, flops_counted=half, tflops_dense_count=round(fwd_flops / t.median / 1e9, 1))
    log(f"retnet fwd: {t.median:.4f} ms -> {fwd_flops / t.median / 1e9:.1f} TFLOP/s (dense-mask FLOPs; zero tiles skipped)")
    with torch.no_grad():
        t = time_launches(lambda: aat.RetNetAttnFunc(q, k, v, mask, arch, False), steps, warmup)
    res["retnet_fwd_dense_walk_b4h8s2048_dqk256_dv512"] = extra(t, fwd_flops)
    log(f"retnet fwd, dense walk: {t.median:.4f} ms -> {fwd_flops / t.median / 1e9:.1f} TFLOP/s")

    t = time_launches(lambda: aat.RetNetAttnFunc(q, k, v, mask, arch).backward(do), steps, warmup, before_each=reset)
    res["retnet_fwd_bwd_b4h8s2048_dqk256_dv512"] = extra(t, (fwd_flops + bwd_flops) / 2, issued_ratio=issued_ratio("retnet_bwd", 1), flops_counted=half,
                                                         tflops_dense_count=round((fwd_flops + bwd_flops) / t.median / 1e9, 1))
    log(f"retnet fwd+bwd: {t.median:.4f} ms -> {(fwd_flops + bwd_flops) / t.median / 1e9:.1f} TFLOP/s (dense-mask FLOPs; zero tiles skipped)")
    # a model applies one mask in every layer and step: the scan taken once and handed to every call
    scan = aat.retnet_mask_scan(mask, arch)
    t = time_launches(lambda: aat.RetNetAttnFunc(q, k, v, mask, arch, scan).backward(do), steps, warmup, before_each=reset)
    res["retnet_fwd_bwd_scan_reused_b4h8s2048_dqk256_dv512"] = extra(t, (fwd_flops + bwd_flops) / 2, issued_ratio=issued_ratio("retnet_bwd", 1),
                                                                     flops_counted=half)
    log(f"retnet fwd+bwd, mask scan reused: {t.median:.4f} ms")
    t = time_launches(lambda: aat.RetNetAttnFunc(q, k, v, mask, arch, False).backward(do), steps, warmup, before_each=reset)
    res["retnet_fwd_bwd_dense_walk_b4h8s2048_dqk256_dv512"] = extra(t, fwd_flops + bwd_flops, issued_ratio=issued_ratio("retnet_bwd", 0))
    log(f"retnet fwd+bwd, dense walk: {t.median:.4f} ms -> {(fwd_flops + bwd_flops) / t.median / 1e9:.1f} TFLOP/s")

    if hasattr(aat, "RetNetDecayAttnFunc"):              # the same decay mask, built in registers from one rate per head
        gamma = 1.0 - torch.pow(2.0, -5.0 - torch.arange(h, dtype=torch.float64))
        t = time_launches(lambda: aat.RetNetDecayAttnFunc(q, k, v, gamma, arch).backward(do), steps, warmup, before_each=reset)
        # tiles above the diagonal are skipped: the roofline fraction is taken on half the dense count
        res["retnet_decay_fwd_bwd_b4h8s2048_dqk256_dv512"] = extra(t, (fwd_flops + bwd_flops) / 2, issued_ratio=issued_ratio("retnet_bwd_decay", 1), flops_counted=half,
                                                                   tflops_dense_count=round((fwd_flops + bwd_flops) / t.median / 1e9, 1))
        log(f"retnet decay fwd+bwd: {t.median:.4f} ms -> {(fwd_flops + bwd_flops) / t.median / 1e9:.1f} TFLOP/s (dense-mask FLOPs)")
    return res


if __name__ == "__main__":
    main()
