"""End-to-end attention benchmark through the public operator, against PyTorch's own GPU attention
(counterpart of reference python/benchmarks/bench_attention.py:34-114).

    python -m attention_autotuner_amd.benchmarks.bench_attention [--causal] [--bwd] [--dims 64 128 192 256]
"""
import argparse
import math

import torch
import torch.nn.functional as F

from .. import MI355X, flash_attn_func
from ..utils import max_abs_err
from .do_bench import do_bench


def torch_attention(q, k, v, scale, causal):
    return F.scaled_dot_product_attention(q, k, v, scale=scale, is_causal=causal)


def run(batch, heads, seq_q, seq_k, dim_qk, dim_v, causal, arch, bwd=False):
    q = torch.randn(batch, heads, seq_q, dim_qk, device="cuda", dtype=torch.float16, requires_grad=bwd)
    k = torch.randn(batch, heads, seq_k, dim_qk, device="cuda", dtype=torch.float16, requires_grad=bwd)
    v = torch.randn(batch, heads, seq_k, dim_v, device="cuda", dtype=torch.float16, requires_grad=bwd)
    scale = 1.0 / math.sqrt(dim_qk)
    o = flash_attn_func(q, k, v, arch, causal, scale)
    err = None
    if dim_qk == dim_v:                                         # torch's fused kernels want equal head sizes
        err = max_abs_err(o, torch_attention(q.float(), k.float(), v.float(), scale, causal))
    flops = 2.0 * batch * heads * seq_q * seq_k * (dim_qk + dim_v) * (0.5 if causal else 1.0)
    with torch.no_grad():
        ms, p20, p80 = do_bench(lambda: flash_attn_func(q, k, v, arch, causal, scale), quantiles=[0.5, 0.2, 0.8])
    line = f"d_qk={dim_qk:3d} d_v={dim_v:3d} causal={int(causal)}  ours {ms:.4f} ms [{p20:.4f}, {p80:.4f}] {flops / ms / 1e9:7.1f} TFLOP/s"
    if dim_qk == dim_v:
        with torch.no_grad():
            ref_ms = do_bench(lambda: torch_attention(q, k, v, scale, causal), quantiles=[0.5])
        line += f"   torch sdpa {ref_ms:.4f} ms {flops / ref_ms / 1e9:7.1f} TFLOP/s   max|err| vs fp32 {err:.2e}"
    print(line, flush=True)
    if not bwd:
        return
    # forward + backward (reference python/benchmarks/bench_attention.py:42-71 times the backward of a kept forward; the
    # operator here has no such split, so both sides are timed as the training step runs them)
    do = torch.randn(batch, heads, seq_q, dim_v, device="cuda", dtype=torch.float16)
    both = 3.5 * flops                                           # 2 (d_qk + d_v) forward + (3 d_qk + 2 d_v) backward at d_qk = d_v
    if dim_qk != dim_v:
        both = flops * (4.0 * dim_qk + 3.0 * dim_v) / (dim_qk + dim_v)
    try:
        ms = do_bench(lambda: flash_attn_func(q, k, v, arch, causal, scale).backward(do), grad_to_none=[q, k, v], quantiles=[0.5])
    except NotImplementedError as e:                             # head sizes the backward does not take
        print(f"d_qk={dim_qk:3d} d_v={dim_v:3d} causal={int(causal)}  fwd+bwd: {e}", flush=True)
        return
    line = f"d_qk={dim_qk:3d} d_v={dim_v:3d} causal={int(causal)}  fwd+bwd ours {ms:.4f} ms {both / ms / 1e9:7.1f} TFLOP/s"
    if dim_qk == dim_v:
        ref_ms = do_bench(lambda: torch_attention(q, k, v, scale, causal).backward(do), grad_to_none=[q, k, v], quantiles=[0.5])
        line += f"   torch sdpa {ref_ms:.4f} ms {both / ref_ms / 1e9:7.1f} TFLOP/s"
    print(line, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--causal", action="store_true")
    ap.add_argument("--bwd", action="store_true", help="also time forward + backward")
    ap.add_argument("--dims", type=int, nargs="*", default=[64, 128, 192, 256])
    ap.add_argument("--shape", type=int, nargs=4, default=[4, 8, 2048, 2048], metavar=("B", "H", "Sq", "Sk"))
    args = ap.parse_args()
    torch.manual_seed(0)
    arch = MI355X()
    for d in args.dims:
        run(*args.shape, d, d, args.causal, arch, args.bwd)


if __name__ == "__main__":
    main()
