"""End-to-end RetNet benchmark through the public operator (forward and forward+backward), against
the same math in plain PyTorch on the GPU (counterpart of reference python/benchmarks/bench_retnet.py:32-116).

    python -m attention_autotuner_amd.benchmarks.bench_retnet [--dims 64 128 192 256] [--dv 512]
"""
import argparse

import torch

from .. import MI355X, RetNetAttnFunc
from ..utils import max_abs_err
from .do_bench import do_bench


def torch_retnet(q, k, v, mask):
    s = (q @ k.transpose(-1, -2)) * mask
    r = s.detach().abs().sum(dim=-1, keepdim=True).clamp(min=1.0)
    return (s / r) @ v


def decay_mask(heads, seq_q, seq_k, device):
    n = torch.arange(seq_q, device=device, dtype=torch.float64).view(1, seq_q, 1)
    m = torch.arange(seq_k, device=device, dtype=torch.float64).view(1, 1, seq_k)
    gamma = (1.0 - torch.pow(2.0, -5.0 - torch.arange(heads, device=device, dtype=torch.float64))).view(heads, 1, 1)
    d = torch.where(n >= m, gamma ** (n - m).clamp(min=0), torch.zeros((), device=device, dtype=torch.float64))
    return d.float().half()


def run(batch, heads, seq_q, seq_k, dim_qk, dim_v, arch, causal):
    mk = lambda *s: torch.randn(*s, device="cuda", dtype=torch.float16, requires_grad=True)
    q, k, v = mk(batch, heads, seq_q, dim_qk), mk(batch, heads, seq_k, dim_qk), mk(batch, heads, seq_k, dim_v)
    do = torch.randn(batch, heads, seq_q, dim_v, device="cuda", dtype=torch.float16)
    mask = decay_mask(heads, seq_q, seq_k, "cuda")
    o = RetNetAttnFunc(q, k, v, mask, arch, causal)
    o_ref = torch_retnet(q.float(), k.float(), v.float(), mask.float())
    err = max_abs_err(o, o_ref)
    fwd = 2.0 * batch * heads * seq_q * seq_k * (dim_qk + dim_v)
    bwd = 2.0 * batch * heads * seq_q * seq_k * (3 * dim_qk + 2 * dim_v)
    with torch.no_grad():
        ms_f = do_bench(lambda: RetNetAttnFunc(q, k, v, mask, arch, causal), quantiles=[0.5])
        ref_f = do_bench(lambda: torch_retnet(q, k, v, mask), quantiles=[0.5])
    ms_fb = do_bench(lambda: RetNetAttnFunc(q, k, v, mask, arch, causal).backward(do), grad_to_none=[q, k, v], quantiles=[0.5])
    ref_fb = do_bench(lambda: torch_retnet(q, k, v, mask).backward(do), grad_to_none=[q, k, v], quantiles=[0.5])
    print(f"d_qk={dim_qk:3d} d_v={dim_v:3d}  fwd {ms_f:.4f} ms {fwd / ms_f / 1e9:6.1f} TFLOP/s (torch {ref_f:.3f} ms)   "
          f"fwd+bwd {ms_fb:.4f} ms {(fwd + bwd) / ms_fb / 1e9:6.1f} TFLOP/s (torch {ref_fb:.3f} ms)   max|err| fwd {err:.2e}")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--dims", type=int, nargs="*", default=[64, 128, 192, 256])
    ap.add_argument("--dv", type=int, default=None, help="value head size (default: same as d_qk)")
    ap.add_argument("--shape", type=int, nargs=4, default=[4, 8, 2048, 2048], metavar=("B", "H", "Sq", "Sk"))
    ap.add_argument("--causal", action="store_true", help="promise a lower-triangular mask so tiles above the diagonal are skipped")
    args = ap.parse_args()
    torch.manual_seed(0)
    arch = MI355X()
    for d in args.dims:
        run(*args.shape, d, args.dv or d, arch, args.causal)


if __name__ == "__main__":
    main()
