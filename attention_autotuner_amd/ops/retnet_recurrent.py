"""``retnet_recurrent_fwd(q, k, v, decay[, device_type[, block_kdim]])`` -- RetNet recurrent form, fp32.

``S_n = decay[h, n] * S_{n-1} + k_n^T v_n``, ``out_n = q_n S_n`` over the first ``block_kdim`` key dims,
with the tensors laid out as the reference's kernel takes them: q, k [B, H, kdim, L], v [B, H, vdim, L]
(sequence contiguous), decay [H, L]; returns out [B, H, vdim, L].

The reference has no Python operator for this path: ``retnet_recurrent_fwd`` is an ``extern "C"`` function
(reference csrc/kernels/retnet/recurrent/recurrent.h:427-463) called from its C++ benchmark only
(benchmarks/retnet/retnet.cu:175-215).  This wrapper binds the same-named entry points of the MI355X
library for PyTorch callers: no autograd, GPU only, no CPU fallback.
"""
import ctypes

import torch

from ..arch import MI355X
from ..autotuner import codegen, library
from ..autotuner.configs import RetRecurrentConfig
from ..autotuner.runtime import KernelLaunchError

_ERRORS = {-2: "unsupported shape: L must be a multiple of 32 (at most 131072), block_kdim a multiple of 64 up to 256 "
               "and <= kdim, vdim a multiple of 64",
           -3: "workspace missing or too small"}


def _library(device_type):
    cfg = RetRecurrentConfig()
    path = codegen.compile_config(cfg, device_type)
    if path is None:
        raise KernelLaunchError(f"could not build kernel library for {cfg.operation}:{cfg} "
                                f"(see {codegen.library_path(cfg)[:-3]}.log)")
    return library.load_recurrent(path)


def workspace_size(nheads, seqlen, device_type=None, batch=1, kdim=128, vdim=128, block_kdim=None):
    """Bytes of workspace one call needs: the decay factors of every (head, 32-position chunk) and, beyond 128
    key dims, a second output-sized buffer (0 for an unsupported shape)."""
    return int(_library(device_type or MI355X()).retnet_recurrent_workspace_size(batch, nheads, kdim, vdim, seqlen,
                                                                                  int(block_kdim or kdim)))


def retnet_recurrent_fwd(q, k, v, decay, device_type=None, block_kdim=None, out=None, workspace=None):
    if not (q.is_cuda and k.is_cuda and v.is_cuda and decay.is_cuda):
        raise RuntimeError("retnet_recurrent_fwd runs on the GPU only (HIP kernels); move q, k, v, decay to a cuda device")
    for t in (q, k, v, decay):
        assert t.dtype == torch.float32, "the recurrent form computes in fp32 (reference recurrent.h:16-17)"
    q, k, v, decay = [x.contiguous() for x in (q, k, v, decay)]
    batch, nheads, kdim, seqlen = q.shape
    vdim = v.shape[2]
    assert k.shape == q.shape and v.shape == (batch, nheads, vdim, seqlen) and decay.shape == (nheads, seqlen)
    block_kdim = int(block_kdim or kdim)
    lib = _library(device_type or MI355X())
    if out is None:
        out = torch.empty_like(v)
    assert out.shape == v.shape and out.dtype == torch.float32 and out.is_contiguous() and out.device == v.device
    need = int(lib.retnet_recurrent_workspace_size(batch, nheads, kdim, vdim, seqlen, block_kdim))
    if workspace is None or workspace.numel() * workspace.element_size() < need:
        workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=q.device)
    with torch.cuda.device(q.device):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.retnet_recurrent_fwd_ex(*[ctypes.c_void_p(t.data_ptr()) for t in (q, k, v, decay, out)], batch, nheads, kdim,
                                         vdim, seqlen, block_kdim, ctypes.c_void_p(workspace.data_ptr()),
                                         ctypes.c_size_t(workspace.numel() * workspace.element_size()), stream)
    if rc != 0:
        raise KernelLaunchError(f"retnet_recurrent_fwd failed with code {rc}: {_ERRORS.get(rc, 'HIP error')}")
    return out
