"""Launcher for one configuration (reference python/autotuner/runtime.py:32-89).

``Runtime(arch, config).apply(torch_array)`` builds (or finds) the configuration's library and
enqueues one launch on the current PyTorch stream.  Unlike the reference, the dlopen handle is kept
for the life of the process, the return code of the kernel entry is checked, and a missing library
is an error -- there is no CPU fallback.
"""
import ctypes
import math
import os

import torch

from . import codegen, library


class KernelLaunchError(RuntimeError):
    pass


_ERRORS = {-2: "sequence lengths are not multiples of the configuration's tile (Br, Bc)",
           -3: "workspace missing or too small"}


# A RetNet backward built with a stored dS asks for B*H*S_q*S_kv fp16 on top of the mask scan and works without them
# (it then evaluates dS twice).  Beyond this many bytes the runtime does not grant the room on its own: a caller who
# wants it there passes a workspace of workspace_size() bytes.
MAX_DS_BYTES = int(os.environ.get("AAT_MAX_DS_BYTES", 2 << 30))


def _wanted(config, need, B, H, Sq, Sk):
    """Bytes of workspace the runtime provides when the caller's is missing or too small."""
    ds_bytes = 2 * B * H * Sq * Sk
    if getattr(config, "operation", "") == "ret_bwd" and getattr(config, "ds_rows", 0) and need >= ds_bytes > MAX_DS_BYTES:
        return need - ds_bytes
    return need


def _grown(workspace, need, device, keep):
    """A workspace of ``need`` bytes.  ``keep``: the one handed in holds a mask scan an earlier launch left (mode
    "scanned") and is smaller than this library wants (a backward that also stores dS): its bytes move to the head of
    the new one, where the library looks for them."""
    new = torch.empty(need, dtype=torch.uint8, device=device)
    if keep:
        if workspace is None:
            raise KernelLaunchError('mask mode "scanned" needs the workspace an earlier "scan" launch filled')
        old = workspace.reshape(-1).view(torch.uint8)
        new[:old.numel()].copy_(old)
    return new


class Runtime:
    def __init__(self, arch, config, tmp_dir=None, libname=None):
        self.arch = arch
        self.config = config
        self.tmp_dir = tmp_dir
        self.libname = libname
        self._lib = None                  # the loaded library and the workspace each problem shape needs, kept between calls
        self._need = {}
        self._asks = {}
        if self.libname is None:
            self.libname = self.compile()
        if self.libname is None:
            log = codegen.library_path(config, tmp_dir)[:-3] + ".log"
            raise KernelLaunchError(f"could not build kernel library for {config.operation}:{config} (see {log})")

    def compile(self, timeout=None):
        return codegen.compile_config(self.config, self.arch, self.tmp_dir, timeout)

    def _path(self):
        if os.path.isabs(self.libname):
            return self.libname
        return os.path.join(self.tmp_dir or codegen.DEFAULT_BUILD_DIR, self.libname)

    def workspace_size(self, B, H, Sq, Sk):
        size = self._asks.get((B, H, Sq, Sk))
        if size is None:
            if self._lib is None:
                self._lib = library.load(self._path(), self.config.operation)
            size = self._asks[(B, H, Sq, Sk)] = int(self._lib.workspace_size(B, H, Sq, Sk))
        return size

    def apply(self, torch_array, device=None, softmax_scale=None, causal=False, workspace=None, lse=None, decay=False):
        """``lse`` (attention forward only): fp32 [B,H,S_q] tensor that receives the log-sum-exp of every row.
        ``decay`` (RetNet only): the mask slot of ``torch_array`` holds log2(gamma) [H] fp32 and the decay
        mask is built in registers; the backward's array then has no dqaccum entry."""
        q, k = torch_array[0], torch_array[1]
        if not q.is_cuda:
            raise KernelLaunchError("kernel libraries run on the GPU only; got CPU tensors")
        B, H, Sq, Sk = q.shape[0], q.shape[1], q.shape[2], k.shape[2]
        op = self.config.operation
        lib = self._lib
        if lib is None:
            lib = self._lib = library.load(self._path(), op)
        need = self._need.get((B, H, Sq, Sk))               # a property of the library and the problem: asked once
        if need is None:
            need = self._need[(B, H, Sq, Sk)] = _wanted(self.config, int(lib.workspace_size(B, H, Sq, Sk)), B, H, Sq, Sk)
        if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
            workspace = _grown(workspace, need, q.device, keep=causal == "scanned")
        ws_ptr = workspace.data_ptr() if workspace is not None else None
        ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
        if op in library.SCALED_OPS:
            scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(q.shape[-1])
            extra = (scale, int(bool(causal)))
        else:
            extra = (mask_mode(causal),)
        # the prototypes are set (library.py), so plain integers convert; the launch goes to the stream that is current
        # on the tensors' device, with that device current
        index = q.device.index
        other = index != torch.cuda.current_device()
        if other:
            previous = torch.cuda.current_device()
            torch.cuda.set_device(index)
        try:
            stream = torch._C._cuda_getCurrentRawStream(index)
            ptrs = [t.data_ptr() for t in torch_array]
            if decay:
                if op not in library.DECAY_OPS:
                    raise KernelLaunchError("only the RetNet operators have a decay-mask variant")
                rc = lib.kernel_entry_decay(*ptrs, B, H, Sq, Sk, ws_ptr, ws_bytes, stream)
            elif lse is not None:
                if op != "attn":
                    raise KernelLaunchError("only the attention forward writes a log-sum-exp")
                rc = lib.kernel_entry_lse(*ptrs, lse.data_ptr(), B, H, Sq, Sk, *extra, ws_ptr, ws_bytes, stream)
            else:
                rc = lib.kernel_entry_ex(*ptrs, B, H, Sq, Sk, *extra, ws_ptr, ws_bytes, stream)
        finally:
            if other:
                torch.cuda.set_device(previous)
        if rc != 0:
            raise KernelLaunchError(f"{op}:{self.config} failed with code {rc}: {_ERRORS.get(rc, 'HIP error')}")
        return rc


    def bind(self, torch_array, softmax_scale=None, causal=False, workspace=None):
        """A zero-argument callable that enqueues one launch of ``kernel_entry_ex`` on ``torch_array``:
        pointers, sizes, the workspace and the stream (the one current NOW) are converted once, so a
        call costs one foreign-function call -- what a serving loop that launches the same problem
        repeatedly would keep.  The tensors (and the returned callable's workspace) must stay alive."""
        q, k = torch_array[0], torch_array[1]
        if not q.is_cuda:
            raise KernelLaunchError("kernel libraries run on the GPU only; got CPU tensors")
        B, H, Sq, Sk = int(q.shape[0]), int(q.shape[1]), int(q.shape[2]), int(k.shape[2])
        op = self.config.operation
        lib = library.load(self._path(), op)
        need = _wanted(self.config, int(lib.workspace_size(B, H, Sq, Sk)), B, H, Sq, Sk)
        if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
            workspace = _grown(workspace, need, q.device, keep=causal == "scanned")
        args = [ctypes.c_void_p(t.data_ptr()) for t in torch_array] + [B, H, Sq, Sk]
        if op in library.SCALED_OPS:
            args.append(ctypes.c_float(softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(q.shape[-1])))
        args += [ctypes.c_int(int(bool(causal)) if op in library.SCALED_OPS else mask_mode(causal)),
                 ctypes.c_void_p(workspace.data_ptr() if workspace is not None else 0),
                 ctypes.c_size_t(workspace.numel() * workspace.element_size() if workspace is not None else 0)]
        with torch.cuda.device(q.device):
            args.append(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        entry, keep, name = lib.kernel_entry_ex, (list(torch_array), workspace), f"{op}:{self.config}"

        def launch():
            rc = entry(*args)
            if rc != 0:
                raise KernelLaunchError(f"{name} failed with code {rc}: {_ERRORS.get(rc, 'HIP error')}")

        launch.keep_alive = keep
        return launch


MASK_MODES = {"dense": 0, "causal": 1, "scan": 2, "scanned": 3}


def mask_mode(causal):
    """The integer the *_ex entry points take as ``causal``: False / True, or for the RetNet operators one of
    "dense", "causal", "scan" (scan the mask tensor for all-zero tiles first, into the workspace) and
    "scanned" (the workspace holds that scan already)."""
    if isinstance(causal, str):
        return MASK_MODES[causal]
    return int(bool(causal))


def compile_parallel(configs, arch, tmp_dir=None):
    return codegen.compile_parallel(configs, arch, tmp_dir)
