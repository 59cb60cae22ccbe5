"""Per-operator tuners (reference python/autotuner/tunner.py:13-225).

Each tuner enumerates the gfx950 space for a ROCm descriptor.  A descriptor of another platform may bring
its own space along (``arch.search_space``: a module with ``forward_candidates`` / ``forward_valid`` /
``backward_candidates`` / ``backward_valid``); such configurations can be enumerated, which is how the
test suite replays the reference's published NVIDIA tuning logs, but not built: ``tune`` refuses.
"""
import ctypes
import math
import os

from . import codegen, gfx950_space
from .base_tunner import BaseTunner


def _is_rocm(arch):
    return getattr(arch, "platform", "") == "ROCm"


def _foreign_space(arch):
    space = getattr(arch, "search_space", None)
    if space is None:
        raise RuntimeError(f"{arch.name}: no search space for platform {getattr(arch, 'platform', '?')!r}")
    return space


class _ForwardTunner(BaseTunner):
    def __init__(self, arch, torch_array, op_name, **kw):
        super().__init__(arch, torch_array, op_name, **kw)
        if _is_rocm(arch):
            self.Br_list = list(gfx950_space.BR_LIST)
            self.Bc_list = list(gfx950_space.BC_LIST)

    def generate_configs(self, Br, Bc, dim_qk, dim_v):
        if not _is_rocm(self.arch):
            return _foreign_space(self.arch).forward_candidates(self.operation, Br, Bc, dim_qk, dim_v)
        return gfx950_space.forward_candidates(self.operation, Br, Bc, dim_qk, dim_v, with_splits=self._wants_splits(Br))

    def _wants_splits(self, Br):
        """kv splitting is worth trying when the row blocks alone cannot occupy the chip."""
        s = self.problem_shape
        blocks = s["B"] * s["H"] * max(1, s["Sq"] // Br)
        return self.operation == "attn" and not self.causal and blocks < 2 * self.arch.compute_max_core

    def _validate(self, config):
        space = gfx950_space if _is_rocm(self.arch) else _foreign_space(self.arch)
        return space.forward_valid(config, self.arch)

    validate_register_fuse = _validate
    validate_shared_fuse = _validate

    def _kernel_matters(self, mangled):
        flags = codegen.template_bools(mangled)
        if self.operation == "ret":                       # <..., DECAY>
            return not flags or flags[-1] == bool(self.decay)
        if "flashattn_fwd_regfuse" in mangled and len(flags) == 5:     # <..., PIPE, CAUSAL, SPLIT, PERSIST, PAIR>
            # the persistent and the paired variant are not launched from a build that spills (the wrapper asks the runtime)
            return flags[1] == bool(self.causal) and not flags[3] and not flags[4]
        if "flashattn_fwd_smemfuse" in mangled and flags:              # <..., CAUSAL>
            return flags[-1] == bool(self.causal)
        return True

    def tune(self, *a, **kw):
        if not _is_rocm(self.arch):
            raise RuntimeError(f"{self.arch.name} configurations can be enumerated but not built on this platform")
        return super().tune(*a, **kw)


def _shipped_cost_model(self):
    """The fitted model ``cost_model_file`` next to the tuning cache, or None (no file, another platform,
    AAT_TUNE_PRUNE=0)."""
    if self.cost_model_file is None:
        return None
    path = os.path.join(self.cost_model_dir, self.cost_model_file)
    if not (_is_rocm(self.arch) and os.environ.get("AAT_TUNE_PRUNE", "1") != "0" and os.path.exists(path)):
        return None
    from .costmodel import CostModel
    try:
        return CostModel.load(path)
    except (OSError, ValueError, KeyError):
        return None


class AttnTunner(_ForwardTunner):
    operation = "attn"
    # the space has a few hundred candidates: with a fitted cost model next to the tuning cache, only the
    # third it ranks best is built and timed (AAT_TUNE_PRUNE=0: time everything, as the reference does)
    cost_model_file = "costmodel_attn.json"
    _shipped_cost_model = _shipped_cost_model

    def __init__(self, arch, torch_array, causal=False, softmax_scale=None):
        super().__init__(arch, torch_array, "attention", causal=causal, softmax_scale=softmax_scale)

    def _ex_args(self):
        scale = self.softmax_scale
        if scale is None:
            scale = 1.0 / math.sqrt(self.problem_key["dim_qk"])
        return [ctypes.c_float(scale), ctypes.c_int(int(self.causal))]


class RetTunner(_ForwardTunner):
    operation = "ret"
    cost_model_file = "costmodel_ret.json"
    _shipped_cost_model = _shipped_cost_model

    def __init__(self, arch, torch_array, causal=False, decay=False, mask_mode=None):
        super().__init__(arch, torch_array, "retnet", causal=causal or decay, decay=decay, mask_mode=mask_mode)


class RetBwdTunner(BaseTunner):
    operation = "ret_bwd"
    cost_model_file = "costmodel_ret_bwd.json"
    _shipped_cost_model = _shipped_cost_model

    def __init__(self, arch, torch_array, causal=False, decay=False, mask_mode=None):
        super().__init__(arch, torch_array, "retnet_bwd", causal=causal or decay, decay=decay, mask_mode=mask_mode)
        if _is_rocm(arch):
            self.Br_list = list(getattr(gfx950_space, "BWD_BR_LIST", (64, 128)))
            self.Bc_list = list(getattr(gfx950_space, "BWD_BC_LIST", (32, 64, 128)))

    def generate_configs(self, Br, Bc, dim_qk, dim_v):
        if _is_rocm(self.arch):
            return gfx950_space.backward_candidates(Br, Bc, dim_qk, dim_v)
        return _foreign_space(self.arch).backward_candidates(Br, Bc, dim_qk, dim_v)

    def validate_kernel(self, config):
        if _is_rocm(self.arch):
            return gfx950_space.backward_valid(config, self.arch)
        return _foreign_space(self.arch).backward_valid(config, self.arch)

    def _kernel_matters(self, mangled):                   # ret_bwd_chain<..., PASS, WPE, DECAY, DS_OUT>; the dK-from-dS kernel has no flags
        flags = codegen.template_bools(mangled)
        return len(flags) != 2 or flags[0] == bool(self.decay)

    def tune(self, *a, **kw):
        if not _is_rocm(self.arch):
            raise RuntimeError(f"{self.arch.name} configurations can be enumerated but not built on this platform")
        return super().tune(*a, **kw)


class AttnBwdTunner(BaseTunner):
    """Tuner for the flash-attention backward (no reference counterpart: reference
    python/ops/attention_interface.py:37-58 leaves the operator empty).  ``torch_array`` is
    [q, k, v, o, dO, lse, dq, dk, dv]."""
    operation = "attn_bwd"
    cost_model_file = "costmodel_attn_bwd.json"
    _shipped_cost_model = _shipped_cost_model

    def __init__(self, arch, torch_array, causal=False, softmax_scale=None):
        super().__init__(arch, torch_array, "attention_bwd", causal=causal, softmax_scale=softmax_scale)
        self.Br_list = list(gfx950_space.ATTN_BWD_BR_LIST)
        self.Bc_list = list(gfx950_space.ATTN_BWD_BC_LIST)

    def generate_configs(self, Br, Bc, dim_qk, dim_v):
        return gfx950_space.attn_backward_candidates(Br, Bc, dim_qk, dim_v)

    def validate_kernel(self, config):
        return gfx950_space.attn_backward_valid(config, self.arch)

    def _ex_args(self):
        scale = self.softmax_scale
        if scale is None:
            scale = 1.0 / math.sqrt(self.problem_key["dim_qk"])
        return [ctypes.c_float(scale), ctypes.c_int(int(self.causal))]

    def tune(self, *a, **kw):
        if not _is_rocm(self.arch):
            raise RuntimeError(f"{self.arch.name} has no attention-backward kernels")
        return super().tune(*a, **kw)
