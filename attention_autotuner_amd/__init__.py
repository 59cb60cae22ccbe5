"""MI355X-native fused attention / RetNet kernels with an autotuner.

Public surface (same names as the reference's python/ tree):
    flash_attn_func(q, k, v, device_type[, causal[, softmax_scale]])
    RetNetAttnFunc(q, k, v, mask, device_type[, causal])      (causal may be a scan from retnet_mask_scan(mask, device_type))
    RetNetDecayAttnFunc(q, k, v, gamma, device_type)          (decay mask built on the fly; not in the reference)
    retnet_recurrent_fwd(q, k, v, decay)                      (recurrent form, fp32; the reference's C entry point of that name)
    arch.MI355X, autotuner.{AttnTunner, RetTunner, RetBwdTunner, Runtime, AttnConfig, RetConfig, RetBwdConfig}
"""
from . import arch, autotuner, ops, utils
from .arch import MI355X, Arch
from .ops import flash_attn_func, RetNetAttnFunc, RetNetDecayAttnFunc, retnet_mask_scan, retnet_recurrent_fwd, REFERENCE_SOFTMAX_SCALE

__all__ = ["arch", "autotuner", "ops", "utils", "MI355X", "Arch", "flash_attn_func", "RetNetAttnFunc", "RetNetDecayAttnFunc", "retnet_mask_scan",
           "retnet_recurrent_fwd", "REFERENCE_SOFTMAX_SCALE"]
