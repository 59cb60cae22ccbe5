from .attention_interface import flash_attn_func, MultiHeadAttnFunc, REFERENCE_SOFTMAX_SCALE
from .retnet_interface import RetNetAttnFunc, RetNetAttn, RetNetDecayAttnFunc, RetNetDecayAttn, retnet_mask_scan
from .retnet_recurrent import retnet_recurrent_fwd

__all__ = ["flash_attn_func", "MultiHeadAttnFunc", "RetNetAttnFunc", "RetNetAttn", "RetNetDecayAttnFunc", "RetNetDecayAttn", "retnet_mask_scan", "retnet_recurrent_fwd",
           "REFERENCE_SOFTMAX_SCALE"]
