from .attention_interface import flash_attn_func, MultiHeadAttnFunc, REFERENCE_SOFTMAX_SCALE
from .retnet_interface import RetNetAttnFunc, RetNetAttn, RetNetDecayAttnFunc, RetNetDecayAttn

__all__ = ["flash_attn_func", "MultiHeadAttnFunc", "RetNetAttnFunc", "RetNetAttn", "RetNetDecayAttnFunc", "RetNetDecayAttn", "REFERENCE_SOFTMAX_SCALE"]
