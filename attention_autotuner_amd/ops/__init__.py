from .attention_interface import flash_attn_func, MultiHeadAttnFunc, REFERENCE_SOFTMAX_SCALE
from .retnet_interface import RetNetAttnFunc, RetNetAttn

__all__ = ["flash_attn_func", "MultiHeadAttnFunc", "RetNetAttnFunc", "RetNetAttn", "REFERENCE_SOFTMAX_SCALE"]
