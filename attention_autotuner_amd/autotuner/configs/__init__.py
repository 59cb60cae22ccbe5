from .base_config import BaseConfig, balanced_wave_split, factor_pairs
from .attention import AttnConfig
from .retnet import RetConfig
from .retnet_bwd import RetBwdConfig
from .attention_bwd import AttnBwdConfig
from .retnet_recurrent import RetRecurrentConfig

supported_configs = {
    "attn": AttnConfig,
    "ret": RetConfig,
    "ret_bwd": RetBwdConfig,
    "attn_bwd": AttnBwdConfig,
    "ret_recurrent": RetRecurrentConfig,
}

__all__ = ["BaseConfig", "AttnConfig", "RetConfig", "RetBwdConfig", "AttnBwdConfig", "RetRecurrentConfig", "supported_configs",
           "balanced_wave_split", "factor_pairs"]
