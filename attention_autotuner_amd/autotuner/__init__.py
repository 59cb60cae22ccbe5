from .configs import AttnConfig, RetConfig, RetBwdConfig, AttnBwdConfig, BaseConfig, supported_configs
from .base_tunner import BaseTunner, CompileResult
from .tunner import AttnTunner, RetTunner, RetBwdTunner, AttnBwdTunner
from .runtime import Runtime, KernelLaunchError

__all__ = ["AttnConfig", "RetConfig", "RetBwdConfig", "AttnBwdConfig", "AttnBwdTunner", "BaseConfig", "supported_configs", "BaseTunner",
           "CompileResult", "AttnTunner", "RetTunner", "RetBwdTunner", "Runtime", "KernelLaunchError"]
