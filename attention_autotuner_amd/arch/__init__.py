from .arch_base import Arch
from .MI355X import MI355X
from .A100 import A100
from .RTX4090 import RTX4090

__all__ = ["Arch", "MI355X", "A100", "RTX4090"]
