from .arch_base import Arch
from .MI355X import MI355X

__all__ = ["Arch", "MI355X"]
