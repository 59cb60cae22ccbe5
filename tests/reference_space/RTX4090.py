"""The package's RTX 4090 descriptor with the reference's NVIDIA search space attached (enumeration checks only,
see A100.py)."""
from attention_autotuner_amd.arch import RTX4090 as _RTX4090

from . import legacy_space


class RTX4090(_RTX4090):
    search_space = legacy_space        # the tuners enumerate a non-ROCm descriptor with the space it brings along
