"""The package's A100 descriptor with the reference's NVIDIA search space attached: kept only so the search-space
enumeration can be checked against the reference's published tuning logs; nothing is compiled or run for it."""
from attention_autotuner_amd.arch import A100 as _A100

from . import legacy_space


class A100(_A100):
    search_space = legacy_space        # the tuners enumerate a non-ROCm descriptor with the space it brings along
