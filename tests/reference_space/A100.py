"""NVIDIA A100 limits.  Kept only so the search-space enumeration can be checked against the
reference's published tuning logs; nothing is compiled or run for this descriptor."""
from attention_autotuner_amd.arch import Arch

from . import legacy_space


class A100(Arch):
    reg_cap = 65536
    smem_cap = 163 * 1024
    max_smem_usage = 164 * 1024
    compute_max_core = 108
    warp_size = 32
    sm_partition = 4
    transaction_size = (32, 128)
    bandwidth = (1319, 16308)
    platform = "CUDA"
    compute_capability = "80"
    register_per_thread = 255
    cutlass_mma = (16, 8, 16)
    search_space = legacy_space        # the tuners enumerate a non-ROCm descriptor with the space it brings along

    def __init__(self):
        super().__init__()
        self.cutlass_mma = type(self).cutlass_mma
