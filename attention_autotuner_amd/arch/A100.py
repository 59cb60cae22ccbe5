"""NVIDIA A100 limits (reference python/arch/A100.py:1-20), importable as in the reference.  A descriptor only: this
package builds and runs kernels for ROCm descriptors (``MI355X``); the tuners enumerate a foreign descriptor only
when it brings a search space along (``search_space``) and refuse to build for it."""
from .arch_base import Arch


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

    def __init__(self):
        super().__init__()
        self.cutlass_mma = type(self).cutlass_mma
