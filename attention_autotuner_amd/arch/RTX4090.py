"""NVIDIA RTX 4090 limits (reference python/arch/RTX4090.py:1-20), importable as in the reference; a descriptor only,
see A100.py."""
from .arch_base import Arch


class RTX4090(Arch):
    reg_cap = 65536
    smem_cap = 100 * 1024
    max_smem_usage = 100 * 1024
    compute_max_core = 128
    warp_size = 32
    sm_partition = 4
    transaction_size = (32, 128)
    bandwidth = (1008, 0)
    platform = "CUDA"
    compute_capability = "89"
    register_per_thread = 255
    cutlass_mma = (16, 8, 16)

    def __init__(self):
        super().__init__()
        self.cutlass_mma = type(self).cutlass_mma
