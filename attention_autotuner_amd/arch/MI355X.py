"""AMD Instinct MI355X (CDNA4, gfx950)."""
from .arch_base import Arch


class MI355X(Arch):
    # 4 SIMDs per CU, 512 unified VGPR/AGPR slots per lane per SIMD, 64 lanes
    reg_cap = 4 * 512 * 64
    smem_cap = 160 * 1024
    max_smem_usage = 160 * 1024
    compute_max_core = 256
    warp_size = 64
    sm_partition = 4
    transaction_size = (64, 1024)      # bytes; a wave's 16 B/lane access covers 1 KB
    bandwidth = (8000, 0)              # GB/s HBM3E; L2/MALL not modelled
    platform = "ROCm"
    compute_capability = "gfx950"
    register_per_thread = 512          # at one wave per SIMD; halves with each extra resident wave
    mfma = (32, 32, 16)                # v_mfma_f32_32x32x16_f16
    lds_banks = 64
    xcds = 8
    peak_tflops = 2500.0               # dense fp16 MFMA
    hipcc_arch = "gfx950"

    def __init__(self):
        super().__init__()
        self.mfma = type(self).mfma
        self.peak_tflops = type(self).peak_tflops
