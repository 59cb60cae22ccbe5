"""Hardware descriptor consumed by the tuner's validity model.

Field names follow reference python/arch/arch_base.py:1-13 so configs written against the reference
keep working; ``mfma`` / ``lds_banks`` / ``peak_tflops`` are additions for CDNA.
"""


class Arch:
    reg_cap = 0                 # 32-bit registers per SIMD/SM partition group usable by one block
    smem_cap = 0                # bytes of LDS / shared memory one block may use
    compute_max_core = 0        # number of CUs / SMs
    warp_size = 0
    sm_partition = 0            # SIMDs per CU / sub-partitions per SM
    transaction_size = (0, 0)   # bytes: smallest and widest coalesced memory transaction
    max_smem_usage = 0
    bandwidth = (0, 0)          # GB/s: device memory, last-level cache
    platform = "unknown"
    compute_capability = "unknown"
    register_per_thread = 0

    def __init__(self):
        # copy class-level defaults so instances serialise with vars()
        for name in ("reg_cap", "smem_cap", "compute_max_core", "warp_size", "sm_partition",
                     "transaction_size", "max_smem_usage", "bandwidth", "platform",
                     "compute_capability", "register_per_thread"):
            setattr(self, name, getattr(type(self), name))

    @property
    def name(self):
        return type(self).__name__

    def __repr__(self):
        return f"{self.name}()"
