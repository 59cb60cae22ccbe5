from .base_config import BaseConfig


class RetConfig(BaseConfig):
    """RetNet parallel forward (reference python/autotuner/configs/retnet.py:4-33)."""
    operation = "ret"
    kernel_subdir = "retnet"
    _log_fields = ("fuse_type", "Br", "Bc", "BlockKSmem", "BlockKSmem2", "num_stages_qk", "num_stages_mask",
                   "num_stages_v", "Nthreads", "unrollLastIter")
    _key_fields = ("fuse_type", "Br", "Bc", "Kd", "D", "BlockKSmem", "BlockKSmem2", "num_stages_qk",
                   "num_stages_mask", "num_stages_v", "Nthreads", "unrollLastIter")

    def __init__(self, Br, Bc, Kd, D, BlockKSmem=256, BlockKSmem2=64, num_stages_qk=1, num_stages_mask=1,
                 num_stages_v=1, Nthreads=256, unrollLastIter=True, warps_mma1_n=None, warps_mma_n=None,
                 waves_per_eu=1):
        super().__init__(Br, Bc, Kd, D, BlockKSmem, num_stages_qk, Nthreads, unrollLastIter)
        self.BlockKSmem2 = BlockKSmem2
        self.num_stages_v = num_stages_v
        self.num_stages_mask = num_stages_mask
        if warps_mma1_n is not None:
            self.warps_mma1_n = warps_mma1_n
        if warps_mma_n is not None:
            self.warps_mma_n = warps_mma_n
        self.waves_per_eu = waves_per_eu
