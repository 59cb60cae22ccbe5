from .base_config import BaseConfig


class AttnConfig(BaseConfig):
    """Flash-attention forward (reference python/autotuner/configs/attention.py:4-30).

    On MI355X: ``num_stages_qk`` / ``num_stages_v`` are the number of LDS buffers for the K and V
    tiles (1 = single buffer refilled behind a barrier, 2 = double buffer filled one tile ahead);
    ``BlockKSmem`` / ``BlockKSmem2`` are the extents staged per buffer and equal Kd / Bc.
    """
    operation = "attn"
    kernel_subdir = "attention"
    _log_fields = ("fuse_type", "Br", "Bc", "BlockKSmem", "BlockKSmem2", "num_stages_qk", "num_stages_v",
                   "Nthreads", "unrollLastIter")
    _key_fields = ("fuse_type", "Br", "Bc", "Kd", "D", "BlockKSmem", "BlockKSmem2", "num_stages_qk",
                   "num_stages_v", "Nthreads", "unrollLastIter")

    def __init__(self, Br, Bc, Kd, D, BlockKSmem=256, BlockKSmem2=64, num_stages_qk=1, num_stages_v=1,
                 Nthreads=256, unrollLastIter=True, warps_mma1_n=None, warps_mma_n=None,
                 waves_per_eu=1, kv_splits=1, sw_pipeline=0):
        super().__init__(Br, Bc, Kd, D, BlockKSmem, num_stages_qk, Nthreads, unrollLastIter)
        self.BlockKSmem2 = BlockKSmem2
        self.num_stages_v = num_stages_v
        if warps_mma1_n is not None:
            self.warps_mma1_n = warps_mma1_n
        if warps_mma_n is not None:
            self.warps_mma_n = warps_mma_n
        self.waves_per_eu = waves_per_eu
        self.kv_splits = kv_splits
        self.sw_pipeline = int(sw_pipeline)
