from .base_config import BaseConfig


class AttnBwdConfig(BaseConfig):
    """Flash-attention backward.  The reference declares the operator and leaves it empty
    (reference python/ops/attention_interface.py:37-58), so there is no reference configuration record;
    this one follows the shape of its RetNet backward record (python/autotuner/configs/retnet_bwd.py:4-26).

    Two kernels share the tile shape: a column kernel (``Br`` kv rows resident per block, q/dO tiles of
    ``Bc`` rows streamed) producing dV and dK, and a row kernel (``Br`` q rows resident, k/v tiles of
    ``Bc`` rows streamed) producing dQ.  ``num_stages_qk`` is the number of LDS buffers of the stream."""
    operation = "attn_bwd"
    kernel_subdir = "attention/bwd"
    _fields = ("Br", "Bc", "Kd", "D", "Nthreads", "num_stages_qk")

    def __init__(self, Br, Bc, Kd, D, Nthreads=256, num_stages_qk=3, waves_per_eu=1):
        super().__init__(Br, Bc, Kd, D, Kd, num_stages_qk, Nthreads, True)
        self.waves_per_eu = waves_per_eu
        self.fuse_type = "bwd"

    def __repr__(self):
        return "AttnBwdConfig(" + ", ".join(f"{f}={getattr(self, f)}" for f in self._fields) + ")"

    def __str__(self):
        return "_".join([self.operation] + [str(getattr(self, f)) for f in self._fields] + self._extras())
