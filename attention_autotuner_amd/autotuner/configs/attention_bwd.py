from .base_config import BaseConfig


class AttnBwdConfig(BaseConfig):
    """Flash-attention backward.  The reference declares the operator and leaves it empty
    (reference python/ops/attention_interface.py:37-58), so there is no reference configuration record;
    this one follows the shape of its RetNet backward record (python/autotuner/configs/retnet_bwd.py:4-26).

    Two kernels share the tile shape: a column kernel (``Br`` kv rows resident per block, q/dO tiles of
    ``Bc`` rows streamed) producing dV and dK, and a row kernel (``Br`` q rows resident, k/v tiles of
    ``Bc`` rows streamed) producing dQ.  ``num_stages_qk`` is the number of LDS buffers of the stream.
    ``row_waves_per_eu`` is the register budget (resident waves per SIMD) the row kernel is compiled for: with
    one output instead of two it fits 256 registers where the column kernel needs the whole file, and two
    waves per SIMD overlap one wave's matrix work with the other's exponentials.  ``row_Bc`` is the row
    kernel's own streamed tile height (the column kernel, alone on its SIMD, likes 64-row tiles; the row kernel
    at two waves per SIMD has no registers to spare for them)."""
    operation = "attn_bwd"
    kernel_subdir = "attention/bwd"
    _fields = ("Br", "Bc", "Kd", "D", "Nthreads", "num_stages_qk")

    def __init__(self, Br, Bc, Kd, D, Nthreads=256, num_stages_qk=3, waves_per_eu=1, row_waves_per_eu=None, row_Bc=None):
        super().__init__(Br, Bc, Kd, D, Kd, num_stages_qk, Nthreads, True)
        self.waves_per_eu = waves_per_eu
        self.row_waves_per_eu = row_waves_per_eu or waves_per_eu
        self.row_Bc = row_Bc or Bc
        self.fuse_type = "bwd"

    @classmethod
    def from_dict(cls, dd):
        cfg = super().from_dict(dd)
        if "row_waves_per_eu" not in dd:                       # records written before the knobs existed
            cfg.row_waves_per_eu = cfg.waves_per_eu
        if "row_Bc" not in dd:
            cfg.row_Bc = cfg.Bc
        return cfg

    def _extras(self):
        out = super()._extras()
        if self.row_waves_per_eu != self.waves_per_eu:
            out.append(f"rw{self.row_waves_per_eu}")
        if self.row_Bc != self.Bc:
            out.append(f"rb{self.row_Bc}")
        return out

    def __repr__(self):
        body = ", ".join(f"{f}={getattr(self, f)}" for f in self._fields)
        if self.waves_per_eu != 1:
            body += f", waves_per_eu={self.waves_per_eu}"
        if self.row_waves_per_eu != self.waves_per_eu:
            body += f", row_waves_per_eu={self.row_waves_per_eu}"
        if self.row_Bc != self.Bc:
            body += f", row_Bc={self.row_Bc}"
        return f"AttnBwdConfig({body})"

    def __str__(self):
        return "_".join([self.operation] + [str(getattr(self, f)) for f in self._fields] + self._extras())
