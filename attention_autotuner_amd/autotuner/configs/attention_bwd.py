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
    at two waves per SIMD has no registers to spare for them).  ``col_split`` builds the column kernel twice,
    once for dV alone and once for dK alone: one more evaluation of the scores, and each half fits a register
    budget (``dv_waves_per_eu`` / ``dk_waves_per_eu``) that the two-output kernel does not -- two waves per SIMD
    at d = 128, and any budget at all at d_qk 256 / d_v 512."""
    operation = "attn_bwd"
    kernel_subdir = "attention/bwd"
    _fields = ("Br", "Bc", "Kd", "D", "Nthreads", "num_stages_qk")

    def __init__(self, Br, Bc, Kd, D, Nthreads=256, num_stages_qk=3, waves_per_eu=1, row_waves_per_eu=None, row_Bc=None,
                 col_split=0, dv_waves_per_eu=None, dk_waves_per_eu=None):
        super().__init__(Br, Bc, Kd, D, Kd, num_stages_qk, Nthreads, True)
        self.waves_per_eu = waves_per_eu
        self.row_waves_per_eu = row_waves_per_eu or waves_per_eu
        self.row_Bc = row_Bc or Bc
        self.col_split = int(col_split)
        self.dv_waves_per_eu = dv_waves_per_eu or waves_per_eu
        self.dk_waves_per_eu = dk_waves_per_eu or waves_per_eu
        self.fuse_type = "bwd"

    @classmethod
    def from_dict(cls, dd):
        cfg = super().from_dict(dd)
        if "row_waves_per_eu" not in dd:                       # records written before the knobs existed
            cfg.row_waves_per_eu = cfg.waves_per_eu
        if "row_Bc" not in dd:
            cfg.row_Bc = cfg.Bc
        if "col_split" not in dd:
            cfg.col_split = 0
        for key in ("dv_waves_per_eu", "dk_waves_per_eu"):
            if key not in dd:
                setattr(cfg, key, cfg.waves_per_eu)
        return cfg

    def _extras(self):
        out = super()._extras()
        if self.row_waves_per_eu != self.waves_per_eu:
            out.append(f"rw{self.row_waves_per_eu}")
        if self.row_Bc != self.Bc:
            out.append(f"rb{self.row_Bc}")
        if self.col_split:
            out.append(f"cs{self.dv_waves_per_eu}{self.dk_waves_per_eu}")
        return out

    def __repr__(self):
        body = ", ".join(f"{f}={getattr(self, f)}" for f in self._fields)
        if self.waves_per_eu != 1:
            body += f", waves_per_eu={self.waves_per_eu}"
        if self.row_waves_per_eu != self.waves_per_eu:
            body += f", row_waves_per_eu={self.row_waves_per_eu}"
        if self.row_Bc != self.Bc:
            body += f", row_Bc={self.row_Bc}"
        if self.col_split:
            body += f", col_split=1, dv_waves_per_eu={self.dv_waves_per_eu}, dk_waves_per_eu={self.dk_waves_per_eu}"
        return f"AttnBwdConfig({body})"

    def __str__(self):
        return "_".join([self.operation] + [str(getattr(self, f)) for f in self._fields] + self._extras())
