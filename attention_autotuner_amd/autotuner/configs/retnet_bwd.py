from .base_config import BaseConfig


class RetBwdConfig(BaseConfig):
    """RetNet parallel backward (reference python/autotuner/configs/retnet_bwd.py:4-26).

    On MI355X the gradient is three passes (dV, dK, dQ) of one chained-contraction kernel: ``Br`` is the
    number of block-resident rows and ``Bc`` the number of streamed rows per step of every pass;
    ``num_stages_qk`` / ``num_stages_dv`` are the LDS buffer counts of the two streams of the dV pass, and
    ``num_stages_ds`` / ``num_stages_dq`` the same counts for the passes that contract over d_v first (dQ, and dK
    where it is a chained pass): their streamed tiles are d_v wide.  The ``mmawarpsN*``
    fields (how the reference splits its warps along the N side of each contraction) are carried for
    file compatibility; every wave here owns whole rows.

    ``ds_rows`` (0, 128 or 256; new on MI355X): with a workspace of B*H*S_q*S_kv fp16 the dQ pass stores the dS
    tiles it forms and dK comes from a kernel of its own that reads them back (``ds_rows`` kv rows per block)
    instead of evaluating dO V^T a second time."""
    operation = "ret_bwd"
    kernel_subdir = "retnet/bwd"
    _fields = ("Br", "Bc", "Kd", "D", "mmawarpsN", "mmawarpsN_dv", "mmawarpsN_dk", "mmawarpsN_dq", "Nthreads",
               "unrollLastIter", "BlockKSmem", "num_stages_qk", "num_stages_mask", "num_stages_dv",
               "num_stages_ds", "num_stages_dq")

    def __init__(self, Br, Bc, Kd, D, mmawarpsN, mmawarpsN_dv, mmawarpsN_dk, mmawarpsN_dq, Nthreads=256,
                 unrollLastIter=True, BlockKSmem=256, num_stages_qk=1, num_stages_mask=1, num_stages_dv=1,
                 num_stages_ds=1, num_stages_dq=1, waves_per_eu=1, ds_rows=0):
        super().__init__(Br, Bc, Kd, D, BlockKSmem, num_stages_qk, Nthreads, unrollLastIter)
        self.num_stages_mask = num_stages_mask
        self.mmawarpsN = mmawarpsN
        self.mmawarpsN_dv = mmawarpsN_dv
        self.mmawarpsN_dk = mmawarpsN_dk
        self.mmawarpsN_dq = mmawarpsN_dq
        self.num_stages_dv = num_stages_dv
        self.num_stages_ds = num_stages_ds
        self.num_stages_dq = num_stages_dq
        self.waves_per_eu = waves_per_eu
        self.ds_rows = int(ds_rows)
        self.fuse_type = "bwd"

    @classmethod
    def from_dict(cls, dd):
        cfg = super().from_dict(dd)
        if "ds_rows" not in dd:                                # records written before the knob existed
            cfg.ds_rows = 0
        return cfg

    def _extras(self):
        out = super()._extras()
        if self.ds_rows:
            out.append(f"ds{self.ds_rows}")
        return out

    def __repr__(self):
        body = ", ".join(f"{f}={getattr(self, f)}" for f in self._fields)
        if self.ds_rows:
            body += f", ds_rows={self.ds_rows}"
        return "RetBwdConfig(" + body + ")"

    def __str__(self):
        return "_".join([self.operation] + [str(getattr(self, f)) for f in self._fields] + self._extras())
