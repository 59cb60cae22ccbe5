from .base_config import BaseConfig


class RetRecurrentConfig(BaseConfig):
    """RetNet recurrent form (reference csrc/kernels/retnet/recurrent/recurrent.h:427-463).  The reference
    has no configuration record for it: one fixed instantiation (128 threads, 16 items per thread, two
    value dims per block, :452-462) is compiled into its benchmark.  Here one library holds every supported
    instantiation and chooses per call, so the record only carries a revision tag that names the library."""
    operation = "ret_recurrent"
    kernel_subdir = "retnet/recurrent"

    def __init__(self, revision=1):
        super().__init__(32, 32, 128, 128, 128, 2, 256, True)
        self.revision = revision

    def __repr__(self):
        return f"RetRecurrentConfig(revision={self.revision})"

    def __str__(self):
        return f"{self.operation}_r{self.revision}"
