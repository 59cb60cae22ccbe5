"""Kernel configuration records.

A configuration is a flat bag of integers (tile sizes, thread count, LDS buffering, ...) plus a fuse
type; ``vars(config)`` is what fills the ``{Br}``-style fields of the wrapper templates and what is
stored in the tuning cache.  Field names, ``repr`` (one line of a tuning log) and ``str`` (the key a
compiled library is filed under) follow reference python/autotuner/configs/base_config.py:30-76 and its
subclasses, so logs and cache files written by the reference remain readable.

New on MI355X: ``waves_per_eu`` (resident waves per SIMD the kernel is compiled for),
``sw_pipeline`` (software-pipelined schedule: the next tile's first contraction is issued between the
current tile's exponentials; needs two K and two V buffers) and ``kv_splits`` (number of kv-range
partitions for long-kv / few-row problems).
"""
import os

_KERNEL_ROOT = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "..", "csrc", "kernels"))


def factor_pairs(n):
    """All (a, b) with a * b == n, ascending in a."""
    return [(a, n // a) for a in range(1, n + 1) if n % a == 0]


def balanced_wave_split(n_waves, rows, cols, atom=16):
    """Split ``n_waves`` into (along rows, along cols) so each wave's sub-tile is as square as the
    divisibility by ``atom`` allows.  Returns None when no split fits.  The cost function and the
    first-minimum-wins tie break are those of reference base_config.py:17-28 (``find_best_pair``)."""
    best, best_cost = None, 1.0
    for a, b in factor_pairs(n_waves):
        if rows % (a * atom) or cols % (b * atom):
            continue
        cost = abs(a * cols / (b * rows + a * cols) - 0.5)
        if cost < best_cost:
            best, best_cost = (a, b), cost
    return best


class BaseConfig:
    operation = None            # "attn" | "ret" | "ret_bwd"
    kernel_subdir = None        # directory under csrc/kernels holding the templates
    _log_fields = ()            # fields printed by repr, in order
    _key_fields = ()            # fields joined by str
    _wave = 32                  # lanes per warp assumed by the wave-split defaults (reference value)

    def __init__(self, Br, Bc, Kd, D, BlockKSmem=256, num_stages_qk=1, Nthreads=256, unrollLastIter=True):
        self.Br, self.Bc, self.Kd, self.D = Br, Bc, Kd, D
        self.BlockKSmem = BlockKSmem
        self.num_stages_qk = num_stages_qk
        self.Nthreads = Nthreads
        self.unrollLastIter = int(unrollLastIter)
        n_waves = max(1, Nthreads // self._wave)
        split1 = balanced_wave_split(n_waves, Br, Bc)
        split2 = balanced_wave_split(n_waves, Br, D)
        self.warps_mma1_n = split1[1] if split1 else None
        self.warps_mma_n = split2[1] if split2 else None
        self.fuse_type = "None"
        self.waves_per_eu = 1
        self.sw_pipeline = 0
        self.kv_splits = 1
        self.operation = type(self).operation
        self.template_dir = os.path.join(_KERNEL_ROOT, type(self).kernel_subdir) if type(self).kernel_subdir else None

    # -- fuse type ---------------------------------------------------------------------------------
    def set_fuse_type(self, fuse_type):
        self.fuse_type = fuse_type
        if fuse_type == "register":
            self.warps_mma1_n = 1
            self.warps_mma_n = 1
        return self

    # -- text forms --------------------------------------------------------------------------------
    def _extras(self):
        """MI355X-only knobs, appended to the key (never to the reference-format log line) when set."""
        out = []
        if getattr(self, "waves_per_eu", 1) != 1:
            out.append(f"w{self.waves_per_eu}")
        if getattr(self, "sw_pipeline", 0):
            out.append("p1")
        if getattr(self, "kv_splits", 1) != 1:
            out.append(f"s{self.kv_splits}")
        return out

    def __repr__(self):
        body = ", ".join(f"{f}={getattr(self, f)}" for f in self._log_fields)
        if self.fuse_type != "register":
            body += f",warps_mma1_n={self.warps_mma1_n},warp_mma_n={self.warps_mma_n}"
        extras = self._extras()
        if extras:
            body += ", " + ", ".join(f"{k}={getattr(self, k)}" for k, d in (("waves_per_eu", 1), ("sw_pipeline", 0), ("kv_splits", 1))
                                     if getattr(self, k, d) != d)
        return f"Config({body})"

    def __str__(self):
        parts = [str(getattr(self, f)) for f in self._key_fields]
        if self.fuse_type != "register":
            parts += [str(self.warps_mma1_n), str(self.warps_mma_n)]
        return "_".join(parts + self._extras())

    def __eq__(self, other):
        return type(self) is type(other) and self.to_dict() == other.to_dict()

    def __hash__(self):
        return hash((type(self).__name__, str(self)))

    # -- (de)serialisation -------------------------------------------------------------------------
    def to_dict(self):
        return {k: v for k, v in vars(self).items() if k != "template_dir"}

    @classmethod
    def from_dict(cls, dd):
        cfg = cls.__new__(cls)
        cfg.waves_per_eu = 1
        cfg.sw_pipeline = 0
        cfg.kv_splits = 1
        vars(cfg).update({k: v for k, v in dd.items() if k != "template_dir"})
        cfg.operation = cls.operation
        cfg.template_dir = os.path.join(_KERNEL_ROOT, cls.kernel_subdir)
        return cfg
