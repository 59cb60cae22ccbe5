"""The set of config libraries built ahead of time (``python -m attention_autotuner_amd.autotuner.prebuilt``).

JIT compilation works anywhere hipcc is installed, but a first call that has to compile is slow and
a machine without a compiler cannot run at all; so the default configuration of every head-size pair
in common use, plus every configuration recorded in the tuning cache, is built into the in-tree
library directory up front.
"""
import glob
import json
import os
import sys

from ..arch import MI355X
from . import codegen, gfx950_space
from .base_tunner import DEFAULT_CACHE_DIR
from .configs import supported_configs

# (operator, d_qk, d_v) pairs whose default configuration is always built
# attention smemfuse variants exercised by the parity suite: (Br, Bc, Nthreads, K bufs, V bufs, W1N, W2N, waves/SIMD)
SHARED_TILES = [(128, 64, 256, 2, 2, 1, 4, 2), (64, 64, 256, 1, 1, 2, 4, 2), (64, 64, 256, 2, 1, 2, 2, 2), (64, 64, 256, 1, 1, 2, 4, 1)]

DEFAULT_PROBLEMS = [
    ("attn", 64, 64), ("attn", 128, 128), ("attn", 256, 256), ("attn", 192, 192), ("attn", 256, 128), ("attn", 64, 128),
    ("attn", 256, 512),
    ("ret", 64, 64), ("ret", 128, 128), ("ret", 256, 256), ("ret", 64, 128), ("ret", 256, 512),
]


# Tile/wave/buffer combinations built for every head-size pair below so that the parity suite can
# show that all of them compute the same thing: (Br, Bc, Nthreads, K buffers, V buffers, waves per SIMD).
PARITY_TILES = [
    (128, 64, 256, 2, 2, 2), (128, 64, 256, 1, 1, 2), (128, 64, 256, 2, 1, 1), (128, 64, 256, 1, 2, 1),
    (128, 32, 256, 2, 2, 2), (128, 128, 256, 1, 1, 1), (64, 64, 128, 2, 2, 2), (128, 64, 128, 1, 1, 1),
    (256, 64, 512, 2, 2, 2), (128, 32, 256, 2, 2, 3), (128, 64, 256, 1, 1, 3),
]
PARITY_DIMS = [(64, 64), (128, 128), (64, 128), (256, 256), (192, 192)]


ATTN_BWD_DIMS = [(64, 64), (128, 128), (64, 128), (128, 64), (256, 128), (256, 256)]
# (Br, Bc, Nthreads, buffers) variants of the attention backward at 128/128 for the parity suite
ATTN_BWD_TILES = [(64, 32, 128, 2), (64, 64, 128, 2), (128, 64, 256, 3), (128, 32, 256, 2)]


def extra_configs(arch=None):
    """Additional libraries built ahead of time: the parity matrix."""
    from .configs import AttnConfig, RetConfig
    arch = arch or MI355X()
    out = []
    # RetNet forward variants at 128/128 (register and both wave grids of the LDS-fused kernel)
    for fuse, extra in (("register", {}), ("shared", dict(warps_mma1_n=1, warps_mma_n=4)), ("shared", dict(warps_mma1_n=2, warps_mma_n=2))):
        for st in ((1, 1), (2, 2)):
            cfg = RetConfig(128 if fuse == "register" else 64, 64, 128, 128, 128, 64, st[0], st[0], st[1], 256, True, waves_per_eu=1, **extra)
            cfg.fuse_type = fuse
            if gfx950_space.forward_valid(cfg, arch):
                out.append(cfg)
    for dims in ((64, 64), (128, 128), (256, 256), (64, 128), (256, 512)):
        out.append(gfx950_space.default_backward_config(*dims, arch, 128, 128))
    # attention backward: the defaults per head-size pair and sequence divisibility, plus tile variants
    from .configs import AttnBwdConfig
    for dims in ATTN_BWD_DIMS:
        for seq in (None, 128, 64):
            out.append(gfx950_space.default_attn_backward_config(*dims, arch, seq, seq))
    for br, bc, nt, st in ATTN_BWD_TILES:
        for row_wpe in (1, 2):
            cfg = AttnBwdConfig(br, bc, 128, 128, nt, st, row_waves_per_eu=row_wpe)
            if gfx950_space.attn_backward_valid(cfg, arch):
                out.append(cfg)
    for dqk, dv in PARITY_DIMS:
        for br, bc, nt, sq, sv, wpe in PARITY_TILES:
            cfg = AttnConfig(br, bc, dqk, dv, dqk, bc, sq, sv, nt, True, waves_per_eu=wpe).set_fuse_type("register")
            if gfx950_space.forward_valid(cfg, arch):
                out.append(cfg)
            if (sq, sv) == (2, 2):
                piped = AttnConfig(br, bc, dqk, dv, dqk, bc, 2, 2, nt, True, waves_per_eu=wpe, sw_pipeline=1).set_fuse_type("register")
                if gfx950_space.forward_valid(piped, arch):
                    out.append(piped)
    for dqk, dv, ns in ((128, 128, 4), (128, 128, 8), (64, 64, 2)):     # kv-splitting variants
        out.append(AttnConfig(128, 64, dqk, dv, dqk, 64, 2, 2, 256, True, waves_per_eu=2, kv_splits=ns).set_fuse_type("register"))
    for dqk, dv in ((64, 64), (128, 128), (256, 512)):
        for br, bc, nt, sq, sv, w1n, w2n, wpe in SHARED_TILES:
            cfg = AttnConfig(br, bc, dqk, dv, dqk, bc, sq, sv, nt, True, w1n, w2n, waves_per_eu=wpe)
            cfg.fuse_type = "shared"
            if gfx950_space.forward_valid(cfg, arch):
                out.append(cfg)
    return out


def cached_configs(cache_dir=None):
    out = []
    for path in sorted(glob.glob(os.path.join(cache_dir or DEFAULT_CACHE_DIR, "best_config_*.json"))):
        try:
            with open(path) as f:
                dd = json.load(f)
            out.append(supported_configs[dd["operation"]].from_dict(dd))
        except (OSError, ValueError, KeyError):
            continue
    return out


def shipping_set(arch=None):
    arch = arch or MI355X()
    cfgs = []
    for op, dqk, dv in DEFAULT_PROBLEMS:
        if op in ("attn", "ret"):
            for seq in (None, 128, 64):          # defaults differ with what the sequence length divides by
                cfgs.append(gfx950_space.default_forward_config(op, dqk, dv, arch, seq, seq))
        if op == "ret":
            cfgs.append(gfx950_space.default_backward_config(dqk, dv, arch))
    cfgs += extra_configs(arch)
    cfgs.append(supported_configs["ret_recurrent"]())
    cfgs += cached_configs()
    seen, unique = set(), []
    for c in cfgs:
        key = (c.operation, str(c))
        if key not in seen:
            seen.add(key)
            unique.append(c)
    return unique


def build_all(arch=None, force=True, timeout=600, verbose=True):
    arch = arch or MI355X()
    cfgs = shipping_set(arch)
    if force:
        for c in cfgs:
            p = codegen.library_path(c)
            if os.path.exists(p):
                os.remove(p)
    libs = codegen.compile_parallel(cfgs, arch, timeout=timeout)
    failed = [c for c, l in zip(cfgs, libs) if l is None]
    if verbose:
        print(f"built {len(cfgs) - len(failed)}/{len(cfgs)} config libraries into {codegen.DEFAULT_BUILD_DIR}")
    if failed:
        raise RuntimeError("hipcc failed for: " + ", ".join(f"{c.operation}:{c}" for c in failed))
    return libs


def prune_stale(build_dir=None):
    """Delete libraries (and their sources / logs) built from an older revision of the kernel sources."""
    root = build_dir or codegen.DEFAULT_BUILD_DIR
    removed = 0
    for op in sorted(os.listdir(root)) if os.path.isdir(root) else []:
        if op not in codegen.SOURCE_DIRS:
            continue
        keep = "-" + codegen.source_digest(op) + "."
        for dirpath, _, files in os.walk(os.path.join(root, op)):
            for fn in files:
                if fn.endswith((".so", ".hip", ".log")) and keep not in fn:
                    os.remove(os.path.join(dirpath, fn))
                    removed += 1
    return removed


if __name__ == "__main__":
    if "--prune" in sys.argv:
        print("removed", prune_stale(), "stale files")
    build_all(force="--force" in sys.argv)
