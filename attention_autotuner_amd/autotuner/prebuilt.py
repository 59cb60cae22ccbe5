"""The set of config libraries built ahead of time (``python -m attention_autotuner_amd.autotuner.prebuilt``).

JIT compilation works anywhere hipcc is installed, but a first call that has to compile is slow and
a machine without a compiler cannot run at all; so the default configuration of every head-size pair
in common use, plus every configuration recorded in the tuning cache, is built into the in-tree
library directory up front.  Callers can add configurations of their own (``extra``).
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
DEFAULT_PROBLEMS = [
    ("attn", 64, 64), ("attn", 128, 128), ("attn", 256, 256), ("attn", 192, 192), ("attn", 256, 128), ("attn", 64, 128), ("attn", 128, 64), ("attn", 128, 192), ("attn", 192, 64),
    ("attn", 256, 512),
    ("ret", 64, 64), ("ret", 128, 128), ("ret", 192, 192), ("ret", 256, 256), ("ret", 64, 128), ("ret", 256, 512),
    ("attn_bwd", 64, 64), ("attn_bwd", 128, 128), ("attn_bwd", 64, 128), ("attn_bwd", 128, 64), ("attn_bwd", 192, 192), ("attn_bwd", 128, 192), ("attn_bwd", 192, 64), ("attn_bwd", 256, 128),
    ("attn_bwd", 256, 256), ("attn_bwd", 256, 512),
]


def default_configs(arch=None):
    """The default configuration of every problem in DEFAULT_PROBLEMS, for each sequence divisibility the
    defaults distinguish."""
    arch = arch or MI355X()
    cfgs = []
    for op, dqk, dv in DEFAULT_PROBLEMS:
        for seq in (None, 128, 64):          # defaults differ with what the sequence length divides by
            if op in ("attn", "ret"):
                cfgs.append(gfx950_space.default_forward_config(op, dqk, dv, arch, seq, seq))
            elif op == "attn_bwd":
                cfgs.append(gfx950_space.default_attn_backward_config(dqk, dv, arch, seq, seq))
        if op == "ret":
            for seq in (None, 128, 64):
                cfgs.append(gfx950_space.default_backward_config(dqk, dv, arch, seq, seq))
    return cfgs


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


def shipping_set(arch=None, extra=()):
    """Defaults, the RetNet recurrent library, every configuration in the tuning cache, and ``extra``
    (e.g. the matrix of tile variants a test suite wants built ahead of time), without duplicates."""
    arch = arch or MI355X()
    cfgs = default_configs(arch)
    cfgs.append(supported_configs["ret_recurrent"]())
    cfgs += cached_configs()
    cfgs += list(extra)
    seen, unique = set(), []
    for c in cfgs:
        key = (c.operation, str(c))
        if key not in seen:
            seen.add(key)
            unique.append(c)
    return unique


def build_all(arch=None, force=True, timeout=600, verbose=True, extra=()):
    arch = arch or MI355X()
    cfgs = shipping_set(arch, extra)
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
                if fn.endswith((".so", ".hip", ".log", ".usage.json")) and keep not in fn:
                    os.remove(os.path.join(dirpath, fn))
                    removed += 1
    return removed


def prune_candidates(extra=(), build_dir=None):
    """Delete every library that is not in the shipping set (+ ``extra``): what a tuning run over a whole search space
    leaves behind.  Returns the number of files removed."""
    root = build_dir or codegen.DEFAULT_BUILD_DIR
    keep = {os.path.basename(codegen.library_path(c, build_dir))[:-3] for c in shipping_set(extra=extra)}
    removed = 0
    for op in sorted(os.listdir(root)) if os.path.isdir(root) else []:
        if op not in codegen.SOURCE_DIRS or op == "ret_recurrent":
            continue
        for dirpath, _, files in os.walk(os.path.join(root, op)):
            for fn in files:
                stem = fn[:-len(".usage.json")] if fn.endswith(".usage.json") else os.path.splitext(fn)[0]
                if fn.endswith((".so", ".hip", ".log", ".usage.json")) and stem not in keep:
                    os.remove(os.path.join(dirpath, fn))
                    removed += 1
    return removed


if __name__ == "__main__":
    if "--prune" in sys.argv:
        print("removed", prune_stale(), "stale files")
    if "--prune-candidates" in sys.argv:          # keep the shipping set and the parity suite's variants only
        from . import prebuilt_extra
        print("removed", prune_candidates(extra=prebuilt_extra.parity_configs()), "files of libraries outside the shipping set")
    build_all(force="--force" in sys.argv)
