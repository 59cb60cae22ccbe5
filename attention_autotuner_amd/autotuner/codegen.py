"""Wrapper generation and hipcc driver.

One configuration -> one ``.hip`` wrapper (template text from ``csrc/kernels/**/profile_code.py`` filled
with ``vars(config)``) -> one shared object exporting the C ABI of include/aat_kernel_abi.h.  Same job
as ``_create_code_for_profiling`` / ``_compile`` in reference python/autotuner/base_tunner.py:25-66 and
``Runtime.compile`` in reference python/autotuner/runtime.py:42-72, with three changes: libraries
are content-addressed (configuration + a hash of every kernel source), they live in a persistent
in-tree directory so a tuned library is never rebuilt, and a failed or timed-out compile yields
``None`` that callers skip instead of crashing on.
"""
import functools
import hashlib
import importlib.util
import json
import os
import re
import shutil
import subprocess
import sys
import threading
from concurrent.futures import ThreadPoolExecutor

_PKG = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
CSRC_DIR = os.path.join(_PKG, "csrc")
INCLUDE_DIR = os.path.normpath(os.path.join(_PKG, "..", "include"))
DEFAULT_BUILD_DIR = os.environ.get("AAT_BUILD_DIR", os.path.join(_PKG, "build"))

# -packed-fp32-ops is switched OFF on purpose: hipcc would otherwise fuse scalar fp32 math into
# v_pk_*_f32 instructions.
# -Rpass-analysis=kernel-resource-usage makes the compiler report registers, scratch and occupancy of every kernel
# it emits; the report is kept next to the library (``resource_usage``) and is what the tuners reject spilling
# candidates by.
HIPCC_FLAGS = ["-std=c++17", "-O3", "-fno-math-errno", "-ffp-contract=fast", "-fno-honor-nans", "-fPIC", "-shared", "-w",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Rpass-analysis=kernel-resource-usage"]


def hipcc_exe():
    exe = os.environ.get("HIPCC")
    if exe:
        return exe
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cand = os.path.join(rocm, "bin", "hipcc")
    return cand if os.path.exists(cand) else (shutil.which("hipcc") or "hipcc")


def _template_file(config):
    sub = {"register": "regfuse", "shared": "smemfuse"}.get(config.fuse_type, "")
    return os.path.join(config.template_dir, sub, "profile_code.py")


@functools.lru_cache(maxsize=None)
def _load_template(path):
    spec = importlib.util.spec_from_file_location("aat_profile_code_" + hashlib.sha1(path.encode()).hexdigest()[:8], path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def render(config, kind="kernel"):
    """Source text of the wrapper for ``config``; ``kind`` is "kernel" or "profile" (the same text
    here, both entry points live in one library)."""
    mod = _load_template(_template_file(config))
    text = mod.kernel_code if kind == "kernel" else mod.profile_code
    fields = dict(vars(config))
    fields["config_name"] = f"{config.operation}:{config}"
    return text.format_map(fields)


# kernel directories (under csrc/kernels) whose files can change the machine code of an operator's libraries;
# csrc/kernels/utils and include/ count for every operator
SOURCE_DIRS = {
    "attn": ("attention/regfuse", "attention/smemfuse"),
    "attn_bwd": ("attention/bwd",),
    "ret": ("retnet/regfuse", "retnet/smemfuse"),
    "ret_bwd": ("retnet/bwd",),
    "ret_recurrent": ("retnet/recurrent",),
}


@functools.lru_cache(maxsize=None)
def source_digest(operation):
    """Hash of every file that can change the machine code of a config library of ``operation``."""
    h = hashlib.sha1()
    h.update(" ".join(HIPCC_FLAGS).encode())
    kernels = os.path.join(CSRC_DIR, "kernels")
    roots = [os.path.join(kernels, "utils")] + [os.path.join(kernels, d) for d in SOURCE_DIRS[operation]] + [INCLUDE_DIR]
    for root in roots:
        for dirpath, dirnames, filenames in sorted(os.walk(root)):
            dirnames.sort()
            for fn in sorted(filenames):
                if fn.endswith((".h", ".py", ".hip")):
                    with open(os.path.join(dirpath, fn), "rb") as f:
                        h.update(os.path.relpath(os.path.join(dirpath, fn), kernels).encode())
                        h.update(f.read())
    return h.hexdigest()[:10]


def library_name(config):
    return f"{config}-{source_digest(config.operation)}.so"


def library_path(config, build_dir=None):
    return os.path.join(build_dir or DEFAULT_BUILD_DIR, config.operation, library_name(config))


def hipcc_command(src, out, arch):
    target = getattr(arch, "hipcc_arch", None) or arch.compute_capability
    return [hipcc_exe(), *HIPCC_FLAGS, f"--offload-arch={target}", f"-I{INCLUDE_DIR}", f"-I{CSRC_DIR}", src, "-o", out]


class MissingLibraryError(RuntimeError):
    """A library would have to be compiled and compiling is switched off (AAT_NO_JIT=1)."""


def jit_allowed():
    """AAT_NO_JIT=1 forbids spawning hipcc from this process: a measurement or profiler run must never
    time a compile, and a process whose GPU a profiler has already initialised must not start children
    that inherit its preloaded libraries.  Build ahead of time with
    ``python -m attention_autotuner_amd.autotuner.prebuilt``."""
    return os.environ.get("AAT_NO_JIT", "0") in ("", "0")


def compile_config(config, arch, build_dir=None, timeout=None, force=False):
    """Build the library for ``config``; returns its path, or None if hipcc failed or timed out.
    Raises MissingLibraryError instead of compiling when AAT_NO_JIT=1."""
    if getattr(arch, "platform", "ROCm") != "ROCm":
        return None
    out = library_path(config, build_dir)
    if os.path.exists(out) and not force:
        return out
    if not jit_allowed():
        raise MissingLibraryError(f"{out} is not built and AAT_NO_JIT=1 forbids compiling it here; "
                                  "run `python -m attention_autotuner_amd.autotuner.prebuilt` first")
    os.makedirs(os.path.dirname(out), exist_ok=True)
    src = out[:-3] + ".hip"
    try:
        text = render(config)
    except (KeyError, FileNotFoundError, AttributeError):
        return None
    with open(src, "w") as f:
        f.write(text)
    tmp = out + f".tmp{os.getpid()}_{threading.get_ident()}"     # two threads of one process may build the same library
    scan = may_hold_numbered_accumulators(config)
    workdir = None
    command = hipcc_command(src, tmp, arch)
    if scan:                                       # keep the compiler's assembly next to a private copy of the output
        workdir = tmp + ".d"
        os.makedirs(workdir, exist_ok=True)
        tmp = os.path.join(workdir, os.path.basename(out))
        command = hipcc_command(src, tmp, arch) + ["-save-temps=obj"]

    def discard():
        if workdir is not None:
            shutil.rmtree(workdir, ignore_errors=True)
        elif os.path.exists(tmp):
            os.remove(tmp)

    try:
        ret = subprocess.run(command, timeout=timeout, capture_output=True, text=True)
    except subprocess.TimeoutExpired:
        discard()
        return None
    if ret.returncode != 0:
        with open(out[:-3] + ".log", "w") as f:
            f.write(ret.stdout + ret.stderr)
        discard()
        return None
    usage = parse_resource_usage(ret.stderr)
    if scan:
        listing = [os.path.join(workdir, f) for f in os.listdir(workdir) if f.endswith(".s") and "-hip-amdgcn" in f]
        clashes = foreign_accumulator_use(open(listing[0]).read()) if len(listing) == 1 else {"<no device assembly found>": 1}
        if clashes:
            # The kernel keeps its output tile in accumulation registers it names itself and the compiler has put values
            # of its own there as well: the library would compute garbage (or fault on a corrupted address).  A failed build.
            with open(out[:-3] + ".log", "w") as f:
                f.write("rejected: the compiler allocated accumulation registers in a kernel that addresses them by number\n")
                for name, n in clashes.items():
                    f.write(f"  {name}: {n} instructions outside the kernel's own asm statements name an accumulation register\n")
            discard()
            return None
    with open(usage_path(out), "w") as f:
        json.dump(usage, f, indent=1)
    os.replace(tmp, out)
    discard()
    return out


def may_hold_numbered_accumulators(config):
    """Configurations whose kernels keep their output tile in accumulation registers addressed by number
    (csrc/kernels/utils/acc_file.h): the one-wave-per-SIMD RetNet kernels.  Their builds are checked by
    ``foreign_accumulator_use``."""
    return getattr(config, "operation", "") in ("ret", "ret_bwd") and getattr(config, "waves_per_eu", 1) == 1


_AGPR_OPERAND = re.compile(r"\ba\d+\b|\ba\[\d+")
_KERNEL_LABEL = re.compile(r"^(_Z\w+):")


NUMBERED_MARK = "aat: accumulation registers addressed by number"      # left in the assembly by acc_claim_all() (utils/acc_file.h)


def foreign_accumulator_use(assembly):
    """{kernel: count} for the kernels of a device assembly listing that address accumulation registers by number (they
    carry NUMBERED_MARK) AND name such registers in instructions the compiler emitted itself (outside the #ASMSTART /
    #ASMEND pairs).  The numbered registers are invisible to the compiler's allocation: with vector registers scarce it
    loads operands or parks values in the same file, and the two uses overwrite each other.  Kernels without the mark
    (ordinary MFMA code, accumulators handed to asm statements as operands) are the compiler's own business."""
    own, foreign = {}, {}
    kernel, in_asm = None, False
    for line in assembly.splitlines():
        m = _KERNEL_LABEL.match(line)
        if m:
            kernel, in_asm = m.group(1), False
            continue
        if kernel is None:
            continue
        if NUMBERED_MARK in line:
            own[kernel] = 1
        if "#ASMSTART" in line:
            in_asm = True
            continue
        if "#ASMEND" in line:
            in_asm = False
            continue
        text = line.split(";")[0].strip()
        if not text or text.startswith("."):
            continue
        if not in_asm and _AGPR_OPERAND.search(text):
            foreign[kernel] = foreign.get(kernel, 0) + 1
    return {k: n for k, n in foreign.items() if own.get(k)}


# ---- the compiler's per-kernel resource report ---------------------------------------------------------
_USAGE_FIELDS = {"TotalSGPRs": "sgprs", "VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch_bytes",
                 "Occupancy [waves/SIMD]": "occupancy", "SGPRs Spill": "sgpr_spills", "VGPRs Spill": "vgpr_spills",
                 "LDS Size [bytes/block]": "lds_bytes"}
_USAGE_LINE = re.compile(r"remark:\s+(.+?):\s+(\S+)\s+\[-Rpass-analysis=kernel-resource-usage\]")


def parse_resource_usage(text):
    """[{"kernel": mangled name, "sgprs", "vgprs", "agprs", "scratch_bytes", "occupancy", "sgpr_spills",
    "vgpr_spills", "lds_bytes"}, ...] from the remarks hipcc prints under -Rpass-analysis=kernel-resource-usage."""
    kernels = []
    for line in text.splitlines():
        m = _USAGE_LINE.search(line)
        if not m:
            continue
        key, value = m.group(1).split(":")[-1].strip(), m.group(2)      # with -save-temps the source position follows "remark:"
        if key == "Function Name":
            kernels.append({"kernel": value})
        elif kernels and key in _USAGE_FIELDS and value.lstrip("-").isdigit():
            kernels[-1][_USAGE_FIELDS[key]] = int(value)
    return kernels


def usage_path(lib_path):
    return lib_path[:-3] + ".usage.json"


def resource_usage(lib_path):
    """The report written when ``lib_path`` was built, or None for a library built without one."""
    try:
        with open(usage_path(lib_path)) as f:
            return json.load(f)
    except (OSError, ValueError):
        return None


def template_bools(mangled):
    """Trailing boolean template arguments of a mangled kernel name, e.g. [False, True] for ...Lb0ELb1EEEv...;
    the kernels here end their template lists with the flags that select a variant (causal, decay, ...)."""
    m = re.search(r"((?:Lb[01]E)+)EEv", mangled)
    return [c == "1" for c in re.findall(r"Lb([01])E", m.group(1))] if m else []


# A few dwords of scratch outside the main loop (a saved address, a loop bound) cost nothing measurable and
# several tuned winners have them; a candidate whose working set does not fit spills hundreds of bytes.
MAX_SCRATCH_BYTES = 64


def spilling_kernels(usage, matters=None, max_bytes=MAX_SCRATCH_BYTES):
    """Entries of ``usage`` that keep more than ``max_bytes`` per lane in scratch memory (register spills or
    stack arrays), restricted to the kernels ``matters(mangled name)`` accepts."""
    return [k for k in usage or [] if k.get("scratch_bytes", 0) > max_bytes and (matters is None or matters(k["kernel"]))]


def compile_parallel(configs, arch, build_dir=None, timeout=None, max_workers=None):
    """Compile many configurations with a pool of hipcc subprocesses; result list is aligned with
    ``configs`` and holds None where a compile failed."""
    workers = max_workers or int(os.environ.get("MAX_JOBS", 0)) or os.cpu_count() or 1
    workers = max(1, min(workers, 16, len(configs) or 1))
    progress = os.environ.get("AAT_PROGRESS", "0") not in ("", "0")      # long builds under a watchdog: say that work goes on
    done = [0]

    first = {}                                     # a configuration listed twice is built once
    for c in configs:
        first.setdefault(library_path(c, build_dir), c)

    def build(c):
        lib = compile_config(c, arch, build_dir, timeout)
        done[0] += 1
        if progress and (done[0] % 8 == 0 or done[0] == len(first)):
            print(f"[build] {done[0]}/{len(first)} libraries", file=sys.stderr, flush=True)
        return lib

    with ThreadPoolExecutor(max_workers=workers) as pool:
        built = dict(zip(first, pool.map(build, first.values())))
    return [built[library_path(c, build_dir)] for c in configs]
