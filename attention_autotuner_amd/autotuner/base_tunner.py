"""Tuning loop: enumerate -> validate -> compile in parallel -> time through the C ABI -> log + cache.

Mirrors reference python/autotuner/base_tunner.py:68-208 (``BaseTunner``) in interface -- a tuner is
built from ``(arch, torch_array)`` and ``tune(log_path)`` returns the best configuration, consulting
an on-disk cache first -- with these deliberate changes:

* the cache key is the whole problem (arch, operator, head dims, B, H, S_q, S_kv, causal), not just
  the two head dims, because the best tile for S_q=256/S_kv=16384 is not the best for 2048/2048;
  the reference's ``best_config_{op}_{dqk}_{dv}.json`` name is still read as a fallback;
* a configuration whose compile fails or times out is skipped (the reference dereferences None);
* timing calls ``profile_ex`` on the caller's stream with the caller's softmax scale / causal flag;
* compiled libraries are kept (content-addressed), so a later ``Runtime`` reuses the tuned binary;
* the winner is run once and compared with plain torch math on the GPU before it is cached; a library
  that is fast but wrong is discarded and the next fastest is tried (``AAT_TUNE_VERIFY=0`` skips this).
"""
import ctypes
import json
import math
import os
import pprint
import re
import time

import torch

from . import codegen, library, verify
from .configs import supported_configs
from .gfx950_space import NoValidConfigError

_PKG = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
DEFAULT_CACHE_DIR = os.environ.get("AAT_CACHE_DIR", os.path.join(_PKG, "cache"))
FAILED = 1e8                          # latency recorded for a configuration that errored at run time

_memo = {}                            # in-process memo of resolved best configs (and of the operators' launch plans)
_UNSET = object()


class CompileResult:
    def __init__(self, config, lib_name):
        self.config = config
        self.lib_name = lib_name


def _stream_ptr():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class BaseTunner:
    operation = None                  # config operation name ("attn", ...)

    def __init__(self, arch, torch_array, op_name, causal=False, softmax_scale=None, decay=False, mask_mode=None):
        self.arch = arch
        # RetNet only: the mask mode the operator will launch with when that is not plain causal / dense ("scan":
        # the library scans the caller's mask for zero tiles).  Candidates are timed and verified in that mode, on the
        # caller's own mask, which need not be zero above the diagonal; the cache entry is the causal walk's.
        self.mask_mode = mask_mode
        self.decay = bool(decay)                  # RetNet only: torch_array[3] is log2(gamma) [H], not a mask
        self.torch_array = torch_array
        self.op_name = op_name
        self.causal = bool(causal)
        self.softmax_scale = softmax_scale
        self.Br_list = [32, 64, 128, 256]
        self.Bc_list = [32, 64, 128, 256]
        self.cache_path = DEFAULT_CACHE_DIR
        self.cost_model_dir = self.cache_path     # a caller that records its results elsewhere still prunes with the shipped model
        self.build_dir = None
        self.verbose = os.environ.get("AAT_VERBOSE", "0") == "1"
        q, k, v = torch_array[0], torch_array[1], torch_array[2]
        self.problem_key = {"dim_qk": int(q.shape[-1]), "dim_v": int(v.shape[-1])}
        self.problem_shape = {"B": int(q.shape[0]), "H": int(q.shape[1]), "Sq": int(q.shape[2]), "Sk": int(k.shape[2])}

    # ---- search space (filled in by subclasses) -------------------------------------------------------
    def generate_configs(self, Br, Bc, dim_qk, dim_v):
        return []

    def validate_register_fuse(self, config):
        return False

    def validate_shared_fuse(self, config):
        return False

    def validate_kernel(self, config):
        return False

    def _is_valid(self, config):
        if config.fuse_type == "register":
            return self.validate_register_fuse(config)
        if config.fuse_type == "shared":
            return self.validate_shared_fuse(config)
        return self.validate_kernel(config)

    def _fits_problem(self, config):
        s = self.problem_shape
        ns = getattr(config, "kv_splits", 1)
        if ns > 1 and (s["Sk"] // config.Bc) % ns:
            return False
        if config.operation in ("ret_bwd", "attn_bwd"):   # both lengths are resident in one pass, streamed in another
            return all(s[n] % config.Br == 0 and s[n] % config.Bc == 0 for n in ("Sq", "Sk")) and \
                s["Sk"] % getattr(config, "row_Bc", config.Bc) == 0
        return s["Sq"] % config.Br == 0 and s["Sk"] % config.Bc == 0

    def get_tuned_configs(self):
        dq, dv = self.problem_key["dim_qk"], self.problem_key["dim_v"]
        return [c for Br in self.Br_list for Bc in self.Bc_list
                for c in self.generate_configs(Br, Bc, dq, dv) if self._is_valid(c)]

    # ---- compile + time --------------------------------------------------------------------------------
    def compile(self, configs, temp_dir=None, timeout=None):
        return [self._result(c, codegen.compile_config(c, self.arch, temp_dir or self.build_dir, timeout)) for c in configs]

    def compile_parallel(self, configs, temp_dir=None, timeout=None):
        libs = codegen.compile_parallel(configs, self.arch, temp_dir or self.build_dir, timeout)
        return [self._result(c, lib) for c, lib in zip(configs, libs)]

    @staticmethod
    def _result(config, lib):
        return CompileResult(config, lib)

    def _ex_args(self):
        """Operator-specific scalar arguments between the sizes and the workspace."""
        if self.mask_mode is not None:
            from .runtime import mask_mode
            return [ctypes.c_int(mask_mode(self.mask_mode))]
        return [ctypes.c_int(int(self.causal))]

    def _workspace(self, lib, config):
        """(tensor or None, bytes): the workspace the runtime would grant ``config`` for this problem -- a stored dS
        beyond the runtime's limit is withheld there too, so what is timed is what will be launched.  Raises
        torch.cuda.OutOfMemoryError like any allocation."""
        from .runtime import _wanted
        s = self.problem_shape
        need = int(lib.workspace_size(s["B"], s["H"], s["Sq"], s["Sk"]))
        if config is not None:
            need = _wanted(config, need, s["B"], s["H"], s["Sq"], s["Sk"])
        ws = torch.empty(need, dtype=torch.uint8, device=self.torch_array[0].device) if need else None
        return ws, need

    def profile(self, libname, device="cuda:0", config=None):
        """Mean milliseconds of one launch of ``libname`` on this tuner's tensors (FAILED on error, and when the
        workspace the candidate asks for cannot be allocated)."""
        lib = library.load(libname, self.operation)
        s = self.problem_shape
        try:
            ws, need = self._workspace(lib, config)
        except torch.cuda.OutOfMemoryError:
            return FAILED
        ptrs = [ctypes.c_void_p(t.data_ptr()) for t in self.torch_array]
        entry = lib.profile_decay if self.decay else lib.profile_ex
        ms = entry(*ptrs, s["B"], s["H"], s["Sq"], s["Sk"], *([] if self.decay else self._ex_args()),
                   ctypes.c_void_p(ws.data_ptr() if ws is not None else 0), ctypes.c_size_t(need), _stream_ptr())
        return FAILED if ms < 0 else float(ms)

    def verify(self, libname, config=None):
        """Run ``libname`` once on this tuner's tensors and compare its outputs with torch math."""
        if not hasattr(self, "_reference"):
            scale = None if len(self._ex_args()) == 1 else self._ex_args()[0].value
            self._reference = verify.reference_outputs(self.operation, self.torch_array, scale, self.causal, self.decay)
        lib = library.load(libname, self.operation)
        s = self.problem_shape
        try:
            ws, need = self._workspace(lib, config)
        except torch.cuda.OutOfMemoryError:
            return False
        for idx in self._reference:
            self.torch_array[idx].zero_()
        ptrs = [ctypes.c_void_p(t.data_ptr()) for t in self.torch_array]
        entry = lib.kernel_entry_decay if self.decay else lib.kernel_entry_ex
        rc = entry(*ptrs, s["B"], s["H"], s["Sq"], s["Sk"], *([] if self.decay else self._ex_args()),
                   ctypes.c_void_p(ws.data_ptr() if ws is not None else 0), ctypes.c_size_t(need), _stream_ptr())
        torch.cuda.synchronize()
        return rc == 0 and verify.outputs_match(self.torch_array, self._reference)

    # ---- cache -----------------------------------------------------------------------------------------
    def _cache_file(self):
        k, s = self.problem_key, self.problem_shape
        return os.path.join(self.cache_path, "best_config_{}_{}_{}_{}_b{}h{}q{}k{}_c{}.json".format(
            self.op_name + ("_decay" if self.decay else ""), self.arch.name, k["dim_qk"], k["dim_v"], s["B"], s["H"], s["Sq"], s["Sk"], int(self.causal)))

    def _legacy_cache_file(self):
        k = self.problem_key
        return os.path.join(self.cache_path, "best_config_{}_{}_{}.json".format(self.op_name, k["dim_qk"], k["dim_v"]))

    def _memo_key(self):
        return (self._cache_file(),)

    def check_cache(self):
        hit = _memo.get(self._memo_key())
        if hit is not None:
            return hit
        for path in (self._cache_file(), self._legacy_cache_file()):
            try:
                with open(path) as f:
                    dd = json.load(f)
                cfg = supported_configs[dd["operation"]].from_dict(dd)
            except (OSError, ValueError, KeyError):
                continue                                  # missing or corrupt cache file: fall through
            if self._fits_problem(cfg):
                _memo[self._memo_key()] = cfg
                return cfg
        return None

    nearest_limit = 12.0       # e.g. one length and the row count a factor 16 apart

    def nearest_cached(self):
        """The tuned configuration of the closest problem this cache holds for the same operator, head sizes and mask
        walk whose tiles also divide this problem's lengths, or None.  For callers that do not want a tuning run on a
        miss: the reference keys its cache by the two head sizes alone (python/autotuner/base_tunner.py:190-208), i.e. it always launches
        whatever was tuned first; here the entry of the nearest lengths and block count stands in, and only then the
        built-in default.  Distance in octaves: lengths count twice (they decide tile sizes and the kv split), the number
        of rows in the launch once (it decides how many blocks a CU gets); an entry more than ``nearest_limit`` away says
        nothing about this problem."""
        s = self.problem_shape
        stem = os.path.basename(self._cache_file()).split("_b%d" % s["B"])[0]
        pat = re.compile(re.escape(stem) + r"_b(\d+)h(\d+)q(\d+)k(\d+)_c%d\.json$" % int(self.causal))
        try:
            names = sorted(os.listdir(self.cache_path))
        except OSError:
            return None
        found = []
        for name in names:
            m = pat.match(name)
            if not m:
                continue
            b, h, sq, sk = (int(x) for x in m.groups())
            far = 2 * abs(math.log2(sq / s["Sq"])) + 2 * abs(math.log2(sk / s["Sk"])) + \
                abs(math.log2((b * h * sq) / (s["B"] * s["H"] * s["Sq"])))
            if far <= self.nearest_limit:
                found.append((far, name))
        for _, name in sorted(found):
            try:
                with open(os.path.join(self.cache_path, name)) as f:
                    dd = json.load(f)
                cfg = supported_configs[dd["operation"]].from_dict(dd)
            except (OSError, ValueError, KeyError):
                continue
            if self._fits_problem(cfg):
                _memo[self._memo_key()] = cfg             # this process keeps launching it for this problem
                return cfg
        return None

    def _write_cache(self, config):
        os.makedirs(self.cache_path, exist_ok=True)
        with open(self._cache_file(), "w") as f:
            json.dump(config.to_dict(), f)
        for key in [k for k in _memo if k[0] == "plan"]:      # launch plans the operators resolved before this entry existed
            del _memo[key]
        _memo[self._memo_key()] = config

    # ---- what is not worth timing ----------------------------------------------------------------------
    def _kernel_matters(self, mangled):
        """Whether a kernel of a candidate library is one this tuner's problem launches (a library holds
        several variants: causal or not, decay mask or mask tensor)."""
        return True

    # A fitted costmodel.CostModel: tune() then times only its best-ranked candidates.  Subclasses name a model file
    # next to the tuning cache; it is read when first asked for, not when the tuner is built: an operator builds a
    # tuner on every call of a problem it has not launched before, and only a tuning run needs the model.
    cost_model_file = None
    _cost_model = _UNSET

    @property
    def cost_model(self):
        if self._cost_model is _UNSET:
            self._cost_model = self._shipped_cost_model()
        return self._cost_model

    @cost_model.setter
    def cost_model(self, model):
        self._cost_model = model

    def _shipped_cost_model(self):
        return None

    keep_fraction = 0.35       # ... this share of them (at least keep_min)
    keep_min = 8

    def prune(self, configs):
        """The candidates worth compiling and timing: all of them without a cost model, else those the
        model ranks in the best ``keep_fraction`` (reference python/tests/export_costmodel_config.py:31-56
        exports (configuration, cycles) pairs for such a model; the model itself is autotuner/costmodel.py)."""
        self.pruned = []
        if self.cost_model is None or len(configs) <= self.keep_min:
            return configs
        shape = (self.problem_shape["B"], self.problem_shape["H"], self.problem_shape["Sq"], self.problem_shape["Sk"])
        ranked = sorted(configs, key=lambda c: self.cost_model.predict(c, shape, self.causal))
        keep = max(self.keep_min, int(len(ranked) * self.keep_fraction + 0.999))
        self.pruned = ranked[keep:]
        return ranked[:keep]

    # ---- the loop --------------------------------------------------------------------------------------
    def tune(self, log_path="../logs/", timeout=120, use_cache=True):
        started = time.time()
        if use_cache:
            cached = self.check_cache()
            if cached is not None:
                return cached
        configs = [c for c in self.get_tuned_configs() if self._fits_problem(c)]
        if not configs:
            raise NoValidConfigError(f"no valid {self.op_name} configuration for {self.problem_key} {self.problem_shape}")
        if self.verbose:
            print("Configs to be tuned: ")
            for c in configs:
                pprint.pprint(c)
        configs = self.prune(configs)
        results = self.compile_parallel(configs, timeout=timeout)
        timings, best, best_ms = {}, None, FAILED
        self.rejected_spills = {}
        for res in results:
            if res.lib_name is None:
                continue                                  # compile failed or timed out
            spills = codegen.spilling_kernels(codegen.resource_usage(res.lib_name), self._kernel_matters)
            if spills and os.environ.get("AAT_TUNE_SPILLS", "0") == "0":
                # the compiler says this candidate keeps part of its working set in scratch memory: not worth timing
                self.rejected_spills[res.config] = max(k.get("scratch_bytes", 0) for k in spills)
                continue
            ms = self.profile(res.lib_name, config=res.config)
            if ms == FAILED and self.verbose:
                pprint.pprint(res.config)
                print("profile runtime error")
            timings[res.config] = ms
            if ms < best_ms:
                best, best_ms = res.config, ms
        if best is not None and os.environ.get("AAT_TUNE_VERIFY", "1") != "0":
            libs = {res.config: res.lib_name for res in results}
            best = None
            for cfg in sorted((c for c, ms in timings.items() if ms < FAILED), key=timings.get):
                if self.verify(libs[cfg], config=cfg):
                    best, best_ms = cfg, timings[cfg]
                    break
                timings[cfg] = FAILED                     # fast but wrong: never cache it
                if self.verbose:
                    print("output mismatch, discarded:", cfg)
        if best is None:
            raise RuntimeError(f"every {self.op_name} candidate failed to compile, run or verify")
        elapsed = time.time() - started
        if self.verbose:
            print("#" * 58)
            print("Operation type: ", best.operation)
            print("Best config: ")
            pprint.pprint(best)
            print("Latency: ", best_ms)
        self._write_log(log_path, timings, best, best_ms, elapsed)
        self._write_cache(best)
        self.last_timings = timings
        return best

    def _write_log(self, log_path, timings, best, best_ms, elapsed):
        """Same text layout as the reference's profile_result_*.txt (base_tunner.py:178-188)."""
        if log_path is None:
            return
        k = self.problem_key
        os.makedirs(log_path, exist_ok=True)
        name = "profile_result_{}_{}_{}.txt".format(best.operation, k["dim_qk"], k["dim_v"])
        with open(os.path.join(log_path, name), "w") as f:
            for cfg, ms in timings.items():
                f.write(repr(cfg) + "\n" + str(ms) + "\n")
            f.write("\nbest config: \n" + repr(best) + "\n" + str(best_ms) + "\n")
            f.write("\nsearch time: " + str(elapsed) + "s")
            # after the reference's layout: what was never timed, and why
            for cfg, nbytes in getattr(self, "rejected_spills", {}).items():
                f.write("\nnot timed (compiler reports " + str(nbytes) + " bytes/lane of scratch): " + str(cfg))
            for cfg in getattr(self, "pruned", []):
                f.write("\nnot timed (ranked out by the cost model): " + str(cfg))
