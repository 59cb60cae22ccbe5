"""Shared by the two operator front ends: pick the configuration to launch."""
import os

import torch

from ..autotuner import base_tunner
from ..autotuner.runtime import Runtime

_PKG = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
DEFAULT_LOG_DIR = os.environ.get("AAT_LOG_DIR", os.path.join(_PKG, "logs"))


def tune_on_miss():
    """The reference tunes whenever its cache has no entry; set AAT_TUNE_ON_MISS=0 to launch the
    configuration tuned for the nearest problem of the same head sizes instead, or the built-in default
    where there is none (no compile storm on first use)."""
    return os.environ.get("AAT_TUNE_ON_MISS", "1") != "0"


def resolve(tuner, default_factory):
    cfg = tuner.check_cache()
    if cfg is not None:
        return cfg
    if tune_on_miss():
        return tuner.tune(log_path=DEFAULT_LOG_DIR)
    return tuner.nearest_cached() or default_factory()


def planned(key, make_tuner, default_factory):
    """``(configuration, Runtime)`` for the problem ``key`` (operator, shapes, mask walk): resolved through a tuner the
    first time this process meets the problem and kept in the tuners' own memo, so that every later call costs one
    dictionary lookup instead of a tuner, a cache-file name and a library path (the reference reads its JSON cache,
    python/autotuner/base_tunner.py:197-206, and opens the library, python/autotuner/runtime.py:74-82, on every call;
    its README.md:113 lists "the performance of python interface?" as open)."""
    k = ("plan", base_tunner.DEFAULT_CACHE_DIR, tune_on_miss()) + key
    plan = base_tunner._memo.get(k)
    if plan is None:
        tuner = make_tuner()
        cc = resolve(tuner, default_factory)
        plan = base_tunner._memo[k] = (cc, Runtime(tuner.arch, cc))
    return plan


class NoGraph:
    """Stands in for the autograd context when no input of a call requires a gradient: the operators then run their
    forward directly (an inference call skips the ~15 us a ``torch.autograd.Function.apply`` costs on the host)."""
    needs_input_grad = (False,) * 8

    def save_for_backward(self, *tensors):
        pass


def wants_graph(*tensors):
    return torch.is_grad_enabled() and any(t.requires_grad for t in tensors)
