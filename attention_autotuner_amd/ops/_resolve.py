"""Shared by the two operator front ends: pick the configuration to launch."""
import os

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
