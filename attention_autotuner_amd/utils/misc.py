"""Small helpers for scripts (reference python/utils/misc.py:4-13)."""
import torch


def is_close_my(a, a_ref, rtol=1e-3, atol=1e-3):
    """``torch.testing.assert_close`` that reports instead of raising; returns True when close."""
    try:
        torch.testing.assert_close(a, a_ref, rtol=rtol, atol=atol)
        return True
    except AssertionError as e:
        print(e)
        return False


def max_abs_err(a, b):
    return (a.detach().float().cpu() - b.detach().float().cpu()).abs().max().item()
