from .misc import is_close_my, max_abs_err

__all__ = ["is_close_my", "max_abs_err"]
