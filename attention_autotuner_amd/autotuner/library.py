"""ctypes binding of a config library (the Python side of include/aat_kernel_abi.h)."""
import ctypes
import threading

_VP, _I, _F, _SZ = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t

# number of device-pointer arguments per operator
N_POINTERS = {"attn": 4, "ret": 6, "ret_bwd": 10, "attn_bwd": 9}
# operators whose extended entry points take a softmax scale in front of the causal flag
SCALED_OPS = ("attn", "attn_bwd")
# operators that also export the reference-signature pair profile / kernel_entry
LEGACY_OPS = ("attn", "ret", "ret_bwd")
# operators with a decay-mask variant (profile_decay / kernel_entry_decay)
DECAY_OPS = ("ret", "ret_bwd")

_handles = {}
_lock = threading.Lock()


class KernelLibraryError(RuntimeError):
    pass


def _bind(lib, op):
    n = N_POINTERS[op]
    ptrs = [_VP] * n
    lib.abi_version.restype = _I
    lib.abi_version.argtypes = []
    lib.config_string.restype = ctypes.c_char_p
    lib.config_string.argtypes = []
    lib.workspace_size.restype = _SZ
    lib.workspace_size.argtypes = [_I] * 4
    if op in LEGACY_OPS:
        lib.profile.restype = _F
        lib.profile.argtypes = ptrs + [_I] * 4
        lib.kernel_entry.restype = _I
        lib.kernel_entry.argtypes = ptrs + [_I] * 4
    extra = [_F, _I] if op in SCALED_OPS else [_I]   # attention: scale + causal; RetNet: causal
    tail = extra + [_VP, _SZ, _VP]                   # workspace, bytes, stream
    if op == "attn":
        lib.kernel_entry_lse.restype = _I
        lib.kernel_entry_lse.argtypes = [_VP] * 5 + [_I] * 4 + tail
    if op in DECAY_OPS:                               # mask slot carries log2(gamma) [H]; dqaccum and causal are gone
        nd = n - 1 if op == "ret_bwd" else n
        lib.profile_decay.restype = _F
        lib.profile_decay.argtypes = [_VP] * nd + [_I] * 4 + [_VP, _SZ, _VP]
        lib.kernel_entry_decay.restype = _I
        lib.kernel_entry_decay.argtypes = [_VP] * nd + [_I] * 4 + [_VP, _SZ, _VP]
    lib.profile_ex.restype = _F
    lib.profile_ex.argtypes = ptrs + [_I] * 4 + tail
    lib.kernel_entry_ex.restype = _I
    lib.kernel_entry_ex.argtypes = ptrs + [_I] * 4 + tail
    return lib


def _bind_recurrent(lib):
    """The RetNet recurrent library: reference-named entry points instead of profile / kernel_entry."""
    lib.abi_version.restype = _I
    lib.abi_version.argtypes = []
    lib.config_string.restype = ctypes.c_char_p
    lib.config_string.argtypes = []
    lib.workspace_size.restype = _SZ
    lib.workspace_size.argtypes = [_I] * 4
    dims = [_I] * 6                                   # batch, heads, kdim, vdim, l, block_kdim
    lib.retnet_recurrent_workspace_size.restype = _SZ
    lib.retnet_recurrent_workspace_size.argtypes = dims
    lib.retnet_recurrent_fwd.restype = None
    lib.retnet_recurrent_fwd.argtypes = [_VP] * 5 + dims
    lib.retnet_recurrent_fwd_ex.restype = _I
    lib.retnet_recurrent_fwd_ex.argtypes = [_VP] * 5 + dims + [_VP, _SZ, _VP]
    lib.retnet_recurrent_profile.restype = _F
    lib.retnet_recurrent_profile.argtypes = [_VP] * 5 + dims + [_VP, _SZ, _VP]
    lib.retnet_recurrent_fwd_noalloc.restype = _I
    lib.retnet_recurrent_fwd_noalloc.argtypes = [_VP] * 5 + dims + [_VP]
    return lib


def load_recurrent(path):
    return load(path, "ret_recurrent")


def load(path, op):
    """dlopen ``path`` once per process and set the prototypes for operator ``op``."""
    key = (path, op)
    lib = _handles.get(key)
    if lib is None:
        with _lock:
            lib = _handles.get(key)
            if lib is None:
                try:
                    lib = _bind_recurrent(ctypes.CDLL(path)) if op == "ret_recurrent" else _bind(ctypes.CDLL(path), op)
                except (OSError, AttributeError) as e:
                    raise KernelLibraryError(f"cannot load kernel library {path}: {e}") from e
                _handles[key] = lib
    return lib
