"""ctypes binding of libparaattn_hip.so (the C ABI declared in include/paraattn_hip.h).

The library is built in-tree by ``paraattention_amd/csrc/Makefile`` (or
``__graft_entry__.build()``).  There is no fallback: if the shared object is
missing, loading raises and every op of this package raises with it.
"""
import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
# PARAATTN_HIP_LIB points at another build of the same ABI (kernel experiments); default = in-tree
LIB_PATH = os.environ.get("PARAATTN_HIP_LIB") or os.path.join(_HERE, "libparaattn_hip.so")

PA_OK = 0
PA_ERR_INVALID = -1
PA_ERR_UNSUPPORTED = -2
PA_ERR_LAUNCH = -3
PA_ERR_WORKSPACE = -4

PA_DTYPE_BF16 = 0
PA_DTYPE_F16 = 1
PA_DTYPE_F32 = 2

PA_NOALLOC_SCRATCH_BYTES = 80 << 20

PA_MASK_BOOL = 1
PA_MASK_F32 = 2
PA_MASK_ACT = 3

ABI_VERSION = 4

_vp = ctypes.c_void_p
_i = ctypes.c_int
_i64 = ctypes.c_int64
_f = ctypes.c_float
_sz = ctypes.c_size_t
_strides = ctypes.POINTER(ctypes.c_int64)
_ptrs = ctypes.POINTER(ctypes.c_void_p)  # host array of device pointers
_floats = ctypes.POINTER(ctypes.c_float)  # host array

# name -> (restype, argtypes); mirrors include/paraattn_hip.h declaration by declaration
SIGNATURES = {
    "pa_abi_version": (_i, []),
    "pa_last_error": (ctypes.c_char_p, []),
    "pa_set_tuning": (_i, [ctypes.c_char_p, _i]),
    "pa_attn_fwd_lse": (
        _i,
        [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _strides, _strides, _strides, _strides, _f, _vp, _i, _vp],
    ),
    "pa_attn_fwd_lse_ws": (
        _i,
        [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _strides, _strides, _strides, _strides, _f, _vp, _i,
         _vp, _sz, _vp],
    ),
    "pa_attn_fwd_masked": (
        _i,
        [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _strides, _strides, _strides, _strides, _f,
         _vp, _i, _strides, _vp, _sz, _vp],
    ),
    "pa_attn_fwd_masked_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _strides, _strides]),
    "pa_attn_fwd_lse_noalloc": (
        _i,
        [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _strides, _strides, _strides, _strides, _f, _vp, _i, _vp],
    ),
    "pa_attn_fwd_accumulate": (
        _i,
        [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _strides, _strides, _strides, _strides, _f, _vp,
         _i, _vp, _sz, _vp],
    ),
    "pa_attn_fwd_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _strides, _strides]),
    "pa_attn_fwd_call_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _strides, _strides, _i, _i]),
    "pa_attn_fwd_sweep": (
        _i,
        [_vp, _ptrs, _ptrs, _i, _i, _vp, _vp, _i, _i, _i, _i, _i, _strides, _strides, _strides, _strides, _f, _vp, _sz, _vp],
    ),
    "pa_attn_fwd_sweep_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _i, _strides, _strides]),
    "pa_attn_fwd_blocksparse": (
        _i,
        [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _strides, _strides, _strides, _strides, _f,
         _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp],
    ),
    "pa_attn_fwd_blocksparse_runs": (
        _i,
        [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _strides, _strides, _strides, _strides, _f,
         _i, _i, _i, _i, _i, _vp, _sz, _vp],
    ),
    "pa_blocksparse_workspace_bytes": (_sz, [_i, _i, _i]),
    "pa_blocksparse_build_runs": (_i, [_vp, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "pa_merge_lse": (_i, [_vp, _i, _vp, _vp, _i, _vp, _vp, _i, _vp, _i64, _i, _vp]),
    "pa_taylorseer_update": (_i, [_vp, _ptrs, _ptrs, _i, _i, _i64, _f, _vp]),
    "pa_taylorseer_value": (_i, [_ptrs, _i, _floats, _floats, _vp, _vp, _i, _i64, _vp]),
    "pa_fbcache_absdiff_ratio": (
        _i,
        [_vp, _vp, _i, _i64, _i64, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _sz, _vp],
    ),
    "pa_fbcache_workspace_bytes": (_sz, []),
    "pa_fbcache_residual_ratio": (_i, [_vp, _vp, _vp, _vp, _i, _i64, _vp, _vp, _vp, _sz, _vp]),
    "pa_fbcache_apply_residual": (_i, [_vp, _vp, _vp, _i, _i64, _vp]),
}

_lib = None
_lock = threading.Lock()


class HipLibraryError(RuntimeError):
    """A call into libparaattn_hip.so returned an error code."""


def load():
    """Load (once) and return the ctypes handle; raises if the library is not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
                "(hipcc, --offload-arch=gfx950). paraattention_amd has no CPU or eager fallback."
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        got = lib.pa_abi_version()
        if got != ABI_VERSION:
            raise ImportError(f"{LIB_PATH}: ABI version {got}, this package expects {ABI_VERSION}; rebuild it")
        _lib = lib
    return _lib


def check(rc, what):
    """Turn a PA_ERR_* return code into the exception the reference's op would raise."""
    if rc == PA_OK:
        return
    msg = load().pa_last_error().decode("utf-8", "replace")
    text = f"{what}: {msg} (code {rc})"
    if rc == PA_ERR_UNSUPPORTED:
        raise NotImplementedError(text)
    if rc == PA_ERR_INVALID:
        raise ValueError(text)
    raise HipLibraryError(text)


def set_tuning(name, value):
    """Set one tuning / test knob of the attention launches (pa_set_tuning in the header): "no_pipe", "bm",
    "no_split", "no_xcd_order", "bound", "stream", "stream_even", "stream_dyn", "stream_solo", "sparse_pair", "wave_rows", "short_keys", "sparse_order".  The PARAATTN_* environment variables only give the initial values."""
    check(load().pa_set_tuning(name.encode(), int(value)), "pa_set_tuning")


def strides3(t):
    """(batch, head, seq) strides of a 4-D tensor as a C int64[3]; size-1 dims get stride 0."""
    st = [0 if t.shape[d] == 1 else t.stride(d) for d in range(3)]
    return (ctypes.c_int64 * 3)(*st)
