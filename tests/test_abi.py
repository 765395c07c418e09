"""The C ABI without a GPU: every declaration of include/paraattn_hip.h is exported by the built library
and bound by the Python loader, and argument validation (which runs before any device work) behaves."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

from paraattention_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "paraattn_hip.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"PA_API\s+[\w\s\*]+?\b(pa_\w+)\s*\(", text)


def test_header_symbols_exported_and_bound():
    names = _declared()
    assert len(names) >= 11 and len(set(names)) == len(names)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
        assert n in _lib.SIGNATURES, f"{n} declared in the header but not bound in _lib.SIGNATURES"
    assert set(_lib.SIGNATURES) == set(names)


def test_only_pa_symbols_are_exported():
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    syms = [l.split()[-1] for l in out.splitlines() if " T " in l]
    assert syms and all(s.startswith("pa_") for s in syms), syms


def test_version_and_error_text():
    lib = _lib.load()
    assert lib.pa_abi_version() == _lib.ABI_VERSION
    rc = lib.pa_merge_lse(None, 0, None, None, 0, None, None, 0, None, 0, 8, None)
    assert rc == _lib.PA_ERR_INVALID and b"null pointer" in lib.pa_last_error()
    with pytest.raises(ValueError):
        _lib.check(rc, "pa_merge_lse")
    with pytest.raises(NotImplementedError):
        _lib.check(_lib.PA_ERR_UNSUPPORTED, "x")
    with pytest.raises(_lib.HipLibraryError):
        _lib.check(_lib.PA_ERR_LAUNCH, "x")


def test_argument_validation_without_device_work():
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    base = p.value + (16 - p.value % 16) % 16
    a = ctypes.c_void_p(base)
    st = (ctypes.c_int64 * 3)(0, 4096, 128)
    # unsupported head_dim, dtype, scale, misalignment
    assert lib.pa_attn_fwd_lse(a, a, a, a, None, 0, 1, 1, 16, 16, 32, st, st, st, st, 1.0, None, 0, None) == _lib.PA_ERR_UNSUPPORTED
    assert b"head_dim" in lib.pa_last_error()
    assert lib.pa_attn_fwd_lse(a, a, a, a, None, 2, 1, 1, 16, 16, 128, st, st, st, st, 1.0, None, 0, None) == _lib.PA_ERR_UNSUPPORTED
    assert lib.pa_attn_fwd_lse(a, a, a, a, None, 0, 1, 1, 16, 16, 128, st, st, st, st, -1.0, None, 0, None) == _lib.PA_ERR_UNSUPPORTED
    odd = ctypes.c_void_p(base + 2)
    assert lib.pa_attn_fwd_lse(odd, a, a, a, None, 0, 1, 1, 16, 16, 128, st, st, st, st, 1.0, None, 0, None) == _lib.PA_ERR_UNSUPPORTED
    bad = (ctypes.c_int64 * 3)(0, 4096, 100)
    assert lib.pa_attn_fwd_lse(a, a, a, a, None, 0, 1, 1, 16, 16, 128, bad, st, st, st, 1.0, None, 0, None) == _lib.PA_ERR_UNSUPPORTED
    assert lib.pa_attn_fwd_lse(None, a, a, a, None, 0, 1, 1, 16, 16, 128, st, st, st, st, 1.0, None, 0, None) == _lib.PA_ERR_INVALID
    # the fused ring step exists for head_dim 128 only, is not causal, and says so before any launch
    # (a head_dim-64 call once slipped through to a kernel without that epilogue and wrote through a null output)
    st64 = (ctypes.c_int64 * 3)(0, 2048, 64)
    assert lib.pa_attn_fwd_accumulate(a, a, a, a, a, None, 0, 1, 1, 16, 16, 64, st64, st64, st64, None, 1.0, None, 1,
                                      None, 0, None) == _lib.PA_ERR_UNSUPPORTED
    assert b"head_dim 128" in lib.pa_last_error()
    assert lib.pa_attn_fwd_accumulate(a, a, a, None, a, None, 0, 1, 1, 16, 16, 128, st, st, st, None, 1.0, None, 1,
                                      None, 0, None) == _lib.PA_ERR_INVALID
    # empty problems succeed without touching the device
    assert lib.pa_attn_fwd_lse(a, a, a, a, None, 0, 0, 1, 16, 16, 128, st, st, st, st, 1.0, None, 0, None) == _lib.PA_OK
    assert lib.pa_merge_lse(a, 2, a, a, 0, a, a, 2, a, 0, 128, None) == _lib.PA_OK
    # merge: head_dim must be a multiple of 8; in-place needs equal dtypes
    assert lib.pa_merge_lse(a, 2, a, a, 0, a, a, 2, a, 4, 12, None) == _lib.PA_ERR_UNSUPPORTED
    assert lib.pa_merge_lse(a, 2, a, a, 0, a, a, 0, a, 4, 16, None) == _lib.PA_ERR_INVALID
    # block-sparse geometry
    assert lib.pa_blocksparse_workspace_bytes(24, 256, 256) == 4 * (24 * 258 + 24 * 258 * 131 * 2 + 2 * 24 * 256)  # counts, ranges, launch order, kept blocks per list
    assert lib.pa_blocksparse_workspace_bytes(0, 1, 1) == 0
    assert lib.pa_blocksparse_build_runs(a, 1, 2, 3, 100, 0, 64, a, 4096, None) == _lib.PA_ERR_INVALID  # 3*64 > 100
    assert lib.pa_blocksparse_build_runs(a, 1, 2, 3, 192, 0, 64, a, 8, None) == _lib.PA_ERR_WORKSPACE
    assert lib.pa_attn_fwd_blocksparse(a, a, a, a, None, 0, 1, 4, 128, 128, 128, st, st, st, st, 1.0, a, 3, 1, 1, 0, 128, 0, 128, a, 4096, None) == _lib.PA_ERR_INVALID
    # fbcache
    assert lib.pa_fbcache_workspace_bytes() >= 16
    assert lib.pa_fbcache_absdiff_ratio(a, a, 0, 0, 8, 8, 1, 8, 1, a, None, a, 1 << 20, None) == _lib.PA_ERR_INVALID
    assert lib.pa_fbcache_absdiff_ratio(a, a, 0, 1, 8, 8, 1, 8, 1, a, None, a, 8, None) == _lib.PA_ERR_WORKSPACE
    assert lib.pa_fbcache_absdiff_ratio(a, a, 7, 1, 8, 8, 1, 8, 1, a, None, a, 1 << 20, None) == _lib.PA_ERR_UNSUPPORTED
    assert lib.pa_fbcache_apply_residual(a, a, a, 0, 0, None) == _lib.PA_OK


def test_tuning_knobs_are_validated():
    lib = _lib.load()
    try:
        assert lib.pa_set_tuning(b"bm", 256) == _lib.PA_OK
        assert lib.pa_set_tuning(b"bm", 100) == _lib.PA_ERR_INVALID and b"bm" in lib.pa_last_error()
        assert lib.pa_set_tuning(b"no_such_knob", 1) == _lib.PA_ERR_INVALID
        assert lib.pa_set_tuning(None, 1) == _lib.PA_ERR_INVALID
        for name in (b"no_pipe", b"no_split", b"no_xcd_order", b"bound", b"stream", b"stream_even", b"stream_dyn", b"stream_solo", b"sparse_pair", b"wave_rows", b"short_keys", b"sparse_order"):
            assert lib.pa_set_tuning(name, 1) == _lib.PA_OK
        with pytest.raises(ValueError):
            _lib.set_tuning("bm", 64)
    finally:
        for name, val in (("no_pipe", 0), ("bm", 0), ("no_split", 0), ("no_xcd_order", 0), ("bound", -1), ("stream", -1), ("stream_even", -1), ("stream_dyn", -1), ("stream_solo", 0), ("sparse_pair", 0), ("wave_rows", 0), ("short_keys", -1), ("sparse_order", 1)):
            _lib.set_tuning(name, val)


def test_missing_library_is_loud():
    code = "import paraattention_amd._lib as l\ntry:\n    l.load()\nexcept ImportError as e:\n    print('IMPORTERROR', 'no CPU or eager fallback' in str(e))\n"
    env = dict(os.environ, PARAATTN_HIP_LIB="/nonexistent/libparaattn_hip.so", PYTHONPATH=ROOT)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env)
    assert "IMPORTERROR True" in out.stdout, out.stdout + out.stderr
