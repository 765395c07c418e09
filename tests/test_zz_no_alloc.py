"""The entry point that allocates nothing (pa_attn_fwd_lse_noalloc): called through the C ABI and compared
with pa_attn_fwd_lse_ws on the same inputs, on two calls in a row (the second smaller, so that it meets the
first call's leftovers in the library's static scratch buffer)."""
import ctypes
import math

import pytest
import torch

from oracle import attention as oattn
from oracle import inputs
from paraattention_amd import _lib

pytestmark = pytest.mark.gpu


def _vp(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _call_ws(lib, q, k, v, causal=0):
    B, H, Sq, D = q.shape
    Skv = k.shape[2]
    out, lse = torch.empty_like(q), torch.empty((B, H, Sq), dtype=torch.float32, device=q.device)
    need = lib.pa_attn_fwd_workspace_bytes(B, H, Sq, Skv, D, _lib.strides3(k), _lib.strides3(v))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    rc = lib.pa_attn_fwd_lse_ws(_vp(q), _vp(k), _vp(v), _vp(out), _vp(lse), 0, B, H, Sq, Skv, D, _lib.strides3(q),
                                _lib.strides3(k), _lib.strides3(v), _lib.strides3(out), 1.0 / math.sqrt(D), None, causal,
                                _vp(ws), need, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, lib.pa_last_error()
    torch.cuda.synchronize()
    return out, lse, need


def _call_noalloc(lib, q, k, v, causal=0):
    B, H, Sq, D = q.shape
    Skv = k.shape[2]
    out, lse = torch.empty_like(q), torch.empty((B, H, Sq), dtype=torch.float32, device=q.device)
    rc = lib.pa_attn_fwd_lse_noalloc(_vp(q), _vp(k), _vp(v), _vp(out), _vp(lse), 0, B, H, Sq, Skv, D, _lib.strides3(q),
                                     _lib.strides3(k), _lib.strides3(v), _lib.strides3(out), 1.0 / math.sqrt(D), None, causal,
                                     ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return rc, out, lse


def test_noalloc_matches_workspace_entry_on_two_calls(cuda, tuning):
    lib = _lib.load()
    tuning("bound", 1)  # the score bound's words at the front of the scratch are used at these small sizes too
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    B, H, D = 2, 4, 128
    tuning("bm", 256)
    # first call: a grid a little over a whole number of rounds, so the launch splits the keys of its last
    # query tiles and parks fp32 partial results in the scratch; second call: fewer rows and keys, another plan
    shapes = [((cus // (B * H) + 5) * 256 - 19, 64 * 40 + 37), (3 * 256 + 77, 64 * 21 + 5)]
    first_need = None
    for Sq, Skv in shapes:
        q, k, v = (t.to(cuda) for t in inputs.qkv(B, H, Sq, Skv, D, seed=Sq))
        want_out, want_lse, need = _call_ws(lib, q, k, v)
        first_need = need if first_need is None else first_need
        before = torch.cuda.memory_allocated()
        rc, out, lse = _call_noalloc(lib, q, k, v)
        assert rc == 0, lib.pa_last_error()
        torch.cuda.synchronize()
        grown = torch.cuda.memory_allocated() - before  # torch's own count: only the two outputs (rounded to its 512-byte blocks)
        assert grown <= out.numel() * 2 + lse.numel() * 4 + 1024
        assert torch.equal(out, want_out) and torch.equal(lse, want_lse), (Sq, Skv)
        ref_out, ref_lse = oattn.sdpa_lse_torch_cpu(q[:, :1].cpu(), k[:, :1].cpu(), v[:, :1].cpu())
        assert (out[:, :1].float().cpu() - ref_out.float()).abs().max().item() <= 2e-2 + 2e-2 * ref_out.float().abs().max().item()
        assert (lse[:, :1].cpu() - ref_lse).abs().max().item() <= 1e-3
    assert first_need > 16384, "the first shape is meant to take the key-split path (partials in the scratch)"


def test_noalloc_with_resident_workgroups(cuda, tuning):
    """The default plan of a dense call (resident workgroups, the ragged last round cut into ranges whose partial
    results lie in the scratch): bit for bit the workspace entry's result, on two calls in a row."""
    lib = _lib.load()
    tuning("bound", 1)
    tuning("stream", 1)  # the second, small problem would by itself go to the kernels with one workgroup per query tile
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    B, D = 1, 128
    for H, Sq, Skv in ((4, (cus // 4 + 25) * 256 - 50, 64 * 30 + 11), (3, 9 * 256 + 3, 64 * 9)):
        q, k, v = (t.to(cuda) for t in inputs.qkv(B, H, Sq, Skv, D, seed=Sq))
        want_out, want_lse, need = _call_ws(lib, q, k, v)
        assert need > 16384, "meant to cut pieces (partial results in the workspace)"
        rc, out, lse = _call_noalloc(lib, q, k, v)
        assert rc == 0, lib.pa_last_error()
        torch.cuda.synchronize()
        assert torch.equal(out, want_out) and torch.equal(lse, want_lse), (H, Sq, Skv)
        ref_out, ref_lse = oattn.sdpa_lse_torch_cpu(q[:, :1].cpu(), k[:, :1].cpu(), v[:, :1].cpu())
        assert (out[:, :1].float().cpu() - ref_out.float()).abs().max().item() <= 2e-2 + 2e-2 * ref_out.float().abs().max().item()
        assert (lse[:, :1].cpu() - ref_lse).abs().max().item() <= 1e-3


def test_noalloc_refuses_what_the_buffer_cannot_hold(cuda, tuning):
    lib = _lib.load()
    tuning("bm", 256)
    tuning("stream", 0)  # the key-split plan (the resident-workgroup plan keeps these 150 pieces whole and needs nothing)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    # one head, a round and 150 query tiles more, long keys: the plan splits the 150 tiles' keys several ways
    B, H, D, Sq, Skv = 1, 1, 128, (cus + 150) * 256, 16384
    q, k, v = (t.to(cuda) for t in inputs.qkv(B, H, Sq, Skv, D, seed=1))
    need = lib.pa_attn_fwd_workspace_bytes(B, H, Sq, Skv, D, _lib.strides3(k), _lib.strides3(v))
    if need <= _lib.PA_NOALLOC_SCRATCH_BYTES:
        pytest.skip(f"this device's plan for the shape needs {need} bytes, which the buffer holds")
    rc, _, _ = _call_noalloc(lib, q, k, v)
    assert rc == _lib.PA_ERR_WORKSPACE and b"static buffer holds" in lib.pa_last_error()
    # the entry with a caller's workspace takes the same problem
    out, lse, _ = _call_ws(lib, q, k, v)
    assert torch.isfinite(lse).all()
    # with is_causal the same shape is taken: a causal launch never cuts its keys and uses the score bound's few KB only
    tuning("bound", 1)
    assert lib.pa_attn_fwd_call_workspace_bytes(B, H, Sq, Skv, D, _lib.strides3(k), _lib.strides3(v), 0, 1) <= 16384
    assert lib.pa_attn_fwd_call_workspace_bytes(B, H, Sq, Skv, D, _lib.strides3(k), _lib.strides3(v), 1, 0) >= need  # the key-split plan (+ the bound's words)
    rc, cout, clse = _call_noalloc(lib, q, k, v, causal=1)
    assert rc == 0, lib.pa_last_error()
    torch.cuda.synchronize()
    want_out, want_lse, _ = _call_ws(lib, q, k, v, causal=1)
    assert torch.equal(cout, want_out) and torch.equal(clse, want_lse)
    rows = torch.tensor([0, 1, 255, 256, 4097, Skv - 1, Skv, Sq - 1])
    keep = (torch.arange(Skv)[None, :] <= rows[:, None])[None, None]
    ref_out, ref_lse = oattn.sdpa_lse_torch_cpu(q[:, :, rows].cpu(), k.cpu(), v.cpu(), attn_mask=keep)
    assert (cout[:, :, rows.to(cuda)].float().cpu() - ref_out.float()).abs().max().item() <= 2e-2 + 2e-2 * ref_out.float().abs().max().item()
    assert (clse[:, :, rows.to(cuda)].cpu() - ref_lse).abs().max().item() <= 1e-3
