"""The interception modes route F.scaled_dot_product_attention to the HIP kernels
(src/para_attn/para_attn_interface.py:395-479, src/para_attn/sparse_attn.py:607-640)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import paraattention_amd
from oracle import attention as oattn
from oracle import inputs
from paraattention_amd import interface

pytestmark = pytest.mark.gpu


def test_unified_attn_mode_routes_to_the_kernel(cuda):
    q, k, v = inputs.qkv(1, 3, 200, 333, 128, seed=12)
    ref_out, _ = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy())
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    assert interface.kernel_takes(qd, kd, vd)
    direct = torch.ops.para_attn.attention_forward(qd, kd, vd)
    with paraattention_amd.UnifiedAttnMode():
        out = F.scaled_dot_product_attention(qd, kd, vd)
        scaled = F.scaled_dot_product_attention(qd, kd, vd, scale=0.05)
        f32 = F.scaled_dot_product_attention(qd.float(), kd.float(), vd.float())  # not the kernel's: aten
    assert torch.equal(out, direct)  # the same kernel, not aten's
    np.testing.assert_allclose(out.float().cpu().numpy(), ref_out, atol=2e-2, rtol=2e-2)
    assert torch.equal(scaled, torch.ops.para_attn.attention_forward(qd, kd, vd, scale=0.05))
    assert f32.dtype == torch.float32
    np.testing.assert_allclose(f32.cpu().numpy(), ref_out, atol=2e-3, rtol=2e-3)
    with paraattention_amd.config.patch(**{"attention.force_dispatch_to_custom_ops": True}):
        with paraattention_amd.UnifiedAttnMode(attn_func=lambda *a, **kw: "never"):
            assert torch.equal(F.scaled_dot_product_attention(qd, kd, vd), direct)
    # [B,S,H,D] memory, as diffusers hands it over
    qs = qd.transpose(1, 2).contiguous().transpose(1, 2)
    with paraattention_amd.UnifiedAttnMode():
        assert torch.equal(F.scaled_dot_product_attention(qs, kd, vd), direct)


def test_sparse_kv_mode(cuda):
    B, H, Sq, Skv, D = 2, 2, 100, 300, 128
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=13)
    keep = torch.arange(Skv)[None, :] < torch.tensor([300, 177])[:, None]
    ref_out, _ = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, keep[:, None, None, :].numpy())
    mask = keep[:, None, None, :].expand(B, 1, Sq, Skv).to(cuda)
    with paraattention_amd.SparseKVAttnMode():
        out = F.scaled_dot_product_attention(q.to(cuda), k.to(cuda), v.to(cuda), attn_mask=mask)
    np.testing.assert_allclose(out.float().cpu().numpy(), ref_out, atol=2e-2, rtol=2e-2)
    assert torch.equal(out, paraattention_amd.sparse_kv_attn_func(q.to(cuda), k.to(cuda), v.to(cuda), attn_mask=mask))
    with paraattention_amd.SparseKVAttnMode():
        with paraattention_amd.SparseKVAttnMode.disable():
            aten = F.scaled_dot_product_attention(q.to(cuda), k.to(cuda), v.to(cuda), attn_mask=mask)
    np.testing.assert_allclose(aten.float().cpu().numpy(), ref_out, atol=2e-2, rtol=2e-2)
    # under the unified mode a key-only mask goes to the kernel as well
    with paraattention_amd.UnifiedAttnMode():
        out2 = F.scaled_dot_product_attention(q.to(cuda), k.to(cuda), v.to(cuda), attn_mask=keep[:, None, None, :].to(cuda))
    assert torch.equal(out2, out)


@pytest.mark.parametrize("is_causal", [False, True])
def test_compiled_function_under_the_mode(cuda, is_causal):
    """The reference's mode test compiled (tests/test_interface.py:94-109): F.scaled_dot_product_attention inside
    torch.compile(fullgraph=True), the mode entered around the call, two calls."""
    q, k, v = (t.to(cuda) for t in inputs.qkv(1, 3, 257, 257, 128, seed=4))

    def func(*args, **kwargs):
        return F.scaled_dot_product_attention(*args, **kwargs)

    compiled = torch.compile(func, fullgraph=True, backend="aot_eager")
    for _ in range(2):
        with paraattention_amd.UnifiedAttnMode():
            out = compiled(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=is_causal)
    assert torch.equal(out, torch.ops.para_attn.attention_forward(q, k, v, is_causal=is_causal))
    keep = oattn.causal_keep(257, 257) if is_causal else None
    ref_out, _ = oattn.sdpa_lse_f64(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), None, keep)
    np.testing.assert_allclose(out.float().cpu().numpy(), ref_out, atol=2e-2, rtol=2e-2)


def _bshd(t):
    """The same values in [B,S,H,D] memory viewed as [B,H,S,D]: what a diffusers processor hands to SDPA."""
    return t.transpose(1, 2).contiguous().transpose(1, 2)


def _strided_cases(cuda):
    q, k, v = (t.to(cuda) for t in inputs.qkv(2, 3, 200, 256, 128, seed=31))
    odd = torch.empty(2, 3, 200, 132, dtype=q.dtype, device=cuda)[..., :128]  # row stride 132: not 16-byte aligned rows
    odd.copy_(q)
    return {"contiguous": q, "bshd": _bshd(q), "unaligned_rows": odd}, k, v


def test_fake_outputs_have_the_real_layout(cuda):
    """Every op that returns attention output is run on real and on fake tensors (torch.library.opcheck's
    test_faketensor: sizes, strides, dtype and device of the fake result must equal the real one's), with the
    query contiguous, in [B,S,H,D] memory (output keeps that layout) and with rows the kernels cannot take in
    place (output contiguous).  The reference's fakes run the aten kernels on FakeTensors
    (src/para_attn/ops/__init__.py:182-201, 226-245), so theirs agree by construction."""
    from torch.library import opcheck

    queries, k, v = _strided_cases(cuda)
    ns = torch.ops.para_attn
    bm = torch.rand(3, 2, 4, generator=torch.Generator().manual_seed(1)) < 0.6
    bm[..., 0] = True
    bm = bm.to(cuda)
    runs = ns.block_sparse_key_runs(bm, 256)
    keymask = (torch.arange(256, device=cuda) < 200)[None, None, None, :]
    for name, q in queries.items():
        real = ns.attention_forward(q, k, v)
        assert real.stride() == (q.stride() if name != "unaligned_rows" else q.contiguous().stride()), name
        checks = [
            (ns.attention_forward_with_lse.default, (q, k, v), {}),
            (ns.attention_forward_with_lse.default, (q, k, v, None, 0.0, True), {}),
            (ns.attention_forward_with_lse.default, (q, k, v, keymask), {"scale": 0.1}),
            (ns.attention_forward.default, (q, k, v), {}),
            (ns.attention_forward_sparse_kv.default, (q, k, v, keymask.expand(2, 1, 1, 256)), {}),
            (ns.attention_forward_sweep.default, (q, [k[:, :, :128], k[:, :, 128:]], [v[:, :, :128], v[:, :, 128:]]), {}),
            (ns.attention_forward_block_sparse.default, (q, k, v, bm), {}),
            (ns.attention_forward_block_sparse_runs.default, (q, k, v, runs, 3, 2, 4), {}),
        ]
        for op, args, kwargs in checks:
            opcheck(op, args, kwargs, test_utils="test_faketensor")
    opcheck(ns.block_sparse_key_runs.default, (bm, 256), test_utils="test_faketensor")
    opcheck(ns.block_sparse_key_runs.default, (bm[0], 512, 128, 384), test_utils="test_faketensor")
    q = queries["bshd"]
    o1, l1 = ns.attention_forward_with_lse(q, k[:, :, :100], v[:, :, :100])
    o2, l2 = ns.attention_forward_with_lse(q, k[:, :, 100:], v[:, :, 100:])
    opcheck(ns.merge_attention_lse.default, (o1, l1, o2, l2), test_utils="test_faketensor")
    opcheck(ns.merge_attention_lse.default, (o1.float(), l1.unsqueeze(-1), o2, l2, torch.bfloat16), test_utils="test_faketensor")
    acc, acc_lse = torch.zeros(q.shape, dtype=torch.float32, device=cuda), torch.zeros(q.shape[:3], dtype=torch.float32, device=cuda)
    ns.attention_forward_accumulate_(acc, acc_lse, q, k[:, :, :100], v[:, :, :100], True)
    opcheck(ns.attention_forward_accumulate_final.default, (acc, acc_lse, q, k[:, :, 100:], v[:, :, 100:]), test_utils="test_faketensor")
    h = torch.randn(1, 64, 512, device=cuda).bfloat16().transpose(1, 2)  # not contiguous
    opcheck(ns.fbcache_apply_residual.default, (h, h), test_utils="test_faketensor")
    opcheck(ns.fbcache_first_residual_diff.default, (h, h, h), test_utils="test_faketensor")
    opcheck(ns.fbcache_residual_diff.default, (h, h), test_utils="test_faketensor")
    opcheck(ns.taylorseer_derivatives.default, (h, [h, h], 2.0), test_utils="test_faketensor")
    opcheck(ns.taylorseer_value.default, ([h, h], 2, h), test_utils="test_faketensor")


def test_operands_on_another_device_are_refused(cuda):
    """A mask (or key, value) that is not on the query's device raises before anything is launched: the kernels take
    raw pointers, and F.scaled_dot_product_attention, which the reference's ops call, raises a device mismatch
    there as well."""
    q, k, v = (t.to(cuda) for t in inputs.qkv(1, 2, 64, 96, 128, seed=2))
    keep = torch.ones(1, 1, 1, 96, dtype=torch.bool)  # on the CPU
    ns = torch.ops.para_attn
    for op in (ns.attention_forward_with_lse, ns.attention_forward, ns.attention_forward_sparse_kv):
        with pytest.raises(ValueError, match="device"):
            op(q, k, v, keep)
        with pytest.raises(ValueError, match="device"):
            op(q, k, v, keep.float())
    with pytest.raises(ValueError, match="device"):
        ns.attention_forward(q, k.cpu(), v)
    torch.cuda.synchronize()
    assert torch.isfinite(ns.attention_forward(q, k, v, keep.to(cuda)).float()).all()


def test_compiled_on_the_default_backend(cuda):
    """The reference's compiled mode test on torch.compile's default backend (tests/test_interface.py:94-109), with
    the consumer every diffusers processor puts behind SDPA (``.transpose(1, 2).flatten(2, 3)``,
    src/para_attn/context_parallel/diffusers_adapters/mochi.py:242-245) and a pointwise op behind that, on
    [B,S,H,D]-memory operands: the compiler plans the consumer against the fake implementation's strides, so this
    passes only if they are the strides the kernel writes.  Two calls, against eager."""
    B, H, S, D = 2, 3, 264, 128
    x = torch.randn(3, B, S, H * D, generator=torch.Generator().manual_seed(7)).bfloat16().to(cuda)

    def block(x):
        q, k, v = (x[i].view(B, S, H, D).transpose(1, 2) for i in range(3))
        o = F.scaled_dot_product_attention(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False)
        o = o.transpose(1, 2).flatten(2, 3)
        return o * 2 + x[0], o

    with paraattention_amd.UnifiedAttnMode():
        want = block(x)
    assert want[1].shape == (B, S, H * D)
    try:
        compiled = torch.compile(block, fullgraph=True)
        with paraattention_amd.UnifiedAttnMode():
            got = compiled(x)
    except Exception as e:  # only a missing or broken inductor toolchain on the box; wrong strides fail the asserts below
        from torch._dynamo.exc import BackendCompilerFailed
        from torch._inductor.exc import InductorError

        if isinstance(e, (BackendCompilerFailed, InductorError)) and "assert_size_stride" not in str(e):
            pytest.skip(f"torch.compile's default backend cannot build kernels here: {type(e).__name__}: {str(e)[:300]}")
        raise
    for _ in range(2):
        with paraattention_amd.UnifiedAttnMode():
            got = compiled(x)
        assert torch.equal(got[1], want[1])
        torch.testing.assert_close(got[0], want[0], atol=2e-2, rtol=2e-2)  # the pointwise tail may fuse its roundings
    # and the op layer's own ops in one compiled graph
    def split_merge(x):
        q, k, v = (x[i].view(B, S, H, D).transpose(1, 2) for i in range(3))
        o1, l1 = torch.ops.para_attn.attention_forward_with_lse(q, k[:, :, :120], v[:, :, :120])
        o2, l2 = torch.ops.para_attn.attention_forward_with_lse(q, k[:, :, 120:], v[:, :, 120:])
        o, l = torch.ops.para_attn.merge_attention_lse(o1, l1, o2, l2, q.dtype)
        return o.transpose(1, 2).flatten(2, 3), l

    w = split_merge(x)
    g = torch.compile(split_merge, fullgraph=True)(x)
    assert torch.equal(g[0], w[0]) and torch.equal(g[1], w[1])


def test_compiled_ops_fullgraph(cuda):
    """attention + merge custom ops inside one compiled graph (src/para_attn/ops/__init__.py registers them for this)."""
    q, k, v = (t.to(cuda) for t in inputs.qkv(1, 2, 300, 200, 128, seed=5))

    def fn(q, k, v):
        o1, l1 = torch.ops.para_attn.attention_forward_with_lse(q, k[:, :, :120], v[:, :, :120])
        o2, l2 = torch.ops.para_attn.attention_forward_with_lse(q, k[:, :, 120:], v[:, :, 120:])
        return torch.ops.para_attn.merge_attention_lse(o1, l1, o2, l2, q.dtype)

    want = fn(q, k, v)
    got = torch.compile(fn, fullgraph=True, backend="aot_eager")(q, k, v)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    full, lse = torch.ops.para_attn.attention_forward_with_lse(q, k, v)
    assert (got[0].float() - full.float()).abs().max().item() <= 2e-2 and (got[1] - lse).abs().max().item() <= 1e-3


def test_in_batch_ring_and_ulysses_on_one_rank(cuda):
    """para_attn_interface.py:88-117, 200-276: on one rank ring and ulysses attention are plain attention, and
    in-batch attention lets every batch element attend the keys of all of them."""
    B, H, Sq, Skv, D = 3, 2, 70, 90, 128
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=8)
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    direct = torch.ops.para_attn.attention_forward(qd, kd, vd)
    assert torch.equal(paraattention_amd.ring_attn_func(qd, kd, vd), direct)
    assert torch.equal(paraattention_amd.ulysses_attn_func(qd, kd, vd), direct)
    with paraattention_amd.RingAttnMode():
        assert torch.equal(F.scaled_dot_product_attention(qd, kd, vd), direct)
    with paraattention_amd.UlyssesAttnMode(skip_small_kv=True):
        assert torch.equal(F.scaled_dot_product_attention(qd, kd, vd), direct)
    # in-batch: queries of every element against the concatenated keys of all elements
    kf = k.permute(1, 0, 2, 3).reshape(1, H, B * Skv, D).float().numpy()
    vf = v.permute(1, 0, 2, 3).reshape(1, H, B * Skv, D).float().numpy()
    qf = q.permute(1, 0, 2, 3).reshape(1, H, B * Sq, D).float().numpy()
    ref, _ = oattn.sdpa_lse_f64(qf, kf, vf)
    ref = ref.reshape(H, B, Sq, D).transpose(1, 0, 2, 3)
    out = paraattention_amd.in_batch_attn_func(qd, kd, vd)
    assert out.shape == (B, H, Sq, D)
    np.testing.assert_allclose(out.float().cpu().numpy(), ref, atol=2e-2, rtol=2e-2)
    with paraattention_amd.InBatchAttnMode():
        out2 = F.scaled_dot_product_attention(qd, kd, vd)
    assert torch.equal(out2, out)
    # [B,S,H,D] memory: the fold is a view, no copy of q, k or v is made
    qs, ks, vs = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (qd, kd, vd))
    folded = qs.permute(1, 0, 2, 3).reshape(1, H, B * Sq, D)
    assert folded.data_ptr() == qs.data_ptr()
    assert torch.equal(paraattention_amd.in_batch_attn_func(qs, ks, vs), out)


@pytest.mark.parametrize("is_causal", [False, True])
def test_torch_ring_loop_calls_the_op(cuda, tmp_path, is_causal):
    """torch's own ring loop with this package's op, the call the reference makes
    (src/para_attn/para_attn_interface.py:164-197: _templated_ring_attention(mesh, seq_dim,
    para_attn_ops.attention_forward_with_lse, q, k, v, attn_mask=, dropout_p=, is_causal=, scale=) with load
    balancing off and fp32 merging).  On a group of one rank the loop issues no collective: it calls the op once
    as op(q, k, v, is_causal=..., **kwargs), unpacks (out, lse, *rest), passes both through _SDPAMerger and casts
    back, so the result must be the op's own, bit for bit."""
    import torch.distributed as dist
    from torch.distributed.tensor.experimental._context_parallel import _attention as tra

    # a one-rank default group: this test's own, or the one an earlier test of this process left behind
    mine = not dist.is_initialized()
    if mine:
        dist.init_process_group("gloo", store=dist.FileStore(str(tmp_path / "rendezvous"), 1), rank=0, world_size=1)
    assert dist.get_world_size() == 1
    saved = (tra._cp_options.enable_load_balance, tra._cp_options.convert_to_f32, tra._cp_options.rotate_method)
    try:
        tra._cp_options.enable_load_balance = False
        tra._cp_options.convert_to_f32 = True
        tra._cp_options.rotate_method = tra._RotateMethod.ALL_TO_ALL
        q, k, v = inputs.qkv(1, 3, 300, 300, 128, seed=21)
        qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
        out, lse = tra._templated_ring_attention(dist.group.WORLD, 2, torch.ops.para_attn.attention_forward_with_lse,
                                                 qd, kd, vd, attn_mask=None, dropout_p=0.0, is_causal=is_causal, scale=None)
        want_out, want_lse = torch.ops.para_attn.attention_forward_with_lse(qd, kd, vd, is_causal=is_causal)
        assert out.dtype == torch.bfloat16 and torch.equal(out, want_out)
        assert lse.dtype == torch.float32 and torch.equal(lse.reshape(want_lse.shape), want_lse)
        keep = oattn.causal_keep(300, 300) if is_causal else None
        ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, keep)
        np.testing.assert_allclose(out.float().cpu().numpy(), ref_out, atol=2e-2, rtol=2e-2)
        np.testing.assert_allclose(lse.reshape(want_lse.shape).cpu().numpy(), ref_lse, atol=1e-3)
    finally:
        (tra._cp_options.enable_load_balance, tra._cp_options.convert_to_f32, tra._cp_options.rotate_method) = saved
        if mine:
            dist.destroy_process_group()
