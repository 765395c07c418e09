"""Parity of the HIP attention kernel (through torch.ops.para_attn.* -> C ABI) with the oracle.

Tolerances are the ones the task states: bf16/fp16 output atol 2e-2 / rtol 2e-2, fp32 LSE 1e-3.
"""
import math

import numpy as np
import pytest
import torch

import paraattention_amd  # noqa: F401
from oracle import attention as oattn
from oracle import inputs

pytestmark = pytest.mark.gpu

OUT_ATOL = OUT_RTOL = 2e-2
LSE_ATOL = 1e-3


def _check(out, lse, ref_out, ref_lse, what=""):
    out = out.float().cpu().numpy().astype(np.float64)
    ref_out = np.asarray(ref_out, dtype=np.float64)
    err = np.abs(out - ref_out)
    tol = OUT_ATOL + OUT_RTOL * np.abs(ref_out)
    assert (err <= tol).all(), f"{what}: out max err {err.max():.4g} (worst excess {(err - tol).max():.4g})"
    if lse is not None:
        lse = lse.cpu().numpy().astype(np.float64)
        ref_lse = np.asarray(ref_lse, dtype=np.float64)
        with np.errstate(invalid="ignore"):
            lerr = np.where(lse == ref_lse, 0.0, np.abs(lse - ref_lse))  # -inf against -inf (a row that keeps nothing) is exact
        assert lse.dtype == np.float64 and (lerr <= LSE_ATOL).all(), f"{what}: lse max err {lerr.max():.4g}"


# ragged sizes the reference's shapes hit: 119056 = 930*128 + 16, 14882 = 116*128 + 34, 32760 = 255*128 + 120
SMALL = [
    (1, 1, 1, 1), (1, 2, 15, 17), (2, 3, 16, 16), (1, 2, 17, 34), (1, 1, 33, 63), (1, 2, 64, 64), (1, 1, 65, 65),
    (1, 2, 120, 129), (1, 1, 128, 128), (1, 3, 129, 120), (2, 2, 257, 300), (1, 2, 300, 1000), (1, 1, 1000, 77),
]


@pytest.mark.parametrize("B,H,Sq,Skv", SMALL)
@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_small_vs_f64(cuda, B, H, Sq, Skv, D, dtype):
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=Sq * 1000 + Skv, dtype=dtype)
    ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy())
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k.to(cuda), v.to(cuda))
    assert out.dtype == dtype and out.shape == (B, H, Sq, D)
    assert lse.dtype == torch.float32 and lse.shape == (B, H, Sq)  # the reference's own assertions, tests/ops/test_ops.py:63-64
    _check(out, lse, ref_out, ref_lse, f"{(B, H, Sq, Skv, D, dtype)}")
    out2 = torch.ops.para_attn.attention_forward(q.to(cuda), k.to(cuda), v.to(cuda))
    assert torch.equal(out2, out)


@pytest.mark.parametrize("scale", [0.05, 1.0, None])
def test_scale_and_large_logits(cuda, scale):
    # scaled logits up to a few hundred: exercises the running-maximum update
    q, k, v = inputs.qkv(1, 2, 200, 500, 128, seed=7)
    q = q * 4
    ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), scale)
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k.to(cuda), v.to(cuda), scale=scale)
    _check(out, lse, ref_out, ref_lse)


def test_increasing_maximum(cuda):
    # keys ordered so that every tile raises the row maximum: the rescale path runs on each tile
    D, Skv = 128, 640
    g = torch.Generator().manual_seed(3)
    q = torch.ones(1, 1, 64, D) * 0.5
    k = torch.randn(1, 1, Skv, D, generator=g) * 0.1 + torch.linspace(-2, 2, Skv)[None, None, :, None]
    v = torch.randn(1, 1, Skv, D, generator=g)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), 1.0)
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k.to(cuda), v.to(cuda), scale=1.0)
    _check(out, lse, ref_out, ref_lse)


def test_closed_forms(cuda):
    D = 128
    q, k, v = inputs.qkv(1, 2, 77, 333, D, seed=11)
    # K = 0: uniform weights -> out = mean(V), lse = ln(Skv)
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), torch.zeros_like(k).to(cuda), v.to(cuda))
    assert torch.allclose(lse.cpu(), torch.full_like(lse.cpu(), math.log(333)), atol=1e-4)
    assert torch.allclose(out.float().cpu(), v.float().mean(2, keepdim=True).expand(-1, -1, 77, -1), atol=2e-2, rtol=2e-2)
    # V constant along keys: out = that constant, exactly representable
    vc = torch.full_like(v, 0.75)
    out, _ = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k.to(cuda), vc.to(cuda))
    assert torch.allclose(out.float().cpu(), vc.float()[:, :, :1].expand(-1, -1, 77, -1), atol=4e-3)


def test_noncontiguous_layouts(cuda):
    # diffusers hands SDPA [B,S,H,D] memory viewed as [B,H,S,D]
    B, H, S, D = 2, 3, 200, 128
    q, k, v = inputs.qkv(B, H, S, S, D, seed=5)
    ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy())
    qt, kt, vt = (t.to(cuda).transpose(1, 2).contiguous().transpose(1, 2) for t in (q, k, v))
    assert not qt.is_contiguous()
    out, lse = torch.ops.para_attn.attention_forward_with_lse(qt, kt, vt)
    assert out.stride() == qt.stride()  # output keeps the query's memory layout
    _check(out, lse, ref_out, ref_lse)
    # sliced views (non-dense strides)
    big = torch.randn(B, H, S + 8, D + 64, generator=torch.Generator().manual_seed(1)).bfloat16()
    qs = big[:, :, 3 : 3 + S, :D]
    ref_out, ref_lse = oattn.sdpa_lse_f64(qs.float().numpy(), k.float().numpy(), v.float().numpy())
    out, lse = torch.ops.para_attn.attention_forward_with_lse(big.to(cuda)[:, :, 3 : 3 + S, :D], k.to(cuda), v.to(cuda))
    _check(out, lse, ref_out, ref_lse)


def test_permutation_invariance(cuda):
    q, k, v = inputs.qkv(1, 2, 130, 515, 128, seed=9)
    perm = torch.randperm(515, generator=torch.Generator().manual_seed(0))
    o1, l1 = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k.to(cuda), v.to(cuda))
    o2, l2 = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k[:, :, perm].to(cuda), v[:, :, perm].to(cuda))
    assert torch.allclose(l1, l2, atol=1e-4)
    assert torch.allclose(o1.float(), o2.float(), atol=2e-2, rtol=2e-2)


def test_flux_shape_vs_torch_cpu(cuda):
    # the FLUX-dev joint-attention shape: B1 H24 S4608 D128 against torch's CPU SDPA on identical bits
    q, k, v = inputs.qkv(1, 24, 4608, 4608, 128, seed=0)
    ref_out, ref_lse = oattn.sdpa_lse_torch_cpu(q, k, v)
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k.to(cuda), v.to(cuda))
    _check(out, lse, ref_out.float().numpy(), ref_lse.numpy(), "flux")


def test_hunyuan_shape_sampled_rows(cuda):
    # the 119k-token HunyuanVideo head-share shape at full size on the GPU; the oracle checks sampled query rows of each head
    B, H, S, D = 1, 3, 119056, 128
    q, k, v = inputs.qkv(B, H, S, S, D, seed=0, rms_norm_qk=True)
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k.to(cuda), v.to(cuda))
    rows = torch.cat([torch.arange(0, 40), torch.arange(S - 40, S), torch.randint(0, S, (176,), generator=torch.Generator().manual_seed(1))])
    ref_out, ref_lse = oattn.sdpa_lse_torch_cpu(q[:, :, rows], k, v)
    _check(out[:, :, rows.to(cuda)], lse[:, :, rows.to(cuda)], ref_out.float().numpy(), ref_lse.numpy(), "hunyuan")
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()


def test_hunyuan_shape_every_row_by_closed_forms(cuda):
    """Properties that hold whatever the size, checked on every query row of the 119k-token shape (the sampled-row
    test above leaves most rows to chance): with zero keys every score is 0, so LSE = ln(Skv) and out = the mean
    of V over the keys; with V constant along the keys, out is that constant whatever the scores; and out is
    linear in V at fixed q, k while LSE does not depend on V."""
    B, H, S, D = 1, 3, 119056, 128
    q, k, v = inputs.qkv(B, H, S, S, D, seed=5, rms_norm_qk=True)
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    op = torch.ops.para_attn.attention_forward_with_lse
    # zero keys
    out, lse = op(qd, torch.zeros_like(kd), vd)
    assert (lse - np.log(S)).abs().max().item() <= 1e-3
    mean_v = vd.float().mean(dim=2, keepdim=True)  # [B,H,1,D]
    assert (out.float() - mean_v).abs().max().item() <= 2e-2
    # V constant along the keys: row d of every key holds c[d]
    c = torch.linspace(-2.0, 2.0, D).bfloat16().to(cuda)
    out_c, lse_c = op(qd, kd, c.expand(B, H, S, D).contiguous())
    assert (out_c.float() - c.float()).abs().max().item() <= 2e-2
    # linearity in V; LSE independent of V
    out1, lse1 = op(qd, kd, vd)
    v2 = torch.roll(vd, 7, dims=2)
    out2, lse2 = op(qd, kd, v2)
    out3, lse3 = op(qd, kd, (0.5 * vd.float() - 0.25 * v2.float()).bfloat16())
    assert torch.equal(lse1, lse2) and torch.equal(lse1, lse3) and torch.equal(lse1, lse_c)
    # three bf16 roundings of outputs that are O(0.01) here; the bound is the parity tolerance itself
    err = (out3.float() - (0.5 * out1.float() - 0.25 * out2.float())).abs()
    assert (err <= 2e-2 + 2e-2 * out3.float().abs()).all(), err.max().item()


def test_wan_cross_attention_shape(cuda):
    # the Wan 2.1 cross-attention leg at full size: 32760 queries x 40 heads against 512 text keys, every row
    # against torch's CPU SDPA on identical bits
    q, k, v = inputs.qkv(1, 40, 32760, 512, 128, seed=2)
    ref_out, ref_lse = oattn.sdpa_lse_torch_cpu(q, k, v)
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k.to(cuda), v.to(cuda))
    _check(out, lse, ref_out.float().numpy(), ref_lse.numpy(), "wan-cross")


def test_wan_self_attention_shape(cuda):
    """The Wan 2.1 self-attention leg at full size, B1 H40 S32760 D128 (32760 = 255*128 + 120: a ragged last query
    tile and a ragged last key tile).  torch's CPU SDPA checks sampled query rows of three heads (first, a middle
    one, last; the first and last rows of the sequence among them); closed forms that hold at any size check
    every row of every head: zero keys give LSE = ln(Skv) and out = mean of V, V constant along the keys gives
    that constant, out is linear in V and LSE does not depend on V."""
    B, H, S, D = 1, 40, 32760, 128
    q, k, v = inputs.qkv(B, H, S, S, D, seed=4)
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    op = torch.ops.para_attn.attention_forward_with_lse
    out, lse = op(qd, kd, vd)
    assert out.shape == (B, H, S, D) and lse.shape == (B, H, S)
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    heads = [0, 17, 39]
    rows = torch.cat([torch.arange(0, 40), torch.arange(S - 130, S), torch.randint(0, S, (86,), generator=torch.Generator().manual_seed(1))])
    ref_out, ref_lse = oattn.sdpa_lse_torch_cpu(q[:, heads][:, :, rows].contiguous(), k[:, heads].contiguous(), v[:, heads].contiguous())
    got_out, got_lse = out[:, heads][:, :, rows.to(cuda)], lse[:, heads][:, :, rows.to(cuda)]
    _check(got_out, got_lse, ref_out.float().numpy(), ref_lse.numpy(), "wan-self")
    # attention_forward is the same launch without the LSE
    assert torch.equal(torch.ops.para_attn.attention_forward(qd, kd, vd), out)
    # zero keys
    out0, lse0 = op(qd, torch.zeros_like(kd), vd)
    assert (lse0 - np.log(S)).abs().max().item() <= 1e-3
    assert (out0.float() - vd.float().mean(dim=2, keepdim=True)).abs().max().item() <= 2e-2
    del out0, lse0
    # V constant along the keys
    c = torch.linspace(-2.0, 2.0, D).bfloat16().to(cuda)
    out_c, lse_c = op(qd, kd, c.expand(B, H, S, D).contiguous())
    assert (out_c.float() - c.float()).abs().max().item() <= 2e-2
    assert torch.equal(lse_c, lse)
    del out_c, lse_c
    # linearity in V at fixed q, k
    v2 = torch.roll(vd, 5, dims=2)
    out2, lse2 = op(qd, kd, v2)
    out3, lse3 = op(qd, kd, (0.5 * vd.float() - 0.25 * v2.float()).bfloat16())
    assert torch.equal(lse2, lse) and torch.equal(lse3, lse)
    err = (out3.float() - (0.5 * out.float() - 0.25 * out2.float())).abs()
    assert (err <= 2e-2 + 2e-2 * out3.float().abs()).all(), err.max().item()


def test_key_mask_and_sparse_kv(cuda):
    B, H, Sq, Skv, D = 2, 2, 150, 333, 128
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=21)
    # prefix mask (valid text length per batch element) and a scattered mask
    lens = [333, 201]
    prefix = torch.arange(Skv)[None, :] < torch.tensor(lens)[:, None]
    scattered = torch.rand(B, Skv, generator=torch.Generator().manual_seed(4)) < 0.6
    for m in (prefix, scattered):
        keep = m[:, None, None, :].numpy()
        ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, keep)
        mask4 = m[:, None, None, :].expand(B, 1, Sq, Skv).to(cuda)
        out = torch.ops.para_attn.attention_forward_sparse_kv(q.to(cuda), k.to(cuda), v.to(cuda), mask4)
        _check(out, None, ref_out, None, "sparse_kv")
        out, lse = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k.to(cuda), v.to(cuda), m[:, None, None, :].to(cuda))
        _check(out, lse, ref_out, ref_lse, "key mask")


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_general_masks_vs_f64(cuda, D, dtype):
    """attn_mask as the reference's dense ops take it (src/para_attn/ops/__init__.py:78-87, 215-223): boolean or
    additive, any shape that broadcasts to [B,H,Sq,Skv] with torch's alignment of trailing dimensions.  Rows that
    keep nothing give out = 0, lse = -inf (the oracle's convention); tiles in which a row keeps nothing at all
    precede kept ones.  Every case against the fp64 oracle with the mask expanded."""
    B, H, Sq, Skv = 2, 3, 150, 333
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=41, dtype=dtype)
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    g = torch.Generator().manual_seed(8)
    op = torch.ops.para_attn.attention_forward_with_lse
    qn, kn, vn = q.float().numpy(), k.float().numpy(), v.float().numpy()
    shapes = [(B, H, Sq, Skv), (1, 1, Sq, Skv), (Sq, Skv), (B, 1, Sq, Skv), (H, 1, Skv), (B, 1, 1, Skv), (Skv,), (1, H, Sq, 1)]
    for shape in shapes:
        keep = torch.rand(shape, generator=g) < 0.4
        if len(shape) >= 2 and shape[-2] == Sq and shape[-1] == Skv:
            keep[..., 3, :] = False        # a row that keeps nothing
            keep[..., 5, :200] = False     # a row whose first three tiles are empty
        ref_out, ref_lse = oattn.sdpa_lse_f64(qn, kn, vn, None, np.broadcast_to(keep.numpy(), (B, H, Sq, Skv)))
        out, lse = op(qd, kd, vd, keep.to(cuda))
        _check(out, lse, ref_out, ref_lse, f"bool mask {shape}")
        assert torch.equal(torch.ops.para_attn.attention_forward(qd, kd, vd, keep.to(cuda)), out)
        # the same mask as an additive one (0 / -inf), in fp32 and in the activation type
        for mdt in (torch.float32, dtype):
            bias = torch.zeros(keep.shape, dtype=mdt).masked_fill_(~keep, float("-inf"))
            out_a, lse_a = op(qd, kd, vd, bias.to(cuda))
            _check(out_a, lse_a, ref_out, ref_lse, f"additive -inf mask {shape} {mdt}")
    # a finite bias: scores + bias before the softmax
    bias = torch.randn(B, 1, Sq, Skv, generator=g)
    s = np.einsum("bhqd,bhkd->bhqk", qn.astype(np.float64), kn.astype(np.float64)) / np.sqrt(D) + bias.numpy().astype(np.float64)
    m = s.max(-1, keepdims=True)
    pw = np.exp(s - m)
    ref_out = (pw @ vn.astype(np.float64)) / pw.sum(-1, keepdims=True)
    ref_lse = (m + np.log(pw.sum(-1, keepdims=True)))[..., 0]
    out, lse = op(qd, kd, vd, bias.to(cuda))
    _check(out, lse, ref_out, ref_lse, "finite additive bias")
    # torch's own CPU SDPA agrees on the same additive mask (independent of the oracle's formula)
    t_out, t_lse = oattn.sdpa_lse_torch_cpu(q, k, v, attn_mask=bias.to(dtype).expand(B, H, Sq, Skv).contiguous())
    out_b, lse_b = op(qd, kd, vd, bias.to(dtype).to(cuda))
    _check(out_b, lse_b, t_out.float().numpy(), t_lse.numpy(), "finite additive bias, torch CPU")
    with pytest.raises(ValueError):
        op(qd, kd, vd, torch.ones(B, Skv, dtype=torch.bool, device=cuda))  # [2,333] is not [Sq,Skv]


def test_key_masks_take_the_fast_kernels_when_prefixes(cuda, tuning):
    """A key-only boolean mask is scanned on the device: prefixes run the dense kernels with per-batch key counts
    (here with the key-split tail and the score bound in play), anything else the per-score kernel; both give the
    oracle's result and neither reads the mask on the host."""
    tuning("bound", 1)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    B, H, D = 2, 4, 128
    Sq, Skv = (cus // (B * H) + 3) * 256 - 19, 64 * 40 + 37
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=43)
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    lens = torch.tensor([Skv - 3, 900])
    prefix = torch.arange(Skv)[None, :] < lens[:, None]
    scattered = prefix.clone()
    scattered[1, 10] = False
    scattered[1, 2000] = True
    rows = torch.cat([torch.arange(0, 30), torch.arange(Sq - 300, Sq, 7)])
    for name, m in (("prefix", prefix), ("scattered", scattered)):
        ref_out, ref_lse = oattn.sdpa_lse_f64(q[:, :, rows].float().numpy(), k.float().numpy(), v.float().numpy(), None, m[:, None, None, :].numpy())
        out, lse = torch.ops.para_attn.attention_forward_with_lse(qd, kd, vd, m[:, None, None, :].to(cuda))
        _check(out[:, :, rows.to(cuda)], lse[:, :, rows.to(cuda)], ref_out, ref_lse, name)
        assert torch.isfinite(lse).all()


@pytest.mark.parametrize("rounds", [-1, 6])
def test_long_launches_with_nearly_full_key_masks(cuda, rounds, tuning):
    """A longer launch (512 key-tile steps per workgroup and more) whose key mask is a prefix that keeps at least 7/8 of
    the keys in every batch element -- a padded text prompt at the end of a video's tokens -- goes to the
    resident-workgroup kernel with the counts as per-batch key limits: pieces end at their batch element's last key,
    ranges of the tail that lie beyond it come out empty (with 6 rounds the last ranges are 32 tiles long and one
    batch element drops 60).  A prefix that keeps less goes to the kernel with one workgroup per query tile.  A mask
    with holes -- one key missing, half of the keys at random, or the text padding of eight ranks' shards inside the
    gathered sequence, as the reference's sequence-parallel HunyuanVideo adapter builds it
    (context_parallel/diffusers_adapters/hunyuan_video.py:86-100) -- has its kept K and V rows gathered into dense
    copies on which the same two kernels run.  Which launches run is decided on the device.  Sampled rows of three
    heads against the fp64 oracle; the nearly full cases also against the same call with the resident-workgroup kernel
    switched off, and bit for bit against a second call; attention_forward_sparse_kv gives the same output."""
    tuning("stream_dyn", rounds)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    B, H, D = 2, 8, 128
    Sq, Skv = cus // 8 * 256 - 77, 64 * 520 + 13  # 2 x 8 x 32 pieces of 521 tiles: 1042 steps per workgroup
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=47)
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    op = torch.ops.para_attn.attention_forward_with_lse
    heads = [0, 3, 7]
    rows = torch.cat([torch.arange(0, 150), torch.randint(0, Sq, (150,), generator=torch.Generator().manual_seed(2)), torch.arange(Sq - 150, Sq)])
    cases = [("nearly full", [Skv - 3, Skv - 64 * 60 - 5]),  # the second batch element is the one whose pieces make up the tail ("full", [Skv, Skv]), ("nearly full, whole tiles", [Skv - 13, Skv - 13 - 128]),
             ("half", [Skv - 3, Skv // 2]), ("nearly full, one hole", None), ("random half", None), ("nearly full, interleaved padding", None)]
    for name, lens in cases:
        if name == "nearly full, one hole":
            m = torch.arange(Skv)[None, :] < torch.tensor([Skv - 3, Skv - 70])[:, None]
            m[1, 10] = False
        elif name == "random half":
            m = torch.rand(B, Skv, generator=torch.Generator().manual_seed(9)) < 0.5
        elif name == "nearly full, interleaved padding":
            shard, text = Skv // 8, 32  # per rank: latent tokens, then 32 text tokens; 100 / 37 of the 256 are valid
            pos = torch.arange(Skv)
            rank, off = pos // shard, pos % shard
            text_index = rank * text + (off - (shard - text))
            m = torch.stack([(off < shard - text) | (text_index < valid) | (pos >= 8 * shard) for valid in (100, 37)])
        else:
            m = torch.arange(Skv)[None, :] < torch.tensor(lens)[:, None]
        mask = m[:, None, None, :].to(cuda)
        ref_out, ref_lse = oattn.sdpa_lse_f64(q[:, heads][:, :, rows].float().numpy(), k[:, heads].float().numpy(), v[:, heads].float().numpy(), None, m[:, None, None, :].numpy())
        out, lse = op(qd, kd, vd, mask)
        _check(out[:, heads][:, :, rows.to(cuda)], lse[:, heads][:, :, rows.to(cuda)], ref_out, ref_lse, f"{name}, rounds={rounds}")
        assert torch.isfinite(lse).all() and torch.isfinite(out.float()).all()
        out2, lse2 = op(qd, kd, vd, mask)
        assert torch.equal(out2, out) and torch.equal(lse2, lse), name
        assert torch.equal(torch.ops.para_attn.attention_forward_sparse_kv(qd, kd, vd, mask.expand(B, 1, Sq, Skv)), out), name
        if name.startswith("nearly"):
            tuning("stream", 0)
            out0, lse0 = op(qd, kd, vd, mask)
            tuning("stream", -1)
            assert (out.float() - out0.float()).abs().max().item() <= 2e-2 and (lse - lse0).abs().max().item() <= 1e-4
            if rounds > 0:  # (whole pieces come out bit-equal from both kernels: the same tiles in the same order)
                assert not torch.equal(out0, out), "meant to run two different kernels"


@pytest.mark.parametrize("Sq,Skv", [(150, 333), (9000, 9011)])
def test_key_masks_that_keep_nothing_in_one_batch_element(cuda, Sq, Skv):
    """A key mask that drops every key of one batch element (out = 0, LSE = -inf there, the oracle's convention), as a
    prefix of length 0 and, with a hole in the other element, as a mask with holes; at a small size (the per-score
    kernel for the mask with holes) and at one where the kept keys are gathered."""
    B, H, D = 2, 8, 128
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=61)
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    rows = torch.cat([torch.arange(0, 60), torch.arange(Sq - 60, Sq)])
    for holes in (False, True):
        m = torch.ones(B, Skv, dtype=torch.bool)
        m[0] = False
        if holes:
            m[1, 7] = False
        ref_out, ref_lse = oattn.sdpa_lse_f64(q[:, :, rows].float().numpy(), k.float().numpy(), v.float().numpy(), None, m[:, None, None, :].numpy())
        out, lse = torch.ops.para_attn.attention_forward_with_lse(qd, kd, vd, m[:, None, None, :].to(cuda))
        _check(out[:, :, rows.to(cuda)], lse[:, :, rows.to(cuda)], ref_out, ref_lse, f"nothing kept in element 0, holes={holes}")
        assert (out[0] == 0).all() and torch.isinf(lse[0]).all() and (lse[0] < 0).all()
        assert torch.isfinite(out[1].float()).all() and torch.isfinite(lse[1]).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_key_masks_with_holes_head_dim_64(cuda, dtype):
    """head_dim 64, large enough (3e11 flop) for the kept keys of a mask with holes to be gathered: a random mask that
    keeps 70 % and one that drops three keys, two batch elements, K in [B,S,H,D] memory; every head's sampled rows
    against the fp64 oracle."""
    B, H, Sq, Skv, D = 2, 6, 10000, 10007, 64
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=53, dtype=dtype)
    qd, vd = q.to(cuda), v.to(cuda)
    kd = k.to(cuda).transpose(1, 2).contiguous().transpose(1, 2)
    rows = torch.cat([torch.arange(0, 100), torch.arange(Sq - 100, Sq)])
    g = torch.Generator().manual_seed(6)
    for name in ("random", "three holes"):
        m = torch.rand(B, Skv, generator=g) < 0.7 if name == "random" else torch.ones(B, Skv, dtype=torch.bool)
        m[0, 5] = m[1, 4000] = m[1, Skv - 1] = False
        ref_out, ref_lse = oattn.sdpa_lse_f64(q[:, :, rows].float().numpy(), k.float().numpy(), v.float().numpy(), None, m[:, None, None, :].numpy())
        out, lse = torch.ops.para_attn.attention_forward_with_lse(qd, kd, vd, m[:, None, None, :].to(cuda))
        _check(out[:, :, rows.to(cuda)], lse[:, :, rows.to(cuda)], ref_out, ref_lse, f"head_dim 64, {name}, {dtype}")
        assert torch.isfinite(out.float()).all()


@pytest.mark.parametrize("D", [128, 64])
def test_empty_inputs(cuda, D):
    """No keys at all (Skv = 0, or a batch element whose mask keeps nothing): out = 0 and lse = -inf, what the
    softmax over an empty set sums to; no queries: empty outputs; all without touching memory out of bounds."""
    q, k, v = (t.to(cuda) for t in inputs.qkv(2, 2, 70, 50, D, seed=2))
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q, k[:, :, :0], v[:, :, :0])
    assert out.shape == q.shape and (out == 0).all() and torch.isneginf(lse).all()
    keep = torch.zeros(2, 1, 1, 50, dtype=torch.bool, device=cuda)
    keep[0] = True
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q, k, v, keep)
    ref_out, ref_lse = oattn.sdpa_lse_f64(q[:1].float().cpu().numpy(), k[:1].float().cpu().numpy(), v[:1].float().cpu().numpy())
    _check(out[:1], lse[:1], ref_out, ref_lse, "kept batch element")
    assert (out[1] == 0).all() and torch.isneginf(lse[1]).all()
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q[:, :, :0], k, v)
    assert out.shape == (2, 2, 0, D) and lse.shape == (2, 2, 0)


@pytest.mark.parametrize("env", [{"no_pipe": 1}, {"bm": 256}])
def test_alternative_kernels(cuda, env, tuning):
    """The kernels without 32-bit offset limits (taken when K or V spans 4 GiB or more) and the 8-wavefront
    workgroup variants compute the same thing as the default kernels, at head_dim 128 and 64."""
    cases = [(1, 2, 300, 434, 128), (2, 1, 129, 1000, 128), (1, 1, 64, 64, 128), (1, 3, 1000, 77, 128),
             (1, 2, 300, 434, 64), (2, 1, 129, 1000, 64), (1, 3, 1000, 77, 64)]
    for B, H, Sq, Skv, D in cases:
        q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=Sq + Skv)
        ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy())
        for name, val in env.items():
            tuning(name, val)
        out, lse = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k.to(cuda), v.to(cuda))
        for name in env:
            tuning(name, 0)
        _check(out, lse, ref_out, ref_lse, f"{env} {(B, H, Sq, Skv)}")


@pytest.mark.parametrize("bm", ["128", "256"])
def test_key_split_tail(cuda, bm, tuning):
    """Grids a little over a whole number of rounds: the query tiles of the last round are computed in key
    shares (fp32 partials in a workspace) and merged.  Checked against the oracle, against the unsplit launch,
    with per-batch key counts that leave some shares empty, and with a strided output."""
    from paraattention_amd import _lib

    lib = _lib.load()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    rows = int(bm)
    slots = cus * (2 if bm == "128" else 1)
    B, H, D = 2, 4, 128
    tiles_per_head = slots // (B * H) + 5   # 40 tiles over a whole round
    Sq = tiles_per_head * rows - 19          # ragged last tile
    Skv = 64 * 40 + 37
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=77)
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    tuning("bm", int(bm))
    need = lib.pa_attn_fwd_workspace_bytes(B, H, Sq, Skv, D, _lib.strides3(kd), _lib.strides3(vd))
    assert need > 0, "this shape is meant to take the key-split path"
    ref_out, ref_lse = oattn.sdpa_lse_torch_cpu(q, k, v)
    out, lse = torch.ops.para_attn.attention_forward_with_lse(qd, kd, vd)
    _check(out, lse, ref_out.float().numpy(), ref_lse.numpy(), f"split bm={bm}")
    tuning("no_split", 1)
    # no partials any more (what remains, if the score bound is asked for at this size, is its 8 KB)
    assert lib.pa_attn_fwd_workspace_bytes(B, H, Sq, Skv, D, _lib.strides3(kd), _lib.strides3(vd)) < 16384
    out1, lse1 = torch.ops.para_attn.attention_forward_with_lse(qd, kd, vd)
    tuning("no_split", 0)
    assert (out.float() - out1.float()).abs().max().item() <= 2e-2
    assert (lse - lse1).abs().max().item() <= 1e-4
    # a workspace that is too short is not an error: the launch is the unsplit one
    import ctypes

    out3, lse3 = torch.empty_like(out), torch.empty_like(lse)
    short = torch.empty(64, dtype=torch.uint8, device=cuda)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    rc = lib.pa_attn_fwd_lse_ws(vp(qd), vp(kd), vp(vd), vp(out3), vp(lse3), 0, B, H, Sq, Skv, D, _lib.strides3(qd),
                                _lib.strides3(kd), _lib.strides3(vd), _lib.strides3(out3), 1.0 / math.sqrt(D), None, 0,
                                vp(short), short.numel(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    # (not bit-equal when the launch above ran without a running maximum: the short workspace has no room for the bound)
    assert (out3.float() - out1.float()).abs().max().item() <= 2e-2 and (lse3 - lse1).abs().max().item() <= 1e-4
    # per-batch key counts: batch 1 keeps 40 keys, so all but one of its shares are empty
    lens = torch.tensor([Skv - 3, 40])
    keep = torch.arange(Skv)[None, :] < lens[:, None]
    ref_out, ref_lse = oattn.sdpa_lse_f64(q[:, :1, -300:].float().numpy(), k[:, :1].float().numpy(), v[:, :1].float().numpy(),
                                          None, keep[:, None, None, :].numpy())
    out, lse = torch.ops.para_attn.attention_forward_with_lse(qd, kd, vd, keep[:, None, None, :].to(cuda))
    _check(out[:, :1, -300:], lse[:, :1, -300:], ref_out, ref_lse, f"split bm={bm} key counts")
    # [B,S,H,D] memory for q and the output
    qs = qd.transpose(1, 2).contiguous().transpose(1, 2)
    out2, lse2 = torch.ops.para_attn.attention_forward_with_lse(qs, kd, vd, keep[:, None, None, :].to(cuda))
    assert torch.equal(out2, out) and torch.equal(lse2, lse)


@pytest.mark.parametrize("even", [-1, 0, 1])
@pytest.mark.parametrize("bound", [0, 1])
@pytest.mark.parametrize("wave_rows", [32, 64])
def test_resident_workgroup_kernel(cuda, even, bound, wave_rows, tuning):
    """The kernel whose workgroups stay resident and walk a list of pieces as one stream of key tiles, forced on
    for every shape here: fewer pieces than compute units (every piece cut into ranges), a few pieces more than a
    whole number of rounds (whole pieces, then a tail cut evenly or into shares that begin at the same keys),
    pieces of one and two key tiles (a new piece's Q and output on every iteration), ragged query and key ends,
    strided memory, both score-bound variants.  Against the fp64 oracle, and against the kernel with one
    workgroup per piece."""
    tuning("stream", 1)
    tuning("stream_even", even)
    tuning("bound", bound)
    tuning("wave_rows", wave_rows)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    op = torch.ops.para_attn.attention_forward_with_lse
    shapes = [(1, 2, 300, 434), (2, 3, 129, 1000), (1, 1, 64, 64), (1, 3, 1000, 77), (2, 2, 700, 128), (1, 5, 2000, 40),
              (1, 2, (cus // 2 + 5) * 256 - 19, 64 * 40 + 37), (2, 4, (2 * cus // 8 + 3) * 256, 100), (1, 1, (cus + 1) * 256, 64)]
    for B, H, Sq, Skv in shapes:
        q, k, v = inputs.qkv(B, H, Sq, Skv, 128, seed=Sq + Skv)
        qd = q.to(cuda).transpose(1, 2).contiguous().transpose(1, 2)
        kd, vd = k.to(cuda), v.to(cuda)
        out, lse = op(qd, kd, vd)
        rows = torch.arange(Sq) if Sq <= 2000 else torch.cat([torch.arange(0, 300), torch.arange(Sq - 600, Sq)])
        ref_out, ref_lse = oattn.sdpa_lse_f64(q[:, :, rows].float().numpy(), k.float().numpy(), v.float().numpy())
        _check(out[:, :, rows.to(cuda)], lse[:, :, rows.to(cuda)], ref_out, ref_lse, f"resident {(B, H, Sq, Skv)} even={even} bound={bound}")
        tuning("stream", 0)
        out0, lse0 = op(qd, kd, vd)
        tuning("stream", 1)
        assert (out.float() - out0.float()).abs().max().item() <= 2e-2 and (lse - lse0).abs().max().item() <= 1e-4
        assert torch.equal(torch.ops.para_attn.attention_forward(qd, kd, vd), out)
    # the shapes the planner picks it for by itself: FLUX's 1.7 rounds and short cross-attention pieces
    # (its partial results are what FLUX's workspace is for: the one-workgroup-per-piece plan has no split there)
    tuning("stream", -1)
    tuning("stream_even", -1)
    from paraattention_amd import _lib

    lib = _lib.load()
    qf = torch.empty(1, 24, 4608, 128, dtype=torch.bfloat16, device=cuda)
    assert lib.pa_attn_fwd_workspace_bytes(1, 24, 4608, 4608, 128, _lib.strides3(qf), _lib.strides3(qf)) > 0
    tuning("stream", 0)
    tuning("bound", 0)
    assert lib.pa_attn_fwd_workspace_bytes(1, 24, 4608, 4608, 128, _lib.strides3(qf), _lib.strides3(qf)) == 0


@pytest.mark.parametrize("rounds", [2, 4, 6])
@pytest.mark.parametrize("wave_rows", [32, 64])
def test_resident_workgroups_draw_their_tail_ranges(cuda, rounds, wave_rows, tuning):
    """The resident-workgroup kernel with its tail cut into rounds of ever shorter ranges that the workgroups draw
    from a counter as they run out of work (by itself the planner does that from 2048 key-tile steps per workgroup
    on; forced here at sizes the oracle can follow): fewer pieces than workgroups, a few pieces beyond a whole round,
    and exactly two rounds of pieces (the plan then gives up a round of whole pieces to have a tail), ragged query
    and key ends, both dtypes.  Sampled rows of three heads against the fp64 oracle; the whole output against the
    plan with one range per workgroup; and bit for bit against a second call (which workgroup drew which range
    differs from call to call and must not show)."""
    import ctypes

    from paraattention_amd import _lib

    lib = _lib.load()
    tuning("stream", 1)
    tuning("wave_rows", wave_rows)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    op = torch.ops.para_attn.attention_forward_with_lse
    shapes = [(1, 8, cus // 16 * 256 + 33, 64 * (260 if rounds > 2 else 130) + 7, torch.bfloat16),
              (2, 5, (cus // 10 + 5) * 256 - 100, 64 * 400 + 1, torch.float16),
              (1, 8, cus // 4 * 256, 64 * 70, torch.bfloat16)]
    for B, H, Sq, Skv, dtype in shapes:
        q, k, v = inputs.qkv(B, H, Sq, Skv, 128, seed=Sq + Skv, dtype=dtype)
        qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
        tuning("stream_dyn", 0)
        need0 = lib.pa_attn_fwd_workspace_bytes(B, H, Sq, Skv, 128, _lib.strides3(kd), _lib.strides3(vd))
        out0, lse0 = op(qd, kd, vd)
        tuning("stream_dyn", rounds)
        need = lib.pa_attn_fwd_workspace_bytes(B, H, Sq, Skv, 128, _lib.strides3(kd), _lib.strides3(vd))
        assert need >= 2 * cus * 2 * 256 * 129 * 4 > need0, "meant to take at least two rounds of ranges"
        out, lse = op(qd, kd, vd)
        heads = [0, H // 2, H - 1]
        rows = torch.cat([torch.arange(0, 200), torch.randint(0, Sq, (200,), generator=torch.Generator().manual_seed(Sq)), torch.arange(Sq - 300, Sq)])
        ref_out, ref_lse = oattn.sdpa_lse_f64(q[:, heads][:, :, rows].float().numpy(), k[:, heads].float().numpy(), v[:, heads].float().numpy())
        _check(out[:, heads][:, :, rows.to(cuda)], lse[:, heads][:, :, rows.to(cuda)], ref_out, ref_lse, f"drawn ranges {(B, H, Sq, Skv, dtype)} rounds={rounds}")
        assert (out.float() - out0.float()).abs().max().item() <= 2e-2 and (lse - lse0).abs().max().item() <= 1e-4
        for _ in range(2):
            out2, lse2 = op(qd, kd, vd)
            assert torch.equal(out2, out) and torch.equal(lse2, lse)
        # a workspace that holds the equal ranges but not the drawn ones: the call falls back to the former
        ws = torch.empty(need0, dtype=torch.uint8, device=cuda)
        out3, lse3 = torch.empty_like(qd), torch.empty_like(lse)
        vp = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
        rc = lib.pa_attn_fwd_lse_ws(vp(qd), vp(kd), vp(vd), vp(out3), vp(lse3), 0 if dtype == torch.bfloat16 else 1, B, H, Sq, Skv, 128,
                                    _lib.strides3(qd), _lib.strides3(kd), _lib.strides3(vd), _lib.strides3(out3), 1.0 / math.sqrt(128), None, 0,
                                    vp(ws), need0, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, lib.pa_last_error()
        torch.cuda.synchronize()
        assert torch.equal(out3, out0) and torch.equal(lse3, lse0)


@pytest.mark.parametrize("rounds", [2, 5])
@pytest.mark.parametrize("wave_rows", [32, 64])
def test_one_workgroup_draws_every_range(cuda, rounds, wave_rows, tuning):
    """A workgroup may draw the range that follows its own: two items in a row then belong to one piece (no new Q, no
    new K/V descriptor), and the first one's partial result must still be written and the accumulators cleared before
    the second begins.  With 256 workgroups drawing at once that is rare; the test aid `stream_solo` has workgroup 0
    draw and compute every range in turn, so every boundary between ranges is of that kind.  Fewer pieces than
    compute units (all work is in the tail); against the fp64 oracle and the plan with one range per workgroup."""
    tuning("stream", 1)
    tuning("wave_rows", wave_rows)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    op = torch.ops.para_attn.attention_forward_with_lse
    B, H, Sq, Skv = 1, 4, cus // 16 * 256 + 33, 64 * 520 + 7
    q, k, v = inputs.qkv(B, H, Sq, Skv, 128, seed=5)
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    tuning("stream_dyn", 0)
    out0, lse0 = op(qd, kd, vd)
    tuning("stream_dyn", rounds)
    tuning("stream_solo", 1)
    out, lse = op(qd, kd, vd)
    rows = torch.cat([torch.arange(0, 300), torch.arange(Sq - 300, Sq)])
    ref_out, ref_lse = oattn.sdpa_lse_f64(q[:, :, rows].float().numpy(), k.float().numpy(), v.float().numpy())
    _check(out[:, :, rows.to(cuda)], lse[:, :, rows.to(cuda)], ref_out, ref_lse, f"one workgroup, {rounds} rounds")
    assert (out.float() - out0.float()).abs().max().item() <= 2e-2 and (lse - lse0).abs().max().item() <= 1e-4
    tuning("stream_solo", 0)
    out2, lse2 = op(qd, kd, vd)  # the same ranges drawn by all workgroups: the same bits
    assert torch.equal(out2, out) and torch.equal(lse2, lse)


def test_drawn_ranges_random_configurations(cuda, tuning):
    """Sixteen seeded random draws for the resident-workgroup kernel with drawn tail ranges forced on: batch, heads,
    query rows and keys such that the work is 300 to 1200 key-tile steps per workgroup (whole rounds of pieces or
    none, tails of every size), 2 to 6 rounds, either dtype, [B,H,S,D] or [B,S,H,D] memory, and in half of the cases a
    prefix key mask that keeps at least 7/8 of the keys of every batch element (the variant with per-batch key counts
    where the launch is long enough for it, the kernel with one workgroup per query tile below).  Sampled rows of up
    to three heads against the fp64 oracle, and the same bits from a second call."""
    tuning("stream", 1)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    rng = np.random.default_rng(2024)
    op = torch.ops.para_attn.attention_forward_with_lse
    for case in range(16):
        B, H = int(rng.integers(1, 3)), int(rng.integers(1, 7))
        steps = int(rng.integers(300, 1200)) * cus          # key-tile steps of the whole launch
        L = int(rng.integers(40, 700))                       # key tiles per piece
        pieces = max(B * H, steps // L)
        Sq = max(1, pieces // (B * H)) * 256 - int(rng.integers(0, 256))
        Skv = L * 64 - int(rng.integers(0, 64))
        dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float16
        tuning("stream_dyn", int(rng.integers(2, 7)))
        q, k, v = inputs.qkv(B, H, Sq, Skv, 128, seed=4000 + case, dtype=dtype)
        keep = None
        if case % 2:
            lens = [int(rng.integers(Skv - Skv // 8, Skv + 1)) for _ in range(B)]
            keep = torch.arange(Skv)[None, :] < torch.tensor(lens)[:, None]
        heads = sorted(set([0, H // 2, H - 1]))
        rows = torch.cat([torch.arange(0, min(Sq, 120)), torch.randint(0, Sq, (120,), generator=torch.Generator().manual_seed(case)), torch.arange(max(0, Sq - 120), Sq)])
        ref_out, ref_lse = oattn.sdpa_lse_f64(q[:, heads][:, :, rows].float().numpy(), k[:, heads].float().numpy(), v[:, heads].float().numpy(),
                                              None, None if keep is None else keep[:, None, None, :].numpy())
        dev = [t.to(cuda) for t in (q, k, v)]
        for i in range(3):
            if rng.random() < 0.4:
                dev[i] = dev[i].transpose(1, 2).contiguous().transpose(1, 2)
        mask = None if keep is None else keep[:, None, None, :].to(cuda)
        out, lse = op(*dev, mask)
        what = f"case {case}: B{B} H{H} Sq{Sq} Skv{Skv} {dtype} masked={keep is not None}"
        _check(out[:, heads][:, :, rows.to(cuda)], lse[:, heads][:, :, rows.to(cuda)], ref_out, ref_lse, what)
        out2, lse2 = op(*dev, mask)
        assert torch.equal(out2, out) and torch.equal(lse2, lse), what


def test_planner_draws_ranges_for_long_launches_only(cuda, tuning):
    """What the planner asks of the workspace says which plan it took: four rounds of ranges (4 x compute units x two
    partial results, and the counter's 256 bytes) from 2048 key-tile steps per workgroup on, at most one range per
    workgroup below."""
    import ctypes

    from paraattention_amd import _lib

    lib = _lib.load()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    tuning("bound", 0)
    per_range = 2 * 256 * 129 * 4

    def need(H, S):
        st = (ctypes.c_int64 * 3)(H * S * 128, S * 128, 128)
        return lib.pa_attn_fwd_workspace_bytes(1, H, S, S, 128, st, st)

    assert need(3, 119056) == 4 * cus * per_range + 256
    assert need(40, 32760) == 4 * cus * per_range + 256
    assert need(24, 4608) <= cus * per_range
    assert need(24, 8192) <= cus * per_range


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_short_key_kernel(cuda, dtype, tuning):
    """The kernel for 449..512 keys per head (cross-attention to a text prompt), forced on for every shape here:
    fewer pieces than workgroups (runs of one piece), several pieces per workgroup with runs that end at a head's
    last query tile and go on in the next head, ragged last key tiles (449, 480, 511 keys) and ragged last query
    tiles, strided memory, several batches.  Every row against the fp64 oracle, and against the
    resident-workgroup kernel."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    op = torch.ops.para_attn.attention_forward_with_lse
    shapes = [(1, 2, 700, 512), (2, 3, 1380, 449), (1, 1, 31, 480), (1, 5, 256 * 3, 511),
              (1, cus // 4 + 3, 9 * 256 - 57, 512), (2, cus // 8 + 1, 5 * 256 + 1, 500)]
    for B, H, Sq, Skv in shapes:
        q, k, v = inputs.qkv(B, H, Sq, Skv, 128, seed=Sq + Skv, dtype=dtype)
        qd = q.to(cuda).transpose(1, 2).contiguous().transpose(1, 2)  # [B,S,H,D] memory
        kd, vd = k.to(cuda), v.to(cuda).transpose(1, 2).contiguous().transpose(1, 2)
        tuning("short_keys", 1)
        out, lse = op(qd, kd, vd)
        assert torch.equal(torch.ops.para_attn.attention_forward(qd, kd, vd), out)
        tuning("short_keys", 0)
        out0, lse0 = op(qd, kd, vd)
        heads = list(range(H)) if H <= 5 else [0, 1, H // 2, H - 2, H - 1]
        ref_out, ref_lse = oattn.sdpa_lse_f64(q[:, heads].float().numpy(), k[:, heads].float().numpy(), v[:, heads].float().numpy())
        _check(out[:, heads], lse[:, heads], ref_out, ref_lse, f"short keys {(B, H, Sq, Skv, dtype)}")
        assert (out.float() - out0.float()).abs().max().item() <= 2e-2 and (lse - lse0).abs().max().item() <= 1e-4
        tuning("short_keys", -1)  # by itself the planner takes it from two query tiles per compute unit on
        out_d, lse_d = op(qd, kd, vd)
        want = (out, lse) if B * H * ((Sq + 255) // 256) >= 2 * cus else (out0, lse0)
        assert torch.equal(out_d, want[0]) and torch.equal(lse_d, want[1]), (B, H, Sq, Skv)


@pytest.mark.parametrize("scale", [1.0, 0.3])
def test_short_key_kernel_large_logits(cuda, scale, tuning):
    """Logits of a few hundred through the kernel for short key sequences: the running maximum rises from tile to
    tile (keys sorted by their projection on a fixed direction, ascending, so that later tiles hold the larger
    scores; both halves of the workgroup, which walk the tiles in different orders), against the fp64 oracle."""
    tuning("short_keys", 1)
    B, H, Sq, Skv = 1, 3, 700, 507
    q, k, v = inputs.qkv(B, H, Sq, Skv, 128, seed=11)
    q = q * 3
    d = torch.randn(128, generator=torch.Generator().manual_seed(1))
    order = torch.argsort((k.float() @ d), dim=2)
    k = torch.gather(k, 2, order[..., None].expand_as(k))
    q = (q.float() + 2.0 * d).bfloat16()
    ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), scale)
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k.to(cuda), v.to(cuda), scale=scale)
    _check(out, lse, ref_out, ref_lse, f"short keys, large logits, scale {scale}")


def test_resident_workgroups_with_a_short_workspace(cuda, tuning):
    """pa_attn_fwd_lse_ws with less workspace than the plan asks for: the tail is cut into as many ranges as the
    workspace holds (still more than its pieces), or, below that, left as whole pieces; with no workspace at all the
    call runs as well.  Every variant against torch's CPU SDPA on sampled rows and against the full-workspace call."""
    import ctypes

    from paraattention_amd import _lib

    lib = _lib.load()
    tuning("bound", 0)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    B, H, D = 1, 2, 128
    Sq, Skv = (cus // 2 + 20) * 256 - 31, 64 * 24 + 9  # one round and 40 pieces more
    q, k, v = (t.to(cuda) for t in inputs.qkv(B, H, Sq, Skv, D, seed=8))
    need = lib.pa_attn_fwd_workspace_bytes(B, H, Sq, Skv, D, _lib.strides3(k), _lib.strides3(v))
    per_range = 2 * 256 * 129 * 4
    assert need > 100 * per_range, "meant to cut the 40 pieces of the tail into more than 100 ranges"
    vp = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None  # noqa: E731
    rows = torch.cat([torch.arange(0, 40), torch.arange(Sq - 300, Sq, 3)])
    ref_out, ref_lse = oattn.sdpa_lse_torch_cpu(q[:, :, rows.to(cuda)].cpu(), k.cpu(), v.cpu())
    results = []
    for nbytes in (need, 100 * per_range + 77, 41 * per_range, 10 * per_range, 0):
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=cuda) if nbytes else None
        out, lse = torch.empty_like(q), torch.empty((B, H, Sq), dtype=torch.float32, device=cuda)
        rc = lib.pa_attn_fwd_lse_ws(vp(q), vp(k), vp(v), vp(out), vp(lse), 0, B, H, Sq, Skv, D, _lib.strides3(q),
                                    _lib.strides3(k), _lib.strides3(v), _lib.strides3(out), 1.0 / math.sqrt(D), None, 0,
                                    vp(ws), nbytes, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, lib.pa_last_error()
        torch.cuda.synchronize()
        _check(out[:, :, rows.to(cuda)], lse[:, :, rows.to(cuda)], ref_out.float().numpy(), ref_lse.numpy(), f"workspace of {nbytes} bytes")
        results.append((out, lse))
    for out, lse in results[1:]:
        assert (out.float() - results[0][0].float()).abs().max().item() <= 2e-2
        assert (lse - results[0][1]).abs().max().item() <= 1e-4
    assert torch.equal(results[3][0], results[4][0])  # too short for any cut and none at all: the same whole-piece plan


@pytest.mark.parametrize("D,bm", [(128, "256"), (64, "128"), (64, "256")])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_score_bound_variants(cuda, dtype, D, bm, tuning):
    """The dense kernels (head_dim 128: 256 rows; head_dim 64: both sizes) drop the running maximum when
    |q| |k| scale bounds every score (computed on the device); forced on at a small size here.  Unit-variance inputs
    sit below the bf16 limit (bound about 23 of 60) and above the fp16 one (14); inputs four times larger exceed
    both, smaller ones neither, so both variants run for each type; every case is checked against the fp64 oracle
    and against the launch without the bound."""
    tuning("bm", int(bm))
    B, H, Sq, Skv = 2, 3, 700, 1500
    op = torch.ops.para_attn.attention_forward_with_lse
    for gain, kgain in ((1.0, 1.0), (4.0, 4.0), (0.25, 1.0), (1.0, 0.0)):
        q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=31, dtype=dtype)
        q, k = (q.float() * gain).to(dtype), (k.float() * kgain).to(dtype)
        ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy())
        tuning("bound", 1)
        out, lse = op(q.to(cuda), k.to(cuda), v.to(cuda))
        _check(out, lse, ref_out, ref_lse, f"bound on, gain {gain} {kgain} {dtype}")
        tuning("bound", 0)
        out0, lse0 = op(q.to(cuda), k.to(cuda), v.to(cuda))
        assert (out.float() - out0.float()).abs().max().item() <= 2e-2 and (lse - lse0).abs().max().item() <= 1e-4


@pytest.mark.parametrize("D,bm", [(128, "256"), (64, "128"), (64, "256")])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("side", ["under", "over"])
def test_score_bound_at_the_limit(cuda, dtype, D, bm, side, tuning):
    """The score bound where dropping the running maximum is riskiest: every q and k row has the same norm, chosen so
    that the device-computed bound |q| |k| scale log2(e) lands just under the limit (about 58 of 60 for bf16, 13.5 of
    14 for fp16: the variant without a maximum runs) or just over it (the variant with the maximum runs), and some
    query rows meet one key aligned with them and one opposed to them, so a single row realises scores at both
    ends of the bound (exp2 of +58 and of -58 in one sum).  Against the fp64 oracle and against the launch with the
    bound switched off."""
    tuning("bm", int(bm))
    limit = 60.0 if dtype == torch.bfloat16 else 14.0
    target = limit - (2.0 if dtype == torch.bfloat16 else 0.5) if side == "under" else limit + (2.0 if dtype == torch.bfloat16 else 0.5)
    c = D ** -0.5 * 1.4426950408889634
    norm = (target / c) ** 0.5
    B, H, Sq, Skv = 1, 2, 600, 1300
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=77, dtype=torch.float32)
    q = q / q.norm(dim=-1, keepdim=True) * norm
    k = k / k.norm(dim=-1, keepdim=True) * norm
    planted = [0, 31, 32, 255, 256, 300, 599]  # first and last rows of wavefronts and workgroups among them
    for n, i in enumerate(planted):
        k[:, :, 7 + 64 * n] = q[:, :, i]         # aligned: the row's largest score, +bound
        k[:, :, 1299 - 97 * n] = -q[:, :, i]     # opposed: its smallest, -bound
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    # what the device computes from the rounded operands (largest row norms, fp32)
    bound = q.float().norm(dim=-1).max().item() * k.float().norm(dim=-1).max().item() * c
    assert (limit - 3 < bound < limit - 0.2) if side == "under" else (limit + 0.2 < bound < limit + 3), bound
    ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy())
    s = np.einsum("bhid,bhjd->bhij", q.float().numpy().astype(np.float64), k.float().numpy().astype(np.float64)) * c
    assert s[:, :, planted].max() > bound - 0.5 and s[:, :, planted].min() < -bound + 0.5  # both ends are realised
    op = torch.ops.para_attn.attention_forward_with_lse
    tuning("bound", 1)
    out, lse = op(q.to(cuda), k.to(cuda), v.to(cuda))
    _check(out, lse, ref_out, ref_lse, f"bound {bound:.2f} of {limit} ({side}) {dtype} D={D}")
    tuning("bound", 0)
    out0, lse0 = op(q.to(cuda), k.to(cuda), v.to(cuda))
    _check(out0, lse0, ref_out, ref_lse, f"no bound, {bound:.2f} {dtype} D={D}")
    assert (out.float() - out0.float()).abs().max().item() <= 2e-2 and (lse - lse0).abs().max().item() <= 1e-3


@pytest.mark.parametrize("D,Dv", [(32, 32), (40, 40), (72, 72), (80, 80), (96, 96), (128, 64), (64, 128), (16, 24), (120, 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_other_head_dims(cuda, D, Dv, dtype):
    """head_dims other than 64 and 128, and values narrower or wider than the keys, as aten's kernels behind the
    reference's op take them (src/para_attn/ops/__init__.py:58-109): the default scale is that of the true head_dim,
    out has the values' width, with and without a mask and is_causal; against the fp64 oracle and torch's CPU SDPA,
    and through F.scaled_dot_product_attention under the mode."""
    B, H, Sq, Skv = 2, 3, 150, 333
    g = torch.Generator().manual_seed(D * 131 + Dv)
    q = torch.randn(B, H, Sq, D, generator=g).to(dtype)
    k = torch.randn(B, H, Skv, D, generator=g).to(dtype)
    v = torch.randn(B, H, Skv, Dv, generator=g).to(dtype)
    ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy())
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    out, lse = torch.ops.para_attn.attention_forward_with_lse(qd, kd, vd)
    assert out.shape == (B, H, Sq, Dv) and out.dtype == dtype and out.is_contiguous() and lse.shape == (B, H, Sq)
    _check(out, lse, ref_out, ref_lse, f"head_dim {D}/{Dv} {dtype}")
    if D == Dv:
        cpu_out, cpu_lse = oattn.sdpa_lse_torch_cpu(q.float(), k.float(), v.float())
        _check(out, lse, cpu_out.numpy(), cpu_lse.numpy(), f"head_dim {D}/{Dv} {dtype} vs torch CPU")
    else:  # torch's CPU flash routine wants one head size; its composite SDPA takes any (no LSE from it)
        cpu_out = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
        _check(out, None, cpu_out.numpy(), None, f"head_dim {D}/{Dv} {dtype} vs torch CPU")
    assert torch.equal(torch.ops.para_attn.attention_forward(qd, kd, vd), out)
    # a scale of the caller's, a key mask that is no prefix, is_causal
    keep = torch.rand(B, 1, 1, Skv, generator=g) < 0.6
    keep[..., 0] = True
    m_out, m_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), 0.2, keep.numpy())
    out, lse = torch.ops.para_attn.attention_forward_with_lse(qd, kd, vd, keep.to(cuda), scale=0.2)
    _check(out, lse, m_out, m_lse, f"head_dim {D}/{Dv} masked")
    assert torch.equal(torch.ops.para_attn.attention_forward_sparse_kv(qd, kd, vd, keep.to(cuda), scale=0.2), out)
    c_out, c_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, oattn.causal_keep(Sq, Skv))
    out, lse = torch.ops.para_attn.attention_forward_with_lse(qd, kd, vd, is_causal=True)
    _check(out, lse, c_out, c_lse, f"head_dim {D}/{Dv} causal")
    import paraattention_amd

    with paraattention_amd.UnifiedAttnMode():
        routed = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd)
    assert torch.equal(routed, torch.ops.para_attn.attention_forward(qd, kd, vd))
    torch.library.opcheck(torch.ops.para_attn.attention_forward_with_lse.default, (qd, kd, vd), test_utils="test_faketensor")
    with pytest.raises(NotImplementedError):
        torch.ops.para_attn.attention_forward(torch.zeros(1, 1, 4, 160, dtype=dtype, device=cuda), torch.zeros(1, 1, 4, 160, dtype=dtype, device=cuda),
                                              torch.zeros(1, 1, 4, 160, dtype=dtype, device=cuda))


CAUSAL = [(1, 2, 1, 1), (1, 1, 17, 17), (2, 2, 64, 64), (1, 2, 129, 129), (1, 1, 300, 300), (1, 2, 700, 700),
          (1, 1, 300, 90), (1, 2, 90, 300), (1, 1, 1000, 1000)]


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("B,H,Sq,Skv", CAUSAL)
def test_causal_vs_f64(cuda, B, H, Sq, Skv, D):
    """is_causal=True as the reference's own op test asks for it (tests/ops/test_ops.py:28-31), plus Sq != Skv with
    torch's top-left alignment.  Every kernel variant must agree with the oracle."""
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=Sq * 7 + Skv)
    ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, oattn.causal_keep(Sq, Skv))
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    out, lse = torch.ops.para_attn.attention_forward_with_lse(qd, kd, vd, is_causal=True)
    _check(out, lse, ref_out, ref_lse, f"causal {(B, H, Sq, Skv, D)}")
    assert torch.equal(torch.ops.para_attn.attention_forward(qd, kd, vd, is_causal=True), out)


@pytest.mark.parametrize("env", [{"no_pipe": 1}, {"bm": 256}, {"bm": 128}])
def test_causal_alternative_kernels(cuda, env, tuning):
    for B, H, Sq, Skv, D in [(1, 2, 700, 700, 128), (1, 1, 300, 90, 128), (1, 2, 90, 300, 128), (2, 1, 513, 513, 128),
                             (1, 2, 700, 700, 64), (1, 1, 300, 90, 64), (2, 1, 513, 513, 64)]:
        q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=Sq + Skv)
        ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, oattn.causal_keep(Sq, Skv))
        for name, val in env.items():
            tuning(name, val)
        out, lse = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k.to(cuda), v.to(cuda), is_causal=True)
        for name in env:
            tuning(name, 0)
        _check(out, lse, ref_out, ref_lse, f"causal {env} {(B, H, Sq, Skv, D)}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 128])
def test_causal_reference_test_shape(cuda, dtype, D):
    """The reference's op test shape (tests/ops/test_ops.py:21-31: B1 H24 S4096, fp16 and bf16, is_causal) against
    torch's CPU SDPA with is_causal, on a subset of heads."""
    B, H, S = 1, 24, 4096
    q, k, v = inputs.qkv(B, H, S, S, D, seed=3, dtype=dtype)
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), k.to(cuda), v.to(cuda), is_causal=True)
    assert lse.dtype == torch.float32 and lse.shape == (B, H, S)
    hs = [0, 11, 23]
    ref_out, ref_lse = oattn.sdpa_lse_torch_cpu(q[:, hs].float(), k[:, hs].float(), v[:, hs].float(), is_causal=True)
    _check(out[:, hs], lse[:, hs], ref_out.numpy(), ref_lse.numpy(), f"causal 4096 {dtype} D={D}")


def test_causal_long_sequence_sampled_rows(cuda):
    """is_causal at a length where the launch has many rounds of workgroups of unequal length (started longest
    first) and most tiles lie below the diagonal: sampled rows against torch's CPU SDPA over each row's own key
    prefix, every row's LSE against the count of keys it sees for zero queries."""
    B, H, S, D = 1, 2, 20000 + 37, 128
    q, k, v = inputs.qkv(B, H, S, S, D, seed=12)
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    out, lse = torch.ops.para_attn.attention_forward_with_lse(qd, kd, vd, is_causal=True)
    g = torch.Generator().manual_seed(4)
    for r in [0, 1, 63, 64, 255, 256, S - 1] + torch.randint(0, S, (10,), generator=g).tolist():
        ro, rl = oattn.sdpa_lse_torch_cpu(q[:, :, r : r + 1], k[:, :, : r + 1], v[:, :, : r + 1])
        _check(out[:, :, r : r + 1], lse[:, :, r : r + 1], ro.float().numpy(), rl.numpy(), f"causal row {r}")
    _, lse0 = torch.ops.para_attn.attention_forward_with_lse(torch.zeros_like(qd), kd, vd, is_causal=True)
    want = torch.log(torch.arange(1, S + 1, dtype=torch.float64))[None, None, :].expand(B, H, S)
    assert (lse0.cpu().double() - want).abs().max().item() <= 1e-3


def test_causal_argument_rules(cuda):
    q, k, v = (t.to(cuda) for t in inputs.qkv(1, 1, 32, 32, 128))
    mask = torch.ones(1, 1, 1, 32, dtype=torch.bool, device=cuda)
    with pytest.raises(ValueError):
        torch.ops.para_attn.attention_forward_with_lse(q, k, v, mask, is_causal=True)
    with pytest.raises(NotImplementedError):
        torch.ops.para_attn.attention_forward_sparse_kv(q, k, v, mask, is_causal=True)


def test_random_configurations(cuda):
    """Sixty seeded random draws over shape, head_dim, dtype, layout, scale, is_causal and per-batch key counts,
    each against the fp64 oracle: the combinations no hand-written case lists."""
    rng = np.random.default_rng(2024)
    for case in range(60):
        B, H = int(rng.integers(1, 3)), int(rng.integers(1, 5))
        Sq, Skv = int(rng.integers(1, 700)), int(rng.integers(1, 700))
        D = int(rng.choice([64, 128]))
        dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float16
        causal = bool(rng.random() < 0.3)
        use_len = (not causal) and bool(rng.random() < 0.3)
        bshd = bool(rng.random() < 0.4)
        scale = None if rng.random() < 0.6 else float(rng.uniform(0.02, 0.3))
        q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=1000 + case, dtype=dtype)
        keep = None
        mask = None
        if causal:
            keep = oattn.causal_keep(Sq, Skv)
        elif use_len:
            lens = rng.integers(1, Skv + 1, size=B)
            kb = np.arange(Skv)[None, :] < lens[:, None]
            keep = kb[:, None, None, :]
            mask = torch.from_numpy(kb)[:, None, None, :].to(cuda)
        ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), scale, keep)
        qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
        if bshd:  # [B,S,H,D] memory behind a [B,H,S,D] view
            qd, kd, vd = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (qd, kd, vd))
        out, lse = torch.ops.para_attn.attention_forward_with_lse(qd, kd, vd, mask, is_causal=causal, scale=scale)
        what = f"case {case}: B{B} H{H} Sq{Sq} Skv{Skv} D{D} {dtype} causal={causal} len={use_len} bshd={bshd} scale={scale}"
        _check(out, lse, ref_out, ref_lse, what)


def test_short_key_kernel_random_configurations(cuda, tuning):
    """Thirty seeded random draws for the kernel for short key sequences (forced on): batch, heads, query rows from a
    handful to several query tiles per workgroup, 449..512 keys, dtype, scale, [B,H,S,D] or [B,S,H,D] memory for each
    of q, k, v -- each against the fp64 oracle."""
    tuning("short_keys", 1)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    rng = np.random.default_rng(77)
    for case in range(30):
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 9))
        big = rng.random() < 0.25  # now and then enough pieces for several per workgroup and runs that cross heads
        Sq = int(rng.integers(256 * cus // (B * H), 3 * 256 * cus // (B * H))) if big else int(rng.integers(1, 1500))
        Skv = int(rng.integers(449, 513))
        dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float16
        scale = None if rng.random() < 0.6 else float(rng.uniform(0.02, 0.3))
        q, k, v = inputs.qkv(B, H, Sq, Skv, 128, seed=3000 + case, dtype=dtype)
        heads = list(range(H)) if not big else sorted(set([0, H // 2, H - 1]))
        rows = torch.arange(Sq) if not big else torch.cat([torch.arange(0, 300), torch.randint(0, Sq, (300,), generator=torch.Generator().manual_seed(case)), torch.arange(Sq - 300, Sq)])
        ref_out, ref_lse = oattn.sdpa_lse_f64(q[:, heads][:, :, rows].float().numpy(), k[:, heads].float().numpy(), v[:, heads].float().numpy(), scale)
        dev = [t.to(cuda) for t in (q, k, v)]
        for i in range(3):
            if rng.random() < 0.4:
                dev[i] = dev[i].transpose(1, 2).contiguous().transpose(1, 2)
        out, lse = torch.ops.para_attn.attention_forward_with_lse(*dev, scale=scale)
        _check(out[:, heads][:, :, rows.to(cuda)], lse[:, heads][:, :, rows.to(cuda)], ref_out, ref_lse,
               f"case {case}: B{B} H{H} Sq{Sq} Skv{Skv} {dtype} scale={scale}")


def test_key_rows_spread_over_4gib(cuda):
    """K and V whose rows lie 1 MiB apart span more than 4 GiB per head: beyond the 32-bit offsets of the
    pipelined kernel, so the launch must pick the kernel without that limit (a wrong pick reads zeros)."""
    B, H, Sq, Skv, D = 1, 1, 200, 4100, 128
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=31)
    ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy())
    stride = 1 << 19  # elements between consecutive key rows
    big = torch.empty(2, Skv * stride, dtype=torch.bfloat16, device=cuda)
    kd = big[0].as_strided((B, H, Skv, D), (0, 0, stride, 1))
    vd = big[1].as_strided((B, H, Skv, D), (0, 0, stride, 1))
    kd.copy_(k.to(cuda))
    vd.copy_(v.to(cuda))
    assert (Skv - 1) * stride * 2 >= 1 << 32
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q.to(cuda), kd, vd)
    _check(out, lse, ref_out, ref_lse, "rows 1 MiB apart")
    with pytest.raises(NotImplementedError):  # the fused ring step has no such fallback and says so
        torch.ops.para_attn.attention_forward_accumulate_(
            torch.empty(B, H, Sq, D, device=cuda), torch.empty(B, H, Sq, device=cuda), q.to(cuda), kd, vd, True)
    del big, kd, vd
    torch.cuda.empty_cache()


def test_unsupported_raise(cuda):
    q, k, v = (t.to(cuda) for t in inputs.qkv(1, 1, 16, 16, 128))
    with pytest.raises(NotImplementedError):
        torch.ops.para_attn.attention_forward_with_lse(q, k, v, dropout_p=0.1)
    big = torch.zeros(1, 1, 16, 160, dtype=q.dtype, device=cuda)
    with pytest.raises(NotImplementedError):  # head_dim above 128 (up to 128 runs, zero-padded where it is not 64 or 128)
        torch.ops.para_attn.attention_forward_with_lse(big, big, big)
    with pytest.raises(NotImplementedError):  # the ops outside the SDPA signature take 64 / 128 only
        torch.ops.para_attn.attention_forward_sweep(q[..., :32], [k[..., :32]], [v[..., :32]])
    with pytest.raises(NotImplementedError):
        torch.ops.para_attn.attention_forward_with_lse(q.float(), k.float(), v.float())
