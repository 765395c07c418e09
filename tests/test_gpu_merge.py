"""Parity of the fused merge kernel and the ring sweep with the oracle and with torch's own merger."""
import numpy as np
import pytest
import torch

import paraattention_amd
from oracle import attention as oattn
from oracle import inputs
from oracle import merge as omerge

pytestmark = pytest.mark.gpu


def _partials(B, H, S, D, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    o1 = torch.randn(B, H, S, D, generator=g).to(dtype)
    o2 = torch.randn(B, H, S, D, generator=g).to(dtype)
    l1 = torch.randn(B, H, S, generator=g) * 3 + 5
    l2 = torch.randn(B, H, S, generator=g) * 3 + 5
    return o1, l1, o2, l2


@pytest.mark.parametrize("shape", [(1, 1, 1, 8), (1, 2, 34, 128), (2, 3, 257, 64), (1, 24, 1000, 128)])
@pytest.mark.parametrize("blk_dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_merge_step_vs_oracle(cuda, shape, blk_dtype):
    B, H, S, D = shape
    o1, l1, o2, l2 = _partials(B, H, S, D, seed=S, dtype=blk_dtype)
    ref_out, ref_lse = omerge.merge_step(o1.float().numpy(), l1.numpy(), o2.float().numpy(), l2.numpy())
    # functional: 16-bit accumulator in (the first real step), fp32 out
    out, lse = torch.ops.para_attn.merge_attention_lse(o1.to(cuda), l1.to(cuda), o2.to(cuda), l2.to(cuda))
    assert out.dtype == torch.float32 and lse.dtype == torch.float32 and lse.shape == l1.shape
    np.testing.assert_allclose(out.cpu().numpy(), ref_out, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(lse.cpu().numpy(), ref_lse, rtol=1e-6, atol=2e-6)
    # in-place on fp32 accumulators
    acc, acc_l = o1.float().to(cuda), l1.clone().to(cuda)
    torch.ops.para_attn.merge_attention_lse_(acc, acc_l, o2.to(cuda), l2.to(cuda))
    assert torch.equal(acc, out) and torch.equal(acc_l, lse)
    # final step writes the activation dtype directly = fp32 result rounded once
    if blk_dtype != torch.float32:
        outb, _ = torch.ops.para_attn.merge_attention_lse(o1.float().to(cuda), l1.to(cuda), o2.to(cuda), l2.to(cuda), blk_dtype)
        assert torch.equal(outb, out.to(blk_dtype))
    # LSE given as [B,H,S,1] (the cuDNN layout torch's merger also accepts)
    out4, lse4 = torch.ops.para_attn.merge_attention_lse(o1.to(cuda), l1[..., None].to(cuda), o2.to(cuda), l2[..., None].to(cuda))
    assert lse4.shape == (B, H, S, 1) and torch.equal(out4, out)


@pytest.mark.parametrize("D", [24, 48, 72, 80, 200])
@pytest.mark.parametrize("acc_dtype", [torch.float32, torch.bfloat16])
def test_merge_in_place_head_dims_off_the_wavefront(cuda, D, acc_dtype):
    """In-place steps at head dims whose 8-element chunk count does not divide 64: a row's threads then straddle
    wavefronts (D = 48: rows 10, 21 ... start in one wavefront and end in the next), and the step must still read
    the old LSE for every chunk.  Many rows, so that every position of a row inside a wavefront and a workgroup
    occurs; checked against the oracle's step and bit for bit against the functional op, which never aliases."""
    B, H, S = 2, 3, 1777
    o1, l1, o2, l2 = _partials(B, H, S, D, seed=D, dtype=acc_dtype)
    # weights far from 0 and 1 on most rows, so an element merged with the new LSE instead of the old one shows
    ref_out, ref_lse = omerge.merge_step(o1.float().numpy(), l1.numpy(), o2.float().numpy(), l2.numpy())
    want, want_l = torch.ops.para_attn.merge_attention_lse(o1.to(cuda), l1.to(cuda), o2.to(cuda), l2.to(cuda), acc_dtype)
    acc, acc_l = o1.to(cuda), l1.clone().to(cuda)
    torch.ops.para_attn.merge_attention_lse_(acc, acc_l, o2.to(cuda), l2.to(cuda))
    assert torch.equal(acc, want) and torch.equal(acc_l, want_l)
    tol = dict(rtol=1e-5, atol=1e-5) if acc_dtype == torch.float32 else dict(rtol=1.6e-2, atol=1e-5)
    np.testing.assert_allclose(acc.float().cpu().numpy(), ref_out, **tol)
    np.testing.assert_allclose(acc_l.cpu().numpy(), ref_lse, rtol=1e-6, atol=2e-6)
    # a second step on the merged pair (the accumulator's LSE now differs from row to row in the last bits)
    o3, l3, _, _ = _partials(B, H, S, D, seed=D + 1, dtype=acc_dtype)
    want2, want_l2 = torch.ops.para_attn.merge_attention_lse(acc.clone(), acc_l.clone(), o3.to(cuda), l3.to(cuda), acc_dtype)
    torch.ops.para_attn.merge_attention_lse_(acc, acc_l, o3.to(cuda), l3.to(cuda))
    assert torch.equal(acc, want2) and torch.equal(acc_l, want_l2)


def test_merge_vs_torch_sdpa_merger(cuda):
    from torch.distributed.tensor.experimental._context_parallel._attention import _SDPAMerger

    B, H, S, D = 1, 4, 300, 128
    g = torch.Generator().manual_seed(0)
    outs = [torch.randn(B, H, S, D, generator=g).bfloat16() for _ in range(5)]
    lses = [torch.randn(B, H, S, generator=g) * 4 for _ in range(5)]
    ref = _SDPAMerger(True, 2)
    mine = paraattention_amd.SDPAMerger(True, 2)
    for o, l in zip(outs, lses):
        ref.step(o, l, False)
        mine.step(o.to(cuda), l.to(cuda), False)
    ro, rl = ref.results()
    mo, ml = mine.results()
    assert mo.dtype == ro.dtype and ml.shape == rl.shape
    torch.testing.assert_close(ml.cpu(), rl, rtol=1e-6, atol=1e-5)
    torch.testing.assert_close(mo.float().cpu(), ro.float(), rtol=1.6e-2, atol=1e-5)  # one bf16 ulp after fp32 merge


def test_merge_empty_partials(cuda):
    # a partial that saw no key (lse = -inf) is the identity, on either side
    o1, l1, o2, l2 = _partials(1, 1, 64, 128, seed=1)
    ninf = torch.full_like(l2, float("-inf"))
    out, lse = torch.ops.para_attn.merge_attention_lse(o1.to(cuda), l1.to(cuda), torch.zeros_like(o2).to(cuda), ninf.to(cuda))
    assert torch.equal(out.cpu(), o1.float()) and torch.equal(lse.cpu(), l1)
    out, lse = torch.ops.para_attn.merge_attention_lse(torch.zeros_like(o1).to(cuda), ninf.to(cuda), o2.to(cuda), l2.to(cuda))
    assert torch.equal(out.cpu(), o2.float()) and torch.equal(lse.cpu(), l2)


@pytest.mark.parametrize("fused", ["sweep", True, False])
def test_ring_sweep_equals_full_attention(cuda, fused):
    # the ring-sweep shape in miniature, ragged like 14882 = 116*128 + 34: 8 blocks of 290 keys
    B, H, Sq, D, nblk, blk = 1, 4, 290, 128, 8, 290
    q, k, v = inputs.qkv(B, H, Sq, nblk * blk, D, seed=3)
    ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy())
    kb = [k[:, :, i * blk : (i + 1) * blk].contiguous().to(cuda) for i in range(nblk)]
    vb = [v[:, :, i * blk : (i + 1) * blk].contiguous().to(cuda) for i in range(nblk)]
    out, lse = paraattention_amd.ring_sweep(q.to(cuda), kb, vb, fused=fused)
    assert out.dtype == torch.bfloat16
    np.testing.assert_allclose(lse.cpu().numpy(), ref_lse, atol=1e-3)
    np.testing.assert_allclose(out.float().cpu().numpy(), ref_out, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("wave_rows", [32, 64])
def test_one_launch_sweep(cuda, dtype, wave_rows, tuning):
    """attention_forward_sweep: blocks at separate addresses walked as one key sequence.  Ragged block length
    (tiles never straddle blocks), ragged query length, [B,S,H,D] memory, 1 to 16 blocks, more pieces than the
    chip has compute units and fewer, with and without the score bound; against the fp64 oracle over the
    concatenated keys and bit for bit against the dense op on the concatenation where both take the same path."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    D = 128
    tuning("wave_rows", wave_rows)  # both forms of the resident-workgroup kernel walk the segments
    for B, H, Sq, blk, n, bound in [(1, 2, 300, 290, 8, -1), (2, 3, 77, 64, 3, -1), (1, 4, 600, 1000, 16, 1), (1, 1, 256, 37, 1, -1),
                                    (1, 2, (cus // 2 + 3) * 256 - 100, 150, 4, 1)]:
        tuning("bound", bound)
        q, k, v = inputs.qkv(B, H, Sq, blk * n, D, seed=blk + n, dtype=dtype)
        rows = torch.arange(Sq) if Sq <= 1000 else torch.cat([torch.arange(0, 50), torch.arange(Sq - 400, Sq, 3)])
        ref_out, ref_lse = oattn.sdpa_lse_f64(q[:, :, rows].float().numpy(), k.float().numpy(), v.float().numpy())
        qd = q.to(cuda).transpose(1, 2).contiguous().transpose(1, 2)
        kb = [t.contiguous().to(cuda) for t in k.split(blk, 2)]
        vb = [t.contiguous().to(cuda) for t in v.split(blk, 2)]
        out, lse = torch.ops.para_attn.attention_forward_sweep(qd, kb, vb)
        assert out.dtype == dtype and out.stride() == qd.stride() and lse.shape == (B, H, Sq)
        np.testing.assert_allclose(lse[:, :, rows.to(cuda)].cpu().numpy(), ref_lse, atol=1e-3)
        np.testing.assert_allclose(out[:, :, rows.to(cuda)].float().cpu().numpy(), ref_out, atol=2e-2, rtol=2e-2)
        # ring_sweep takes this path by default
        ro, rl = paraattention_amd.ring_sweep(qd, kb, vb)
        assert torch.equal(ro, out) and torch.equal(rl, lse)
    with pytest.raises(NotImplementedError):
        q64, k64, v64 = (t.to(cuda) for t in inputs.qkv(1, 1, 16, 16, 64))
        torch.ops.para_attn.attention_forward_sweep(q64, [k64, k64], [v64, v64])
    with pytest.raises(ValueError):
        torch.ops.para_attn.attention_forward_sweep(qd, kb, vb[:-1])


@pytest.mark.parametrize("wave_rows", [32, 64])
def test_fused_accumulate_steps(cuda, wave_rows, tuning):
    """attention_forward_accumulate_ / _final against the oracle's merge of the oracle's partials, on a grid that
    takes the key-split tail (so the split merge folds the accumulator too), with a strided query."""
    from oracle import merge as omerge
    from paraattention_amd import _lib

    tuning("wave_rows", wave_rows)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    B, H, D = 1, 8, 128
    Sq = (cus // (B * H) + 3) * 256 - 77
    blks = [64 * 40 + 5, 64 * 33, 64 * 47 + 63]
    q, k, v = inputs.qkv(B, H, Sq, sum(blks), D, seed=5)
    qd = q.to(cuda).transpose(1, 2).contiguous().transpose(1, 2)
    ks, vs = k.split(blks, 2), v.split(blks, 2)
    assert _lib.load().pa_attn_fwd_workspace_bytes(B, H, Sq, blks[0], D, _lib.strides3(ks[0]), _lib.strides3(vs[0])) > 0
    acc = torch.full((B, H, Sq, D), float("nan"), device=cuda)       # first=True must not read it
    acc_l = torch.full((B, H, Sq), float("nan"), device=cuda)
    rows = torch.cat([torch.arange(0, 40), torch.arange(Sq - 300, Sq)])  # unsplit head and split tail tiles
    parts = [oattn.sdpa_lse_f64(q[:, :, rows].float().numpy(), kk.float().numpy(), vv.float().numpy()) for kk, vv in zip(ks, vs)]
    for i in range(2):
        torch.ops.para_attn.attention_forward_accumulate_(acc, acc_l, qd, ks[i].to(cuda), vs[i].to(cuda), i == 0)
        ro, rl = omerge.merge_all([p[0] for p in parts[: i + 1]], [p[1] for p in parts[: i + 1]])
        np.testing.assert_allclose(acc_l[:, :, rows].cpu().numpy(), rl, atol=1e-3)
        np.testing.assert_allclose(acc[:, :, rows].cpu().numpy(), ro, atol=2e-2, rtol=2e-2)
    before = acc.clone()
    out = torch.ops.para_attn.attention_forward_accumulate_final(acc, acc_l, qd, ks[2].to(cuda), vs[2].to(cuda))
    assert out.dtype == torch.bfloat16 and torch.equal(acc, before)
    ref_out, ref_lse = oattn.sdpa_lse_f64(q[:, :, rows].float().numpy(), k.float().numpy(), v.float().numpy())
    np.testing.assert_allclose(acc_l[:, :, rows].cpu().numpy(), ref_lse, atol=1e-3)
    np.testing.assert_allclose(out[:, :, rows].float().cpu().numpy(), ref_out, atol=2e-2, rtol=2e-2)
    # unsplit launch gives the same (to rounding)
    tuning("no_split", 1)
    acc_l2 = acc_l.clone()
    torch.ops.para_attn.attention_forward_accumulate_(acc, acc_l2, qd, ks[0].to(cuda), vs[0].to(cuda), True)
    torch.ops.para_attn.attention_forward_accumulate_(acc, acc_l2, qd, ks[1].to(cuda), vs[1].to(cuda))
    out2 = torch.ops.para_attn.attention_forward_accumulate_final(acc, acc_l2, qd, ks[2].to(cuda), vs[2].to(cuda))
    assert (out2.float() - out.float()).abs().max().item() <= 2e-2 and (acc_l2 - acc_l).abs().max().item() <= 1e-4
    # unsupported shapes say so
    q64, k64, v64 = (t.to(cuda) for t in inputs.qkv(1, 1, 16, 16, 64))
    with pytest.raises(NotImplementedError):
        torch.ops.para_attn.attention_forward_accumulate_(torch.zeros(1, 1, 16, 64, device=cuda), torch.zeros(1, 1, 16, device=cuda), q64, k64, v64, True)


def test_ring_sweep_full_shape_sampled(cuda):
    # the ring-sweep shape at full size (Q block 14882 x 24 heads against 8 KV blocks of 14882);
    # the oracle checks sampled rows of two heads against one full-length SDPA over 119056 keys
    B, H, Sq, D, nblk = 1, 24, 14882, 128, 8
    g = torch.Generator().manual_seed(0)
    q = torch.randn(B, H, Sq, D, generator=g).bfloat16()
    kb_cpu = [torch.randn(B, H, Sq, D, generator=g).bfloat16() for _ in range(nblk)]
    vb_cpu = [torch.randn(B, H, Sq, D, generator=g).bfloat16() for _ in range(nblk)]
    out, lse = paraattention_amd.ring_sweep(q.to(cuda), [t.to(cuda) for t in kb_cpu], [t.to(cuda) for t in vb_cpu])
    rows = torch.cat([torch.arange(0, 16), torch.arange(Sq - 40, Sq), torch.randint(0, Sq, (72,), generator=g)])
    for h in (0, 23):
        kf = torch.cat([t[:, h : h + 1] for t in kb_cpu], 2)
        vf = torch.cat([t[:, h : h + 1] for t in vb_cpu], 2)
        ro, rl = oattn.sdpa_lse_torch_cpu(q[:, h : h + 1, rows], kf, vf)
        np.testing.assert_allclose(lse[:, h : h + 1, rows.to(cuda)].cpu().numpy(), rl.numpy(), atol=1e-3)
        np.testing.assert_allclose(out[:, h : h + 1, rows.to(cuda)].float().cpu().numpy(), ro.float().numpy(), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("fused", [True, False])
def test_ring_sweep_full_shape_every_row_by_closed_forms(cuda, fused):
    """Every row of the ring-sweep shape, by properties that need no oracle run: with zero keys in all 8 blocks
    LSE = ln(8 * 14882) and out = the mean of V over all blocks' keys; with V constant within a block the sweep
    gives the mean of the blocks' constants."""
    B, H, Sq, D, nblk = 1, 24, 14882, 128, 8
    g = torch.Generator().manual_seed(4)
    q = torch.randn(B, H, Sq, D, generator=g).bfloat16().to(cuda)
    vb = [torch.randn(B, H, Sq, D, generator=g).bfloat16().to(cuda) for _ in range(nblk)]
    zero = [torch.zeros(B, H, Sq, D, dtype=torch.bfloat16, device=cuda) for _ in range(nblk)]
    out, lse = paraattention_amd.ring_sweep(q, zero, vb, fused=fused)
    assert (lse - np.log(nblk * Sq)).abs().max().item() <= 1e-3
    mean_v = torch.stack([t.float().mean(dim=2) for t in vb]).mean(dim=0)[:, :, None]  # equal block sizes
    assert (out.float() - mean_v).abs().max().item() <= 2e-2
    # V constant within a block, a different constant per block, zero keys: out = the mean of the constants
    consts = [torch.full((B, H, Sq, D), float(i - 3), dtype=torch.bfloat16, device=cuda) for i in range(nblk)]
    out_c, _ = paraattention_amd.ring_sweep(q, zero, consts, fused=fused)
    assert (out_c.float() - (sum(range(nblk)) / nblk - 3.0)).abs().max().item() <= 2e-2
