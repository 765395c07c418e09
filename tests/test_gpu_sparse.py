"""Block-sparse attention: device-built runs must reproduce the mask exactly; out/LSE must match
dense attention with -inf on the dropped tiles."""
import numpy as np
import pytest
import torch

import paraattention_amd
from paraattention_amd import ops
from oracle import attention as oattn
from oracle import inputs
from oracle import sparse as osparse

pytestmark = pytest.mark.gpu


def _runs_to_mask(count, ranges, nK, kv_lo, kb):
    """Rebuild the boolean mask rows from the device's range lists (segments 1..nQ)."""
    Hm, nseg = count.shape
    out = np.zeros((Hm, nseg - 2, nK), dtype=bool)
    for h in range(Hm):
        for s in range(1, nseg - 1):
            for r in range(count[h, s]):
                b, e = ranges[h, s, r]
                b, e = max(b, kv_lo), min(e, kv_lo + nK * kb)
                if e > b:
                    assert (b - kv_lo) % kb == 0 and (e - kv_lo) % kb == 0
                    out[h, s - 1, (b - kv_lo) // kb : (e - kv_lo) // kb] = True
    return out


@pytest.mark.parametrize("Hm,nQ,nK", [(1, 1, 1), (1, 4, 7), (3, 16, 16), (24, 256, 256)])
def test_runs_reproduce_mask_bit_exact(cuda, Hm, nQ, nK):
    mask, _ = inputs.block_mask(Hm, nQ, nK, seed=nK)
    kb = 128
    count, ranges = ops.block_sparse_runs(mask.to(cuda), Skv=nK * kb)
    count, ranges = count.cpu().numpy(), ranges.cpu().numpy()
    assert np.array_equal(_runs_to_mask(count, ranges, nK, 0, kb), mask.numpy())
    # and the runs are the reference's runs (sparse_attn.py:215-234)
    for h in range(Hm):
        for i in range(nQ):
            want = [(s * kb, e * kb) for s, e in osparse.mask_row_runs(mask[h, i].tolist())]
            got = [tuple(ranges[h, i + 1, r]) for r in range(count[h, i + 1])]
            assert got == want
    assert (count[:, 0] == 1).all() and (count[:, -1] == 1).all()


@pytest.mark.parametrize("Hm,nQ,nK,kb", [(1, 1, 1, 128), (2, 9, 7, 100), (3, 40, 33, 16), (24, 256, 256, 128)])
def test_launch_order_is_longest_list_first(cuda, Hm, nQ, nK, kb):
    mask, _ = inputs.block_mask(Hm, nQ, nK, seed=nQ)
    Skv = nK * kb + 40
    order = ops.block_sparse_launch_order(mask.to(cuda), Skv=Skv, kv_lo=24, kv_hi=24 + nK * kb).cpu().numpy()
    for h in range(Hm):
        want = np.argsort(-mask[h].sum(-1).numpy(), kind="stable")  # falling number of kept key blocks, ties by block number
        assert np.array_equal(order[h], want), h


def test_launch_order_leaves_results_alone(cuda, tuning):
    """Which query block a workgroup takes (knob "sparse_order") changes when a block is computed, not what: the
    same bits either way, with margins, several tiles per block, per-head masks and both head dims."""
    op = torch.ops.para_attn.attention_forward_block_sparse
    rng = np.random.default_rng(11)
    for case, (H, nQ, nK, qb, kb, q_lo, q_tail, kv_lo, kv_tail, D, per_head) in enumerate([
        (3, 12, 10, 128, 128, 0, 0, 0, 0, 128, True), (2, 5, 9, 256, 64, 256, 37, 24, 12, 128, True),
        (2, 7, 6, 128, 100, 128, 50, 8, 0, 64, False), (1, 20, 16, 64, 32, 0, 0, 0, 64, 128, True),
    ]):
        Sq, Skv = q_lo + nQ * qb + q_tail, kv_lo + nK * kb + kv_tail
        bm = torch.from_numpy(rng.random((H if per_head else 1, nQ, nK)) < rng.uniform(0.1, 0.9, size=(1, nQ, 1)))
        bm2 = bm if per_head else bm[0]
        q, k, v = (t.to(cuda) for t in inputs.qkv(1, H, Sq, Skv, D, seed=700 + case))
        args = (q, k, v, bm2.to(cuda), q_lo, q_lo + nQ * qb, kv_lo, kv_lo + nK * kb)
        tuning("sparse_order", 0)
        out0, lse0 = op(*args)
        tuning("sparse_order", 1)
        out1, lse1 = op(*args)
        assert torch.equal(out0, out1) and torch.equal(lse0, lse1), case


def test_runs_word_boundaries(cuda):
    # rows that exercise the 64-block voting words: kept block at bit 63, runs crossing words, all kept, none kept
    nK = 200
    rows = torch.zeros(8, nK, dtype=torch.bool)
    rows[0, 63] = True
    rows[1, 60:70] = True
    rows[2, :] = True
    rows[4, 0] = True; rows[4, 127:129] = True; rows[4, 199] = True
    rows[5, 64:128] = True
    rows[6, 1::2] = True
    rows[7, 63:65] = True; rows[7, 191:193] = True
    count, ranges = ops.block_sparse_runs(rows[None].to(cuda), Skv=nK * 16)
    count, ranges = count.cpu().numpy(), ranges.cpu().numpy()
    for i in range(8):
        want = [(s * 16, e * 16) for s, e in osparse.mask_row_runs(rows[i].tolist())]
        got = [tuple(ranges[0, i + 1, r]) for r in range(count[0, i + 1])]
        assert got == want, i


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("per_head", [False, True])
@pytest.mark.parametrize("qb,kb", [(128, 128), (64, 32), (50, 70), (200, 24)])
def test_small_vs_masked_dense(cuda, per_head, qb, kb, D):
    B, H, nQ, nK = 2, 3, 5, 6
    Sq, Skv = nQ * qb, nK * kb
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=qb + kb)
    mask, _ = inputs.block_mask(H if per_head else 1, nQ, nK, seed=1, window=0, sinks=1, density=0.5)
    bm = mask if per_head else mask[0]
    keep = osparse.expand_block_mask(bm.numpy(), Sq, Skv)
    ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, keep)
    out, lse = torch.ops.para_attn.attention_forward_block_sparse(q.to(cuda), k.to(cuda), v.to(cuda), bm.to(cuda))
    np.testing.assert_allclose(lse.cpu().numpy(), ref_lse, atol=1e-3)
    np.testing.assert_allclose(out.float().cpu().numpy(), ref_out, atol=2e-2, rtol=2e-2)
    if not per_head:
        # the reference's own algorithm (runs + merges) agrees as well
        ref2, _ = osparse.struct_sparse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), bm.numpy())
        np.testing.assert_allclose(out.float().cpu().numpy(), ref2, atol=2e-2, rtol=2e-2)


def test_sparse_ranges_with_dense_margins(cuda):
    # sparse_range_query / sparse_range_key_value: dense margins on both sides (text tokens in video DiTs)
    B, H, D = 1, 2, 128
    Sq, Skv = 37 + 4 * 60 + 19, 20 + 5 * 48 + 33
    q_range, kv_range = (37, 37 + 240), (20, 20 + 240)
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=77)
    bm = torch.tensor([[1, 0, 0, 1, 1], [0, 0, 1, 0, 0], [1, 1, 1, 1, 1], [0, 1, 0, 1, 0]], dtype=torch.bool)
    ref_out, ref_lse = osparse.struct_sparse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), bm.numpy(), None, q_range, kv_range)
    keep = osparse.expand_block_mask(bm.numpy(), Sq, Skv, q_range, kv_range)
    ref_out2, ref_lse2 = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, keep)
    np.testing.assert_allclose(ref_out, ref_out2, atol=1e-9)
    np.testing.assert_allclose(ref_lse, ref_lse2, atol=1e-9)
    out = paraattention_amd.struct_sparse_attn_func(
        q.to(cuda), k.to(cuda), v.to(cuda), sparse_mask=bm, sparse_range_query=q_range, sparse_range_key_value=kv_range
    )
    np.testing.assert_allclose(out.float().cpu().numpy(), ref_out, atol=2e-2, rtol=2e-2)
    with paraattention_amd.StructSparseAttnMode(sparse_mask=bm, sparse_range_query=q_range, sparse_range_key_value=kv_range):
        out2 = torch.nn.functional.scaled_dot_product_attention(q.to(cuda), k.to(cuda), v.to(cuda))
        # the class-wide switch of the reference's mode (sparse_attn.py:679-692): dense attention while it is off
        with paraattention_amd.StructSparseAttnMode.disable():
            assert paraattention_amd.StructSparseAttnMode.disabled
            dense = torch.nn.functional.scaled_dot_product_attention(q.to(cuda), k.to(cuda), v.to(cuda))
        assert not paraattention_amd.StructSparseAttnMode.disabled
    assert torch.equal(out, out2)
    ref_dense, _ = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy())
    np.testing.assert_allclose(dense.float().cpu().numpy(), ref_dense, atol=2e-2, rtol=2e-2)


def test_prebuilt_runs_entry(cuda):
    """A mask that serves many calls is scanned once: attention_forward_block_sparse_runs with the ranges from
    block_sparse_key_runs gives bit for bit what attention_forward_block_sparse gives, for shared and per-head
    masks, with margins, on keys of another content; the mode caches the ranges and follows in-place edits."""
    B, H, D = 1, 3, 128
    Sq, Skv = 16 + 4 * 128 + 40, 24 + 6 * 64 + 8
    q_range, kv_range = (16, 16 + 512), (24, 24 + 384)
    q, k, v = (t.to(cuda) for t in inputs.qkv(B, H, Sq, Skv, D, seed=5))
    g = torch.Generator().manual_seed(9)
    for shape in ((4, 6), (H, 4, 6)):
        bm = torch.rand(shape, generator=g) < 0.5
        bm[..., 0] = True
        want_out, want_lse = torch.ops.para_attn.attention_forward_block_sparse(q, k, v, bm.to(cuda), *q_range, *kv_range)
        runs = torch.ops.para_attn.block_sparse_key_runs(bm.to(cuda), Skv, *kv_range)
        hm = 1 if bm.ndim == 2 else H
        for kk, vv in ((k, v), (v, k)):  # the ranges depend on the mask only
            w_out, w_lse = torch.ops.para_attn.attention_forward_block_sparse(q, kk, vv, bm.to(cuda), *q_range, *kv_range)
            out, lse = torch.ops.para_attn.attention_forward_block_sparse_runs(q, kk, vv, runs, hm, 4, 6, *q_range)
            assert torch.equal(out, w_out) and torch.equal(lse, w_lse)
        with pytest.raises(ValueError):
            torch.ops.para_attn.attention_forward_block_sparse_runs(q, k, v, runs[:10], hm, 4, 6, *q_range)
        # ranges built for a longer key sequence (a longer dense right margin) are cut at the keys there are:
        # the walk never leaves the tensors, and here the cut lists are those of the true length
        longer = torch.ops.para_attn.block_sparse_key_runs(bm.to(cuda), Skv + 200, *kv_range)
        out, lse = torch.ops.para_attn.attention_forward_block_sparse_runs(q, k, v, longer, hm, 4, 6, *q_range)
        assert torch.equal(out, want_out) and torch.equal(lse, want_lse)
    bm = torch.rand((4, 6), generator=g) < 0.5
    bm[:, 0] = True
    with paraattention_amd.StructSparseAttnMode(sparse_mask=bm, sparse_range_query=q_range, sparse_range_key_value=kv_range) as mode:
        cache = mode._sparse["runs_cache"]
        o1 = torch.nn.functional.scaled_dot_product_attention(q, k, v)
        (held,) = cache.values()
        o2 = torch.nn.functional.scaled_dot_product_attention(q, k, v)
        assert next(iter(cache.values())) is held and torch.equal(o1, o2)  # second call: no new scan
        want, _ = torch.ops.para_attn.attention_forward_block_sparse(q, k, v, bm.to(cuda), *q_range, *kv_range)
        assert torch.equal(o1, want)
        bm[1] = ~bm[1]
        bm[1, 0] = True  # edited in place: the version counter moves, the ranges are rebuilt
        o3 = torch.nn.functional.scaled_dot_product_attention(q, k, v)
        want3, _ = torch.ops.para_attn.attention_forward_block_sparse(q, k, v, bm.to(cuda), *q_range, *kv_range)
        assert torch.equal(o3, want3) and len(cache) == 1 and next(iter(cache.values())) is not held
        # a second key length through the same mode: its own entry, and the first one is still there afterwards
        k2, v2 = k[:, :, : kv_range[1]].contiguous(), v[:, :, : kv_range[1]].contiguous()
        o4 = torch.nn.functional.scaled_dot_product_attention(q, k2, v2)
        want4, _ = torch.ops.para_attn.attention_forward_block_sparse(q, k2, v2, bm.to(cuda), *q_range, *kv_range)
        assert torch.equal(o4, want4) and len(cache) == 2
        entries = list(cache.values())
        assert torch.equal(torch.nn.functional.scaled_dot_product_attention(q, k, v), want3)
        assert torch.equal(torch.nn.functional.scaled_dot_product_attention(q, k2, v2), want4)
        assert len(cache) == 2 and all(a is b for a, b in zip(cache.values(), entries))  # both served from the cache


def test_paired_query_blocks(cuda, tuning):
    """Two adjacent 128-row query blocks in one 256-row workgroup over the union of their key ranges (tuning knob
    "sparse_pair"): the same results as one workgroup per block to the kernels' tolerance, and as float64 dense
    attention over the kept tiles; with margins, per-head masks, rows of a pair that keep nothing, key blocks
    smaller than a tile."""
    rng = np.random.default_rng(5)
    op = torch.ops.para_attn.attention_forward_block_sparse
    for case, (H, nQ, nK, kb, q_lo, q_tail, kv_lo, kv_tail, dens, per_head) in enumerate([
        (2, 4, 6, 128, 0, 0, 0, 0, 0.5, True),
        (3, 6, 9, 64, 256, 37, 24, 12, 0.4, True),
        (1, 2, 5, 100, 0, 130, 8, 0, 0.3, False),
        (2, 8, 16, 32, 0, 0, 0, 64, 0.25, True),
        (2, 4, 4, 128, 0, 0, 0, 0, 1.0, False),
    ]):
        Sq, Skv = q_lo + nQ * 128 + q_tail, kv_lo + nK * kb + kv_tail
        bm = torch.from_numpy(rng.random((H if per_head else 1, nQ, nK)) < dens)
        if case == 1:
            bm[:, 3] = False  # the upper block of a pair keeps nothing (margins aside)
        bm2 = bm if per_head else bm[0]
        q, k, v = inputs.qkv(1, H, Sq, Skv, 128, seed=900 + case)
        q_range, kv_range = (q_lo, q_lo + nQ * 128), (kv_lo, kv_lo + nK * kb)
        keep = osparse.expand_block_mask(bm2.numpy(), Sq, Skv, q_range, kv_range)
        ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, keep)
        args = (q.to(cuda), k.to(cuda), v.to(cuda), bm2.to(cuda), *q_range, *kv_range)
        tuning("sparse_pair", 0)
        out0, lse0 = op(*args)
        tuning("sparse_pair", 1)
        out1, lse1 = op(*args)
        tuning("sparse_pair", 0)
        what = f"case {case}"
        got_lse, got_out = lse1.cpu().numpy(), out1.float().cpu().numpy()
        dead = np.isneginf(ref_lse)
        assert (np.isneginf(got_lse) == dead).all(), what
        np.testing.assert_allclose(np.where(dead, 0, got_lse), np.where(dead, 0, ref_lse), atol=1e-3, err_msg=what)
        np.testing.assert_allclose(got_out, np.where(dead[..., None], 0, ref_out), atol=2e-2, rtol=2e-2, err_msg=what)
        assert (np.where(dead, 0, got_lse - lse0.cpu().numpy()) == 0).all() or np.abs(np.where(dead, 0, got_lse - lse0.cpu().numpy())).max() < 1e-4, what
        assert (out1.float() - out0.float()).abs().max().item() <= 2e-2, what


def test_row_without_kept_block(cuda):
    # the reference asserts out on such a row (torch _SDPAMerger.results() with nothing merged);
    # the kernel defines it: out = 0, lse = -inf
    q, k, v = inputs.qkv(1, 1, 256, 256, 128, seed=1)
    bm = torch.tensor([[True, False], [False, False]])
    out, lse = torch.ops.para_attn.attention_forward_block_sparse(q.to(cuda), k.to(cuda), v.to(cuda), bm.to(cuda))
    assert (out[:, :, 128:] == 0).all() and torch.isneginf(lse[:, :, 128:]).all()
    assert torch.isfinite(lse[:, :, :128]).all()


def test_config5_shape_sampled(cuda):
    # the block-sparse benchmark shape: B1 H24 S32768 D128, 128x128 tiles, ~30% density; the oracle checks sampled
    # query blocks of sampled heads by gathering their kept key blocks (torch CPU SDPA)
    B, H, S, D, nb = 1, 24, 32768, 128, 256
    q, k, v = inputs.qkv(B, H, S, S, D, seed=0)
    mask, density = inputs.block_mask(H, nb, nb, seed=0)
    assert 0.28 < density < 0.32
    out, lse = torch.ops.para_attn.attention_forward_block_sparse(q.to(cuda), k.to(cuda), v.to(cuda), mask.to(cuda))
    g = torch.Generator().manual_seed(2)
    for h in (0, 11, 23):
        for i in [0, 255] + torch.randint(1, 255, (4,), generator=g).tolist():
            rows = slice(i * 128, (i + 1) * 128)
            idx = torch.nonzero(mask[h, i]).flatten()
            ks = k[:, h : h + 1].reshape(1, 1, nb, 128, D)[:, :, idx].reshape(1, 1, -1, D)
            vs = v[:, h : h + 1].reshape(1, 1, nb, 128, D)[:, :, idx].reshape(1, 1, -1, D)
            ro, rl = oattn.sdpa_lse_torch_cpu(q[:, h : h + 1, rows], ks, vs)
            np.testing.assert_allclose(lse[:, h : h + 1, rows].cpu().numpy(), rl.numpy(), atol=1e-3)
            np.testing.assert_allclose(out[:, h : h + 1, rows].float().cpu().numpy(), ro.float().numpy(), atol=2e-2, rtol=2e-2)
    assert torch.isfinite(out.float()).all()


def test_config5_shape_every_row_by_closed_forms(cuda):
    """Every row of the benchmark shape, by properties that need no oracle run: with zero keys all kept scores
    are 0, so LSE = ln(number of kept keys) of the row's (head, query block) and out = the mean of V over the kept
    keys; with V constant along the keys out is that constant."""
    B, H, S, D, nb = 1, 24, 32768, 128, 256
    q, k, v = inputs.qkv(B, H, S, S, D, seed=3)
    mask, _ = inputs.block_mask(H, nb, nb, seed=0)
    qd, vd, md = q.to(cuda), v.to(cuda), mask.to(cuda)
    op = torch.ops.para_attn.attention_forward_block_sparse
    out, lse = op(qd, torch.zeros_like(qd), vd, md)
    kept = mask.sum(dim=2).to(torch.float64) * (S // nb)                      # [H, nb] kept keys per query block
    want_lse = torch.log(kept).repeat_interleave(S // nb, dim=1)[None]          # [1, H, S]
    assert (lse.cpu().double() - want_lse).abs().max().item() <= 1e-3
    # mean of V over the kept key blocks: block means [H, nb, D], averaged with the mask row as weights
    blk_mean = vd.float().reshape(B, H, nb, S // nb, D).mean(dim=3)[0]          # [H, nb, D]
    want_out = torch.einsum("hij,hjd->hid", md.float(), blk_mean) / md.float().sum(dim=2, keepdim=True)
    want_out = want_out.repeat_interleave(S // nb, dim=1)[None]                 # [1, H, S, D]
    assert (out.float() - want_out).abs().max().item() <= 2e-2
    c = torch.linspace(-2.0, 2.0, D).bfloat16().to(cuda)
    out_c, _ = op(qd, k.to(cuda), c.expand(B, H, S, D).contiguous(), md)
    assert (out_c.float() - c.float()).abs().max().item() <= 2e-2


def test_random_configurations(cuda):
    """Forty seeded random draws over block sizes, block counts, dense margins, mask density (rows that keep
    nothing included), per-head masks, head_dim and dtype, each against dense attention with -inf on the dropped tiles."""
    rng = np.random.default_rng(77)
    for case in range(40):
        B, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
        D = int(rng.choice([64, 128]))
        dtype = torch.bfloat16 if rng.random() < 0.7 else torch.float16
        nQ, nK = int(rng.integers(1, 7)), int(rng.integers(1, 9))
        qb, kb = int(rng.choice([8, 37, 64, 128, 130, 256])), int(rng.choice([5, 32, 64, 100, 128]))
        q_lo, q_tail = (int(rng.integers(0, 90)), int(rng.integers(0, 90))) if rng.random() < 0.5 else (0, 0)
        kv_lo, kv_tail = (int(rng.integers(0, 90)), int(rng.integers(0, 90))) if rng.random() < 0.5 else (0, 0)
        Sq, Skv = q_lo + nQ * qb + q_tail, kv_lo + nK * kb + kv_tail
        per_head = bool(rng.random() < 0.4)
        dens = float(rng.choice([0.1, 0.3, 0.6, 1.0]))
        bm = torch.from_numpy(rng.random((H if per_head else 1, nQ, nK)) < dens)
        bm2 = bm if per_head else bm[0]
        q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=500 + case, dtype=dtype)
        q_range, kv_range = (q_lo, q_lo + nQ * qb), (kv_lo, kv_lo + nK * kb)
        keep = osparse.expand_block_mask(bm2.numpy(), Sq, Skv, q_range, kv_range)
        ref_out, ref_lse = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, keep)
        out, lse = torch.ops.para_attn.attention_forward_block_sparse(
            q.to(cuda), k.to(cuda), v.to(cuda), bm2.to(cuda), q_range[0], q_range[1], kv_range[0], kv_range[1])
        what = f"case {case}: B{B} H{H} D{D} {dtype} nQ{nQ}x{qb} nK{nK}x{kb} margins q({q_lo},{q_tail}) kv({kv_lo},{kv_tail}) per_head={per_head} density={dens}"
        got_lse = lse.cpu().numpy().astype(np.float64)
        both_inf = np.isneginf(got_lse) & np.isneginf(ref_lse)
        assert (np.isneginf(got_lse) == np.isneginf(ref_lse)).all(), what
        assert (np.abs(np.where(both_inf, 0.0, got_lse - np.where(both_inf, 0.0, ref_lse))) <= 1e-3).all(), what
        err = np.abs(out.float().cpu().numpy().astype(np.float64) - ref_out)
        assert (err <= 2e-2 + 2e-2 * np.abs(ref_out)).all(), what + f" max err {err.max():.4g}"
