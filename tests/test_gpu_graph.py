"""The ops are capturable into a HIP graph (no host synchronisation, no allocation outside torch's allocator,
no memset nodes) and every replay reproduces the eager result: replays are interleaved with eager work and
synchronisations, and inputs are rewritten in place between them."""
import pytest
import torch

import paraattention_amd
from oracle import inputs

pytestmark = pytest.mark.gpu


def _eager(q, kb, vb, prev, cur, key_mask, block_mask):
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q, kb[0], vb[0])
    # masked calls: whether the key mask is a prefix is decided on the device, inside the captured work
    mo, ml = torch.ops.para_attn.attention_forward_with_lse(q, kb[0], vb[0], key_mask)
    so = torch.ops.para_attn.attention_forward_sparse_kv(q, kb[0], vb[0], key_mask.expand(-1, -1, q.shape[2], -1))
    ro, rl = paraattention_amd.ring_sweep(q, kb, vb, fused=True)
    uo, ul = paraattention_amd.ring_sweep(q, kb, vb, fused=False)
    wo, wl = paraattention_amd.ring_sweep(q, kb, vb)  # all blocks in one launch
    # block-sparse with the ranges extracted inside the captured work
    bo, bl = torch.ops.para_attn.attention_forward_block_sparse(q[:, :, :1024], kb[0][:, :, :2560], vb[0][:, :, :2560], block_mask)
    ratio = torch.ops.para_attn.fbcache_residual_diff(prev, cur)
    applied = torch.ops.para_attn.fbcache_apply_residual(prev, cur)
    tv = torch.ops.para_attn.taylorseer_value([cur, prev], 2, prev)
    # 500 keys: the kernel for short key sequences (forced on by the test)
    co, cl = torch.ops.para_attn.attention_forward_with_lse(q, kb[1][:, :, :500], vb[1][:, :, :500])
    return [out, lse, ro, rl, uo, ul, ratio, applied, tv, mo, ml, so, wo, wl, bo, bl, co, cl]


def test_graph_replays_match_eager(cuda, tuning):
    tuning("short_keys", 1)
    tuning("stream_dyn", 2)  # the sweep in one launch is long enough for two rounds of tail ranges drawn from a counter, which a small kernel clears
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    B, H, D = 1, 4, 128
    Sq = (cus // H + 2) * 256 - 40  # a grid that takes the key-split tail and its workspace
    q, k, v = inputs.qkv(B, H, Sq, 3 * 2600, D, seed=1)
    q = q.to(cuda)
    kb = [t.contiguous().to(cuda) for t in k.split(2600, 2)]
    vb = [t.contiguous().to(cuda) for t in v.split(2600, 2)]
    prev, cur = (t.to(cuda) for t in inputs.fbcache_pair((1, 700, 512), seed=2))
    key_mask = (torch.arange(2600)[None, None, None, :] < 2000).to(cuda)  # a prefix at capture time
    block_mask = (torch.rand(8, 20, generator=torch.Generator().manual_seed(3)) < 0.5).to(cuda)  # 128-row x 128-key blocks
    _eager(q, kb, vb, prev, cur, key_mask, block_mask)  # warm-up outside capture (library load, function attributes)
    key_mask[..., 5] = False
    _eager(q, kb, vb, prev, cur, key_mask, block_mask)  # and the per-score kernel's
    key_mask[..., 5] = True
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        _eager(q, kb, vb, prev, cur, key_mask, block_mask)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            captured = _eager(q, kb, vb, prev, cur, key_mask, block_mask)
    torch.cuda.synchronize()
    g = torch.Generator().manual_seed(5)
    for rep in range(4):
        if rep:  # new values in the captured input buffers
            q.copy_(torch.randn(q.shape, generator=g).bfloat16())
            kb[1].copy_(torch.randn(kb[1].shape, generator=g).bfloat16())
            cur.copy_((prev.float().cpu() + 0.05 * (rep + 1) * torch.randn(prev.shape, generator=g)).bfloat16())
            # the mask changes between replays: a shorter prefix, then a scattered mask, then a prefix again
            key_mask.copy_(((torch.arange(2600) < 2000 - 300 * rep) ^ (torch.arange(2600) == 7 if rep == 2 else torch.zeros(2600, dtype=torch.bool)))[None, None, None, :])
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = _eager(q, kb, vb, prev, cur, key_mask, block_mask)
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), f"replay {rep}: output {i} differs from the eager run"


def test_graph_replays_of_a_masked_call_whose_mask_changes(cuda):
    """A masked call large enough for the kept keys of a mask with holes to be gathered (3e11 flop), captured once and
    replayed with a prefix mask, a mask with holes, a mask that keeps half of the keys at random and a prefix again:
    which of the enqueued launches run is decided on the device at every replay."""
    B, H, Sq, Skv, D = 1, 8, 9000, 9011, 128
    q, k, v = (t.to(cuda) for t in inputs.qkv(B, H, Sq, Skv, D, seed=3))
    mask = torch.ones(1, 1, 1, Skv, dtype=torch.bool, device=cuda)
    op = torch.ops.para_attn.attention_forward_with_lse
    op(q, k, v, mask)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        op(q, k, v, mask)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            captured = op(q, k, v, mask)
    torch.cuda.synchronize()
    g = torch.Generator().manual_seed(4)
    masks = [torch.arange(Skv) < Skv - 100, (torch.arange(Skv) < Skv - 100) & (torch.arange(Skv) != 77), torch.rand(Skv, generator=g) < 0.5,
             torch.arange(Skv) < 3000]
    for rep, m in enumerate(masks):
        mask.copy_(m[None, None, None, :])
        q.copy_(torch.randn(q.shape, generator=g).bfloat16())
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = op(q, k, v, mask)
        torch.cuda.synchronize()
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), f"replay {rep}"
        kept = m.nonzero()[:, 0].to(cuda)
        ref = op(q, k[:, :, kept], v[:, :, kept])
        assert (got[0].float() - ref[0].float()).abs().max().item() <= 2e-2 and (got[1] - ref[1]).abs().max().item() <= 1e-4, f"replay {rep}"
