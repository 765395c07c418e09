"""The ops are capturable into a HIP graph (no host synchronisation, no allocation outside torch's allocator,
no memset nodes) and every replay reproduces the eager result: replays are interleaved with eager work and
synchronisations, and inputs are rewritten in place between them."""
import pytest
import torch

import paraattention_amd
from oracle import inputs

pytestmark = pytest.mark.gpu


def _eager(q, kb, vb, prev, cur):
    out, lse = torch.ops.para_attn.attention_forward_with_lse(q, kb[0], vb[0])
    ro, rl = paraattention_amd.ring_sweep(q, kb, vb, fused=True)
    uo, ul = paraattention_amd.ring_sweep(q, kb, vb, fused=False)
    ratio = torch.ops.para_attn.fbcache_residual_diff(prev, cur)
    applied = torch.ops.para_attn.fbcache_apply_residual(prev, cur)
    tv = torch.ops.para_attn.taylorseer_value([cur, prev], 2, prev)
    return [out, lse, ro, rl, uo, ul, ratio, applied, tv]


def test_graph_replays_match_eager(cuda):
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    B, H, D = 1, 4, 128
    Sq = (cus // H + 2) * 256 - 40  # a grid that takes the key-split tail and its workspace
    q, k, v = inputs.qkv(B, H, Sq, 3 * 2600, D, seed=1)
    q = q.to(cuda)
    kb = [t.contiguous().to(cuda) for t in k.split(2600, 2)]
    vb = [t.contiguous().to(cuda) for t in v.split(2600, 2)]
    prev, cur = (t.to(cuda) for t in inputs.fbcache_pair((1, 700, 512), seed=2))
    _eager(q, kb, vb, prev, cur)  # warm-up outside capture (library load, function attributes)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        _eager(q, kb, vb, prev, cur)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            captured = _eager(q, kb, vb, prev, cur)
    torch.cuda.synchronize()
    g = torch.Generator().manual_seed(5)
    for rep in range(4):
        if rep:  # new values in the captured input buffers
            q.copy_(torch.randn(q.shape, generator=g).bfloat16())
            kb[1].copy_(torch.randn(kb[1].shape, generator=g).bfloat16())
            cur.copy_((prev.float().cpu() + 0.05 * (rep + 1) * torch.randn(prev.shape, generator=g)).bfloat16())
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = _eager(q, kb, vb, prev, cur)
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), f"replay {rep}: output {i} differs from the eager run"
