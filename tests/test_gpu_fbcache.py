"""FBCache reduction: the ratio and the hit/miss decision must be bit-exact against the oracle."""
import numpy as np
import pytest
import torch

import paraattention_amd
from paraattention_amd import fbcache
from oracle import fbcache as ofb
from oracle import inputs

pytestmark = pytest.mark.gpu

NAMES = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}


@pytest.mark.parametrize("shape", [(1,), (7,), (1, 33, 40), (2, 257, 129), (1, 3276, 5120)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("noise", [0.05, 0.2])
def test_ratio_bit_exact(cuda, shape, dtype, noise):
    prev, cur = inputs.fbcache_pair(shape, seed=sum(shape), noise=noise, dtype=dtype)
    want, _, _ = ofb.residual_diff_ratio(prev.float().numpy(), cur.float().numpy(), NAMES[dtype])
    got = torch.ops.para_attn.fbcache_residual_diff(prev.to(cuda), cur.to(cuda))
    assert got.dtype == dtype and got.ndim == 0
    if dtype == torch.float32:
        assert abs(got.item() - want) <= 2e-6 * abs(want)  # fp32 means: summation order differs in the last bits
    else:
        assert got.item() == want
    # called again on the same stream: the workspace must have been left clean
    assert torch.ops.para_attn.fbcache_residual_diff(prev.to(cuda), cur.to(cuda)).item() == got.item()


def test_wan_shape_decision(cuda):
    # the Wan 2.1 shape: bf16 [1,32760,5120] pair, threshold 0.12 -> hit; 0.2 noise -> miss
    prev, cur = inputs.fbcache_pair((1, 32760, 5120), seed=1234, noise=0.05)
    want, md, mt = ofb.residual_diff_ratio(prev.float().numpy(), cur.float().numpy())
    got = torch.ops.para_attn.fbcache_residual_diff(prev.to(cuda), cur.to(cuda)).item()
    assert got == want == 0.050048828125 and (md, mt) == (0.039794921875, 0.796875)
    assert fbcache.are_two_tensors_similar(prev.to(cuda), cur.to(cuda), threshold=0.12) is True
    prev, cur = inputs.fbcache_pair((1, 32760, 5120), seed=1234, noise=0.2)
    want, _, _ = ofb.residual_diff_ratio(prev.float().numpy(), cur.float().numpy())
    assert torch.ops.para_attn.fbcache_residual_diff(prev.to(cuda), cur.to(cuda)).item() == want
    assert fbcache.are_two_tensors_similar(prev.to(cuda), cur.to(cuda), threshold=0.12) is False


def test_known_answers(cuda):
    prev, cur = inputs.fbcache_pair((2, 100, 64), seed=3)
    p = prev.to(cuda)
    assert torch.ops.para_attn.fbcache_residual_diff(p, p).item() == 0.0  # identical -> 0 -> similar
    assert fbcache.are_two_tensors_similar(p, p, threshold=1e-9) is True
    z = torch.zeros_like(p)
    assert torch.ops.para_attn.fbcache_residual_diff(p, z).item() == 1.0  # cur = 0 -> ratio 1
    assert fbcache.are_two_tensors_similar(p, z, threshold=0.12) is False
    assert fbcache.are_two_tensors_similar(p, p, threshold=0.0) is False  # utils.py:222-223
    assert fbcache.are_two_tensors_similar(p, p[:, :50], threshold=0.5) is False  # utils.py:225-226


def test_near_threshold_decisions(cuda):
    # thresholds one bf16 step either side of the computed ratio: strict "<" must flip exactly there
    prev, cur = inputs.fbcache_pair((1, 999, 320), seed=8, noise=0.1)
    ratio, _, _ = ofb.residual_diff_ratio(prev.float().numpy(), cur.float().numpy())
    p, c = prev.to(cuda), cur.to(cuda)
    assert fbcache.are_two_tensors_similar(p, c, threshold=ratio) is False
    assert fbcache.are_two_tensors_similar(p, c, threshold=float(np.nextafter(np.float32(ratio), np.float32(1)))) is True
    assert fbcache.are_two_tensors_similar(p, c, threshold=float(np.nextafter(np.float32(ratio), np.float32(0)))) is False


@pytest.mark.parametrize("k", [2, 3, 4])
def test_downsample_and_gates(cuda, k):
    shape = (1, 300, 512)
    prev_full, cur = inputs.fbcache_pair(shape, seed=k, noise=0.08)
    ctx = fbcache.create_cache_context(residual_diff_threshold=0.12, downsample_factor=k, warmup_steps=1)
    with fbcache.cache_context(ctx):
        ctx.mark_step_begin()  # step 0 = warm-up
        assert fbcache.get_can_use_cache(cur.to(cuda)) is False  # warm-up gate, utils.py:271
        fbcache.set_first_hidden_states_residual(prev_full.to(cuda))
        stored = fbcache.get_first_hidden_states_residual()
        assert stored.shape[-1] == len(range(0, 512, k)) and stored.is_contiguous()
        ctx.mark_step_begin()
        want = ofb.get_can_use_cache(prev_full.float().numpy()[..., ::k], cur.float().numpy(), 0.12, downsample_factor=k)
        assert fbcache.get_can_use_cache(cur.to(cuda)) is want
        # ratio itself on the strided view
        r, _, _ = ofb.residual_diff_ratio(prev_full.float().numpy()[..., ::k], cur.float().numpy()[..., ::k])
        assert torch.ops.para_attn.fbcache_residual_diff(stored, cur.to(cuda)[..., ::k]).item() == r
    ctx2 = fbcache.create_cache_context(residual_diff_threshold=0.12)
    with fbcache.cache_context(ctx2):
        ctx2.mark_step_begin()
        assert fbcache.get_can_use_cache(cur.to(cuda)) is False  # no previous residual, utils.py:280


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_first_block_step(cuda, dtype):
    # residual = hidden - hidden0 fused with the reduction; must equal the two-step form bit for bit
    shape = (1, 777, 520)
    g = torch.Generator().manual_seed(5)
    h0 = torch.randn(shape, generator=g).to(dtype)
    prev = torch.randn(shape, generator=g).to(dtype)
    h = (h0.float() + prev.float() + 0.07 * torch.randn(shape, generator=g)).to(dtype)
    resid_ref = (h - h0)  # torch CPU: rounded to dtype
    want, _, _ = ofb.residual_diff_ratio(prev.float().numpy(), resid_ref.float().numpy(), NAMES[dtype])
    resid, ratio = torch.ops.para_attn.fbcache_first_residual_diff(h.to(cuda), h0.to(cuda), prev.to(cuda))
    assert torch.equal(resid.cpu(), resid_ref) and ratio.item() == want
    resid2, ratio2 = torch.ops.para_attn.fbcache_first_residual_diff(h.to(cuda), h0.to(cuda), None)
    assert torch.equal(resid2.cpu(), resid_ref) and ratio2.item() == float("inf")
    applied = torch.ops.para_attn.fbcache_apply_residual(resid, h.to(cuda))
    assert torch.equal(applied.cpu(), resid_ref + h)
    ctx = fbcache.create_cache_context(residual_diff_threshold=0.12)
    with fbcache.cache_context(ctx):
        r1, hit1 = fbcache.first_block_step(h.to(cuda), h0.to(cuda))
        assert hit1 is False and torch.equal(r1.cpu(), resid_ref)
        fbcache.set_first_hidden_states_residual(prev.to(cuda))
        r2, hit2 = fbcache.first_block_step(h.to(cuda), h0.to(cuda))
        assert hit2 is (want < 0.12)
