"""Pins oracle.fbcache against torch's eager bf16/fp16 op chain on CPU (the seven ops of the reference's
are_two_tensors_similar, src/para_attn/first_block_cache/utils.py:228-233), on the committed golden
vectors, on near-threshold cases and on the decision table of get_can_use_cache (utils.py:269-286)."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import fbcache as ofb
from oracle import inputs
from oracle.bf16 import round_bf16

NAMES = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _torch_chain(t1, t2):
    mean_diff = (t1 - t2).abs().mean()
    mean_t1 = t1.abs().mean()
    return (mean_diff / mean_t1).item(), mean_diff.item(), mean_t1.item()


def test_round_bf16_matches_torch():
    x = torch.randn(100000, generator=torch.Generator().manual_seed(0)) * 37
    x = torch.cat([x, torch.tensor([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, 1e-40, float("inf")])])
    assert np.array_equal(round_bf16(x.numpy()), x.bfloat16().float().numpy())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(5,), (1, 33, 40), (2, 257, 129), (1, 2000, 512)])
@pytest.mark.parametrize("noise", [0.03, 0.12, 0.5])
def test_ratio_equals_torch_chain(dtype, shape, noise):
    prev, cur = inputs.fbcache_pair(shape, seed=len(shape) * 7 + int(noise * 100), noise=noise, dtype=dtype)
    want = _torch_chain(prev, cur)
    got = ofb.residual_diff_ratio(prev.float().numpy(), cur.float().numpy(), NAMES[dtype])
    if dtype == torch.float32:
        np.testing.assert_allclose(got, want, rtol=3e-6)  # fp32 means: torch's summation order is its own
    else:
        assert got == want


def test_near_threshold_sweep():
    """Many noise levels close to 0.12: the decision must equal torch's for every one of them."""
    agree = 0
    for i in range(60):
        noise = 0.114 + 0.0002 * i  # ratios around 0.114 .. 0.126 (the ratio is about the noise level)
        prev, cur = inputs.fbcache_pair((1, 700, 64), seed=i, noise=noise)
        r_t = _torch_chain(prev, cur)[0]
        r_o = ofb.residual_diff_ratio(prev.float().numpy(), cur.float().numpy())[0]
        assert r_o == r_t
        assert ofb.are_two_tensors_similar(prev.float().numpy(), cur.float().numpy(), 0.12) == (r_t < 0.12)
        agree += r_t < 0.12
    assert 0 < agree < 60  # the sweep really straddles the threshold


def test_golden_vectors():
    with open(os.path.join(GOLDEN, "fbcache_cases.json")) as f:
        cases = json.load(f)
    data = np.load(os.path.join(GOLDEN, "fbcache_inputs.npz"))
    assert len(cases) >= 8
    for c in cases:
        prev = data[c["name"] + "_prev"].astype(np.float32)
        cur = data[c["name"] + "_cur"].astype(np.float32)
        if c["dtype"] == "bf16":  # stored as raw bf16 bit patterns
            prev = (data[c["name"] + "_prev"].astype(np.uint32) << 16).view(np.float32)
            cur = (data[c["name"] + "_cur"].astype(np.uint32) << 16).view(np.float32)
        got = ofb.residual_diff_ratio(prev, cur, c["dtype"])
        assert got == (c["ratio"], c["mean_diff"], c["mean_t1"]), c["name"]
        assert ofb.are_two_tensors_similar(prev, cur, c["threshold"], c["dtype"]) is c["similar"], c["name"]


def test_decision_table():
    prev, cur = inputs.fbcache_pair((2, 50, 64), seed=9, noise=0.05)
    p, c = prev.float().numpy(), cur.float().numpy()
    assert ofb.are_two_tensors_similar(p, c, 0.0) is False  # utils.py:222-223
    assert ofb.are_two_tensors_similar(p, c, -1.0) is False
    assert ofb.are_two_tensors_similar(p, c[:, :25], 0.5) is False  # shape mismatch, utils.py:225-226
    assert ofb.are_two_tensors_similar(p, p, 1e-9) is True  # identical -> ratio 0
    assert ofb.residual_diff_ratio(p, np.zeros_like(p))[0] == 1.0  # t2 = 0 -> ratio 1
    assert ofb.are_two_tensors_similar(p, np.zeros_like(p), 0.12) is False
    assert ofb.get_can_use_cache(p, c, 0.12, in_warmup=True) is False  # utils.py:271
    assert ofb.get_can_use_cache(None, c, 0.12) is False  # utils.py:280
    assert ofb.get_can_use_cache(p, c, 0.0) is False  # utils.py:273-275
    assert ofb.get_can_use_cache(p, c, 0.12) is True
    # down-sampling: the fresh residual is sliced [..., ::k], the stored one already is (utils.py:276-278, 289-295)
    k = 4
    want = _torch_chain(prev[..., ::k].contiguous(), cur[..., ::k])[0] < 0.12
    assert ofb.get_can_use_cache(p[..., ::k], c, 0.12, downsample_factor=k) is want


def test_wan_row_slice_known_answer():
    """A 1/16 row slice of the Wan 2.1 shape (the full [1,32760,5120] pair is checked in the GPU suite,
    where the host has the memory bandwidth for it): torch's chain and the oracle agree to the bit."""
    prev, cur = inputs.fbcache_pair((1, 2048, 5120), seed=1234, noise=0.05)
    got = ofb.residual_diff_ratio(prev.float().numpy(), cur.float().numpy())
    assert got == _torch_chain(prev, cur)
    assert abs(got[0] - 0.05) < 1e-3 and ofb.are_two_tensors_similar(prev.float().numpy(), cur.float().numpy(), 0.12)
