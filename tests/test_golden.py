"""Committed golden vectors (tests/golden, written by make_golden.py from torch's CPU routines): the oracle
must reproduce them on the CPU; the GPU half of this file checks the HIP kernels against the same files."""
import os

import numpy as np
import pytest
import torch

from oracle import attention as oattn
from oracle import merge as omerge

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _bf16(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def _t(bits):
    return torch.from_numpy(bits.astype(np.int16)).view(torch.bfloat16)


def test_oracle_reproduces_attention_vectors():
    d = np.load(os.path.join(GOLDEN, "attention_cases.npz"))
    for name in ("a", "b"):
        o, l = oattn.sdpa_lse_f64(_bf16(d[name + "_q"]), _bf16(d[name + "_k"]), _bf16(d[name + "_v"]))
        np.testing.assert_allclose(o, _bf16(d[name + "_out"]), atol=2e-2, rtol=2e-2)
        np.testing.assert_allclose(l, d[name + "_lse"], atol=1e-3)


def test_oracle_reproduces_merge_vectors():
    d = np.load(os.path.join(GOLDEN, "merge_cases.npz"))
    acc_o, acc_l = _bf16(d["out0"]), d["lse0"]
    for i in range(1, 4):
        acc_o, acc_l = omerge.merge_step(acc_o, acc_l, _bf16(d[f"out{i}"]), d[f"lse{i}"])
        np.testing.assert_allclose(acc_o, d[f"acc_out{i}"], rtol=2e-6, atol=2e-6)
        np.testing.assert_allclose(acc_l, d[f"acc_lse{i}"], rtol=1e-6, atol=2e-6)


@pytest.mark.gpu
def test_gpu_attention_vectors(cuda):
    import paraattention_amd  # noqa: F401

    d = np.load(os.path.join(GOLDEN, "attention_cases.npz"))
    for name in ("a", "b"):
        q, k, v = (_t(d[f"{name}_{n}"]).to(cuda) for n in "qkv")
        out, lse = torch.ops.para_attn.attention_forward_with_lse(q, k, v)
        np.testing.assert_allclose(out.float().cpu().numpy(), _bf16(d[name + "_out"]), atol=2e-2, rtol=2e-2)
        np.testing.assert_allclose(lse.cpu().numpy(), d[name + "_lse"], atol=1e-3)


@pytest.mark.gpu
def test_gpu_merge_vectors(cuda):
    import paraattention_amd

    d = np.load(os.path.join(GOLDEN, "merge_cases.npz"))
    m = paraattention_amd.SDPAMerger(True, 2)
    for i in range(4):
        m.step(_t(d[f"out{i}"]).to(cuda), torch.from_numpy(d[f"lse{i}"]).to(cuda))
        if i:
            np.testing.assert_allclose(m._out.cpu().numpy(), d[f"acc_out{i}"], rtol=1e-5, atol=1e-5)
            np.testing.assert_allclose(m._lse.cpu().numpy(), d[f"acc_lse{i}"], rtol=1e-6, atol=2e-6)
    out, lse = m.results()
    assert out.dtype == torch.bfloat16
    np.testing.assert_allclose(out.float().cpu().numpy(), _bf16(d["result_out"]), rtol=8e-3, atol=1e-6)
    np.testing.assert_allclose(lse.cpu().numpy(), d["result_lse"], rtol=1e-6, atol=2e-6)


@pytest.mark.gpu
def test_gpu_fbcache_vectors(cuda):
    import json

    import paraattention_amd  # noqa: F401
    from paraattention_amd import fbcache

    cases = json.load(open(os.path.join(GOLDEN, "fbcache_cases.json")))
    d = np.load(os.path.join(GOLDEN, "fbcache_inputs.npz"))
    for c in cases:
        if c["dtype"] == "bf16":
            prev, cur = _t(d[c["name"] + "_prev"]).to(cuda), _t(d[c["name"] + "_cur"]).to(cuda)
        else:
            prev, cur = torch.from_numpy(d[c["name"] + "_prev"]).to(cuda), torch.from_numpy(d[c["name"] + "_cur"]).to(cuda)
        assert torch.ops.para_attn.fbcache_residual_diff(prev, cur).item() == c["ratio"], c["name"]
        assert fbcache.are_two_tensors_similar(prev, cur, threshold=c["threshold"]) is c["similar"], c["name"]
