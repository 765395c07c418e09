"""Pins oracle.attention without the GPU: closed forms, invariants, brute force on tiny inputs and
torch's CPU SDPA library routine.  Each check is chosen so that a plausible mistake (dropped scale,
wrong log base, transposed operand, mask sign) fails it."""
import math

import numpy as np
import pytest
import torch

from oracle import attention as oattn
from oracle import inputs


def _brute(q, k, v, scale, keep=None):
    """Scalar loops, no shared code with the oracle."""
    Sq, D = q.shape
    Skv, Dv = v.shape
    out = np.zeros((Sq, Dv))
    lse = np.zeros(Sq)
    for i in range(Sq):
        logits = []
        for j in range(Skv):
            if keep is not None and not keep[i, j]:
                continue
            logits.append((j, scale * sum(float(q[i, d]) * float(k[j, d]) for d in range(D))))
        if not logits:
            lse[i] = -math.inf
            continue
        m = max(x for _, x in logits)
        z = sum(math.exp(x - m) for _, x in logits)
        lse[i] = m + math.log(z)
        for j, x in logits:
            w = math.exp(x - m) / z
            for d in range(Dv):
                out[i, d] += w * float(v[j, d])
    return out, lse


@pytest.mark.parametrize("Sq,Skv,D", [(1, 1, 4), (3, 5, 8), (7, 2, 16), (5, 9, 3)])
def test_brute_force_tiny(Sq, Skv, D):
    rng = np.random.default_rng(Sq * 100 + Skv)
    q, k, v = rng.standard_normal((Sq, D)), rng.standard_normal((Skv, D)), rng.standard_normal((Skv, D + 1))
    keep = rng.random((Sq, Skv)) < 0.7
    for kp in (None, keep):
        for scale in (0.37, None):
            sc = scale if scale is not None else 1.0 / math.sqrt(D)
            want_o, want_l = _brute(q, k, v, sc, kp)
            got_o, got_l = oattn.sdpa_lse_f64(q, k, v, scale, kp)
            np.testing.assert_allclose(got_o, want_o, atol=1e-12)
            np.testing.assert_allclose(got_l, want_l, atol=1e-12)


def test_closed_forms():
    rng = np.random.default_rng(0)
    q, k, v = rng.standard_normal((4, 6, 16)), rng.standard_normal((4, 9, 16)), rng.standard_normal((4, 9, 16))
    # K = 0 -> uniform weights: out = mean(V), lse = ln(Skv) (natural log, not log2)
    o, l = oattn.sdpa_lse_f64(q, np.zeros_like(k), v)
    np.testing.assert_allclose(l, math.log(9), atol=1e-12)
    np.testing.assert_allclose(o, np.broadcast_to(v.mean(1, keepdims=True), o.shape), atol=1e-12)
    # V constant -> out = constant
    o, _ = oattn.sdpa_lse_f64(q, k, np.full_like(v, -2.5))
    np.testing.assert_allclose(o, -2.5, atol=1e-12)
    # Skv = 1 -> out = v, lse = scale * q.k
    o, l = oattn.sdpa_lse_f64(q, k[:, :1], v[:, :1], 0.5)
    np.testing.assert_allclose(o, np.broadcast_to(v[:, :1], o.shape), atol=1e-12)
    np.testing.assert_allclose(l, 0.5 * np.einsum("bqd,bd->bq", q, k[:, 0]), atol=1e-12)
    # one dominant key -> out ~ its value, lse ~ its logit
    kd = k.copy()
    kd[:, 3] = 50 * q[:, 0] / np.linalg.norm(q[:, 0], axis=-1, keepdims=True)
    o, l = oattn.sdpa_lse_f64(q[:, :1], kd, v, 1.0)
    np.testing.assert_allclose(o[:, 0], v[:, 3], atol=1e-6)
    # default scale is 1/sqrt(D) (src/para_attn/ops/__init__.py passes scale=None through to aten)
    o1, l1 = oattn.sdpa_lse_f64(q, k, v)
    o2, l2 = oattn.sdpa_lse_f64(q, k, v, 0.25)
    np.testing.assert_allclose(o1, o2, atol=1e-14)
    np.testing.assert_allclose(l1, l2, atol=1e-14)


def test_invariants():
    rng = np.random.default_rng(1)
    q, k, v = rng.standard_normal((2, 5, 8)), rng.standard_normal((2, 11, 8)), rng.standard_normal((2, 11, 8))
    o, l = oattn.sdpa_lse_f64(q, k, v)
    perm = rng.permutation(11)
    o2, l2 = oattn.sdpa_lse_f64(q, k[:, perm], v[:, perm])
    np.testing.assert_allclose(o, o2, atol=1e-12)
    np.testing.assert_allclose(l, l2, atol=1e-12)
    # a masked key is the same as a removed key; a fully masked row gives out 0, lse -inf
    keep = np.ones((2, 5, 11), dtype=bool)
    keep[:, :, 4] = False
    keep[0, 2, :] = False
    o3, l3 = oattn.sdpa_lse_f64(q, k, v, None, keep)
    idx = [j for j in range(11) if j != 4]
    o4, l4 = oattn.sdpa_lse_f64(q, k[:, idx], v[:, idx])
    rows = np.ones((2, 5), dtype=bool)
    rows[0, 2] = False
    np.testing.assert_allclose(o3[rows], o4[rows], atol=1e-12)
    np.testing.assert_allclose(l3[rows], l4[rows], atol=1e-12)
    assert (o3[0, 2] == 0).all() and l3[0, 2] == -np.inf
    # lse is logsumexp of the scaled scores
    s = np.einsum("bqd,bkd->bqk", q, k) / math.sqrt(8)
    np.testing.assert_allclose(l, np.log(np.exp(s).sum(-1)), atol=1e-12)


@pytest.mark.parametrize("shape", [(1, 2, 33, 70, 64), (2, 3, 17, 129, 128), (1, 1, 120, 34, 128)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_matches_torch_cpu_sdpa(shape, dtype):
    """The library routine (torch CPU flash kernel == F.scaled_dot_product_attention on CPU) agrees with the
    closed form within the tolerance the GPU tests use, and its LSE is the natural-log logsumexp."""
    B, H, Sq, Skv, D = shape
    q, k, v = inputs.qkv(B, H, Sq, Skv, D, seed=5, dtype=dtype)
    o64, l64 = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy())
    o, l = oattn.sdpa_lse_torch_cpu(q, k, v)
    assert o.dtype == dtype and l.dtype == torch.float32 and l.shape == (B, H, Sq)
    np.testing.assert_allclose(o.float().numpy(), o64, atol=2e-2, rtol=2e-2)
    np.testing.assert_allclose(l.numpy(), l64, atol=1e-3)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v)
    assert torch.equal(ref, o)
    # boolean and additive masks mean the same thing
    keep = torch.rand(B, 1, Sq, Skv, generator=torch.Generator().manual_seed(0)) < 0.8
    keep[..., 0] = True
    om, lm = oattn.sdpa_lse_torch_cpu(q, k, v, None, keep)
    o64m, l64m = oattn.sdpa_lse_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, keep.numpy())
    np.testing.assert_allclose(om.float().numpy(), o64m, atol=2e-2, rtol=2e-2)
    np.testing.assert_allclose(lm.numpy(), l64m, atol=1e-3)


@pytest.mark.parametrize("Sq,Skv", [(1, 1), (5, 5), (7, 3), (3, 7), (70, 70), (33, 100), (100, 33)])
def test_causal_keep_matches_torch(Sq, Skv):
    """The causal mask: by its definition on tiny cases (row i keeps exactly min(i + 1, Skv) leading keys), against
    torch's own is_causal (CPU SDPA) and against torch's documented construction ones(L, S).tril()."""
    keep = oattn.causal_keep(Sq, Skv)
    assert keep.shape == (Sq, Skv)
    for i in range(Sq):
        n = min(i + 1, Skv)
        assert keep[i, :n].all() and not keep[i, n:].any()
    assert np.array_equal(keep, torch.ones(Sq, Skv, dtype=torch.bool).tril(diagonal=0).numpy())
    g = torch.Generator().manual_seed(Sq * 100 + Skv)
    q, k, v = torch.randn(1, 2, Sq, 32, generator=g), torch.randn(1, 2, Skv, 32, generator=g), torch.randn(1, 2, Skv, 32, generator=g)
    out, lse = oattn.sdpa_lse_f64(q.numpy(), k.numpy(), v.numpy(), None, keep)
    t_out, t_lse = oattn.sdpa_lse_torch_cpu(q, k, v, is_causal=True)
    np.testing.assert_allclose(out, t_out.numpy(), atol=2e-5, rtol=2e-5)
    np.testing.assert_allclose(lse, t_lse.numpy(), atol=2e-5, rtol=2e-5)
