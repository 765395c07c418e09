"""Pins oracle.merge: torch's own _SDPAMerger (the code the reference calls), the logaddexp closed form,
identity on an empty partial, and split-KV attention + merge == full attention."""
import numpy as np
import pytest
import torch

from oracle import attention as oattn
from oracle import merge as omerge


def _rand_partials(n, shape, seed):
    g = torch.Generator().manual_seed(seed)
    outs = [torch.randn(*shape, generator=g) for _ in range(n)]
    lses = [torch.randn(*shape[:-1], generator=g) * 4 for _ in range(n)]
    return outs, lses


@pytest.mark.parametrize("n", [2, 3, 8])
def test_against_torch_sdpa_merger(n):
    from torch.distributed.tensor.experimental._context_parallel._attention import _SDPAMerger

    outs, lses = _rand_partials(n, (2, 3, 17, 16), n)
    m = _SDPAMerger(True, 2)
    for o, l in zip(outs, lses):
        m.step(o.bfloat16(), l, False)
    ro, rl = m.results()
    go, gl = omerge.merge_all([o.bfloat16().float().numpy() for o in outs], [l.numpy() for l in lses])
    np.testing.assert_allclose(gl, rl.numpy(), rtol=1e-6, atol=1e-6)
    # torch casts the fp32 result back to bf16 in results(); compare before that cast within one bf16 ulp
    np.testing.assert_allclose(go, ro.float().numpy(), rtol=8e-3, atol=1e-6)


def test_closed_form_and_symmetry():
    outs, lses = _rand_partials(2, (1, 2, 9, 8), 0)
    a, b = outs[0].double().numpy(), outs[1].double().numpy()
    la, lb = lses[0].double().numpy(), lses[1].double().numpy()
    o, l = omerge.merge_step(a, la, b, lb, dtype=np.float64)
    want_l = np.logaddexp(la, lb)
    want_o = (np.exp(la - want_l)[..., None] * a) + (np.exp(lb - want_l)[..., None] * b)
    np.testing.assert_allclose(l, want_l, atol=1e-12)
    np.testing.assert_allclose(o, want_o, atol=1e-12)
    o2, l2 = omerge.merge_step(b, lb, a, la, dtype=np.float64)  # commutative
    np.testing.assert_allclose(o, o2, atol=1e-12)
    np.testing.assert_allclose(l, l2, atol=1e-12)


def test_empty_partial_is_identity():
    outs, lses = _rand_partials(1, (1, 1, 5, 8), 1)
    a, la = outs[0].numpy(), lses[0].numpy()
    ninf = np.full_like(la, -np.inf)
    o, l = omerge.merge_step(a, la, np.zeros_like(a), ninf)
    assert np.array_equal(o, a) and np.array_equal(l, la)
    o, l = omerge.merge_step(np.zeros_like(a), ninf, a, la)
    assert np.array_equal(o, a) and np.array_equal(l, la)


def test_split_kv_plus_merge_equals_full():
    rng = np.random.default_rng(0)
    q, k, v = rng.standard_normal((1, 2, 7, 8)), rng.standard_normal((1, 2, 40, 8)), rng.standard_normal((1, 2, 40, 8))
    full_o, full_l = oattn.sdpa_lse_f64(q, k, v)
    cuts = [0, 5, 6, 23, 40]  # ragged blocks, ring order = block after block
    parts = [oattn.sdpa_lse_f64(q, k[:, :, a:b], v[:, :, a:b]) for a, b in zip(cuts[:-1], cuts[1:])]
    o, l = omerge.merge_all([p[0] for p in parts], [p[1] for p in parts], dtype=np.float64)
    np.testing.assert_allclose(o, full_o, atol=1e-12)
    np.testing.assert_allclose(l, full_l, atol=1e-12)
