"""Pins oracle.sparse: the run scan against brute force over every mask row of up to 8 blocks, and the
reference's run-by-run algorithm against dense attention with -inf on dropped tiles."""
import itertools

import numpy as np
import pytest

from oracle import attention as oattn
from oracle import sparse as osparse


def test_run_scan_exhaustive():
    for n in range(1, 9):
        for bits in itertools.product([False, True], repeat=n):
            runs = osparse.mask_row_runs(list(bits))
            rebuilt = [False] * n
            for s, e in runs:
                assert 0 <= s < e <= n and all(bits[s:e])
                assert (s == 0 or not bits[s - 1]) and (e == n or not bits[e])  # maximal
                for j in range(s, e):
                    assert not rebuilt[j]
                    rebuilt[j] = True
            assert tuple(rebuilt) == bits
            assert runs == sorted(runs)


def test_expand_block_mask():
    bm = np.array([[1, 0, 1], [0, 1, 0]], dtype=bool)
    keep = osparse.expand_block_mask(bm, 2 + 4 + 1, 3 + 6 + 2, (2, 6), (3, 9))
    assert keep.shape == (7, 11)
    assert keep[:2].all() and keep[6:].all()  # dense query margins
    assert keep[:, :3].all() and keep[:, 9:].all()  # dense key margins
    assert np.array_equal(keep[2:4, 3:9], np.repeat(bm[0], 2)[None].repeat(2, 0))
    assert np.array_equal(keep[4:6, 3:9], np.repeat(bm[1], 2)[None].repeat(2, 0))


@pytest.mark.parametrize("ranges", [(None, None), ((3, 11), (2, 14)), ((0, 8), (4, 16)), ((4, 12), (0, 12))])
def test_reference_algorithm_equals_masked_dense(ranges):
    rng = np.random.default_rng(3)
    Sq, Skv, D = 12, 16, 8
    q, k, v = rng.standard_normal((2, 2, Sq, D)), rng.standard_normal((2, 2, Skv, D)), rng.standard_normal((2, 2, Skv, D))
    q_range, kv_range = ranges
    nQ = ((q_range[1] - q_range[0]) if q_range else Sq) // 4
    nK = ((kv_range[1] - kv_range[0]) if kv_range else Skv) // 4
    for trial in range(6):
        bm = rng.random((nQ, nK)) < 0.5
        if not q_range and not kv_range:
            bm[:, 0] |= ~bm.any(1)  # the reference needs >= 1 kept tile per row when there are no margins
        if kv_range == (0, 12) or kv_range is None:
            pass
        keep = osparse.expand_block_mask(bm, Sq, Skv, q_range, kv_range)
        want_o, want_l = oattn.sdpa_lse_f64(q, k, v, None, keep)
        got_o, got_l = osparse.struct_sparse_f64(q, k, v, bm, None, q_range, kv_range)
        np.testing.assert_allclose(got_o, want_o, atol=1e-10)
        np.testing.assert_allclose(got_l, want_l, atol=1e-10)
