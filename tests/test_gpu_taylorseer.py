"""Parity of the TaylorSeer kernels (through torch.ops.para_attn.* -> C ABI) with the oracle: bit-exact, as the
chain is elementwise with torch's own roundings."""
import numpy as np
import pytest
import torch

import paraattention_amd
from oracle import taylorseer as ots
from paraattention_amd import fbcache
from test_oracle_taylorseer import golden_cases

pytestmark = pytest.mark.gpu

TORCH = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}


def _dev(a, dt, cuda):
    return torch.from_numpy(np.ascontiguousarray(a)).to(TORCH[dt]).to(cuda)


def _np(t):
    return t.float().cpu().numpy()


def test_golden_vectors_bit_exact(cuda):
    for c, v in golden_cases():
        dt = c["dtype"]
        y, prev = _dev(v["y"], dt, cuda), [_dev(p, dt, cuda) for p in v["prev"]]
        cur = torch.ops.para_attn.taylorseer_derivatives(y, prev, float(c["window"]))
        for got, want in zip(cur, v["cur"]):
            assert got.dtype == TORCH[dt] and np.array_equal(_np(got), want), c["name"]
        derivs = [y] + list(cur)
        assert np.array_equal(_np(torch.ops.para_attn.taylorseer_value(derivs, c["elapsed"])), v["value"]), c["name"]
        hid = _dev(v["hidden"], dt, cuda)
        assert np.array_equal(_np(torch.ops.para_attn.taylorseer_value(derivs, c["elapsed"], hid)), v["applied"]), c["name"]


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("numel", [1, 7, 8, 4099, 1 << 20])
def test_random_chains_match_oracle(cuda, dt, numel):
    g = torch.Generator().manual_seed(numel)
    mk = lambda s: (torch.randn(numel, generator=g) * s).to(TORCH[dt])  # noqa: E731
    y, prev, hidden = mk(3.0), [mk(2.0), mk(1.0), mk(0.5), mk(0.25)], mk(1.0)
    for n, window, elapsed in [(1, 1, 1), (2, 3, 2), (4, 5, 3)]:
        cur = torch.ops.para_attn.taylorseer_derivatives(y.to(cuda), [p.to(cuda) for p in prev[:n]], float(window))
        ref = ots.finite_differences(_np(y), [_np(p) for p in prev[:n]], window, dt)
        for a, b in zip(cur, ref):
            assert np.array_equal(_np(a), b)
        derivs = [y.to(cuda)] + list(cur)
        assert np.array_equal(_np(torch.ops.para_attn.taylorseer_value(derivs, elapsed)), ots.extrapolate([_np(y)] + ref, elapsed, dt))
        got = torch.ops.para_attn.taylorseer_value(derivs, elapsed, hidden.to(cuda))
        assert np.array_equal(_np(got), ots.extrapolate([_np(y)] + ref, elapsed, dt, hidden=_np(hidden)))


def test_class_follows_the_oracle_class(cuda):
    """A run of the class over 14 steps (computed and skipped ones) against the oracle's class, bit for bit."""
    g = torch.Generator().manual_seed(3)
    kw = dict(n_derivatives=2, warmup_steps=3, skip_interval_steps=3)
    mine, ref = paraattention_amd.TaylorSeer(**kw), ots.TaylorSeer(**kw, dtype_name="bf16")
    base = torch.randn(2, 50, 64, generator=g)
    for t in range(14):
        y = (base * (1 + 0.1 * t) + 0.05 * torch.randn(2, 50, 64, generator=g)).bfloat16()
        out, want = mine.step(y.to(cuda)), ref.step(_np(y))
        assert mine.should_compute_full() == ref.should_compute_full()
        assert np.array_equal(_np(out), want), f"step {t}"


def test_cache_context_taylorseer_path(cuda):
    """set_hidden_states_residual / get_hidden_states_residual / apply_prev_hidden_states_residual with TaylorSeer on
    (src/para_attn/first_block_cache/utils.py:237-243, 297-312)."""
    g = torch.Generator().manual_seed(9)
    ctx = fbcache.create_cache_context(enable_taylorseer=True, taylorseer_kwargs=dict(n_derivatives=1, warmup_steps=2, skip_interval_steps=2))
    ref = ots.TaylorSeer(n_derivatives=1, warmup_steps=2, skip_interval_steps=2, dtype_name="bf16")
    with fbcache.cache_context(ctx):
        assert fbcache.is_taylorseer_enabled()
        for t in range(6):
            ctx.mark_step_begin()
            ref.mark_step_begin()
            r = (torch.randn(1, 33, 40, generator=g) + t).bfloat16()
            h = torch.randn(1, 33, 40, generator=g).bfloat16()
            if fbcache.get_taylorseer().should_compute_full():
                fbcache.set_hidden_states_residual(r.to(cuda))
                ref.update(_np(r))
            else:
                want = ref.approximate_value()
                assert np.array_equal(_np(fbcache.get_hidden_states_residual()), want)
                hs, enc = fbcache.apply_prev_hidden_states_residual(h.to(cuda), "untouched")
                assert enc == "untouched"
                assert np.array_equal(_np(hs), ots.extrapolate([d for d in ref.state["dY_current"] if d is not None],
                                                                ref.current_step - ref.last_non_approximated_step, "bf16", hidden=_np(h)))
        fbcache.set_encoder_hidden_states_residual(h)
        assert fbcache.get_encoder_hidden_states_residual() is None


def test_bad_arguments(cuda):
    y = torch.zeros(16, device=cuda, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        torch.ops.para_attn.taylorseer_derivatives(y, [torch.zeros(8, device=cuda, dtype=torch.bfloat16)], 1.0)
    with pytest.raises(ValueError):
        torch.ops.para_attn.taylorseer_derivatives(y, [y], 0.0)
    with pytest.raises(NotImplementedError):
        torch.ops.para_attn.taylorseer_derivatives(y, [y] * 5, 1.0)
    with pytest.raises(NotImplementedError):
        torch.ops.para_attn.taylorseer_value([y.to(torch.int32)], 1)
