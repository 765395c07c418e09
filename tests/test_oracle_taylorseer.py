"""Pins oracle/taylorseer.py: against torch's CPU eager ops evaluating the reference's expressions
(committed golden vectors and fresh random cases), against closed forms of the extrapolation, and against the
compute/skip schedule written out by hand."""
import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import taylorseer as ots

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "taylorseer_cases.npz")


def _dec(arr, dtype):
    if dtype == "bf16":
        return (arr.astype(np.uint32) << 16).view(np.float32)
    return arr.astype(np.float32)


def golden_cases():
    d = np.load(GOLDEN)
    for c in json.loads(str(d["cases"])):
        name, dt, n = c["name"], c["dtype"], c["n"]
        yield c, {
            "y": _dec(d[name + "_y"], dt), "hidden": _dec(d[name + "_hidden"], dt),
            "prev": [_dec(d[f"{name}_prev{i}"], dt) for i in range(n)],
            "cur": [_dec(d[f"{name}_cur{i + 1}"], dt) for i in range(n)],
            "value": _dec(d[name + "_value"], dt), "applied": _dec(d[name + "_applied"], dt),
        }


def test_golden_vectors_bit_exact():
    seen = 0
    for c, v in golden_cases():
        cur = ots.finite_differences(v["y"], v["prev"], c["window"], c["dtype"])
        for got, want in zip(cur, v["cur"]):
            assert np.array_equal(got, want), c["name"]
        derivs = [v["y"]] + v["cur"]
        assert np.array_equal(ots.extrapolate(derivs, c["elapsed"], c["dtype"]), v["value"]), c["name"]
        assert np.array_equal(ots.extrapolate(derivs, c["elapsed"], c["dtype"], hidden=v["hidden"]), v["applied"]), c["name"]
        seen += 1
    assert seen == 5


@pytest.mark.parametrize("dtype,name", [(torch.bfloat16, "bf16"), (torch.float16, "f16"), (torch.float32, "f32")])
@pytest.mark.parametrize("window,elapsed", [(1, 1), (2, 3), (3, 1), (7, 5)])
def test_matches_torch_eager_chain(dtype, name, window, elapsed):
    g = torch.Generator().manual_seed(window * 10 + elapsed)
    y = (torch.randn(4097, generator=g) * 3).to(dtype)
    prev = [torch.randn(4097, generator=g).to(dtype) for _ in range(3)]
    cur = [y]
    for i in range(3):
        cur.append((cur[i] - prev[i]) / window)
    output = 0
    for i, d in enumerate(cur):
        output += (1 / math.factorial(i)) * d * (elapsed**i)
    f = lambda t: t.float().numpy()  # noqa: E731
    mine = ots.finite_differences(f(y), [f(p) for p in prev], window, name)
    for a, b in zip(mine, cur[1:]):
        assert np.array_equal(a, f(b))
    assert np.array_equal(ots.extrapolate([f(y)] + mine, elapsed, name), f(output))


def test_minus_zero_becomes_plus_zero():
    # output = 0; output += t  ->  0 + (-0.0) = +0.0
    out = ots.extrapolate([np.array([-0.0, 1.0], dtype=np.float32)], 3, "bf16")
    assert not np.signbit(out[0]) and out[1] == 1.0


def test_linear_sequence_is_extrapolated_exactly():
    # y(t) = a + b t: first difference b, second 0, so the prediction at t + e is y(t) + b e (fp32, exact integers)
    a, b = np.array([3.0, -7.0, 0.5], dtype=np.float32), np.array([2.0, 5.0, -1.5], dtype=np.float32)
    ts = ots.TaylorSeer(n_derivatives=2, warmup_steps=3, skip_interval_steps=4, dtype_name="f32")
    for t in range(12):
        out = ts.step(a + b * t)
        np.testing.assert_array_equal(out, a + b * t)  # computed or predicted, the value is exact


def test_quadratic_closed_form():
    # y = t^2, unit window: d1 = 2t - 1, d2 = 2, prediction at t + e = t^2 + (2t - 1) e + e^2 = (t + e)^2 - e
    # (the second difference exists from the fourth computed step on: it needs a stored first difference)
    ts = ots.TaylorSeer(n_derivatives=2, warmup_steps=4, skip_interval_steps=100, dtype_name="f32")
    for t in range(4):
        ts.step(np.array([float(t * t)], dtype=np.float32))
    for e in range(1, 6):
        out = ts.step(np.array([np.nan], dtype=np.float32))  # skipped steps never look at their input
        assert out[0] == (3 + e) ** 2 - e
    # a dropped 1/2 on the second-order term, or e instead of e^2, would give (t+e)^2 + e^2 - e or t^2 + 2te


def test_schedule_by_enumeration():
    ts = ots.TaylorSeer(n_derivatives=2, warmup_steps=2, skip_interval_steps=3)
    # step < 2 -> full; afterwards full when (step - 2 + 1) % 3 == 0: steps 4, 7, 10
    assert [ts.should_compute_full(s) for s in range(12)] == [True, True, False, False, True, False, False, True, False, False, True, False]
    ts = ots.TaylorSeer(compute_step_map=[True, False, True])
    assert [ts.should_compute_full(s) for s in range(3)] == [True, False, True]


def test_orders_appear_one_update_at_a_time():
    # differences need current_step > 1 and a stored previous value of the order below (taylorseer.py:34)
    ts = ots.TaylorSeer(n_derivatives=2, warmup_steps=10, dtype_name="f32")
    counts = []
    for t in range(5):
        ts.step(np.array([float(t**3)], dtype=np.float32))
        counts.append(sum(d is not None for d in ts.state["dY_current"]))
    assert counts == [1, 1, 2, 3, 3]
    # third differences of t^3 with unit steps: d1 = 3t^2 - 3t + 1, d2 = 6t - 6
    assert ts.state["dY_current"][1][0] == 3 * 16 - 12 + 1 and ts.state["dY_current"][2][0] == 18
