"""TaylorSeer (src/para_attn/first_block_cache/taylorseer.py:4-64) restated over numpy arrays
with torch's eager rounding chain.  Test infrastructure only.

Values are fp32 arrays holding numbers representable in ``dtype_name`` ("bf16", "f16",
"f32"); every tensor operation of the reference is one fp32 operation followed by a rounding
to that type, Python scalars enter as fp32 (torch's op-math type for 16-bit tensors).
"""
import math

import numpy as np

from .bf16 import round_to


def finite_differences(y, prev, window, dtype_name="bf16"):
    """approximate_derivative's loop body (taylorseer.py:33-35) for the orders in ``prev``:
    x0 = y;  x_{i+1} = (x_i - prev[i]) / window.  Returns [x1, ..., xn]."""
    out = []
    x = np.asarray(y, dtype=np.float32)
    w = np.float32(window)
    for p in prev:
        d = round_to(x - np.asarray(p, dtype=np.float32), dtype_name)
        x = round_to(d / w, dtype_name)
        out.append(x)
    return out


def extrapolate(derivs, elapsed, dtype_name="bf16", hidden=None):
    """approximate_value (taylorseer.py:40-48): ``output = 0; output += (1 / i!) * d * elapsed**i``;
    with ``hidden``, followed by ``output + hidden`` (first_block_cache/utils.py:242)."""
    out = None
    for i, d in enumerate(derivs):
        a = round_to(np.float32(1 / math.factorial(i)) * np.asarray(d, dtype=np.float32), dtype_name)
        t = round_to(a * np.float32(elapsed**i), dtype_name)
        out = round_to(np.float32(0) + t, dtype_name) if out is None else round_to(out + t, dtype_name)
    if hidden is not None:
        out = round_to(out + np.asarray(hidden, dtype=np.float32), dtype_name)
    return out


class TaylorSeer:
    """The reference class (taylorseer.py:4-64) over the two functions above."""

    def __init__(self, n_derivatives=2, warmup_steps=1, skip_interval_steps=1, compute_step_map=None, dtype_name="bf16"):
        self.n_derivatives = n_derivatives
        self.ORDER = n_derivatives + 1
        self.warmup_steps = warmup_steps
        self.skip_interval_steps = skip_interval_steps
        self.compute_step_map = compute_step_map
        self.dtype_name = dtype_name
        self.reset_cache()

    def reset_cache(self):
        self.state = {"dY_prev": [None] * self.ORDER, "dY_current": [None] * self.ORDER}
        self.current_step = -1
        self.last_non_approximated_step = -1

    def should_compute_full(self, step=None):  # taylorseer.py:21-27
        step = self.current_step if step is None else step
        if self.compute_step_map is not None:
            return self.compute_step_map[step]
        return step < self.warmup_steps or (step - self.warmup_steps + 1) % self.skip_interval_steps == 0

    def approximate_derivative(self, Y):  # taylorseer.py:29-38
        cur = [None] * self.ORDER
        cur[0] = np.asarray(Y, dtype=np.float32)
        window = self.current_step - self.last_non_approximated_step
        prev = []
        for i in range(self.n_derivatives):
            if self.state["dY_prev"][i] is not None and self.current_step > 1:
                prev.append(self.state["dY_prev"][i])
            else:
                break
        for i, d in enumerate(finite_differences(cur[0], prev, window, self.dtype_name)):
            cur[i + 1] = d
        return cur

    def approximate_value(self):  # taylorseer.py:40-48
        elapsed = self.current_step - self.last_non_approximated_step
        ds = []
        for d in self.state["dY_current"]:
            if d is None:
                break
            ds.append(d)
        return extrapolate(ds, elapsed, self.dtype_name)

    def mark_step_begin(self):
        self.current_step += 1

    def update(self, Y):  # taylorseer.py:53-56
        self.state["dY_prev"] = self.state["dY_current"]
        self.state["dY_current"] = self.approximate_derivative(Y)
        self.last_non_approximated_step = self.current_step

    def step(self, Y):  # taylorseer.py:58-64
        self.mark_step_begin()
        if self.should_compute_full():
            self.update(Y)
            return np.asarray(Y, dtype=np.float32)
        return self.approximate_value()
