"""TaylorSeer with the reference's interface
(src/para_attn/first_block_cache/taylorseer.py:4-64): the step bookkeeping is the
reference's, the tensor arithmetic of ``approximate_derivative`` and
``approximate_value`` runs as one kernel each instead of one torch launch per
operation.
"""
from . import ops


class TaylorSeer:
    def __init__(self, n_derivatives=2, warmup_steps=1, skip_interval_steps=1, compute_step_map=None):
        if n_derivatives > 4:
            raise NotImplementedError("at most 4 finite-difference orders")
        self.n_derivatives = n_derivatives
        self.ORDER = n_derivatives + 1
        self.warmup_steps = warmup_steps
        self.skip_interval_steps = skip_interval_steps
        self.compute_step_map = compute_step_map
        self.reset_cache()

    def reset_cache(self):
        self.state = {
            "dY_prev": [None] * self.ORDER,
            "dY_current": [None] * self.ORDER,
        }
        self.current_step = -1
        self.last_non_approximated_step = -1

    def should_compute_full(self, step=None):
        """taylorseer.py:21-27."""
        step = self.current_step if step is None else step
        if self.compute_step_map is not None:
            return self.compute_step_map[step]
        if step < self.warmup_steps or (step - self.warmup_steps + 1) % self.skip_interval_steps == 0:
            return True
        return False

    def _usable_orders(self):
        """How many differences approximate_derivative builds (taylorseer.py:33-37): consecutive
        orders whose previous value exists, none before the third step."""
        n = 0
        if self.current_step > 1:
            while n < self.n_derivatives and self.state["dY_prev"][n] is not None:
                n += 1
        return n

    def approximate_derivative(self, Y):
        dY_current = [None] * self.ORDER
        dY_current[0] = Y
        window = self.current_step - self.last_non_approximated_step
        n = self._usable_orders()
        if n:
            dY_current[1 : n + 1] = ops.taylorseer_derivatives(Y, self.state["dY_prev"][:n], float(window))
        return dY_current

    def _stored(self):
        ds = []
        for d in self.state["dY_current"]:
            if d is None:
                break
            ds.append(d)
        return ds

    def approximate_value(self):
        elapsed = self.current_step - self.last_non_approximated_step
        ds = self._stored()
        if not ds:
            return 0  # what the reference's empty sum returns
        return ops.taylorseer_value(ds, elapsed)

    def approximate_value_plus(self, hidden_states):
        """``approximate_value() + hidden_states`` in one pass (the cache-hit path of
        src/para_attn/first_block_cache/utils.py:239-243)."""
        elapsed = self.current_step - self.last_non_approximated_step
        return ops.taylorseer_value(self._stored(), elapsed, hidden_states)

    def mark_step_begin(self):
        self.current_step += 1

    def update(self, Y):
        self.state["dY_prev"] = self.state["dY_current"]
        self.state["dY_current"] = self.approximate_derivative(Y)
        self.last_non_approximated_step = self.current_step

    def step(self, Y):
        self.mark_step_begin()
        if self.should_compute_full():
            self.update(Y)
            return Y
        return self.approximate_value()
