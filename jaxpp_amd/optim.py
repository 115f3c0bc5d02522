"""The step behind the loop: the optimizer applied to what ``treduce`` returns.

The reference's train step ends with

    updates, opt_state = optimizer.update(grad, opt_state, pars)
    new_pars = optax.apply_updates(pars, updates)

(README.md:90-93; examples/basic.py:234 builds ``optimizer`` with ``optax.adam``).  ``adam``
here has optax's interface - ``init``, ``update`` - and ``apply_updates`` adds the updates;
both run on the GPU (``jpp_adam_step``, ``jpp_grad_accum_f32``), leaf by leaf over pytrees of
float32 host arrays, in the arithmetic ``optax.adam`` uses: f32 tensors, every scalar formed in
double and rounded once.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from jaxpp_amd import tracing


def _zip_map(f, *trees):
    a = trees[0]
    if isinstance(a, (tuple, list)):
        return type(a)(_zip_map(f, *ts) for ts in zip(*trees))
    if isinstance(a, dict):
        return {k: _zip_map(f, *(t[k] for t in trees)) for k in a}
    return f(*trees)


@dataclass(frozen=True)
class adam:
    """``optax.adam(learning_rate, b1, b2, eps)``: no weight decay, bias-corrected moments."""

    learning_rate: float
    b1: float = 0.9
    b2: float = 0.999
    eps: float = 1e-8

    def init(self, params) -> dict:
        zeros = lambda a: np.zeros(np.shape(a), np.float32)
        return {"count": 0, "mu": tracing.tree_map(zeros, params),
                "nu": tracing.tree_map(zeros, params)}

    def update(self, grads, state: dict, params=None):
        """-> (updates, new state); ``updates = -lr * m_hat / (sqrt(v_hat) + eps)``."""
        from jaxpp_amd import runtime as rt
        rt.require_gpu()
        step = int(state["count"]) + 1

        def leaf(g, m, v):
            g = np.ascontiguousarray(g, dtype=np.float32)
            n = g.size
            dg, dm, dv = (rt.DeviceBuffer.from_numpy(np.ascontiguousarray(a, dtype=np.float32))
                          for a in (g, m, v))
            du = rt.DeviceBuffer(4 * n)
            du.zero()
            # weights that start at zero end as the update itself
            rt.adam_step(n, dg.ptr, dm.ptr, dv.ptr, step, master=du.ptr, lr=self.learning_rate,
                         b1=self.b1, b2=self.b2, eps=self.eps)
            rt.sync()
            return (du.download(np.float32, g.shape), dm.download(np.float32, g.shape),
                    dv.download(np.float32, g.shape))

        trio = _zip_map(leaf, grads, state["mu"], state["nu"])
        pick = lambda k: _zip_map(lambda g, t: t[k], grads, trio)
        return pick(0), {"count": step, "mu": pick(1), "nu": pick(2)}


def apply_updates(params, updates):
    """``optax.apply_updates``: ``params + updates``, leaf by leaf, in f32 on the GPU."""
    from jaxpp_amd import runtime as rt
    rt.require_gpu()

    def leaf(p, u):
        p = np.ascontiguousarray(p, dtype=np.float32)
        dp = rt.DeviceBuffer.from_numpy(p)
        du = rt.DeviceBuffer.from_numpy(np.ascontiguousarray(u, dtype=np.float32))
        rt.check(rt.load().jpp_grad_accum_f32(None, dp.ptr, du.ptr, p.size, 1))
        rt.sync()
        return dp.download(np.float32, p.shape)

    return _zip_map(leaf, params, updates)
