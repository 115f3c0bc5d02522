"""Symbolic values for tracing one microbatch of the loop body.

The reference traces the user's function into a jaxpr and cuts it at the
``pipeline_yield`` equations (src/jaxpp/core.py:958-1015).  The host here has
no jaxpr: the body is a chain of transformer layers, stage markers and a loss,
recorded as a flat op list by running the user's function on ``Traced``
placeholders.  Clustering that list at the markers gives the same
stage -> layers assignment the reference derives.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

import numpy as np

_active = None


@dataclass
class Trace:
    ops: list = field(default_factory=list)       # ("layer", spec, params) | ("yield", stage, name) | ("mse", scale)
    n_values: int = 0

    def fresh(self, shape, producer) -> "Traced":
        self.n_values += 1
        return Traced(self, self.n_values, tuple(shape), producer)


@dataclass(frozen=True, eq=False)
class Traced:
    """Placeholder for a per-microbatch activation of shape ``shape``."""
    trace: Trace
    uid: int
    shape: tuple
    producer: Any

    def _scalar_op(self, other, what):
        if self.producer is None or self.producer[0] != "mse":
            raise TypeError(f"only a loss value can be {what}; got {self}")
        return self.trace.fresh((), ("mse", self.producer[1] * other if what == "scaled"
                                     else self.producer[1] / other))

    def __truediv__(self, other):
        return self._scalar_op(float(other), "divided")

    def __mul__(self, other):
        return self._scalar_op(float(other), "scaled")

    __rmul__ = __mul__


@dataclass(frozen=True)
class GradOf:
    """Stands for d(loss)/d(parameter leaf) of one microbatch."""
    leaf_id: int
    shape: tuple


def current() -> Trace | None:
    return _active


class tracing:
    def __enter__(self):
        global _active
        if _active is not None:
            raise RuntimeError("nested loop-body traces are not supported")
        _active = Trace()
        return _active

    def __exit__(self, *exc):
        global _active
        _active = None
        return False


def tree_map(f, tree):
    if isinstance(tree, (tuple, list)):
        return type(tree)(tree_map(f, t) for t in tree)
    if isinstance(tree, dict):
        return {k: tree_map(f, v) for k, v in tree.items()}
    return f(tree)


def tree_leaves(tree) -> list:
    out = []
    tree_map(out.append, tree)
    return out


def mark_values(anchor, stage_id: int, name):
    tr = current()
    if tr is None:
        return anchor
    leaves = [v for v in tree_leaves(anchor) if isinstance(v, Traced)]
    if not leaves:
        raise TypeError("mark_stage_end needs at least one traced activation in its anchor")
    tr.ops.append(("yield", stage_id, name))
    return tree_map(lambda v: tr.fresh(v.shape, ("yield", stage_id)) if isinstance(v, Traced) else v,
                    anchor)
