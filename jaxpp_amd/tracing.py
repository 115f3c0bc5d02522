"""Symbolic values for tracing one microbatch of the loop body.

The reference traces the user's function into a jaxpr and cuts it at the
``pipeline_yield`` equations (src/jaxpp/core.py:958-1015).  The host here has
no jaxpr: the body is a chain of transformer layers, stage markers and a loss,
recorded as a flat op list by running the user's function on ``Traced``
placeholders.  Clustering that list at the markers gives the same
stage -> layers assignment the reference derives.

What a trace records
  * ``inputs``: the microbatched arrays the body indexes with the loop index
    (``take(x, i, axis)``, the counterpart of the reference's
    ``jnp.take(x, i, axis)`` in ``treduce``, src/jaxpp/training.py:232-235),
    each with its placeholder;
  * ``ops``: ``("layer", spec, params, in_uid, out_uid)``,
    ``("yield", stage_id, name, in_uids, out_uids)``,
    ``("mse", pred_uid, target)`` with ``target`` either ``("input", k)`` - the
    k-th microbatched input - or ``("const", array)``;
  * ``differentiated``: the value ``value_and_grad`` differentiates.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

import numpy as np

_active = None


class MicrobatchIndex:
    """The loop index ``i`` of ``treduce_i``'s body while it is traced."""

    def __repr__(self):
        return "MicrobatchIndex()"


@dataclass
class Trace:
    ops: list = field(default_factory=list)
    inputs: list = field(default_factory=list)    # [(array with the microbatch axis first, Traced)]
    n_values: int = 0
    index: MicrobatchIndex = field(default_factory=MicrobatchIndex)
    differentiated: Any = None                    # Traced scalar, set by value_and_grad

    def fresh(self, shape, producer) -> "Traced":
        self.n_values += 1
        return Traced(self, self.n_values, tuple(shape), producer)

    def add_input(self, x: np.ndarray, axis: int) -> "Traced":
        x = np.moveaxis(np.asarray(x), axis, 0)
        for arr, sym in self.inputs:              # the same array indexed twice is one input
            if (arr.shape, arr.strides, arr.dtype, arr.__array_interface__["data"][0]) == \
                    (x.shape, x.strides, x.dtype, x.__array_interface__["data"][0]):
                return sym
        sym = self.fresh(x.shape[1:], ("input", len(self.inputs)))
        self.inputs.append((x, sym))
        return sym


@dataclass(frozen=True, eq=False)
class Traced:
    """Placeholder for a per-microbatch value of shape ``shape``."""
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
    out = tree_map(lambda v: tr.fresh(v.shape, ("yield", stage_id)) if isinstance(v, Traced) else v,
                   anchor)
    outs = [v for v in tree_leaves(out) if isinstance(v, Traced)]
    tr.ops.append(("yield", stage_id, name, tuple(v.uid for v in leaves),
                   tuple(v.uid for v in outs)))
    return out
