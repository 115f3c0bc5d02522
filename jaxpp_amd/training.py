"""``treduce``: the temporal reduce over microbatches
(reference: src/jaxpp/training.py:106-340).

    state = tree_map(lambda a, op: op.state(n, a), fun(xs[0]), operation)
    for i in range(n):
        state = tree_map(lambda op, s, v: op.update(s, v, i), operation, state, fun(xs[i]))

The loop body is traced once on a symbolic microbatch; under
``mpmd_jit_with_loop`` the traced body is cut at its ``mark_stage_end``
markers, unrolled over the microbatches and executed on the GPU in the order
the schedule's task table dictates (see jaxpp_amd/core.py).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

import numpy as np

from jaxpp_amd import tracing
from jaxpp_amd.pipelining import yield_scope
from jaxpp_amd.schedules import BaseSchedule


@dataclass(frozen=True)
class AddT:
    """Element-wise sum; the accumulator has the dtype of the value
    (reference: training.py:112-123)."""

    def state(self, _: int, a) -> np.ndarray:
        return np.zeros(a.shape, a.dtype)

    def update(self, l, r, _: int):
        return l + r


Add = AddT()


@dataclass(frozen=True)
class Concat:
    """Stacks the per-microbatch values along ``axis``
    (reference: training.py:126-148)."""

    axis: int = 0

    def state(self, n: int, a) -> np.ndarray:
        assert n > 0
        shape = tuple(a.shape[: self.axis]) + (n,) + tuple(a.shape[self.axis:])
        return np.zeros(shape, a.dtype)

    def update(self, state, update, index: int):
        idx = [slice(None)] * state.ndim
        idx[self.axis] = index
        state[tuple(idx)] = update
        return state


@dataclass(frozen=True)
class MaxT:
    """Element-wise maximum (reference: training.py:151-166)."""

    def state(self, _: int, a) -> np.ndarray:
        lo = -np.inf if np.issubdtype(a.dtype, np.floating) else np.iinfo(a.dtype).min
        return np.full(a.shape, lo, a.dtype)

    def update(self, l, r, _: int):
        return np.maximum(l, r)


Max = MaxT()
default_op = (Concat(), Add)


def broadcast_ops(operation, outputs):
    """``operation`` is a prefix tree of ``outputs``: an op standing where the
    outputs have a subtree applies to every leaf below
    (reference: training.py:302-304)."""
    if hasattr(operation, "state") and hasattr(operation, "update"):
        return tracing.tree_map(lambda _: operation, outputs)
    if isinstance(operation, (tuple, list)):
        if not isinstance(outputs, (tuple, list)) or len(operation) != len(outputs):
            raise ValueError("`operation` is not a prefix of the function's output structure")
        return type(outputs)(broadcast_ops(o, v) for o, v in zip(operation, outputs))
    if isinstance(operation, dict):
        return {k: broadcast_ops(operation[k], v) for k, v in outputs.items()}
    raise TypeError(f"unexpected operation {operation!r}")


def take(x, i, axis: int = 0):
    """``x`` at position ``i`` of ``axis`` - ``jnp.take(x, i, axis)`` of the reference's loop
    body (training.py:232-235).  With the loop index of ``treduce_i`` it makes ``x`` a
    microbatched input of the loop and returns its per-microbatch placeholder; with an integer
    it is ``numpy.take``."""
    if isinstance(i, tracing.MicrobatchIndex):
        tr = tracing.current()
        if tr is None or tr.index is not i:
            raise RuntimeError("the loop index is only meaningful while its loop body is traced")
        return tr.add_input(x, axis)
    return np.take(x, i, axis=axis)


def treduce(fun: Callable, xs, schedule: BaseSchedule, axis: int = 0, operation=default_op):
    """Temporally reduces ``fun`` over the microbatch axis of ``xs``, a pytree of arrays
    (signature and meaning as the reference's, training.py:172-239)."""
    flat = tracing.tree_leaves(xs)
    n = flat[0].shape[axis]
    if any(a.shape[axis] != n for a in flat):
        raise AssertionError("Leading dimensions differing among xs")

    def wrap(i):
        return fun(tracing.tree_map(lambda x: take(x, i, axis), xs))

    return treduce_i(wrap, n, schedule=schedule, operation=operation)


def treduce_i(fun: Callable, length: int, schedule: BaseSchedule, operation=default_op):
    """``treduce`` with an explicit length: ``fun(i)`` is the i-th microbatch's value
    (reference: training.py:248-340); the body picks its microbatch with ``take(x, i, axis)``.
    The body is traced once on the symbolic index; every array it indexes must have ``length``
    entries along the indexed axis."""
    from jaxpp_amd import core
    if length <= 0:
        raise ValueError(f"treduce_i: length must be positive, got {length}")
    with tracing.tracing() as tr, yield_scope():
        outputs = fun(tr.index)
    if not tr.inputs:
        raise TypeError("the loop body never indexed an array with the loop index "
                        "(take(x, i, axis)): there is nothing to iterate over")
    for x, _ in tr.inputs:
        if x.shape[0] != length:
            raise AssertionError(f"an array indexed by the loop has {x.shape[0]} entries along "
                                 f"the indexed axis, the loop runs {length} times")
    ops = broadcast_ops(operation, outputs)
    return core.run_loop(tr, outputs, ops, length, schedule)
