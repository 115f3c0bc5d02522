"""``mark_stage_end``: the stage-boundary marker
(reference: src/jaxpp/pipelining.py:25-81).

Inside a ``yield_scope`` (opened by ``treduce`` while it traces the loop body)
each call tags its anchor with the next stage id, counting from 0; outside it
is the identity, exactly as in the reference.  The marker is linear: the
backward of stage k's marker is the boundary at which stage k's backward
receives its cotangent (src/jaxpp/jax_primitives.py:546-554).
"""
from __future__ import annotations

import warnings
from contextlib import contextmanager
from typing import Any

_current_stage = None


@contextmanager
def yield_scope(enabled: bool = True):
    global _current_stage
    prev = _current_stage
    _current_stage = 0 if enabled else None
    try:
        yield
    finally:
        _current_stage = prev


def mark_stage_end(anchor: Any, name: str | None = None) -> Any:
    """Marks the end of a pipeline stage at ``anchor`` (a traced value or a
    pytree - tuple / list / dict - of them) and returns a pytree of the same
    structure."""
    global _current_stage
    if _current_stage is None:
        return anchor
    stage_id = _current_stage
    _current_stage += 1
    from jaxpp_amd.tracing import mark_values
    return mark_values(anchor, stage_id, name)


def pipeline_enter_stage(anchor: Any, name: str | None = None) -> Any:
    warnings.warn("pipeline_enter_stage is deprecated, use mark_stage_end instead.",
                  DeprecationWarning, stacklevel=2)
    return mark_stage_end(anchor, name)
