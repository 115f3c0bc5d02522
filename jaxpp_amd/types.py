"""Task vocabulary shared by the schedules and the stage executor.

Mirrors the jax-free part of the reference's ``src/jaxpp/types.py``
(``TaskType`` at types.py:79-96, ``MpmdIdx`` at types.py:36).  The sharding
metadata kept beside them in the reference is out of scope: one GPU executes
one pipeline rank's share.
"""
from __future__ import annotations

from enum import Enum
from typing import NewType

MpmdIdx = NewType("MpmdIdx", int)


class TaskType(Enum):
    """Kind of a schedule slot (reference: types.py:79-96).

    The integer values are part of the C ABI (``jpp_task_kind``)."""

    FWD = 1
    BWD = 2
    BWD_I = 3
    BWD_W = 4

    def __repr__(self):
        return f"{type(self).__name__}.{self.name}"

    @property
    def default_latency(self) -> int:
        # A full backward costs two forward units, every other kind one.
        return 2 if self is TaskType.BWD else 1


#: name prefix per kind (reference: schedules.py:742-752)
TASK_PREFIX = {
    TaskType.FWD: "fwd_",
    TaskType.BWD: "bwd_",
    TaskType.BWD_I: "bwdA_",
    TaskType.BWD_W: "bwdW_",
}
