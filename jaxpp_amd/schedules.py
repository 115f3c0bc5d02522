"""Pipeline schedules: per-rank task tables, bit-exact with the reference.

Behavioural restatement of the reference's ``src/jaxpp/schedules.py`` in a
row-wise, closed-form style: every ``tasks(n)`` builds one rank's row at a
time from the slot ranges the reference fills step by step.  The public names,
constructor arguments, validation messages and the tables themselves
(including the ``None`` bubble slots) are identical; each class cites the
reference lines it follows.

A table is ``list[list[Task | FusedTask | None]]``: one list per pipeline
rank, whose entries are executed in order by that rank.
"""
from __future__ import annotations

import dataclasses
import os
from abc import ABCMeta, abstractmethod
from collections import defaultdict
from dataclasses import dataclass, field
from typing import Any, Iterable, Sequence

from jaxpp_amd.types import TASK_PREFIX, MpmdIdx, TaskType

__all__ = [
    "Task", "FusedTask", "ScheduleTasks", "BaseSchedule",
    "InterleavedBaseSchedule", "Std1F1B", "Eager1F1B", "GPipe", "ZeroBubble",
    "Interleaved1F1B", "KimiK2", "DualPipeV", "dualpipev_tasks",
    "preprocess_schedule_tasks", "schedule_task_fusion_disabled",
    "check_and_strip_adjecent_bwd_a_bwd_w",
    "strip_nones", "unpack_fused_tasks_fn", "mk_task_name",
]


def mk_task_name(stage_id, ty: TaskType, mubatch_idx: int | None = None) -> str:
    """``fwd_3``, ``bwdA_1__7`` ... (reference: schedules.py:742-752)."""
    tail = "" if mubatch_idx is None else f"__{mubatch_idx}"
    return f"{TASK_PREFIX[ty]}{stage_id}{tail}"


@dataclass(frozen=True)
class Task:
    """One (stage, microbatch, kind) unit of work (reference: schedules.py:25-45).

    ``latency`` takes no part in equality or hashing, so a first-stage
    backward whose W half was merged into it still equals the plain task."""

    stage_id: int
    mubatch_idx: int
    fwd_or_bwd: TaskType
    latency: int = field(hash=False, compare=False)

    @classmethod
    def make(cls, stage_id: int, mubatch_idx: int, fwd_or_bwd: TaskType,
             latency: int | None = None) -> "Task":
        return cls(stage_id, mubatch_idx, fwd_or_bwd,
                   fwd_or_bwd.default_latency if latency is None else latency)

    def __str__(self) -> str:
        return mk_task_name(self.stage_id, self.fwd_or_bwd, self.mubatch_idx)


class FusedTask(tuple):
    """Tasks issued as one unit (reference: schedules.py:48-54)."""

    @property
    def latency(self) -> int:
        return sum(t.latency for t in self)

    def __str__(self) -> str:
        return f"FusedTask({', '.join(map(str, self))})"


ScheduleTasks = list  # list[list[Task | FusedTask | None]]

_F, _B, _BI, _BW = TaskType.FWD, TaskType.BWD, TaskType.BWD_I, TaskType.BWD_W


class _Dispenser:
    """Hands out microbatch indices in ascending order per (stage, kind)
    (reference: schedules.py:64-97)."""

    def __init__(self, split_backward: bool = False):
        self.issued: dict = defaultdict(int)
        self.split_backward = split_backward

    def take(self, stage: int, kind: TaskType) -> Task:
        mb = self.issued[stage, kind]
        self.issued[stage, kind] = mb + 1
        return Task.make(stage, mb, kind)

    def fwd(self, stage: int) -> Task:
        return self.take(stage, _F)

    def bwd_a(self, stage: int) -> Task:
        return self.take(stage, _BI)

    def bwd_w(self, stage: int) -> Task:
        return self.take(stage, _BW)

    def bwd(self, stage: int):
        if self.split_backward:
            return FusedTask((self.bwd_a(stage), self.bwd_w(stage)))
        return self.take(stage, _B)

    def fwd_bwd(self, fwd_stage: int, bwd_stage: int) -> FusedTask:
        back = self.bwd(bwd_stage)
        back = (back,) if isinstance(back, Task) else tuple(back)
        return FusedTask((self.fwd(fwd_stage),) + back)


# ---------------------------------------------------------------------------
# base classes
# ---------------------------------------------------------------------------
@dataclass(eq=True, frozen=True)
class BaseSchedule(metaclass=ABCMeta):
    """reference: schedules.py:195-218"""

    num_stages: int
    is_partial_bwd: bool = field(default=False, init=False)

    def __post_init__(self):
        if self.num_stages <= 0:
            # message text as in the reference (schedules.py:200-202)
            raise ValueError("The argument `num_stages` must be `>= 0`")

    def get_mpmd_idx(self, stage_id: int) -> MpmdIdx:
        return MpmdIdx(stage_id)

    @abstractmethod
    def tasks(self, n_mubatches: int) -> ScheduleTasks:
        raise NotImplementedError


@dataclass(eq=True, frozen=True)
class InterleavedBaseSchedule(BaseSchedule):
    """Several stages per rank, round-robin (reference: schedules.py:221-236)."""

    mpmd_dim: int

    def __post_init__(self):
        super().__post_init__()
        if self.mpmd_dim <= 0:
            raise ValueError("The argument `mpmd_dim` must be `>= 0`")
        if self.num_stages % self.mpmd_dim:
            raise ValueError(
                f"{self.num_stages=} can not be evenly divided by {self.mpmd_dim=}. "
                f"Remainder: {divmod(self.num_stages, self.mpmd_dim)=}"
            )

    def get_mpmd_idx(self, stage_id: int) -> MpmdIdx:
        return MpmdIdx(stage_id % self.mpmd_dim)


# ---------------------------------------------------------------------------
# non-interleaved schedules: one stage per rank, tables with bubble slots
# ---------------------------------------------------------------------------
def _one_f_one_b_row(stage: int, n_stages: int, n: int, n_warm_cols: int) -> list:
    """Row of a 1F1B-style table.

    Forwards fill columns ``stage .. stage+n_warm_cols-1``; from column
    ``2*n_stages-1-stage`` on, slots alternate BWD, FWD, BWD, ... and a slot
    whose kind has run out of microbatches stays ``None``."""
    width = 2 * (n + n_stages - 1)
    row: list = [None] * width
    issued = {_F: 0, _B: 0}

    def put(col: int, kind: TaskType):
        if issued[kind] < n:
            row[col] = Task.make(stage, issued[kind], kind)
            issued[kind] += 1

    for col in range(stage, stage + n_warm_cols):
        put(col, _F)
    first_back = 2 * n_stages - 1 - stage
    for col in range(first_back, width):
        put(col, _B if (col - first_back) % 2 == 0 else _F)
    return row


@dataclass(eq=True, frozen=True)
class Std1F1B(BaseSchedule):
    """Warm-up of ``num_stages - stage`` forwards, then one backward per
    forward (reference: schedules.py:239-273)."""

    def tasks(self, n_mubatches: int) -> ScheduleTasks:
        S = self.num_stages
        return [_one_f_one_b_row(s, S, n_mubatches, S - s) for s in range(S)]


@dataclass(eq=True, frozen=True)
class Eager1F1B(BaseSchedule):
    """1F1B whose warm-up runs ``2*(num_stages-stage)-1`` forwards, right up
    to the stage's first backward slot (reference: schedules.py:276-312)."""

    def tasks(self, n_mubatches: int) -> ScheduleTasks:
        S = self.num_stages
        return [_one_f_one_b_row(s, S, n_mubatches, 2 * (S - s) - 1)
                for s in range(S)]


@dataclass(eq=True, frozen=True)
class GPipe(BaseSchedule):
    """All forwards, then all backwards (reference: schedules.py:315-343)."""

    def tasks(self, n_mubatches: int) -> ScheduleTasks:
        S, n = self.num_stages, n_mubatches
        half = n + S - 1
        table = []
        for s in range(S):
            row: list = [None] * (2 * half)
            for mb in range(n):
                row[s + mb] = Task.make(s, mb, _F)
                row[half + (S - 1 - s) + mb] = Task.make(s, mb, _B)
            table.append(row)
        return table


@dataclass(eq=True, frozen=True)
class ZeroBubble(BaseSchedule):
    """ZB-H1 style table with the backward split into BWD_I and BWD_W
    (reference: schedules.py:346-446)."""

    def __post_init__(self):
        super().__post_init__()
        object.__setattr__(self, "is_partial_bwd", True)

    def tasks(self, n_mubatches: int) -> ScheduleTasks:
        return self.build_schedule(n_mubatches)

    def build_schedule(self, n_mubatches: int) -> ScheduleTasks:
        S, n = self.num_stages, n_mubatches
        assert n >= S, (
            f"Expect num of microbatches >= num of stages, but {n} "
            f"microbatches and {S} stages found")
        if S == 1:
            # The reference reads a variable that only its warm-up loop binds,
            # and that loop has no iteration for a single stage
            # (schedules.py:439); the failure mode is kept.
            raise UnboundLocalError(
                "local variable 'next_kind' referenced before assignment")
        width = 3 * n + S - 1
        rotation = (_BI, _BW, _F)
        table = []
        for s in range(S):
            row: list = [None] * width
            issued = {_F: 0, _BI: 0, _BW: 0}

            def put(col: int, kind: TaskType):
                row[col] = Task.make(s, issued[kind], kind)
                issued[kind] += 1

            for col in range(s, S):                       # forwards only
                put(col, _F)
            lo = 2 * S - 1 - s
            for col in range(lo, lo + 2 * s):             # BI, F, BI, F ...
                put(col, _BI if (col - lo) % 2 == 0 else _F)
            at = 0                                        # BI -> BW -> F
            for col in range(lo + 2 * s, width):
                for _ in range(3):
                    kind = rotation[at]
                    at = (at + 1) % 3
                    if issued[kind] < n:
                        put(col, kind)
                        break
                else:
                    raise ValueError(
                        "All tasks have been already scheduled for all mubatches")
            table.append(row)
        return table


# ---------------------------------------------------------------------------
# interleaved schedules: dense per-rank lists, no bubble slots
# ---------------------------------------------------------------------------
@dataclass(eq=True, frozen=True)
class Interleaved1F1B(InterleavedBaseSchedule):
    """Interleaved 1F1B over ``vp = num_stages / mpmd_dim`` chunks per rank
    (reference: schedules.py:450-556).  A steady-state (fwd, bwd) pair is
    fused when ``fuse_steady_state`` is set or the forward belongs to the
    last stage."""

    fuse_steady_state: bool = False

    def __post_init__(self):
        super().__post_init__()
        vp, rem = divmod(self.num_stages, self.mpmd_dim)
        if rem:
            raise ValueError(
                f"{self.num_stages=} must be divisible by {self.mpmd_dim=}")
        object.__setattr__(self, "vp", vp)
        object.__setattr__(self, "is_partial_bwd", False)

    def microbatches_per_round(self, n_microbatches: int) -> int:
        rounds = max(1, n_microbatches // self.mpmd_dim)
        per_round, rem = divmod(n_microbatches, rounds)
        if rem:
            raise ValueError("n_microbatches must be divisible by mpmd_dim")
        return per_round

    def _get_rank_warmup_ops(self, mpmd_idx: int, n_microbatches: int) -> int:
        per_round = self.microbatches_per_round(n_microbatches)
        hops_from_last = self.mpmd_dim - 1 - mpmd_idx
        return (self.vp - 1) * per_round + 2 * hops_from_last

    def get_rank_warmup_ops(self, mpmd_idx: int, n_microbatches: int) -> int:
        return min(self._get_rank_warmup_ops(mpmd_idx, n_microbatches),
                   n_microbatches * self.vp)

    def forward_stage_index(self, mpmd_idx: int, step: int,
                            microbatches_per_round: int) -> int:
        chunk = (step // microbatches_per_round) % self.vp
        return chunk * self.mpmd_dim + mpmd_idx

    def backward_stage_index(self, step: int, warmup_ops: int,
                             microbatches_per_round: int, mpmd_idx: int) -> int:
        chunk = self.vp - 1 - ((step - warmup_ops) // microbatches_per_round) % self.vp
        return chunk * self.mpmd_dim + mpmd_idx

    def _tasks_for_rank(self, mpmd_idx: int, n_mubatches: int) -> list:
        total = self.vp * n_mubatches
        warm = self.get_rank_warmup_ops(mpmd_idx, n_mubatches)
        per_round = self.microbatches_per_round(n_mubatches)
        give = _Dispenser(split_backward=self.is_partial_bwd)
        last_stage = self.num_stages - 1
        out: list = []
        for step in range(total + warm):
            fwd_stage = bwd_stage = None
            if step < total:
                fwd_stage = self.forward_stage_index(mpmd_idx, step, per_round)
            if step >= warm:
                bwd_stage = self.backward_stage_index(step, warm, per_round, mpmd_idx)
            if bwd_stage is None:                          # warm-up
                out.append(give.fwd(fwd_stage))
            elif fwd_stage is None:                        # cool-down
                out.append(give.bwd(bwd_stage))
            else:                                          # steady state
                f, b = give.fwd(fwd_stage), give.bwd(bwd_stage)
                if self.fuse_steady_state or fwd_stage == last_stage:
                    b = (b,) if isinstance(b, Task) else tuple(b)
                    out.append(FusedTask((f,) + b))
                else:
                    out += [f, b]
        return out

    def tasks(self, n_mubatches: int) -> ScheduleTasks:
        return [self._tasks_for_rank(r, n_mubatches) for r in range(self.mpmd_dim)]


class KimiK2(Interleaved1F1B):
    """Interleaved 1F1B with one extra warm-up forward per rank
    (reference: schedules.py:559-561)."""

    def _get_rank_warmup_ops(self, mpmd_idx: int, n_microbatches: int) -> int:
        return super()._get_rank_warmup_ops(mpmd_idx, n_microbatches) + 1


def dualpipev_tasks(mpmd_dim: int, mpmd_idx: int, n_mubatches: int) -> list:
    """One rank's DualPipeV list (reference: schedules.py:100-192).

    The rank owns stage ``near = mpmd_idx`` (descending leg of the V) and
    ``far = 2*mpmd_dim-1-mpmd_idx`` (ascending leg)."""
    P, r, n = mpmd_dim, mpmd_idx, n_mubatches
    near, far = r, 2 * P - 1 - r
    behind = P - 1 - r                  # ranks between this one and the V turn
    give = _Dispenser(split_backward=True)
    out: list = []

    out += [give.fwd(near) for _ in range(2 * behind)]              # 1: F0
    for _ in range(r + 1):                                          # 2: F0 F1
        out += [give.fwd(near), give.fwd(far)]
    for _ in range(behind):                                         # 3: B1 W1 F1
        out += [give.bwd_a(far), give.bwd_w(far), give.fwd(far)]
    for i in range(n - 2 * P + r + 1):                              # 4: F0B1 F1B0
        if i == 0 and r == P - 1:
            out += [give.fwd(near), give.bwd(far)]
        else:
            out.append(give.fwd_bwd(near, far))
        out.append(give.fwd_bwd(far, near))
    for _ in range(behind):                                         # 5: B1 F1B0
        out += [give.bwd(far), give.fwd_bwd(far, near)]
    zb_from = (r + 1) // 2
    for i in range(r + 1):                                          # 6: B1 B0
        defer_w = i >= zb_from
        out.append(give.bwd_a(far) if defer_w and r % 2 == 1 else give.bwd(far))
        # the first stage's backward is never split
        out.append(give.bwd_a(near) if defer_w and r % 2 == 0 and near != 0
                   else give.bwd(near))
    for _ in range(behind):                                         # 7: B0
        out.append(give.bwd(near) if near == 0 else give.bwd_a(near))
    pending = {(stage, done) for (stage, kind), done in give.issued.items()
               if kind is _BW}                                      # 8: left-over W
    assert len(pending) == 2
    tail = [give.bwd_w(stage) for stage, done in pending for _ in range(done, n)]
    out += sorted(tail, key=lambda t: (t.mubatch_idx, t.stage_id))
    return out


@dataclass(eq=True, frozen=True)
class DualPipeV(InterleavedBaseSchedule):
    """V-shaped placement of ``2*mpmd_dim`` stages with split backward
    (reference: schedules.py:622-652)."""

    def __post_init__(self):
        super().__post_init__()
        if divmod(self.num_stages, self.mpmd_dim) != (2, 0):
            raise ValueError(
                f"{DualPipeV.__name__} only supports 2 * mpmd_dim stages,"
                f" {self.num_stages=} requested with {self.mpmd_dim=}"
            )
        object.__setattr__(self, "is_partial_bwd", True)

    def get_mpmd_idx(self, stage_id: int) -> MpmdIdx:
        leg, pos = divmod(stage_id, self.mpmd_dim)
        return pos if leg % 2 == 0 else self.mpmd_dim - 1 - pos

    def tasks(self, n_mubatches: int) -> ScheduleTasks:
        if not (n_mubatches > 0 and n_mubatches >= self.num_stages):
            raise ValueError(
                f"{DualPipeV.__name__} requires {n_mubatches=} >= "
                f"{self.num_stages=} ({self.mpmd_dim=})"
            )
        return [dualpipev_tasks(self.mpmd_dim, r, n_mubatches)
                for r in range(self.mpmd_dim)]


# ---------------------------------------------------------------------------
# table -> what a rank actually executes
# ---------------------------------------------------------------------------
def strip_nones(ts: Iterable) -> list:
    return [t for t in ts if t is not None]


def unpack_fused_tasks_fn(ts: Iterable) -> list:
    flat: list = []
    for entry in ts:
        flat.extend(entry if isinstance(entry, FusedTask) else (entry,))
    return flat


def check_and_strip_adjecent_bwd_a_bwd_w(tasks: Sequence, first_stage_id: Any) -> list:
    """Fold every first-stage ``BWD_I`` and the ``BWD_W`` right behind it into
    one ``BWD_I`` of summed latency; the first stage's backward is never split
    (reference: schedules.py:671-721, name kept).  A first-stage ``BWD_I``
    followed by anything else raises ``NotImplementedError``; one in the very
    last position is passed through, as in the reference."""

    def fold_group(group: FusedTask):
        inner = check_and_strip_adjecent_bwd_a_bwd_w(list(group), first_stage_id)
        return inner[0] if len(inner) == 1 else FusedTask(inner)

    out: list = []
    i, last = 0, len(tasks) - 1
    while i <= last:
        t = tasks[i]
        if isinstance(t, FusedTask):
            out.append(fold_group(t))
        elif (i < last and t.stage_id == first_stage_id and t.fwd_or_bwd is _BI):
            nxt = tasks[i + 1]
            if (isinstance(nxt, FusedTask) or nxt.stage_id != first_stage_id
                    or nxt.fwd_or_bwd is not _BW):
                raise NotImplementedError(
                    f"{_BI} is not followed by {_BW} for "
                    f"first_stage {first_stage_id} at tasks {i} {tasks[i:i+2]}.\n"
                    f"{[str(_) for _ in tasks]}"
                )
            out.append(dataclasses.replace(t, latency=t.latency + nxt.latency))
            i += 1
        else:
            out.append(t)
        i += 1
    return out


def schedule_task_fusion_disabled() -> bool:
    """The reference's ``JAXPP_DISABLE_SCHEDULE_TASK_FUSION`` switch (src/jaxpp/env_vars.py:10-12,
    read where the loop is unrolled, src/jaxpp/core.py:2559-2563): when set, fused entries of a
    schedule's table are run as their members, one after the other.  Same spellings as the
    reference's ``parse_bool`` (src/jaxpp/utils.py:87-92); anything else is an error."""
    v = os.environ.get("JAXPP_DISABLE_SCHEDULE_TASK_FUSION")
    if v is None:
        return False
    if v.lower() in ("true", "1", "t", "y", "yes"):
        return True
    if v.lower() in ("false", "0", "f", "n", "no"):
        return False
    raise ValueError(f"Unsupported value JAXPP_DISABLE_SCHEDULE_TASK_FUSION={v}")


def preprocess_schedule_tasks(schedule: ScheduleTasks, first_stage_id,
                              unpack_fused_tasks: bool) -> list:
    """Bubble slots removed, fused groups optionally flattened, first-stage
    backward re-joined (reference: schedules.py:724-739)."""
    rows = [strip_nones(row) for row in schedule]
    if unpack_fused_tasks:
        rows = [unpack_fused_tasks_fn(row) for row in rows]
    return [check_and_strip_adjecent_bwd_a_bwd_w(row, first_stage_id=first_stage_id)
            for row in rows]
