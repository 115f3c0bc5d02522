"""From a schedule's task table to what one rank executes.

Follows the reference's loop unrolling for a single rank
(src/jaxpp/core.py:2550-2589): the table is preprocessed
(``preprocess_schedule_tasks`` with ``first_stage_id=0``) and the rank runs its
row in order, the members of a fused group back to back.  Residual lifetimes
are what ``infer_donation`` / ``add_deletes`` produce
(src/jaxpp/core.py:1732-1890): a forward's residuals die with the task that
last reads them, so the number of slots a rank needs is the peak number of
forwards whose BWD (or BWD_W) has not yet run.
"""
from __future__ import annotations

from dataclasses import dataclass, field

from jaxpp_amd.schedules import (BaseSchedule, FusedTask, Task, preprocess_schedule_tasks,
                                 schedule_task_fusion_disabled)
from jaxpp_amd.types import TaskType


@dataclass(frozen=True)
class PlannedTask:
    task: Task              # the table's entry
    exec_kind: TaskType     # what the executor runs (a merged first-stage BWD_I runs BWD)
    chunk: int              # index of the stage among this rank's stages
    group: int              # position of the (possibly fused) entry in the row


@dataclass
class RankPlan:
    rank: int
    stages: list            # stage ids this rank owns, ascending; chunk = index
    tasks: list = field(default_factory=list)
    max_live: int = 0
    split_backward: bool = False

    @property
    def n_chunks(self) -> int:
        return len(self.stages)


def stages_of_rank(schedule: BaseSchedule, rank: int) -> list:
    return [s for s in range(schedule.num_stages) if int(schedule.get_mpmd_idx(s)) == rank]


def make_rank_plan(schedule: BaseSchedule, n_mubatches: int, rank: int,
                   unpack_fused_tasks: bool | None = None, first_stage_id: int = 0) -> RankPlan:
    """`unpack_fused_tasks` None: as the environment says (JAXPP_DISABLE_SCHEDULE_TASK_FUSION,
    the reference's switch, read where it unrolls the loop: src/jaxpp/core.py:2559-2563)."""
    if unpack_fused_tasks is None:
        unpack_fused_tasks = schedule_task_fusion_disabled()
    rows = preprocess_schedule_tasks(schedule.tasks(n_mubatches), first_stage_id,
                                     unpack_fused_tasks)
    if not 0 <= rank < len(rows):
        raise ValueError(f"rank {rank} out of range for a table of {len(rows)} rows")
    stages = stages_of_rank(schedule, rank)
    chunk_of = {s: i for i, s in enumerate(stages)}
    plan = RankPlan(rank=rank, stages=stages)
    live = 0
    pending_w = set()
    for gi, entry in enumerate(rows[rank]):
        members = tuple(entry) if isinstance(entry, FusedTask) else (entry,)
        for t in members:
            if t.stage_id not in chunk_of:
                raise ValueError(f"{t} is scheduled on rank {rank}, which does not own its stage")
            kind = t.fwd_or_bwd
            if kind is TaskType.BWD_I and t.stage_id == first_stage_id and t.latency > 1:
                kind = TaskType.BWD           # W half was folded into it
            if kind is TaskType.FWD:
                live += 1
                plan.max_live = max(plan.max_live, live)
            elif kind is TaskType.BWD:
                live -= 1
            elif kind is TaskType.BWD_I:
                pending_w.add((t.stage_id, t.mubatch_idx))
                plan.split_backward = True
            elif kind is TaskType.BWD_W:
                if (t.stage_id, t.mubatch_idx) not in pending_w:
                    raise ValueError(f"{t} precedes its BWD_I")
                pending_w.discard((t.stage_id, t.mubatch_idx))
                live -= 1
            plan.tasks.append(PlannedTask(t, kind, chunk_of[t.stage_id], gi))
    if live != 0 or pending_w:
        raise ValueError(f"row of rank {rank} leaves {live} residual sets alive")
    return plan
