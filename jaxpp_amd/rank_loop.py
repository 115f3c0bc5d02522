"""Runs one rank's row of the task table on a stage executor.

The reference turns the members of a ``FusedTask`` into one task whose parts
the compiler is free to overlap (src/jaxpp/core.py:2444-2513, ``fuse_groups``;
src/jaxpp/schedules.py:48-54).  Here the forward member of a fused entry goes
out on a second stream and the backward member on the first one - unless they
belong to the same microbatch: that backward reads the forward's residuals, so
the two run in order.  The streams meet again at the end of the entry, so
everything after it sees both results.
"""
from __future__ import annotations

from itertools import groupby

from jaxpp_amd import runtime as rt
from jaxpp_amd.types import TaskType


class RankLoop:
    def __init__(self, executor: "rt.StageExecutor", plan, overlap_fused: bool = True):
        self.ex, self.plan = executor, plan
        self.entries = [list(g) for _, g in groupby(plan.tasks, key=lambda pt: pt.group)]
        self.overlap = overlap_fused and any(len(e) > 1 for e in self.entries)
        if self.overlap:
            self.aux = rt.Stream()
            self.fork, self.join = rt.Event(), rt.Event()

    def run(self, io, stream=None):
        """``io(pt, lane)`` -> (in_ptr, out_ptr) for a FWD / BWD / BWD_I task (lane 1: the task
        runs beside another one and needs an output buffer of its own); BWD_W tasks take
        none.  Everything is queued on `stream` (a stream pointer; None: the null stream),
        fused forwards on the loop's second stream."""
        ex = self.ex
        for entry in self.entries:
            fwd_mbs = {pt.task.mubatch_idx for pt in entry if pt.exec_kind is TaskType.FWD}
            bwd_mbs = {pt.task.mubatch_idx for pt in entry if pt.exec_kind is not TaskType.FWD}
            # A fused entry may hold the forward and the backward of one microbatch (the last
            # stage's, back to back): the backward reads what that forward leaves behind, so
            # such members run one after the other; side by side only when the forward
            # belongs to another microbatch than every backward of the entry.
            beside = self.overlap and bool(fwd_mbs) and bool(bwd_mbs) and not (fwd_mbs & bwd_mbs)
            if beside:
                self.fork.record(stream)
                self.aux.wait(self.fork)
            for pt in entry:
                m = pt.task.mubatch_idx
                if pt.exec_kind is TaskType.BWD_W:
                    ex.run_task(pt.exec_kind, pt.chunk, m, stream=stream)
                    continue
                on_aux = beside and pt.exec_kind is TaskType.FWD
                inp, out = io(pt, 1 if on_aux else 0)
                ex.run_task(pt.exec_kind, pt.chunk, m, inp, out, self.aux.ptr if on_aux else stream)
            if beside:
                self.join.record(self.aux.ptr)
                rt.stream_wait(stream, self.join)
