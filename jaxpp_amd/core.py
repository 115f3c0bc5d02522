"""Driver: ``mpmd_jit_with_loop`` and what it runs.

Reference anchors
  * ``mpmd_jit_with_loop`` / ``TraceableFunction`` - src/jaxpp/core.py:3892-3923,
    :3151-3259: a decorator taking the MPMD mesh; the object it returns has
    ``compile(*args)`` and ``__call__``.
  * clustering the loop body at the stage markers - core.py:958-1180 - here
    ``cluster_ops``; marker count must equal ``schedule.num_stages``.
  * unrolling over microbatches and list-scheduling the unrolled tasks against
    the per-rank tables - core.py:1896-2098 - here ``order_tasks``, with the
    reference's two failure messages.
  * ``task_impl`` dispatch of each task - src/jaxpp/jax_primitives.py:776-859 -
    here one ``StageExecutor.run_task`` per task, all MPMD groups on one GPU.
"""
from __future__ import annotations

import contextlib
import ctypes as C
import time
from collections import defaultdict
from dataclasses import dataclass
from typing import Any, Callable, Iterable, Sequence

import numpy as np

from jaxpp_amd import tracing
from jaxpp_amd.mesh import MpmdMesh
from jaxpp_amd.schedules import (BaseSchedule, FusedTask, Task, mk_task_name,
                                 preprocess_schedule_tasks, schedule_task_fusion_disabled)
from jaxpp_amd.types import TaskType

# ---------------------------------------------------------------------------
# per-task timings (reference: collect_task_times_ms, jax_primitives.py:742-773)
# ---------------------------------------------------------------------------
_statistics = None


@contextlib.contextmanager
def collect_task_times_ms(enabled: bool = True):
    """``with collect_task_times_ms() as stats`` -> ``{task_name: [ms, ...]}``;
    while active every task is bracketed by device synchronisation, as in the
    reference.  ``enabled=False`` yields ``None``."""
    global _statistics
    if not enabled:
        yield
        return
    old, _statistics = _statistics, defaultdict(list)
    try:
        yield _statistics
    finally:
        _statistics = old


# ---------------------------------------------------------------------------
# autodiff marker for the traced body
# ---------------------------------------------------------------------------
def value_and_grad(fun: Callable, has_aux: bool = False) -> Callable:
    """Like ``jax.value_and_grad`` for a loss traced through
    ``jaxpp_amd.nn``: differentiates with respect to the first argument (the
    parameter pytree).  The gradients are symbolic; ``treduce`` materialises
    their sum over microbatches."""

    def wrapped(params, *args):
        if tracing.current() is None:
            raise RuntimeError("value_and_grad(...) evaluates inside jaxpp_amd.treduce")
        out = fun(params, *args)
        value = out[0] if has_aux else out
        if not (isinstance(value, tracing.Traced) and value.shape == () and
                value.producer[0] == "mse"):
            raise TypeError("value_and_grad differentiates a scalar loss (the first element of "
                            "the function's result with has_aux)")
        tracing.current().differentiated = value
        grads = tracing.tree_map(lambda a: tracing.GradOf(id(a), tuple(np.shape(a))), params)
        return out, grads

    return wrapped


# ---------------------------------------------------------------------------
# loop body -> stages
# ---------------------------------------------------------------------------
@dataclass
class StagedBody:
    stage_layers: list          # per stage: [(spec, params dict), ...]
    has_loss: bool              # the last stage ends in an mse loss
    leaf_owner: dict            # id(param array) -> (stage, layer index, name)
    input_index: int            # which microbatched input feeds the first layer
    target: tuple | None        # ("input", k) | ("const", array): what the loss compares with
    final_uid: int = 0          # the value the last stage hands out (the prediction)


def cluster_ops(tr: tracing.Trace, target_num_stages: int) -> StagedBody:
    """Cuts the traced body at its markers (reference: ``cluster_by_yield_eqns`` /
    ``clusters_to_tasks``, src/jaxpp/core.py:958-1118: a task is whatever lies between two
    markers).  The body must be one chain: a microbatched input through layers and markers to
    the prediction the loss reads."""
    stages, cur, mse = [], [], None
    producer_of = {sym.uid: ("input", k) for k, (_, sym) in enumerate(tr.inputs)}
    head = None                    # uid of the value the chain has reached
    input_index = None
    for op in tr.ops:
        if op[0] == "layer":
            if mse is not None:
                raise AssertionError("layers after the loss are not part of any stage")
            _, spec, params, in_uid, out_uid = op
            if head is None:
                src = producer_of.get(in_uid)
                if src is None:
                    raise NotImplementedError("the first layer must read a microbatched input "
                                              "of the loop")
                input_index = src[1]
            elif in_uid != head:
                raise NotImplementedError("the loop body must be a single chain of layers: a "
                                          "layer reads the value the previous layer or marker "
                                          "produced")
            head = out_uid
            cur.append((spec, params))
        elif op[0] == "yield":
            ins, outs = op[3], op[4]
            if head is None or head not in ins:
                raise NotImplementedError("mark_stage_end must be applied to the value the "
                                          "chain of layers has reached")
            head = outs[ins.index(head)]
            stages.append(cur)
            cur = []
        elif op[0] == "mse":
            if mse is not None:
                raise NotImplementedError("one loss per loop body")
            mse = op
    if cur and stages:            # trailing layers join the last stage, like trailing eqns
        stages[-1] = stages[-1] + cur
    found = len(stages)
    if found != target_num_stages:
        raise AssertionError(f"Unexpected number of pipeline markers: found {found} "
                             f"expected {target_num_stages}.\n")
    owner = {}
    for s_, layers in enumerate(stages):
        if not layers:
            raise AssertionError(f"Empty stage {(s_, TaskType.FWD)}")
        for li, (_, params) in enumerate(layers):
            for name, arr in params.items():
                owner[id(arr)] = (s_, li, name)
    target = None
    if mse is not None:
        _, pred_uid, target = mse
        # trailing layers (after the last marker) move `head` past the marker's output
        if pred_uid != head:
            raise NotImplementedError("the loss must read the output of the last layer of the "
                                      "last stage")
    shapes = {(sp.tokens, sp.hidden, sp.dtype) for layers in stages for sp, _ in layers}
    if len(shapes) != 1:
        raise NotImplementedError("every layer of the body must keep the activation's shape "
                                  f"(tokens, hidden) and element type; found {sorted(shapes)}")
    return StagedBody(stages, mse is not None, owner, input_index, target, head)


# ---------------------------------------------------------------------------
# unrolled task graph + list scheduling
# ---------------------------------------------------------------------------
def task_dependencies(t: Task, num_stages: int, split: set) -> list:
    """Tasks whose results ``t`` consumes.  ``split`` holds the stages whose
    backward runs as BWD_I + BWD_W."""
    s, m, k = t.stage_id, t.mubatch_idx, t.fwd_or_bwd
    back = lambda st: TaskType.BWD_I if st in split else TaskType.BWD
    deps = []
    if k is TaskType.FWD:
        if s > 0:
            deps.append(Task.make(s - 1, m, TaskType.FWD))
    elif k is TaskType.BWD_W:
        deps.append(Task.make(s, m, TaskType.BWD_I))
    else:
        deps.append(Task.make(s, m, TaskType.FWD))
        if s + 1 < num_stages:
            deps.append(Task.make(s + 1, m, back(s + 1)))
    if m > 0 and k is not TaskType.FWD:       # accumulators are loop carries
        deps.append(Task.make(s, m - 1, k))
    return deps


@dataclass(frozen=True)
class TimedEntry:
    start_time: int
    end_time: int
    rank: int
    entry: Any                   # Task | FusedTask


def order_tasks(rows: list, num_stages: int) -> list:
    """Global order of the per-rank rows: repeatedly advance the rank whose
    next entry is ready and can start earliest (ties: lowest rank), then sort
    by (start, end).  Restates ``reorder_nodes_with_schedule``
    (src/jaxpp/core.py:1966-2098) including its two errors."""
    split = {t.stage_id for row in rows for e in row
             for t in (e if isinstance(e, FusedTask) else (e,))
             if t.fwd_or_bwd is TaskType.BWD_W}
    # a first-stage BWD_I that swallowed its BWD_W stands for the whole backward
    all_tasks = [t for row in rows for e in row for t in (e if isinstance(e, FusedTask) else (e,))]
    present = set(all_tasks)
    done_at: dict = {}
    pos = [0] * len(rows)
    clock = [0] * len(rows)
    out = []
    remaining = len(all_tasks)
    while remaining:
        best = None
        for r, row in enumerate(rows):
            if pos[r] >= len(row):
                continue
            entry = row[pos[r]]
            members = tuple(entry) if isinstance(entry, FusedTask) else (entry,)
            ready, inside, ok = clock[r], set(), True
            for t in members:
                for d in task_dependencies(t, num_stages, split):
                    if d not in present or d in inside:
                        continue
                    if d not in done_at:
                        ok = False
                        break
                    ready = max(ready, done_at[d])
                if not ok:
                    break
                inside.add(t)
            if ok and (best is None or ready < best[0]):
                best = (ready, r, entry, members)
        if best is None:
            where = {r: (pos[r], rows[r][pos[r]]) for r in range(len(rows)) if pos[r] < len(rows[r])}
            raise AssertionError("Schedule does not honor data dependencies.\n"
                                 f"Current position in schedule for ranks {where}.")
        start, r, entry, members = best
        end = start
        for t in members:
            end += t.latency
            done_at[t] = end
        out.append(TimedEntry(start, end, r, entry))
        pos[r] += 1
        clock[r] = end
        remaining -= len(members)
    for r, row in enumerate(rows):
        if pos[r] != len(row):
            raise AssertionError("Loop tasks have ended but schedule contains other tasks. "
                                 f"{row[pos[r]:]}")
    return sorted(out, key=lambda e: (e.start_time, e.end_time))


def validate_schedule(schedule: BaseSchedule, n_mubatches: int,
                      unpack_fused_tasks: bool | None = None) -> list:
    """Preprocess the table and check it against the task graph; returns the
    global order.  `unpack_fused_tasks` None: as JAXPP_DISABLE_SCHEDULE_TASK_FUSION says."""
    if unpack_fused_tasks is None:
        unpack_fused_tasks = schedule_task_fusion_disabled()
    rows = preprocess_schedule_tasks(schedule.tasks(n_mubatches), 0, unpack_fused_tasks)
    seen = set()
    for row in rows:
        for e in row:
            for t in (e if isinstance(e, FusedTask) else (e,)):
                seen.add((t.stage_id, t.mubatch_idx, t.fwd_or_bwd))
    for s in range(schedule.num_stages):
        for m in range(n_mubatches):
            if (s, m, TaskType.FWD) not in seen:
                raise AssertionError("Loop tasks have ended but schedule contains other tasks. "
                                     f"missing fwd_{s}__{m}")
    return order_tasks(rows, schedule.num_stages)


# ---------------------------------------------------------------------------
# the decorator
# ---------------------------------------------------------------------------
_active_function = None


class TraceableFunction:
    def __init__(self, fun: Callable, mpmd_mesh: MpmdMesh, options: dict):
        self.fun, self.mpmd_mesh, self.options = fun, mpmd_mesh, options
        self._executors = {}        # key -> {(stage, segment): StageExecutor}
        self.last_order = None      # TimedEntry list of the last loop
        self.__wrapped__ = fun

    def compile(self, *args, **kwargs):
        """Runs the function once so that executors exist and kernels are
        loaded; returns ``self`` (the compiled callable)."""
        self(*args, **kwargs)
        return self

    def __call__(self, *args, **kwargs):
        global _active_function
        if _active_function is not None:
            raise RuntimeError("nested mpmd_jit_with_loop calls are not supported")
        _active_function = self
        try:
            with self.mpmd_mesh:
                return self.fun(*args, **kwargs)
        finally:
            _active_function = None

    def close(self):
        for group in self._executors.values():
            for ex in group.values():
                ex.close()
        self._executors.clear()


def mpmd_jit_with_loop(fun: Callable | None = None, mpmd_mesh: MpmdMesh | None = None, *,
                       in_shardings=None, out_shardings=None, in_specs=None, out_specs=None,
                       static_argnums: int | Sequence[int] | None = None,
                       static_argnames: str | Iterable[str] | None = None,
                       donate_argnums: int | Sequence[int] | None = None,
                       donate_argnames: str | Iterable[str] | None = None,
                       compiler_options: dict | None = None) -> TraceableFunction:
    """Signature of the reference's decorator (core.py:3892-3905).  Sharding,
    static and donation arguments are accepted and validated the same way;
    with one device per MPMD group there is nothing for them to change."""
    if in_specs is not None and in_shardings is not None:
        raise ValueError("Can't pass both in_shardings and in_specs")
    if out_specs is not None and out_shardings is not None:
        raise ValueError("Can't pass both out_shardings and out_specs")
    if mpmd_mesh is None:
        raise TypeError("mpmd_jit_with_loop() missing required argument: 'mpmd_mesh'")
    opts = dict(in_shardings=in_shardings or in_specs, out_shardings=out_shardings or out_specs,
                static_argnums=static_argnums, static_argnames=static_argnames,
                donate_argnums=donate_argnums, donate_argnames=donate_argnames,
                compiler_options=compiler_options)
    if fun is None:
        return lambda f: TraceableFunction(f, mpmd_mesh, opts)
    return TraceableFunction(fun, mpmd_mesh, opts)


# ---------------------------------------------------------------------------
# running the loop
# ---------------------------------------------------------------------------
@dataclass
class _Segment:
    """Consecutive layers of one stage that share a layer shape: one stage executor."""
    spec: Any
    layers: list                # parameter dicts
    first: int                  # index of its first layer inside the stage
    ex: Any = None


def _segments(layers: list) -> list:
    segs = []
    for li, (spec, params) in enumerate(layers):
        if segs and segs[-1].spec == spec:
            segs[-1].layers.append(params)
        else:
            segs.append(_Segment(spec, [params], li))
    return segs


def _stage_lifetimes(rows: list, num_stages: int) -> tuple:
    """Per stage: peak number of forwards whose residuals are still needed, and whether its
    backward arrives split into BWD_I and BWD_W tasks."""
    peak, live, split = [0] * num_stages, [0] * num_stages, [False] * num_stages
    for row in rows:
        for e in row:
            for t in (e if isinstance(e, FusedTask) else (e,)):
                s_, k = t.stage_id, t.fwd_or_bwd
                if k is TaskType.FWD:
                    live[s_] += 1
                    peak[s_] = max(peak[s_], live[s_])
                elif k is TaskType.BWD or k is TaskType.BWD_W or \
                        (k is TaskType.BWD_I and s_ == 0 and t.latency > 1):
                    live[s_] -= 1
                if k is TaskType.BWD_W:
                    split[s_] = True
    return peak, split


def run_loop(tr, outputs, ops, n: int, schedule: BaseSchedule):
    from jaxpp_amd import runtime as rt
    fn = _active_function
    if fn is None:
        raise RuntimeError("treduce executes under mpmd_jit_with_loop (it needs the MPMD mesh)")
    mesh = fn.mpmd_mesh
    body = cluster_ops(tr, schedule.num_stages)
    S = schedule.num_stages
    # (src/jaxpp/core.py:2559-2563: the environment decides whether fused entries stay fused)
    rows = preprocess_schedule_tasks(schedule.tasks(n), 0, schedule_task_fusion_disabled())
    if len(rows) != mesh.mpmd_dim:
        raise AssertionError(f"schedule places tasks on {len(rows)} MPMD groups, the mesh has "
                             f"{mesh.mpmd_dim}")
    order = order_tasks(rows, S)
    fn.last_order = order
    peak, split = _stage_lifetimes(rows, S)

    # One executor per run of equally shaped layers inside a stage (a task is whatever lies
    # between two markers: stages may differ in depth and in layer family).
    stage_segs = [_segments(layers) for layers in body.stage_layers]
    spec0 = body.stage_layers[0][0][0]
    lib = rt.load()
    key = (tuple(tuple((sg.spec, len(sg.layers)) for sg in segs) for segs in stage_segs),
           type(schedule).__name__, S, n, tuple(peak), tuple(split))
    if key not in fn._executors:
        fn.close()
        group = {}
        for s_, segs in enumerate(stage_segs):
            for g, sg in enumerate(segs):
                group[s_, g] = rt.StageExecutor(sg.spec, 1, len(sg.layers), peak[s_], split[s_], True)
        fn._executors[key] = group
    execs = fn._executors[key]
    for s_, segs in enumerate(stage_segs):
        for g, sg in enumerate(segs):
            sg.ex = execs[s_, g]
            for li, params in enumerate(sg.layers):
                sg.ex.set_params(0, li, params)
            sg.ex.zero_grads()

    tokens, hidden = spec0.tokens, spec0.hidden
    act_elems = tokens * hidden
    f32 = spec0.dtype == "f32"           # an f32 model runs through the f32 operators
    any_ex = execs[0, 0]

    def microbatches(x):
        if x.shape[1:] != (tokens, hidden):
            if int(np.prod(x.shape[1:])) != act_elems:
                raise ValueError(f"a microbatch of shape {x.shape[1:]} does not hold "
                                 f"{tokens} x {hidden} values")
            x = x.reshape(n, tokens, hidden)
        return [any_ex.upload_activation(x[m]) for m in range(n)]

    xs_dev = microbatches(tr.inputs[body.input_index][0])
    tgt_dev = None
    if body.has_loss:
        kind, what = body.target
        if kind == "input":
            tgt_dev = xs_dev if what == body.input_index else microbatches(tr.inputs[what][0])
        else:
            const = any_ex.upload_activation(np.ascontiguousarray(what).reshape(tokens, hidden))
            tgt_dev = [const] * n
    act, cot = {}, {}                   # (stage, mb) -> DeviceBuffer
    free = []

    def take():
        return free.pop() if free else any_ex.new_activation()

    def run_fwd(s_, m, src, dst):
        segs = stage_segs[s_]
        cur = src
        for g, sg in enumerate(segs):
            out = dst if g + 1 == len(segs) else take()
            sg.ex.run_task(TaskType.FWD, 0, m, cur.ptr, out.ptr)
            if cur is not src:
                free.append(cur)        # the executor keeps its own copy of a task's input
            cur = out

    def run_bwd(s_, m, kind, src, dst):
        segs = stage_segs[s_]
        cur = src
        for g in reversed(range(len(segs))):
            out = dst if g == 0 else take()
            segs[g].ex.run_task(kind, 0, m, cur.ptr, out.ptr)
            if cur is not src:
                free.append(cur)
            cur = out

    loss_dev = rt.DeviceBuffer(4 * n)
    partial = rt.DeviceBuffer(4 * rt.NORM_PARTIALS)
    want_pred = any(isinstance(v, tracing.Traced) and v.shape != () for v in tracing.tree_leaves(outputs))
    preds = {}
    # the scale of the value that is differentiated sets the cotangent; loss values returned
    # with another scale are rescaled from it
    diff = tr.differentiated
    loss_scales = [v.producer[1] for v in tracing.tree_leaves(outputs)
                   if isinstance(v, tracing.Traced) and v.shape == () and v.producer[0] == "mse"]
    loss_scale = diff.producer[1] if diff is not None else (loss_scales[0] if loss_scales else 1.0)

    for te in order:
        members = tuple(te.entry) if isinstance(te.entry, FusedTask) else (te.entry,)
        for t in members:
            s, m = t.stage_id, t.mubatch_idx
            kind = t.fwd_or_bwd
            if kind is TaskType.BWD_I and s == 0 and t.latency > 1:
                kind = TaskType.BWD
            t0 = None
            if _statistics is not None:
                rt.sync()
                t0 = time.perf_counter()
            if kind is TaskType.FWD:
                src = xs_dev[m] if s == 0 else act.pop((s, m))
                dst = take()
                run_fwd(s, m, src, dst)
                if s > 0:
                    free.append(src)
                if s + 1 < S:
                    act[s + 1, m] = dst
                else:
                    if not body.has_loss:
                        raise AssertionError("the last stage has no loss to differentiate")
                    d = take()
                    if f32:
                        rt.check(lib.jpp_mse_loss_f32(None, dst.ptr, tgt_dev[m].ptr, act_elems,
                                                      float(loss_scale), loss_dev.ptr + 4 * m,
                                                      d.ptr))
                    else:
                        rt.check(lib.jpp_mse_loss(None, dst.ptr, tgt_dev[m].ptr, act_elems,
                                                  float(loss_scale), loss_dev.ptr + 4 * m, d.ptr,
                                                  partial.ptr))
                    cot[s, m] = d
                    if want_pred:
                        preds[m] = any_ex.download_activation(dst, (tokens, hidden))
                    free.append(dst)
            elif kind is TaskType.BWD_W:
                for sg in reversed(stage_segs[s]):
                    sg.ex.run_task(kind, 0, m)
            else:
                src = cot.pop((s, m))
                dst = take()
                run_bwd(s, m, kind, src, dst)
                free.append(src)
                if s > 0:
                    cot[s - 1, m] = dst
                else:
                    free.append(dst)
            if t0 is not None:
                rt.sync()
                _statistics[mk_task_name(s, t.fwd_or_bwd)].append((time.perf_counter() - t0) * 1e3)
    rt.sync()
    losses = loss_dev.download(np.float32, (n,))
    grads = {}
    for s_, segs in enumerate(stage_segs):
        grads[s_] = []
        for sg in segs:
            grads[s_] += [sg.ex.get_grads(0, li) for li in range(len(sg.layers))]

    def reduce_leaf(v, op):
        if isinstance(v, tracing.GradOf):
            if type(op).__name__ != "AddT":
                raise NotImplementedError("gradients are reduced with Add")
            if diff is None:
                raise AssertionError("gradients need value_and_grad around the loss")
            s, li, name = body.leaf_owner[v.leaf_id]
            return grads[s][li][name].reshape(v.shape)
        if isinstance(v, tracing.Traced):
            if v.shape == ():
                if v.producer[0] != "mse":
                    raise NotImplementedError(f"cannot return {v} from the loop body")
                rescale = np.float32(v.producer[1] / loss_scale)
                per_mb = [np.float32(losses[m]) * rescale for m in range(n)]
            else:
                if v.uid != body.final_uid:
                    raise NotImplementedError("the only activation the loop can return is the "
                                              "output of the last stage")
                per_mb = [preds[m].reshape(v.shape) for m in range(n)]
            state = op.state(n, per_mb[0])
            for m in range(n):
                state = op.update(state, per_mb[m], m)
            return state
        return v

    def walk(v, op):
        if isinstance(v, (tuple, list)):
            return type(v)(walk(a, b) for a, b in zip(v, op))
        if isinstance(v, dict):
            return {k: walk(v[k], op[k]) for k in v}
        return reduce_leaf(v, op)

    return walk(outputs, ops)
