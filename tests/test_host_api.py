"""Host-side logic that needs no GPU: the API surface, markers, reduction
ops, the list scheduler and its failure modes, rank plans."""
from functools import partial

import numpy as np
import pytest

import jaxpp_amd as jaxpp
from jaxpp_amd import core, schedules as S, tracing
from jaxpp_amd.model import LayerSpec
from jaxpp_amd.plan import make_rank_plan
from jaxpp_amd.types import TaskType

SPEC = LayerSpec("bert", 128, 2, 256, 128, 1)


def test_public_names_of_the_reference_api():
    # src/jaxpp/api.py:19-45 (the part this package builds)
    for name in ["mark_stage_end", "pipeline_enter_stage", "treduce", "treduce_i", "Add", "Concat",
                 "Max", "mpmd_jit_with_loop", "MpmdMesh", "BaseSchedule", "DualPipeV", "Eager1F1B",
                 "Interleaved1F1B", "KimiK2", "Std1F1B", "ZeroBubble", "collect_task_times_ms"]:
        assert hasattr(jaxpp, name), name


def test_mark_stage_end_is_identity_outside_a_loop():
    x = np.ones(3)
    assert jaxpp.mark_stage_end(x) is x
    with pytest.deprecated_call():
        assert jaxpp.pipeline_enter_stage(x) is x


def test_markers_number_stages_from_zero_per_scope():
    from jaxpp_amd.pipelining import yield_scope
    for _ in range(2):
        with tracing.tracing() as tr, yield_scope():
            v = tr.fresh((4, 4), ("input",))
            v = jaxpp.mark_stage_end(v, name="a")
            v, w = jaxpp.mark_stage_end((v, v))
        assert [op[:2] for op in tr.ops] == [("yield", 0), ("yield", 1)]
    assert jaxpp.mark_stage_end(5) == 5          # scope closed again


def test_reduction_ops():
    a = np.arange(6, dtype=np.float32).reshape(2, 3)
    st = jaxpp.Add.state(4, a)
    assert st.shape == (2, 3) and st.dtype == np.float32 and not st.any()
    np.testing.assert_array_equal(jaxpp.Add.update(st, a, 0), a)
    c = jaxpp.Concat(axis=1)
    st = c.state(4, a)
    assert st.shape == (2, 4, 3)
    st = c.update(st, a, 2)
    np.testing.assert_array_equal(st[:, 2], a)
    assert not st[:, 1].any()
    m = jaxpp.Max.state(4, a)
    assert np.isneginf(m).all()
    np.testing.assert_array_equal(jaxpp.Max.update(m, a, 0), a)
    from jaxpp_amd.training import broadcast_ops
    ops = broadcast_ops((jaxpp.Concat(), jaxpp.Add), ((1, (2, 3)), {"w": 4}))
    assert isinstance(ops[0][1][0], jaxpp.Concat) and ops[1]["w"] is jaxpp.Add


def test_treduce_checks_leading_dimensions():
    with pytest.raises(AssertionError, match="Leading dimensions differing among xs"):
        jaxpp.treduce(lambda x: x, (np.zeros((4, 2)), np.zeros((3, 2))), S.Std1F1B(1))
    with pytest.raises(RuntimeError, match="under mpmd_jit_with_loop"):
        model = jaxpp.nn.TransformerStack(SPEC, 1, 1)
        jaxpp.treduce(lambda x: jaxpp.nn.mse_loss(model.apply(model.init(), x), x),
                      np.zeros((2, 128, 128), np.float32), S.Std1F1B(1), operation=jaxpp.Concat())


def test_wrong_marker_count_is_reported_like_the_reference():
    model = jaxpp.nn.TransformerStack(SPEC, 4, 2)            # 2 markers
    mesh = jaxpp.MpmdMesh(jaxpp.DeviceMesh(np.arange(4).reshape(4, 1), ("mpmd", "data")), "mpmd")
    params = model.init()

    @partial(jaxpp.mpmd_jit_with_loop, mpmd_mesh=mesh)
    def step(batch):
        return jaxpp.treduce(lambda x: jaxpp.nn.mse_loss(model.apply(params, x), x), batch,
                             S.Std1F1B(4), operation=jaxpp.Concat())
    with pytest.raises(AssertionError,
                       match="Unexpected number of pipeline markers: found 2 expected 4"):
        step(np.zeros((4, 128, 128), np.float32))


def test_mpmd_mesh():
    mesh = jaxpp.MpmdMesh(jaxpp.DeviceMesh(np.arange(8).reshape(2, 1, 4), ("mpmd", "data", "model")),
                          "mpmd")
    assert mesh.mpmd_dim == 2 and mesh.mpmd_axis == 0
    assert mesh.lowering_mesh().shape == {"mpmd": 1, "data": 1, "model": 4}   # README.md:104
    assert [m.devices.ravel().tolist() for m in mesh.unstack] == [[0, 1, 2, 3], [4, 5, 6, 7]]
    assert mesh.device_mpmd_idx[5] == 1
    assert mesh.mpmd_submesh([1]).jax_mesh.devices.ravel().tolist() == [4, 5, 6, 7]
    with mesh:
        assert jaxpp.MpmdMesh.mesh_stack[-1] is mesh
    assert mesh not in jaxpp.MpmdMesh.mesh_stack
    with pytest.raises(ValueError):
        jaxpp.MpmdMesh(mesh.jax_mesh, "pipe")


def test_decorator_argument_checks():
    mesh = jaxpp.MpmdMesh(jaxpp.DeviceMesh(np.arange(2).reshape(2), ("mpmd",)), "mpmd")
    with pytest.raises(ValueError, match="Can't pass both in_shardings and in_specs"):
        jaxpp.mpmd_jit_with_loop(lambda: 0, mesh, in_shardings=1, in_specs=1)
    with pytest.raises(ValueError, match="Can't pass both out_shardings and out_specs"):
        jaxpp.mpmd_jit_with_loop(lambda: 0, mesh, out_shardings=1, out_specs=1)
    f = jaxpp.mpmd_jit_with_loop(lambda a: a + 1, mesh)
    assert f(1) == 2 and f.compile(1) is f


GRID = [(S.Std1F1B(1), 4), (S.Std1F1B(2), 4), (S.Eager1F1B(3), 5), (S.Interleaved1F1B(1, 1), 1),
        (S.Interleaved1F1B(8, 4), 1), (S.KimiK2(8, 4, fuse_steady_state=True), 1),
        (S.Interleaved1F1B(4, 2), 12), (S.ZeroBubble(4), 4), (S.ZeroBubble(4), 8),
        (S.DualPipeV(6, 3), 6), (S.DualPipeV(6, 3), 10), (S.Interleaved1F1B(48, 8), 64),
        (S.DualPipeV(16, 8), 18), (S.GPipe(3), 5), (S.ZeroBubble(8), 24), (S.DualPipeV(8, 4), 16)]


@pytest.mark.parametrize("sched,n", GRID, ids=lambda v: str(v))
def test_every_reference_schedule_orders_the_task_graph(sched, n):
    """The grids of tests/test_transformations.py:140-155 and :194-200 must
    schedule without a dependency violation; start times respect dependencies
    and no rank runs two things at once."""
    order = core.validate_schedule(sched, n)
    rows = S.preprocess_schedule_tasks(sched.tasks(n), 0, False)
    assert sum(len(r) for r in rows) == len(order)
    end = {}
    busy = {}
    for te in order:
        assert te.start_time >= busy.get(te.rank, 0)
        busy[te.rank] = te.end_time
        for t in (te.entry if isinstance(te.entry, S.FusedTask) else (te.entry,)):
            end[t] = te.end_time
    assert [te.start_time for te in order] == sorted(te.start_time for te in order)
    # per-rank order is the row's order
    for r, row in enumerate(rows):
        assert [te.entry for te in order if te.rank == r] == row


def test_scheduler_errors():
    rows = S.preprocess_schedule_tasks(S.Std1F1B(2).tasks(2), 0, False)
    bad = [rows[0], rows[1][::-1]]
    with pytest.raises(AssertionError, match="Schedule does not honor data dependencies"):
        core.order_tasks(bad, 2)
    F = lambda s, m: S.Task.make(s, m, TaskType.FWD)
    # bwd_0__0 waits for bwd_1__0, which no row holds... but a task nobody can
    # ever start leaves the rest of the row unscheduled
    stuck = [[F(0, 0), S.Task.make(0, 0, TaskType.BWD)], [S.Task.make(1, 0, TaskType.BWD), F(1, 0)]]
    with pytest.raises(AssertionError, match="does not honor data dependencies"):
        core.order_tasks(stuck, 2)


@pytest.mark.parametrize("sched,n,rank,stages,live,split", [
    (S.Std1F1B(4), 16, 0, [0], 4, False),
    (S.Interleaved1F1B(8, 4), 32, 0, [0, 4], 11, False),
    (S.ZeroBubble(8), 24, 1, [1], 8, True),
    (S.ZeroBubble(8), 24, 0, [0], 8, False),
    (S.DualPipeV(8, 4), 16, 0, [0, 7], 8, True),
    (S.DualPipeV(8, 4), 16, 1, [1, 6], 8, True),
])
def test_rank_plans_for_the_benchmark_configs(sched, n, rank, stages, live, split):
    plan = make_rank_plan(sched, n, rank)
    assert plan.stages == stages and plan.split_backward == split
    assert plan.max_live <= live + 4 and plan.max_live >= 1
    fw = [p for p in plan.tasks if p.exec_kind is TaskType.FWD]
    assert len(fw) == n * len(stages)
    if rank == 0:       # the first stage's backward is never split
        assert all(p.exec_kind is not TaskType.BWD_W for p in plan.tasks if p.task.stage_id == 0)


# ---------------------------------------------------------------------------
# tracing the loop body: what a stage may contain, and what the loss may read
# ---------------------------------------------------------------------------
def _trace(body):
    from jaxpp_amd.pipelining import yield_scope
    with tracing.tracing() as tr, yield_scope():
        out = body(tr.index)
    return tr, out


def test_a_stage_is_whatever_lies_between_two_markers():
    """Stages of different depth and of different layer families (reference:
    clusters_to_tasks, src/jaxpp/core.py:1063-1118); examples/basic.py:125-131 places its
    markers in front of layer i for i % n == 0, which splits 4 layers 3 + 1."""
    dec = LayerSpec("decoder", 128, 2, 256, 128, 1, causal=True)
    bert, block = jaxpp.nn.TransformerLayer(SPEC), jaxpp.nn.TransformerLayer(dec)
    x = np.zeros((4, 128, 128), np.float32)
    params = [bert.init(0, i) for i in range(3)] + [block.init(0, 3)]

    def body(i):
        h = jaxpp.take(x, i, 0)
        for li, p in enumerate(params):
            if li == 3:
                h = jaxpp.mark_stage_end(h)
            h = (bert if li < 3 else block).apply(p, h)
        h = jaxpp.mark_stage_end(h)
        return jaxpp.nn.mse_loss(h, jaxpp.take(x, i, 0)) / 4

    tr, _ = _trace(body)
    staged = core.cluster_ops(tr, 2)
    assert [len(s) for s in staged.stage_layers] == [3, 1]
    assert [sp.family for sp, _ in staged.stage_layers[0]] == ["bert"] * 3
    assert staged.stage_layers[1][0][0].family == "decoder"
    assert staged.input_index == 0 and staged.target == ("input", 0) and staged.has_loss
    assert len(tr.inputs) == 1                    # the same array taken twice is one input
    segs = core._segments(staged.stage_layers[0] + staged.stage_layers[1])
    assert [(sg.spec.family, len(sg.layers), sg.first) for sg in segs] == [("bert", 3, 0), ("decoder", 1, 3)]
    with pytest.raises(AssertionError, match="found 2 expected 3"):
        core.cluster_ops(tr, 3)


def test_loss_target_must_be_an_input_or_a_constant():
    layer = jaxpp.nn.TransformerLayer(SPEC)
    p = layer.init()
    x, y = np.zeros((2, 128, 128), np.float32), np.ones((2, 128, 128), np.float32)

    def second_input(i):
        h = jaxpp.mark_stage_end(layer.apply(p, jaxpp.take(x, i)))
        return jaxpp.nn.mse_loss(h, jaxpp.take(y, i))
    tr, _ = _trace(second_input)
    staged = core.cluster_ops(tr, 1)
    assert staged.input_index == 0 and staged.target == ("input", 1) and len(tr.inputs) == 2

    const = np.full((128, 128), 0.5, np.float32)
    tr, _ = _trace(lambda i: jaxpp.nn.mse_loss(jaxpp.mark_stage_end(layer.apply(p, jaxpp.take(x, i))), const))
    kind, arr = core.cluster_ops(tr, 1).target
    assert kind == "const" and arr is not None and arr.shape == (128, 128)

    def computed_target(i):
        h = layer.apply(p, jaxpp.take(x, i))
        return jaxpp.nn.mse_loss(jaxpp.mark_stage_end(h), h)
    with pytest.raises(NotImplementedError, match="microbatched input of the loop or a constant"):
        _trace(computed_target)
    with pytest.raises(ValueError, match="target of shape"):
        _trace(lambda i: jaxpp.nn.mse_loss(layer.apply(p, jaxpp.take(x, i)), np.zeros((3, 3))))

    def loss_on_an_earlier_value(i):
        h0 = layer.apply(p, jaxpp.take(x, i))
        jaxpp.mark_stage_end(layer.apply(p, h0))
        return jaxpp.nn.mse_loss(h0, jaxpp.take(x, i))
    tr, _ = _trace(loss_on_an_earlier_value)
    with pytest.raises(NotImplementedError, match="output of the last layer of the last stage"):
        core.cluster_ops(tr, 1)

    def not_a_chain(i):
        a = layer.apply(p, jaxpp.take(x, i))
        b = layer.apply(p, jaxpp.take(x, i))          # reads the input again, not `a`
        return jaxpp.nn.mse_loss(jaxpp.mark_stage_end(b), jaxpp.take(x, i))
    tr, _ = _trace(not_a_chain)
    with pytest.raises(NotImplementedError, match="single chain"):
        core.cluster_ops(tr, 1)


def test_value_and_grad_remembers_what_it_differentiates():
    layer = jaxpp.nn.TransformerLayer(SPEC)
    p = layer.init()
    x = np.zeros((2, 128, 128), np.float32)

    def loss_fn(pars, mb):
        res = jaxpp.mark_stage_end(layer.apply(pars, mb))
        raw = jaxpp.nn.mse_loss(res, mb)
        return raw / 2, (raw, res)            # differentiated: raw / 2; returned too: raw

    tr, out = _trace(lambda i: jaxpp.value_and_grad(loss_fn, has_aux=True)(p, jaxpp.take(x, i)))
    (scaled, (raw, _)), grads = out
    assert tr.differentiated is scaled and scaled.producer == ("mse", 0.5) and raw.producer == ("mse", 1.0)
    assert set(grads) == set(p) and all(isinstance(g, tracing.GradOf) for g in grads.values())
    with pytest.raises(TypeError, match="differentiates a scalar loss"):
        _trace(lambda i: jaxpp.value_and_grad(lambda pars, mb: layer.apply(pars, mb))(p, jaxpp.take(x, i)))


def test_treduce_i_takes_the_loop_index():
    x = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    np.testing.assert_array_equal(jaxpp.take(x, 1, axis=1), x[:, 1])
    with pytest.raises(ValueError, match="length must be positive"):
        jaxpp.treduce_i(lambda i: i, 0, S.Std1F1B(1))
    with pytest.raises(TypeError, match="never indexed an array"):
        jaxpp.treduce_i(lambda i: 0, 2, S.Std1F1B(1))
    with pytest.raises(AssertionError, match="has 2 entries along the indexed axis, the loop runs 3"):
        jaxpp.treduce_i(lambda i: jaxpp.take(x, i), 3, S.Std1F1B(1))
    with pytest.raises(RuntimeError, match="only meaningful while its loop body is traced"):
        jaxpp.take(x, tracing.MicrobatchIndex())


def test_stage_lifetimes_per_stage():
    rows = S.preprocess_schedule_tasks(S.ZeroBubble(2).tasks(4), 0, False)
    peak, split = core._stage_lifetimes(rows, 2)
    assert split == [False, True] and peak == [2, 2]
    rows = S.preprocess_schedule_tasks(S.Interleaved1F1B(4, 2).tasks(4), 0, False)
    peak, split = core._stage_lifetimes(rows, 4)
    assert split == [False] * 4 and all(1 <= p <= 4 for p in peak)


def test_schedule_task_fusion_switch(monkeypatch):
    """JAXPP_DISABLE_SCHEDULE_TASK_FUSION (src/jaxpp/env_vars.py:10-12, read at
    src/jaxpp/core.py:2559-2563): with it set, a rank's plan and the global order run the
    members of a fused table entry one after the other; spellings as the reference's
    parse_bool, anything else an error."""
    sched, n = S.Interleaved1F1B(num_stages=4, mpmd_dim=2, fuse_steady_state=True), 8
    monkeypatch.delenv("JAXPP_DISABLE_SCHEDULE_TASK_FUSION", raising=False)
    fused = make_rank_plan(sched, n, 0)
    groups = [pt.group for pt in fused.tasks]
    assert len(set(groups)) < len(groups)                  # some entries hold two tasks
    for spelling in ("1", "true", "T", "yes", "Y"):
        monkeypatch.setenv("JAXPP_DISABLE_SCHEDULE_TASK_FUSION", spelling)
        assert S.schedule_task_fusion_disabled()
        flat = make_rank_plan(sched, n, 0)
        assert len({pt.group for pt in flat.tasks}) == len(flat.tasks)
        assert [pt.task for pt in flat.tasks] == [pt.task for pt in fused.tasks]
        assert flat.max_live == fused.max_live
        order = core.validate_schedule(sched, n)
        assert all(not isinstance(e.entry, S.FusedTask) for e in order)
    for spelling in ("0", "false", "no"):
        monkeypatch.setenv("JAXPP_DISABLE_SCHEDULE_TASK_FUSION", spelling)
        assert not S.schedule_task_fusion_disabled()
        assert [pt.group for pt in make_rank_plan(sched, n, 0).tasks] == groups
    # an explicit argument wins over the environment
    monkeypatch.setenv("JAXPP_DISABLE_SCHEDULE_TASK_FUSION", "1")
    assert [pt.group for pt in make_rank_plan(sched, n, 0, unpack_fused_tasks=False).tasks] == groups
    monkeypatch.setenv("JAXPP_DISABLE_SCHEDULE_TASK_FUSION", "maybe")
    with pytest.raises(ValueError, match="Unsupported value JAXPP_DISABLE_SCHEDULE_TASK_FUSION=maybe"):
        make_rank_plan(sched, n, 0)
