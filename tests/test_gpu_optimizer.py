"""The step after the loop (Adam on the accumulated gradients) through the C ABI against
the oracle's `adam_step`, which tests/test_oracle_stage.py pins on torch.optim.Adam.

Bar: f32 state within 2e-6 of the tensor's largest magnitude after every step (the kernel
contracts multiply-adds and divides by the bias corrections rounded to f32; the oracle
works in numpy f32 with f64 scalars); the bf16 parameters are exactly the rounding of the
kernel's own f32 weights."""
import numpy as np
import pytest

import parity

from jaxpp_amd import runtime as rt
from jaxpp_amd import schedules as S
from jaxpp_amd.model import LayerSpec, boundary_tensor, init_layer_params
from jaxpp_amd.plan import make_rank_plan
from jaxpp_amd.rank_loop import RankLoop
from jaxpp_amd.types import TaskType
from oracle import layers as L
from oracle import stage as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    rt.require_gpu()


close = parity.close


@pytest.mark.parametrize("count", [8 * 256 * 33, 8 * 1000 + 5, 3])
@pytest.mark.parametrize("with_master", [True, False])
def test_adam_flat(count, with_master):
    rng = np.random.default_rng(count + with_master)
    lr, b1, b2, eps, gs = 5e-3, 0.9, 0.999, 1e-8, 0.25
    w0 = L.bf16_round((rng.standard_normal(count) * 0.02).astype(np.float32))
    ms, vs = {"w": np.zeros(count, np.float32)}, {"w": np.zeros(count, np.float32)}
    w = w0.copy()
    d_w = rt.DeviceBuffer.from_numpy(w0) if with_master else None
    d_p = rt.DeviceBuffer.from_numpy(rt.to_bf16_bits(w0))
    d_m = rt.DeviceBuffer.from_numpy(ms["w"])
    d_v = rt.DeviceBuffer.from_numpy(vs["w"])
    for step in (1, 2, 3):
        g = (rng.standard_normal(count) * (10.0 ** rng.integers(-4, 1))).astype(np.float32)
        g[rng.integers(0, count, max(1, count // 50))] = 0.0   # exact zeros: 0 / (0 + eps)
        d_g = rt.DeviceBuffer.from_numpy(g)
        zero = step == 2
        rt.adam_step(count, d_g.ptr, d_m.ptr, d_v.ptr, step,
                     master=d_w.ptr if with_master else None, param=d_p.ptr, lr=lr, b1=b1, b2=b2,
                     eps=eps, grad_scale=gs, zero_grad=zero)
        rt.sync()
        want = O.adam_step({"w": w}, {"w": g * np.float32(gs)}, ms, vs, step, lr, b1, b2,
                           eps)["w"]
        got_m = d_m.download(np.float32, (count,))
        got_v = d_v.download(np.float32, (count,))
        got_p = rt.from_bf16_bits(d_p.download(np.uint16, (count,)))
        close(got_m, ms["w"], 2e-6, f"m step {step}")
        close(got_v, vs["w"], 2e-6, f"v step {step}")
        if with_master:
            got_w = d_w.download(np.float32, (count,))
            close(got_w, want, 2e-6, f"weights step {step}")
            assert np.array_equal(got_p, L.bf16_round(got_w)), "bf16 copy is the rounded f32 weight"
            w = want
        else:
            # the bf16 tensor is the only copy: one rounding per step, compared at its precision
            close(got_p, L.bf16_round(want), 2 ** -7, f"bf16 weights step {step}")
            w = got_p.copy()
        got_g = d_g.download(np.float32, (count,))
        assert np.array_equal(got_g, np.zeros_like(g) if zero else g), "gradient cleared iff asked"


def test_adam_empty_tensor_is_a_no_op():
    buf = rt.DeviceBuffer(64)
    rt.adam_step(0, buf.ptr, buf.ptr, buf.ptr, 1, master=buf.ptr)


def test_adam_rejects_bad_arguments():
    buf = rt.DeviceBuffer(1024)
    with pytest.raises(rt.JppError, match="step counts from 1"):
        rt.adam_step(8, buf.ptr, buf.ptr, buf.ptr, 0, master=buf.ptr)
    with pytest.raises(rt.JppError, match="null operand"):
        rt.adam_step(8, buf.ptr, buf.ptr, buf.ptr, 1)
    with pytest.raises(rt.JppError, match="16-byte aligned"):
        rt.adam_step(8, buf.ptr + 4, buf.ptr, buf.ptr, 1, master=buf.ptr)
    with pytest.raises(rt.JppError, match=r"\[0, 1\)"):
        rt.adam_step(8, buf.ptr, buf.ptr, buf.ptr, 1, master=buf.ptr, b1=1.0)


LLAMA = LayerSpec("llama", 256, 2, 384, 128, 2, n_kv_heads=1, head_dim=128, causal=True,
                  rope_theta=5e5, eps=1e-5)
BERT = LayerSpec("bert", 128, 2, 256, 128, 1, eps=1e-12)


@pytest.mark.parametrize("spec,two_streams", [(LLAMA, False), (LLAMA, True), (BERT, False)])
def test_stage_adam_after_loop(spec, two_streams):
    """Two train steps of one rank: loop, Adam, loop on the updated bf16 parameters, Adam.
    The oracle's Adam consumes the gradients the GPU accumulated, so each step is compared
    on its own."""
    schedule, n_mb, rank, lpc = S.Interleaved1F1B(4, 2), 4, 0, 1
    plan = make_rank_plan(schedule, n_mb, rank)
    shape = (spec.tokens, spec.hidden)
    ex = rt.StageExecutor(spec, plan.n_chunks, lpc, plan.max_live, plan.split_backward, True,
                          two_streams)
    host = {}
    for c, stage in enumerate(plan.stages):
        host[c] = {k: L.bf16_round(v) for k, v in
                   init_layer_params(spec, 3, stage, perturb=True).items()}
        ex.set_params(c, 0, host[c])
    ex.optimizer_init()
    bufs = {}

    def io(pt, lane=0):
        kind = "x" if pt.exec_kind is TaskType.FWD else "dy"
        key = (kind, pt.task.stage_id, pt.task.mubatch_idx)
        if key not in bufs:
            bufs[key] = (rt.DeviceBuffer.from_f32_as_bf16(
                boundary_tensor(kind, pt.task.stage_id, pt.task.mubatch_idx, shape, 0)),
                rt.DeviceBuffer(spec.tokens * spec.hidden * 2))
        return bufs[key][0].ptr, bufs[key][1].ptr

    m = {c: {k: np.zeros_like(v, dtype=np.float32) for k, v in host[c].items()} for c in host}
    v = {c: {k: np.zeros_like(v_, dtype=np.float32) for k, v_ in host[c].items()} for c in host}
    w = {c: {k: a.astype(np.float32) for k, a in host[c].items()} for c in host}
    lr = 1e-2
    for step in (1, 2):
        RankLoop(ex, plan).run(io)
        grads = {c: ex.get_grads(c, 0) for c in host}
        ex.adam_step(step, lr=lr, grad_scale=1.0 / n_mb)
        rt.sync()
        for c in host:
            g = {k: a * np.float32(1.0 / n_mb) for k, a in grads[c].items()}
            w[c] = O.adam_step(w[c], g, m[c], v[c], step, lr)
            state = ex.get_opt_state(c, 0)
            new_p = ex.get_params(c, 0)
            for k in host[c]:
                gw, gm, gv = (a.reshape(host[c][k].shape) for a in state[k])
                close(gm, m[c][k], 2e-6, f"step {step} chunk {c} m[{k}]")
                close(gv, v[c][k], 2e-6, f"step {step} chunk {c} v[{k}]")
                close(gw, w[c][k], 2e-6, f"step {step} chunk {c} weights[{k}]")
                assert np.array_equal(new_p[k].reshape(gw.shape), L.bf16_round(gw)), k
                assert np.abs(gw - host[c][k]).max() > 0, f"{k} did not move"
            zeros = ex.get_grads(c, 0)
            assert all(not a.any() for a in zeros.values()), "accumulators cleared by the step"
    ex.close()


def test_adam_step_runs_weight_gradients_that_are_still_held_back():
    """With grouped weight gradients the last group of a row may be incomplete (3 microbatches
    in pairs): the optimizer step must run what is pending before it reads the accumulators.
    Same loop and step with and without grouping: the same weights (f32 reassociation aside)."""
    spec, schedule, n_mb, lpc = LLAMA, S.Std1F1B(1), 3, 2
    plan = make_rank_plan(schedule, n_mb, 0)
    shape = (spec.tokens, spec.hidden)
    results = []
    for group in (0, 2):
        ex = rt.StageExecutor(spec, plan.n_chunks, lpc, plan.max_live, plan.split_backward, True,
                              False, wgrad_group=group)
        for li in range(lpc):
            ex.set_params(0, li, {k: L.bf16_round(v) for k, v in
                                  init_layer_params(spec, 3, li, perturb=True).items()})
        ex.optimizer_init()
        bufs = {}

        def io(pt, lane=0):
            kind = "x" if pt.exec_kind is TaskType.FWD else "dy"
            key = (kind, pt.task.stage_id, pt.task.mubatch_idx)
            if key not in bufs:
                bufs[key] = (rt.DeviceBuffer.from_f32_as_bf16(
                    boundary_tensor(kind, pt.task.stage_id, pt.task.mubatch_idx, shape, 0)),
                    rt.DeviceBuffer(spec.tokens * spec.hidden * 2))
            return bufs[key][0].ptr, bufs[key][1].ptr

        RankLoop(ex, plan).run(io)
        if group:
            assert ex.live_slots() == 1, "the third microbatch waits for a partner"
        ex.adam_step(1, lr=1e-2, grad_scale=1.0 / n_mb)          # no join, no get_grads before it
        rt.sync()
        assert ex.live_slots() == 0
        results.append([ex.get_opt_state(0, li) for li in range(lpc)])
        ex.close()
    for li in range(lpc):
        for k in results[0][li]:
            for what, a, b in zip(("weights", "m", "v"), results[0][li][k], results[1][li][k]):
                assert np.abs(a).max() > 0
                close(b, a, 1e-5, f"layer {li} {what}[{k}]")


def test_stage_adam_needs_init():
    plan = make_rank_plan(S.Std1F1B(2), 2, 0)
    ex = rt.StageExecutor(BERT, plan.n_chunks, 1, plan.max_live, plan.split_backward, True, False)
    with pytest.raises(rt.JppError, match="optimizer_init has not run"):
        ex.adam_step(1)
    ex.close()


def test_bf16_parameters_are_written_once_per_step_by_the_adam_pass():
    """The reference hoists the cast of the f32 weights to bf16 out of the microbatch loop
    (loop-invariant code motion, src/jaxpp/licm.py:531-644; PERF_GUIDE.md:29-41): the loop
    reads a bf16 copy made once per step.  Here that copy is the stage's parameter storage:
    no task of the loop writes it (its bits are the same after every task of the row), the
    only launches of a step that touch it are the loop's reads and one Adam launch, and after
    that launch it is exactly the rounded f32 weights."""
    spec, schedule, n_mb, rank, lpc = LLAMA, S.Interleaved1F1B(4, 2), 4, 0, 1
    plan = make_rank_plan(schedule, n_mb, rank)
    shape = (spec.tokens, spec.hidden)
    ex = rt.StageExecutor(spec, plan.n_chunks, lpc, plan.max_live, plan.split_backward, True, False)
    for c, stage in enumerate(plan.stages):
        ex.set_params(c, 0, {k: L.bf16_round(v) for k, v in
                             init_layer_params(spec, 3, stage, perturb=True).items()})
    ex.optimizer_init()
    lib = rt.load()

    def param_bits():
        out = []
        for c in range(plan.n_chunks):
            for name, rows, cols in ex.params:
                ptr = ex._ptr(lib.jpp_stage_param_ptr, c, 0, name)
                out.append(rt.download_ptr(ptr, np.uint16, (rows * cols,)))
        return np.concatenate(out)

    x = rt.DeviceBuffer.from_f32_as_bf16(boundary_tensor("x", 0, 0, shape, 0))
    out = rt.DeviceBuffer(spec.tokens * spec.hidden * 2)
    for step in (1, 2):
        before = param_bits()
        with rt.probe("adam") as pr:
            for pt in plan.tasks:
                ex.run_task(pt.exec_kind, pt.chunk, pt.task.mubatch_idx, x.ptr, out.ptr)
                rt.sync()
                np.testing.assert_array_equal(param_bits(), before,
                                              err_msg=f"step {step}: {pt.task} wrote the parameters")
            ex.adam_step(step, lr=1e-2, grad_scale=1.0 / n_mb)
            rt.sync()
        assert pr.launches == 1, "one Adam launch per step rewrites the bf16 copy"
        after = param_bits()
        assert (after != before).any(), "the Adam pass must rewrite the bf16 parameters"
        for c in range(plan.n_chunks):
            state, new_p = ex.get_opt_state(c, 0), ex.get_params(c, 0)
            for k, (w, _, _) in state.items():
                assert np.array_equal(new_p[k].reshape(w.shape), L.bf16_round(w)), k
    ex.close()
