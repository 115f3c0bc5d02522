"""The README's train step (README.md:74-94) through the public API on the
GPU, against the CPU oracle's whole-pipeline executor with the same
parameters and microbatches.  bf16 compute, fp32 accumulation: 2e-2."""
from functools import partial

import numpy as np
import pytest

import parity

import jaxpp_amd as jaxpp
from jaxpp_amd import runtime as rt
from jaxpp_amd.model import LayerSpec
from oracle import layers as L
from oracle import stage as O

pytestmark = pytest.mark.gpu


def close(got, want, what, rtol=2e-2):
    parity.close_stage(np.asarray(got, np.float32), np.asarray(want), rtol, what)


@pytest.mark.parametrize("schedule,n_mb,mpmd", [
    (jaxpp.Std1F1B(2), 8, 2), (jaxpp.Interleaved1F1B(4, 2), 4, 2), (jaxpp.ZeroBubble(2), 4, 2),
    (jaxpp.DualPipeV(4, 2), 4, 2),
], ids=["std1f1b", "interleaved", "zerobubble", "dualpipev"])
def test_train_step_matches_oracle_pipeline(schedule, n_mb, mpmd):
    rt.require_gpu()
    print(f"api case {schedule}", flush=True)
    spec = LayerSpec("bert", 256, 4, 1024, 128, 1, eps=1e-12)       # cfg1's layer, one sequence
    n_stages = schedule.num_stages
    model = jaxpp.nn.TransformerStack(spec, n_layers=n_stages, layers_per_stage=1)
    params = model.init(seed=0, perturb=True)
    params = {"layers": [{k: L.bf16_round(v) for k, v in p.items()} for p in params["layers"]]}
    rng = np.random.default_rng(1)
    batch = L.bf16_round(rng.standard_normal((n_mb, spec.tokens, spec.hidden)).astype(np.float32))
    mesh = jaxpp.MpmdMesh(jaxpp.DeviceMesh(np.arange(mpmd).reshape(mpmd, 1), ("mpmd", "data")),
                          "mpmd")

    def loss_fn(pars, mb):
        res = model.apply(pars, mb)
        return jaxpp.nn.mse_loss(res, mb) / n_mb, (res, 4)

    @partial(jaxpp.mpmd_jit_with_loop, mpmd_mesh=mesh)
    def pp_train_step(pars, batch):
        mubatch_grad = partial(jaxpp.value_and_grad(loss_fn, has_aux=True), pars)
        (losses, (pred, _)), grad = jaxpp.treduce(mubatch_grad, batch, schedule=schedule)
        return losses, pred, grad

    with jaxpp.collect_task_times_ms() as stats:
        losses, pred, grad = pp_train_step(params, batch)
    assert losses.shape == (n_mb,) and pred.shape == batch.shape
    assert set(stats) >= {"fwd_0", f"fwd_{n_stages - 1}"}
    assert sum(len(v) for v in stats.values()) == len(
        [t for te in pp_train_step.last_order
         for t in (te.entry if isinstance(te.entry, tuple) else (te.entry,))])

    cfg = L.LayerCfg(**spec.as_dict())
    stages = [[p] for p in params["layers"]]
    want_pred = []
    want_loss, want_acc = O.treduce_sequential(cfg, stages, list(batch), L.Numerics.bf16(),
                                               preds=want_pred)
    close(losses, want_loss, "losses")
    for m in range(n_mb):                   # the returned activation: every microbatch's, stacked
        close(pred[m], want_pred[m], f"prediction of microbatch {m}")
    for s in range(n_stages):
        for k, v in want_acc[s][0].items():
            close(grad["layers"][s][k], v.reshape(grad["layers"][s][k].shape), f"grad {s}/{k}")
    # second call reuses the executors and gives the same numbers
    losses2, _, grad2 = pp_train_step(params, batch)
    np.testing.assert_array_equal(losses, losses2)
    np.testing.assert_array_equal(grad["layers"][0]["Wqkv"], grad2["layers"][0]["Wqkv"])
    pp_train_step.close()


def test_example_model_train_step():
    """The reference's example (examples/basic.py): a stack of pre-LN causal decoder blocks with
    a stage marker after every `num_layers // pp` layers, loss mean((res - batch)**2) /
    num_ubatches, Std1F1B over 2 stages - here 4 blocks of hidden 256 in two stages."""
    rt.require_gpu()
    spec = LayerSpec("decoder", 256, 2, 512, 128, 1, causal=True, eps=1e-6, gelu_tanh=True)
    n_mb, pp, n_layers = 4, 2, 4
    schedule = jaxpp.Std1F1B(pp)
    model = jaxpp.nn.TransformerStack(spec, n_layers=n_layers, layers_per_stage=n_layers // pp)
    params = model.init(seed=0, perturb=True)
    params = {"layers": [{k: L.bf16_round(v) for k, v in p.items()} for p in params["layers"]]}
    rng = np.random.default_rng(2)
    batch = L.bf16_round(rng.uniform(size=(n_mb, spec.tokens, spec.hidden)).astype(np.float32))
    mesh = jaxpp.MpmdMesh(jaxpp.DeviceMesh(np.arange(pp).reshape(pp, 1), ("mpmd", "data")), "mpmd")

    def loss_fn(pars, mb):
        res = model.apply(pars, mb)
        return jaxpp.nn.mse_loss(res, mb) / n_mb, (res, 4)

    @partial(jaxpp.mpmd_jit_with_loop, mpmd_mesh=mesh)
    def train_step(pars, batch):
        mubatch_grad = partial(jaxpp.value_and_grad(loss_fn, has_aux=True), pars)
        (losses, (pred, _)), grad = jaxpp.treduce(mubatch_grad, batch, schedule=schedule)
        return losses, pred, grad

    losses, pred, grad = train_step(params, batch)
    cfg = L.LayerCfg(**spec.as_dict())
    per = n_layers // pp
    stages = [params["layers"][s * per:(s + 1) * per] for s in range(pp)]
    want_pred = []
    want_loss, want_acc = O.treduce_sequential(cfg, stages, list(batch), L.Numerics.bf16(),
                                               preds=want_pred)
    close(losses, want_loss, "losses")
    assert pred.shape == batch.shape
    for m in range(n_mb):
        close(pred[m], want_pred[m], f"prediction of microbatch {m}")
    for s in range(pp):
        for li in range(per):
            for k, v in want_acc[s][li].items():
                got = grad["layers"][s * per + li][k]
                close(got, v.reshape(got.shape), f"grad {s}/{li}/{k}")
    train_step.close()


def _mesh(pp):
    return jaxpp.MpmdMesh(jaxpp.DeviceMesh(np.arange(pp).reshape(pp, 1), ("mpmd", "data")), "mpmd")


def test_uneven_stages_and_mixed_layer_families():
    """A task is whatever lies between two markers (reference: clusters_to_tasks,
    src/jaxpp/core.py:1063-1118).  Three post-LN encoder layers in the first stage and, in the
    second, one encoder layer followed by a pre-LN decoder block - stages of different depth
    and a stage whose layers are of two families - with the markers placed by hand as
    examples/basic.py:125-131 does.  ZeroBubble(2), so the second stage's backward runs split
    across both of its executors.  Against the sequential loop of the oracle."""
    rt.require_gpu()
    bert = LayerSpec("bert", 256, 4, 512, 128, 1, eps=1e-12)
    dec = LayerSpec("decoder", 256, 4, 512, 128, 1, causal=True, eps=1e-6, gelu_tanh=True)
    enc, blk = jaxpp.nn.TransformerLayer(bert), jaxpp.nn.TransformerLayer(dec)
    n_mb, schedule = 4, jaxpp.ZeroBubble(2)
    rnd = lambda p: {k: L.bf16_round(v) for k, v in p.items()}
    params = [rnd(enc.init(0, i, perturb=True)) for i in range(4)] + [rnd(blk.init(0, 4, perturb=True))]
    layers = [enc, enc, enc, enc, blk]
    batch = L.bf16_round(np.random.default_rng(3).standard_normal(
        (n_mb, bert.tokens, bert.hidden)).astype(np.float32))

    def loss_fn(pars, mb):
        h = mb
        for i, (layer, p) in enumerate(zip(layers, pars)):
            if i == 3:
                h = jaxpp.mark_stage_end(h)
            h = layer.apply(p, h)
        h = jaxpp.mark_stage_end(h)
        return jaxpp.nn.mse_loss(h, mb) / n_mb

    @partial(jaxpp.mpmd_jit_with_loop, mpmd_mesh=_mesh(2))
    def train_step(pars, batch):
        return jaxpp.treduce(partial(jaxpp.value_and_grad(loss_fn), pars), batch, schedule=schedule)

    losses, grad = train_step(params, batch)
    cfgs = {0: [L.LayerCfg(**bert.as_dict())] * 3,
            1: [L.LayerCfg(**bert.as_dict()), L.LayerCfg(**dec.as_dict())]}
    want_loss, want_acc = O.treduce_sequential(cfgs[0][0], [params[:3], params[3:]], list(batch),
                                               L.Numerics.bf16(), layer_cfgs=cfgs)
    close(losses, want_loss, "losses")
    for i in range(5):
        s, li = (0, i) if i < 3 else (1, i - 3)
        for k, v in want_acc[s][li].items():
            close(grad[i][k], v.reshape(grad[i][k].shape), f"grad layer {i}/{k}")
    train_step.close()


@pytest.mark.parametrize("target_kind", ["second-input", "constant"])
def test_loss_against_a_target_that_is_not_the_input(target_kind):
    """Two microbatched arrays in `xs` (hidden states and targets), or a constant target held by
    the closure: the loss and its cotangent must come from that target, and a loss value
    returned with another scale than the differentiated one must be reported with its own."""
    rt.require_gpu()
    spec = LayerSpec("bert", 256, 4, 512, 128, 1, eps=1e-12)
    n_mb, pp = 4, 2
    model = jaxpp.nn.TransformerStack(spec, n_layers=2, layers_per_stage=1)
    params = model.init(seed=0, perturb=True)
    params = {"layers": [{k: L.bf16_round(v) for k, v in p.items()} for p in params["layers"]]}
    rng = np.random.default_rng(5)
    batch = L.bf16_round(rng.standard_normal((n_mb, spec.tokens, spec.hidden)).astype(np.float32))
    if target_kind == "second-input":
        targets = L.bf16_round(rng.standard_normal(batch.shape).astype(np.float32))
        xs = {"hidden": batch, "target": targets}
    else:
        const = L.bf16_round(rng.standard_normal(batch.shape[1:]).astype(np.float32))
        targets = np.stack([const] * n_mb)
        xs = {"hidden": batch}

    def loss_fn(pars, mb):
        res = model.apply(pars, mb["hidden"])
        raw = jaxpp.nn.mse_loss(res, mb["target"] if target_kind == "second-input" else const)
        return raw / n_mb, raw

    @partial(jaxpp.mpmd_jit_with_loop, mpmd_mesh=_mesh(pp))
    def train_step(pars, xs):
        fun = partial(jaxpp.value_and_grad(loss_fn, has_aux=True), pars)
        (losses, raw), grad = jaxpp.treduce(fun, xs, schedule=jaxpp.Std1F1B(pp),
                                            operation=((jaxpp.Concat(), jaxpp.Concat()), jaxpp.Add))
        return losses, raw, grad

    losses, raw, grad = train_step(params, xs)
    cfg = L.LayerCfg(**spec.as_dict())
    stages = [[p] for p in params["layers"]]
    want_loss, want_acc = O.treduce_sequential(cfg, stages, list(batch), L.Numerics.bf16(),
                                               targets=list(targets))
    close(losses, want_loss, "losses")
    close(raw, want_loss * n_mb, "unscaled losses")
    # the loss really is against the target: against the input it would be far off
    assert abs(float(losses[0]) - float(L.mse_loss(batch[0], batch[0], n_mb)[0])) > 0.1 * float(want_loss[0])
    for s in range(pp):
        for k, v in want_acc[s][0].items():
            close(grad["layers"][s][k], v.reshape(grad["layers"][s][k].shape), f"grad {s}/{k}")
    train_step.close()


def test_reductions_other_than_the_default_ones():
    """operation=((Add, (Max, Concat(axis=1))), Add): the losses summed to the step's loss, the
    element-wise maximum of the predictions over the microbatches, and the predictions stacked
    along their second axis (reference: training.py:112-166)."""
    rt.require_gpu()
    spec = LayerSpec("bert", 256, 4, 512, 128, 1, eps=1e-12)
    n_mb, pp = 3, 2
    model = jaxpp.nn.TransformerStack(spec, n_layers=2, layers_per_stage=1)
    params = model.init(seed=1, perturb=True)
    params = {"layers": [{k: L.bf16_round(v) for k, v in p.items()} for p in params["layers"]]}
    batch = L.bf16_round(np.random.default_rng(11).standard_normal(
        (n_mb, spec.tokens, spec.hidden)).astype(np.float32))

    def loss_fn(pars, mb):
        res = model.apply(pars, mb)
        return jaxpp.nn.mse_loss(res, mb) / n_mb, (res, res)

    @partial(jaxpp.mpmd_jit_with_loop, mpmd_mesh=_mesh(pp))
    def train_step(pars, xs):
        fun = partial(jaxpp.value_and_grad(loss_fn, has_aux=True), pars)
        return jaxpp.treduce(fun, xs, schedule=jaxpp.Std1F1B(pp),
                             operation=((jaxpp.Add, (jaxpp.Max, jaxpp.Concat(axis=1))), jaxpp.Add))

    (loss, (top, side_by_side)), grad = train_step(params, batch)
    want_pred = []
    want_loss, want_acc = O.treduce_sequential(L.LayerCfg(**spec.as_dict()),
                                               [[p] for p in params["layers"]], list(batch),
                                               L.Numerics.bf16(), preds=want_pred)
    assert np.shape(loss) == ()
    np.testing.assert_allclose(float(loss), float(want_loss.astype(np.float64).sum()), rtol=2e-2)
    assert side_by_side.shape == (spec.tokens, n_mb, spec.hidden)
    for m in range(n_mb):
        close(side_by_side[:, m], want_pred[m], f"prediction of microbatch {m}")
    # the maximum of the GPU's own predictions exactly, and of the oracle's to the bf16 bar
    np.testing.assert_array_equal(top, np.max(np.asarray(side_by_side), axis=1))
    close(top, np.maximum.reduce(want_pred), "maximum over the microbatches")
    for s in range(pp):
        for k, v in want_acc[s][0].items():
            close(grad["layers"][s][k], v.reshape(grad["layers"][s][k].shape), f"grad {s}/{k}")
    train_step.close()


def test_treduce_i_with_an_explicit_length():
    """treduce_i(fun, length): the body picks its microbatch with take(x, i, axis) - here along
    axis 1 of an array laid out [tokens, microbatch, hidden] (reference: training.py:248-340)."""
    rt.require_gpu()
    spec = LayerSpec("bert", 256, 4, 512, 128, 1, eps=1e-12)
    n_mb = 2
    layer = jaxpp.nn.TransformerLayer(spec)
    p = {k: L.bf16_round(v) for k, v in layer.init(0, 0, perturb=True).items()}
    batch = L.bf16_round(np.random.default_rng(7).standard_normal(
        (n_mb, spec.tokens, spec.hidden)).astype(np.float32))
    laid_out = np.ascontiguousarray(batch.transpose(1, 0, 2))      # [tokens, microbatch, hidden]

    def body(pars, i):
        mb = jaxpp.take(laid_out, i, axis=1)
        return jaxpp.nn.mse_loss(jaxpp.mark_stage_end(layer.apply(pars, mb)), mb) / n_mb

    @partial(jaxpp.mpmd_jit_with_loop, mpmd_mesh=_mesh(1))
    def train_step(pars):
        return jaxpp.treduce_i(partial(jaxpp.value_and_grad(body), pars), n_mb,
                               schedule=jaxpp.Std1F1B(1))

    losses, grad = train_step(p)
    want_loss, want_acc = O.treduce_sequential(L.LayerCfg(**spec.as_dict()), [[p]], list(batch),
                                               L.Numerics.bf16())
    close(losses, want_loss, "losses")
    for k, v in want_acc[0][0].items():
        close(grad[k], v.reshape(grad[k].shape), f"grad {k}")
    train_step.close()


def test_the_example_script_runs_and_learns():
    """examples/basic.py: Std1F1B against the microbatches in turn, bit for bit (checked inside
    the script), Adam applied through the public API; the loss on its fixed batch goes down."""
    import importlib.util
    import os
    rt.require_gpu()
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "examples", "basic.py")
    spec = importlib.util.spec_from_file_location("example_basic", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    for argv in (["--steps", "4"], ["--steps", "3", "--dtype", "f32", "--pp", "3", "--num-ubatches", "6"]):
        history = mod.main(argv)
        assert all(np.isfinite(history)) and history[-1] < history[0], history
