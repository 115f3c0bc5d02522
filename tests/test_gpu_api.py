"""The README's train step (README.md:74-94) through the public API on the
GPU, against the CPU oracle's whole-pipeline executor with the same
parameters and microbatches.  bf16 compute, fp32 accumulation: 2e-2."""
from functools import partial

import numpy as np
import pytest

import jaxpp_amd as jaxpp
from jaxpp_amd import runtime as rt
from jaxpp_amd.model import LayerSpec
from oracle import layers as L
from oracle import stage as O

pytestmark = pytest.mark.gpu


def close(got, want, what, rtol=2e-2):
    scale = float(np.abs(want).max()) + 1e-30
    err = float(np.abs(np.asarray(got, np.float32) - want).max())
    assert err <= rtol * scale, f"{what}: {err:.4g} vs {scale:.4g}"


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
    want_loss, want_acc = O.treduce_sequential(cfg, stages, list(batch), L.Numerics.bf16())
    close(losses, want_loss, "losses")
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
    want_loss, want_acc = O.treduce_sequential(cfg, stages, list(batch), L.Numerics.bf16())
    close(losses, want_loss, "losses")
    for s in range(pp):
        for li in range(per):
            for k, v in want_acc[s][li].items():
                got = grad["layers"][s * per + li][k]
                close(got, v.reshape(got.shape), f"grad {s}/{li}/{k}")
    train_step.close()
