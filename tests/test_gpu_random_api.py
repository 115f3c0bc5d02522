"""Seeded random train steps through the public API (mark_stage_end / treduce /
mpmd_jit_with_loop) against the oracle's sequential loop: random layer family, stage depth,
schedule, pipeline width and microbatch count.

The loss is taken against a target that is independent of the input.  (With the input as the
target, as in the README's autoencoder step, a pre-LN residual stack is ill-conditioned: the
cotangent 2 (pred - x) / N is the difference of two nearly equal bf16 tensors, and a one-ulp
difference in pred is a few per cent of it.  That is a property of that loss, not of the
executor, and the fixed cases of test_gpu_api.py cover that step.)  A whole pipeline of up to
eight layers compounds the rounding of every layer behind it: pipelines of more than four
layers are granted 4e-3 of a tensor's elements outside the elementwise bound instead of the
stage-level 1e-3 (the worst of them 4 x the bound, as everywhere).  That is what the oracle's own
arithmetic does at this depth: evaluated twice on the sweep's six-layer BERT pipeline, with
float32 and with float64 accumulation, it disagrees with itself on 2.5e-3 of the first layer's
QKV weight gradient, by up to 2.5 x (tests/test_oracle_stage.py,
test_bf16_sensitivity_of_a_six_layer_pipeline).  At eight layers a fixed figure stops being one:
a further draw of this sweep (offset 200000, seed 4: BERT, 4 stages of 2 layers) has 4.65e-3 of
that tensor outside the bound while the device is as close to the float32 run as the bf16 oracle
is (0.99 x in the Frobenius norm) and the float32 run itself has 2.4e-2 of its elements outside
the same bound around the bf16 oracle.  (A four-layer one of the same sweep, seed 5, has 1.5e-3 against the
stage-level 1e-3 in the same way.)  So where the float32 run exists, a gradient is also
granted half of that run's own count: the device may disagree with the bf16 oracle on half as
many elements as the unrounded computation does (seen: a fifth at most), and its worst element
may be 1.5 x as far outside the bound as that run's worst is (of 360 further draws one six-layer
pipeline had an element at 4.1 x, with the float32 run's worst of that tensor at 4.0 x; the
float32 run's worst elements sit at 3 - 7 x, the device's at 0.5 - 1.0 of them).  How good the bf16 results are is held separately: no farther from the float32 computation than the bf16 oracle's own
(parity.close_to_truth).  The sweep is for dataflow errors - a wrong slot, a microbatch counted
twice, a stage out of order - which put whole tensors off by their own magnitude."""
import os
from functools import partial

import numpy as np
import pytest

import parity

import jaxpp_amd as jaxpp
from jaxpp_amd import runtime as rt
from jaxpp_amd import schedules as S
from jaxpp_amd.model import LayerSpec
from oracle import layers as L
from oracle import stage as O

pytestmark = pytest.mark.gpu

# further draws on demand: JPP_SWEEP_OFFSET=100000 python -m pytest <this file> (the committed runs use 0)
SWEEP_OFFSET = int(os.environ.get("JPP_SWEEP_OFFSET", "0"))

SPECS = [
    LayerSpec("bert", 256, 4, 512, 128, 1, eps=1e-12),
    LayerSpec("decoder", 256, 2, 512, 128, 1, causal=True, eps=1e-6, gelu_tanh=True),
    LayerSpec("llama", 256, 2, 384, 128, 1, n_kv_heads=1, head_dim=128, causal=True,
              rope_theta=5e5, eps=1e-5),
]


def draw(seed):
    rng = np.random.default_rng(2000 + SWEEP_OFFSET + seed)
    while True:
        spec = SPECS[rng.integers(len(SPECS))]
        p = int(rng.integers(1, 4))
        kind = int(rng.integers(6))
        if kind == 0:
            sched = jaxpp.Std1F1B(p)
        elif kind == 1:
            sched = S.GPipe(p)                           # (not among the reference's exports)
        elif kind == 2:
            sched = jaxpp.Eager1F1B(p)
        elif kind == 3:
            sched = jaxpp.ZeroBubble(p)
        elif kind == 4:
            sched = jaxpp.Interleaved1F1B(p * int(rng.integers(2, 4)), p)
        else:
            sched = jaxpp.DualPipeV(2 * p, p)
        n_mb = int(rng.integers(1, 4)) * p if kind >= 4 else int(rng.integers(1, 7))
        per = int(rng.integers(1, 3))
        try:
            sched.tasks(n_mb)
        except Exception:                               # the schedule rejects the combination
            continue
        if sched.num_stages * per > 8:
            continue
        return spec, sched, p, n_mb, per


# fraction of a tensor's elements granted outside the elementwise bound: the stage-level
# figure, and what pipelines of more than four layers get (see the module's text)
DEEP_BAD_FRAC = 4e-3
# ... and what any gradient gets of the count of the float32 run's elements outside the same bound
# around the bf16 oracle
DEEP_TRUTH_SHARE = 0.5
# ... and how far outside it the worst element may be, in units of that run's worst
TRUTH_EXCESS = 1.5


@pytest.mark.parametrize("seed", range(40))
def test_random_train_step_matches_sequential_loop(seed):
    rt.require_gpu()
    spec, sched, p, n_mb, per = draw(seed)
    n_stages = sched.num_stages
    print(f"seed {seed}: {spec.family} {type(sched).__name__} stages={n_stages} ranks={p} "
          f"n_mb={n_mb} layers/stage={per}", flush=True)
    model = jaxpp.nn.TransformerStack(spec, n_layers=n_stages * per, layers_per_stage=per)
    params = model.init(seed=seed, perturb=True)
    params = {"layers": [{k: L.bf16_round(v) for k, v in q.items()} for q in params["layers"]]}
    rng = np.random.default_rng(seed)
    batch = L.bf16_round(rng.standard_normal((n_mb, spec.tokens, spec.hidden)).astype(np.float32))
    targets = L.bf16_round(rng.standard_normal(batch.shape).astype(np.float32))
    mesh = jaxpp.MpmdMesh(jaxpp.DeviceMesh(np.arange(p).reshape(p, 1), ("mpmd", "data")), "mpmd")

    def loss_fn(pars, mb):
        res = model.apply(pars, mb["hidden"])
        return jaxpp.nn.mse_loss(res, mb["target"]) / n_mb, res

    @partial(jaxpp.mpmd_jit_with_loop, mpmd_mesh=mesh)
    def train_step(pars, batch):
        mubatch_grad = partial(jaxpp.value_and_grad(loss_fn, has_aux=True), pars)
        (losses, pred), grad = jaxpp.treduce(mubatch_grad, batch, schedule=sched)
        return losses, pred, grad

    losses, pred, grad = train_step(params, {"hidden": batch, "target": targets})
    cfg = L.LayerCfg(**spec.as_dict())
    stages = [params["layers"][s * per:(s + 1) * per] for s in range(n_stages)]
    want_pred = []
    want_loss, want_acc = O.treduce_sequential(cfg, stages, list(batch), L.Numerics.bf16(),
                                               targets=list(targets), preds=want_pred)
    # the unrounded computation (float32 on the same bf16-valued inputs): the device may be no
    # farther from it than the bf16 oracle is (expert layers aside: the float32 run may route
    # a token to another expert)
    BAD_FRAC = DEEP_BAD_FRAC if n_stages * per > 4 else parity.STAGE_BAD_FRAC
    EXCESS = parity.MAX_EXCESS
    truth_pred = []
    truth = None if spec.family == "mixtral" else O.treduce_sequential(
        cfg, stages, list(batch), L.Numerics.f32(), targets=list(targets), preds=truth_pred)
    parity.close(np.asarray(losses, np.float32), np.asarray(want_loss), 2e-2, "losses")
    assert pred.shape == batch.shape
    for m in range(n_mb):
        got = np.asarray(pred[m], np.float32)
        parity.close(got, want_pred[m], 2e-2, f"prediction of microbatch {m}", BAD_FRAC, EXCESS)
        if truth:
            parity.close_to_truth(got, want_pred[m], truth_pred[m], f"prediction of microbatch {m}")
    for s in range(n_stages):
        for li in range(per):
            for k, v in want_acc[s][li].items():
                got = np.asarray(grad["layers"][s * per + li][k], np.float32)
                frac, excess = BAD_FRAC, EXCESS
                if truth:
                    t_bad, t_n, t_worst = parity.violations(
                        np.asarray(truth[1][s][li][k], np.float32).reshape(got.shape),
                        np.asarray(v, np.float32).reshape(got.shape), 2e-2)
                    frac = max(frac, DEEP_TRUTH_SHARE * t_bad / max(t_n, 1))
                    excess = max(excess, TRUTH_EXCESS * t_worst)
                parity.close(got, v.reshape(got.shape), 2e-2, f"grad {s}/{li}/{k}", frac, excess)
                if truth:
                    parity.close_to_truth(got, v, truth[1][s][li][k], f"grad {s}/{li}/{k}")
    train_step.close()
