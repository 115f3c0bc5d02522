"""A pipelined train step with jaxpp_amd, in the spelling of the reference's example
(examples/basic.py there: a stack of pre-LN decoder blocks, a stage marker after every
`num_layers // pp` blocks, loss mean((out - in)^2) / num_ubatches, Std1F1B, Adam).

    python examples/basic.py [--pp 2] [--num-ubatches 4] [--steps 3] [--dtype bf16|f32]

The step runs twice per iteration - once with the schedule asked for and once with the
microbatches one after the other (a one-stage-at-a-time GPipe order) - and the two must agree
bit for bit: the order the schedule puts the tasks in changes no result.  Needs an MI355X and
the built library (`python -m jaxpp_amd.build`).
"""
from __future__ import annotations

import argparse
import os
import sys
import time
from functools import partial

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import jaxpp_amd as jaxpp                     # noqa: E402
from jaxpp_amd import schedules               # noqa: E402
from jaxpp_amd.model import LayerSpec         # noqa: E402


def make_train_step(model, optimizer, mesh, schedule, num_ubatches):
    def loss_fn(params, ubatch):
        out = model.apply(params, ubatch)      # marks the end of a stage every few blocks
        return jaxpp.nn.mse_loss(out, ubatch) / num_ubatches, out

    @partial(jaxpp.mpmd_jit_with_loop, mpmd_mesh=mesh)
    def train_step(opt_state, params, batch):
        ubatch_grad = partial(jaxpp.value_and_grad(loss_fn, has_aux=True), params)
        (losses, preds), grad = jaxpp.treduce(ubatch_grad, batch, schedule=schedule)
        updates, opt_state = optimizer.update(grad, opt_state, params)
        return opt_state, jaxpp.optim.apply_updates(params, updates), losses, preds

    return train_step


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--pp", type=int, default=2, help="pipeline stages (one MPMD group each)")
    ap.add_argument("--num-ubatches", type=int, default=4)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--dtype", choices=["bf16", "f32"], default="bf16")
    ap.add_argument("--hidden", type=int, default=256)
    ap.add_argument("--seq", type=int, default=128)
    args = ap.parse_args(argv)

    spec = LayerSpec("decoder", args.hidden, args.hidden // 128, 3 * args.hidden, args.seq, 2,
                     causal=True, eps=1e-6, gelu_tanh=True, dtype=args.dtype)
    model = jaxpp.nn.TransformerStack(spec, n_layers=2 * args.pp, layers_per_stage=2)
    mesh = jaxpp.MpmdMesh(jaxpp.DeviceMesh(np.arange(args.pp).reshape(args.pp, 1), ("stages", "data")),
                          "stages")
    optimizer = jaxpp.optim.adam(1e-3)
    pipelined = make_train_step(model, optimizer, mesh, jaxpp.Std1F1B(args.pp), args.num_ubatches)
    in_turn = make_train_step(model, optimizer, mesh, schedules.GPipe(args.pp), args.num_ubatches)

    params = model.init(seed=0)
    opt_state = optimizer.init(params)
    batch = np.random.default_rng(0).uniform(
        size=(args.num_ubatches, spec.tokens, spec.hidden)).astype(np.float32)
    history = []
    for step in range(args.steps):
        t0 = time.perf_counter()
        new_state, new_params, losses, preds = pipelined(opt_state, params, batch)
        dt = time.perf_counter() - t0
        _, ref_params, ref_losses, ref_preds = in_turn(opt_state, params, batch)
        np.testing.assert_array_equal(np.asarray(losses), np.asarray(ref_losses))
        np.testing.assert_array_equal(np.asarray(preds), np.asarray(ref_preds))
        for got, want in zip(new_params["layers"], ref_params["layers"]):
            for name in got:
                np.testing.assert_array_equal(np.asarray(got[name]), np.asarray(want[name]), err_msg=name)
        opt_state, params = new_state, new_params
        history.append(float(np.sum(losses)))
        print(f"step {step}: loss {float(np.sum(losses)):.6f}  ({dt * 1e3:.1f} ms incl. host round "
              f"trips; same losses, predictions and parameters with the microbatches in turn)")
    pipelined.close()
    in_turn.close()
    return history


if __name__ == "__main__":
    main()
