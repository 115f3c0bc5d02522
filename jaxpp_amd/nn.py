"""Model-side building blocks a user's train step is written with: a stack of
transformer layers with stage markers, and the mean-squared-error loss of the
reference's examples (README.md:46-78, examples/basic.py:94-133, :247-250).

Layer arithmetic runs in the HIP kernels; these classes only describe it."""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from jaxpp_amd import tracing
from jaxpp_amd.model import LayerSpec, init_layer_params
from jaxpp_amd.pipelining import mark_stage_end


@dataclass(frozen=True)
class TransformerStack:
    """``n_layers`` identical layers; ``mark_stage_end`` after every
    ``layers_per_stage`` layers (the README's ``(i + 1) % n == 0`` placement)."""

    spec: LayerSpec
    n_layers: int
    layers_per_stage: int

    def init(self, seed: int = 0, perturb: bool = False) -> dict:
        return {"layers": [init_layer_params(self.spec, seed, i, perturb)
                           for i in range(self.n_layers)]}

    def apply(self, params: dict, hidden):
        tr = tracing.current()
        if tr is None or not isinstance(hidden, tracing.Traced):
            raise RuntimeError("TransformerStack.apply runs inside jaxpp_amd.treduce under "
                               "mpmd_jit_with_loop (there is no eager CPU path)")
        want = (self.spec.tokens, self.spec.hidden)
        if tuple(hidden.shape) != want:
            raise ValueError(f"microbatch of shape {hidden.shape}, layer expects {want}")
        for i, layer_params in enumerate(params["layers"]):
            tr.ops.append(("layer", self.spec, layer_params))
            hidden = tr.fresh(want, ("layer", i))
            if (i + 1) % self.layers_per_stage == 0:
                hidden = mark_stage_end(hidden)
        return hidden


def mse_loss(pred, target):
    """``mean((pred - target) ** 2)`` of one microbatch; divide the result by
    the number of microbatches as the reference's examples do."""
    tr = tracing.current()
    if tr is None or not isinstance(pred, tracing.Traced):
        raise RuntimeError("mse_loss runs inside jaxpp_amd.treduce")
    tr.ops.append(("mse", pred.uid, getattr(target, "uid", None)))
    return tr.fresh((), ("mse", 1.0))
