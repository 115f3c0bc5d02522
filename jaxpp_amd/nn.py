"""Model-side building blocks a user's train step is written with: transformer
layers (singly, or as a stack with stage markers) and the mean-squared-error
loss of the reference's examples (README.md:46-78, examples/basic.py:94-133,
:247-250).

Layer arithmetic runs in the HIP kernels; these classes only describe it."""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from jaxpp_amd import tracing
from jaxpp_amd.model import LayerSpec, init_layer_params
from jaxpp_amd.pipelining import mark_stage_end


@dataclass(frozen=True)
class TransformerLayer:
    """One layer of the family ``spec.family``.  A body is a chain of these with
    ``mark_stage_end`` wherever the user wants a stage to end - after every
    ``n`` layers (README.md:67), in front of layer ``i`` for ``i % n == 0``
    (examples/basic.py:125-131, which gives uneven stages), between layers of
    different families."""

    spec: LayerSpec

    def init(self, seed: int = 0, index: int = 0, perturb: bool = False) -> dict:
        return init_layer_params(self.spec, seed, index, perturb)

    def apply(self, params: dict, hidden):
        tr = tracing.current()
        if tr is None or not isinstance(hidden, tracing.Traced):
            raise RuntimeError("a layer is applied inside jaxpp_amd.treduce under "
                               "mpmd_jit_with_loop (there is no eager CPU path)")
        want = (self.spec.tokens, self.spec.hidden)
        if tuple(hidden.shape) != want:
            raise ValueError(f"microbatch of shape {hidden.shape}, layer expects {want}")
        out = tr.fresh(want, ("layer", len(tr.ops)))
        tr.ops.append(("layer", self.spec, params, hidden.uid, out.uid))
        return out


@dataclass(frozen=True)
class TransformerStack:
    """``n_layers`` identical layers; ``mark_stage_end`` after every
    ``layers_per_stage`` layers (the README's ``(i + 1) % n == 0`` placement);
    ``layers_per_stage = 0`` places no markers."""

    spec: LayerSpec
    n_layers: int
    layers_per_stage: int = 0

    def init(self, seed: int = 0, perturb: bool = False) -> dict:
        return {"layers": [init_layer_params(self.spec, seed, i, perturb)
                           for i in range(self.n_layers)]}

    def apply(self, params: dict, hidden):
        layer = TransformerLayer(self.spec)
        for i, layer_params in enumerate(params["layers"]):
            hidden = layer.apply(layer_params, hidden)
            if self.layers_per_stage and (i + 1) % self.layers_per_stage == 0:
                hidden = mark_stage_end(hidden)
        return hidden


def mse_loss(pred, target):
    """``mean((pred - target) ** 2)`` of one microbatch; divide the result by
    the number of microbatches as the reference's examples do.  ``target`` is a
    microbatched input of the loop (the hidden states themselves in the
    reference's examples, or a second array of ``xs``) or a constant array of
    ``pred``'s shape."""
    tr = tracing.current()
    if tr is None or not isinstance(pred, tracing.Traced):
        raise RuntimeError("mse_loss runs inside jaxpp_amd.treduce")
    if isinstance(target, tracing.Traced):
        if target.producer[0] != "input":
            raise NotImplementedError("the target of mse_loss is a microbatched input of the loop "
                                      "or a constant array, not a computed value")
        tgt = ("input", target.producer[1])
    else:
        arr = np.asarray(target, dtype=np.float32)
        if arr.shape != tuple(pred.shape):
            raise ValueError(f"mse_loss: target of shape {arr.shape}, prediction {pred.shape}")
        tgt = ("const", arr)
    tr.ops.append(("mse", pred.uid, tgt))
    return tr.fresh((), ("mse", 1.0))
