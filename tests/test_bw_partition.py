"""Which operations of a stage's backward go into BWD_I and which into BWD_W.

The reference splits a backward task with ``partition_eqns(eqns, tgt_vars,
is_partial_bwd=True, memory_scarce=True)`` (src/jaxpp/jaxpr_utils.py:105-169, called at
src/jaxpp/core.py:1080-1085).  ``partition`` below restates that rule on a plain description
of an operation graph (primitive kind, operands, results, byte sizes):

1. walking the operations backwards, everything the target variables (the cotangent handed to
   the previous stage) depend on is scheduled first - the input-gradient task;
2. then, walking the remaining operations forwards, an operation also moves to the first task
   unless it is a ``dot_general``, or reads something defined by an operation that stays
   behind, or its results are larger than its operands;
3. what stays behind is the weight-gradient task.

The graphs are the backward of each layer family as ``oracle/layers.py`` computes it, written
down operation by operation; the test checks that the rule puts into the two tasks exactly what
``layer_bwd_i`` and ``layer_bwd_w`` (and, on the device, ``layer_bwd_i`` / ``layer_bwd_w`` of
``csrc/stage.hip``, which the GPU tests hold against them) return.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import pytest

from oracle import layers as L

DOT = "dot_general"


@dataclass(frozen=True)
class Op:
    name: str
    prim: str
    ins: tuple
    outs: tuple


def partition(ops, sizes, targets):
    """src/jaxpp/jaxpr_utils.py:105-169 with memory_scarce=True (no remat equations)."""
    used = set(targets)
    left = list(ops)
    first_rev = []
    for i in reversed(range(len(ops))):                         # :126-139
        if any(o in used for o in ops[i].outs):
            left[i] = None
            first_rev.append(ops[i])
            used.update(ops[i].ins)
    first = list(reversed(first_rev))

    def nbytes(names):                                          # :141-142
        return sum(sizes[n] for n in names)

    if first and any(op is not None for op in left):            # :144
        defined_behind = set()
        for i, op in enumerate(left):                           # :156-171
            if op is None:
                continue
            if op.prim == DOT or any(v in defined_behind for v in op.ins):
                defined_behind.update(op.outs)
                continue
            if nbytes(op.outs) <= nbytes(op.ins):
                first.append(op)
                left[i] = None
            else:
                defined_behind.update(op.outs)
    return first, [op for op in left if op is not None]


def task_types(first, behind):
    """src/jaxpp/core.py:1086-1094: the non-empty parts are zipped with (BWD_I, BWD_W), so a
    stage whose first part is empty - nothing to hand to a previous stage - becomes one task of
    type BWD_I holding everything."""
    parts = [p for p in (first, behind) if p]
    return list(zip(parts, ("BWD_I", "BWD_W")))


# ---------------------------------------------------------------------------
# the backward of one layer as an operation graph
# ---------------------------------------------------------------------------
class Graph:
    def __init__(self, tokens, hidden, ffn, qkv_width, param_bytes, act_bytes):
        self.ops, self.sizes = [], {}
        self.T, self.h, self.f, self.w = tokens, hidden, ffn, qkv_width
        self.pb, self.ab = param_bytes, act_bytes

    def var(self, name, elems, nbytes_per):
        self.sizes[name] = elems * nbytes_per
        return name

    def act(self, name, cols):
        return self.var(name, self.T * cols, self.ab)

    def op(self, name, prim, ins, outs):
        self.ops.append(Op(name, prim, tuple(ins), tuple(outs)))

    def weight_grad(self, w, rows, cols, lhs, cot):
        """dot_general -> (convert to the accumulator's type) -> add, as the reference's
        weight-gradient task holds them."""
        self.var(f"d{w}", rows * cols, self.ab)
        self.var(f"acc_{w}", rows * cols, 4)
        self.var(f"acc_{w}'", rows * cols, 4)
        self.op(f"dot:{w}", DOT, [lhs, cot], [f"d{w}"])
        src = f"d{w}"
        if self.ab != 4:
            self.var(f"d{w}_f32", rows * cols, 4)
            self.op(f"convert:{w}", "convert_element_type", [src], [f"d{w}_f32"])
            src = f"d{w}_f32"
        self.op(f"add:{w}", "add", [f"acc_{w}", src], [f"acc_{w}'"])

    def small_grad(self, name, cols, ins, f32_sum):
        """Column sum of a cotangent (bias) or of cotangent x normalised input (norm scale).
        f32_sum: the sum comes out in the accumulator's type (as the device kernels emit it);
        otherwise in the activation type, followed by a convert."""
        out_b = 4 if (f32_sum or self.ab == 4) else self.ab
        self.var(f"g_{name}", cols, out_b)
        self.var(f"acc_{name}", cols, 4)
        self.var(f"acc_{name}'", cols, 4)
        self.op(f"sum:{name}", "reduce_sum", ins, [f"g_{name}"])
        src = f"g_{name}"
        if out_b != 4:
            self.var(f"g_{name}_f32", cols, 4)
            self.op(f"convert:{name}", "convert_element_type", [src], [f"g_{name}_f32"])
            src = f"g_{name}_f32"
        self.op(f"add:{name}", "add", [f"acc_{name}", src], [f"acc_{name}'"])


def llama_backward(act_bytes, f32_small_sums=True, moe=False):
    """oracle/layers.py:436-460 (input gradients) and :474-481 (weight gradients)."""
    g = Graph(tokens=64, hidden=32, ffn=48, qkv_width=64, param_bytes=act_bytes, act_bytes=act_bytes)
    T, h, f, w = g.T, g.h, g.f, g.w
    for name, cols in (("dy", h), ("gu", 2 * f), ("s", f), ("n2", h), ("h1", h), ("ctx", h),
                       ("qkv", w), ("n1", h), ("x", h)):
        g.act(name, cols)
    for name, n in (("Wd", f * h), ("Wgu", h * 2 * f), ("Wo", h * h), ("Wqkv", h * w),
                    ("rms1_g", h), ("rms2_g", h)):
        g.var(name, n, g.pb)
    for name in ("rstd1", "rstd2", "lse"):
        g.var(name, T, 4)
    g.act("ds", f); g.act("dgu", 2 * f); g.act("dn2", h); g.act("dh1_", h); g.act("dh1", h)
    g.act("dctx", h); g.act("dqkv", w); g.act("dn1", h); g.act("dx_", h); g.act("dx", h)
    g.op("dot:ds", DOT, ["dy", "Wd"], ["ds"])
    g.op("swiglu_bwd", "mul", ["gu", "ds"], ["dgu"])
    g.op("dot:dn2", DOT, ["dgu", "Wgu"], ["dn2"])
    g.op("rms2_bwd_dx", "rmsnorm_bwd", ["dn2", "h1", "rstd2", "rms2_g"], ["dh1_"])
    g.op("add:dh1", "add", ["dh1_", "dy"], ["dh1"])
    g.op("dot:dctx", DOT, ["dh1", "Wo"], ["dctx"])
    g.op("attention_bwd+rope", "attention_bwd", ["qkv", "ctx", "dctx", "lse"], ["dqkv"])
    g.op("dot:dn1", DOT, ["dqkv", "Wqkv"], ["dn1"])
    g.op("rms1_bwd_dx", "rmsnorm_bwd", ["dn1", "x", "rstd1", "rms1_g"], ["dx_"])
    g.op("add:dx", "add", ["dx_", "dh1"], ["dx"])
    g.small_grad("rms2_g", h, ["dn2", "h1", "rstd2"], f32_small_sums)
    g.small_grad("rms1_g", h, ["dn1", "x", "rstd1"], f32_small_sums)
    g.weight_grad("Wd", f, h, "s", "dy")
    g.weight_grad("Wgu", h, 2 * f, "n2", "dgu")
    g.weight_grad("Wo", h, h, "ctx", "dh1")
    g.weight_grad("Wqkv", h, w, "n1", "dqkv")
    return g


def bert_backward(act_bytes, f32_small_sums=True):
    """oracle/layers.py:390-412 and :468-470."""
    g = Graph(tokens=64, hidden=32, ffn=128, qkv_width=96, param_bytes=act_bytes, act_bytes=act_bytes)
    T, h, f, w = g.T, g.h, g.f, g.w
    for name, cols in (("dy", h), ("c", h), ("u", f), ("g", f), ("x1", h), ("a", h), ("ctx", h),
                       ("qkv", w), ("x", h)):
        g.act(name, cols)
    for name, n in (("W2", f * h), ("W1", h * f), ("Wo", h * h), ("Wqkv", h * w),
                    ("ln1_g", h), ("ln2_g", h)):
        g.var(name, n, g.pb)
    for name in ("mean1", "rstd1", "mean2", "rstd2", "lse"):
        g.var(name, T, 4)
    for name, cols in (("dc", h), ("dg", f), ("du", f), ("t1", h), ("dx1", h), ("da", h),
                       ("dctx", h), ("dqkv", w), ("t2", h), ("dx", h)):
        g.act(name, cols)
    g.op("ln2_bwd_dx", "layernorm_bwd", ["dy", "c", "mean2", "rstd2", "ln2_g"], ["dc"])
    g.op("dot:dg", DOT, ["dc", "W2"], ["dg"])
    g.op("gelu_bwd", "mul", ["dg", "u"], ["du"])
    g.op("dot:t1", DOT, ["du", "W1"], ["t1"])
    g.op("add:dx1", "add", ["t1", "dc"], ["dx1"])
    g.op("ln1_bwd_dx", "layernorm_bwd", ["dx1", "a", "mean1", "rstd1", "ln1_g"], ["da"])
    g.op("dot:dctx", DOT, ["da", "Wo"], ["dctx"])
    g.op("attention_bwd", "attention_bwd", ["qkv", "ctx", "dctx", "lse"], ["dqkv"])
    g.op("dot:t2", DOT, ["dqkv", "Wqkv"], ["t2"])
    g.op("add:dx", "add", ["t2", "da"], ["dx"])
    g.small_grad("ln2_g", h, ["dy", "c", "mean2", "rstd2"], f32_small_sums)
    g.small_grad("ln2_b", h, ["dy"], f32_small_sums)
    g.small_grad("ln1_g", h, ["dx1", "a", "mean1", "rstd1"], f32_small_sums)
    g.small_grad("ln1_b", h, ["dx1"], f32_small_sums)
    g.small_grad("b2", h, ["dc"], f32_small_sums)
    g.small_grad("b1", f, ["du"], f32_small_sums)
    g.small_grad("bo", h, ["da"], f32_small_sums)
    g.small_grad("bqkv", w, ["dqkv"], f32_small_sums)
    g.weight_grad("W2", f, h, "g", "dc")
    g.weight_grad("W1", h, f, "x1", "du")
    g.weight_grad("Wo", h, h, "ctx", "da")
    g.weight_grad("Wqkv", h, w, "x", "dqkv")
    return g


def oracle_membership(family):
    """The parameters whose gradients layer_bwd_i (its `small`) and layer_bwd_w return, from a
    run of the oracle itself on a small layer."""
    if family == "bert":
        cfg = L.LayerCfg("bert", 32, 2, 64, 16, 1, eps=1e-5)
    else:
        cfg = L.LayerCfg("llama", 32, 2, 48, 16, 1, n_kv_heads=1, head_dim=16, causal=True,
                         rope_theta=1e4, eps=1e-5)
    rng = np.random.default_rng(0)
    p = {k: rng.standard_normal(s).astype(np.float32) * 0.1 for k, s in L.param_shapes(cfg).items()}
    nm = L.Numerics.f32()
    x = rng.standard_normal((cfg.tokens, cfg.hidden)).astype(np.float32)
    _, st = L.layer_fwd(cfg, p, x, nm)
    _, wst, small = L.layer_bwd_i(cfg, p, st, x, nm)
    return set(small), set(L.layer_bwd_w(cfg, st, wst, nm))


def names(ops, kind):
    return {op.name.split(":", 1)[1] for op in ops if op.name.startswith(kind + ":")}


@pytest.mark.parametrize("family,build", [("llama", llama_backward), ("bert", bert_backward)])
@pytest.mark.parametrize("act_bytes", [4, 2])
def test_split_backward_membership_follows_the_reference_rule(family, build, act_bytes):
    g = build(act_bytes)
    first, behind = partition(g.ops, g.sizes, ["dx"])
    small, weights = oracle_membership(family)
    # BWD_I: the whole input-gradient chain (its dot_generals included: they are on the path
    # to the target) plus every small gradient's sum and accumulate
    chain = [op.name for op in g.ops if op.name.split(":")[0] not in ("sum", "convert", "add")
             or op.name in ("add:dx", "add:dh1", "add:dx1")]
    chain = [n for n in chain if not (n.startswith("dot:") and n.split(":")[1] in weights)]
    assert [op.name for op in first[:len(chain)]] == chain
    assert names(first, "sum") == small
    assert names(first, "add") - {"dx", "dh1", "dx1"} == small
    # BWD_W: dot_general -> (convert) -> add of every weight, nothing else
    assert names(behind, "dot") == weights
    assert names(behind, "add") == weights
    assert {op.prim for op in behind} <= {DOT, "convert_element_type", "add"}
    assert [t for _, t in task_types(first, behind)] == ["BWD_I", "BWD_W"]


def test_an_operation_that_grows_its_operand_stays_behind():
    """With small gradients summed in the activation type and converted afterwards (what a
    bf16 model followed by an astype(float32) traces to), the convert - 2 bytes in, 4 out - and
    the add that reads it stay in BWD_W, while the sums themselves still move to BWD_I.  The
    device kernels emit these sums in fp32 directly (no convert exists), which is the
    first case above; the accumulated values are the same either way."""
    g = llama_backward(2, f32_small_sums=False)
    first, behind = partition(g.ops, g.sizes, ["dx"])
    assert names(first, "sum") == {"rms1_g", "rms2_g"}
    assert {"rms1_g", "rms2_g"} <= names(behind, "convert")
    assert {"rms1_g", "rms2_g"} <= names(behind, "add")
    # and an operation that reads something defined behind stays behind whatever its size
    assert all(op.name.split(":")[0] != "sum" for op in behind)


def test_first_stage_is_not_split():
    """Stage 0 hands no cotangent to a previous stage: no target variables, the first part is
    empty, and the whole backward becomes one task of type BWD_I (src/jaxpp/core.py:1086-1094;
    ZeroBubble tables accordingly carry no BWD_W for stage 0)."""
    g = llama_backward(2)
    first, behind = partition(g.ops, g.sizes, [])
    assert first == [] and len(behind) == len(g.ops)
    assert [t for _, t in task_types(first, behind)] == ["BWD_I"]
    from jaxpp_amd import schedules as S
    from jaxpp_amd.plan import make_rank_plan
    from jaxpp_amd.types import TaskType
    plan0 = make_rank_plan(S.ZeroBubble(4), 8, 0)
    assert not plan0.split_backward
    assert all(pt.exec_kind is not TaskType.BWD_W for pt in plan0.tasks)
    plan1 = make_rank_plan(S.ZeroBubble(4), 8, 1)
    assert plan1.split_backward and any(pt.exec_kind is TaskType.BWD_W for pt in plan1.tasks)
