"""CPU oracle: one pipeline rank's share of the microbatch loop, the whole
pipeline, and the sequential loop every schedule must equal.

TEST INFRASTRUCTURE ONLY (see oracle/layers.py).

Follows the reference's run-time structure:

* ``treduce`` semantics: ``state = op.state(...)``; for each microbatch in
  order ``state = op.update(state, fun(xs[i]), i)`` with losses concatenated
  and gradients added (src/jaxpp/training.py:106-169, :187-194;
  sequential definition in src/jaxpp/jax_primitives.py:579-607).
* a rank executes its row of the preprocessed task table in order
  (src/jaxpp/core.py:2550-2589); fused groups run their members in order.
* accumulate-adds live in the backward task of the stage that produced the
  gradient and microbatches ascend per (stage, kind), so per-parameter
  summation order does not depend on the schedule
  (src/jaxpp/core.py:903-918, src/jaxpp/schedules.py:64-72).
* a residual lives from the forward task that made it to its last consumer:
  BWD, or BWD_W when the backward is split (src/jaxpp/core.py:1812-1890).
"""
from __future__ import annotations

import numpy as np

from . import layers as L


def _flatten(row):
    out = []
    for e in row:
        if e is None:
            continue
        if isinstance(e, tuple) and not hasattr(e, "stage_id"):
            out.extend(e)
        else:
            out.append(e)
    return out


class RankOracle:
    """One rank holding one or more stages ("chunks"), each a list of layers."""

    def __init__(self, cfg: L.LayerCfg, chunks: dict, nm: L.Numerics,
                 round_wgrad: bool = False, layer_cfgs: dict | None = None):
        """``layer_cfgs``: stage_id -> [LayerCfg per layer] for stages whose layers differ
        in shape or family; every other layer is a ``cfg`` layer."""
        self.cfg, self.nm, self.round_wgrad = cfg, nm, round_wgrad
        self.layer_cfgs = layer_cfgs or {}
        self.chunks = chunks                       # stage_id -> [param dict per layer]
        self.acc = {s: [{k: np.zeros(v.shape, np.float32) for k, v in p.items()}
                        for p in ps] for s, ps in chunks.items()}
        self.stash, self.wstash = {}, {}
        self.live = self.peak_live = 0
        # mixture layers: per (stage, microbatch) and layer, every token's gap between its
        # last selected router logit and the best one left out (a small gap = a near tie,
        # where top-k selection is discontinuous)
        self.router_margin = {}
        # (stage, microbatch) -> [expert ids [T, top_k] per layer] to impose on mixture layers
        # (see layers.layer_fwd), and how many tokens that changed per layer
        self.forced_ids = {}
        self.forced_changes = {}

    # -- tasks -----------------------------------------------------------
    def cfg_of(self, stage, li):
        return self.layer_cfgs[stage][li] if stage in self.layer_cfgs else self.cfg

    def fwd(self, stage, mb, x):
        sts = []
        for li, p in enumerate(self.chunks[stage]):
            forced = self.forced_ids.get((stage, mb))
            x, st = L.layer_fwd(self.cfg_of(stage, li), p, x, self.nm,
                                forced[li] if forced is not None else None)
            sts.append(st)
            if forced is not None and "own_ids" in st:
                changed = (np.sort(st["own_ids"], -1) != np.sort(st["ids"], -1)).any(-1)
                self.forced_changes.setdefault((stage, mb), []).append(changed)
            if "logits" in st:
                k = self.cfg_of(stage, li).top_k
                srt = np.sort(st["logits"].astype(np.float64), axis=-1)
                self.router_margin.setdefault((stage, mb), []).append(srt[:, -k] - srt[:, -k - 1])
        self.stash[stage, mb] = sts
        self.live += 1
        self.peak_live = max(self.peak_live, self.live)
        return x

    def _add(self, stage, li, name, g):
        a = self.acc[stage][li][name]
        a += np.asarray(g, dtype=np.float32)

    def bwd_i(self, stage, mb, dy):
        sts = self.stash[stage, mb]
        wsts = [None] * len(sts)
        for li in reversed(range(len(sts))):
            dy, wst, small = L.layer_bwd_i(self.cfg_of(stage, li), self.chunks[stage][li], sts[li], dy,
                                           self.nm)
            wsts[li] = wst
            for name, g in small.items():
                self._add(stage, li, name, g)
        self.wstash[stage, mb] = wsts
        return dy

    def bwd_w(self, stage, mb):
        sts, wsts = self.stash.pop((stage, mb)), self.wstash.pop((stage, mb))
        for li in reversed(range(len(sts))):
            for name, g in L.layer_bwd_w(self.cfg_of(stage, li), sts[li], wsts[li], self.nm).items():
                if self.round_wgrad:
                    g = self.nm.rt(g.astype(np.float32))
                self._add(stage, li, name, g)
        self.live -= 1

    def bwd(self, stage, mb, dy):
        dx = self.bwd_i(stage, mb, dy)
        self.bwd_w(stage, mb)
        return dx

    # -- a row of the table ------------------------------------------------
    def run_row(self, row, x_in, dy_in, first_stage_id=0):
        """``x_in(stage, mb)`` / ``dy_in(stage, mb)`` supply the boundary
        tensors.  A first-stage BWD_I stands for the whole backward (the
        table's W half was merged into it).  Returns {(stage, mb): y} and
        {(stage, mb): dx}."""
        ys, dxs = {}, {}
        for t in _flatten(row):
            kind, s, m = t.fwd_or_bwd.name, t.stage_id, t.mubatch_idx
            if kind == "FWD":
                ys[s, m] = self.fwd(s, m, x_in(s, m))
            elif kind == "BWD" or (kind == "BWD_I" and s == first_stage_id and t.latency == 2):
                dxs[s, m] = self.bwd(s, m, dy_in(s, m))
            elif kind == "BWD_I":
                dxs[s, m] = self.bwd_i(s, m, dy_in(s, m))
            elif kind == "BWD_W":
                self.bwd_w(s, m)
            else:
                raise ValueError(kind)
        assert not self.stash and not self.wstash, "table left residuals alive"
        return ys, dxs


# ---------------------------------------------------------------------------
# whole model: sequential loop and scheduled pipeline (cfg "CPU plumbing")
# ---------------------------------------------------------------------------
def treduce_sequential(cfg, stage_layers, xs, nm, round_wgrad=False, targets=None,
                       layer_cfgs=None, preds=None):
    """The loop as ``treduce`` defines it: microbatches in order, every stage
    forward then backward; losses concatenated, gradients summed.  The loss
    compares the last stage's output with ``targets[m]`` (default: the
    microbatch itself, as in the reference's examples).  A list passed as
    ``preds`` receives the last stage's output of every microbatch, in order."""
    n = len(xs)
    targets = xs if targets is None else targets
    ro = RankOracle(cfg, dict(enumerate(stage_layers)), nm, round_wgrad, layer_cfgs)
    losses = np.zeros(n, np.float32)
    S = len(stage_layers)
    for m in range(n):
        a = xs[m]
        for s in range(S):
            a = ro.fwd(s, m, a)
        if preds is not None:
            preds.append(a)
        losses[m], d = L.mse_loss(a, targets[m], n, nm.acc)
        d = nm.rt(d.astype(np.float32))
        for s in reversed(range(S)):
            d = ro.bwd(s, m, d)
    return losses, ro.acc


def run_pipeline(cfg, stage_layers, rows, mpmd_idx_of_stage, xs, nm, round_wgrad=False):
    """Every rank runs its preprocessed row; a task waits for the boundary
    tensor it consumes.  Ranks are polled round-robin, which is one valid
    interleaving of the per-rank orders; a row that can never progress raises
    like the reference's scheduler does (src/jaxpp/core.py:2050-2060)."""
    n, S = len(xs), len(stage_layers)
    n_ranks = len(rows)
    ranks = []
    for r in range(n_ranks):
        chunks = {s: stage_layers[s] for s in range(S) if mpmd_idx_of_stage[s] == r}
        ranks.append(RankOracle(cfg, chunks, nm, round_wgrad))
    act, cot = {}, {}                       # (stage, mb) -> input activation / cotangent
    for m in range(n):
        act[0, m] = xs[m]
    losses = np.zeros(n, np.float32)
    pos = [0] * n_ranks
    flat = [_flatten(r) for r in rows]
    while any(pos[r] < len(flat[r]) for r in range(n_ranks)):
        progressed = False
        for r in range(n_ranks):
            if pos[r] >= len(flat[r]):
                continue
            t = flat[r][pos[r]]
            kind, s, m = t.fwd_or_bwd.name, t.stage_id, t.mubatch_idx
            ro = ranks[r]
            if kind == "FWD":
                if (s, m) not in act:
                    continue
                y = ro.fwd(s, m, act.pop((s, m)))
                if s == S - 1:
                    losses[m], d = L.mse_loss(y, xs[m], n, nm.acc)
                    cot[s, m] = nm.rt(d.astype(np.float32))
                else:
                    act[s + 1, m] = y
            elif kind == "BWD_W":
                if (s, m) not in ro.wstash:
                    continue
                ro.bwd_w(s, m)
            else:
                if (s, m) not in cot or (s, m) not in ro.stash:
                    continue
                whole = kind == "BWD" or (s == 0 and t.latency == 2)
                d = cot.pop((s, m))
                dx = ro.bwd(s, m, d) if whole else ro.bwd_i(s, m, d)
                if s > 0:
                    cot[s - 1, m] = dx
            pos[r] += 1
            progressed = True
        if not progressed:
            raise AssertionError("Schedule does not honor data dependencies.")
    acc = {}
    for ro in ranks:
        acc.update(ro.acc)
    return losses, acc, max(ro.peak_live for ro in ranks)


def adam_step(params, grads, m, v, step, lr=1e-3, b1=0.9, b2=0.999, eps=1e-8):
    """optax.adam defaults (examples/basic.py:234 uses the same transform)."""
    out = {}
    for k in params:
        g = grads[k].astype(np.float32)
        m[k] = b1 * m[k] + (1 - b1) * g
        v[k] = b2 * v[k] + (1 - b2) * g * g
        mh = m[k] / (1 - b1 ** step)
        vh = v[k] / (1 - b2 ** step)
        out[k] = (params[k].astype(np.float32) - lr * mh / (np.sqrt(vh) + eps)).astype(params[k].dtype)
    return out
