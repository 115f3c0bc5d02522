"""Parity at the sizes the bench runs (Llama-3-8B-shaped layer: hidden 4096, 32/8 heads of
128, SwiGLU 14336, 4096 tokens), where the small cases of the other files do not reach: K
loops long enough for the accumulate GEMM to stream its output tile and for the deep-stage
tiles, tile grids of several rounds per CU, attention over 64 key blocks.

* GEMMs: checksums that any dropped, duplicated or misplaced tile breaks - row sums and
  column sums of the f32 result against matrix-vector products of the operands (f64 on the
  host), plus a dense comparison of a few full rows and columns.
* One whole layer (forward, backward, weight gradients) against the numpy oracle, and
  exact doubling of the accumulators when the same microbatch is run twice.

Tolerances: f32 GEMM results 1e-4 sqrt(K) of the largest magnitude, bf16 GEMM results 1e-2 (as
for the small cases); bf16 tensors of the layer 2e-2 of the tensor's largest magnitude."""
import math

import numpy as np
import pytest

import parity

from jaxpp_amd import runtime as rt
from jaxpp_amd import schedules as S
from jaxpp_amd.model import LayerSpec
from jaxpp_amd.plan import make_rank_plan
from oracle import layers as L

from test_gpu_stage import assert_close_to_truth, close, make_params, run_on_gpu, run_on_oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    rt.require_gpu()


def rnd(rng, *shape, scale=1.0):
    return L.bf16_round((rng.standard_normal(shape, dtype=np.float32) * np.float32(scale)))


# (layout, M, N, K, epilogue, tile): the shapes of the bench's GEMM classes and the tiles
# that the small cases cannot drive into their long-K code paths
FULL = [
    ("nn", 4096, 28672, 4096, rt.EPI_F32, 0),       # gate/up projection
    ("nt", 4096, 4096, 14336, rt.EPI_BF16, 0),      # input gradient of the down projection
    ("tn", 4096, 28672, 4096, rt.EPI_ACC_F32, 0),   # weight gradient, streamed accumulator
    ("tn", 14336, 4096, 4096, rt.EPI_ACC_F32, 0),
    ("tn", 1024, 1024, 4096, rt.EPI_ACC_F32, 1),    # 128x128, 3 LDS stages
    ("nn", 1024, 1024, 4096, rt.EPI_F32, 1),        # 128x128, 4 LDS stages
    ("nt", 2048, 1024, 4096, rt.EPI_BF16, 2),       # 256x128
    ("tn", 1024, 2048, 4096, rt.EPI_ACC_F32, 3),    # 128x256, streamed accumulator
    ("nn", 1152, 2048, 4096, rt.EPI_F32, 3),
    # Llama-70B-shaped stage: hidden 8192, 64 + 2 x 8 heads of 128, SwiGLU 28672
    ("nt", 4096, 8192, 28672, rt.EPI_BF16, 0),      # input gradient of the down projection: 448 K-steps
    ("tn", 8192, 10240, 4096, rt.EPI_ACC_F32, 0),   # QKV weight gradient: five full rounds of tiles
]


@pytest.mark.parametrize("lay,m,n,k,epi,tile", FULL, ids=[f"{c[0]}-{c[1]}x{c[2]}x{c[3]}-t{c[5]}" for c in FULL])
def test_gemm_checksums_at_full_size(lay, m, n, k, epi, tile):
    print(f"full-size gemm {lay} {m}x{n}x{k} epi={epi} tile={tile}", flush=True)
    rng = np.random.default_rng(m + n + k)
    ta, tb = {"nn": (0, 1), "nt": (0, 0), "tn": (1, 1)}[lay]
    A = rnd(rng, m, k)                       # logical [M, K]
    B = rnd(rng, n, k, scale=0.05)           # logical [N, K]
    a_h = np.ascontiguousarray(A.T) if ta else A
    b_h = np.ascontiguousarray(B.T) if tb else B
    da, db = rt.DeviceBuffer.from_f32_as_bf16(a_h), rt.DeviceBuffer.from_f32_as_bf16(b_h)
    prev = None
    if epi == rt.EPI_ACC_F32:
        prev = rng.standard_normal((m, n), dtype=np.float32)
        dc = rt.DeviceBuffer.from_numpy(prev)
    else:
        dc = rt.DeviceBuffer(m * n * (2 if epi == rt.EPI_BF16 else 4))
    rt.gemm(da.ptr, db.ptr, dc.ptr, m, n, k, a_h.shape[1], b_h.shape[1], n, ta, tb, epi, tile=tile)
    rt.sync()
    got = (dc.download_bf16((m, n)) if epi == rt.EPI_BF16
           else dc.download(np.float32, (m, n))).astype(np.float64)
    assert np.isfinite(got).all()
    A64, B64 = A.astype(np.float64), B.astype(np.float64)
    p64 = prev.astype(np.float64) if prev is not None else None
    # per-element bound, as for the small cases (a bf16 result: 1e-2, of which rounding to
    # 8 bits takes 2^-8); a sum of n such errors grows like sqrt(n)
    elem = (1e-2 if epi == rt.EPI_BF16 else 1e-4 * math.sqrt(k)) * float(np.abs(got).max())
    row_want = A64 @ B64.sum(axis=0) + (p64.sum(axis=1) if prev is not None else 0.0)
    col_want = B64 @ A64.sum(axis=0) + (p64.sum(axis=0) if prev is not None else 0.0)
    assert np.abs(got.sum(axis=1) - row_want).max() <= elem * math.sqrt(n), "row checksums"
    assert np.abs(got.sum(axis=0) - col_want).max() <= elem * math.sqrt(m), "column checksums"
    rows = sorted(set(int(r) for r in rng.integers(0, m, 6)) | {0, m - 1, 255, 256})
    cols = sorted(set(int(c) for c in rng.integers(0, n, 6)) | {0, n - 1, 255, 256})
    want_rows = A64[rows] @ B64.T + (p64[rows] if prev is not None else 0.0)
    want_cols = A64 @ B64[cols].T + (p64[:, cols] if prev is not None else 0.0)
    assert np.abs(got[rows] - want_rows).max() <= elem, "dense rows"
    assert np.abs(got[:, cols] - want_cols).max() <= elem, "dense columns"


def test_grouped_gemms_at_full_size():
    """The expert products of the Mixtral-shaped stage (8 experts, hidden 4096, SwiGLU 14336,
    2 x 8192 token copies): the down projection over ragged 256-row-padded groups and its
    weight gradient, one output per expert.  Row checksums per expert (a misplaced or dropped
    tile, or a group that multiplies another group's weights, breaks them), dense rows at the
    group edges, untouched padding; for the weight gradient row and column checksums per expert
    and the bit pattern of an expert without rows."""
    print("full-size grouped gemms", flush=True)
    rng = np.random.default_rng(5)
    E, h, f = 8, 4096, 14336
    counts = [3000, 1, 2304, 0, 4095, 2048, 2560, 2376]          # 16384 token copies
    seg = np.zeros(E + 1, np.int32)
    for e, c in enumerate(counts):
        seg[e + 1] = seg[e] + (c + 255) // 256 * 256
    cap = int(seg[E]) + 256
    s_h = np.zeros((cap, f), np.float32)                          # SwiGLU outputs, grouped rows
    for e, c in enumerate(counts):
        s_h[seg[e]:seg[e] + c] = rnd(rng, c, f)
    w2 = rnd(rng, E, f, h, scale=0.05)
    b_seg = rt.DeviceBuffer.from_numpy(seg)
    b_rows = rt.DeviceBuffer.from_numpy(np.array(counts, np.int32))
    b_s, b_w = rt.DeviceBuffer.from_f32_as_bf16(s_h), rt.DeviceBuffer.from_f32_as_bf16(w2)
    out = rt.DeviceBuffer(cap * h * 2)
    out.zero()
    rt.gemm(b_s.ptr, b_w.ptr, out.ptr, cap, h, f, f, h, h, 0, 1, rt.EPI_BF16, seg=b_seg.ptr, n_seg=E,
            group_mode=1, stride_b=f * h, seg_rows=b_rows.ptr)
    rt.sync()
    got = out.download_bf16((cap, h)).astype(np.float64)
    assert np.isfinite(got).all()
    assert not got[seg[E]:].any(), "tiles past the last group must not be written"
    elem = 1e-2 * float(np.abs(got).max())
    for e, c in enumerate(counts):
        if not c:
            continue
        rows = slice(int(seg[e]), int(seg[e]) + c)
        want = s_h[rows].astype(np.float64) @ w2[e].astype(np.float64).sum(axis=1)
        assert np.abs(got[rows].sum(axis=1) - want).max() <= elem * math.sqrt(h), f"row checksums, expert {e}"
        edge = [int(seg[e]), int(seg[e]) + c - 1]
        dense = s_h[edge].astype(np.float64) @ w2[e].astype(np.float64)
        assert np.abs(got[edge] - dense).max() <= elem, f"dense rows, expert {e}"
        assert not got[int(seg[e]) + c:int(seg[e + 1])].any(), f"padding rows of expert {e}"
    # weight gradient of the same projection: dW2[e] += s_e^T dy_e
    dy = np.zeros((cap, h), np.float32)
    for e, c in enumerate(counts):
        dy[seg[e]:seg[e] + c] = rnd(rng, c, h, scale=0.05)
    del out, b_w
    acc0 = rng.standard_normal((E, f, h), dtype=np.float32)
    b_dy, b_acc = rt.DeviceBuffer.from_f32_as_bf16(dy), rt.DeviceBuffer.from_numpy(acc0)
    rt.gemm(b_s.ptr, b_dy.ptr, b_acc.ptr, f, h, 0, f, h, h, 1, 1, rt.EPI_ACC_F32, seg=b_seg.ptr,
            n_seg=E, group_mode=2, stride_c=f * h, seg_rows=b_rows.ptr)
    rt.sync()
    gw = b_acc.download(np.float32, (E, f, h))
    np.testing.assert_array_equal(gw[3], acc0[3])                 # expert without rows
    for e, c in enumerate(counts):
        if not c:
            continue
        rows = slice(int(seg[e]), int(seg[e]) + c)
        se, de = s_h[rows].astype(np.float64), dy[rows].astype(np.float64)
        d = gw[e].astype(np.float64) - acc0[e]
        tol = 1e-4 * math.sqrt(max(c, 64)) * max(float(np.abs(gw[e]).max()), 1.0)
        assert np.abs(d.sum(axis=1) - se.T @ de.sum(axis=1)).max() <= tol * math.sqrt(h), f"dW row checksums, expert {e}"
        assert np.abs(d.sum(axis=0) - de.T @ se.sum(axis=1)).max() <= tol * math.sqrt(f), f"dW column checksums, expert {e}"
        cols = [0, 255, 256, h - 1]
        assert np.abs(d[:, cols] - se.T @ de[:, cols]).max() <= tol, f"dW dense columns, expert {e}"


LLAMA_8B_LAYER = LayerSpec("llama", 4096, 32, 14336, 4096, 1, n_kv_heads=8, head_dim=128,
                           causal=True, rope_theta=5e5, eps=1e-5)


def test_llama_8b_layer_matches_oracle():
    """One layer of the bench's stage at full size: forward, backward and weight gradients of
    one microbatch against the oracle; a second pass over the same microbatch must double
    every accumulator up to f32 rounding (the GEMM folds the old value into its running sums
    part-way through the K loop, so the second sum is rounded differently from the first)."""
    spec, lpc = LLAMA_8B_LAYER, 1
    sched = S.Std1F1B(1)
    plan1 = make_rank_plan(sched, 1, 0)
    params = make_params(spec, plan1.stages, lpc)
    row = S.preprocess_schedule_tasks(sched.tasks(1), 0, False)[0]
    print("full-size layer: oracle", flush=True)
    ys_w, dxs_w, acc_w = run_on_oracle(spec, plan1, params, row)
    print("full-size layer: gpu", flush=True)
    ys, dxs, grads = run_on_gpu(spec, plan1, lpc, params, two_streams=False)
    for key in ys_w:
        parity.close_stage(ys[key], ys_w[key], 2e-2, f"y{key}")
    for key in dxs_w:
        parity.close_stage(dxs[key], dxs_w[key], 2e-2, f"dx{key}")
    for pname, want in acc_w[0][0].items():
        got = grads[0][0][pname]
        parity.close_stage(got, want.reshape(got.shape), 2e-2, f"grad {pname}")
    print("full-size layer: oracle in float32", flush=True)
    assert_close_to_truth(spec, plan1, lpc, params, row, (ys, dxs, grads), (ys_w, dxs_w, acc_w))
    # the same microbatch twice (boundary tensors depend on the microbatch index, so the
    # second pass is a second run of microbatch 0 into the same accumulators)
    shape = (spec.tokens, spec.hidden)
    from jaxpp_amd.model import boundary_tensor
    from jaxpp_amd.types import TaskType
    ex = rt.StageExecutor(spec, 1, lpc, 1, False, True, False)
    ex.set_params(0, 0, params[0][0])
    x = rt.DeviceBuffer.from_f32_as_bf16(boundary_tensor("x", 0, 0, shape, 0))
    dy = rt.DeviceBuffer.from_f32_as_bf16(boundary_tensor("dy", 0, 0, shape, 0))
    out = rt.DeviceBuffer(spec.tokens * spec.hidden * 2)
    for _ in range(2):
        ex.run_task(TaskType.FWD, 0, 0, x.ptr, out.ptr)
        ex.run_task(TaskType.BWD, 0, 0, dy.ptr, out.ptr)
    rt.sync()
    twice = ex.get_grads(0, 0)
    ex.close()
    for pname, once in grads[0][0].items():
        close(twice[pname], 2.0 * once, 1e-5, f"accumulated twice: {pname}")


BERT_LARGE_LAYER = LayerSpec("bert", 1024, 16, 4096, 512, 8, eps=1e-12)


@pytest.mark.parametrize("two_streams", [False, True], ids=["one-stream", "two-streams"])
def test_bert_large_layers_match_oracle(two_streams):
    """Two layers of the BERT-large stage at full size (8 x 512 tokens, hidden 1024, heads of
    64), two microbatches of a 1F1B row, against the oracle."""
    spec, lpc, n = BERT_LARGE_LAYER, 2, 2
    sched = S.Std1F1B(2)
    plan = make_rank_plan(sched, n, 1)
    params = make_params(spec, plan.stages, lpc)
    row = S.preprocess_schedule_tasks(sched.tasks(n), 0, False)[1]
    ys_w, dxs_w, acc_w = run_on_oracle(spec, plan, params, row)
    ys, dxs, grads = run_on_gpu(spec, plan, lpc, params, two_streams=two_streams)
    for key in ys_w:
        parity.close_stage(ys[key], ys_w[key], 2e-2, f"y{key}")
    for key in dxs_w:
        parity.close_stage(dxs[key], dxs_w[key], 2e-2, f"dx{key}")
    for s_ in plan.stages:
        for li in range(lpc):
            for pname, want in acc_w[s_][li].items():
                got = grads[s_][li][pname]
                parity.close_stage(got, want.reshape(got.shape), 2e-2, f"grad {s_}/{li}/{pname}")
    if two_streams:
        assert_close_to_truth(spec, plan, lpc, params, row, (ys, dxs, grads), (ys_w, dxs_w, acc_w))


# ---------------------------------------------------------------------------
# Stage-level parity at the shapes of the 70B-shaped and the Mixtral-shaped stages, and the
# bench's own rows against the same work in sequential order
# ---------------------------------------------------------------------------
def big_params(spec, stages, layers_per_chunk, seed=7):
    """Parameters of large layers without minutes of host random-number generation: matrices are
    windows of one N(0, 0.02^2) pool of 2^26 values at per-tensor offsets (the router scaled to
    unit-variance logits), gains 1 + 0.1 N(0,1), shifts 0.02 N(0,1); all rounded to bf16."""
    rng = np.random.default_rng(seed)
    pool = L.bf16_round(rng.standard_normal(1 << 26, dtype=np.float32) * np.float32(0.02))
    out, k = {}, 0
    for s in stages:
        out[s] = []
        for _ in range(layers_per_chunk):
            p = {}
            for name, shape in spec.param_shapes().items():
                n = int(np.prod(shape))
                k += 1
                if len(shape) >= 2:
                    off = (k * 7919 * 4099) % (pool.size // 2)
                    a = np.resize(pool[off:], n).reshape(shape)
                    if name == "Wr":
                        a = L.bf16_round(a * np.float32(1.0 / (0.02 * math.sqrt(spec.hidden))))
                elif name.endswith("_g"):
                    a = L.bf16_round(1 + 0.1 * rng.standard_normal(shape, dtype=np.float32))
                else:
                    a = L.bf16_round(0.02 * rng.standard_normal(shape, dtype=np.float32))
                p[name] = a
            out[s].append(p)
    return out


def run_on_gpu_with_routing(spec, plan, lpc, params, seed=0, wgrad_group=0):
    """The rank's row, one task at a time; after every forward of a mixture stage the routing
    it chose is read back (jpp_stage_routing).  Returns run_on_gpu's triple and
    {(stage, microbatch): [expert ids per layer]}."""
    from jaxpp_amd.model import boundary_tensor
    from jaxpp_amd.types import TaskType
    shape = (spec.tokens, spec.hidden)
    ex = rt.StageExecutor(spec, plan.n_chunks, lpc, plan.max_live, plan.split_backward, True, False,
                          wgrad_group=wgrad_group)
    for c, stage in enumerate(plan.stages):
        for li in range(lpc):
            ex.set_params(c, li, params[stage][li])
    outs, routing = {}, {}
    for pt in plan.tasks:
        t = pt.task
        if pt.exec_kind is TaskType.BWD_W:
            ex.run_task(pt.exec_kind, pt.chunk, t.mubatch_idx)
            continue
        kind = "x" if pt.exec_kind is TaskType.FWD else "dy"
        src = ex.upload_activation(boundary_tensor(kind, t.stage_id, t.mubatch_idx, shape, seed))
        dst = ex.new_activation()
        ex.run_task(pt.exec_kind, pt.chunk, t.mubatch_idx, src.ptr, dst.ptr)
        rt.sync()
        outs[kind, t.stage_id, t.mubatch_idx] = ex.download_activation(dst, shape)
        if pt.exec_kind is TaskType.FWD and spec.family == "mixtral":
            routing[t.stage_id, t.mubatch_idx] = [ex.routing(pt.chunk, t.mubatch_idx, li)[0]
                                                  for li in range(lpc)]
    ex.join()
    rt.sync()
    assert ex.live_slots() == 0
    ys = {k[1:]: v for k, v in outs.items() if k[0] == "x"}
    dxs = {k[1:]: v for k, v in outs.items() if k[0] == "dy"}
    grads = {stage: [ex.get_grads(c, li) for li in range(lpc)] for c, stage in enumerate(plan.stages)}
    ex.close()
    return ys, dxs, grads, routing


# Top-2 selection is discontinuous.  The router logits of the GPU and of the oracle differ by a
# few 1e-3 at hidden 4096 (the normalised activations they are computed from agree only to a
# bf16 ulp per element), so a token whose second and third logits are closer than that goes to
# another expert on the two sides, and then its whole row of the layer's output differs.  The
# oracle is therefore held to the routing the device chose (layers.layer_fwd `forced_ids`): the
# comparison then covers everything but the choice itself, which is checked separately - the
# device may differ from the oracle's own choice only for tokens whose deciding logits the
# oracle sees within NEAR_TIE_MARGIN of each other, and only for a few per cent of the tokens.
NEAR_TIE_MARGIN = 2e-2


def check_rank_row(spec, sched, n, rank, lpc, bad_frac=parity.STAGE_BAD_FRAC, wgrad_group=0):
    from jaxpp_amd.model import boundary_tensor
    from oracle import stage as O
    plan = make_rank_plan(sched, n, rank)
    params = big_params(spec, plan.stages, lpc)
    row = S.preprocess_schedule_tasks(sched.tasks(n), 0, False)[rank]
    shape = (spec.tokens, spec.hidden)
    print(f"  gpu: {len(plan.tasks)} tasks", flush=True)
    ys, dxs, grads, routing = run_on_gpu_with_routing(spec, plan, lpc, params, wgrad_group=wgrad_group)
    print("  oracle", flush=True)
    ro = O.RankOracle(L.LayerCfg(**spec.as_dict()), {s_: params[s_] for s_ in plan.stages},
                      L.Numerics.bf16())
    ro.forced_ids = routing
    ys_w, dxs_w = ro.run_row(row, lambda s_, m: L.bf16_round(boundary_tensor("x", s_, m, shape, 0)),
                             lambda s_, m: L.bf16_round(boundary_tensor("dy", s_, m, shape, 0)))
    assert set(ys) == set(ys_w) and set(dxs) == set(dxs_w)
    for key, per_layer in ro.forced_changes.items():
        for li, changed in enumerate(per_layer):
            margin = ro.router_margin[key][li]
            assert changed.sum() <= 0.03 * spec.tokens, f"{key} layer {li}: {changed.sum()} tokens rerouted"
            assert (margin[changed] < NEAR_TIE_MARGIN).all(), (
                f"{key} layer {li}: a token was routed differently although its deciding "
                f"logits are {margin[changed].max():.3g} apart")
            print(f"  {key} layer {li}: {int(changed.sum())} of {spec.tokens} tokens routed at a "
                  f"near tie (largest margin {margin[changed].max() if changed.any() else 0:.2g})",
                  flush=True)
    for key in ys_w:
        parity.close(ys[key], ys_w[key], 2e-2, f"y{key}", bad_frac)
    for key in dxs_w:
        parity.close(dxs[key], dxs_w[key], 2e-2, f"dx{key}", bad_frac)
    for s_ in plan.stages:
        for li in range(lpc):
            for pname, want in ro.acc[s_][li].items():
                got = grads[s_][li][pname]
                parity.close(got, want.reshape(got.shape), 2e-2, f"grad {s_}/{li}/{pname}", bad_frac)


LLAMA_70B_LAYER = LayerSpec("llama", 8192, 64, 28672, 4096, 1, n_kv_heads=8, head_dim=128,
                            causal=True, rope_theta=5e5, eps=1e-5)


def test_llama_70b_layer_on_a_zero_bubble_row_matches_oracle():
    """One layer of the 70B-shaped stage at full size - hidden 8192, 64 query / 8 key-value
    heads of 128, SwiGLU 28672, 4096 tokens - on rank 1 of ZeroBubble(2), two microbatches:
    forward, BWD_I and the deferred BWD_W tasks of a split backward through
    jpp_stage_run_task, against the oracle (outputs, input cotangents, every accumulator).

    Fraction of elements allowed outside the elementwise bound: 4e-3 (none more than 4 x out).
    At this shape the layer's bf16 arithmetic itself is that sensitive: two evaluations of the
    oracle that differ only in accumulating in f32 or in f64 (tests/test_oracle_layers.py,
    test_bf16_sensitivity_of_a_70b_shaped_layer) disagree on 1.0e-3 of the elements of the QKV
    weight gradient - all of them in its key columns, as here - by up to 2.9 x the bound, and on
    2e-4 of the input cotangent's, the first tokens of the sequence ahead; the GPU against the
    oracle: 1.6e-3 (up to 3.7 x) and 4.9e-4 (2.6 x)."""
    print("70B-shaped layer, ZeroBubble(2) rank 1", flush=True)
    # weight gradients of the two microbatches as one product per weight, as the bench runs them
    check_rank_row(LLAMA_70B_LAYER, S.ZeroBubble(2), 2, 1, 1, bad_frac=4e-3, wgrad_group=2)


# The oracle multiplies on the host: at the bench's 2 x 4096 tokens the eight layer passes of a
# DualPipeV(4, 2) row are 1.6e14 FLOP there (minutes), so the sequences are 512 long here.  All
# widths are the bench's: hidden 4096, 32 / 8 heads, 8 experts of SwiGLU 14336, top-2.  The
# expert products over the bench's 16 384 token copies are covered by
# test_grouped_gemms_at_full_size.
MIXTRAL_8X7B_LAYER = LayerSpec("mixtral", 4096, 32, 14336, 512, 2, n_kv_heads=8, head_dim=128,
                               causal=True, rope_theta=5e5, eps=1e-5, n_experts=8, top_k=2)


def test_mixtral_8x7b_layer_on_a_dualpipev_row_matches_oracle():
    """One Mixtral-8x7B-shaped layer per stage on rank 0 of DualPipeV(4, 2) (stages 0 and 3:
    an unsplit first-stage backward and a split one), four microbatches, against the oracle."""
    print("Mixtral-shaped layers, DualPipeV(4,2) rank 0", flush=True)
    # weight gradients in pairs of microbatches, the experts' with each microbatch's own row
    # groups, as the bench runs them
    check_rank_row(MIXTRAL_8X7B_LAYER, S.DualPipeV(4, 2), 4, 0, 1, wgrad_group=2)


@pytest.mark.parametrize("name,peak", [("cfg3", 11), ("cfg2", 4)])
def test_bench_row_equals_sequential_order(name, peak):
    """The rows bench.py times, at full size and with its own device state (bench.Workbench):
    cfg3 = Interleaved1F1B(8, 4) rank 0, 32 microbatches, 2 x 4 Llama-3-8B-shaped layers;
    cfg2 = Std1F1B(4) rank 0, 16 microbatches, 6 BERT-large layers (its ungrouped passes with the
    weight gradients on the stage's second stream, which bench.py offers as an option).  No oracle at
    this size; instead the reference's own invariant (tests/test_transformations.py:187-191):
    the scheduled row must give bit-identical results to the same work in sequential order
    (every microbatch forward then backward, chunk by chunk) - every task's output and every
    gradient accumulator - and the number of live residual slots must peak at the schedule's
    figure (11 / 4), which exercises every slot of the ring and both chunks."""
    import bench
    from jaxpp_amd.model import workloads
    from jaxpp_amd.types import TaskType
    wl = workloads()[name]
    two = wl.layer.hidden < 2048
    print(f"bench row {name}: {wl.schedule}{wl.schedule_kwargs} rank {wl.rank}", flush=True)
    wb = bench.Workbench(wl, fused=True, two_streams=two)
    ex, plan = wb.ex, wb.plan
    act = wl.layer.tokens * wl.layer.hidden
    outs = {(pt.exec_kind, pt.chunk, pt.task.mubatch_idx): rt.DeviceBuffer(act * 2)
            for pt in plan.tasks if pt.exec_kind is not TaskType.BWD_W}

    def io(pt, lane=0):
        m = pt.task.mubatch_idx
        src = wb.x_in if pt.exec_kind is TaskType.FWD else wb.dy_in
        return src[pt.chunk, m].ptr, outs[pt.exec_kind, pt.chunk, m].ptr

    def snapshot():
        ex.join()
        rt.sync()
        o = {k: b.download(np.uint16, (act,)) for k, b in outs.items()}
        g = [ex.get_grads(c, li) for c in range(plan.n_chunks) for li in range(wl.layers_per_stage)]
        return o, g

    # the schedule's order, one task at a time so that the peak of live slots is seen
    ex.zero_grads()
    live_peak = 0
    for pt in plan.tasks:
        if pt.exec_kind is TaskType.BWD_W:
            ex.run_task(pt.exec_kind, pt.chunk, pt.task.mubatch_idx)
        else:
            ex.run_task(pt.exec_kind, pt.chunk, pt.task.mubatch_idx, *io(pt))
        live_peak = max(live_peak, ex.live_slots())
    assert live_peak == peak == plan.max_live
    assert ex.live_slots() == 0
    outs_sched, grads_sched = snapshot()
    # ... and through the loop the bench uses (fused entries beside each other on two streams)
    ex.zero_grads()
    for b in outs.values():
        b.zero()
    wb.loop.run(io)
    outs_loop, grads_loop = snapshot()
    # sequential order: microbatch by microbatch, forward then backward of every chunk
    ex.zero_grads()
    for b in outs.values():
        b.zero()
    bwd_kinds = {}
    for pt in plan.tasks:
        if pt.exec_kind is not TaskType.FWD:
            bwd_kinds.setdefault((pt.chunk, pt.task.mubatch_idx), []).append(pt)
    for m in range(wl.n_mubatches):
        for c in range(plan.n_chunks):
            ex.run_task(TaskType.FWD, c, m, wb.x_in[c, m].ptr, outs[TaskType.FWD, c, m].ptr)
        for c in reversed(range(plan.n_chunks)):
            for pt in bwd_kinds[c, m]:
                if pt.exec_kind is TaskType.BWD_W:
                    ex.run_task(pt.exec_kind, c, m)
                else:
                    ex.run_task(pt.exec_kind, c, m, *io(pt))
        assert ex.live_slots() == 0
    outs_seq, grads_seq = snapshot()
    for what, (o, g) in {"task order": (outs_sched, grads_sched), "rank loop": (outs_loop, grads_loop)}.items():
        for k, v in outs_seq.items():
            assert v.any(), f"output of {k} was never written"
            np.testing.assert_array_equal(o[k], v, err_msg=f"{what}: output of {k}")
        for i, gd in enumerate(grads_seq):
            for pname, v in gd.items():
                np.testing.assert_array_equal(g[i][pname], v, err_msg=f"{what}: grad {i}/{pname}")
    ex.close()
    group = bench.default_wgrad_group(wl, False)
    if group > 1:
        # the mode the bench runs by default: weight gradients of `group` microbatches as one
        # product per weight.  Outputs bit-identical; accumulators equal up to f32
        # reassociation; a microbatch held back keeps its slot, so the peak is higher.
        del wb, outs_sched, outs_loop, grads_sched, grads_loop
        wb = bench.Workbench(wl, fused=True, two_streams=False, wgrad_group=group)
        ex = wb.ex
        ex.zero_grads()
        for b in outs.values():
            b.zero()
        live_peak = 0
        for pt in plan.tasks:
            ex.run_task(pt.exec_kind, pt.chunk, pt.task.mubatch_idx, *io(pt))
            live_peak = max(live_peak, ex.live_slots())
        assert peak < live_peak <= peak + plan.n_chunks * (group - 1)
        outs_grp, grads_grp = snapshot()
        assert ex.live_slots() == 0
        for k, v in outs_seq.items():
            np.testing.assert_array_equal(outs_grp[k], v, err_msg=f"grouped: output of {k}")
        for i, gd in enumerate(grads_seq):
            for pname, v in gd.items():
                # sums of 32 x 4096 products in another order: a few fp32 ulps of the terms
                parity.close(grads_grp[i][pname], v, 3e-5, f"grouped: grad {i}/{pname}")
        ex.close()


@pytest.mark.parametrize("name", ["cfg4", "cfg5"])
def test_deep_bench_rows_equal_sequential_order(name):
    """The two other rows bench.py times, at their real depth in microbatches and at the full
    layer widths, on bench's own device state and with its own weight-gradient grouping:
    cfg4 = ZeroBubble(8) rank 1, 24 microbatches, split backward with the BWD_W tasks in the
    table's bubble slots, Llama-70B-shaped layers; cfg5 = DualPipeV(8, 4) rank 0, 16
    microbatches, both V-chunks on the rank, Mixtral-8x7B-shaped layers.  Two layers per stage
    instead of ten / four (memory and time; the slot ring, the held-back weight gradients and
    the order of tasks - what depth in microbatches exercises - do not depend on the layer
    count).  As for cfg3 there is no oracle at this size; the scheduled row must give
    bit-identical results to the same work in sequential order (the reference's own invariant,
    tests/test_transformations.py:187-191): every task's output and every accumulator, the
    latter kept on the device (a copy per parameter) and compared one parameter at a time."""
    import dataclasses

    import bench
    from jaxpp_amd.model import workloads
    from jaxpp_amd.types import TaskType
    wl = dataclasses.replace(workloads()[name], layers_per_stage=2)
    group = bench.default_wgrad_group(wl, False)
    assert group == 2
    print(f"bench row {name}: {wl.schedule}{wl.schedule_kwargs} rank {wl.rank}, "
          f"{wl.n_mubatches} microbatches, weight gradients in groups of {group}", flush=True)
    wb = bench.Workbench(wl, fused=True, two_streams=False, wgrad_group=group)
    ex, plan = wb.ex, wb.plan
    lib = rt.load()
    act = wl.layer.tokens * wl.layer.hidden
    keys = [(pt.exec_kind, pt.chunk, pt.task.mubatch_idx) for pt in plan.tasks
            if pt.exec_kind is not TaskType.BWD_W]
    outs = [{k: rt.DeviceBuffer(act * 2) for k in keys} for _ in range(2)]

    def io_into(which):
        def io(pt, lane=0):
            m = pt.task.mubatch_idx
            src = wb.x_in if pt.exec_kind is TaskType.FWD else wb.dy_in
            return src[pt.chunk, m].ptr, outs[which][pt.exec_kind, pt.chunk, m].ptr
        return io

    def grad_ptrs():
        for c in range(plan.n_chunks):
            for li in range(wl.layers_per_stage):
                for pname, rows, cols in ex.params:
                    yield (c, li, pname), ex._ptr(lib.jpp_stage_grad_ptr, c, li, pname), rows * cols * 4

    # the schedule's order, one task at a time so that the peak of live slots is seen
    ex.zero_grads()
    live_peak, io = 0, io_into(0)
    for pt in plan.tasks:
        if pt.exec_kind is TaskType.BWD_W:
            ex.run_task(pt.exec_kind, pt.chunk, pt.task.mubatch_idx)
        else:
            ex.run_task(pt.exec_kind, pt.chunk, pt.task.mubatch_idx, *io(pt))
        live_peak = max(live_peak, ex.live_slots())
    ex.join()
    rt.sync()
    assert ex.live_slots() == 0
    assert plan.max_live <= live_peak <= plan.max_live + plan.n_chunks * (group - 1), (
        f"live slots peaked at {live_peak}; the plan says {plan.max_live}, a group holds "
        f"{plan.n_chunks * (group - 1)} more")
    print(f"  live slots peaked at {live_peak} (plan {plan.max_live})", flush=True)
    kept = {}
    for key, ptr, nbytes in grad_ptrs():
        kept[key] = rt.DeviceBuffer(nbytes)
        rt.check(lib.jpp_memcpy_d2d_async(kept[key].ptr, ptr, nbytes, None))
    rt.sync()

    # sequential order: microbatch by microbatch, forward then backward of every chunk
    ex.zero_grads()
    io = io_into(1)
    bwd_kinds = {}
    for pt in plan.tasks:
        if pt.exec_kind is not TaskType.FWD:
            bwd_kinds.setdefault((pt.chunk, pt.task.mubatch_idx), []).append(pt)
    for m in range(wl.n_mubatches):
        for c in range(plan.n_chunks):
            ex.run_task(TaskType.FWD, c, m, wb.x_in[c, m].ptr, outs[1][TaskType.FWD, c, m].ptr)
        for c in reversed(range(plan.n_chunks)):
            for pt in bwd_kinds[c, m]:
                if pt.exec_kind is TaskType.BWD_W:
                    ex.run_task(pt.exec_kind, c, m)
                else:
                    ex.run_task(pt.exec_kind, c, m, *io(pt))
    ex.join()
    rt.sync()
    assert ex.live_slots() == 0

    for k in keys:
        a, b = outs[0][k].download(np.uint16, (act,)), outs[1][k].download(np.uint16, (act,))
        assert b.any(), f"output of {k} was never written"
        np.testing.assert_array_equal(a, b, err_msg=f"output of {k}")
    for key, ptr, nbytes in grad_ptrs():
        a = kept[key].download(np.float32, (nbytes // 4,))
        b = rt.download_ptr(ptr, np.float32, (nbytes // 4,))
        assert np.isfinite(b).all() and (b.any() or key[2].startswith("b")), f"accumulator {key}"
        np.testing.assert_array_equal(a, b, err_msg=f"accumulator {key}")
        kept[key].free()
    wb.close()
