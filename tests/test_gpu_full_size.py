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

from jaxpp_amd import runtime as rt
from jaxpp_amd import schedules as S
from jaxpp_amd.model import LayerSpec
from jaxpp_amd.plan import make_rank_plan
from oracle import layers as L

from test_gpu_stage import close, make_params, run_on_gpu, run_on_oracle

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
        close(ys[key], ys_w[key], 2e-2, f"y{key}")
    for key in dxs_w:
        close(dxs[key], dxs_w[key], 2e-2, f"dx{key}")
    for pname, want in acc_w[0][0].items():
        got = grads[0][0][pname]
        close(got, want.reshape(got.shape), 2e-2, f"grad {pname}")
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
        close(ys[key], ys_w[key], 2e-2, f"y{key}")
    for key in dxs_w:
        close(dxs[key], dxs_w[key], 2e-2, f"dx{key}")
    for s_ in plan.stages:
        for li in range(lpc):
            for pname, want in acc_w[s_][li].items():
                got = grads[s_][li][pname]
                close(got, want.reshape(got.shape), 2e-2, f"grad {s_}/{li}/{pname}")
