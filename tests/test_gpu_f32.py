"""The f32 operators (jpp_*_f32) against numpy in float64, through the C ABI.

Tolerance 1e-5 of a tensor's largest magnitude for single operators (fp32 arithmetic in a
fixed order against float64), 1e-4 - the bound stated for fp32 results - for whole stages."""
import ctypes as C
import math

import numpy as np
import pytest

import parity

from jaxpp_amd import runtime as rt
from oracle import layers as L

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    rt.require_gpu()


close = parity.close


def dev(a):
    return rt.DeviceBuffer.from_numpy(np.ascontiguousarray(a, dtype=np.float32))


GEMMS = [("nn", 128, 192, 64), ("nn", 512, 768, 256), ("nt", 512, 256, 1024), ("tn", 256, 1024, 512)]


@pytest.mark.parametrize("lay,m,n,k", GEMMS, ids=[f"{c[0]}-{c[1]}x{c[2]}x{c[3]}" for c in GEMMS])
def test_gemm_f32_epilogues(lay, m, n, k):
    print(f"gemm_f32 {lay} {m}x{n}x{k}", flush=True)
    rng = np.random.default_rng(m + n + k)
    ta, tb = {"nn": (0, 1), "nt": (0, 0), "tn": (1, 1)}[lay]
    A = rng.standard_normal((m, k), dtype=np.float32)
    B = rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.1)
    bias = rng.standard_normal(n, dtype=np.float32)
    resid = rng.standard_normal((m, n), dtype=np.float32)
    aux = rng.standard_normal((m, n), dtype=np.float32)
    a_h = np.ascontiguousarray(A.T) if ta else A
    b_h = np.ascontiguousarray(B.T) if tb else B
    da, db, dbias, dres, daux = dev(a_h), dev(b_h), dev(bias), dev(resid), dev(aux)
    prod = A.astype(np.float64) @ B.astype(np.float64).T
    lda, ldb = a_h.shape[1], b_h.shape[1]

    def run(epi, c0=None, **kw):
        dc = dev(c0 if c0 is not None else np.zeros((m, n), np.float32))
        rt.gemm(da.ptr, db.ptr, dc.ptr, m, n, k, lda, ldb, n, ta, tb, epi, f32=True, **kw)
        rt.sync()
        return dc.download(np.float32, (m, n))

    close(run(rt.EPI_BF16), prod, 1e-5, "store")
    close(run(rt.EPI_F32), prod, 1e-5, "f32 store")
    close(run(rt.EPI_BF16, bias=dbias.ptr, resid=dres.ptr, ldresid=n), prod + bias + resid, 1e-5,
          "bias + residual")
    c0 = rng.standard_normal((m, n), dtype=np.float32)
    close(run(rt.EPI_ACC_F32, c0), prod + c0, 1e-5, "accumulate")
    for tanh_form in (0, 1):
        u = prod + bias
        if tanh_form:
            t = np.tanh(0.7978845608028654 * (u + 0.044715 * u ** 3))
            g = 0.5 * u * (1 + t)
        else:
            erf = np.vectorize(math.erf)
            g = 0.5 * u * (1 + erf(u / math.sqrt(2)))
        dc2 = dev(np.zeros((m, n), np.float32))
        got_u = run(rt.EPI_GELU, bias=dbias.ptr, c2=dc2.ptr, ldc2=n, gelu_tanh=tanh_form)
        close(got_u, u, 1e-5, "gelu pre-activation")
        close(dc2.download(np.float32, (m, n)), g, 1e-5, "gelu")
        x = aux.astype(np.float64)
        if tanh_form:
            t = np.tanh(0.7978845608028654 * (x + 0.044715 * x ** 3))
            gp = 0.5 * (1 + t) + 0.5 * x * (1 - t * t) * 0.7978845608028654 * (1 + 0.134145 * x * x)
        else:
            erf = np.vectorize(math.erf)
            gp = 0.5 * (1 + erf(x / math.sqrt(2))) + x * np.exp(-0.5 * x * x) / math.sqrt(2 * math.pi)
        close(run(rt.EPI_DGELU, aux=daux.ptr, ldaux=n, gelu_tanh=tanh_form), prod * gp, 1e-5, "dgelu")


def test_gemm_f32_swiglu_epilogues_and_rope():
    rng = np.random.default_rng(21)
    m, f, k = 128, 192, 64                 # gate/up interleaved in blocks of 32 columns
    A = rng.standard_normal((m, k), dtype=np.float32)
    W = rng.standard_normal((k, 2 * f), dtype=np.float32) * np.float32(0.2)   # [gate | up]
    c = np.arange(2 * f)
    q, w = c // 64, c % 64
    order = np.where(w < 32, 32 * q + w, f + 32 * q + w - 32)                 # device column -> host column
    da, dw = dev(A), dev(W[:, order])
    gu, s_out = rt.DeviceBuffer(m * 2 * f * 4), rt.DeviceBuffer(m * f * 4)
    rt.gemm(da.ptr, dw.ptr, gu.ptr, m, 2 * f, k, k, 2 * f, 2 * f, 0, 1, rt.EPI_SWIGLU, c2=s_out.ptr,
            ldc2=f, f32=True)
    rt.sync()
    prod = A.astype(np.float64) @ W.astype(np.float64)
    g64, u64 = prod[:, :f], prod[:, f:]
    close(gu.download(np.float32, (m, 2 * f)), prod[:, order], 1e-5, "gate/up")
    close(s_out.download(np.float32, (m, f)), g64 / (1 + np.exp(-g64)) * u64, 1e-5, "swiglu")
    # gradient: d(gate/up) from ds = dy Wd^T, C of width 2f in the interleaved layout
    h = 64
    dy = rng.standard_normal((m, h), dtype=np.float32)
    Wd = rng.standard_normal((f, h), dtype=np.float32) * np.float32(0.2)
    ddy, dwd, dgu = dev(dy), dev(Wd), rt.DeviceBuffer(m * 2 * f * 4)
    rt.gemm(ddy.ptr, dwd.ptr, dgu.ptr, m, f, h, h, h, 2 * f, 0, 0, rt.EPI_DSWIGLU, aux=gu.ptr,
            ldaux=2 * f, f32=True)
    rt.sync()
    ds = dy.astype(np.float64) @ Wd.astype(np.float64).T
    sg = 1 / (1 + np.exp(-g64))
    want = np.concatenate([ds * u64 * sg * (1 + g64 * (1 - sg)), ds * g64 * sg], 1)
    close(dgu.download(np.float32, (m, 2 * f)), want[:, order], 1e-5, "d gate/up")
    # rotary embedding and its inverse
    B, S, heads, d = 2, 64, 3, 128
    ld = (heads + 1) * d
    x = rng.standard_normal((B * S, ld), dtype=np.float32)
    ang = np.arange(S)[:, None] * (5e5 ** (-2.0 * np.arange(d // 2) / d))[None, :]
    cs, sn = np.cos(ang), np.sin(ang)
    bx, bc, bs = dev(x), dev(cs), dev(sn)
    lib = rt.load()
    rt.check(lib.jpp_rope_f32(None, bx.ptr, ld, bc.ptr, bs.ptr, B, S, heads, d, 0))
    rt.sync()
    want = x.astype(np.float64).copy()
    xr = want[:, :heads * d].reshape(B, S, heads, d)
    a, b = xr[..., :d // 2].copy(), xr[..., d // 2:].copy()
    xr[..., :d // 2] = a * cs[None, :, None, :] - b * sn[None, :, None, :]
    xr[..., d // 2:] = b * cs[None, :, None, :] + a * sn[None, :, None, :]
    want[:, :heads * d] = xr.reshape(B * S, heads * d)
    close(bx.download(np.float32, (B * S, ld)), want, 1e-5, "rope (last head untouched)")
    rt.check(lib.jpp_rope_f32(None, bx.ptr, ld, bc.ptr, bs.ptr, B, S, heads, d, 1))
    rt.sync()
    close(bx.download(np.float32, (B * S, ld)), x.astype(np.float64), 1e-5, "rope then inverse")


def test_gemm_f32_grouped_modes():
    rng = np.random.default_rng(12)
    E, h, f = 8, 128, 192
    counts = [300, 0, 256, 17, 700, 1, 255, 512]
    seg = np.zeros(E + 1, np.int32)
    for e, c in enumerate(counts):
        seg[e + 1] = seg[e] + (c + 255) // 256 * 256
    cap = int(seg[E]) + 256
    xp = np.zeros((cap, h), np.float32)
    dy = np.zeros((cap, f), np.float32)
    for e, c in enumerate(counts):
        xp[seg[e]:seg[e] + c] = rng.standard_normal((c, h), dtype=np.float32)
        dy[seg[e]:seg[e] + c] = rng.standard_normal((c, f), dtype=np.float32)
    w = rng.standard_normal((E, h, f), dtype=np.float32) * np.float32(0.1)
    b_seg = rt.DeviceBuffer.from_numpy(seg)
    b_xp, b_w, b_dy = dev(xp), dev(w), dev(dy)
    out = dev(np.zeros((cap, f), np.float32))
    rt.gemm(b_xp.ptr, b_w.ptr, out.ptr, cap, f, h, h, f, f, 0, 1, rt.EPI_BF16, seg=b_seg.ptr, n_seg=E,
            group_mode=1, stride_b=h * f, f32=True)
    rt.sync()
    got = out.download(np.float32, (cap, f))
    for e in range(E):
        if counts[e]:
            close(got[seg[e]:seg[e + 1]], xp[seg[e]:seg[e + 1]].astype(np.float64) @ w[e], 1e-5, f"group {e}")
    assert not got[seg[E]:].any(), "tiles past the last group must not be written"
    acc0 = rng.standard_normal((E, h, f), dtype=np.float32)
    b_acc = dev(acc0)
    rt.gemm(b_xp.ptr, b_dy.ptr, b_acc.ptr, h, f, 0, h, f, f, 1, 1, rt.EPI_ACC_F32, seg=b_seg.ptr,
            n_seg=E, group_mode=2, stride_c=h * f, f32=True)
    rt.sync()
    gw = b_acc.download(np.float32, (E, h, f))
    for e in range(E):
        want = acc0[e] + xp[seg[e]:seg[e + 1]].astype(np.float64).T @ dy[seg[e]:seg[e + 1]]
        close(gw[e], want, 1e-5, f"dW group {e}")
    np.testing.assert_array_equal(gw[1], acc0[1])       # empty group: untouched


def test_gemm_f32_rejects_what_it_does_not_do():
    d = rt.DeviceBuffer(64 * 64 * 4)
    with pytest.raises(rt.JppError, match="multiples of 64"):
        rt.gemm(d.ptr, d.ptr, d.ptr, 32, 64, 16, 16, 64, 64, 0, 1, f32=True)
    with pytest.raises(rt.JppError, match="SwiGLU epilogue needs c2"):
        rt.gemm(d.ptr, d.ptr, d.ptr, 64, 64, 16, 16, 64, 64, 0, 1, rt.EPI_SWIGLU, f32=True)
    with pytest.raises(rt.JppError, match="grouped problem needs seg"):
        rt.gemm(d.ptr, d.ptr, d.ptr, 64, 64, 16, 16, 64, 64, 0, 1, f32=True, group_mode=1)


@pytest.mark.parametrize("ln", [True, False], ids=["layernorm", "rmsnorm"])
def test_norm_f32(ln):
    rng = np.random.default_rng(3)
    rows, cols, eps = 200, 320, 1e-5
    x = rng.standard_normal((rows, cols), dtype=np.float32) * 2 + 0.5
    gamma = rng.standard_normal(cols, dtype=np.float32)
    beta = rng.standard_normal(cols, dtype=np.float32)
    dy = rng.standard_normal((rows, cols), dtype=np.float32)
    resid = rng.standard_normal((rows, cols), dtype=np.float32)
    x64 = x.astype(np.float64)
    mean = x64.mean(-1, keepdims=True) if ln else np.zeros((rows, 1))
    var = ((x64 - mean) ** 2).mean(-1, keepdims=True)
    rstd = 1.0 / np.sqrt(var + eps)
    xh = (x64 - mean) * rstd
    y_w = xh * gamma + (beta if ln else 0.0)
    dg = dy.astype(np.float64) * gamma
    s1 = dg.mean(-1, keepdims=True) if ln else 0.0
    s2 = (dg * xh).mean(-1, keepdims=True)
    dx_w = (dg - s1 - xh * s2) * rstd + resid
    b = {k: dev(v) for k, v in dict(x=x, gamma=gamma, beta=beta, dy=dy, resid=resid).items()}
    y, dx = rt.DeviceBuffer(rows * cols * 4), rt.DeviceBuffer(rows * cols * 4)
    mean_d, rstd_d = rt.DeviceBuffer(rows * 4), rt.DeviceBuffer(rows * 4)
    g0 = rng.standard_normal(cols, dtype=np.float32)
    b0 = rng.standard_normal(cols, dtype=np.float32)
    dgam, dbet = dev(g0), dev(b0)
    a = rt.NormArgs(b["x"].ptr, b["gamma"].ptr, b["beta"].ptr if ln else None, y.ptr,
                    mean_d.ptr if ln else None, rstd_d.ptr, b["dy"].ptr, b["resid"].ptr, dx.ptr,
                    dgam.ptr, dbet.ptr if ln else None, None, rows, cols, eps)
    lib = rt.load()
    rt.check(lib.jpp_norm_fwd_f32(None, C.byref(a)))
    rt.check(lib.jpp_norm_bwd_f32(None, C.byref(a)))
    rt.sync()
    close(y.download(np.float32, (rows, cols)), y_w, 1e-5, "y")
    close(rstd_d.download(np.float32, (rows,)), rstd[:, 0], 1e-5, "rstd")
    if ln:
        close(mean_d.download(np.float32, (rows,)), mean[:, 0], 1e-5, "mean")
    close(dx.download(np.float32, (rows, cols)), dx_w, 1e-5, "dx")
    close(dgam.download(np.float32, (cols,)), g0 + (dy * xh).sum(0), 1e-5, "dgamma")
    if ln:
        close(dbet.download(np.float32, (cols,)), b0 + dy.astype(np.float64).sum(0), 1e-5, "dbeta")


ATTN = [(2, 128, 4, 4, 64, False), (1, 256, 4, 2, 128, True), (2, 64, 2, 1, 64, True),
        (1, 192, 2, 2, 128, False)]


@pytest.mark.parametrize("B,S,Hq,Hkv,d,causal", ATTN,
                         ids=[f"b{c[0]}s{c[1]}h{c[2]}kv{c[3]}d{c[4]}{'c' if c[5] else ''}" for c in ATTN])
def test_attention_f32(B, S, Hq, Hkv, d, causal):
    print(f"attention_f32 B{B} S{S} Hq{Hq} Hkv{Hkv} d{d} causal={causal}", flush=True)
    rng = np.random.default_rng(S + d)
    w = (Hq + 2 * Hkv) * d
    qkv = rng.standard_normal((B * S, w), dtype=np.float32)
    do = rng.standard_normal((B * S, Hq * d), dtype=np.float32)
    q = qkv[:, :Hq * d].reshape(B, S, Hq, d)
    k = qkv[:, Hq * d:(Hq + Hkv) * d].reshape(B, S, Hkv, d)
    v = qkv[:, (Hq + Hkv) * d:].reshape(B, S, Hkv, d)
    o_w, lse_w = L.attention_fwd(q, k, v, causal, np.float64)
    dq_w, dk_w, dv_w = L.attention_bwd(q, k, v, o_w, do.reshape(B, S, Hq, d).astype(np.float64),
                                       lse_w, causal, np.float64)
    b_qkv, b_do = dev(qkv), dev(do)
    o, lse = rt.DeviceBuffer(B * S * Hq * d * 4), rt.DeviceBuffer(B * Hq * S * 4)
    dqkv, delta = rt.DeviceBuffer(B * S * w * 4), rt.DeviceBuffer(2 * B * Hq * S * 4)
    a = rt.AttnArgs(b_qkv.ptr, b_qkv.ptr + Hq * d * 4, b_qkv.ptr + (Hq + Hkv) * d * 4, o.ptr, lse.ptr,
                    b_do.ptr, dqkv.ptr, dqkv.ptr + Hq * d * 4, dqkv.ptr + (Hq + Hkv) * d * 4, delta.ptr,
                    w, w, w, Hq * d, Hq * d, w, w, w, B, S, Hq, Hkv, d, int(causal))
    lib = rt.load()
    rt.check(lib.jpp_attn_fwd_f32(None, C.byref(a)))
    rt.check(lib.jpp_attn_bwd_f32(None, C.byref(a)))
    rt.sync()
    close(o.download(np.float32, (B, S, Hq, d)), o_w, 1e-5, "o")
    close(lse.download(np.float32, (B, Hq, S)), lse_w, 1e-5, "lse")
    got = dqkv.download(np.float32, (B * S, w))
    close(got[:, :Hq * d].reshape(B, S, Hq, d), dq_w, 1e-5, "dq")
    close(got[:, Hq * d:(Hq + Hkv) * d].reshape(B, S, Hkv, d), dk_w, 1e-5, "dk")
    close(got[:, (Hq + Hkv) * d:].reshape(B, S, Hkv, d), dv_w, 1e-5, "dv")


def test_colsum_and_mse_f32():
    rng = np.random.default_rng(9)
    rows, cols, ld = 300, 200, 256
    x = rng.standard_normal((rows, ld), dtype=np.float32)
    acc0 = rng.standard_normal(cols, dtype=np.float32)
    bx, acc = dev(x), dev(acc0)
    lib = rt.load()
    rt.check(lib.jpp_colsum_accum_f32(None, bx.ptr, ld, rows, cols, acc.ptr))
    rt.sync()
    close(acc.download(np.float32, (cols,)), acc0 + x[:, :cols].astype(np.float64).sum(0), 1e-5, "colsum")
    n = 5000
    out, tgt = rng.standard_normal(n, dtype=np.float32), rng.standard_normal(n, dtype=np.float32)
    bo, bt, loss, dout = dev(out), dev(tgt), rt.DeviceBuffer(4), rt.DeviceBuffer(n * 4)
    rt.check(lib.jpp_mse_loss_f32(None, bo.ptr, bt.ptr, n, 0.125, loss.ptr, dout.ptr))
    rt.sync()
    d = out.astype(np.float64) - tgt
    close(loss.download(np.float32, (1,)), np.array([0.125 * (d * d).mean()]), 1e-5, "loss")
    close(dout.download(np.float32, (n,)), 0.125 * 2 * d / n, 1e-5, "dout")


# ---------------------------------------------------------------------------
# whole stages in f32 against the oracle's f32 numerics
# ---------------------------------------------------------------------------
from jaxpp_amd import schedules as S                      # noqa: E402
from jaxpp_amd.model import LayerSpec, init_layer_params  # noqa: E402
from jaxpp_amd.plan import make_rank_plan                 # noqa: E402

from test_gpu_stage import run_on_gpu, run_on_oracle      # noqa: E402

# the CPU-runnable configuration: post-LN encoder layers of hidden 256, 4 heads, FFN 1024,
# 128-token sequences in microbatches of 4, two stages of two layers, Std1F1B, 8 microbatches
CFG1 = LayerSpec("bert", 256, 4, 1024, 128, 4, eps=1e-12, dtype="f32")
DECODER_F32 = LayerSpec("decoder", 256, 2, 512, 128, 2, causal=True, eps=1e-6, gelu_tanh=True,
                        dtype="f32")
BERT_D64_F32 = LayerSpec("bert", 128, 2, 256, 256, 1, eps=1e-5, dtype="f32")

LLAMA_F32 = LayerSpec("llama", 256, 2, 384, 128, 2, n_kv_heads=1, head_dim=128, causal=True,
                      rope_theta=5e5, eps=1e-5, dtype="f32")
LLAMA_D64_F32 = LayerSpec("llama", 256, 4, 256, 256, 1, n_kv_heads=2, head_dim=64, causal=True,
                          rope_theta=1e4, eps=1e-5, dtype="f32")

MIXTRAL_F32 = LayerSpec("mixtral", 256, 2, 256, 128, 2, n_kv_heads=1, head_dim=128, causal=True,
                        rope_theta=5e5, eps=1e-5, n_experts=8, top_k=2, dtype="f32")

STAGES_F32 = [
    ("mixtral-1f1b", MIXTRAL_F32, S.Std1F1B(2), 3, 1, 2),
    ("mixtral-dualpipev", MIXTRAL_F32, S.DualPipeV(4, 2), 4, 0, 1),
    ("mixtral-zb", MIXTRAL_F32, S.ZeroBubble(2), 3, 1, 1),
    ("llama-interleaved", LLAMA_F32, S.Interleaved1F1B(4, 2), 4, 0, 2),
    ("llama-zb", LLAMA_D64_F32, S.ZeroBubble(3), 3, 1, 2),
    ("llama-dualpipev", LLAMA_F32, S.DualPipeV(4, 2), 4, 1, 1),
    ("cfg1-rank0", CFG1, S.Std1F1B(2), 8, 0, 2),
    ("cfg1-rank1", CFG1, S.Std1F1B(2), 8, 1, 2),
    ("bert-zb", BERT_D64_F32, S.ZeroBubble(2), 3, 1, 2),
    ("bert-zb-first-stage", BERT_D64_F32, S.ZeroBubble(2), 2, 0, 1),
    ("decoder-1f1b", DECODER_F32, S.Std1F1B(2), 3, 1, 2),
    ("decoder-zb", DECODER_F32, S.ZeroBubble(2), 3, 1, 1),
    ("decoder-interleaved", DECODER_F32, S.Interleaved1F1B(4, 2), 4, 0, 1),
]


@pytest.mark.parametrize("two_streams", [False, True], ids=["one-stream", "two-streams"])
@pytest.mark.parametrize("name,spec,sched,n,rank,lpc", STAGES_F32, ids=[c[0] for c in STAGES_F32])
def test_f32_stage_matches_oracle(name, spec, sched, n, rank, lpc, two_streams):
    print(f"f32 stage case {name} two_streams={two_streams}", flush=True)
    plan = make_rank_plan(sched, n, rank)
    params = {s: [init_layer_params(spec, 3, s * lpc + li, perturb=True) for li in range(lpc)]
              for s in plan.stages}
    row = S.preprocess_schedule_tasks(sched.tasks(n), 0, False)[rank]
    ys_w, dxs_w, acc_w = run_on_oracle(spec, plan, params, row)
    ys, dxs, grads = run_on_gpu(spec, plan, lpc, params, two_streams=two_streams)
    assert set(ys) == set(ys_w) and set(dxs) == set(dxs_w)
    for k in ys_w:
        close(ys[k], ys_w[k].astype(np.float64), 1e-4, f"y{k}")
    for k in dxs_w:
        close(dxs[k], dxs_w[k].astype(np.float64), 1e-4, f"dx{k}")
    for s in plan.stages:
        for li in range(lpc):
            for pname, want in acc_w[s][li].items():
                got = grads[s][li][pname]
                close(got, want.reshape(got.shape).astype(np.float64), 1e-4, f"grad {s}/{li}/{pname}")


def test_f32_stage_accumulates_in_the_gemm():
    with pytest.raises(rt.JppError, match="f32 stages accumulate in the weight-gradient GEMM"):
        rt.StageExecutor(CFG1, 1, 1, 1, fused_wgrad_accum=False)


def test_cfg1_train_step_through_the_public_api():
    """The CPU-runnable configuration end to end in float32: 4 post-LN encoder layers of hidden
    256 in 2 stages, 8 microbatches of 4 x 128 tokens, Std1F1B, loss mean((out - in)^2) / 8 -
    losses and accumulated gradients against the sequential loop in the oracle's f32 numerics,
    to the 1e-4 stated for fp32 results."""
    from functools import partial

    import jaxpp_amd as jaxpp
    from oracle import stage as O

    n_mb, pp, n_layers = 8, 2, 4
    model = jaxpp.nn.TransformerStack(CFG1, n_layers=n_layers, layers_per_stage=n_layers // pp)
    params = model.init(seed=0, perturb=True)
    batch = np.random.default_rng(1).standard_normal((n_mb, CFG1.tokens, CFG1.hidden),
                                                     dtype=np.float32)
    mesh = jaxpp.MpmdMesh(jaxpp.DeviceMesh(np.arange(pp).reshape(pp, 1), ("mpmd", "data")), "mpmd")
    schedule = jaxpp.Std1F1B(pp)

    def loss_fn(pars, mb):
        res = model.apply(pars, mb)
        return jaxpp.nn.mse_loss(res, mb) / n_mb, (res, 4)

    @partial(jaxpp.mpmd_jit_with_loop, mpmd_mesh=mesh)
    def train_step(pars, batch):
        mubatch_grad = partial(jaxpp.value_and_grad(loss_fn, has_aux=True), pars)
        (losses, (pred, _)), grad = jaxpp.treduce(mubatch_grad, batch, schedule=schedule)
        return losses, pred, grad

    losses, pred, grad = train_step(params, batch)
    cfg = L.LayerCfg(**CFG1.as_dict())
    per = n_layers // pp
    stages = [params["layers"][s * per:(s + 1) * per] for s in range(pp)]
    want_pred = []
    want_loss, want_acc = O.treduce_sequential(cfg, stages, list(batch), L.Numerics.f32(),
                                               preds=want_pred)
    close(losses, want_loss.astype(np.float64), 1e-4, "losses")
    assert pred.shape == batch.shape and np.isfinite(pred).all()
    for m in range(n_mb):
        close(pred[m], want_pred[m].astype(np.float64), 1e-4, f"prediction of microbatch {m}")
    for s in range(pp):
        for li in range(per):
            for k, v in want_acc[s][li].items():
                got = grad["layers"][s * per + li][k]
                close(got, v.reshape(got.shape).astype(np.float64), 1e-4, f"grad {s}/{li}/{k}")
    train_step.close()


def test_cfg1_two_train_steps_with_adam_through_the_public_api():
    """cfg1 with its optimizer: the train step of the reference's README (README.md:83-93) -
    treduce, then `optimizer.update` and `apply_updates` - returning the updated parameters,
    twice in a row with Adam lr 1e-3, against the oracle's sequential loop and Adam at 1e-4."""
    from functools import partial

    import jaxpp_amd as jaxpp
    from oracle import stage as O

    n_mb, pp, n_layers = 8, 2, 4
    model = jaxpp.nn.TransformerStack(CFG1, n_layers=n_layers, layers_per_stage=n_layers // pp)
    params = model.init(seed=0, perturb=True)
    rng = np.random.default_rng(1)
    mesh = jaxpp.MpmdMesh(jaxpp.DeviceMesh(np.arange(pp).reshape(pp, 1), ("mpmd", "data")), "mpmd")
    schedule = jaxpp.Std1F1B(pp)
    optimizer = jaxpp.optim.adam(1e-3)

    def loss_fn(pars, mb):
        res = model.apply(pars, mb)
        return jaxpp.nn.mse_loss(res, mb) / n_mb, (res, 4)

    @partial(jaxpp.mpmd_jit_with_loop, mpmd_mesh=mesh)
    def pp_train_step(opt_state, pars, batch):
        mubatch_grad = partial(jaxpp.value_and_grad(loss_fn, has_aux=True), pars)
        (losses, (preds, _)), grad = jaxpp.treduce(mubatch_grad, batch, schedule=schedule)
        updates, opt_state = optimizer.update(grad, opt_state, pars)
        new_pars = jaxpp.optim.apply_updates(pars, updates)
        return opt_state, new_pars, losses, preds

    cfg = L.LayerCfg(**CFG1.as_dict())
    per = n_layers // pp
    want_p = [dict(p) for p in params["layers"]]
    want_m = [{k: np.zeros_like(v) for k, v in p.items()} for p in want_p]
    want_v = [{k: np.zeros_like(v) for k, v in p.items()} for p in want_p]
    opt_state = optimizer.init(params)
    for step in (1, 2):
        batch = rng.standard_normal((n_mb, CFG1.tokens, CFG1.hidden), dtype=np.float32)
        opt_state, params, losses, _ = pp_train_step(opt_state, params, batch)
        stages = [want_p[s * per:(s + 1) * per] for s in range(pp)]
        want_loss, want_acc = O.treduce_sequential(cfg, stages, list(batch), L.Numerics.f32())
        close(losses, want_loss.astype(np.float64), 1e-4, f"step {step} losses")
        for i in range(n_layers):
            g = {k: v.reshape(want_p[i][k].shape) for k, v in want_acc[i // per][i % per].items()}
            want_p[i] = O.adam_step(want_p[i], g, want_m[i], want_v[i], step, lr=1e-3)
            for k in want_p[i]:
                close(params["layers"][i][k], want_p[i][k].astype(np.float64), 1e-4,
                      f"step {step} layer {i} {k}")
                close(opt_state["mu"]["layers"][i][k], want_m[i][k].astype(np.float64), 1e-4,
                      f"step {step} layer {i} m[{k}]")
                close(opt_state["nu"]["layers"][i][k], want_v[i][k].astype(np.float64), 1e-4,
                      f"step {step} layer {i} v[{k}]")
        assert opt_state["count"] == step
    pp_train_step.close()


def test_f32_stage_adam_after_loop():
    """Two train steps of an f32 rank: the parameters are their own f32 weights (no second
    copy), Adam rewrites them in place and clears the accumulators."""
    from jaxpp_amd.model import boundary_tensor
    from jaxpp_amd.rank_loop import RankLoop
    from jaxpp_amd.types import TaskType
    from oracle import stage as O

    spec, schedule, n_mb, rank, lpc = CFG1, S.Std1F1B(2), 4, 1, 2
    plan = make_rank_plan(schedule, n_mb, rank)
    shape = (spec.tokens, spec.hidden)
    ex = rt.StageExecutor(spec, plan.n_chunks, lpc, plan.max_live, plan.split_backward, True, False)
    host = [init_layer_params(spec, 3, li, perturb=True) for li in range(lpc)]
    for li in range(lpc):
        ex.set_params(0, li, host[li])
    ex.optimizer_init()
    bufs = {}

    def io(pt, lane=0):
        kind = "x" if pt.exec_kind is TaskType.FWD else "dy"
        key = (kind, pt.task.stage_id, pt.task.mubatch_idx)
        if key not in bufs:
            bufs[key] = (ex.upload_activation(boundary_tensor(kind, *key[1:], shape, 0)),
                         ex.new_activation())
        return bufs[key][0].ptr, bufs[key][1].ptr

    m = [{k: np.zeros_like(v) for k, v in p.items()} for p in host]
    v = [{k: np.zeros_like(v_) for k, v_ in p.items()} for p in host]
    w = [dict(p) for p in host]
    for step in (1, 2):
        RankLoop(ex, plan).run(io)
        grads = [ex.get_grads(0, li) for li in range(lpc)]
        ex.adam_step(step, lr=1e-3, grad_scale=1.0 / n_mb)
        rt.sync()
        for li in range(lpc):
            g = {k: a.reshape(host[li][k].shape) * np.float32(1.0 / n_mb) for k, a in grads[li].items()}
            w[li] = O.adam_step(w[li], g, m[li], v[li], step, 1e-3)
            state, new_p = ex.get_opt_state(0, li), ex.get_params(0, li)
            for k in host[li]:
                gw, gm, gv = (a.reshape(host[li][k].shape) for a in state[k])
                close(gm, m[li][k].astype(np.float64), 2e-6, f"step {step} m[{k}]")
                close(gv, v[li][k].astype(np.float64), 2e-6, f"step {step} v[{k}]")
                close(gw, w[li][k].astype(np.float64), 2e-6, f"step {step} weights[{k}]")
                assert np.array_equal(new_p[k].reshape(gw.shape), gw), k
                assert np.abs(gw - host[li][k]).max() > 0, f"{k} did not move"
            assert all(not a.any() for a in ex.get_grads(0, li).values())
    ex.close()


def test_example_model_train_step_in_float32():
    """The reference's example at its default dtype (examples/basic.py:36, :72, :100: float32): a
    stack of pre-LN causal decoder blocks, a stage marker after every `num_layers // pp`
    layers, uniform inputs (:238), loss mean((res - batch)**2) / num_ubatches, Std1F1B over two
    stages; losses and gradients against the sequential loop at 1e-4."""
    from functools import partial

    import jaxpp_amd as jaxpp
    from oracle import stage as O

    spec = LayerSpec("decoder", 256, 2, 512, 128, 1, causal=True, eps=1e-6, gelu_tanh=True,
                     dtype="f32")
    n_mb, pp, n_layers = 4, 2, 4
    schedule = jaxpp.Std1F1B(pp)
    model = jaxpp.nn.TransformerStack(spec, n_layers=n_layers, layers_per_stage=n_layers // pp)
    params = model.init(seed=0, perturb=True)
    batch = np.random.default_rng(2).uniform(size=(n_mb, spec.tokens, spec.hidden)).astype(np.float32)
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
    per = n_layers // pp
    stages = [params["layers"][s * per:(s + 1) * per] for s in range(pp)]
    want_loss, want_acc = O.treduce_sequential(L.LayerCfg(**spec.as_dict()), stages, list(batch),
                                               L.Numerics.f32())
    close(losses, want_loss.astype(np.float64), 1e-4, "losses")
    for s in range(pp):
        for li in range(per):
            for k, v in want_acc[s][li].items():
                got = grad["layers"][s * per + li][k]
                close(got, v.reshape(got.shape).astype(np.float64), 1e-4, f"grad {s}/{li}/{k}")
    train_step.close()
