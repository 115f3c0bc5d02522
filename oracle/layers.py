"""CPU oracle: transformer-layer forward / backward for one pipeline stage.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
module; it exists so the HIP path can be checked against an independent
restatement (tests, the smoke check, and the CPU-baseline leg of the bench).

What the reference fixes and what it does not
---------------------------------------------
The reference (NVIDIA/jaxpp) holds no layer arithmetic of its own: a stage's
task is whatever jaxpr the user's model traced to, compiled by XLA
(src/jaxpp/jax_primitives.py:704-722).  Its examples show the layer shapes
(examples/basic.py:33-91 pre-LN GELU decoder block; README.md:46-72 a post-LN
BERT encoder stack) and its compiler fixes the *structure*:

* a stage's forward task returns the boundary activation plus residuals for
  the backward task (src/jaxpp/core.py:1063-1118);
* with a split backward, BWD_I is the reverse dataflow slice that produces the
  cotangent for the previous stage, plus every remaining non-``dot_general``
  equation whose output is no larger than its inputs; BWD_W is what is left:
  the weight-gradient ``dot_general``s and their accumulate adds
  (src/jaxpp/jaxpr_utils.py:105-169, called with ``memory_scarce=True`` at
  src/jaxpp/core.py:1080-1085).  Here that puts bias gradients (column sums)
  and norm scale/shift gradients in ``bwd_i`` and the four weight-gradient
  GEMMs of a layer in ``bwd_w``.

Layer numerics are therefore pinned by mathematics, not by reference vectors
(the reference's tests hold none): tests/test_oracle_layers.py checks every
function here against float64 central finite differences, against torch
autograd on an independently written torch model, against brute-force
per-row attention, and against scipy special functions.

Precision model: ``rt`` is the storage rounding applied to every tensor the
device path writes to HBM (identity for fp32, round-to-nearest-even bf16
otherwise); products accumulate in fp32 (``acc``=float32) or float64.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np

try:  # scipy is test-time only; erf falls back to math.erf vectorised
    from scipy.special import erf as _erf
except Exception:  # pragma: no cover
    _erf = np.vectorize(math.erf)


# ---------------------------------------------------------------------------
# storage rounding
# ---------------------------------------------------------------------------
def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round float32 to the nearest bf16 (ties to even), returned as float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    r = (u + np.uint32(0x7FFF) + lsb) & np.uint32(0xFFFF0000)
    out = r.view(np.float32)
    nan = np.isnan(x)
    if nan.any():
        out = np.where(nan, x, out)
    return out


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    return (bf16_round(x).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def identity(x):
    return x


@dataclass(frozen=True)
class LayerCfg:
    """Shape of one transformer layer and the conventions it uses."""

    family: str                      # "bert" | "decoder" | "llama" | "mixtral"
    hidden: int
    n_heads: int
    ffn: int
    seq: int
    batch: int                       # sequences per microbatch
    n_kv_heads: int | None = None    # None -> n_heads
    head_dim: int | None = None      # None -> hidden // n_heads
    causal: bool = False
    rope_theta: float = 5e5
    eps: float = 1e-12
    gelu_tanh: bool = False
    n_experts: int = 0
    top_k: int = 0
    dtype: str = "bf16"              # element type of parameters and activations: "bf16" | "f32"

    @property
    def kvh(self) -> int:
        return self.n_kv_heads or self.n_heads

    @property
    def d(self) -> int:
        return self.head_dim or self.hidden // self.n_heads

    @property
    def tokens(self) -> int:
        return self.seq * self.batch

    @property
    def qkv_width(self) -> int:
        return (self.n_heads + 2 * self.kvh) * self.d


def param_shapes(cfg: LayerCfg) -> dict:
    h, f = cfg.hidden, cfg.ffn
    if cfg.family in ("bert", "decoder"):
        return {"Wqkv": (h, 3 * h), "bqkv": (3 * h,), "Wo": (h, h), "bo": (h,),
                "ln1_g": (h,), "ln1_b": (h,), "W1": (h, f), "b1": (f,),
                "W2": (f, h), "b2": (h,), "ln2_g": (h,), "ln2_b": (h,)}
    if cfg.family == "llama":
        return {"rms1_g": (h,), "Wqkv": (h, cfg.qkv_width),
                "Wo": (cfg.n_heads * cfg.d, h), "rms2_g": (h,),
                "Wgu": (h, 2 * f), "Wd": (f, h)}
    if cfg.family == "mixtral":
        E = cfg.n_experts
        return {"rms1_g": (h,), "Wqkv": (h, cfg.qkv_width),
                "Wo": (cfg.n_heads * cfg.d, h), "rms2_g": (h,),
                "Wr": (h, E), "Wgu": (E, h, 2 * f), "Wd": (E, f, h)}
    raise ValueError(cfg.family)


# ---------------------------------------------------------------------------
# primitive ops (forward and backward), all on [rows, features] float arrays
# ---------------------------------------------------------------------------
def layernorm_fwd(x, g, b, eps, acc=np.float32):
    xa = x.astype(acc)
    mean = xa.mean(-1, keepdims=True)
    var = ((xa - mean) ** 2).mean(-1, keepdims=True)
    rstd = 1.0 / np.sqrt(var + eps)
    y = (xa - mean) * rstd * g.astype(acc) + b.astype(acc)
    return y, mean[..., 0], rstd[..., 0]


def layernorm_bwd(dy, x, mean, rstd, g, acc=np.float32):
    xa, dya = x.astype(acc), dy.astype(acc)
    xh = (xa - mean[..., None]) * rstd[..., None]
    dyg = dya * g.astype(acc)
    m1 = dyg.mean(-1, keepdims=True)
    m2 = (dyg * xh).mean(-1, keepdims=True)
    dx = (dyg - m1 - xh * m2) * rstd[..., None]
    return dx, (dya * xh).sum(0), dya.sum(0)


def rmsnorm_fwd(x, g, eps, acc=np.float32):
    xa = x.astype(acc)
    rstd = 1.0 / np.sqrt((xa * xa).mean(-1, keepdims=True) + eps)
    return xa * rstd * g.astype(acc), rstd[..., 0]


def rmsnorm_bwd(dy, x, rstd, g, acc=np.float32):
    xa, dya = x.astype(acc), dy.astype(acc)
    xh = xa * rstd[..., None]
    dyg = dya * g.astype(acc)
    m2 = (dyg * xh).mean(-1, keepdims=True)
    return (dyg - xh * m2) * rstd[..., None], (dya * xh).sum(0)


_SQRT_2_OVER_PI = math.sqrt(2.0 / math.pi)


def gelu(u, tanh=False):
    if tanh:
        return 0.5 * u * (1.0 + np.tanh(_SQRT_2_OVER_PI * (u + 0.044715 * u ** 3)))
    return 0.5 * u * (1.0 + _erf(u / math.sqrt(2.0)))


def gelu_grad(u, tanh=False):
    if tanh:
        t = np.tanh(_SQRT_2_OVER_PI * (u + 0.044715 * u ** 3))
        return 0.5 * (1 + t) + 0.5 * u * (1 - t * t) * _SQRT_2_OVER_PI * (1 + 3 * 0.044715 * u * u)
    return 0.5 * (1.0 + _erf(u / math.sqrt(2.0))) + u * np.exp(-0.5 * u * u) / math.sqrt(2 * math.pi)


def sigmoid(a):
    return 1.0 / (1.0 + np.exp(-a))


def swiglu(gu, f):
    a, b = gu[..., :f], gu[..., f:]
    return a * sigmoid(a) * b


def swiglu_bwd(gu, ds, f):
    a, b = gu[..., :f], gu[..., f:]
    s = sigmoid(a)
    da = ds * b * s * (1.0 + a * (1.0 - s))
    db = ds * a * s
    return np.concatenate([da, db], -1)


def rope_tables(seq, d, theta, acc=np.float64):
    """cos/sin of pos * theta^(-2i/d), i < d/2; computed in float64 and
    rounded once, so the device path can be handed the same table."""
    inv = theta ** (-np.arange(0, d // 2, dtype=np.float64) * 2.0 / d)
    ang = np.arange(seq, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang).astype(acc), np.sin(ang).astype(acc)


def rope_apply(x, cos, sin, inverse=False):
    """Half-split rotary embedding on [B, S, H, d]; ``inverse`` rotates by
    the negative angle (the transpose, used for the backward)."""
    d2 = x.shape[-1] // 2
    x1, x2 = x[..., :d2], x[..., d2:]
    c, s = cos[None, :, None, :], sin[None, :, None, :]
    if inverse:
        s = -s
    return np.concatenate([x1 * c - x2 * s, x2 * c + x1 * s], -1)


def attention_fwd(q, k, v, causal, acc=np.float32, rt=identity):
    """q: [B,S,Hq,d]; k,v: [B,S,Hkv,d].  Returns o [B,S,Hq,d] and the row
    log-sum-exp of the scaled scores [B,Hq,S].  ``rt`` rounds the probabilities
    where they become an operand of the second product (a bf16 path multiplies
    bf16 probabilities; the row sum is taken before rounding)."""
    B, S, Hq, d = q.shape
    Hkv = k.shape[2]
    grp = Hq // Hkv
    scale = 1.0 / math.sqrt(d)
    qa = q.astype(acc).transpose(0, 2, 1, 3)                       # B,Hq,S,d
    ka = np.repeat(k.astype(acc).transpose(0, 2, 1, 3), grp, 1)
    va = np.repeat(v.astype(acc).transpose(0, 2, 1, 3), grp, 1)
    s = np.matmul(qa, ka.transpose(0, 1, 3, 2)) * scale            # B,Hq,S,S
    if causal:
        s = np.where(np.tril(np.ones((S, S), bool)), s, -np.inf)
    m = s.max(-1, keepdims=True)
    p = np.exp(s - m)
    l = p.sum(-1, keepdims=True)
    o = np.matmul(p / l, va) if rt is identity else np.matmul(rt(p).astype(acc), va) / l
    lse = (m + np.log(l))[..., 0]
    return o.transpose(0, 2, 1, 3), lse


def attention_bwd(q, k, v, o, do, lse, causal, acc=np.float32, rt=identity):
    """``rt`` rounds the recomputed probabilities and the score cotangents where
    they become operands of the three gradient products; the softmax scale that
    belongs on the score cotangents is applied to the finished dq and dk (a
    blocked attention backward carries it out of the inner loop this way)."""
    B, S, Hq, d = q.shape
    Hkv = k.shape[2]
    grp = Hq // Hkv
    scale = 1.0 / math.sqrt(d)
    qa = q.astype(acc).transpose(0, 2, 1, 3)
    ka = np.repeat(k.astype(acc).transpose(0, 2, 1, 3), grp, 1)
    va = np.repeat(v.astype(acc).transpose(0, 2, 1, 3), grp, 1)
    oa = o.astype(acc).transpose(0, 2, 1, 3)
    doa = do.astype(acc).transpose(0, 2, 1, 3)
    s = np.matmul(qa, ka.transpose(0, 1, 3, 2)) * scale
    if causal:
        s = np.where(np.tril(np.ones((S, S), bool)), s, -np.inf)
    p = np.exp(s - lse.astype(acc)[..., None])
    dv = np.matmul(rt(p).astype(acc).transpose(0, 1, 3, 2), doa)
    dp = np.matmul(doa, va.transpose(0, 1, 3, 2))
    delta = (doa * oa).sum(-1, keepdims=True)
    ds = rt(p * (dp - delta)).astype(acc)
    dq = np.matmul(ds, ka) * acc(scale)
    dk = np.matmul(ds.transpose(0, 1, 3, 2), qa)
    dk = dk.reshape(B, Hkv, grp, S, d).sum(2) * acc(scale)
    dv = dv.reshape(B, Hkv, grp, S, d).sum(2)
    return (dq.transpose(0, 2, 1, 3), dk.transpose(0, 2, 1, 3), dv.transpose(0, 2, 1, 3))


def mm(a, b, acc=np.float32):
    return np.matmul(a.astype(acc), b.astype(acc))


# ---------------------------------------------------------------------------
# layer forward / backward-input / backward-weight
# ---------------------------------------------------------------------------
@dataclass
class Numerics:
    """``rt``: storage rounding; ``acc``: accumulation dtype."""
    rt: callable = identity
    acc: type = np.float32

    @staticmethod
    def bf16():
        return Numerics(bf16_round, np.float32)

    @staticmethod
    def f32():
        return Numerics(identity, np.float32)

    @staticmethod
    def f64():
        return Numerics(identity, np.float64)


def _split_qkv(cfg: LayerCfg, qkv):
    B, S, d = cfg.batch, cfg.seq, cfg.d
    nq, nk = cfg.n_heads * d, cfg.kvh * d
    q = qkv[:, :nq].reshape(B, S, cfg.n_heads, d)
    k = qkv[:, nq:nq + nk].reshape(B, S, cfg.kvh, d)
    v = qkv[:, nq + nk:].reshape(B, S, cfg.kvh, d)
    return q, k, v


def _join_qkv(cfg: LayerCfg, q, k, v):
    T = cfg.tokens
    return np.concatenate([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], -1)


def layer_fwd(cfg: LayerCfg, p: dict, x, nm: Numerics, forced_ids=None):
    """Forward of one layer.  Returns (y, stash); the stash is what the
    forward task hands to the backward task(s) of the same microbatch.
    ``forced_ids`` ([T, top_k] expert ids, mixture layers only) replaces the
    layer's own top-k selection; the gates are the softmax over the logits of
    the forced experts.  Tests use it to hold the oracle to the routing the
    device chose where a token's logits tie within rounding."""
    rt, acc = nm.rt, nm.acc
    T, h = cfg.tokens, cfg.hidden
    assert x.shape == (T, h)
    st = {"x": x}
    if cfg.family == "bert":
        qkv = rt(mm(x, p["Wqkv"], acc) + p["bqkv"].astype(acc))
        q, k, v = _split_qkv(cfg, qkv)
        o, lse = attention_fwd(q, k, v, cfg.causal, acc, rt)
        ctx = rt(o.reshape(T, -1))
        a = rt(mm(ctx, p["Wo"], acc) + p["bo"].astype(acc) + x.astype(acc))
        y1, mean1, rstd1 = layernorm_fwd(a, p["ln1_g"], p["ln1_b"], cfg.eps, acc)
        x1 = rt(y1)
        u_full = mm(x1, p["W1"], acc) + p["b1"].astype(acc)
        u = rt(u_full)
        g = rt(gelu(u_full, cfg.gelu_tanh))
        c = rt(mm(g, p["W2"], acc) + p["b2"].astype(acc) + x1.astype(acc))
        y2, mean2, rstd2 = layernorm_fwd(c, p["ln2_g"], p["ln2_b"], cfg.eps, acc)
        y = rt(y2)
        st.update(qkv=qkv, ctx=ctx, lse=lse, a=a, mean1=mean1, rstd1=rstd1, x1=x1,
                  u=u, g=g, c=c, mean2=mean2, rstd2=rstd2)
        return y, st
    if cfg.family == "decoder":
        # pre-LN block of the reference's example model (examples/basic.py:72-91): x + attention
        # of the normalised input, then x + GELU feed-forward of the normalised sum; causal
        # mask and tanh GELU (jax.nn.gelu's default) are the spec's `causal` / `gelu_tanh`
        y1, mean1, rstd1 = layernorm_fwd(x, p["ln1_g"], p["ln1_b"], cfg.eps, acc)
        n1 = rt(y1)
        qkv = rt(mm(n1, p["Wqkv"], acc) + p["bqkv"].astype(acc))
        q, k, v = _split_qkv(cfg, qkv)
        o, lse = attention_fwd(q, k, v, cfg.causal, acc, rt)
        ctx = rt(o.reshape(T, -1))
        h1 = rt(mm(ctx, p["Wo"], acc) + p["bo"].astype(acc) + x.astype(acc))
        y2, mean2, rstd2 = layernorm_fwd(h1, p["ln2_g"], p["ln2_b"], cfg.eps, acc)
        n2 = rt(y2)
        u_full = mm(n2, p["W1"], acc) + p["b1"].astype(acc)
        u = rt(u_full)
        g = rt(gelu(u_full, cfg.gelu_tanh))
        y = rt(mm(g, p["W2"], acc) + p["b2"].astype(acc) + h1.astype(acc))
        st.update(mean1=mean1, rstd1=rstd1, n1=n1, qkv=qkv, ctx=ctx, lse=lse, h1=h1,
                  mean2=mean2, rstd2=rstd2, n2=n2, u=u, g=g)
        return y, st
    if cfg.family in ("llama", "mixtral"):
        y1, rstd1 = rmsnorm_fwd(x, p["rms1_g"], cfg.eps, acc)
        n1 = rt(y1)
        qkv = rt(mm(n1, p["Wqkv"], acc))
        q, k, v = _split_qkv(cfg, qkv)
        cos, sin = rope_tables(cfg.seq, cfg.d, cfg.rope_theta, acc)
        q = rt(rope_apply(q.astype(acc), cos, sin))
        k = rt(rope_apply(k.astype(acc), cos, sin))
        qkv = _join_qkv(cfg, q, k, v)
        o, lse = attention_fwd(q, k, v, cfg.causal, acc, rt)
        ctx = rt(o.reshape(T, -1))
        h1 = rt(mm(ctx, p["Wo"], acc) + x.astype(acc))
        y2, rstd2 = rmsnorm_fwd(h1, p["rms2_g"], cfg.eps, acc)
        n2 = rt(y2)
        st.update(rstd1=rstd1, n1=n1, qkv=qkv, ctx=ctx, lse=lse, h1=h1, rstd2=rstd2, n2=n2)
        if cfg.family == "llama":
            gu = rt(mm(n2, p["Wgu"], acc))
            s = rt(swiglu(gu.astype(acc), cfg.ffn))
            y = rt(mm(s, p["Wd"], acc) + h1.astype(acc))
            st.update(gu=gu, s=s)
            return y, st
        return _moe_fwd(cfg, p, n2, h1, st, nm, forced_ids)
    raise ValueError(cfg.family)


def layer_bwd_i(cfg: LayerCfg, p: dict, st: dict, dy, nm: Numerics):
    """Input-gradient half of the backward.  Returns (dx, wst, small) where
    ``wst`` holds the per-GEMM output cotangents the weight-gradient half
    needs and ``small`` the bias / norm gradients (fp32, unrounded sums)."""
    rt, acc = nm.rt, nm.acc
    T = cfg.tokens
    small, wst = {}, {}
    if cfg.family == "bert":
        dc_, small["ln2_g"], small["ln2_b"] = layernorm_bwd(
            dy, st["c"], st["mean2"], st["rstd2"], p["ln2_g"], acc)
        dc = rt(dc_)
        du = rt(mm(dc, p["W2"].T, acc) * gelu_grad(st["u"].astype(acc), cfg.gelu_tanh))
        dx1 = rt(mm(du, p["W1"].T, acc) + dc.astype(acc))
        da_, small["ln1_g"], small["ln1_b"] = layernorm_bwd(
            dx1, st["a"], st["mean1"], st["rstd1"], p["ln1_g"], acc)
        da = rt(da_)
        dctx = rt(mm(da, p["Wo"].T, acc))
        q, k, v = _split_qkv(cfg, st["qkv"])
        B, S, d = cfg.batch, cfg.seq, cfg.d
        dq, dk, dv = attention_bwd(q, k, v, st["ctx"].reshape(B, S, cfg.n_heads, d),
                                   dctx.reshape(B, S, cfg.n_heads, d), st["lse"],
                                   cfg.causal, acc, rt)
        dqkv = rt(_join_qkv(cfg, dq, dk, dv))
        dx = rt(mm(dqkv, p["Wqkv"].T, acc) + da.astype(acc))
        small["b2"] = dc.astype(acc).sum(0)
        small["b1"] = du.astype(acc).sum(0)
        small["bo"] = da.astype(acc).sum(0)
        small["bqkv"] = dqkv.astype(acc).sum(0)
        wst.update(dc=dc, du=du, da=da, dqkv=dqkv)
        return dx, wst, small
    if cfg.family == "decoder":
        du = rt(mm(dy, p["W2"].T, acc) * gelu_grad(st["u"].astype(acc), cfg.gelu_tanh))
        dn2 = rt(mm(du, p["W1"].T, acc))
        dh1_, small["ln2_g"], small["ln2_b"] = layernorm_bwd(
            dn2, st["h1"], st["mean2"], st["rstd2"], p["ln2_g"], acc)
        dh1 = rt(dh1_ + dy.astype(acc))
        dctx = rt(mm(dh1, p["Wo"].T, acc))
        q, k, v = _split_qkv(cfg, st["qkv"])
        B, S, d = cfg.batch, cfg.seq, cfg.d
        dq, dk, dv = attention_bwd(q, k, v, st["ctx"].reshape(B, S, cfg.n_heads, d),
                                   dctx.reshape(B, S, cfg.n_heads, d), st["lse"],
                                   cfg.causal, acc, rt)
        dqkv = rt(_join_qkv(cfg, dq, dk, dv))
        dn1 = rt(mm(dqkv, p["Wqkv"].T, acc))
        dx_, small["ln1_g"], small["ln1_b"] = layernorm_bwd(
            dn1, st["x"], st["mean1"], st["rstd1"], p["ln1_g"], acc)
        dx = rt(dx_ + dh1.astype(acc))
        small["b2"] = dy.astype(acc).sum(0)
        small["b1"] = du.astype(acc).sum(0)
        small["bo"] = dh1.astype(acc).sum(0)
        small["bqkv"] = dqkv.astype(acc).sum(0)
        wst.update(dy=dy, du=du, dh1=dh1, dqkv=dqkv)
        return dx, wst, small
    if cfg.family in ("llama", "mixtral"):
        if cfg.family == "llama":
            ds = rt(mm(dy, p["Wd"].T, acc))
            dgu = rt(swiglu_bwd(st["gu"].astype(acc), ds.astype(acc), cfg.ffn))
            dn2 = rt(mm(dgu, p["Wgu"].T, acc))
            wst.update(dy=dy, dgu=dgu)
        else:
            dn2 = _moe_bwd_i(cfg, p, st, dy, wst, small, nm)
        dh1_, small["rms2_g"] = rmsnorm_bwd(dn2, st["h1"], st["rstd2"], p["rms2_g"], acc)
        dh1 = rt(dh1_ + dy.astype(acc))
        dctx = rt(mm(dh1, p["Wo"].T, acc))
        q, k, v = _split_qkv(cfg, st["qkv"])
        B, S, d = cfg.batch, cfg.seq, cfg.d
        dq, dk, dv = attention_bwd(q, k, v, st["ctx"].reshape(B, S, cfg.n_heads, d),
                                   dctx.reshape(B, S, cfg.n_heads, d), st["lse"],
                                   cfg.causal, acc, rt)
        cos, sin = rope_tables(cfg.seq, cfg.d, cfg.rope_theta, acc)
        dq = rope_apply(rt(dq).astype(acc), cos, sin, inverse=True)
        dk = rope_apply(rt(dk).astype(acc), cos, sin, inverse=True)
        dqkv = rt(_join_qkv(cfg, dq, dk, rt(dv)))
        dn1 = rt(mm(dqkv, p["Wqkv"].T, acc))
        dx_, small["rms1_g"] = rmsnorm_bwd(dn1, st["x"], st["rstd1"], p["rms1_g"], acc)
        dx = rt(dx_ + dh1.astype(acc))
        wst.update(dh1=dh1, dqkv=dqkv)
        return dx, wst, small
    raise ValueError(cfg.family)


def layer_bwd_w(cfg: LayerCfg, st: dict, wst: dict, nm: Numerics):
    """Weight-gradient half: one transposed GEMM per weight matrix, fp32 (or
    ``acc``) results that the caller adds to its accumulators."""
    acc = nm.acc
    if cfg.family == "bert":
        return {"W2": mm(st["g"].T, wst["dc"], acc), "W1": mm(st["x1"].T, wst["du"], acc),
                "Wo": mm(st["ctx"].T, wst["da"], acc), "Wqkv": mm(st["x"].T, wst["dqkv"], acc)}
    if cfg.family == "decoder":
        return {"W2": mm(st["g"].T, wst["dy"], acc), "W1": mm(st["n2"].T, wst["du"], acc),
                "Wo": mm(st["ctx"].T, wst["dh1"], acc), "Wqkv": mm(st["n1"].T, wst["dqkv"], acc)}
    if cfg.family == "llama":
        return {"Wd": mm(st["s"].T, wst["dy"], acc), "Wgu": mm(st["n2"].T, wst["dgu"], acc),
                "Wo": mm(st["ctx"].T, wst["dh1"], acc), "Wqkv": mm(st["n1"].T, wst["dqkv"], acc)}
    if cfg.family == "mixtral":
        out = _moe_bwd_w(cfg, st, wst, nm)
        out["Wo"] = mm(st["ctx"].T, wst["dh1"], acc)
        out["Wqkv"] = mm(st["n1"].T, wst["dqkv"], acc)
        return out
    raise ValueError(cfg.family)


# ---------------------------------------------------------------------------
# Mixtral-style top-k mixture of SwiGLU experts
# ---------------------------------------------------------------------------
def moe_route(logits, top_k):
    """Top-k by value (ties -> lower expert index), gates = softmax over the
    selected logits.  Returns (expert ids [T,k], gates [T,k])."""
    order = np.argsort(-logits, axis=-1, kind="stable")[:, :top_k]
    sel = np.take_along_axis(logits, order, -1)
    e = np.exp(sel - sel.max(-1, keepdims=True))
    return order, e / e.sum(-1, keepdims=True)


def _moe_fwd(cfg, p, n2, h1, st, nm, forced_ids=None):
    rt, acc = nm.rt, nm.acc
    T, f, E = cfg.tokens, cfg.ffn, cfg.n_experts
    logits = mm(n2, p["Wr"], acc).astype(acc)
    ids, gates = moe_route(logits, cfg.top_k)
    st["own_ids"] = ids
    if forced_ids is not None:
        ids = np.asarray(forced_ids).reshape(T, cfg.top_k).astype(ids.dtype)
        sel = np.take_along_axis(logits, ids, -1)
        e = np.exp(sel - sel.max(-1, keepdims=True))
        gates = e / e.sum(-1, keepdims=True)
    y = h1.astype(acc).copy()
    gu_all = np.zeros((T, cfg.top_k, 2 * f), acc)
    s_all = np.zeros((T, cfg.top_k, f), acc)
    eo_all = np.zeros((T, cfg.top_k, cfg.hidden), acc)
    for e in range(E):
        tok, slot = np.nonzero(ids == e)
        if tok.size == 0:
            continue
        gu = rt(mm(n2[tok], p["Wgu"][e], acc))
        s = rt(swiglu(gu.astype(acc), f))
        eo = rt(mm(s, p["Wd"][e], acc))
        gu_all[tok, slot], s_all[tok, slot], eo_all[tok, slot] = gu, s, eo
    for kk in range(cfg.top_k):
        y += gates[:, kk:kk + 1].astype(acc) * eo_all[:, kk].astype(acc)
    st.update(logits=logits, ids=ids, gates=gates, gu=gu_all, s=s_all, eo=eo_all)
    return rt(y), st


def _moe_bwd_i(cfg, p, st, dy, wst, small, nm):
    rt, acc = nm.rt, nm.acc
    T, f, E, K = cfg.tokens, cfg.ffn, cfg.n_experts, cfg.top_k
    ids, gates = st["ids"], st["gates"].astype(acc)
    dya = dy.astype(acc)
    dgate = np.stack([(dya * st["eo"][:, kk].astype(acc)).sum(-1) for kk in range(K)], -1)
    # softmax over the selected logits
    dsel = gates * (dgate - (gates * dgate).sum(-1, keepdims=True))
    dlogits = np.zeros((T, E), acc)
    np.put_along_axis(dlogits, ids, dsel, -1)
    dlogits = dlogits.astype(acc)
    dn2 = mm(dlogits, p["Wr"].T, acc)
    deo_all = np.zeros((T, K, cfg.hidden), acc)
    dgu_all = np.zeros((T, K, 2 * f), acc)
    for e in range(E):
        tok, slot = np.nonzero(ids == e)
        if tok.size == 0:
            continue
        deo = rt(gates[tok, slot][:, None] * dya[tok])
        ds = rt(mm(deo, p["Wd"][e].T, acc))
        dgu = rt(swiglu_bwd(st["gu"][tok, slot].astype(acc), ds.astype(acc), f))
        dn2[tok] += mm(dgu, p["Wgu"][e].T, acc)
        deo_all[tok, slot], dgu_all[tok, slot] = deo, dgu
    wst.update(deo=deo_all, dgu=dgu_all, dlogits=dlogits)
    return rt(dn2)


def _moe_bwd_w(cfg, st, wst, nm):
    acc = nm.acc
    E, f, h = cfg.n_experts, cfg.ffn, cfg.hidden
    ids = st["ids"]
    dWgu = np.zeros((E, h, 2 * f), acc)
    dWd = np.zeros((E, f, h), acc)
    for e in range(E):
        tok, slot = np.nonzero(ids == e)
        if tok.size == 0:
            continue
        dWd[e] = mm(st["s"][tok, slot].T, wst["deo"][tok, slot], acc)
        dWgu[e] = mm(st["n2"][tok].T, wst["dgu"][tok, slot], acc)
    return {"Wr": mm(st["n2"].T, wst["dlogits"], acc), "Wgu": dWgu, "Wd": dWd}


# ---------------------------------------------------------------------------
# loss of the last stage (README.md:76-78, examples/basic.py:248-250)
# ---------------------------------------------------------------------------
def mse_loss(out, target, n_mubatches, acc=np.float32):
    diff = out.astype(acc) - target.astype(acc)
    loss = (diff * diff).mean() / n_mubatches
    dout = 2.0 * diff / (diff.size * n_mubatches)
    return loss, dout
