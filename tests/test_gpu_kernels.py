"""HIP kernels against the CPU oracle, called through the C ABI.

Tolerances: outputs stored as bf16 are compared with rtol 2e-2 relative to the
tensor's largest magnitude (the bar the north star sets for bf16), fp32
accumulators with rtol 1e-4 where the arithmetic is fp32 end to end."""
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


def dev_bf16(a):
    return rt.DeviceBuffer.from_f32_as_bf16(a)


def rnd(rng, *shape, scale=1.0):
    return L.bf16_round((rng.standard_normal(shape) * scale).astype(np.float32))


def close(got, want, rtol=2e-2, what="", max_bad_frac=0.0):
    parity.close(got, want, rtol, what, max_bad_frac)


def interleave32(gate, up):
    """[.., f] gate and up -> [.., 2f] with blocks of 32 gate columns followed by their 32 ups."""
    f = gate.shape[-1]
    out = np.empty(gate.shape[:-1] + (2 * f,), gate.dtype)
    o = out.reshape(gate.shape[:-1] + (f // 32, 64))
    o[..., :32] = gate.reshape(gate.shape[:-1] + (f // 32, 32))
    o[..., 32:] = up.reshape(up.shape[:-1] + (f // 32, 32))
    return out


GEMM_CASES = [  # (trans_a, trans_b, epilogue)
    (0, 1, rt.EPI_BF16), (0, 1, rt.EPI_GELU), (0, 1, rt.EPI_F32), (0, 1, rt.EPI_ACC_F32),
    (0, 0, rt.EPI_BF16), (0, 0, rt.EPI_DGELU),
    (1, 1, rt.EPI_ACC_F32), (1, 1, rt.EPI_BF16), (1, 1, rt.EPI_F32),
]


@pytest.mark.parametrize("ta,tb,epi", GEMM_CASES)
@pytest.mark.parametrize("tile,m,n,k", [(1, 128, 384, 192), (2, 512, 128, 64), (4, 256, 512, 320), (4, 512, 256, 192),
                                        (3, 384, 512, 192),
                                        (0, 768, 256, 128),
                                        # 384 tiles of 256x256: the half-filled second round runs as
                                        # a launch of 128x256 tiles over the last columns / rows
                                        (0, 4096, 6144, 128), (0, 6144, 4096, 192),
                                        # two rounds of 256x256 tiles and more, the second
                                        # with a 128x256 launch for the last half round
                                        (0, 4096, 8192, 128), (0, 8192, 5120, 192)])
def test_gemm(ta, tb, epi, tile, m, n, k):
    print(f"gemm ta={ta} tb={tb} epi={epi} tile={tile} {m}x{n}x{k}", flush=True)
    rng = np.random.default_rng(m + n + k + 7 * epi)
    A = rnd(rng, m, k)
    B = rnd(rng, n, k)
    want = A @ B.T
    a_h = A.T.copy() if ta else A
    b_h = B.T.copy() if tb else B
    da, db = dev_bf16(a_h), dev_bf16(b_h)
    lda, ldb = a_h.shape[1], b_h.shape[1]
    kw = {}
    keep = []
    if epi in (rt.EPI_BF16, rt.EPI_GELU):
        bias = rnd(rng, n)
        keep.append(dev_bf16(bias))
        kw["bias"] = keep[-1].ptr
        want = want + bias
    if epi == rt.EPI_BF16:
        resid = rnd(rng, m, n)
        keep.append(dev_bf16(resid))
        kw.update(resid=keep[-1].ptr, ldresid=n)
        want = want + resid
    if epi == rt.EPI_DGELU:
        aux = rnd(rng, m, n)
        keep.append(dev_bf16(aux))
        kw.update(aux=keep[-1].ptr, ldaux=n)
        want = want * L.gelu_grad(aux.astype(np.float64)).astype(np.float32)
    f32_out = epi in (rt.EPI_ACC_F32, rt.EPI_F32)
    if epi == rt.EPI_ACC_F32:
        prev = rng.standard_normal((m, n)).astype(np.float32)
        dc = rt.DeviceBuffer.from_numpy(prev)
        want = want + prev
    else:
        dc = rt.DeviceBuffer(m * n * (4 if f32_out else 2))
    if epi == rt.EPI_GELU:
        dc2 = rt.DeviceBuffer(m * n * 2)
        kw.update(c2=dc2.ptr, ldc2=n)
    rt.gemm(da.ptr, db.ptr, dc.ptr, m, n, k, lda, ldb, n, ta, tb, epi, tile=tile, **kw)
    rt.sync()
    if f32_out:
        got = dc.download(np.float32, (m, n))
        close(got, want, 1e-4 * math.sqrt(k), "gemm f32")
    else:
        close(dc.download_bf16((m, n)), want, 1e-2, "gemm bf16")
    if epi == rt.EPI_GELU:
        close(dc2.download_bf16((m, n)), L.gelu(want.astype(np.float64)).astype(np.float32), 1e-2,
              "gemm gelu")


@pytest.mark.parametrize("parts,m,n,k,tile", [(2, 256, 512, 192, 4), (4, 512, 256, 640, 4), (3, 1024, 768, 1024, 3),
                                              (4, 4096, 3072, 512, 0), (2, 4096, 6144, 2048, 0),
                                              (2, 8192, 4096, 256, 0)])   # two rounds of tiles
def test_gemm_contraction_over_several_operand_pairs(parts, m, n, k, tile):
    """C += sum_i A_i^T B_i in one launch (the weight gradients of several microbatches):
    against numpy on the concatenated operands, and bit-identical to ... nothing else: the
    summation order is the launch's own, so the check is numerical."""
    rng = np.random.default_rng(parts + m + n + k)
    As = [rnd(rng, k, m) for _ in range(parts)]          # stored [K, M]: trans_a = 1
    Bs = [rnd(rng, k, n, scale=0.05) for _ in range(parts)]
    prev = rng.standard_normal((m, n)).astype(np.float32)
    want = prev + sum(a.astype(np.float64).T @ b.astype(np.float64) for a, b in zip(As, Bs))
    dA, dB = [dev_bf16(a) for a in As], [dev_bf16(b) for b in Bs]
    dc = rt.DeviceBuffer.from_numpy(prev)
    rt.gemm(dA[0].ptr, dB[0].ptr, dc.ptr, m, n, k, m, n, n, 1, 1, rt.EPI_ACC_F32, tile=tile,
            more=[(a.ptr, b.ptr) for a, b in zip(dA[1:], dB[1:])])
    rt.sync()
    close(dc.download(np.float32, (m, n)), want, 1e-4 * math.sqrt(k * parts), "gemm over operand pairs")
    with pytest.raises(rt.JppError, match="operand pair 1 is null"):
        rt.gemm(dA[0].ptr, dB[0].ptr, dc.ptr, m, n, k, m, n, n, 1, 1, rt.EPI_ACC_F32, more=[(None, dB[0].ptr)])
    with pytest.raises(rt.JppError, match="several operand pairs are supported for"):
        rt.gemm(dA[0].ptr, dB[0].ptr, dc.ptr, m, n, k, m, n, n, 1, 1, rt.EPI_F32, tile=4,
                more=[(dA[0].ptr, dB[0].ptr)])


@pytest.mark.parametrize("parts,k,shapes", [
    (1, 192, [(512, 256), (256, 768)]),
    (4, 128, [(1536, 1024), (1024, 1024), (1024, 7168), (3584, 1024)]),   # 13 x 64 tiles
    (2, 256, [(4096, 6144), (4096, 4096), (256, 256)])])                  # 384 + 256 + 1 tiles
def test_gemm_several_weight_gradients_in_one_launch(parts, k, shapes):
    """jpp_gemm_bf16_multi: independent accumulated weight gradients as one grid of tiles.
    Against numpy, and bit for bit against the same problems launched one by one (contractions
    this short add the old accumulator value in the epilogue whatever the tile, so an output
    element sees the same sum in the same order whichever launch computes it)."""
    rng = np.random.default_rng(parts + k + len(shapes))
    probs, keep, wants, prevs = [], [], [], []
    for m, n in shapes:
        As = [rnd(rng, k, m) for _ in range(parts)]
        Bs = [rnd(rng, k, n, scale=0.05) for _ in range(parts)]
        prev = rng.standard_normal((m, n)).astype(np.float32)
        wants.append(prev + sum(a.astype(np.float64).T @ b.astype(np.float64) for a, b in zip(As, Bs)))
        dA, dB = [dev_bf16(a) for a in As], [dev_bf16(b) for b in Bs]
        dc = rt.DeviceBuffer.from_numpy(prev)
        keep.append((dA, dB, dc))
        prevs.append(prev)
        probs.append(dict(a=dA[0].ptr, b=dB[0].ptr, c=dc.ptr, m=m, n=n, k=k, lda=m, ldb=n, ldc=n,
                          more=[(a.ptr, b.ptr) for a, b in zip(dA[1:], dB[1:])]))
    rt.gemm_multi(probs)
    rt.sync()
    got = [dc.download(np.float32, shp) for (_, _, dc), shp in zip(keep, shapes)]
    for g, w, shp in zip(got, wants, shapes):
        close(g, w, 1e-4 * math.sqrt(k * parts), f"multi {shp}")
    for (dA, dB, dc), prev, (m, n), g in zip(keep, prevs, shapes, got):
        dc.upload(prev)
        # (several operand pairs: the library takes the 256-wide tiles built for that itself)
        rt.gemm(dA[0].ptr, dB[0].ptr, dc.ptr, m, n, k, m, n, n, 1, 1, rt.EPI_ACC_F32,
                more=[(a.ptr, b.ptr) for a, b in zip(dA[1:], dB[1:])])
        rt.sync()
        np.testing.assert_array_equal(dc.download(np.float32, (m, n)), g)
    with pytest.raises(rt.JppError, match="differs from problem 0 in k or k_parts"):
        rt.gemm_multi([probs[0], dict(probs[1], k=64)])
    with pytest.raises(rt.JppError, match="not a plain accumulated weight gradient"):
        rt.gemm_multi([probs[0], dict(probs[1], epilogue=rt.EPI_F32)])
    with pytest.raises(rt.JppError, match="1 to 4 problems"):
        rt.gemm_multi([probs[0]] * 5)


def test_gemm_rejects_bad_shapes():
    d = rt.DeviceBuffer(1 << 16)
    with pytest.raises(rt.JppError, match="multiples of 128"):
        rt.gemm(d.ptr, d.ptr, d.ptr, 100, 128, 64, 64, 64, 128, 0, 0)
    with pytest.raises(rt.JppError, match="unsupported combination"):
        rt.gemm(d.ptr, d.ptr, d.ptr, 128, 128, 64, 128, 64, 128, 1, 0)
    with pytest.raises(rt.JppError, match="null operand"):
        rt.gemm(None, d.ptr, d.ptr, 128, 128, 64, 64, 64, 128, 0, 0)


@pytest.mark.parametrize("batch,seq,heads,rot_heads,d,k,tile", [
    (2, 256, 8, 6, 128, 256, 0),        # 128 x 128 tiles
    (2, 256, 12, 10, 128, 512, 4),      # 256 x 256 tiles
    (1, 256, 8, 6, 64, 256, 0),         # heads of 64
    (1, 512, 16, 12, 64, 128, 3),       # 128 x 256 tiles, four heads per tile
    (1, 4096, 48, 40, 128, 256, 0),     # 384 tiles: a full round and a tail of 128 x 256 tiles
                                        # over the last columns (the Llama-3-8B QKV projection)
    (5, 1024, 32, 32, 128, 128, 0),     # 320 tiles: the tail over the last rows (positions
                                        # continue behind the split)
])
def test_gemm_with_rotary_epilogue(batch, seq, heads, rot_heads, d, k, tile):
    """The forward product that rotates its first rot_heads heads in the epilogue leaves the
    very bits jpp_rope leaves when run over the plain product."""
    print(f"gemm+rope b={batch} s={seq} heads={heads}/{rot_heads} d={d} k={k} tile={tile}", flush=True)
    rng = np.random.default_rng(batch + seq + heads + d)
    m, n = batch * seq, heads * d
    a, w = rnd(rng, m, k), rnd(rng, k, n, scale=0.1)
    cos, sin = L.rope_tables(seq, d, 5e5, np.float32)
    ba, bw = dev_bf16(a), dev_bf16(w)
    bc, bs = rt.DeviceBuffer.from_numpy(cos), rt.DeviceBuffer.from_numpy(sin)
    plain, fused = rt.DeviceBuffer(m * n * 2), rt.DeviceBuffer(m * n * 2)
    rt.gemm(ba.ptr, bw.ptr, plain.ptr, m, n, k, k, n, n, 0, 1, rt.EPI_BF16, tile=tile)
    rt.check(rt.load().jpp_rope(None, plain.ptr, n, bc.ptr, bs.ptr, batch, seq, rot_heads, d, 0))
    rt.gemm(ba.ptr, bw.ptr, fused.ptr, m, n, k, k, n, n, 0, 1, rt.EPI_BF16, tile=tile,
            rope=(bc.ptr, bs.ptr, rot_heads * d, seq, d))
    rt.sync()
    want = plain.download_bf16((m, n))
    got = fused.download_bf16((m, n))
    np.testing.assert_array_equal(got, want)
    # and the pass it replaces does what the oracle says (rotated heads only)
    ref = L.bf16_round(a.astype(np.float64) @ w.astype(np.float64)).reshape(batch, seq, heads, d)
    ref[:, :, :rot_heads] = L.rope_apply(ref[:, :, :rot_heads], cos, sin)
    close(got, ref.reshape(m, n), 2e-2, "rotated product")
    with pytest.raises(rt.JppError, match="rotary"):
        rt.gemm(ba.ptr, bw.ptr, fused.ptr, m, n, k, k, n, n, 0, 1, rt.EPI_BF16,
                rope=(bc.ptr, bs.ptr, rot_heads * d + 8, seq, d))
    with pytest.raises(rt.JppError, match="rotary"):
        rt.gemm(ba.ptr, bw.ptr, fused.ptr, m, n, k, k, n, n, 0, 1, rt.EPI_BF16, resid=ba.ptr,
                ldresid=n, rope=(bc.ptr, bs.ptr, rot_heads * d, seq, d))


@pytest.mark.parametrize("d,causal,hq,hkv,batch,seq", [
    (64, 0, 4, 4, 2, 256), (64, 1, 2, 2, 1, 384), (128, 1, 8, 2, 1, 512),
    (128, 0, 2, 1, 2, 128), (128, 1, 4, 4, 1, 256),
    # shortest causal sequence with grouped heads; an odd number of 128-query blocks; head
    # counts that switch on the per-XCD work order (8 kv heads); the BERT-large head shape
    (128, 1, 4, 1, 2, 128), (64, 1, 8, 2, 2, 640), (128, 1, 32, 8, 1, 512), (64, 0, 16, 16, 2, 512),
    (64, 1, 16, 8, 1, 1024),
    # eight query heads per key-value head (the 70B-shaped layer's grouping)
    (128, 1, 16, 2, 1, 512), (128, 1, 64, 8, 1, 256),
    # head 128 with an odd number of 128-query blocks: the last workgroup of the dQ kernel is half
    # empty, and its last loads go to the slot its first waves stage their output through
    (128, 1, 8, 2, 1, 640),
])
def test_attention_fwd_bwd(d, causal, hq, hkv, batch, seq):
    print(f"attention d={d} causal={causal} hq={hq} hkv={hkv} b={batch} s={seq}", flush=True)
    rng = np.random.default_rng(d + seq + hq)
    T, width = batch * seq, (hq + 2 * hkv) * d
    qkv = rnd(rng, T, width)
    do = rnd(rng, T, hq * d)
    q = qkv[:, :hq * d].reshape(batch, seq, hq, d)
    k = qkv[:, hq * d:(hq + hkv) * d].reshape(batch, seq, hkv, d)
    v = qkv[:, (hq + hkv) * d:].reshape(batch, seq, hkv, d)
    # the oracle rounds the probabilities (and, backward, the score cotangents) to bf16 where
    # they become matrix-product operands, as any bf16 path does
    o_w, lse_w = L.attention_fwd(q, k, v, bool(causal), rt=L.bf16_round)
    dq_w, dk_w, dv_w = L.attention_bwd(q, k, v, L.bf16_round(o_w),
                                       do.reshape(batch, seq, hq, d), lse_w, bool(causal),
                                       rt=L.bf16_round)
    dqkv_w = np.concatenate([dq_w.reshape(T, -1), dk_w.reshape(T, -1), dv_w.reshape(T, -1)], -1)

    dqkv_d = rt.DeviceBuffer(T * width * 2)
    dqkv_d.zero()
    b_qkv, b_o, b_do = dev_bf16(qkv), rt.DeviceBuffer(T * hq * d * 2), dev_bf16(do)
    b_lse = rt.DeviceBuffer(batch * hq * seq * 4)
    b_delta = rt.DeviceBuffer(2 * batch * hq * seq * 4)
    a = rt.AttnArgs(b_qkv.ptr, b_qkv.ptr + hq * d * 2, b_qkv.ptr + (hq + hkv) * d * 2, b_o.ptr,
                    b_lse.ptr, b_do.ptr, dqkv_d.ptr, dqkv_d.ptr + hq * d * 2,
                    dqkv_d.ptr + (hq + hkv) * d * 2, b_delta.ptr,
                    width, width, width, hq * d, hq * d, width, width, width,
                    batch, seq, hq, hkv, d, causal)
    rt.check(rt.load().jpp_attn_fwd(None, C.byref(a)))
    rt.sync()
    close(b_o.download_bf16((T, hq * d)), o_w.reshape(T, -1), 2e-2, "attn out")
    np.testing.assert_allclose(b_lse.download(np.float32, (batch, hq, seq)), lse_w, rtol=0,
                               atol=2e-2)
    # the backward is checked on the oracle's forward results: `o` enters the row term
    # sum(dO * O) that every score cotangent of the row shares, so a one-ulp difference in a
    # few elements of `o` would otherwise be charged to the backward kernels
    b_o.upload(rt.to_bf16_bits(o_w.reshape(T, -1)))
    b_lse.upload(np.ascontiguousarray(lse_w, dtype=np.float32))
    rt.check(rt.load().jpp_attn_bwd(None, C.byref(a)))
    rt.sync()
    got = dqkv_d.download_bf16((T, width))
    close(got[:, :hq * d], dqkv_w[:, :hq * d], 2e-2, "dq")
    close(got[:, hq * d:(hq + hkv) * d], dqkv_w[:, hq * d:(hq + hkv) * d], 2e-2, "dk")
    close(got[:, (hq + hkv) * d:], dqkv_w[:, (hq + hkv) * d:], 2e-2, "dv")
    # with rotary tables the backward writes dq and dk already rotated back: the same values
    # a pass of jpp_rope(inverse) over the plain result leaves (q and k heads are adjacent)
    cos, sin = L.rope_tables(seq, d, 5e5, np.float32)
    bc, bs = rt.DeviceBuffer.from_numpy(cos), rt.DeviceBuffer.from_numpy(sin)
    rt.check(rt.load().jpp_rope(None, dqkv_d.ptr, width, bc.ptr, bs.ptr, batch, seq, hq + hkv, d, 1))
    rt.sync()
    want_r = dqkv_d.download_bf16((T, width))
    dqkv_d.zero()
    a.rope_cos, a.rope_sin = bc.ptr, bs.ptr
    rt.check(rt.load().jpp_attn_bwd(None, C.byref(a)))
    rt.sync()
    np.testing.assert_array_equal(dqkv_d.download_bf16((T, width)), want_r)
    # the kernels read the tables 16 bytes at a time: a table that is not aligned so is refused
    a.rope_cos = bc.ptr + 4
    with pytest.raises(rt.JppError, match="rotary tables must be 16-byte aligned"):
        rt.check(rt.load().jpp_attn_bwd(None, C.byref(a)))
    a.rope_cos, a.rope_sin = bc.ptr, None
    with pytest.raises(rt.JppError, match="rope_cos and rope_sin go together"):
        rt.check(rt.load().jpp_attn_bwd(None, C.byref(a)))


@pytest.mark.parametrize("d,causal,slope", [(128, 1, 40.0), (128, 0, 40.0), (64, 1, 12.0),
                                            (128, 1, -40.0), (64, 0, 300.0)])
def test_attention_forward_with_drifting_row_maxima(d, causal, slope):
    """Scores that grow (or fall) steadily along the key axis: the running maximum of every row
    moves in every block of keys, so the rescale of the running sums and outputs carries weight
    in the result.  slope is the growth of the scaled score over the whole sequence (300: a jump
    of 2^27 per block; negative: the first block holds every maximum)."""
    print(f"attention drift d={d} causal={causal} slope={slope}", flush=True)
    rng = np.random.default_rng(int(abs(slope)) + d + causal)
    batch, seq, hq, hkv = 1, 1024, 4, 2
    T, width = batch * seq, (hq + 2 * hkv) * d
    u = np.ones(d, np.float32) / np.sqrt(d)
    ramp = (np.arange(seq, dtype=np.float32) / seq)[:, None]
    q = 0.3 * rng.standard_normal((T, hq, d)).astype(np.float32) + np.sqrt(np.sqrt(d) * abs(slope)) * u
    k = 0.3 * rng.standard_normal((T, hkv, d)).astype(np.float32) + \
        (np.sign(slope) * np.sqrt(np.sqrt(d) * abs(slope)) * ramp * u)[:, None, :]
    v = rng.standard_normal((T, hkv, d)).astype(np.float32)
    qkv = L.bf16_round(np.concatenate([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], -1))
    q4 = qkv[:, :hq * d].reshape(batch, seq, hq, d)
    k4 = qkv[:, hq * d:(hq + hkv) * d].reshape(batch, seq, hkv, d)
    v4 = qkv[:, (hq + hkv) * d:].reshape(batch, seq, hkv, d)
    o_w, lse_w = L.attention_fwd(q4, k4, v4, bool(causal), rt=L.bf16_round)
    # the case is what it claims: along the keys a row's scaled scores span about |slope|
    s0 = (q4[0, -1, 0] @ k4[0, :, 0].T) / np.sqrt(d)
    assert abs(float(s0[-1] - s0[0])) > 0.6 * abs(slope)
    b_qkv, b_o = dev_bf16(qkv), rt.DeviceBuffer(T * hq * d * 2)
    b_lse = rt.DeviceBuffer(batch * hq * seq * 4)
    a = rt.AttnArgs(b_qkv.ptr, b_qkv.ptr + hq * d * 2, b_qkv.ptr + (hq + hkv) * d * 2, b_o.ptr,
                    b_lse.ptr, None, None, None, None, None,
                    width, width, width, hq * d, hq * d, width, width, width,
                    batch, seq, hq, hkv, d, causal)
    rt.check(rt.load().jpp_attn_fwd(None, C.byref(a)))
    rt.sync()
    got = b_o.download_bf16((T, hq * d))
    assert np.isfinite(got).all()
    close(got, o_w.reshape(T, -1), 2e-2, "attn out")
    np.testing.assert_allclose(b_lse.download(np.float32, (batch, hq, seq)), lse_w, rtol=2e-3,
                               atol=2e-2)


@pytest.mark.parametrize("ln,rows,cols", [(True, 300, 256), (True, 1024, 1024), (False, 512, 4096),
                                          (False, 130, 8192), (False, 64, 128), (True, 261, 4096),
                                          (True, 1030, 8192), (True, 140, 6144), (False, 140, 5120)])
def test_norm_fwd_bwd(ln, rows, cols):
    print(f"norm ln={ln} {rows}x{cols}", flush=True)
    rng = np.random.default_rng(rows + cols)
    x, dy, resid = rnd(rng, rows, cols, scale=2.0), rnd(rng, rows, cols), rnd(rng, rows, cols)
    g = L.bf16_round(1 + 0.1 * rng.standard_normal(cols).astype(np.float32))
    b = L.bf16_round(0.1 * rng.standard_normal(cols).astype(np.float32))
    eps = 1e-5
    if ln:
        y_w, mean_w, rstd_w = L.layernorm_fwd(x, g, b, eps)
        dx_w, dg_w, db_w = L.layernorm_bwd(dy, x, mean_w, rstd_w, g)
    else:
        y_w, rstd_w = L.rmsnorm_fwd(x, g, eps)
        dx_w, dg_w = L.rmsnorm_bwd(dy, x, rstd_w, g)
    dx_w = dx_w + resid
    bx, bg, bb, bdy, br = dev_bf16(x), dev_bf16(g), dev_bf16(b), dev_bf16(dy), dev_bf16(resid)
    by, bdx = rt.DeviceBuffer(rows * cols * 2), rt.DeviceBuffer(rows * cols * 2)
    bmean, brstd = rt.DeviceBuffer(rows * 4), rt.DeviceBuffer(rows * 4)
    prev_g = rng.standard_normal(cols).astype(np.float32)
    prev_b = rng.standard_normal(cols).astype(np.float32)
    bdg, bdb = rt.DeviceBuffer.from_numpy(prev_g), rt.DeviceBuffer.from_numpy(prev_b)
    part = rt.DeviceBuffer(2 * rt.NORM_PARTIALS * cols * 4)
    a = rt.NormArgs(bx.ptr, bg.ptr, bb.ptr if ln else None, by.ptr, bmean.ptr if ln else None,
                    brstd.ptr, bdy.ptr, br.ptr, bdx.ptr, bdg.ptr, bdb.ptr if ln else None,
                    part.ptr, rows, cols, eps)
    rt.check(rt.load().jpp_norm_fwd(None, C.byref(a)))
    rt.check(rt.load().jpp_norm_bwd(None, C.byref(a)))
    rt.sync()
    close(by.download_bf16((rows, cols)), y_w, 1e-2, "norm y")
    np.testing.assert_allclose(brstd.download(np.float32, (rows,)), rstd_w, rtol=1e-4)
    if ln:
        np.testing.assert_allclose(bmean.download(np.float32, (rows,)), mean_w, rtol=1e-3, atol=1e-5)
    close(bdx.download_bf16((rows, cols)), dx_w, 1e-2, "norm dx")
    close(bdg.download(np.float32, (cols,)), prev_g + dg_w, 1e-3, "dgamma")
    if ln:
        close(bdb.download(np.float32, (cols,)), prev_b + db_w, 1e-3, "dbeta")


def test_swiglu_rope_accum_colsum_cast():
    rng = np.random.default_rng(5)
    lib = rt.load()
    rows, f = 96, 1024
    gu, ds = rnd(rng, rows, 2 * f, scale=2.0), rnd(rng, rows, f)
    bgu, bds = dev_bf16(gu), dev_bf16(ds)
    bs, bdgu = rt.DeviceBuffer(rows * f * 2), rt.DeviceBuffer(rows * 2 * f * 2)
    rt.check(lib.jpp_swiglu_fwd(None, bgu.ptr, bs.ptr, rows, f, 0))
    rt.check(lib.jpp_swiglu_bwd(None, bgu.ptr, bds.ptr, bdgu.ptr, rows, f, 0))
    rt.sync()
    close(bs.download_bf16((rows, f)), L.swiglu(gu, f), 1e-2, "swiglu")
    dgu_w = L.swiglu_bwd(gu, ds, f)
    close(bdgu.download_bf16((rows, 2 * f)), dgu_w, 1e-2, "swiglu bwd")
    # the same through the layout with gate and up interleaved in blocks of 32 columns
    bgi = dev_bf16(interleave32(gu[:, :f], gu[:, f:]))
    rt.check(lib.jpp_swiglu_fwd(None, bgi.ptr, bs.ptr, rows, f, 1))
    rt.check(lib.jpp_swiglu_bwd(None, bgi.ptr, bds.ptr, bdgu.ptr, rows, f, 1))
    rt.sync()
    close(bs.download_bf16((rows, f)), L.swiglu(gu, f), 1e-2, "swiglu, interleaved")
    close(bdgu.download_bf16((rows, 2 * f)), interleave32(dgu_w[:, :f], dgu_w[:, f:]), 1e-2,
          "swiglu bwd, interleaved")

    batch, seq, heads, d, extra = 2, 64, 6, 128, 2
    ld = (heads + extra) * d
    x = rnd(rng, batch * seq, ld)
    cos, sin = L.rope_tables(seq, d, 5e5, np.float32)
    bc, bsn = rt.DeviceBuffer.from_numpy(cos), rt.DeviceBuffer.from_numpy(sin)
    for inverse in (0, 1):
        bx = dev_bf16(x)
        rt.check(lib.jpp_rope(None, bx.ptr, ld, bc.ptr, bsn.ptr, batch, seq, heads, d, inverse))
        rt.sync()
        want = x.copy()
        rot = L.rope_apply(x[:, :heads * d].reshape(batch, seq, heads, d), cos, sin, bool(inverse))
        want[:, :heads * d] = rot.reshape(batch * seq, -1)
        got = bx.download_bf16((batch * seq, ld))
        close(got, want, 1e-2, "rope")
        np.testing.assert_array_equal(got[:, heads * d:], x[:, heads * d:])

    for n, f32 in [(8 * 1000 + 3, 0), (4096, 1), (5, 0)]:
        acc = rng.standard_normal(n).astype(np.float32)
        g = rng.standard_normal(n).astype(np.float32)
        if not f32:
            g = L.bf16_round(g)
        bacc = rt.DeviceBuffer.from_numpy(acc)
        bg = rt.DeviceBuffer.from_numpy(g if f32 else rt.to_bf16_bits(g))
        rt.check(lib.jpp_grad_accum_f32(None, bacc.ptr, bg.ptr, n, f32))
        rt.sync()
        np.testing.assert_array_equal(bacc.download(np.float32, (n,)), acc + g)

    rows, cols = 1000, 3072
    xx = rnd(rng, rows, cols)
    acc = rng.standard_normal(cols).astype(np.float32)
    bacc, bx = rt.DeviceBuffer.from_numpy(acc), dev_bf16(xx)
    part = rt.DeviceBuffer(rt.NORM_PARTIALS * cols * 4)
    rt.check(lib.jpp_colsum_accum(None, bx.ptr, cols, rows, cols, bacc.ptr, part.ptr))
    rt.sync()
    close(bacc.download(np.float32, (cols,)), acc + xx.sum(0), 1e-4, "colsum")
    # several tensors at once (a layer's bias gradients): widths 256 / 1024 / 8 / 3072, one of
    # them a column slice of a wider tensor
    widths, lds = [256, 1024, 8, 3072], [256, 1024, 64, 3072]
    xs = [rnd(rng, rows, ld) for ld in lds]
    accs = [rng.standard_normal(w).astype(np.float32) for w in widths]
    bxs, baccs = [dev_bf16(x) for x in xs], [rt.DeviceBuffer.from_numpy(a) for a in accs]
    items = (rt.ColsumItem * 4)(*[rt.ColsumItem(bx.ptr, ld, w, ba.ptr)
                                  for bx, ld, w, ba in zip(bxs, lds, widths, baccs)])
    part = rt.DeviceBuffer(rt.NORM_PARTIALS * sum(widths) * 4)
    rt.check(lib.jpp_colsum_accum_multi(None, 4, items, rows, part.ptr))
    rt.sync()
    for x, w, a, ba in zip(xs, widths, accs, baccs):
        close(ba.download(np.float32, (w,)), a + x[:, :w].sum(0), 1e-4, f"colsum of {w} columns")
    assert lib.jpp_colsum_accum_multi(None, 5, items, rows, part.ptr) == -1

    src = rng.standard_normal(1001).astype(np.float32)
    bsrc, bdst = rt.DeviceBuffer.from_numpy(src), rt.DeviceBuffer(1001 * 2)
    rt.check(lib.jpp_cast_f32_to_bf16(None, bsrc.ptr, bdst.ptr, 1001))
    rt.sync()
    np.testing.assert_array_equal(bdst.download(np.uint16, (1001,)), L.f32_to_bf16_bits(src))
    np.testing.assert_array_equal(rt.to_bf16_bits(src), L.f32_to_bf16_bits(src))


def moe_setup(rng, T, h):
    lib = rt.load()
    E = 8
    x = rnd(rng, T, h)
    wr = rnd(rng, h, E, scale=1.0 / math.sqrt(h))
    cap = lib.jpp_moe_capacity(T, E, 2)
    bufs = dict(x=dev_bf16(x), wr=dev_bf16(wr), ids=rt.DeviceBuffer(T * 8),
                gates=rt.DeviceBuffer(T * 8), row_of=rt.DeviceBuffer(T * 8),
                tok_of=rt.DeviceBuffer(cap * 4), gate_of=rt.DeviceBuffer(cap * 4),
                seg=rt.DeviceBuffer(64 * 4), work=rt.DeviceBuffer(2 * ((T + 255) // 256) * E * 4 + 256))
    a = rt.MoeArgs(bufs["x"].ptr, bufs["wr"].ptr, bufs["ids"].ptr, bufs["gates"].ptr,
                   bufs["row_of"].ptr, bufs["tok_of"].ptr, bufs["gate_of"].ptr, bufs["seg"].ptr,
                   bufs["work"].ptr, T, h, E, 2)
    return lib, a, bufs, x, wr, cap


def test_moe_routing_and_permutation():
    check_moe(11, 1000, 256)


def check_moe(seed, T, h):
    """Routing, the token permutation it implies, gather / combine and their backward, the
    router's weight gradient: T tokens of width h over the 8 experts."""
    rng = np.random.default_rng(seed)
    E = 8
    lib, a, b, x, wr, cap = moe_setup(rng, T, h)
    rt.check(lib.jpp_moe_route(None, C.byref(a)))
    rt.sync()
    ids = b["ids"].download(np.int32, (T, 2))
    gates = b["gates"].download(np.float32, (T, 2))
    logits = (x.astype(np.float64) @ wr.astype(np.float64))
    ids_w, gates_w = L.moe_route(logits, 2)
    # a routing decision may differ only where two logits are within rounding of each other
    diff = np.nonzero((ids != ids_w).any(1))[0]
    for t in diff:
        top3 = np.sort(logits[t])[::-1][:3]
        assert min(top3[0] - top3[1], top3[1] - top3[2]) < 1e-4, (t, top3)
    same = np.setdiff1d(np.arange(T), diff)
    np.testing.assert_allclose(gates[same], gates_w[same], rtol=1e-4, atol=1e-6)
    seg_all = b["seg"].download(np.int32, (2 * E + 1,))
    seg, seg_rows = seg_all[:E + 1], seg_all[E + 1:]
    np.testing.assert_array_equal(seg_rows, [(ids == e).any(1).sum() for e in range(E)])
    row_of = b["row_of"].download(np.int32, (T, 2))
    tok_of = b["tok_of"].download(np.int32, (cap,))
    gate_of = b["gate_of"].download(np.float32, (cap,))
    assert seg[0] == 0 and (seg % 256 == 0).all() and seg[E] <= cap
    for e in range(E):
        toks = np.nonzero((ids == e).any(1))[0]            # token order inside the group
        rows = np.arange(seg[e], seg[e] + len(toks))
        np.testing.assert_array_equal(tok_of[rows], toks)
        assert (tok_of[seg[e] + len(toks):seg[e + 1]] == -1).all()
        slot = (ids[toks] == e).argmax(1)
        np.testing.assert_array_equal(row_of[toks, slot], rows)
        np.testing.assert_array_equal(gate_of[rows], gates[toks, slot])

    # gather / combine forward / backward helpers
    xp = rt.DeviceBuffer(cap * h * 2)
    rt.check(lib.jpp_moe_gather(None, C.byref(a), b["x"].ptr, xp.ptr))
    rt.sync()
    xp_h = xp.download_bf16((cap, h))
    valid = tok_of >= 0
    np.testing.assert_array_equal(xp_h[:seg[E]][valid[:seg[E]]], x[tok_of[:seg[E]][valid[:seg[E]]]])
    assert not xp_h[:seg[E]][~valid[:seg[E]]].any()
    eo, resid, dy = rnd(rng, cap, h), rnd(rng, T, h), rnd(rng, T, h)
    b_eo, b_res, b_dy = dev_bf16(eo), dev_bf16(resid), dev_bf16(dy)
    y = rt.DeviceBuffer(T * h * 2)
    rt.check(lib.jpp_moe_combine_fwd(None, C.byref(a), b_eo.ptr, b_res.ptr, y.ptr))
    want = resid + gates[:, :1] * eo[row_of[:, 0]] + gates[:, 1:] * eo[row_of[:, 1]]
    rt.sync()
    close(y.download_bf16((T, h)), want, 1e-2, "moe combine")
    dlog, deo = rt.DeviceBuffer(T * E * 4), rt.DeviceBuffer(cap * h * 2)
    rt.check(lib.jpp_moe_bwd_prepare(None, C.byref(a), b_dy.ptr, b_eo.ptr, dlog.ptr, deo.ptr))
    rt.sync()
    dgate = np.stack([(dy * eo[row_of[:, k]]).sum(-1) for k in range(2)], -1)
    dsel = gates * (dgate - (gates * dgate).sum(-1, keepdims=True))
    dl_w = np.zeros((T, E), np.float32)
    np.put_along_axis(dl_w, ids.astype(np.int64), dsel, -1)
    close(dlog.download(np.float32, (T, E)), dl_w, 1e-4, "dlogits")
    deo_w = np.zeros((cap, h), np.float32)
    deo_w[row_of[:, 0]] = gates[:, :1] * dy
    deo_w[row_of[:, 1]] = gates[:, 1:] * dy
    close(deo.download_bf16((cap, h))[:seg[E]], deo_w[:seg[E]], 1e-2, "deo")
    dx = rt.DeviceBuffer(T * h * 2)
    rt.check(lib.jpp_moe_combine_bwd(None, C.byref(a), b_eo.ptr, dlog.ptr, dx.ptr))
    rt.sync()
    close(dx.download_bf16((T, h)), eo[row_of[:, 0]] + eo[row_of[:, 1]] + dl_w @ wr.T, 1e-2, "moe dx")
    acc0 = rng.standard_normal((h, E)).astype(np.float32)
    acc, part = rt.DeviceBuffer.from_numpy(acc0), rt.DeviceBuffer(64 * h * E * 4)
    rt.check(lib.jpp_moe_router_wgrad(None, C.byref(a), b["x"].ptr, dlog.ptr, acc.ptr, part.ptr))
    rt.sync()
    close(acc.download(np.float32, (h, E)), acc0 + x.T @ dl_w, 1e-4, "dWr")


def test_grouped_gemm():
    rng = np.random.default_rng(12)
    E, h, f = 8, 256, 512
    counts = [300, 0, 256, 17, 700, 1, 255, 512]
    seg = np.zeros(E + 1, np.int32)
    for e, c in enumerate(counts):
        seg[e + 1] = seg[e] + (c + 255) // 256 * 256
    cap = int(seg[E]) + 512                      # capacity beyond the last group
    xp = np.zeros((cap, h), np.float32)
    for e, c in enumerate(counts):
        xp[seg[e]:seg[e] + c] = rnd(rng, c, h)
    w = rnd(rng, E, h, f, scale=0.1)
    b_seg, b_xp, b_w = rt.DeviceBuffer.from_numpy(seg), dev_bf16(xp), dev_bf16(w)
    out = rt.DeviceBuffer(cap * f * 2)
    out.zero()
    rt.gemm(b_xp.ptr, b_w.ptr, out.ptr, cap, f, h, h, f, f, 0, 1, rt.EPI_BF16, seg=b_seg.ptr, n_seg=E,
            group_mode=1, stride_b=h * f)
    rt.sync()
    got = out.download_bf16((cap, f))
    for e in range(E):
        if counts[e]:
            close(got[seg[e]:seg[e + 1]], xp[seg[e]:seg[e + 1]] @ w[e], 1e-2, f"group {e}")
    assert not got[seg[E]:].any(), "tiles past the last group must not be written"
    # row counts change nothing for row-grouped products: same bits
    b_rows = rt.DeviceBuffer.from_numpy(np.array(counts, np.int32))
    out2 = rt.DeviceBuffer(cap * f * 2)
    out2.zero()
    rt.gemm(b_xp.ptr, b_w.ptr, out2.ptr, cap, f, h, h, f, f, 0, 1, rt.EPI_BF16, seg=b_seg.ptr, n_seg=E,
            group_mode=1, stride_b=h * f, seg_rows=b_rows.ptr)
    rt.sync()
    np.testing.assert_array_equal(out2.download_bf16((cap, f)), got)
    # weight gradients: per-expert contraction over the expert's rows, accumulated
    dy = np.zeros((cap, f), np.float32)
    dy[:seg[E]] = rnd(rng, int(seg[E]), f)
    acc0 = rng.standard_normal((E, h, f)).astype(np.float32)
    b_dy, b_acc = dev_bf16(dy), rt.DeviceBuffer.from_numpy(acc0)
    rt.gemm(b_xp.ptr, b_dy.ptr, b_acc.ptr, h, f, 0, h, f, f, 1, 1, rt.EPI_ACC_F32, seg=b_seg.ptr,
            n_seg=E, group_mode=2, stride_c=h * f)
    rt.sync()
    got = b_acc.download(np.float32, (E, h, f))
    for e in range(E):
        want = acc0[e] + xp[seg[e]:seg[e + 1]].T @ dy[seg[e]:seg[e + 1]]
        close(got[e], want, 1e-3, f"dW group {e}")
    np.testing.assert_array_equal(got[1], acc0[1])       # empty group: untouched
    # with the groups' row counts, steps of the contraction that hold only padding are left out
    b_acc2 = rt.DeviceBuffer.from_numpy(acc0)
    rt.gemm(b_xp.ptr, b_dy.ptr, b_acc2.ptr, h, f, 0, h, f, f, 1, 1, rt.EPI_ACC_F32, seg=b_seg.ptr,
            n_seg=E, group_mode=2, stride_c=h * f, seg_rows=b_rows.ptr)
    rt.sync()
    got2 = b_acc2.download(np.float32, (E, h, f))
    for e in range(E):
        want = acc0[e] + xp[seg[e]:seg[e + 1]].T @ dy[seg[e]:seg[e + 1]]
        close(got2[e], want, 1e-3, f"dW group {e}, padding steps skipped")
    np.testing.assert_array_equal(got2[1], acc0[1])
    # several operand pairs, each with its own row groups (the expert weight gradients of
    # several microbatches, routed differently): one launch adds all of them
    counts_b = [0, 300, 256, 1, 0, 515, 70, 64]
    seg_b = np.zeros(E + 1, np.int32)
    for e, c in enumerate(counts_b):
        seg_b[e + 1] = seg_b[e] + (c + 255) // 256 * 256
    cap_b = int(seg_b[E]) + 256
    xp_b, dy_b = np.zeros((cap_b, h), np.float32), np.zeros((cap_b, f), np.float32)
    for e, c in enumerate(counts_b):
        xp_b[seg_b[e]:seg_b[e] + c] = rnd(rng, c, h)
        dy_b[seg_b[e]:seg_b[e] + c] = rnd(rng, c, f)
    d_seg_b, d_rows_b = rt.DeviceBuffer.from_numpy(seg_b), rt.DeviceBuffer.from_numpy(np.array(counts_b, np.int32))
    d_xp_b, d_dy_b = dev_bf16(xp_b), dev_bf16(dy_b)
    b_acc3 = rt.DeviceBuffer.from_numpy(acc0)
    rt.gemm(b_xp.ptr, b_dy.ptr, b_acc3.ptr, h, f, 0, h, f, f, 1, 1, rt.EPI_ACC_F32, seg=b_seg.ptr,
            n_seg=E, group_mode=2, stride_c=h * f, seg_rows=b_rows.ptr, tile=4,
            more=[(d_xp_b.ptr, d_dy_b.ptr), (b_xp.ptr, b_dy.ptr)],
            more_seg=[(d_seg_b.ptr, d_rows_b.ptr), (b_seg.ptr, b_rows.ptr)])
    rt.sync()
    got3 = b_acc3.download(np.float32, (E, h, f))
    for e in range(E):
        want = (acc0[e] + 2 * (xp[seg[e]:seg[e + 1]].T @ dy[seg[e]:seg[e + 1]])
                + xp_b[seg_b[e]:seg_b[e + 1]].T @ dy_b[seg_b[e]:seg_b[e + 1]])
        close(got3[e], want, 2e-3, f"dW group {e} over three operand pairs")
    with pytest.raises(rt.JppError, match="needs its row groups"):
        rt.gemm(b_xp.ptr, b_dy.ptr, b_acc3.ptr, h, f, 0, h, f, f, 1, 1, rt.EPI_ACC_F32, seg=b_seg.ptr,
                n_seg=E, group_mode=2, stride_c=h * f, tile=4, more=[(d_xp_b.ptr, d_dy_b.ptr)])


@pytest.mark.parametrize("trans_b", [1, 0], ids=["nn", "nt"])
@pytest.mark.parametrize("counts,h", [
    ([520, 300, 256, 1100, 700, 300, 255, 513], 128),    # 20 tile rows x 16: last round 64 tiles -> 4 rows split off
    ([520, 300, 256, 1100, 700, 300, 255, 513], 2048),   # ... with the deeper prefetch of a long contraction
    ([512, 512, 512, 512, 512, 512, 512, 512], 128),     # 16 x 16 = one full round: nothing to split
    ([1024, 512, 512, 512, 512, 512, 512, 600], 128),    # 19 x 16: 48 tiles -> 3 rows split off
    ([1024, 512, 512, 512, 512, 512, 512, 1300], 128),   # 22 x 16: 96 tiles -> 6 rows split off, as 128x256 tiles
    ([1024, 512, 512, 512, 512, 512, 512, 1300], 2048),
    ([2048, 512, 512, 512, 512, 512, 512, 1300], 128),   # 26 x 16: 160 tiles in the last round: no split
    ([256, 0, 0, 0, 0, 0, 0, 1], 128),                   # 2 x 16: less than a round: no split
    # 69 tile rows in groups of 8 - 10 (72 with the capacity: the XCDs split the tile columns and
    # walk them group by group); 80 tiles in the last round -> 5 rows split off
    ([2300, 2048, 1900, 2200, 2100, 2500, 1800, 2000], 128),
    ([5000, 0, 300, 6100, 2100, 40, 1800, 2000], 128),   # groups of 20, 0, 2, 24, 9, 1, 8, 8 tile rows
], ids=["rest64", "rest64-long", "full", "rest48", "rest96", "rest96-long", "rest160", "small",
        "tall", "tall-uneven"])
def test_grouped_gemm_last_round(counts, h, trans_b):
    """Row-grouped products whose 256x256 tiles end in a round that fills at most half of the
    CUs run that round's rows as 128x128 tiles (up to 64 tiles of 256x256) or 128x256 tiles (up
    to 128) in launches of their own; where the split falls is decided on the device from the
    rows in use.  Bit for bit the single launch on 256x256
    tiles (the caller's choice of tile switches the split off), and right against numpy."""
    rng = np.random.default_rng(sum(counts) + trans_b)
    E, f = 8, 4096
    seg = np.zeros(E + 1, np.int32)
    for e, c in enumerate(counts):
        seg[e + 1] = seg[e] + (c + 255) // 256 * 256
    cap = int(seg[E]) + 768                       # the grid covers the capacity, not the rows in use
    xp = np.zeros((cap, h), np.float32)
    for e, c in enumerate(counts):
        xp[seg[e]:seg[e] + c] = rnd(rng, c, h)
    w = rnd(rng, E, h, f, scale=0.1 if h < 1024 else 0.03)
    wd = np.ascontiguousarray(w.transpose(0, 2, 1)) if not trans_b else w     # [E, f, h] for nt
    b_seg, b_xp, b_w = rt.DeviceBuffer.from_numpy(seg), dev_bf16(xp), dev_bf16(wd)
    outs = []
    for tile in (0, 4):
        out = rt.DeviceBuffer(cap * f * 2)
        out.zero()
        print(f"grouped product, counts {counts}, h {h}, trans_b {trans_b}, tile {tile}", flush=True)
        rt.gemm(b_xp.ptr, b_w.ptr, out.ptr, cap, f, h, h, f if trans_b else h, f, 0, trans_b,
                rt.EPI_BF16, seg=b_seg.ptr, n_seg=E, group_mode=1, stride_b=h * f, tile=tile)
        rt.sync()
        outs.append(out.download_bf16((cap, f)))
    np.testing.assert_array_equal(outs[0], outs[1])
    xb = xp
    for e in range(E):
        if counts[e]:
            close(outs[0][seg[e]:seg[e + 1]], xb[seg[e]:seg[e + 1]] @ w[e], 1e-2, f"group {e}")
    assert not outs[0][seg[E]:].any(), "rows past the last group must not be written"


@pytest.mark.parametrize("tile,m,f,k", [(1, 128, 128, 64), (2, 256, 256, 128), (4, 512, 256, 192),
                                        (3, 384, 256, 128),
                                        # split into 256x256 + 128x256 launches: the forward at
                                        # f = 3072 (N = 6144), the backward at f = 6144
                                        (0, 4096, 3072, 128), (0, 4096, 6144, 64),
                                        (0, 8192, 4096, 128)])   # several rounds of tiles
def test_gemm_swiglu_epilogues(tile, m, f, k):
    rng = np.random.default_rng(21)
    x = rnd(rng, m, k)
    wg, wu = rnd(rng, k, f, scale=0.2), rnd(rng, k, f, scale=0.2)
    w = interleave32(wg, wu)                       # device layout of the fused projection
    gu, s = rt.DeviceBuffer(m * 2 * f * 2), rt.DeviceBuffer(m * f * 2)
    dx, dw = dev_bf16(x), dev_bf16(w)
    rt.gemm(dx.ptr, dw.ptr, gu.ptr, m, 2 * f, k, k, 2 * f, 2 * f, 0, 1, rt.EPI_SWIGLU, c2=s.ptr,
            ldc2=f, tile=tile)
    rt.sync()
    g_w, u_w = L.bf16_round(x @ wg), L.bf16_round(x @ wu)
    gu_h = gu.download_bf16((m, 2 * f))
    close(gu_h, interleave32(g_w, u_w), 1e-2, "gate/up")
    # the second output follows from the first exactly as the separate kernel computes it
    g_h = gu_h.reshape(m, f // 32, 64)[..., :32].reshape(m, f)
    u_h = gu_h.reshape(m, f // 32, 64)[..., 32:].reshape(m, f)
    close(s.download_bf16((m, f)), g_h / (1 + np.exp(-g_h)) * u_h, 1e-2, "swiglu")
    # backward: ds = dy Wd^T, then through SwiGLU, written interleaved
    n_out = 128
    dy, wd = rnd(rng, m, n_out), rnd(rng, f, n_out, scale=0.2)
    ddy, dwd, dgu = dev_bf16(dy), dev_bf16(wd), rt.DeviceBuffer(m * 2 * f * 2)
    rt.gemm(ddy.ptr, dwd.ptr, dgu.ptr, m, f, n_out, n_out, n_out, 2 * f, 0, 0, rt.EPI_DSWIGLU,
            aux=gu.ptr, ldaux=2 * f, tile=tile)
    rt.sync()
    ds = L.bf16_round(dy @ wd.T)
    sg = 1 / (1 + np.exp(-g_h))
    want = interleave32(ds * u_h * sg * (1 + g_h * (1 - sg)), ds * g_h * sg)
    close(dgu.download_bf16((m, 2 * f)), want, 1e-2, "dgate/dup")


def test_mfma_rate_diagnostic():
    """The measurement aid runs and lands between a tenth of and just above the published peak."""
    for shape in (16, 32):
        for rnd in (False, True):
            t = rt.mfma_rate(shape, rnd, iters=4000)
            assert 250.0 < t < 2600.0, (shape, rnd, t)
    with pytest.raises(rt.JppError, match="shape is 16"):
        rt.mfma_rate(8, False)


def test_split_contraction():
    """A contraction split over workgroups: JPP_GROUP_K with an f32 epilogue leaves one partial
    product per token range, jpp_sum_accum_f32 adds them to the accumulator in order."""
    rng = np.random.default_rng(31)
    m, n, T, parts = 256, 384, 2048, 4
    x, dy = rnd(rng, T, m), rnd(rng, T, n)
    acc0 = rng.standard_normal((m, n)).astype(np.float32)
    seg = np.arange(parts + 1, dtype=np.int32) * (T // parts)
    b_x, b_dy, b_seg = dev_bf16(x), dev_bf16(dy), rt.DeviceBuffer.from_numpy(seg)
    ws, b_acc = rt.DeviceBuffer(parts * m * n * 4), rt.DeviceBuffer.from_numpy(acc0)
    rt.gemm(b_x.ptr, b_dy.ptr, ws.ptr, m, n, 0, m, n, n, 1, 1, rt.EPI_F32, tile=1, seg=b_seg.ptr,
            n_seg=parts, group_mode=2, stride_c=m * n)
    rt.check(rt.load().jpp_sum_accum_f32(None, b_acc.ptr, ws.ptr, parts, m * n))
    rt.sync()
    part_h = ws.download(np.float32, (parts, m, n))
    for k in range(parts):
        rows = slice(seg[k], seg[k + 1])
        close(part_h[k], x[rows].T @ dy[rows], 1e-4 * math.sqrt(T // parts), f"part {k}")
    got = b_acc.download(np.float32, (m, n))
    # the sum is taken in the order of the parts, exactly
    want = part_h[0].copy()
    for k in range(1, parts):
        want += part_h[k]
    np.testing.assert_array_equal(got, acc0 + want)
    with pytest.raises(rt.JppError, match="multiple of 4"):
        rt.check(rt.load().jpp_sum_accum_f32(None, b_acc.ptr, ws.ptr, parts, 6))
