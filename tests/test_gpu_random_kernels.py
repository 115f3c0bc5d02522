"""Seeded random shapes through the operator seam (GEMM with every epilogue and tile choice,
several operand pairs, attention with grouped heads, norms) against numpy / the oracle.  The
fixed cases of test_gpu_kernels.py name the shapes that matter; this sweep is for the ones
nobody thought of (odd tile counts, splits of the last round along either side, leading
dimensions larger than the row)."""
import ctypes as C
import math

import os

import numpy as np
import pytest

import parity
import test_gpu_kernels as K

from jaxpp_amd import runtime as rt
from oracle import layers as L

pytestmark = pytest.mark.gpu

# further draws on demand: JPP_SWEEP_OFFSET=100000 python -m pytest <this file> (the committed runs use 0)
SWEEP_OFFSET = int(os.environ.get("JPP_SWEEP_OFFSET", "0"))


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    rt.require_gpu()


def pad_cols(a, ld):
    """`a` in a buffer whose rows are `ld` long (the padding holds junk that must not be read
    as data nor written)."""
    out = np.full((a.shape[0], ld), 7.0, np.float32)
    out[:, :a.shape[1]] = a
    return out


@pytest.mark.parametrize("seed", range(48))
def test_random_gemm(seed):
    rng = np.random.default_rng(3000 + SWEEP_OFFSET + seed)
    ta, tb, epi = K.GEMM_CASES[rng.integers(len(K.GEMM_CASES))]
    big = rng.integers(4) == 0                     # now and then: several rounds of 256x256 tiles
    m = int(rng.integers(1, 33 if big else 9)) * 128
    n = int(rng.integers(1, 33 if big else 9)) * 128
    k = int(rng.integers(1, 5 if big else 9)) * 64
    tile = int(rng.integers(0, 5))
    parts = int(rng.integers(1, 5)) if (ta, tb, epi) == (1, 1, rt.EPI_ACC_F32) and rng.integers(2) else 1
    if parts > 1:
        tile = 4 if (m % 256 == 0 and n % 256 == 0) else 3 if n % 256 == 0 else -1
        if tile < 0:
            parts = 1
            tile = 0
    pad_a, pad_b, pad_c = (int(rng.integers(0, 3)) * 8 for _ in range(3))
    print(f"seed {seed}: ta={ta} tb={tb} epi={epi} tile={tile} {m}x{n}x{k} parts={parts} "
          f"pads {pad_a},{pad_b},{pad_c}", flush=True)
    As = [K.rnd(rng, m, k) for _ in range(parts)]
    Bs = [K.rnd(rng, n, k, scale=0.3) for _ in range(parts)]
    want = sum(a.astype(np.float64) @ b.astype(np.float64).T for a, b in zip(As, Bs)).astype(np.float32)
    a_h = [a.T.copy() if ta else a for a in As]
    b_h = [b.T.copy() if tb else b for b in Bs]
    lda, ldb, ldc = a_h[0].shape[1] + pad_a, b_h[0].shape[1] + pad_b, n + pad_c
    dA = [K.dev_bf16(pad_cols(a, lda)) for a in a_h]
    dB = [K.dev_bf16(pad_cols(b, ldb)) for b in b_h]
    kw, keep = {}, []
    if epi in (rt.EPI_BF16, rt.EPI_GELU) and rng.integers(2):
        bias = K.rnd(rng, n)
        keep.append(K.dev_bf16(bias))
        kw["bias"] = keep[-1].ptr
        want = want + bias
    if epi == rt.EPI_BF16 and rng.integers(2):
        resid = K.rnd(rng, m, n)
        keep.append(K.dev_bf16(resid))
        kw.update(resid=keep[-1].ptr, ldresid=n)
        want = want + resid
    if epi == rt.EPI_DGELU:
        aux = K.rnd(rng, m, n)
        keep.append(K.dev_bf16(aux))
        kw.update(aux=keep[-1].ptr, ldaux=n)
        want = want * L.gelu_grad(aux.astype(np.float64)).astype(np.float32)
    f32_out = epi in (rt.EPI_ACC_F32, rt.EPI_F32)
    prev = rng.standard_normal((m, ldc)).astype(np.float32)
    if f32_out:
        dc = rt.DeviceBuffer.from_numpy(prev)
        if epi == rt.EPI_ACC_F32:
            want = want + prev[:, :n]
    else:
        dc = K.dev_bf16(prev)
    if epi == rt.EPI_GELU:
        dc2 = rt.DeviceBuffer(m * n * 2)
        kw.update(c2=dc2.ptr, ldc2=n)
    rt.gemm(dA[0].ptr, dB[0].ptr, dc.ptr, m, n, k, lda, ldb, ldc, ta, tb, epi, tile=tile,
            more=[(a.ptr, b.ptr) for a, b in zip(dA[1:], dB[1:])], **kw)
    rt.sync()
    got = dc.download(np.float32, (m, ldc)) if f32_out else dc.download_bf16((m, ldc))
    if pad_c:   # the padding of C is not the kernel's to write
        np.testing.assert_array_equal(got[:, n:], prev[:, n:] if f32_out else L.bf16_round(prev[:, n:]))
    if f32_out:
        K.close(got[:, :n], want, 1e-4 * math.sqrt(k * parts), "gemm f32")
    else:
        K.close(got[:, :n], want, 1e-2, "gemm bf16")
    if epi == rt.EPI_GELU:
        K.close(dc2.download_bf16((m, n)), L.gelu(want.astype(np.float64)).astype(np.float32), 1e-2,
                "gemm gelu")


@pytest.mark.parametrize("seed", range(24))
def test_random_attention(seed):
    rng = np.random.default_rng(4000 + SWEEP_OFFSET + seed)
    d = int(rng.choice([64, 128]))
    hkv = int(rng.integers(1, 4))
    hq = hkv * int(rng.choice([1, 2, 4]))
    batch = int(rng.integers(1, 3))
    seq = int(rng.integers(1, 7)) * 128
    causal = int(rng.integers(2))
    print(f"seed {seed}: d={d} heads {hq}/{hkv} batch={batch} seq={seq} causal={causal}", flush=True)
    K.test_attention_fwd_bwd(d, bool(causal), hq, hkv, batch, seq)


@pytest.mark.parametrize("seed", range(24))
def test_random_norm(seed):
    rng = np.random.default_rng(5000 + SWEEP_OFFSET + seed)
    ln = bool(rng.integers(2))
    rows = int(rng.integers(1, 1500))
    cols = int(rng.integers(16, 1025)) * 8
    K.test_norm_fwd_bwd(ln, rows, cols)


@pytest.mark.parametrize("seed", range(16))
def test_random_moe(seed):
    rng = np.random.default_rng(6000 + SWEEP_OFFSET + seed)
    T = int(rng.integers(1, 3000))                 # any count: groups are padded to 256 rows
    h = int(rng.integers(2, 65)) * 8
    print(f"seed {seed}: {T} tokens of width {h}", flush=True)
    K.check_moe(seed, T, h)
