// Fused attention for gfx950: forward with online softmax, and a two-kernel
// deterministic backward (dQ per query block, dK/dV per key block; no atomics).
//
// Everything runs on v_mfma_f32_32x32x16_bf16.  Scores are computed transposed
// where that lets the probabilities feed the next MFMA straight from the
// accumulator registers:
//
//   forward / dQ kernel (contraction of the second GEMM runs over keys):
//     S^T[key,q] = K Q^T            A = K   (LDS),  B = Q  (registers)
//     O^T[dv,q] += V^T P^T          A = V^T (LDS),  B = P^T from S^T registers
//   dK/dV kernel (contraction of the second GEMM runs over queries):
//     S[q,key]   = Q K^T            A = Q   (LDS),  B = K  (registers)
//     dV^T[dv,key] += dO^T P        A = dO^T(LDS),  B = P from S registers
//
// An accumulator tile enumerates its row index as (reg/4, lane/32, reg%4); the
// LDS-side operand of the second GEMM is stored with bits 2 and 3 of the
// contraction index swapped (TileLoader KPERM) so that 8 consecutive
// accumulator registers form one 16-element MFMA step.
#include <math.h>

#include "common.h"

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct AttnParams {
  const bf16_t* q; const bf16_t* k; const bf16_t* v;
  bf16_t* o; float* lse;
  const bf16_t* d_o;
  bf16_t* dq; bf16_t* dk; bf16_t* dv;
  float* delta;
  long ldq, ldk, ldv, ldo, lddo, lddq, lddk, lddv;
  int batch, seq, n_heads, n_kv_heads;
  float scale;
};

// 8 consecutive accumulator registers -> one bf16 MFMA operand
__device__ __forceinline__ bf16x8 acc_to_frag(const f32x16& a, int base) {
  bf16x8 f;
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = (__bf16)a[base + e];
  return f;
}

// row-major operand fragment straight from HBM (lane: row = lane&31, 8
// contraction elements of step ks)
__device__ __forceinline__ bf16x8 global_frag(const bf16_t* base, long ld, int ks, int lane) {
  return *(const bf16x8*)(base + (long)(lane & 31) * ld + ks * 16 + (lane >> 5) * 8);
}

template <int D>
__device__ __forceinline__ bf16x8 slabs_frag(const uint8_t* slabs, int rows_per_slab, int row0,
                                             int ks, int lane) {
  // a [rows][D] operand is held as D/64 slabs of [rows][64]
  return slab_frag(slabs + (ks >> 2) * rows_per_slab * 128, row0, ks & 3, lane);
}

// ---------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------
template <int D, bool CAUSAL>
__global__ __launch_bounds__(256) void attn_fwd_kernel(AttnParams p) {
  constexpr int KS = D / 16;  // MFMA steps over the head dimension
  constexpr int DT = D / 32;  // output tiles over the head dimension
  constexpr int NSLAB = D / 64;
  __shared__ __align__(16) uint8_t lds_k[NSLAB * 64 * 128];
  __shared__ __align__(16) uint8_t lds_vt[D * 128];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int qb = CAUSAL ? (gridDim.x - 1 - blockIdx.x) : blockIdx.x;  // heavy blocks first
  const int h = blockIdx.y, b = blockIdx.z;
  const int hk = h / (p.n_heads / p.n_kv_heads);
  const long row0 = (long)b * p.seq;
  const int q0 = qb * 128 + wave * 32;
  const int qi = q0 + (lane & 31);  // this lane's query position

  bf16x8 qf[KS];
  {
    const bf16_t* qbase = p.q + (row0 + q0) * p.ldq + h * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = global_frag(qbase, p.ldq, ks, lane);
  }

  f32x16 oacc[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float sc = p.scale * kLog2e;

  using LK = TileLoader<64, false>;
  using LV = TileLoader<D, true, true>;
  typename LK::Regs rk[NSLAB];
  typename LV::Regs rv;
  const bf16_t* kbase = p.k + row0 * p.ldk + hk * D;
  const bf16_t* vbase = p.v + row0 * p.ldv + hk * D;
  const int nblk = CAUSAL ? (qb * 128 + 128) / 64 : p.seq / 64;

#pragma unroll
  for (int c = 0; c < NSLAB; ++c) LK::load(rk[c], kbase + c * 64, p.ldk, tid);
  LV::load(rv, vbase, p.ldv, tid);

  for (int blk = 0; blk < nblk; ++blk) {
    const int k0 = blk * 64;
    if (blk) __syncthreads();
#pragma unroll
    for (int c = 0; c < NSLAB; ++c) LK::store(rk[c], lds_k + c * 64 * 128, tid);
    LV::store(rv, lds_vt, tid);
    __syncthreads();
    {
      const int kn = min(blk + 1, nblk - 1) * 64;
#pragma unroll
      for (int c = 0; c < NSLAB; ++c) LK::load(rk[c], kbase + (long)kn * p.ldk + c * 64, p.ldk, tid);
      LV::load(rv, vbase + (long)kn * p.ldv, p.ldv, tid);
    }
    if (CAUSAL && k0 > q0 + 31) continue;  // whole block above this wave's diagonal

    f32x16 s[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[t][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        s[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(slabs_frag<D>(lds_k, 64, t * 32, ks, lane),
                                                       qf[ks], s[t], 0, 0, 0);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float v = s[t][r] * sc;
        if (CAUSAL) {
          const int key = k0 + t * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
          if (key > qi) v = -INFINITY;
        }
        s[t][r] = v;
        mx = fmaxf(mx, v);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = exp2f(m_run - m_new);
    m_run = m_new;
    float rs = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float e = exp2f(s[t][r] - m_new);
        s[t][r] = e;
        rs += e;
      }
    l_run = l_run * alpha + rs;
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      const bf16x8 pf = acc_to_frag(s[st >> 1], (st & 1) * 8);
#pragma unroll
      for (int i = 0; i < DT; ++i)
        oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(slab_frag(lds_vt, i * 32, st, lane), pf,
                                                          oacc[i], 0, 0, 0);
    }
  }

  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.0f / l_tot;
  bf16_t* orow = p.o + (row0 + qi) * p.ldo + h * D;
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int dv = i * 32 + g * 8 + (lane >> 5) * 4;
      *(uint2*)(orow + dv) =
          make_uint2(pack_bf16x2(oacc[i][4 * g] * inv, oacc[i][4 * g + 1] * inv),
                     pack_bf16x2(oacc[i][4 * g + 2] * inv, oacc[i][4 * g + 3] * inv));
    }
  if (lane < 32) p.lse[((long)b * p.n_heads + h) * p.seq + qi] = m_run * kLn2 + logf(l_tot);
}

// ---------------------------------------------------------------------------
// backward, step 0: delta[b,h,q] = sum_d dO * O
// ---------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void attn_delta_kernel(AttnParams p) {
  constexpr int LPH = D / 8;  // lanes per head
  const long item = (long)blockIdx.x * 256 + threadIdx.x;
  const long total = (long)p.batch * p.seq * p.n_heads * LPH;
  float s = 0.f;
  long row = 0;
  int h = 0;
  if (item < total) {
    const int c = (int)(item % LPH);
    const long rh = item / LPH;
    h = (int)(rh % p.n_heads);
    row = rh / p.n_heads;
    const uint4 a = *(const uint4*)(p.o + row * p.ldo + h * D + c * 8);
    const uint4 g = *(const uint4*)(p.d_o + row * p.lddo + h * D + c * 8);
    s = bf16lo_to_f32(a.x) * bf16lo_to_f32(g.x) + bf16hi_to_f32(a.x) * bf16hi_to_f32(g.x) +
        bf16lo_to_f32(a.y) * bf16lo_to_f32(g.y) + bf16hi_to_f32(a.y) * bf16hi_to_f32(g.y) +
        bf16lo_to_f32(a.z) * bf16lo_to_f32(g.z) + bf16hi_to_f32(a.z) * bf16hi_to_f32(g.z) +
        bf16lo_to_f32(a.w) * bf16lo_to_f32(g.w) + bf16hi_to_f32(a.w) * bf16hi_to_f32(g.w);
  }
#pragma unroll
  for (int o = LPH / 2; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if (item < total && (item % LPH) == 0) {
    const long b = row / p.seq, qpos = row % p.seq;
    p.delta[(b * p.n_heads + h) * p.seq + qpos] = s;
  }
}

// ---------------------------------------------------------------------------
// backward, dQ: one workgroup per 128 queries of one head
// ---------------------------------------------------------------------------
template <int D, bool CAUSAL>
__global__ __launch_bounds__(256) void attn_bwd_dq_kernel(AttnParams p) {
  constexpr int KS = D / 16, DT = D / 32, NSLAB = D / 64;
  __shared__ __align__(16) uint8_t lds_k[NSLAB * 64 * 128];
  __shared__ __align__(16) uint8_t lds_v[NSLAB * 64 * 128];
  __shared__ __align__(16) uint8_t lds_kt[D * 128];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int qb = CAUSAL ? (gridDim.x - 1 - blockIdx.x) : blockIdx.x;
  const int h = blockIdx.y, b = blockIdx.z;
  const int hk = h / (p.n_heads / p.n_kv_heads);
  const long row0 = (long)b * p.seq;
  const int q0 = qb * 128 + wave * 32;
  const int qi = q0 + (lane & 31);

  bf16x8 qf[KS], dof[KS];
  {
    const bf16_t* qbase = p.q + (row0 + q0) * p.ldq + h * D;
    const bf16_t* dobase = p.d_o + (row0 + q0) * p.lddo + h * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = global_frag(qbase, p.ldq, ks, lane);
      dof[ks] = global_frag(dobase, p.lddo, ks, lane);
    }
  }
  const long stat = ((long)b * p.n_heads + h) * p.seq + qi;
  const float lse2 = p.lse[stat] * kLog2e;
  const float dlt = p.delta[stat];
  const float sc = p.scale * kLog2e;

  f32x16 dqacc[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) dqacc[i][r] = 0.f;

  using LK = TileLoader<64, false>;
  using LT = TileLoader<D, true, true>;
  typename LK::Regs rk[NSLAB], rv[NSLAB];
  typename LT::Regs rkt;
  const bf16_t* kbase = p.k + row0 * p.ldk + hk * D;
  const bf16_t* vbase = p.v + row0 * p.ldv + hk * D;
  const int nblk = CAUSAL ? (qb * 128 + 128) / 64 : p.seq / 64;

#pragma unroll
  for (int c = 0; c < NSLAB; ++c) {
    LK::load(rk[c], kbase + c * 64, p.ldk, tid);
    LK::load(rv[c], vbase + c * 64, p.ldv, tid);
  }
  LT::load(rkt, kbase, p.ldk, tid);

  for (int blk = 0; blk < nblk; ++blk) {
    const int k0 = blk * 64;
    if (blk) __syncthreads();
#pragma unroll
    for (int c = 0; c < NSLAB; ++c) {
      LK::store(rk[c], lds_k + c * 64 * 128, tid);
      LK::store(rv[c], lds_v + c * 64 * 128, tid);
    }
    LT::store(rkt, lds_kt, tid);
    __syncthreads();
    {
      const long kn = (long)min(blk + 1, nblk - 1) * 64;
#pragma unroll
      for (int c = 0; c < NSLAB; ++c) {
        LK::load(rk[c], kbase + kn * p.ldk + c * 64, p.ldk, tid);
        LK::load(rv[c], vbase + kn * p.ldv + c * 64, p.ldv, tid);
      }
      LT::load(rkt, kbase + kn * p.ldk, p.ldk, tid);
    }
    if (CAUSAL && k0 > q0 + 31) continue;

    f32x16 s[2], dp[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int r = 0; r < 16; ++r) { s[t][r] = 0.f; dp[t][r] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        s[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(slabs_frag<D>(lds_k, 64, t * 32, ks, lane),
                                                       qf[ks], s[t], 0, 0, 0);
        dp[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(slabs_frag<D>(lds_v, 64, t * 32, ks, lane),
                                                        dof[ks], dp[t], 0, 0, 0);
      }
    }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float pr = exp2f(s[t][r] * sc - lse2);
        if (CAUSAL) {
          const int key = k0 + t * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
          if (key > qi) pr = 0.f;
        }
        s[t][r] = pr * (dp[t][r] - dlt) * p.scale;
      }
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      const bf16x8 dsf = acc_to_frag(s[st >> 1], (st & 1) * 8);
#pragma unroll
      for (int i = 0; i < DT; ++i)
        dqacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(slab_frag(lds_kt, i * 32, st, lane), dsf,
                                                           dqacc[i], 0, 0, 0);
    }
  }

  bf16_t* drow = p.dq + (row0 + qi) * p.lddq + h * D;
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = i * 32 + g * 8 + (lane >> 5) * 4;
      *(uint2*)(drow + d) = make_uint2(pack_bf16x2(dqacc[i][4 * g], dqacc[i][4 * g + 1]),
                                       pack_bf16x2(dqacc[i][4 * g + 2], dqacc[i][4 * g + 3]));
    }
}

// ---------------------------------------------------------------------------
// backward, dK and dV: one workgroup per 128 keys of one kv head; loops over
// the query heads that share it and over 64-query blocks
// ---------------------------------------------------------------------------
template <int D, bool CAUSAL>
__global__ __launch_bounds__(256) void attn_bwd_dkv_kernel(AttnParams p) {
  constexpr int KS = D / 16, DT = D / 32, NSLAB = D / 64;
  extern __shared__ __align__(16) uint8_t dkv_smem[];  // 4 * D * 128 + 512 bytes
  uint8_t* lds_q = dkv_smem;
  uint8_t* lds_do = lds_q + D * 128;
  uint8_t* lds_qt = lds_do + D * 128;
  uint8_t* lds_dot = lds_qt + D * 128;
  float* lds_lse = (float*)(lds_dot + D * 128);
  float* lds_delta = lds_lse + 64;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int kb = blockIdx.x, hk = blockIdx.y, b = blockIdx.z;
  const int grp = p.n_heads / p.n_kv_heads;
  const long row0 = (long)b * p.seq;
  const int k0 = kb * 128 + wave * 32;
  const int ki = k0 + (lane & 31);

  bf16x8 kf[KS], vf[KS];
  {
    const bf16_t* kbase = p.k + (row0 + k0) * p.ldk + hk * D;
    const bf16_t* vbase = p.v + (row0 + k0) * p.ldv + hk * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kf[ks] = global_frag(kbase, p.ldk, ks, lane);
      vf[ks] = global_frag(vbase, p.ldv, ks, lane);
    }
  }
  f32x16 dkacc[DT], dvacc[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dkacc[i][r] = 0.f; dvacc[i][r] = 0.f; }
  const float sc = p.scale * kLog2e;

  using LR = TileLoader<64, false>;
  using LT = TileLoader<D, true, true>;
  typename LR::Regs rq[NSLAB], rdo[NSLAB];
  typename LT::Regs rqt, rdot;
  float rstat = 0.f;

  const int qblk0 = CAUSAL ? (kb * 128) / 64 : 0;
  const int nqb = p.seq / 64 - qblk0;
  const int iters = grp * nqb;

  auto fetch = [&](int it) {
    const int hh = hk * grp + it / nqb;
    const long q0 = (long)(qblk0 + it % nqb) * 64;
    const bf16_t* qsrc = p.q + (row0 + q0) * p.ldq + hh * D;
    const bf16_t* dsrc = p.d_o + (row0 + q0) * p.lddo + hh * D;
#pragma unroll
    for (int c = 0; c < NSLAB; ++c) {
      LR::load(rq[c], qsrc + c * 64, p.ldq, tid);
      LR::load(rdo[c], dsrc + c * 64, p.lddo, tid);
    }
    LT::load(rqt, qsrc, p.ldq, tid);
    LT::load(rdot, dsrc, p.lddo, tid);
    const long stat = ((long)b * p.n_heads + hh) * p.seq + q0;
    if (tid < 64) rstat = p.lse[stat + tid] * kLog2e;
    else if (tid < 128) rstat = p.delta[stat + tid - 64];
  };

  fetch(0);
  for (int it = 0; it < iters; ++it) {
    const int q0 = (qblk0 + it % nqb) * 64;
    if (it) __syncthreads();
#pragma unroll
    for (int c = 0; c < NSLAB; ++c) {
      LR::store(rq[c], lds_q + c * 64 * 128, tid);
      LR::store(rdo[c], lds_do + c * 64 * 128, tid);
    }
    LT::store(rqt, lds_qt, tid);
    LT::store(rdot, lds_dot, tid);
    if (tid < 64) lds_lse[tid] = rstat;
    else if (tid < 128) lds_delta[tid - 64] = rstat;
    __syncthreads();
    fetch(min(it + 1, iters - 1));
    if (CAUSAL && q0 + 63 < k0) continue;  // every query of the block precedes this wave's keys

    f32x16 s[2], dp[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int r = 0; r < 16; ++r) { s[t][r] = 0.f; dp[t][r] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        s[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(slabs_frag<D>(lds_q, 64, t * 32, ks, lane),
                                                       kf[ks], s[t], 0, 0, 0);
        dp[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(slabs_frag<D>(lds_do, 64, t * 32, ks, lane),
                                                        vf[ks], dp[t], 0, 0, 0);
      }
    }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int ql = t * 32 + g * 8 + (lane >> 5) * 4;
        const float4 l4 = *(const float4*)(lds_lse + ql);
        const float4 d4 = *(const float4*)(lds_delta + ql);
        const float ls[4] = {l4.x, l4.y, l4.z, l4.w};
        const float dl[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = 4 * g + e;
          float pr = exp2f(s[t][r] * sc - ls[e]);
          if (CAUSAL && ki > q0 + ql + e) pr = 0.f;
          s[t][r] = pr;
          dp[t][r] = pr * (dp[t][r] - dl[e]) * p.scale;
        }
      }
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      const bf16x8 pf = acc_to_frag(s[st >> 1], (st & 1) * 8);
      const bf16x8 dsf = acc_to_frag(dp[st >> 1], (st & 1) * 8);
#pragma unroll
      for (int i = 0; i < DT; ++i) {
        dvacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(slab_frag(lds_dot, i * 32, st, lane), pf,
                                                           dvacc[i], 0, 0, 0);
        dkacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(slab_frag(lds_qt, i * 32, st, lane), dsf,
                                                           dkacc[i], 0, 0, 0);
      }
    }
  }

  bf16_t* dkrow = p.dk + (row0 + ki) * p.lddk + hk * D;
  bf16_t* dvrow = p.dv + (row0 + ki) * p.lddv + hk * D;
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = i * 32 + g * 8 + (lane >> 5) * 4;
      *(uint2*)(dkrow + d) = make_uint2(pack_bf16x2(dkacc[i][4 * g], dkacc[i][4 * g + 1]),
                                        pack_bf16x2(dkacc[i][4 * g + 2], dkacc[i][4 * g + 3]));
      *(uint2*)(dvrow + d) = make_uint2(pack_bf16x2(dvacc[i][4 * g], dvacc[i][4 * g + 1]),
                                        pack_bf16x2(dvacc[i][4 * g + 2], dvacc[i][4 * g + 3]));
    }
}

int check_common(const jpp_attn_args* a, const char* who) {
  JPP_REQUIRE(a && a->q && a->k && a->v && a->o && a->lse, "%s: null operand", who);
  JPP_REQUIRE(a->head_dim == 64 || a->head_dim == 128, "%s: head_dim must be 64 or 128, got %d",
              who, a->head_dim);
  JPP_REQUIRE(a->batch > 0 && a->seq > 0 && a->seq % 128 == 0,
              "%s: seq must be a positive multiple of 128, got %d", who, a->seq);
  JPP_REQUIRE(a->n_heads > 0 && a->n_kv_heads > 0 && a->n_heads % a->n_kv_heads == 0,
              "%s: n_heads %d not a multiple of n_kv_heads %d", who, a->n_heads, a->n_kv_heads);
  JPP_REQUIRE(a->ldq >= (int64_t)a->n_heads * a->head_dim &&
                  a->ldk >= (int64_t)a->n_kv_heads * a->head_dim &&
                  a->ldv >= (int64_t)a->n_kv_heads * a->head_dim &&
                  a->ldo >= (int64_t)a->n_heads * a->head_dim,
              "%s: leading dimension too small", who);
  JPP_REQUIRE((a->ldq | a->ldk | a->ldv | a->ldo) % 8 == 0 &&
                  ((uintptr_t)a->q | (uintptr_t)a->k | (uintptr_t)a->v | (uintptr_t)a->o) % 16 == 0,
              "%s: operands must keep 16-byte alignment", who);
  return JPP_OK;
}

AttnParams make_params(const jpp_attn_args* a) {
  AttnParams p;
  p.q = (const bf16_t*)a->q; p.k = (const bf16_t*)a->k; p.v = (const bf16_t*)a->v;
  p.o = (bf16_t*)a->o; p.lse = a->lse; p.d_o = (const bf16_t*)a->d_o;
  p.dq = (bf16_t*)a->dq; p.dk = (bf16_t*)a->dk; p.dv = (bf16_t*)a->dv; p.delta = a->delta;
  p.ldq = a->ldq; p.ldk = a->ldk; p.ldv = a->ldv; p.ldo = a->ldo;
  p.lddo = a->lddo; p.lddq = a->lddq; p.lddk = a->lddk; p.lddv = a->lddv;
  p.batch = a->batch; p.seq = a->seq; p.n_heads = a->n_heads; p.n_kv_heads = a->n_kv_heads;
  p.scale = 1.0f / sqrtf((float)a->head_dim);
  return p;
}

}  // namespace

extern "C" int jpp_attn_fwd(void* stream, const jpp_attn_args* a) {
  if (int rc = check_common(a, "attn_fwd")) return rc;
  AttnParams p = make_params(a);
  dim3 grid(a->seq / 128, a->n_heads, a->batch);
  hipStream_t st = (hipStream_t)stream;
  const double fl = 4.0 * a->batch * a->seq * (double)a->seq * a->n_heads * a->head_dim *
                    (a->causal ? 0.5 : 1.0);
  ProbeScope probe(st, "attn_fwd", fl, 0);
#define JPP_AF(D_, C_) hipLaunchKernelGGL((attn_fwd_kernel<D_, C_>), grid, dim3(256), 0, st, p)
  if (a->head_dim == 64) { if (a->causal) JPP_AF(64, true); else JPP_AF(64, false); }
  else { if (a->causal) JPP_AF(128, true); else JPP_AF(128, false); }
#undef JPP_AF
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

extern "C" int jpp_attn_bwd(void* stream, const jpp_attn_args* a) {
  if (int rc = check_common(a, "attn_bwd")) return rc;
  JPP_REQUIRE(a->d_o && a->dq && a->dk && a->dv && a->delta, "attn_bwd: null operand");
  JPP_REQUIRE(a->lddo >= (int64_t)a->n_heads * a->head_dim &&
                  a->lddq >= (int64_t)a->n_heads * a->head_dim &&
                  a->lddk >= (int64_t)a->n_kv_heads * a->head_dim &&
                  a->lddv >= (int64_t)a->n_kv_heads * a->head_dim,
              "attn_bwd: leading dimension too small");
  JPP_REQUIRE((a->lddo | a->lddq | a->lddk | a->lddv) % 8 == 0 &&
                  ((uintptr_t)a->d_o | (uintptr_t)a->dq | (uintptr_t)a->dk | (uintptr_t)a->dv) % 16 == 0,
              "attn_bwd: operands must keep 16-byte alignment");
  AttnParams p = make_params(a);
  hipStream_t st = (hipStream_t)stream;
  const long items = (long)a->batch * a->seq * a->n_heads * (a->head_dim / 8);
  dim3 gdelta((unsigned)((items + 255) / 256));
  dim3 gq(a->seq / 128, a->n_heads, a->batch);
  dim3 gkv(a->seq / 128, a->n_kv_heads, a->batch);
  const double fl = 8.0 * a->batch * a->seq * (double)a->seq * a->n_heads * a->head_dim *
                    (a->causal ? 0.5 : 1.0);
#define JPP_AB(D_, C_)                                                             \
  do {                                                                             \
    hipLaunchKernelGGL((attn_delta_kernel<D_>), gdelta, dim3(256), 0, st, p);      \
    {                                                                              \
      ProbeScope probe(st, "attn_bwd_dq", fl * 0.4, 0);                            \
      hipLaunchKernelGGL((attn_bwd_dq_kernel<D_, C_>), gq, dim3(256), 0, st, p);   \
    }                                                                              \
    ProbeScope probe(st, "attn_bwd_dkv", fl * 0.6, 0);                             \
    JPP_CHECK_HIP(hipFuncSetAttribute((const void*)attn_bwd_dkv_kernel<D_, C_>,    \
                                      hipFuncAttributeMaxDynamicSharedMemorySize,  \
                                      4 * D_ * 128 + 512));                        \
    hipLaunchKernelGGL((attn_bwd_dkv_kernel<D_, C_>), gkv, dim3(256),              \
                       4 * D_ * 128 + 512, st, p);                                 \
  } while (0)
  if (a->head_dim == 64) { if (a->causal) JPP_AB(64, true); else JPP_AB(64, false); }
  else { if (a->causal) JPP_AB(128, true); else JPP_AB(128, false); }
#undef JPP_AB
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}
