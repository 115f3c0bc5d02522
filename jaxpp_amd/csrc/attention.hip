// Fused attention for gfx950: forward with online softmax, and a two-kernel
// deterministic backward (dQ per query block, attention_dq.hip; dK/dV per key block, here
// without a mask and in attention_dkv.hip under one; no atomics).
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
// LDS-side operand of the second GEMM is read in the same order (slab_frag_tr), so
// that 8 consecutive accumulator registers form one 16-element MFMA step.
#include "attention_common.h"

using namespace jpp_attn;

namespace {

// ---------------------------------------------------------------------------
// forward: one workgroup per 128 queries of one head, 32 queries per wave;
// K/V blocks of 64 keys double-buffered in LDS
// ---------------------------------------------------------------------------
template <int D, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void attn_fwd_kernel(AttnParams p) {
  constexpr int KS = D / 16;  // MFMA steps over the head dimension
  constexpr int DT = D / 32;  // output tiles over the head dimension
  constexpr int TILE = D * 128;  // bytes of a [64][D] tile
  constexpr int STAGE = 2 * TILE;
  extern __shared__ __align__(1024) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: scalar branches and addresses
  const Work w = xcd_work();
  const int qb = CAUSAL ? (gridDim.x - 1 - w.x) : w.x;  // heavy blocks first
  const int h = w.h, b = w.b;
  const int hk = h / (p.n_heads / p.n_kv_heads);
  const long row0 = (long)b * p.seq;
  const int q0 = qb * 128 + wave * 32;
  const int qi = q0 + (lane & 31);  // this lane's query position

  f32x16 oacc[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;  // running max of the raw scores, running sum
  const float sc = p.scale * kLog2e;

  const bf16_t* kbase = p.k + row0 * p.ldk + hk * D;
  const bf16_t* vbase = p.v + row0 * p.ldv + hk * D;
  const int nblk = CAUSAL ? (qb * 128 + 128) / 64 : p.seq / 64;
  Tile64::Offsets offk, offv;
  Tile64::offsets(offk, p.ldk, wave, lane);
  Tile64::offsets(offv, p.ldv, wave, lane);
  const uint32_t lds0 = lds_address(smem);

  // The workgroup's 128 rows of Q come through LDS like the K / V tiles (two tiles, in the
  // stage the loop fills second): a fragment taken from HBM directly touches 32 rows with 32
  // bytes each, and the CU's path to memory takes such a load line by line.
  bf16x8 qf[KS];
  {
    Tile64::Offsets offq;
    Tile64::offsets(offq, p.ldq, wave, lane);
    const bf16_t* qbase = p.q + (row0 + (long)qb * 128) * p.ldq + h * D;
    dma_tile<D>(qbase, offq, lds0 + STAGE, wave);
    dma_tile<D>(qbase + 64 * p.ldq, offq, lds0 + STAGE + TILE, wave);
  }
  dma_tile<D>(kbase, offk, lds0, wave);
  dma_tile<D>(vbase, offv, lds0 + TILE, wave);
  dma_wait_all();
  __syncthreads();
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    qf[ks] = slabs_frag<D>(smem + STAGE + (wave >> 1) * TILE, (wave & 1) * 32, ks, lane);
  settle(qf);
  __syncthreads();  // the stage is block 1's from the first trip on

  for (int blk = 0; blk < nblk; ++blk) {
    const int k0 = blk * 64;
    const uint8_t* lds_k = smem + (blk & 1) * STAGE;
    const uint8_t* lds_v = lds_k + TILE;
    {
      const long kn = (long)min(blk + 1, nblk - 1) * 64;
      const uint32_t dst = lds0 + ((blk + 1) & 1) * STAGE;
      dma_tile<D>(kbase + kn * p.ldk, offk, dst, wave);
      dma_tile<D>(vbase + kn * p.ldv, offv, dst + TILE, wave);
    }
    if (!(CAUSAL && k0 > q0 + 31)) {  // else: whole block above this wave's diagonal
      // Fragments are read from LDS in batches ahead of the MFMAs that consume them, so
      // the MFMAs wait for the oldest read only (LDS returns in order), not for each one.
      f32x16 s[2];
      {
        bf16x8 kfr[2][KS];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) kfr[t][ks] = slabs_frag<D>(lds_k, t * 32, ks, lane);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
          for (int r = 0; r < 16; ++r) s[t][r] = 0.f;
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            s[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[t][ks], qf[ks], s[t], 0, 0, 0);
        }
      }
      // Wave priority: low (0) for the score MFMAs above, raised for the softmax arithmetic and
      // again for the output MFMAs, back to 0 behind them.  A CU holds two workgroups, two waves per SIMD, and the
      // vector ALU is what a block's time is made of: a wave that has its scores gets the ALU
      // ahead of one that is still multiplying, so the two fall out of step - one in the matrix
      // core while the other does its softmax - instead of taking turns instruction by
      // instruction (164 -> 156 us at the Llama-3-8B shape, 19.4 -> 18.3 at the BERT-large one;
      // raising it for the MFMAs and not the softmax: 167).
      __builtin_amdgcn_s_setprio(2);
      // V^T fragments: requested now, they arrive under the softmax arithmetic
      bf16x8 vfr[4][DT];
#pragma unroll
      for (int st = 0; st < 4; ++st)
#pragma unroll
        for (int i = 0; i < DT; ++i) vfr[st][i] = slab_frag_tr(lds_v, 64, i * 32, st, lane);
      if (CAUSAL && k0 + 63 > q0) {  // block touches the diagonal
        // the empty asm keeps this wave-uniform branch a branch (not selects on every block)
        asm volatile("" ::: "memory");
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = k0 + t * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            if (key > qi) s[t][r] = -INFINITY;
          }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[t][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      // (Moving the reference point only when a maximum has grown by a margin - keeping an older,
      // smaller reference meanwhile - saves the rescale of the 64 accumulator registers in
      // almost every block, 5 % of this kernel.  It is not done: the probabilities are rounded
      // to bf16 for the second product, and against a reference other than the row's maximum
      // they round differently from a plain softmax's, which cost a factor of 20 in elements
      // that differ from such a computation by an ulp of the output.)
      const float m_new = fmaxf(m_run, mx);
      const float neg = -m_new * sc;
      float rs = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float e = fast_exp2(fmaf(s[t][r], sc, neg));
          s[t][r] = e;
          rs += e;
        }
      if (__any(m_new != m_run)) {  // rescale only when some row's maximum moved
        const float alpha = fast_exp2((m_run - m_new) * sc);
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < DT; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
        m_run = m_new;
      }
      l_run += rs;
      __builtin_amdgcn_s_setprio(3);
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        const bf16x8 pf = acc_to_frag(s[st >> 1], (st & 1) * 8);
#pragma unroll
        for (int i = 0; i < DT; ++i)
          oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfr[st][i], pf, oacc[i], 0, 0, 0);
      }
      __builtin_amdgcn_s_setprio(0);
    }
    dma_wait_all();
    __syncthreads();
  }

  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.0f / l_tot;
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[i][r] *= inv;
  // (the K / V stages are idle: the loop ends behind a barrier)
  store_tile_by_rows<D, DT>(oacc, lds0 + wave * (32 * D * 2), p.o + (row0 + q0) * p.ldo + h * D,
                            p.ldo, lane);
  if (lane < 32)
    p.lse[((long)b * p.n_heads + h) * p.seq + qi] = m_run * p.scale + logf(l_tot);
}

// ---------------------------------------------------------------------------
// backward, dQ without a causal mask (short sequences; under a mask: attention_dq.hip):
// one workgroup per 128 queries of one head, 32 per wave, two workgroups per CU
// ---------------------------------------------------------------------------
template <int D, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void attn_bwd_dq_kernel(AttnParams p) {
  constexpr int KS = D / 16, DT = D / 32;
  constexpr int TILE = D * 128, STAGE = 2 * TILE;
  extern __shared__ __align__(1024) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: scalar branches and addresses
  const Work w = xcd_work();
  const int qb = CAUSAL ? (gridDim.x - 1 - w.x) : w.x;
  const int h = w.h, b = w.b;
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
  float lse2 = p.lse[stat] * kLog2e;
  // The row term delta = sum_d dO * O of this wave's 32 rows: a lane holds half of its row of
  // dO already (the chunks the MFMA fragment gives it) and reads the same half of O; the other
  // half is with lane ^ 32.  Written out for the dK/dV kernel, which runs behind this one, in
  // the form that kernel consumes: per 64 rows, -delta[64] and then the log-sum-exp[64] in
  // the exp2 domain.
  float dlt = 0.f;
  {
    const bf16_t* obase = p.o + (row0 + q0) * p.ldo + h * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const uint4 ov = *(const uint4*)(obase + (long)(lane & 31) * p.ldo + ks * 16 + (lane >> 5) * 8);
      float of[8], gf[8];
      unpack8(ov, of);
      unpack8(__builtin_bit_cast(uint4, dof[ks]), gf);
#pragma unroll
      for (int e = 0; e < 8; ++e) dlt = fmaf(of[e], gf[e], dlt);
    }
    dlt += __shfl_xor(dlt, 32);
    if (lane < 32) {
      float* st = p.delta + 2 * (stat & ~63L) + (stat & 63);  // (seq is a multiple of 64)
      st[0] = -dlt;
      st[64] = lse2;
    }
  }
  const float sc = p.scale * kLog2e;
  settle(qf);
  settle(dof);
  settle(lse2);
  settle(dlt);

  f32x16 dqacc[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) dqacc[i][r] = 0.f;

  const bf16_t* kbase = p.k + row0 * p.ldk + hk * D;
  const bf16_t* vbase = p.v + row0 * p.ldv + hk * D;
  const int nblk = CAUSAL ? (qb * 128 + 128) / 64 : p.seq / 64;
  Tile64::Offsets offk, offv;
  Tile64::offsets(offk, p.ldk, wave, lane);
  Tile64::offsets(offv, p.ldv, wave, lane);
  const uint32_t lds0 = lds_address(smem);

  dma_tile<D>(kbase, offk, lds0, wave);
  dma_tile<D>(vbase, offv, lds0 + TILE, wave);
  dma_wait_all();
  __syncthreads();

  for (int blk = 0; blk < nblk; ++blk) {
    const int k0 = blk * 64;
    const uint8_t* lds_k = smem + (blk & 1) * STAGE;
    const uint8_t* lds_v = lds_k + TILE;
    {
      const long kn = (long)min(blk + 1, nblk - 1) * 64;
      const uint32_t dst = lds0 + ((blk + 1) & 1) * STAGE;
      dma_tile<D>(kbase + kn * p.ldk, offk, dst, wave);
      dma_tile<D>(vbase + kn * p.ldv, offv, dst + TILE, wave);
    }
    if (!(CAUSAL && k0 > q0 + 31)) {
      const bool diag = CAUSAL && k0 + 63 > q0;
#pragma unroll
      for (int t = 0; t < 2; ++t) {  // 32 keys at a time keeps the live scores small
        f32x16 s, dp;
        {
          bf16x8 kfr[KS], vfr[KS];  // read ahead of the MFMAs that consume them
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            kfr[ks] = slabs_frag<D>(lds_k, t * 32, ks, lane);
            vfr[ks] = slabs_frag<D>(lds_v, t * 32, ks, lane);
          }
#pragma unroll
          for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[ks], qf[ks], s, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfr[ks], dof[ks], dp, 0, 0, 0);
          }
        }
        // (wave priority by phase as in the forward kernel: -3 % at the BERT-large shape)
        __builtin_amdgcn_s_setprio(2);
        bf16x8 ktr[2][DT];  // K^T fragments arrive under the elementwise arithmetic
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
          for (int i = 0; i < DT; ++i) ktr[h2][i] = slab_frag_tr(lds_k, 64, i * 32, 2 * t + h2, lane);
        if (diag) {  // wave-uniform; the empty asm keeps it a branch
          asm volatile("" ::: "memory");
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = k0 + t * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            if (key > qi) s[r] = -INFINITY;
          }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float pr = fast_exp2(fmaf(s[r], sc, -lse2));  // exp2(-inf) = 0 where masked
          s[r] = pr * (dp[r] - dlt);  // (the softmax scale is applied to dQ at the end)
        }
        __builtin_amdgcn_s_setprio(3);
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
          const bf16x8 dsf = acc_to_frag(s, h2 * 8);
#pragma unroll
          for (int i = 0; i < DT; ++i)
            dqacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktr[h2][i], dsf, dqacc[i], 0, 0, 0);
        }
        __builtin_amdgcn_s_setprio(0);
      }
    }
    dma_wait_all();
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) dqacc[i][r] *= p.scale;
  if (p.rope_cos) rope_back<D, DT>(dqacc, p.rope_cos, p.rope_sin, qi, lane);
  // (the K / V stages are idle: the loop ends behind a barrier)
  store_tile_by_rows<D, DT>(dqacc, lds0 + wave * (32 * D * 2), p.dq + (row0 + q0) * p.lddq + h * D,
                            p.lddq, lane);
}

// ---------------------------------------------------------------------------
// backward, dK and dV without a causal mask (every key block carries the same
// work): one workgroup per 128 keys of one kv head; loops over the query heads
// that share it and over 64-query blocks, the four waves sharing each Q / dO tile
// ---------------------------------------------------------------------------
template <int D, bool CAUSAL>
__global__ __launch_bounds__(256, (D > 64 ? 1 : 2)) void attn_bwd_dkv_wide_kernel(AttnParams p) {
  constexpr int KS = D / 16, DT = D / 32;
  constexpr int TILE = D * 128, STAGE = 2 * TILE + 512;
  extern __shared__ __align__(1024) uint8_t smem[];  // 2 stages: Q tile, dO tile, lse[64], delta[64]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const Work w = xcd_work();
  const int kb = w.x, hk = w.h, b = w.b;
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
  settle(kf);
  settle(vf);
  f32x16 dkacc[DT], dvacc[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dkacc[i][r] = 0.f; dvacc[i][r] = 0.f; }
  const float sc = p.scale * kLog2e;

  const int qblk0 = CAUSAL ? (kb * 128) / 64 : 0;
  const int nqb = p.seq / 64 - qblk0;
  const int iters = grp * nqb;
  Tile64::Offsets offq, offdo;
  Tile64::offsets(offq, p.ldq, wave, lane);
  Tile64::offsets(offdo, p.lddo, wave, lane);
  const uint32_t lds0 = lds_address(smem);

  // Q / dO tiles go HBM -> LDS directly; the 64 lse and 64 delta values of a
  // block (as the dQ kernel left them: exp2 domain, -delta) travel through
  // one register per thread and are parked in LDS at the end of the previous
  // iteration, so waiting for them never stalls the tiles.
  float rstat = 0.f;
  auto fetch = [&](int it, int stage) {
    const int hh = hk * grp + it / nqb;
    const long q0 = (long)(qblk0 + it % nqb) * 64;
    const long stat = ((long)b * p.n_heads + hh) * p.seq + q0;
    // one unconditional load, consumed only in park(): nothing in between waits for it
    const int st = tid & 127;
    rstat = p.delta[2 * stat + (st ^ 64)];  // lse[64], then -delta[64]
    const uint32_t dst = lds0 + stage * STAGE;
    dma_tile<D>(p.q + (row0 + q0) * p.ldq + hh * D, offq, dst, wave);
    dma_tile<D>(p.d_o + (row0 + q0) * p.lddo + hh * D, offdo, dst + TILE, wave);
  };
  auto park = [&](int stage) {
    float* st = (float*)(smem + stage * STAGE + 2 * TILE);
    if (tid < 128) st[tid] = rstat;
  };

  fetch(0, 0);
  park(0);
  dma_wait_all();
  __syncthreads();

  for (int it = 0; it < iters; ++it) {
    const int q0 = (qblk0 + it % nqb) * 64;
    const uint8_t* lds_q = smem + (it & 1) * STAGE;
    const uint8_t* lds_do = lds_q + TILE;
    const float* lds_lse = (const float*)(lds_do + TILE);
    const float* lds_delta = lds_lse + 64;
    fetch(min(it + 1, iters - 1), (it + 1) & 1);
    if (!(CAUSAL && q0 + 63 < k0)) {  // else: every query of the block precedes this wave's keys
      const bool diag = CAUSAL && q0 < k0 + 31;
      // TB score tiles (32 queries each) are in flight together: both when the
      // wave owns the whole register file (independent chains to interleave),
      // one when two workgroups share a CU.
      constexpr int TB = D > 64 ? 2 : 1;
#pragma unroll
      for (int t0 = 0; t0 < 2; t0 += TB) {
        f32x16 s[TB], dp[TB];
#pragma unroll
        for (int u = 0; u < TB; ++u) {
          const int t = t0 + u;
#pragma unroll
          for (int r = 0; r < 16; ++r) { s[u][r] = 0.f; dp[u][r] = 0.f; }
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            s[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(slabs_frag<D>(lds_q, t * 32, ks, lane),
                                                           kf[ks], s[u], 0, 0, 0);
            dp[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(slabs_frag<D>(lds_do, t * 32, ks, lane),
                                                            vf[ks], dp[u], 0, 0, 0);
          }
        }
        // (wave priority by phase as in the forward kernel: -2 % at the BERT-large shape)
        __builtin_amdgcn_s_setprio(2);
#pragma unroll
        for (int u = 0; u < TB; ++u) {
          const int t = t0 + u;
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
              float pr = fast_exp2(fmaf(s[u][r], sc, -ls[e]));
              if (diag && ki > q0 + ql + e) pr = 0.f;
              s[u][r] = pr;
              dp[u][r] = pr * (dp[u][r] + dl[e]);  // (the softmax scale is applied to dK at the end)
            }
          }
        }
        __builtin_amdgcn_s_setprio(3);
#pragma unroll
        for (int u = 0; u < TB; ++u) {
          const int t = t0 + u;
#pragma unroll
          for (int h2 = 0; h2 < 2; ++h2) {
            const bf16x8 pf = acc_to_frag(s[u], h2 * 8);
            const bf16x8 dsf = acc_to_frag(dp[u], h2 * 8);
#pragma unroll
            for (int i = 0; i < DT; ++i) {
              dvacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                  slab_frag_tr(lds_do, 64, i * 32, 2 * t + h2, lane), pf, dvacc[i], 0, 0, 0);
              dkacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                  slab_frag_tr(lds_q, 64, i * 32, 2 * t + h2, lane), dsf, dkacc[i], 0, 0, 0);
            }
          }
        }
        __builtin_amdgcn_s_setprio(0);
      }
    }
    park((it + 1) & 1);
    dma_wait_all();
    __syncthreads();
  }

  bf16_t* dkrow = p.dk + (row0 + ki) * p.lddk + hk * D;
  bf16_t* dvrow = p.dv + (row0 + ki) * p.lddv + hk * D;
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = i * 32 + g * 8 + (lane >> 5) * 4;
      *(uint2*)(dkrow + d) =
          make_uint2(pack_bf16x2(dkacc[i][4 * g] * p.scale, dkacc[i][4 * g + 1] * p.scale),
                     pack_bf16x2(dkacc[i][4 * g + 2] * p.scale, dkacc[i][4 * g + 3] * p.scale));
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
  p.rope_cos = nullptr;
  p.rope_sin = nullptr;
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
#define JPP_AF(D_, C_)                                                                  \
  do {                                                                                  \
    if (int rc = set_smem(attn_fwd_kernel<D_, C_>, 4 * D_ * 128)) return rc;            \
    hipLaunchKernelGGL((attn_fwd_kernel<D_, C_>), grid, dim3(256), 4 * D_ * 128, st, p); \
  } while (0)
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
  JPP_REQUIRE(!a->rope_cos == !a->rope_sin, "attn_bwd: rope_cos and rope_sin go together");
  JPP_REQUIRE(((uintptr_t)a->rope_cos | (uintptr_t)a->rope_sin) % 16 == 0,
              "attn_bwd: rotary tables must be 16-byte aligned");
  AttnParams p = make_params(a);
  // the causal kernels rotate dq / dk back themselves; without a mask a pass of its own does
  const bool fused_rope = a->rope_cos && a->causal;
  if (fused_rope) { p.rope_cos = a->rope_cos; p.rope_sin = a->rope_sin; }
  hipStream_t st = (hipStream_t)stream;
  dim3 gq(a->seq / 128, a->n_heads, a->batch);
  // causal: 64-key blocks, a workgroup takes blocks x and n-1-x; else 128-key blocks
  dim3 gkv(a->seq / 128, a->n_kv_heads, a->batch);
  const double fl = 8.0 * a->batch * a->seq * (double)a->seq * a->n_heads * a->head_dim *
                    (a->causal ? 0.5 : 1.0);
#define JPP_AB(D_, C_)                                                              \
  do {                                                                              \
    {                                                                               \
      ProbeScope probe(st, "attn_bwd_dq", fl * 0.4, 0);                             \
      if (C_) {                                                                     \
        if (int rc = launch_dq(st, p, D_, true)) return rc;                         \
      } else {                                                                      \
        if (int rc = set_smem(attn_bwd_dq_kernel<D_, false>, 4 * D_ * 128)) return rc; \
        hipLaunchKernelGGL((attn_bwd_dq_kernel<D_, false>), gq, dim3(256), 4 * D_ * 128, st, p); \
      }                                                                             \
    }                                                                               \
    ProbeScope probe(st, "attn_bwd_dkv", fl * 0.6, 0);                              \
    if (C_) {                                                                       \
      if (int rc = launch_dkv_causal(st, p, D_, gkv)) return rc;                      \
    } else {                                                                        \
      if (int rc = set_smem(attn_bwd_dkv_wide_kernel<D_, false>, 4 * D_ * 128 + 1024)) return rc; \
      hipLaunchKernelGGL((attn_bwd_dkv_wide_kernel<D_, false>), gkv, dim3(256), 4 * D_ * 128 + 1024, st, p); \
    }                                                                               \
  } while (0)
  if (a->head_dim == 64) { if (a->causal) JPP_AB(64, true); else JPP_AB(64, false); }
  else { if (a->causal) JPP_AB(128, true); else JPP_AB(128, false); }
#undef JPP_AB
  JPP_LAUNCH_CHECK();
  if (a->rope_cos && !fused_rope) {
    if (int rc = jpp_rope(stream, a->dq, a->lddq, a->rope_cos, a->rope_sin, a->batch, a->seq,
                          a->n_heads, a->head_dim, 1))
      return rc;
    return jpp_rope(stream, a->dk, a->lddk, a->rope_cos, a->rope_sin, a->batch, a->seq,
                    a->n_kv_heads, a->head_dim, 1);
  }
  return JPP_OK;
}
