// dK/dV of causal attention (see attention.hip for the conventions).  This kernel has one
// wave per SIMD and nothing to hide its latencies behind but its own instruction order; it
// is compiled with LLVM's iterative ILP scheduler, which orders it 4 % faster than the
// default one does (and the other attention kernels slower, hence the separate file).
#include "attention_common.h"

namespace jpp_attn {
namespace {

// ---------------------------------------------------------------------------
// backward, dK and dV.  A workgroup owns 64 keys of one kv head: wave w works
// on keys 32 (w & 1) .. +31 and on every second (query head, 64-query block)
// pair of the list the key block has to visit, starting with pair w >> 1.  The
// two wave pairs stream their own Q / dO tiles through their own LDS stages,
// and their partial dK / dV meet in LDS at the end (fixed order: deterministic).
// Under a causal mask a key block sees only the queries behind it, so a
// workgroup takes block x and then block n-1-x: every workgroup of the launch
// carries the same amount of work.
// ---------------------------------------------------------------------------
using Tile64H = DmaTile<64, false, 2>;  // a [64][64] slab copied by the two waves of a pair
template <int D>
__device__ __forceinline__ void dma_tile_pair(const bf16_t* src, const Tile64H::Offsets& off,
                                              uint32_t lds, int wave_in_pair) {
#pragma unroll
  for (int c = 0; c < D / 64; ++c)
    Tile64H::issue<0, Tile64H::INSTS>(uniform_ptr(src + c * 64), off, lds + c * 8192, wave_in_pair);
}

template <int D, bool CAUSAL>
__global__ __launch_bounds__(256, (D > 64 ? 1 : 2)) void attn_bwd_dkv_kernel(AttnParams p) {
  constexpr int KS = D / 16, DT = D / 32;
  constexpr int TILE = D * 128, STAGE = 2 * TILE + 512;  // Q tile, dO tile, lse[64], delta[64]
  constexpr int PAIR = 2 * STAGE;                        // two stages per wave pair
  extern __shared__ __align__(1024) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ksb = wave & 1, half = wave >> 1;
  const Work w = xcd_work();
  const int hk = w.h, b = w.b;
  const int grp = p.n_heads / p.n_kv_heads;
  const long row0 = (long)b * p.seq;
  const int nkb = p.seq / 64;
  const float sc = p.scale * kLog2e;
  uint8_t* const my = smem + half * PAIR;  // this pair's stages
  const uint32_t lds0 = lds_address(my);
  const int ht = tid & 127;                // thread index within the pair

  Tile64H::Offsets offq, offdo;
  Tile64H::offsets(offq, p.ldq, ksb, lane);
  Tile64H::offsets(offdo, p.lddo, ksb, lane);

  for (int seg = 0; seg < (CAUSAL ? 2 : 1); ++seg) {
    const int kb = CAUSAL ? (seg == 0 ? w.x : nkb - 1 - w.x) : w.x;
    const int k0 = kb * 64 + ksb * 32;
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

    const int qblk0 = CAUSAL ? kb : 0;
    const int nqb = nkb - qblk0;
    // (query block, head) pairs to visit: from the last query block down, heads innermost.
    // Every workgroup of a kv head starts at the same tiles and walks them at the same
    // pace, so a tile is fetched into the XCD's L2 once and found there by the others.
    const int total = grp * nqb;
    const int trips = (total + 1) / 2;    // per wave pair; the last one may be empty for pair 1

    // Q / dO tiles go HBM -> LDS directly; the 64 lse and 64 delta values of a
    // block travel through one register per thread and are parked in LDS at the
    // end of the previous trip, so waiting for them never stalls the tiles.
    float rstat = 0.f;
    auto fetch = [&](int trip, int stage) {
      const int it = min(2 * trip + half, total - 1);
      const int hh = hk * grp + it % grp;
      const long q0 = (long)(nkb - 1 - it / grp) * 64;
      const long stat = ((long)b * p.n_heads + hh) * p.seq + q0;
      // one unconditional load, consumed only in park(): nothing in between waits for it
      rstat = *(ht < 64 ? p.lse + stat + ht : p.delta + stat + (ht - 64));
      const uint32_t dst = lds0 + stage * STAGE;
      dma_tile_pair<D>(p.q + (row0 + q0) * p.ldq + hh * D, offq, dst, ksb);
      dma_tile_pair<D>(p.d_o + (row0 + q0) * p.lddo + hh * D, offdo, dst + TILE, ksb);
    };
    auto park = [&](int stage) {
      // lse in the exp2 domain; delta scaled, so that scale (dP - delta) is one fma per element
      ((float*)(my + stage * STAGE + 2 * TILE))[ht] = ht < 64 ? rstat * kLog2e : rstat * p.scale;
    };

    // one 32-query tile against this wave's 32 keys
    auto tile = [&](bool diag, const uint8_t* lds_q, const uint8_t* lds_do, const float* lds_lse,
                    const float* lds_delta, int q0, int t) {
      f32x16 s, dp;
      {
        bf16x8 qfr[KS], dofr[KS];  // read ahead of the MFMAs that consume them
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          qfr[ks] = slabs_frag<D>(lds_q, t * 32, ks, lane);
          dofr[ks] = slabs_frag<D>(lds_do, t * 32, ks, lane);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qfr[ks], kf[ks], s, 0, 0, 0);
          dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dofr[ks], vf[ks], dp, 0, 0, 0);
        }
      }
      bf16x8 dotr[2][DT], qtr[2][DT];  // transposed fragments arrive under the arithmetic below
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
        for (int i = 0; i < DT; ++i) {
          dotr[h2][i] = slab_frag_tr(lds_do, 64, i * 32, 2 * t + h2, lane);
          qtr[h2][i] = slab_frag_tr(lds_q, 64, i * 32, 2 * t + h2, lane);
        }
      if (CAUSAL && diag) {
        // only tiles on the diagonal pay for the mask: the empty asm keeps the compiler from
        // turning this (wave-uniform) branch into selects on every tile
        asm volatile("" ::: "memory");
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int q = q0 + t * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
          if (ki > q) s[r] = -INFINITY;
        }
      }
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
          const float pr = fast_exp2(fmaf(s[r], sc, -ls[e]));  // exp2(-inf) = 0 where masked
          s[r] = pr;
          dp[r] = pr * fmaf(dp[r], p.scale, -dl[e]);
        }
      }
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const bf16x8 pf = acc_to_frag(s, h2 * 8);
        const bf16x8 dsf = acc_to_frag(dp, h2 * 8);
#pragma unroll
        for (int i = 0; i < DT; ++i) {
          dvacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dotr[h2][i], pf, dvacc[i], 0, 0, 0);
          dkacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qtr[h2][i], dsf, dkacc[i], 0, 0, 0);
        }
      }
    };

    fetch(0, 0);
    park(0);
    dma_wait_all();
    __syncthreads();

    for (int trip = 0; trip < trips; ++trip) {
      const int it = 2 * trip + half;
      const int q0 = (nkb - 1 - it / grp) * 64;
      const uint8_t* lds_q = my + (trip & 1) * STAGE;
      const uint8_t* lds_do = lds_q + TILE;
      const float* lds_lse = (const float*)(lds_do + TILE);
      const float* lds_delta = lds_lse + 64;
      fetch(min(trip + 1, trips - 1), (trip + 1) & 1);
      if (it < total) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const int qt = q0 + t * 32;  // first query of the tile
          if (CAUSAL && qt + 31 < k0) continue;  // every query of the tile precedes the keys
          tile(qt < k0 + 31, lds_q, lds_do, lds_lse, lds_delta, q0, t);
        }
      }
      park((trip + 1) & 1);
      dma_wait_all();
      __syncthreads();
    }

    // pair 1 hands its partial sums to pair 0 through LDS: [ksb][register][lane] floats
    float* xch = (float*)smem + ksb * (2 * DT * 16 * 64) + lane;
    if (half == 1) {
#pragma unroll
      for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          xch[(i * 16 + r) * 64] = dkacc[i][r];
          xch[((DT + i) * 16 + r) * 64] = dvacc[i][r];
        }
    }
    __syncthreads();
    if (half == 0) {
      bf16_t* dkrow = p.dk + (row0 + ki) * p.lddk + hk * D;
      bf16_t* dvrow = p.dv + (row0 + ki) * p.lddv + hk * D;
#pragma unroll
      for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          dkacc[i][r] += xch[(i * 16 + r) * 64];
          dvacc[i][r] += xch[((DT + i) * 16 + r) * 64];
        }
      if (p.rope_cos) rope_back<D, DT>(dkacc, p.rope_cos, p.rope_sin, ki, lane);
#pragma unroll
      for (int i = 0; i < DT; ++i) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int d = i * 32 + g * 8 + (lane >> 5) * 4;
          *(uint2*)(dkrow + d) = make_uint2(pack_bf16x2(dkacc[i][4 * g], dkacc[i][4 * g + 1]),
                                            pack_bf16x2(dkacc[i][4 * g + 2], dkacc[i][4 * g + 3]));
          *(uint2*)(dvrow + d) = make_uint2(pack_bf16x2(dvacc[i][4 * g], dvacc[i][4 * g + 1]),
                                            pack_bf16x2(dvacc[i][4 * g + 2], dvacc[i][4 * g + 3]));
        }
      }
    }
    __syncthreads();  // the exchange area is stage memory of the next key block
  }
}

}  // namespace

int launch_dkv_causal(hipStream_t stream, const AttnParams& p, int head_dim, dim3 grid) {
  if (head_dim == 64) {
    if (int rc = set_smem(attn_bwd_dkv_kernel<64, true>, 8 * 64 * 128 + 2048)) return rc;
    hipLaunchKernelGGL((attn_bwd_dkv_kernel<64, true>), grid, dim3(256), 8 * 64 * 128 + 2048,
                       stream, p);
  } else {
    if (int rc = set_smem(attn_bwd_dkv_kernel<128, true>, 8 * 128 * 128 + 2048)) return rc;
    hipLaunchKernelGGL((attn_bwd_dkv_kernel<128, true>), grid, dim3(256), 8 * 128 * 128 + 2048,
                       stream, p);
  }
  return JPP_OK;
}

}  // namespace jpp_attn
