// dK/dV of causal attention (see attention.hip for the conventions).  One wave per SIMD:
// nothing hides a wave's latencies but its own instruction order, so the kernel is
// software-pipelined by hand - the matrix products of the tiles before and after run under
// the elementwise arithmetic of the tile in the middle.
#include <type_traits>

#include "attention_common.h"

namespace jpp_attn {
namespace {

// ---------------------------------------------------------------------------
// A workgroup owns 64 keys of one kv head and walks the (query head, 64-query block) items
// that see them, from the last query block down, heads innermost (the workgroups of a kv
// head start at the same tiles and walk at the same pace, so a tile is fetched into the
// XCD's L2 once).  Wave w works on keys 32 (w & 1) .. +31 against queries 32 (w >> 1) .. +31
// of every item; the two query halves meet in LDS at the end (fixed order: deterministic).
// Under the mask a key block sees only the queries behind it, so a workgroup takes block x
// and then block n-1-x: every workgroup of the launch carries the same amount of work.
//
// Items travel HBM -> LDS through a ring of four slots (Q tile, dO tile, the rows' scaled
// delta and log-sum-exp), fetched three items ahead.  Per item a wave runs
//   1. S = Q K^T, dP = dO V^T                         (16 MFMAs at head 128)
//   2. P = exp2(S - lse), dS = P (dP - delta)          (elementwise)
//   3. dV += P^T dO, dK += dS^T Q                      (16 MFMAs)
// and one trip of the loop issues 3 of the item before, then 1 of the item after with 2 of
// the item in the middle between its MFMAs; two sets of score registers alternate.
// ---------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256, 1) void attn_bwd_dkv_kernel(AttnParams p) {
  constexpr int KS = D / 16, DT = D / 32;
  constexpr int TILE = D * 128;              // bytes of a [64][D] tile
  constexpr int SLOT = 2 * TILE + 1024;      // Q, dO, {delta, lse}[64] | 512 unused
  constexpr int NLOAD = 4 * (D / 64) + 1;    // wave-level loads per wave and item
  extern __shared__ __align__(1024) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ksb = wave & 1, qh = wave >> 1;
  const Work w = xcd_work();
  const int hk = w.h, b = w.b;
  const int grp = p.n_heads / p.n_kv_heads;
  const long row0 = (long)b * p.seq;
  const int nkb = p.seq / 64;
  const float sc = p.scale * kLog2e;
  const uint32_t lds0 = lds_address(smem);

  Tile64::Offsets offq, offdo;
  Tile64::offsets(offq, p.ldq, wave, lane);
  Tile64::offsets(offdo, p.lddo, wave, lane);
  // one 16-byte load per lane brings an item's row statistics, 64 {scaled delta, lse} pairs
  // as the dQ kernel left them; the upper half of the wave repeats the lower one into the
  // unused part of the slot
  const uint32_t offst = (uint32_t)((lane & 31) * 16);
  const int ql0 = qh * 32 + (lane >> 5) * 4;  // first of this lane's rows within a 64-query block

  for (int seg = 0; seg < 2; ++seg) {
    const int kb = seg == 0 ? w.x : nkb - 1 - w.x;
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
    // (waits for the loads here, and names where the fragments live: the accumulation
    // registers, where the MFMAs of the trips read them)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+a"(kf[ks]), "+a"(vf[ks]));
    f32x16 dkacc[DT], dvacc[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) { dkacc[i][r] = 0.f; dvacc[i][r] = 0.f; }

    const int total = grp * (nkb - kb);   // items; the last grp of them lie on the diagonal

    // The fetch cursor walks the items - running pointers, advanced with selects (the trips of
    // the main loop are one basic block) - and stays on the last item once they are exhausted,
    // so every trip issues the same number of loads (the waits below count them).
    const long head_back = (long)(grp - 1) * D;  // from the last head of a group to the first
    const bf16_t* f_q = p.q + (row0 + (long)(nkb - 1) * 64) * p.ldq + (long)hk * grp * D;
    const bf16_t* f_do = p.d_o + (row0 + (long)(nkb - 1) * 64) * p.lddo + (long)hk * grp * D;
    const float* f_st = p.delta + 2 * (((long)b * p.n_heads + hk * grp) * p.seq + (long)(nkb - 1) * 64);
    int f_h = 0, f_left = total;
    // part j of an item's loads (NLOAD of them per wave: the Q tile's, the dO tile's, the row
    // statistics); the last part moves the cursor on
    auto fetch_part = [&](int slot, int j) __attribute__((always_inline)) {
      const uint32_t dst = lds0 + slot * SLOT;
      constexpr int PER = Tile64::INSTS;  // loads per wave and 64-column slab
      if (j < NLOAD - 1) {
        const int t = j / (PER * (D / 64)), c = (j / PER) % (D / 64), k = j % PER;
        dma_load16(uniform_ptr((t ? f_do : f_q) + c * 64), (t ? offdo : offq)[k],
                   dst + t * TILE + c * 8192 + (wave * PER + k) * 1024);
        return;
      }
      dma_load16(uniform_ptr((const bf16_t*)f_st), offst, dst + 2 * TILE);
      const bool go = f_left > 1;
      const bool wrap = go && f_h + 1 == grp;   // next: first head of the query block before
      f_left -= go ? 1 : 0;
      f_h = wrap ? 0 : f_h + (go ? 1 : 0);
      f_q += wrap ? -(head_back + 64 * p.ldq) : (go ? D : 0);
      f_do += wrap ? -(head_back + 64 * p.lddo) : (go ? D : 0);
      f_st += wrap ? -2 * ((long)(grp - 1) * p.seq + 64) : (go ? 2 * (long)p.seq : 0);
    };
    auto fetch = [&](int slot) __attribute__((always_inline)) {
#pragma unroll
      for (int j = 0; j < NLOAD; ++j) fetch_part(slot, j);
    };

    // S and dP of an item (its tiles in `slot`) against this wave's keys
    auto scores = [&](const uint8_t* slot, f32x16& s, f32x16& dp) __attribute__((always_inline)) {
      bf16x8 qfr[KS], dofr[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        qfr[ks] = slabs_frag<D>(slot, qh * 32, ks, lane);
        dofr[ks] = slabs_frag<D>(slot + TILE, qh * 32, ks, lane);
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qfr[ks], kf[ks], s, 0, 0, 0);
        dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dofr[ks], vf[ks], dp, 0, 0, 0);
      }
    };
    // Items of the key block's own query block are masked: the query half behind the keys
    // sees all of them, the half in front none, the one on the diagonal what lies at or
    // before each query.  Items past the end (an odd count is rounded up) count as unseen.
    auto mask = [&](f32x16& s, int item) __attribute__((always_inline)) {
      if (item >= total - grp) {  // wave-uniform
        if (item >= total || qh < ksb) {
#pragma unroll
          for (int r = 0; r < 16; ++r) s[r] = -INFINITY;
        } else if (qh == ksb) {
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if ((lane & 31) > (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3)) s[r] = -INFINITY;
        }
      }
    };

    bf16x8 pf[2], dsf[2], dotr[2][DT], qtr[2][DT];  // of the item whose step 3 is still to run
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
#pragma unroll
      for (int e = 0; e < 8; ++e) { pf[h2][e] = (__bf16)0.f; dsf[h2][e] = (__bf16)0.f; }
#pragma unroll
      for (int i = 0; i < DT; ++i) { dotr[h2][i] = pf[h2]; qtr[h2][i] = pf[h2]; }
    }
    auto grads = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
        for (int i = 0; i < DT; ++i) {
          dvacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dotr[h2][i], pf[h2], dvacc[i], 0, 0, 0);
          dkacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qtr[h2][i], dsf[h2], dkacc[i], 0, 0, 0);
        }
    };

    // One trip: item i is in the middle (its scores in s_c / dp_c), i - 1 before, i + 1 after.
    // A wave issues in order: an MFMA that finds the matrix core busy holds back whatever
    // follows it, so the elementwise work and the LDS reads have to sit between the MFMAs in
    // the instruction stream.  The MFMAs of a trip are volatile asm statements (they keep
    // their order, and LDS reads do not cross them); the elementwise work is tied to its place
    // by empty asm statements on its inputs and results.
    auto trip = [&](auto tail, int i, f32x16& s_c, f32x16& dp_c, f32x16& s_n, f32x16& dp_n) __attribute__((always_inline)) {
      constexpr bool TAIL = decltype(tail)::value;
      const uint8_t* sl_c = smem + (i & 3) * SLOT;
      const uint8_t* sl_n = smem + ((i + 1) & 3) * SLOT;
      // Q / dO fragments of item i + 1: the first half now, the second while the first is used
      bf16x8 qfr[KS], dofr[KS];
#pragma unroll
      for (int ks = 0; ks < KS / 2; ++ks) {
        qfr[ks] = slabs_frag<D>(sl_n, qh * 32, ks, lane);
        dofr[ks] = slabs_frag<D>(sl_n + TILE, qh * 32, ks, lane);
      }
      // row statistics of item i: {scaled delta, lse} pairs, two rows per 16-byte read
      const float* st = (const float*)(sl_c + 2 * TILE) + 2 * ql0;
      auto stats = [&](int r) __attribute__((always_inline)) { return *(const float4*)(st + 2 * ((r >> 2) * 8 + (r & 3))); };
      float4 st_q[3] = {stats(0), stats(2), stats(4)};  // read two pairs of rows ahead of their use
      // dV / dK products of item i - 1 from registers (the reads above arrive under them);
      // behind each pair, the transposed fragments of item i take over its registers
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
        for (int ii = 0; ii < DT; ++ii) {
          mfma_avv(dvacc[ii], dotr[h2][ii], pf[h2]);
          mfma_avv(dkacc[ii], qtr[h2][ii], dsf[h2]);
          dotr[h2][ii] = slab_frag_tr(sl_c + TILE, 64, ii * 32, 2 * qh + h2, lane);
          qtr[h2][ii] = slab_frag_tr(sl_c, 64, ii * 32, 2 * qh + h2, lane);
          // item i + 3 into the slot item i - 1 has left (its scalar address work runs under
          // the MFMAs)
          // (a load or two behind every pair of MFMAs rather than all at once)
          {
            constexpr int GROUPS = 2 * DT, EACH = (NLOAD + GROUPS - 1) / GROUPS;
            const int g = h2 * DT + ii;
#pragma unroll
            for (int j = g * EACH; j < (g + 1) * EACH && j < NLOAD; ++j) fetch_part((i + 3) & 3, j);
          }
        }
      // S and dP of item i + 1, two MFMAs at a time, with P and dS of EPG elements of item i
      // behind each pair
      constexpr int EPG = 16 / KS;
      uint32_t pw[8], dw[8];  // P and dS as bf16 pairs
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks == 0) {
          mfma_vva_first(s_n, qfr[0], kf[0]);
          mfma_vva_first(dp_n, dofr[0], vf[0]);
        } else {
          mfma_vva(s_n, qfr[ks], kf[ks]);
          mfma_vva(dp_n, dofr[ks], vf[ks]);
        }
        if (ks < KS / 2) {
          qfr[ks + KS / 2] = slabs_frag<D>(sl_n, qh * 32, ks + KS / 2, lane);
          dofr[ks + KS / 2] = slabs_frag<D>(sl_n + TILE, qh * 32, ks + KS / 2, lane);
        }
#pragma unroll
        for (int r = ks * EPG; r < ks * EPG + EPG; r += 2) {
          const float4 x = st_q[(r >> 1) % 3];
          if (r + 6 < 16) st_q[(r >> 1) % 3] = stats(r + 6);
          float s0 = s_c[r], s1 = s_c[r + 1], g0 = dp_c[r], g1 = dp_c[r + 1];
          asm volatile("" : "+v"(s0), "+v"(s1), "+v"(g0), "+v"(g1));
          const float p0 = fast_exp2(fmaf(s0, sc, -x.y));  // exp2(-inf) = 0 where masked
          const float p1 = fast_exp2(fmaf(s1, sc, -x.w));
          pw[r >> 1] = pack2(p0, p1);
          dw[r >> 1] = pack2(p0 * fmaf(g0, p.scale, -x.x), p1 * fmaf(g1, p.scale, -x.z));
          asm volatile("" : "+v"(pw[r >> 1]), "+v"(dw[r >> 1]));
        }
      }
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 pv = {pw[4 * h2], pw[4 * h2 + 1], pw[4 * h2 + 2], pw[4 * h2 + 3]};
        const u32x4 dv = {dw[4 * h2], dw[4 * h2 + 1], dw[4 * h2 + 2], dw[4 * h2 + 3]};
        pf[h2] = __builtin_bit_cast(bf16x8, pv);
        dsf[h2] = __builtin_bit_cast(bf16x8, dv);
      }
      // The compiler does not know that the asm statements above are MFMAs, whose results
      // take 11 issue slots to land: whatever it does with the new scores (copies included)
      // has to wait behind this statement, which the elementwise work of the last MFMA pair
      // (ten instructions and more, tied in front of it) and four idle slots keep clear.
      asm volatile("s_nop 3" : "+v"(s_n), "+v"(dp_n));
      if constexpr (TAIL) mask(s_n, i + 1);
      lds_wait_all();       // this wave has read all it needs of item i's slot ...
      dma_wait<NLOAD>();    // ... and its share of item i + 2 has landed (i + 3 may be on its way)
      __syncthreads();
    };

    fetch(0);
    fetch(1);
    fetch(2);
    dma_wait<NLOAD>();
    __syncthreads();
    f32x16 s_a, dp_a, s_b, dp_b;
    scores(smem, s_a, dp_a);
    mask(s_a, 0);
    int i = 0;
    for (; i + 2 < total - grp; i += 2) {  // neither trip computes the scores of a masked item
      trip(std::false_type{}, i, s_a, dp_a, s_b, dp_b);
      trip(std::false_type{}, i + 1, s_b, dp_b, s_a, dp_a);
    }
    for (; i < total; i += 2) {
      trip(std::true_type{}, i, s_a, dp_a, s_b, dp_b);
      trip(std::true_type{}, i + 1, s_b, dp_b, s_a, dp_a);
    }
    grads();  // of the last item
    dma_wait_all();  // the cursor's repeated fetches of the last item
    __syncthreads();

    // the upper query half hands its partial sums to the lower one through LDS:
    // [ksb][register][lane] floats
    float* xch = (float*)smem + ksb * (2 * DT * 16 * 64) + lane;
    if (qh == 1) {
#pragma unroll
      for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          xch[(i * 16 + r) * 64] = dkacc[i][r];
          xch[((DT + i) * 16 + r) * 64] = dvacc[i][r];
        }
    }
    __syncthreads();
    if (qh == 0) {
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
    __syncthreads();  // the exchange area is slot memory of the next key block
  }
}

}  // namespace

int launch_dkv_causal(hipStream_t stream, const AttnParams& p, int head_dim, dim3 grid) {
  if (head_dim == 64) {
    constexpr int LDS = 4 * (2 * 64 * 128 + 1024);
    if (int rc = set_smem(attn_bwd_dkv_kernel<64>, LDS)) return rc;
    hipLaunchKernelGGL((attn_bwd_dkv_kernel<64>), grid, dim3(256), LDS, stream, p);
  } else {
    constexpr int LDS = 4 * (2 * 128 * 128 + 1024);
    if (int rc = set_smem(attn_bwd_dkv_kernel<128>, LDS)) return rc;
    hipLaunchKernelGGL((attn_bwd_dkv_kernel<128>), grid, dim3(256), LDS, stream, p);
  }
  return JPP_OK;
}

}  // namespace jpp_attn
