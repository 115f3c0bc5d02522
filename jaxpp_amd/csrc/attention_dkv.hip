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
// Items travel HBM -> LDS through a ring of four slots (Q tile, dO tile, the rows' -delta
// and log-sum-exp), fetched three items ahead.  Per item a wave runs
//   1. S = Q K^T, dP - delta = dO V^T - delta          (16 MFMAs at head 128; the accumulator
//                                                       of the second starts from -delta, read
//                                                       from LDS straight into its registers)
//   2. P = exp2(S - lse), dS = P (dP - delta)          (elementwise; the softmax scale that
//                                                       belongs on dS is applied to dK at the end)
//   3. dV += P^T dO, dK += dS^T Q                      (16 MFMAs)
// and one trip of the loop issues 3 of the item before, then 1 of the item after with 2 of
// the item in the middle between its MFMAs; two sets of score registers alternate.
//
// With one wave per SIMD the kernel is bound by the number of instructions a trip issues, so
// the LDS addresses of a trip are a handful of per-lane constants plus the slot's offset, and
// every read is one of those registers plus an immediate.
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
  // one 16-byte load per lane brings an item's row statistics, -delta[64] then lse[64] as the
  // dQ kernel left them; the upper half of the wave repeats the lower one into the unused
  // part of the slot
  const uint32_t offst = (uint32_t)((lane & 31) * 16);
  typedef __attribute__((address_space(3))) const bf16x8* lds_frag;
  typedef __attribute__((address_space(3))) const f32x4* lds_f4;
  typedef __attribute__((address_space(3))) s16x4* lds_s16x4;

  // Per-lane parts of the LDS addresses, in bytes from the start of a slot.
  // Row fragment (tile t, step ks) of this wave's 32 queries:
  //   t TILE + (ks >> 2) 8192 + (a_row ^ (ks & 3) << 5)
  // (the chunk 2 (ks & 3) + lane / 32 enters the swizzle by XOR, and 2 (ks & 3) has bit 0 clear)
  const uint32_t a_row = lds0 + (uint32_t)slab_off(qh * 32 + (lane & 31), lane >> 5);
  // Transposed fragment (tile t, columns 32 ii.., steps 2 qh + h2, half hi) - slab_frag_tr()
  // with its address split into the lane's part and the rest:
  //   t TILE + (ii >> 1) 8192 + h2 2048 + hi 1024 + (a_tr ^ ((ii & 1) ^ hi) << 6)
  uint32_t a_tr;
  {
    const int g = lane >> 4, s = lane & 15;
    const int k0 = qh * 32 + ((g >> 1) << 2) + (s >> 2);
    const int c0 = ((g & 1) << 1) + ((s & 3) >> 1);
    a_tr = lds0 + (uint32_t)(((s & 1) << 3) + slab_off(k0, c0));
  }
  // Row statistics: the lane's rows 8 g + 4 (lane / 32) + 0..3 of its query half, four floats
  // per read:  2 TILE + [256 for lse] + 32 g + a_st
  const uint32_t a_st = lds0 + (uint32_t)(2 * TILE + (qh * 32 + (lane >> 5) * 4) * 4);

  for (int seg = 0; seg < 2; ++seg) {
    const int kb = seg == 0 ? w.x : nkb - 1 - w.x;
    const int k0 = kb * 64 + ksb * 32;

    // The key block's K and V tiles come through LDS like every other tile (into the slot the
    // ring uses last): a fragment taken from HBM directly touches 32 rows with 32 bytes each,
    // and the CU's path to memory takes such a load line by line.
    bf16x8 kf[KS], vf[KS];
    {
      Tile64::Offsets offk, offv;
      Tile64::offsets(offk, p.ldk, wave, lane);
      Tile64::offsets(offv, p.ldv, wave, lane);
      dma_tile<D>(p.k + (row0 + (long)kb * 64) * p.ldk + hk * D, offk, lds0 + 3 * SLOT, wave);
      dma_tile<D>(p.v + (row0 + (long)kb * 64) * p.ldv + hk * D, offv, lds0 + 3 * SLOT + TILE, wave);
    }
    f32x16 dkacc[DT], dvacc[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) { dkacc[i][r] = 0.f; dvacc[i][r] = 0.f; }

    const int total = grp * (nkb - kb);   // items; the last grp of them lie on the diagonal

    // The fetch cursor walks the items - running addresses, advanced with selects (the trips of
    // the main loop are one basic block) - and stays on the last item once they are exhausted,
    // so every trip issues the same number of loads (the waits below count them).
    uint64_t f_q = uniform_u64((uint64_t)(p.q + (row0 + (long)(nkb - 1) * 64) * p.ldq + (long)hk * grp * D));
    uint64_t f_do = uniform_u64((uint64_t)(p.d_o + (row0 + (long)(nkb - 1) * 64) * p.lddo + (long)hk * grp * D));
    uint64_t f_st = uniform_u64((uint64_t)(p.delta + 2 * (((long)b * p.n_heads + hk * grp) * p.seq + (long)(nkb - 1) * 64)));
    // bytes from one item to the next: the next head, or (from the last head of a group) the
    // first head of the query block before
    const int64_t step_qd = 2 * D, step_st = 8 * (int64_t)p.seq;
    const int64_t wrap_q = -2 * ((int64_t)(grp - 1) * D + 64 * p.ldq);
    const int64_t wrap_do = -2 * ((int64_t)(grp - 1) * D + 64 * p.lddo);
    const int64_t wrap_st = -8 * ((int64_t)(grp - 1) * p.seq + 64);
    int f_h = 0, f_left = total;
    // part J of an item's loads (NLOAD of them per wave: the Q tile's, the dO tile's, the row
    // statistics) into the slot at `dst` (this wave's share of it); the last part moves the
    // cursor on
    auto fetch_part = [&](uint32_t dst, auto j_c) __attribute__((always_inline)) {
      constexpr int J = decltype(j_c)::value;
      constexpr int PER = Tile64::INSTS;  // loads per wave and 64-column slab
      if constexpr (J < NLOAD - 1) {
        constexpr int t = J / (PER * (D / 64)), c = (J / PER) % (D / 64), k = J % PER;
        dma_load16_at<t * TILE + c * 8192 + k * 1024, c * 128>(t ? f_do : f_q, (t ? offdo : offq)[k], dst);
      } else {
        dma_load16_at<2 * TILE, 0>(f_st, offst, dst - wave * (PER * 1024));
        const bool go = f_left > 1;
        const bool wrap = go && f_h + 1 == grp;
        f_left -= go ? 1 : 0;
        f_h = wrap ? 0 : f_h + (go ? 1 : 0);
        f_q += wrap ? wrap_q : (go ? step_qd : 0);
        f_do += wrap ? wrap_do : (go ? step_qd : 0);
        f_st += wrap ? wrap_st : (go ? step_st : 0);
      }
    };
    const uint32_t lds_w = lds0 + wave * (Tile64::INSTS * 1024);
    auto fetch = [&](int slot) __attribute__((always_inline)) {
      const uint32_t dst = lds_w + (uint32_t)slot * SLOT;
      static_for<0, NLOAD>([&](auto j_c) __attribute__((always_inline)) { fetch_part(dst, j_c); });
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
      for (int g = 0; g < 4; ++g) {
        const f32x4 nd = *(lds_f4)(uintptr_t)(a_st + (uint32_t)(slot - smem) + 32 * g);
        dp[4 * g] = nd.x; dp[4 * g + 1] = nd.y; dp[4 * g + 2] = nd.z; dp[4 * g + 3] = nd.w;
      }
      // (the same statements as in the trips: compiler-chosen MFMAs would leave their results
      // in the accumulation registers, and the loop would copy its scores there and back)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks == 0) mfma_vaa_first(s, qfr[0], kf[0]);
        else mfma_vaa(s, qfr[ks], kf[ks]);
        mfma_vaa(dp, dofr[ks], vf[ks]);
      }
      asm volatile("s_nop 15" : "+v"(s), "+v"(dp));
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
    // A wave issues in order, and an MFMA that finds the matrix core busy (32 cycles per
    // MFMA) holds back whatever follows it.  So the MFMAs go out one at a time, each followed
    // by its share of the trip's other instructions - about as much as issues in those 32
    // cycles - and never two in a row, where the second would hold up the wave while nothing
    // else issues.  MFMAs and elementwise instructions are volatile asm statements (they
    // keep their order, and LDS reads do not cross the MFMAs).
    auto trip = [&](auto tail, int i, f32x16& s_c, f32x16& dp_c, f32x16& s_n, f32x16& dp_n) __attribute__((always_inline)) {
      constexpr bool TAIL = decltype(tail)::value;
      constexpr int NB = 4 * DT;    // MFMAs of step 3
      constexpr int NR = KS + 8;    // reads for steps 1 and 2: KS/2 Q and KS/2 dO row fragments, 4 x -delta, 4 x lse
      constexpr int EPG = 16 / KS;  // elements of step 2 per MFMA pair of step 1
      uint32_t b_row[4], b_tr[2], b_stc, b_stn;  // this trip's address registers
      bf16x8 qfr[KS], dofr[KS];     // Q / dO fragments of item i + 1
      f32x4 lse_r[4];             // lse of item i's rows
      auto row_frag = [&](int t, int ks) __attribute__((always_inline)) {
        return *(lds_frag)(uintptr_t)(b_row[ks & 3] + (t * TILE + (ks >> 2) * 8192));
      };
      auto tr_frag = [&](int t, int ii, int h2) __attribute__((always_inline)) {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4)(uintptr_t)(
            b_tr[ii & 1] + (t * TILE + (ii >> 1) * 8192 + h2 * 2048)));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4)(uintptr_t)(
            b_tr[(ii & 1) ^ 1] + (t * TILE + (ii >> 1) * 8192 + h2 * 2048 + 1024)));
        const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(bf16x8, v);
      };
      auto early_read = [&](int n) __attribute__((always_inline)) {
        if (n < KS) {  // first half of the row fragments (the second follows while the first is used)
          if (n & 1) dofr[n >> 1] = row_frag(1, n >> 1);
          else qfr[n >> 1] = row_frag(0, n >> 1);
        } else if (n < KS + 4) {  // -delta of item i + 1's rows: where its dP products start from
          const int g = n - KS;
          const f32x4 nd = *(lds_f4)(uintptr_t)(b_stn + 32 * g);
          dp_n[4 * g] = nd.x; dp_n[4 * g + 1] = nd.y; dp_n[4 * g + 2] = nd.z; dp_n[4 * g + 3] = nd.w;
        } else {
          const int g = n - KS - 4;
          lse_r[g] = *(lds_f4)(uintptr_t)(b_stc + (256 + 32 * g));
        }
      };
      // dV / dK products of item i - 1 from registers; behind each, the transposed fragments
      // of item i take over its operand's registers, and a share of: the reads for steps 1
      // and 2, the loads of item i + 3 into the slot item i - 1 has left
      uint32_t dst = lds_w + (uint32_t)((i + 3) & 3) * SLOT;
      asm volatile("" : "+s"(dst));
      // The loads of item i + 3 (into the slot item i - 1 has left) go behind the MFMAs of step
      // 3, evenly spread.  (Behind those of step 1 as well they cost 6 % of the kernel, and so
      // did starting the four waves of a trip 16 cycles apart - tried because a CU's waves
      // share one path to memory, 16 cycles per wave-level load, and wait for each other when
      // they reach their loads together.)
      auto dma_slot = [&](int m) __attribute__((always_inline)) {  // m: constant after unrolling
        static_for<0, NLOAD>([&](auto j_c) __attribute__((always_inline)) {
          if (decltype(j_c)::value * NB / NLOAD == m) fetch_part(dst, j_c);
        });
      };
      static_for<0, NB>([&](auto m_c) __attribute__((always_inline)) {
        constexpr int m = decltype(m_c)::value;
        constexpr int h2 = m / (2 * DT), ii = (m >> 1) % DT;
        if (m & 1) mfma_avv(dkacc[ii], qtr[h2][ii], dsf[h2]);
        else mfma_avv(dvacc[ii], dotr[h2][ii], pf[h2]);
        if (m == 0) {
          // (slot offsets are multiples of 1024: adding them commutes with the XORs; the
          // offsets pass through an asm statement so that this work stays behind the MFMA)
          uint32_t o_c = (uint32_t)(i & 3) * SLOT, o_n = (uint32_t)((i + 1) & 3) * SLOT;
          asm volatile("" : "+s"(o_c), "+s"(o_n));
          b_stc = a_st + o_c;
          b_stn = a_st + o_n;
          b_row[0] = a_row + o_n;
#pragma unroll
          for (int j = 1; j < 4; ++j) b_row[j] = b_row[0] ^ (j << 5);
          b_tr[0] = a_tr + o_c;
          b_tr[1] = b_tr[0] ^ 64;
          asm volatile("" : "+v"(b_row[0]), "+v"(b_row[1]), "+v"(b_row[2]), "+v"(b_row[3]),
                            "+v"(b_tr[0]), "+v"(b_tr[1]), "+v"(b_stc), "+v"(b_stn));
        }
        if (m & 1) qtr[h2][ii] = tr_frag(0, ii, h2);
        else dotr[h2][ii] = tr_frag(1, ii, h2);
#pragma unroll
        for (int n = m * NR / NB; n < (m + 1) * NR / NB; ++n) early_read(n);
        dma_slot(m);
      });
      // S and dP of item i + 1, with P and dS of EPG elements of item i behind each pair:
      // behind the first MFMA the exponentials (and the arguments of the next pair's), behind
      // the second the products and the packing to bf16.  No instruction reads the result of
      // the one before it.
      auto lse_of = [&](int r) __attribute__((always_inline)) {
        const f32x4 l4 = lse_r[r >> 2];
        return (r & 3) == 0 ? l4.x : (r & 3) == 1 ? l4.y : (r & 3) == 2 ? l4.z : l4.w;
      };
      float t[EPG], tn[EPG], pe[EPG], de[EPG];
      uint32_t pw[8], dw[8];  // P and dS as bf16 pairs
#define JPP_EXP_ARGS(KS_, DST)                                                              \
  _Pragma("unroll") for (int e = 0; e < EPG; ++e) {                                         \
    const float l = lse_of((KS_) * EPG + e);                                                \
    asm volatile("v_fma_f32 %0, %1, %2, -%3"                                                \
                 : "=v"(DST[e]) : "v"(s_c[(KS_) * EPG + e]), "s"(sc), "v"(l));              \
  }
      JPP_EXP_ARGS(0, t)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks == 0) mfma_vaa_first(s_n, qfr[0], kf[0]);
        else mfma_vaa(s_n, qfr[ks], kf[ks]);
#pragma unroll
        for (int e = 0; e < EPG; ++e)  // exp2(-inf) = 0 where masked
          asm volatile("v_exp_f32 %0, %1" : "=v"(pe[e]) : "v"(t[e]));
        if (ks + 1 < KS) { JPP_EXP_ARGS(ks + 1, tn) }
        if (ks < KS / 2) qfr[ks + KS / 2] = row_frag(0, ks + KS / 2);
        mfma_vaa(dp_n, dofr[ks], vf[ks]);
#pragma unroll
        for (int e = 0; e < EPG; ++e)
          asm volatile("v_mul_f32 %0, %1, %2" : "=v"(de[e]) : "v"(pe[e]), "v"(dp_c[ks * EPG + e]));
#pragma unroll
        for (int e = 0; e < EPG; e += 2) {
          asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(pw[(ks * EPG + e) >> 1]) : "v"(pe[e]), "v"(pe[e + 1]));
          asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(dw[(ks * EPG + e) >> 1]) : "v"(de[e]), "v"(de[e + 1]));
        }
        if (ks < KS / 2) dofr[ks + KS / 2] = row_frag(1, ks + KS / 2);
#pragma unroll
        for (int e = 0; e < EPG; ++e) t[e] = tn[e];
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
      // has to wait behind this statement, which the elementwise work behind the last MFMA
      // (four instructions or more) and eight idle slots keep clear.
#undef JPP_EXP_ARGS
      asm volatile("s_nop 7" : "+v"(s_n), "+v"(dp_n));
      if constexpr (TAIL) mask(s_n, i + 1);
      lds_wait_all();       // this wave has read all it needs of item i's slot ...
      dma_wait<NLOAD>();    // ... and its share of item i + 2 has landed (i + 3 may be on its way)
      __syncthreads();
    };

    fetch(0);
    fetch(1);
    fetch(2);
    dma_wait<3 * NLOAD>();  // the K / V tiles are in
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kf[ks] = slabs_frag<D>(smem + 3 * SLOT, ksb * 32, ks, lane);
      vf[ks] = slabs_frag<D>(smem + 3 * SLOT + TILE, ksb * 32, ks, lane);
    }
    // (names where the fragments live: the accumulation registers, where the MFMAs of the
    // trips read them)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+a"(kf[ks]), "+a"(vf[ks]));
    lds_wait_all();  // the slot is item 3's from the first trip on
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

    // (what follows is computed from a lane index the compiler cannot trace back: addresses
    // worked out ahead of the loop would sit in registers through all of it)
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    // the upper query half hands its partial sums to the lower one through LDS:
    // [ksb][register][lane] floats
    float* xch = (float*)smem + ksb * (2 * DT * 16 * 64) + lane_e;
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
      const int ki = k0 + (lane_e & 31);
#pragma unroll
      for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          dkacc[i][r] = (dkacc[i][r] + xch[(i * 16 + r) * 64]) * p.scale;
          dvacc[i][r] += xch[((DT + i) * 16 + r) * 64];
        }
      if (p.rope_cos) rope_back<D, DT>(dkacc, p.rope_cos, p.rope_sin, ki, lane_e);
      // (staged in ring memory behind the exchange area; the ring is idle until the barrier below)
      constexpr uint32_t XCH = 2 * (2 * DT * 16 * 64 * 4);
      const uint32_t stage = lds0 + XCH + wave * (2 * 32 * D * 2);
      store_tile_by_rows<D, DT>(dkacc, stage, p.dk + (row0 + k0) * p.lddk + hk * D, p.lddk, lane_e);
      store_tile_by_rows<D, DT>(dvacc, stage + 32 * D * 2, p.dv + (row0 + k0) * p.lddv + hk * D, p.lddv, lane_e);
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
