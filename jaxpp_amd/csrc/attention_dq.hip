// dQ of the attention backward (see attention.hip for the conventions), and the row term
// delta = sum(dO * O) that the dK/dV kernel behind it consumes.  One wave per SIMD, 64 queries
// per wave: every K / V fragment read from LDS feeds two MFMAs (one per 32-query tile), and
// a 64-key block fetched into LDS serves 256 queries.  The kernel is software-pipelined by
// hand: the matrix products of the tiles before and after run under the elementwise
// arithmetic of the tile in the middle.
#include <type_traits>

#include "attention_common.h"

namespace jpp_attn {
namespace {

// ---------------------------------------------------------------------------
// A workgroup owns 256 queries of one head, wave w queries 64 w .. +63 as two tiles of 32
// (qt = 0, 1), and walks the 64-key blocks that see them; the blocks travel HBM -> LDS
// through a ring of four slots, fetched three ahead.  A block is four tiles (kt, qt) of 32
// keys x 32 queries, taken in the order a = (0,0), b = (0,1), c = (1,0), d = (1,1); per tile
//   1. S^T = K Q^T, dP^T = V dO^T                         (16 MFMAs at head 128)
//   2. dS^T = exp2(S^T - lse) (dP^T - delta)              (elementwise)
//   3. dQ^T += K^T dS^T                                   (8 MFMAs)
// and one trip issues the MFMAs of 3 of the tile before and of 1 of the tile after, one at a
// time, with a share of 2 of the tile in the middle and of the trip's loads behind each: a
// wave issues in order, and an MFMA that finds the matrix core busy (32 cycles per MFMA)
// holds back whatever follows it, so two MFMAs in a row would stall the wave while nothing
// else issues.  The K / V row fragments of a 32-key tile stay in registers for its two query
// tiles, and so do its transposed K fragments; they are replaced, register by register,
// behind the MFMAs that read them last.  The softmax scale that belongs on dS is applied to
// the finished dQ.
//
// Under the mask a wave's last block is the one on its diagonal (tile c unseen, a and d
// masked elementwise); it then only helps to fetch for the waves behind it.
// ---------------------------------------------------------------------------
template <int D, bool CAUSAL>
__global__ __launch_bounds__(256, 1) void attn_bwd_dq_kernel(AttnParams p) {
  constexpr int KS = D / 16, DT = D / 32;
  constexpr int TILE = D * 128;            // bytes of a [64][D] tile
  constexpr int SLOT = 2 * TILE;           // K tile, V tile
  constexpr int NLOAD = 4 * (D / 64);      // wave-level loads per wave and block
  constexpr int EPG = 16 / KS;             // elements per pair of score MFMAs
  extern __shared__ __align__(1024) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const Work w = xcd_work();
  const int qb = CAUSAL ? (gridDim.x - 1 - w.x) : w.x;  // heavy blocks first
  const int h = w.h, b = w.b;
  const int hk = h / (p.n_heads / p.n_kv_heads);
  const long row0 = (long)b * p.seq;
  const int q0 = qb * 256 + wave * 64;
  const bool active = q0 < p.seq;          // a sequence of an odd number of 128 rows ends early
  const int nblk = CAUSAL ? min(qb * 256 + 256, p.seq) / 64 : p.seq / 64;
  const int my_last = !active ? -1 : CAUSAL ? q0 / 64 : nblk - 1;
  const float sc = p.scale * kLog2e;
  const uint32_t lds0 = lds_address(smem);

  const bf16_t* kbase = p.k + row0 * p.ldk + hk * D;
  const bf16_t* vbase = p.v + row0 * p.ldv + hk * D;
  Tile64::Offsets offk, offv;
  Tile64::offsets(offk, p.ldk, wave, lane);
  Tile64::offsets(offv, p.ldv, wave, lane);

  // Per-lane parts of the LDS addresses, in bytes from the start of a slot (a block's K tile,
  // then its V tile).  Row fragment (tile t, key tile kt, step ks):
  //   t TILE + (ks >> 2) 8192 + kt 4096 + (a_row ^ (ks & 3) << 5)
  // (the chunk 2 (ks & 3) + lane / 32 enters the swizzle by XOR, and 2 (ks & 3) has bit 0 clear).
  // Transposed K fragment (columns 32 i.., key tile kt, steps 2 kt + h2, half hi) - what
  // slab_frag_tr() reads, the address split into the lane's part and the rest:
  //   (i >> 1) 8192 + kt 4096 + h2 2048 + hi 1024 + (a_tr ^ ((i & 1) ^ hi) << 6)
  const uint32_t a_row = lds0 + (uint32_t)slab_off(lane & 31, lane >> 5);
  uint32_t a_tr;
  {
    const int g = lane >> 4, s = lane & 15;
    a_tr = lds0 + (uint32_t)(((s & 1) << 3) + slab_off(((g >> 1) << 2) + (s >> 2), ((g & 1) << 1) + ((s & 3) >> 1)));
  }
  typedef __attribute__((address_space(3))) const bf16x8* lds_frag;
  typedef __attribute__((address_space(3))) s16x4* lds_s16x4;

  // The fetch cursor: the K / V rows of the block that is fetched next, advanced block by block
  // and left on the last one (every trip of the loop issues the same number of loads: the
  // waits below count them).  Part j of a block's loads goes to `dst` + its place in the slot;
  // the source of a tile's second 64-column slab is an immediate offset.
  uint64_t f_k = uniform_u64((uint64_t)kbase), f_v = uniform_u64((uint64_t)vbase);
  const uint64_t f_dk = (uint64_t)p.ldk * 128, f_dv = (uint64_t)p.ldv * 128;  // bytes per 64 rows
  int f_left = nblk - 1;
  const uint32_t lds_w = lds0 + wave * (Tile64::INSTS * 1024);
  auto fetch_part = [&](uint32_t dst, auto j_c) __attribute__((always_inline)) {
    constexpr int J = decltype(j_c)::value;
    constexpr int PER = Tile64::INSTS;  // loads per wave and 64-column slab
    constexpr int t = J / (PER * (D / 64)), c = (J / PER) % (D / 64), k = J % PER;
    dma_load16_at<t * TILE + c * 8192 + k * 1024, c * 128>(t ? f_v : f_k, (t ? offv : offk)[k], dst);
  };
  auto fetch_advance = [&]() __attribute__((always_inline)) {
    const bool go = f_left > 0;
    f_left -= go ? 1 : 0;
    f_k += go ? f_dk : 0;
    f_v += go ? f_dv : 0;
  };
  auto fetch = [&](int slot) __attribute__((always_inline)) {
    const uint32_t dst = lds_w + (uint32_t)slot * SLOT;
    static_for<0, NLOAD>([&](auto j_c) __attribute__((always_inline)) { fetch_part(dst, j_c); });
    fetch_advance();
  };
  // This wave's Q and dO as MFMA operands (accumulation registers), and per query tile the
  // row's log-sum-exp (exp2 domain) and delta = sum_d dO * O: a lane holds half of its row of
  // dO (the chunks the fragments give it) and the same half of O, the other half is with
  // lane ^ 32.  The wave's 64 rows of Q, dO and O come through LDS, one after the other
  // through 64 * D * 2 bytes that only this wave uses (half of the ring's last slot, or of a
  // slot's worth of LDS behind the ring), as the swizzled slabs slabs_frag() reads: a fragment
  // taken from HBM directly touches 32 rows with 32 bytes each, and the CU's path to memory
  // takes such a load line by line (the three tensors that way: 19 k cycles per workgroup).
  // One load instruction brings 8 rows x 128 bytes; which 16 bytes a lane brings depends on
  // the row's swizzle, which differs between even and odd groups of 8 rows by chunk bit 2.
  const uint32_t stg_off = (wave < 2 ? 3 * SLOT : 4 * SLOT) + (wave & 1) * (SLOT / 2);
  auto stage_rows = [&](const bf16_t* base, long ld) __attribute__((always_inline)) {
    const int r8 = lane >> 3, c_e = (lane & 7) ^ slab_swz(r8);
    const uint32_t off_e = (uint32_t)(r8 * ld * 2 + (c_e << 4)), off_o = (uint32_t)(r8 * ld * 2 + ((c_e ^ 4) << 4));
    uint64_t src = uniform_u64((uint64_t)base);
    const uint64_t step = (uint64_t)ld * 16;  // 8 rows
    static_for<0, 8>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value;
      static_for<0, D / 64>([&](auto c_c) __attribute__((always_inline)) {
        constexpr int c = decltype(c_c)::value;
        dma_load16_at<c * 8192 + i * 1024, c * 128>(src, (i & 1) ? off_o : off_e, lds0 + stg_off);
      });
      src += step;
    });
  };
  auto staged_frag = [&](int qt, int ks) __attribute__((always_inline)) {
    return slabs_frag<D>(smem + stg_off, qt * 32, ks, lane);
  };
  bf16x8 qf[2][KS], dof[2][KS];
  uint4 ov[2][KS];
  float lse2[2] = {0.f, 0.f}, dlt[2] = {0.f, 0.f};
  const long rows = row0 + q0;
  if (active) {
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
      lse2[qt] = p.lse[((long)b * p.n_heads + h) * p.seq + q0 + qt * 32 + (lane & 31)];
    stage_rows(p.q + rows * p.ldq + h * D, p.ldq);
  }
  // the first three key blocks are on their way while this wave's own operands arrive
  fetch(0);
  fetch(1);
  fetch(2);
  if (active) {
    dma_wait<3 * NLOAD>();  // Q is in (loads complete in order)
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) qf[qt][ks] = staged_frag(qt, ks);
    lds_wait_all();
    stage_rows(p.d_o + rows * p.lddo + h * D, p.lddo);
    dma_wait_all();
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) dof[qt][ks] = staged_frag(qt, ks);
    lds_wait_all();
    stage_rows(p.o + rows * p.ldo + h * D, p.ldo);
    dma_wait_all();
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ov[qt][ks] = __builtin_bit_cast(uint4, staged_frag(qt, ks));
    lds_wait_all();  // (the ring's last slot is block 3's from the first trips on)
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
      const long stat = ((long)b * p.n_heads + h) * p.seq + q0 + qt * 32 + (lane & 31);
      lse2[qt] *= kLog2e;
      float acc = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        float of[8], gf[8];
        unpack8(ov[qt][ks], of);
        unpack8(__builtin_bit_cast(uint4, dof[qt][ks]), gf);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc = fmaf(of[e], gf[e], acc);
      }
      acc += __shfl_xor(acc, 32);
      dlt[qt] = acc;
      // for the dK/dV kernel, in the form it consumes: per 64 rows, -delta[64] then lse[64]
      if (lane < 32) {
        float* st = p.delta + 2 * (stat & ~63L) + (stat & 63);  // (seq is a multiple of 64)
        st[0] = -acc;
        st[64] = lse2[qt];
      }
    }
  } else {
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int e = 0; e < 8; ++e) { qf[qt][ks][e] = (__bf16)0.f; dof[qt][ks][e] = (__bf16)0.f; }
  }
  // (names where the fragments live from here on)
#pragma unroll
  for (int qt = 0; qt < 2; ++qt)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+a"(qf[qt][ks]), "+a"(dof[qt][ks]));
  settle(lse2[0]); settle(lse2[1]); settle(dlt[0]); settle(dlt[1]);
  // dP - delta comes out of the matrix core: one more MFMA per tile adds, to every key's row
  // of dP^T, the queries' -delta - as the product of a [keys x 16] operand of ones in three
  // columns with a [16 x queries] operand that holds -delta in those three rows, split into
  // three bf16 terms (24 bits of it)
  bf16x8 ones_f, nd_f[2];
#pragma unroll
  for (int e = 0; e < 8; ++e) ones_f[e] = (__bf16)((lane < 32 && e < 3) ? 1.f : 0.f);
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    const float nd = -dlt[qt];
    const __bf16 hi = (__bf16)nd;
    const __bf16 mid = (__bf16)(nd - (float)hi);
    const __bf16 lo = (__bf16)(nd - (float)hi - (float)mid);
#pragma unroll
    for (int e = 0; e < 8; ++e) nd_f[qt][e] = (__bf16)0.f;
    if (lane < 32) { nd_f[qt][0] = hi; nd_f[qt][1] = mid; nd_f[qt][2] = lo; }
  }

  f32x16 dqacc[2][DT];
#pragma unroll
  for (int qt = 0; qt < 2; ++qt)
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) dqacc[qt][i][r] = 0.f;

  // state of the pipeline between trips
  bf16x8 kfr[KS], vfr[KS];   // K / V rows of the 32-key tile whose scores come next
  bf16x8 ktr[2][DT];         // transposed K of the 32-key tile whose dQ products come next
  bf16x8 dsf_x[2], dsf_y[2]; // dS^T of the tile whose dQ products come next (two sets alternate)
  f32x16 s_a, dp_a, s_b, dp_b;  // scores of the query tiles 0 / 1
#pragma unroll
  for (int h2 = 0; h2 < 2; ++h2) {
#pragma unroll
    for (int e = 0; e < 8; ++e) { dsf_x[h2][e] = (__bf16)0.f; dsf_y[h2][e] = (__bf16)0.f; }
#pragma unroll
    for (int i = 0; i < DT; ++i) ktr[h2][i] = dsf_x[h2];
  }

  // Masks the scores of tile (kt, qt) of `block` just computed: on the wave's diagonal block
  // tile c is unseen and a, d see the keys at or before each query; blocks behind it are not
  // this wave's.
  auto mask = [&](f32x16& s, int block, int kt, int qt) __attribute__((always_inline)) {
    if (!CAUSAL || block < my_last) return;
    if (block > my_last || kt > qt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = -INFINITY;
    } else if (kt == qt) {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if ((r >> 2) * 8 + (lane >> 5) * 4 + (r & 3) > (lane & 31)) s[r] = -INFINITY;
    }
  };

  // One trip.  QP / QC / QN: query tile of the tile before / in the middle / after.  TR:
  // behind their last use the transposed fragments are replaced by those of key tile TR_KT of
  // the K tile whose address registers are b_tr; ROW: likewise the row fragments, by those of
  // key tile ROW_KT of the K / V tiles whose address registers are b_row.  CALC: which address
  // registers this trip works out behind its first MFMAs (1: b_tr and b_row from slot offset
  // `o`; 2: b_row).  PART0: with NLOAD / 4 loads of the block to `dst` per trip, this trip's first
  // (a trip without TR issues its own and those of the trip before it).  dS of
  // the tile in the middle leaves in ds_out; the dQ products of the tile before read ds_in.
  // The statements below are issued in the order they are written (MFMAs and elementwise
  // instructions are volatile asm statements, LDS reads do not cross the MFMAs).  Of the
  // elementwise work on a pair of elements,
  //   dS = exp2(S sc - lse) (dP - delta),
  // three MFMAs share the nine instructions so that each sees at most one exponential (16
  // cycles, the others 4 to 8) and no instruction reads the result of the one before it.
  auto trip = [&](auto qp_c, auto qc_c, auto qn_c, auto tr_c, auto row_c, auto tr_kt_c, auto row_kt_c,
                  auto calc_c, auto part0_c, uint32_t o, uint32_t dst, uint32_t (&b_tr)[2],
                  uint32_t (&b_row)[4], f32x16& s_c, f32x16& dp_c, f32x16& s_n, f32x16& dp_n,
                  const bf16x8 (&ds_in)[2], bf16x8 (&ds_out)[2]) __attribute__((always_inline)) {
    constexpr int QP = decltype(qp_c)::value, QC = decltype(qc_c)::value,
                  QN = decltype(qn_c)::value;
    constexpr bool TR = decltype(tr_c)::value, ROW = decltype(row_c)::value;
    constexpr int TR_KT = decltype(tr_kt_c)::value, ROW_KT = decltype(row_kt_c)::value;
    constexpr int CALC = decltype(calc_c)::value, PART0 = decltype(part0_c)::value;
    constexpr int PARTS = NLOAD / 4;
    constexpr int NSLOT = 2 * DT + 1 + 2 * KS;  // MFMAs of the trip
    const float sc_l = sc, lse_l = lse2[QC];
    float t0, t1, p0, p1, d0, d1;
    uint32_t dw[8];
    auto arg = [&](float& t, int r) __attribute__((always_inline)) {
      asm volatile("v_fma_f32 %0, %1, %2, -%3" : "=v"(t) : "v"(s_c[r]), "s"(sc_l), "v"(lse_l));
    };
    // step 3 g + ph of the elementwise work on elements 2 g, 2 g + 1 (dp_c holds dP - delta)
    auto step = [&](int stp) __attribute__((always_inline)) {
      const int g = stp / 3, ph = stp % 3, r = 2 * g;
      if (ph == 0) {
        asm volatile("v_exp_f32 %0, %1" : "=v"(p0) : "v"(t0));  // exp2(-inf) = 0 where masked
        if (g > 0) asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(dw[g - 1]) : "v"(d0), "v"(d1));
      } else if (ph == 1) {
        asm volatile("v_exp_f32 %0, %1" : "=v"(p1) : "v"(t1));
        asm volatile("v_mul_f32 %0, %1, %2" : "=v"(d0) : "v"(p0), "v"(dp_c[r]));
      } else {
        asm volatile("v_mul_f32 %0, %1, %2" : "=v"(d1) : "v"(p1), "v"(dp_c[r + 1]));
        if (g < 7) { arg(t0, r + 2); arg(t1, r + 3); }
      }
    };
#pragma unroll
    for (int m = 0; m < NSLOT; ++m) {
      if (m < 2 * DT) {
        // dQ products of the tile before
        const int h2 = m / DT, i = m % DT;
        mfma_avv(dqacc[QP][i], ktr[h2][i], ds_in[h2]);
        if (m == 0) { arg(t0, 0); arg(t1, 1); }
        // (slot offsets are multiples of 1024: adding them commutes with the XORs)
        if (CALC == 1 && m == 0) {
          b_tr[0] = a_tr + o;
          b_tr[1] = b_tr[0] ^ 64;
          asm volatile("" : "+v"(b_tr[0]), "+v"(b_tr[1]));
        }
        if (CALC != 0 && m == 1) {
          b_row[0] = a_row + o;
#pragma unroll
          for (int k = 1; k < 4; ++k) b_row[k] = b_row[0] ^ (k << 5);
          asm volatile("" : "+v"(b_row[0]), "+v"(b_row[1]), "+v"(b_row[2]), "+v"(b_row[3]));
        }
        if (TR) {
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4)(uintptr_t)(
              b_tr[i & 1] + ((i >> 1) * 8192 + TR_KT * 4096 + h2 * 2048)));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4)(uintptr_t)(
              b_tr[(i & 1) ^ 1] + ((i >> 1) * 8192 + TR_KT * 4096 + h2 * 2048 + 1024)));
          ktr[h2][i] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
        // the block's loads go out in the trips that read nothing from LDS, half in each (3 %
        // of the kernel against a quarter in every trip)
        if constexpr (!TR) if (m < 2 * PARTS)
          static_for<0, 2 * PARTS>([&](auto q_c) __attribute__((always_inline)) {
            if (decltype(q_c)::value == m)
              fetch_part(dst, std::integral_constant<int, PART0 - PARTS + decltype(q_c)::value>{});
          });
      } else if (m == 2 * DT) {
        // -delta of the tile after's queries: where its dP products start from
        mfma_vvv_first(dp_n, ones_f, nd_f[QN]);
      } else {
        // scores of the tile after
        const int ks = (m - 2 * DT - 1) >> 1;
        if ((m - 2 * DT - 1) & 1) {
          mfma_vva(dp_n, vfr[ks], dof[QN][ks]);
          if (ROW) vfr[ks] = *(lds_frag)(uintptr_t)(b_row[ks & 3] + (TILE + (ks >> 2) * 8192 + ROW_KT * 4096));
        } else {
          if (ks == 0) mfma_vva_first(s_n, kfr[0], qf[QN][0]);
          else mfma_vva(s_n, kfr[ks], qf[QN][ks]);
          if (ROW) kfr[ks] = *(lds_frag)(uintptr_t)(b_row[ks & 3] + ((ks >> 2) * 8192 + ROW_KT * 4096));
        }
      }
#pragma unroll
      for (int stp = m * 24 / NSLOT; stp < (m + 1) * 24 / NSLOT; ++stp) step(stp);
    }
    asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(dw[7]) : "v"(d0), "v"(d1));
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      const u32x4 dv = {dw[4 * h2], dw[4 * h2 + 1], dw[4 * h2 + 2], dw[4 * h2 + 3]};
      ds_out[h2] = __builtin_bit_cast(bf16x8, dv);
    }
    // The compiler does not know that the asm statements above are MFMAs, whose results take
    // 11 issue slots to land: whatever it does with the new scores (copies included) has to
    // wait behind this statement, which the elementwise work behind the last MFMA (three
    // instructions or more, and the one above) and eight idle slots keep clear.
    asm volatile("s_nop 7" : "+v"(s_n), "+v"(dp_n));
  };

  using T = std::true_type;
  using F = std::false_type;
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  constexpr int PARTS = NLOAD / 4;
  static_assert(PARTS >= 1 && PARTS <= 2 && PARTS <= 2 * DT, "a trip issues one or two loads");
  // The four trips of block j (tiles a, b in s_a, s_b; then c, d).  TAIL: the scores computed
  // here may need the mask (the wave's last block and the one before it).
  uint32_t b_tr[2] = {0, 0}, b_row[4] = {0, 0, 0, 0};
  auto block_trips = [&](auto tail, int j) __attribute__((always_inline)) {
    constexpr bool TAIL = decltype(tail)::value;
    // this block's slot (transposed fragments, row fragments of its second key tile), the next
    // block's (row fragments of its first key tile), and where block j + 3 goes
    uint32_t o0 = (uint32_t)(j & 3) * SLOT, o1 = (uint32_t)((j + 1) & 3) * SLOT;
    uint32_t dst = lds_w + (uint32_t)((j + 3) & 3) * SLOT;
    asm volatile("" : "+s"(o0), "+s"(o1), "+s"(dst));
    // a in the middle: dQ of d of the block before (its transposed fragments give way to
    // this block's first key tile), scores of b (the row fragments give way to the second
    // key tile's)
    trip(I1{}, I0{}, I1{}, T{}, T{}, I0{}, I1{}, I1{}, std::integral_constant<int, 0 * PARTS>{}, o0, dst,
         b_tr, b_row, s_a, dp_a, s_b, dp_b, dsf_x, dsf_y);
    if (TAIL) mask(s_b, j, 0, 1);
    // b in the middle: dQ of a, scores of c
    trip(I0{}, I1{}, I0{}, F{}, F{}, I0{}, I0{}, I0{}, std::integral_constant<int, 1 * PARTS>{}, o0, dst,
         b_tr, b_row, s_b, dp_b, s_a, dp_a, dsf_y, dsf_x);
    if (TAIL) mask(s_a, j, 1, 0);
    // c in the middle: dQ of b (transposed fragments: second key tile moves in), scores of d
    // (row fragments: the next block's first key tile moves in)
    trip(I1{}, I0{}, I1{}, T{}, T{}, I1{}, I0{}, I2{}, std::integral_constant<int, 2 * PARTS>{}, o1, dst,
         b_tr, b_row, s_a, dp_a, s_b, dp_b, dsf_x, dsf_y);
    if (TAIL) mask(s_b, j, 1, 1);
    // d in the middle: dQ of c, scores of the next block's a
    trip(I0{}, I1{}, I0{}, F{}, F{}, I0{}, I0{}, I0{}, std::integral_constant<int, 3 * PARTS>{}, o1, dst,
         b_tr, b_row, s_b, dp_b, s_a, dp_a, dsf_y, dsf_x);
    if (TAIL) mask(s_a, j + 1, 0, 0);
    fetch_advance();
  };

  dma_wait<NLOAD>();   // blocks 0 and 1 are in (block 2 may be on its way)
  __syncthreads();
  if (active) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kfr[ks] = slabs_frag<D>(smem, 0, ks, lane);
      vfr[ks] = slabs_frag<D>(smem + TILE, 0, ks, lane);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks == 0) {
        mfma_vva_first(s_a, kfr[0], qf[0][0]);
        mfma_vvv_first(dp_a, ones_f, nd_f[0]);
        mfma_vva(dp_a, vfr[0], dof[0][0]);
      } else {
        mfma_vva(s_a, kfr[ks], qf[0][ks]);
        mfma_vva(dp_a, vfr[ks], dof[0][ks]);
      }
    }
    asm volatile("s_nop 15" : "+v"(s_a), "+v"(dp_a));
    mask(s_a, 0, 0, 0);
  }

  // end of a block: this wave has read all it needs of block j's slot, and its share of block
  // j + 2 has landed (j + 3 may be on its way)
  auto block_end = [&]() __attribute__((always_inline)) {
    lds_wait_all();
    dma_wait<NLOAD>();
    __syncthreads();
  };
  // three loops in a row rather than one with a three-way choice per block: no register
  // state has to be reconciled between the variants
  int j = 0;
  const int first_tail = CAUSAL ? my_last - 1 : my_last + 1;
  for (; j < first_tail; ++j) {
    block_trips(F{}, j);
    block_end();
  }
  for (; j <= my_last; ++j) {
    block_trips(T{}, j);
    if (j == my_last) {
      // dQ of the wave's last tile
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
        for (int i = 0; i < DT; ++i) mfma_avv(dqacc[1][i], ktr[h2][i], dsf_x[h2]);
    }
    block_end();
  }
  if (!CAUSAL && active) {
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
      for (int i = 0; i < DT; ++i) mfma_avv(dqacc[1][i], ktr[h2][i], dsf_x[h2]);
  }
  for (; j < nblk; ++j) {
    fetch((j + 3) & 3);  // its share of the loads for the waves still at work
    block_end();
  }
  // every wave's loads have landed before the ring serves as the output's staging space (the
  // last trips fetch the last block again, into slots the staging may share)
  dma_wait_all();
  __syncthreads();
  if (!active) return;

  // (the MFMAs above are asm statements: their results are settled before the compiler's
  // own code reads them)
#pragma unroll
  for (int qt = 0; qt < 2; ++qt)
#pragma unroll
    for (int i = 0; i < DT; ++i) asm volatile("s_nop 15" : "+a"(dqacc[qt][i]));
  // the softmax scale that belongs on dS
#pragma unroll
  for (int qt = 0; qt < 2; ++qt)
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) dqacc[qt][i][r] *= p.scale;
  if (p.rope_cos) {
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
      rope_back<D, DT>(dqacc[qt], p.rope_cos, p.rope_sin, q0 + qt * 32 + (lane & 31), lane);
  }
#pragma unroll
  for (int qt = 0; qt < 2; ++qt)
    store_tile_by_rows<D, DT>(dqacc[qt], lds0 + (wave * 2 + qt) * (32 * D * 2),
                              p.dq + (row0 + q0 + qt * 32) * p.lddq + h * D, p.lddq, lane);
}

}  // namespace

// dQ and the row term; grid (ceil(seq / 256), heads, batch)
int launch_dq(hipStream_t stream, const AttnParams& p, int head_dim, bool causal) {
  const dim3 grid((p.seq + 255) / 256, p.n_heads, p.batch);
#define JPP_DQ(D_, C_)                                                                  \
  do {                                                                                  \
    constexpr int LDS = 5 * 2 * D_ * 128;  /* the ring, and a slot's worth for the prologue */ \
    if (int rc = set_smem(attn_bwd_dq_kernel<D_, C_>, LDS)) return rc;                  \
    hipLaunchKernelGGL((attn_bwd_dq_kernel<D_, C_>), grid, dim3(256), LDS, stream, p);  \
  } while (0)
  if (head_dim == 64) { if (causal) JPP_DQ(64, true); else JPP_DQ(64, false); }
  else { if (causal) JPP_DQ(128, true); else JPP_DQ(128, false); }
#undef JPP_DQ
  return JPP_OK;
}

}  // namespace jpp_attn
