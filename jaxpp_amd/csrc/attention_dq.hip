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
// and one trip issues 3 of the tile before, then 1 of the tile after with 2 of the tile in
// the middle between its MFMAs.  The K / V row fragments of a 32-key tile stay in registers
// for its two query tiles, and so do its transposed K fragments; they are replaced, register
// by register, behind the last MFMAs that read them.
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

  // part j of the loads of `block` (clamped to the last one, so that every trip of the loop
  // issues the same number of loads: the waits below count them)
  auto fetch_part = [&](int block, int j) __attribute__((always_inline)) {
    const long kn = (long)min(block, nblk - 1) * 64;
    const uint32_t dst = lds0 + (block & 3) * SLOT;
    constexpr int PER = Tile64::INSTS;  // loads per wave and 64-column slab
    const int t = j / (PER * (D / 64)), c = (j / PER) % (D / 64), k = j % PER;
    const bf16_t* src = t ? vbase + kn * p.ldv : kbase + kn * p.ldk;
    dma_load16(uniform_ptr(src + c * 64), (t ? offv : offk)[k],
               dst + t * TILE + c * 8192 + (wave * PER + k) * 1024);
  };
  auto fetch = [&](int block) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < NLOAD; ++j) fetch_part(block, j);
  };
  // the first three key blocks are on their way while this wave's own operands arrive
  fetch(0);
  fetch(1);
  fetch(2);

  // This wave's Q and dO as MFMA operands (accumulation registers), and per query tile the
  // row's log-sum-exp (exp2 domain) and delta = sum_d dO * O:
  // a lane holds half of its row of dO (the chunks the fragments give it) and reads the same
  // half of O, the other half is with lane ^ 32.  All loads are issued before the first of
  // them is waited for.
  bf16x8 qf[2][KS], dof[2][KS];
  uint4 ov[2][KS];
  float lse2[2] = {0.f, 0.f}, dlt[2] = {0.f, 0.f};
  if (active) {
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
      const long r = row0 + q0 + qt * 32;
      const bf16_t* qbase = p.q + r * p.ldq + h * D;
      const bf16_t* dobase = p.d_o + r * p.lddo + h * D;
      const bf16_t* obase = p.o + r * p.ldo + h * D;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        qf[qt][ks] = global_frag(qbase, p.ldq, ks, lane);
        dof[qt][ks] = global_frag(dobase, p.lddo, ks, lane);
        ov[qt][ks] = *(const uint4*)(obase + (long)(lane & 31) * p.ldo + ks * 16 + (lane >> 5) * 8);
      }
      lse2[qt] = p.lse[((long)b * p.n_heads + h) * p.seq + q0 + qt * 32 + (lane & 31)];
    }
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
  bf16x8 dsf[2];             // dS^T of the tile whose dQ products come next
  f32x16 s_a, dp_a, s_b, dp_b;  // scores of the query tiles 0 / 1
#pragma unroll
  for (int h2 = 0; h2 < 2; ++h2) {
#pragma unroll
    for (int e = 0; e < 8; ++e) dsf[h2][e] = (__bf16)0.f;
#pragma unroll
    for (int i = 0; i < DT; ++i) ktr[h2][i] = dsf[h2];
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
  // behind their last use the transposed fragments are replaced by those of key tile `tr_kt`
  // of the K tile at `tr_src`; ROW: likewise the row fragments, by those of key tile
  // `row_kt` of the K / V tiles at `row_src`.  `part0`: first of the NLOAD / 4 loads of block
  // `fetch_block` issued in this trip.  The order of the instructions below is the order they
  // are issued in: a wave issues in order, and an MFMA that finds the matrix core busy holds
  // back whatever follows it, so loads and elementwise work sit between the MFMAs.
  auto trip = [&](auto qp_c, auto qc_c, auto qn_c, auto tr_c, auto row_c, const uint8_t* tr_src,
                  int tr_kt, const uint8_t* row_src, int row_kt, int fetch_block, int part0,
                  f32x16& s_c, f32x16& dp_c, f32x16& s_n, f32x16& dp_n) __attribute__((always_inline)) {
    constexpr int QP = decltype(qp_c)::value, QC = decltype(qc_c)::value,
                  QN = decltype(qn_c)::value;
    constexpr bool TR = decltype(tr_c)::value, ROW = decltype(row_c)::value;
    constexpr int PARTS = NLOAD / 4;
    // dQ products of the tile before
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
      for (int i = 0; i < DT; ++i) {
        mfma_avv(dqacc[QP][i], ktr[h2][i], dsf[h2]);
        if (TR) ktr[h2][i] = slab_frag_tr(tr_src, 64, i * 32, 2 * tr_kt + h2, lane);
        if (h2 * DT + i < PARTS) fetch_part(fetch_block, part0 + h2 * DT + i);
      }
    // scores of the tile after, two MFMAs at a time, with dS of EPG elements of the tile in
    // the middle behind each pair
    uint32_t dw[8];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks == 0) {
        mfma_vva_first(s_n, kfr[0], qf[QN][0]);
        mfma_vva_first(dp_n, vfr[0], dof[QN][0]);
      } else {
        mfma_vva(s_n, kfr[ks], qf[QN][ks]);
        mfma_vva(dp_n, vfr[ks], dof[QN][ks]);
      }
      if (ROW) {
        kfr[ks] = slabs_frag<D>(row_src, row_kt * 32, ks, lane);
        vfr[ks] = slabs_frag<D>(row_src + TILE, row_kt * 32, ks, lane);
      }
#pragma unroll
      for (int r = ks * EPG; r < ks * EPG + EPG; r += 2) {
        float s0 = s_c[r], s1 = s_c[r + 1], g0 = dp_c[r], g1 = dp_c[r + 1];
        asm volatile("" : "+v"(s0), "+v"(s1), "+v"(g0), "+v"(g1));
        const float p0 = fast_exp2(fmaf(s0, sc, -lse2[QC]));  // exp2(-inf) = 0 where masked
        const float p1 = fast_exp2(fmaf(s1, sc, -lse2[QC]));
        dw[r >> 1] = pack2(p0 * (g0 - dlt[QC]), p1 * (g1 - dlt[QC]));
        asm volatile("" : "+v"(dw[r >> 1]));
      }
    }
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      const u32x4 dv = {dw[4 * h2], dw[4 * h2 + 1], dw[4 * h2 + 2], dw[4 * h2 + 3]};
      dsf[h2] = __builtin_bit_cast(bf16x8, dv);
    }
    // The compiler does not know that the asm statements above are MFMAs, whose results take
    // 11 issue slots to land: whatever it does with the new scores (copies included) has to
    // wait behind this statement, which the elementwise work of the last MFMA pair (nine
    // instructions and more, tied in front of it) and four idle slots keep clear.
    asm volatile("s_nop 3" : "+v"(s_n), "+v"(dp_n));
  };

  using T = std::true_type;
  using F = std::false_type;
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  constexpr int PARTS = NLOAD / 4;
  // The four trips of block j (tiles a, b in s_a, s_b; then c, d).  TAIL: the scores computed
  // here may need the mask (the wave's last block and the one before it).
  auto block_trips = [&](auto tail, int j) __attribute__((always_inline)) {
    constexpr bool TAIL = decltype(tail)::value;
    const uint8_t* sl = smem + (j & 3) * SLOT;
    const uint8_t* sl1 = smem + ((j + 1) & 3) * SLOT;
    // a in the middle: dQ of d of the block before (its transposed fragments give way to
    // this block's first key tile), scores of b (the row fragments give way to the second
    // key tile's)
    trip(I1{}, I0{}, I1{}, T{}, T{}, sl, 0, sl, 1, j + 3, 0 * PARTS, s_a, dp_a, s_b, dp_b);
    if (TAIL) mask(s_b, j, 0, 1);
    // b in the middle: dQ of a, scores of c
    trip(I0{}, I1{}, I0{}, F{}, F{}, sl, 0, sl, 0, j + 3, 1 * PARTS, s_b, dp_b, s_a, dp_a);
    if (TAIL) mask(s_a, j, 1, 0);
    // c in the middle: dQ of b (transposed fragments: second key tile moves in), scores of d
    // (row fragments: the next block's first key tile moves in)
    trip(I1{}, I0{}, I1{}, T{}, T{}, sl, 1, sl1, 0, j + 3, 2 * PARTS, s_a, dp_a, s_b, dp_b);
    if (TAIL) mask(s_b, j, 1, 1);
    // d in the middle: dQ of c, scores of the next block's a
    trip(I0{}, I1{}, I0{}, F{}, F{}, sl, 0, sl, 0, j + 3, 3 * PARTS, s_b, dp_b, s_a, dp_a);
    if (TAIL) mask(s_a, j + 1, 0, 0);
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
        mfma_vva_first(dp_a, vfr[0], dof[0][0]);
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
        for (int i = 0; i < DT; ++i) mfma_avv(dqacc[1][i], ktr[h2][i], dsf[h2]);
    }
    block_end();
  }
  if (!CAUSAL && active) {
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
      for (int i = 0; i < DT; ++i) mfma_avv(dqacc[1][i], ktr[h2][i], dsf[h2]);
  }
  for (; j < nblk; ++j) {
    fetch(j + 3);  // its share of the loads for the waves still at work
    block_end();
  }
  dma_wait_all();
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
  for (int qt = 0; qt < 2; ++qt) {
    const int qi = q0 + qt * 32 + (lane & 31);
    bf16_t* drow = p.dq + (row0 + qi) * p.lddq + h * D;
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = i * 32 + g * 8 + (lane >> 5) * 4;
        *(uint2*)(drow + d) =
            make_uint2(pack_bf16x2(dqacc[qt][i][4 * g], dqacc[qt][i][4 * g + 1]),
                       pack_bf16x2(dqacc[qt][i][4 * g + 2], dqacc[qt][i][4 * g + 3]));
      }
  }
}

}  // namespace

// dQ and the row term; grid (ceil(seq / 256), heads, batch)
int launch_dq(hipStream_t stream, const AttnParams& p, int head_dim, bool causal) {
  const dim3 grid((p.seq + 255) / 256, p.n_heads, p.batch);
#define JPP_DQ(D_, C_)                                                                  \
  do {                                                                                  \
    constexpr int LDS = 4 * 2 * D_ * 128;                                               \
    if (int rc = set_smem(attn_bwd_dq_kernel<D_, C_>, LDS)) return rc;                  \
    hipLaunchKernelGGL((attn_bwd_dq_kernel<D_, C_>), grid, dim3(256), LDS, stream, p);  \
  } while (0)
  if (head_dim == 64) { if (causal) JPP_DQ(64, true); else JPP_DQ(64, false); }
  else { if (causal) JPP_DQ(128, true); else JPP_DQ(128, false); }
#undef JPP_DQ
  return JPP_OK;
}

}  // namespace jpp_attn
