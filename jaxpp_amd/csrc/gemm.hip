// bf16 GEMM on gfx950 matrix cores (v_mfma_f32_16x16x32_bf16), operand tiles staged through
// LDS, with the epilogues a pipeline stage needs.
//
//   C[m,n] = epilogue( sum_k Aop[m,k] * Bop[n,k] )
//
// A workgroup of 4 or 8 waves owns a BM x BN output tile and walks K in steps
// of 64.  Operand tiles travel HBM -> LDS without passing through registers
// (global_load_lds_dwordx4), keeping the layout they have in HBM: an operand
// whose contraction index is contiguous in memory lands as swizzled [rows][64]
// slabs and is read back with 16-byte LDS reads; one whose contraction index
// is the slow one (the weights in a forward GEMM, both operands of a
// weight-gradient GEMM) lands as [64][rows] and is read back with the
// transposing 8-byte LDS reads (ds_read_b64_tr_b16).
//
// The weight operand is fed to the MFMA "A" port and the activation operand to
// the "B" port, so a lane ends up holding 4 consecutive n for one m; the
// epilogues regroup the tile through LDS and write whole rows.
//
// The 16x16x32 shape is chosen for what the device sustains, not for issue rate: on
// operands that change from one MFMA to the next it holds a higher clock than the
// 32x32x16 shape (2.03 against 1.82 PFLOP/s in a register-only loop; jpp_mfma_rate).
#include <math.h>
#include <stdio.h>
#include <string.h>

#include <mutex>
#include <string>

#include "common.h"

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {

struct GemmParams {
  const bf16_t* a;
  const bf16_t* b;
  // a contraction spread over several operand pairs of k elements each (see k_parts in the
  // header): pair i > 0 is (a_more[i-1], b_more[i-1]); kt_part = K-steps per pair
  const bf16_t* a_more[3];
  const bf16_t* b_more[3];
  int k_parts, kt_part;
  // JPP_GROUP_K over several pairs: row groups of pair i > 0
  const int* seg_more[3];
  const int* seg_rows_more[3];
  void* c;
  void* c2;
  const bf16_t* bias;
  const bf16_t* resid;
  const bf16_t* aux;
  int m, n, k;
  long lda, ldb, ldc, ldc2, ldresid, ldaux;
  int gelu_tanh;
  int tiles_m, tiles_n;
  // grouped (mixture-of-experts) problems: seg[0..n_seg] are row offsets, multiples of 256
  const int* seg;
  const int* seg_rows;
  int n_seg, group_mode;
  int64_t group_rows;
  long stride_b, stride_c;
  // rotary embedding in the bf16 epilogue of the forward kernels (NULL: none): columns
  // [0, rope_cols) are heads of rope_hd elements, row r is position (rope_row0 + r) % rope_seq
  const float* rope_cos;
  const float* rope_sin;
  int rope_cols, rope_seq, rope_hd;
  long rope_row0;
  // JPP_GROUP_M with a bf16 epilogue as three launches (see group_head_rows): 1 = the 256x256
  // tiles of the rows before the split, 2 / 3 = 128x128 / 128x256 tiles over the rows behind
  // it (one of the two finds work), 0 = one launch for all rows
  int tail_split;
};

// One more problem of a launch that covers several independent products of one kind (same
// orientations, epilogue, contraction length and number of operand pairs): its operands and
// its place in the grid.  Workgroups first .. first + tiles_m tiles_n - 1 work on it.
struct GemmProblem {
  const bf16_t* a[4];
  const bf16_t* b[4];
  void* c;
  long lda, ldb, ldc;
  int tiles_m, tiles_n, first;
};
// kernel arguments: one problem, or (MP) up to four
template <bool MP>
struct GemmArgs {
  GemmParams p;
};
template <>
struct GemmArgs<true> {
  GemmParams p;          // problem 0 and everything the problems share
  GemmProblem more[3];   // problems 1..3; `first` past the grid for those not in use
};

// erf(u / sqrt 2) and exp(-u^2 / 2) for the exact GELU and its derivative: the rational
// approximation 7.1.26 of Abramowitz & Stegun (one reciprocal, one exponential, five fused
// multiply-adds; absolute error 6e-7 in fp32, that of a float erf 1e-7 - either is three
// orders below half a bf16 ulp of the results, and on bf16-valued N(0, 1.5) inputs as many
// of the rounded results differ from a float64 evaluation's as with the library's erff: 2e-3
// of gelu's - tiny values of the negative tail -, 4e-4 of its derivative's).  The library
// call costs about 35 instructions, and an epilogue of a 256 x 256 tile makes 128 of them per
// lane: 17 - 23 us of a 52 - 58 us GEMM at 4096 x 4096 x 1024.
__device__ __forceinline__ void erf_and_gauss(float u, float& erf_x, float& gauss) {
  const float ax = fabsf(u) * 0.7071067811865476f;
  const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, ax, 1.0f));
  gauss = __expf(-ax * ax);
  float poly = fmaf(1.061405429f, t, -1.453152027f);
  poly = fmaf(poly, t, 1.421413741f);
  poly = fmaf(poly, t, -0.284496736f);
  poly = fmaf(poly, t, 0.254829592f);
  erf_x = copysignf(fmaf(-poly * t, gauss, 1.0f), u);
}

__device__ __forceinline__ float gelu_f(float u, int tanh_form) {
  if (tanh_form) {
    float t = tanhf(0.7978845608028654f * (u + 0.044715f * u * u * u));
    return 0.5f * u * (1.0f + t);
  }
  float e, g;
  erf_and_gauss(u, e, g);
  return 0.5f * u * (1.0f + e);
}

__device__ __forceinline__ float gelu_grad_f(float u, int tanh_form) {
  if (tanh_form) {
    float t = tanhf(0.7978845608028654f * (u + 0.044715f * u * u * u));
    return 0.5f * (1.0f + t) +
           0.5f * u * (1.0f - t * t) * 0.7978845608028654f * (1.0f + 0.134145f * u * u);
  }
  float e, g;
  erf_and_gauss(u, e, g);
  return 0.5f * (1.0f + e) + u * g * 0.3989422804014327f;
}

// (sigmoid through the hardware reciprocal, 1 ulp: a correctly rounded division is ten
// instructions, and an epilogue evaluates 64 - 128 of these per lane)
__device__ __forceinline__ float swiglu_f(float g, float u) {
  return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u;
}
__device__ __forceinline__ void swiglu_grad_f(float g, float u, float d, float& dg, float& du) {
  const float sg = __builtin_amdgcn_rcpf(1.0f + __expf(-g));
  dg = d * u * sg * (1.0f + g * (1.0f - sg));
  du = d * g * sg;
}

// Output tile of a workgroup.  Consecutive workgroup ids land on different
// XCDs (8 of them, each with its own L2); give every XCD a contiguous range of
// tiles, and inside a range walk GROUP tile-rows at a time so the B panels in
// flight stay L2 resident.
constexpr int kColumnSplitRows = 64;  // tile rows from which XCDs split by columns

template <bool WGRAD = false>
__device__ __forceinline__ void tile_of_block(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int nwg = tiles_m * tiles_n;
  if ((tiles_n & 7) == 0 && tiles_m >= kColumnSplitRows) {
    // Very tall outputs (the experts' row-grouped products: 16 384 token copies and more):
    // every XCD owns an eighth of the tile columns and walks them 8 tile-rows at a time, so a
    // B panel - which changes from expert to expert - is fetched by one XCD only.  The split
    // below would hand whole row groups to single XCDs and have each of them stream every
    // column of B (+1.3 % on the Mixtral-shaped stage and, through the 112-tile-row weight
    // gradient of its down projection, +0.8 % on the 70B-shaped one; at 16 tile-rows it costs
    // 2.5 %, at 56 it changes nothing).
    const int x = pid & 7, l = pid >> 3, cols_per = tiles_n >> 3;
    const int group = l / (8 * cols_per), within = l - group * 8 * cols_per;
    const int gsize = min(tiles_m - group * 8, 8);
    tm = group * 8 + within % gsize;
    tn = x * cols_per + within / gsize;
    return;
  }
  if ((nwg & 7) == 0) pid = (pid & 7) * (nwg >> 3) + (pid >> 3);
  // Tile rows an XCD walks at a time.  Weight gradients (both operands activations, a panel
  // 8 MiB and more) whose output is at most 16 tiles high or wide take 4: measured, A/B on
  // one box, -0.7 % on the weight-gradient launches of the Llama-3-8B- and Mixtral-shaped
  // stages (-0.2 % step time); 4 for every weight gradient cost the 70B-shaped stage 0.6 %
  // (32 x 40 .. 32 x 224 tiles), 16 for every product cost 1.8 %.
  const int GROUP = WGRAD && (tiles_m <= 16 || tiles_n <= 16) ? 4 : 8;
  const int width = GROUP * tiles_n;
  const int group = pid / width;
  const int first = group * GROUP;
  const int gsize = min(tiles_m - first, GROUP);
  tm = first + (pid % width) % gsize;
  tn = (pid % width) / gsize;
}

// Operand tile of K-step kt when the contraction runs over up to four operand pairs: pair i
// starts at K-step c_i (c_0 = 0; c_1 <= c_2 <= c_3, equal where a pair has no steps).  All
// arguments are wave-uniform.
__device__ __forceinline__ const bf16_t* part_ptr(const bf16_t* p0, const bf16_t* p1,
                                                  const bf16_t* p2, const bf16_t* p3, int kt,
                                                  int c1, int c2, int c3, long step) {
  const int part = (kt >= c1) + (kt >= c2) + (kt >= c3);
  const bf16_t* base = part == 0 ? p0 : part == 1 ? p1 : part == 2 ? p2 : p3;
  const int start = part == 0 ? 0 : part == 1 ? c1 : part == 2 ? c2 : c3;
  return base + (long)(kt - start) * step;
}
// Row-grouped products know the number of rows in use (`rows`, a multiple of 256) on the
// device only; the grid covers the buffer's capacity.  When the 256x256 tiles of those rows
// end in a round that fills at most half of the 256 CUs, the tile rows of that round are
// left to a second launch of smaller tiles: 128x128 when the round holds at most 64 tiles
// (at most one round of the small tiles, about 0.43 of the time), 128x256 when it holds up to
// 128 (one round again, about 0.6).  Returns the first row of that part (`rows` when there
// is none) and which of the two launches it belongs to (tail_split values 2 and 3).
__device__ __forceinline__ long group_head_rows(int rows, int n, int& tail_kind) {
  const int tm = rows / 256, tn = n / 256, total = tm * tn, rest = total % 256;
  const bool split = total > 256 && rest > 0 && rest <= 128 && rest % tn == 0;
  tail_kind = rest <= 64 ? 2 : 3;
  return split ? (long)(tm - rest / tn) * 256 : (long)rows;
}
// K-steps that hold data of row group e of a grouped contraction
__device__ __forceinline__ int group_steps(const int* seg, const int* seg_rows, int e) {
  const int rows = seg_rows ? min(seg_rows[e], seg[e + 1] - seg[e]) : seg[e + 1] - seg[e];
  return (rows + 63) / 64;
}

template <int BM, int BN, bool TA, bool TB, int EPI, int NW, int NS, bool KP = false, bool MP = false>
__global__ __launch_bounds__(NW * 64) void gemm_kernel(GemmArgs<MP> args) {
  GemmParams p = args.p;
  int bid = blockIdx.x;  // this workgroup's tile within its problem
  if constexpr (MP) {
    // which problem this workgroup belongs to (wave-uniform: scalar compares and selects,
    // field by field - never an index into the kernel arguments)
    const bool s1 = bid >= args.more[0].first, s2 = bid >= args.more[1].first,
               s3 = bid >= args.more[2].first;
#define JPP_PICK(own, field) \
  (s3 ? args.more[2].field : s2 ? args.more[1].field : s1 ? args.more[0].field : (own))
    p.a = JPP_PICK(p.a, a[0]);
    p.b = JPP_PICK(p.b, b[0]);
    p.a_more[0] = JPP_PICK(p.a_more[0], a[1]);
    p.a_more[1] = JPP_PICK(p.a_more[1], a[2]);
    p.a_more[2] = JPP_PICK(p.a_more[2], a[3]);
    p.b_more[0] = JPP_PICK(p.b_more[0], b[1]);
    p.b_more[1] = JPP_PICK(p.b_more[1], b[2]);
    p.b_more[2] = JPP_PICK(p.b_more[2], b[3]);
    p.c = JPP_PICK(p.c, c);
    p.lda = JPP_PICK(p.lda, lda);
    p.ldb = JPP_PICK(p.ldb, ldb);
    p.ldc = JPP_PICK(p.ldc, ldc);
    p.tiles_m = JPP_PICK(p.tiles_m, tiles_m);
    p.tiles_n = JPP_PICK(p.tiles_n, tiles_n);
    bid -= JPP_PICK(0, first);
#undef JPP_PICK
  }
  // Which waves issue the HBM -> LDS copies.  With two waves per SIMD the older one is served
  // first whenever it has an instruction ready, so it runs ahead and then waits at the
  // K-step's barrier for the younger one, whose K-step is therefore what a tile's time is made
  // of - and a wave issues in order: every copy it issues (16 cycles of the CU's path to
  // memory, longer when other waves' copies are queued) holds back its next MFMA.  So the four
  // older waves issue all copies (twice as many each) in the time they would wait anyway, and
  // the younger ones only read fragments and multiply: 2.4 - 3.3 % of the step on the Llama-
  // and Mixtral-shaped stages, 2 % on the BERT-large-shaped one (single GEMMs: TN -5 %,
  // NN / NT -2.5 % at 4096 x 28672 x 4096; two shapes of twelve +1 - 2 %).
  constexpr int DW = NW == 8 ? 4 : NW;
  using TileA = DmaTile<BM, TA, DW>;
  using TileB = DmaTile<BN, TB, DW>;
  constexpr int A_BYTES = TileA::BYTES, STAGE = TileA::BYTES + TileB::BYTES;
  constexpr int WN = NW / 2;                        // waves: 2 along m, NW/2 along n
  // 16x16 MFMA tiles per wave.  A K-step runs them in 2 HS blocks of TMH x TN (32 contraction
  // elements each); large wave tiles take the rows in two halves so that the fragments of
  // two blocks fit in registers beside the accumulators
  constexpr int TM = BM / 32, TN = BN / (16 * WN), HS = TM * TN >= 32 ? 2 : 1, TMH = TM / HS;
  constexpr int NB = 2 * HS;
  extern __shared__ __align__(1024) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  // (wave-uniform where the waves differ in what they do: a scalar branch around the copies)
  const int wave = DW == NW ? tid >> 6 : __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool dma_wave = wave < DW;
  const int wm = wave / WN, wn = wave % WN;
  int tm, tn;
  const int tiles = p.tiles_m * p.tiles_n;
  tile_of_block<TA && TB>(p.group_mode == JPP_GROUP_K ? bid % tiles : bid, p.tiles_m, p.tiles_n, tm, tn);
  long m0 = (long)tm * BM;
  const long n0 = (long)tn * BN;
  if constexpr (EPI == JPP_EPI_BF16 && !KP && !MP) {   // (the launcher splits these only)
    if (p.group_mode == JPP_GROUP_M && p.tail_split) {
      int tail_kind;
      const long head = group_head_rows(p.seg[p.n_seg], p.n, tail_kind);
      if (p.tail_split == 1 ? m0 >= head : p.tail_split != tail_kind) return;
      if (p.tail_split != 1) m0 += head;
    }
  }

  const long a_off = TA ? m0 : m0 * p.lda, b_off = TB ? n0 : n0 * p.ldb;
  const bf16_t* a_src = p.a + a_off;
  const bf16_t* b_src = p.b + b_off;
  int kt_n = p.k / 64 * (KP ? p.k_parts : 1);
  // several operand pairs: first K-step of pairs 1..3 and their operands at this tile
  int c1 = p.kt_part, c2 = 2 * p.kt_part, c3 = 3 * p.kt_part;
  const bf16_t* a1 = KP ? p.a_more[0] + a_off : a_src;
  const bf16_t* a2 = KP ? p.a_more[1] + a_off : a_src;
  const bf16_t* a3 = KP ? p.a_more[2] + a_off : a_src;
  const bf16_t* b1 = KP ? p.b_more[0] + b_off : b_src;
  const bf16_t* b2 = KP ? p.b_more[1] + b_off : b_src;
  const bf16_t* b3 = KP ? p.b_more[2] + b_off : b_src;
  if (p.group_mode == JPP_GROUP_M) {
    // rows of A and C are grouped by expert; each group multiplies its own B
    if (m0 >= p.seg[p.n_seg]) return;
    int e = 0;
    while (p.seg[e + 1] <= m0) ++e;
    b_src += (long)e * p.stride_b;
  } else if (p.group_mode == JPP_GROUP_K) {
    // one output per expert; the contraction runs over the expert's rows
    const int e = bid / tiles;
    const long r0 = p.seg[e];
    // rows past the group's data are zero padding: steps made of nothing else are skipped
    kt_n = group_steps(p.seg, p.seg_rows, e);
    a_src += r0 * p.lda;
    b_src += r0 * p.ldb;
    if constexpr (KP) {
      // every further pair brings its own row groups (pair by pair, never an index into the
      // kernel arguments); a pair past k_parts starts where the contraction ends
      c1 = c2 = c3 = kt_n;
      if (p.k_parts > 1) {
        const long r = p.seg_more[0][e];
        a1 += r * p.lda; b1 += r * p.ldb;
        kt_n += group_steps(p.seg_more[0], p.seg_rows_more[0], e);
        c2 = c3 = kt_n;
      }
      if (p.k_parts > 2) {
        const long r = p.seg_more[1][e];
        a2 += r * p.lda; b2 += r * p.ldb;
        kt_n += group_steps(p.seg_more[1], p.seg_rows_more[1], e);
        c3 = kt_n;
      }
      if (p.k_parts > 3) {
        const long r = p.seg_more[2][e];
        a3 += r * p.lda; b3 += r * p.ldb;
        kt_n += group_steps(p.seg_more[2], p.seg_rows_more[2], e);
      }
    }
    p.c = EPI == JPP_EPI_BF16 ? (void*)((bf16_t*)p.c + (long)e * p.stride_c)
                              : (void*)((float*)p.c + (long)e * p.stride_c);
    if (kt_n == 0 && EPI == JPP_EPI_ACC_F32) return;
  }
  const long a_step = TA ? 64 * p.lda : 64;
  const long b_step = TB ? 64 * p.ldb : 64;
  // operand tiles of K-step kt: with several operand pairs the steps run through pair 0,
  // then pair 1, ... (kt and the pair index are wave-uniform: scalar arithmetic; the pair
  // pointers are picked by a chain of selects, never by indexing the kernel arguments)
  // (kernels built without KP take one pair and keep the plain address arithmetic)
#define a_at(kt) (KP ? part_ptr(a_src, a1, a2, a3, (kt), c1, c2, c3, a_step) : a_src + (long)(kt) * a_step)
#define b_at(kt) (KP ? part_ptr(b_src, b1, b2, b3, (kt), c1, c2, c3, b_step) : b_src + (long)(kt) * b_step)

  // of tile (i, j) a lane holds row wm BM/2 + 16 i + lane % 16 and the four columns
  // wn BN/WN + 16 j + 4 (lane / 16) + {0..3}
  f32x4 acc[TM][TN];
  // C += A B (EPI_ACC_F32): the epilogue only stores; the fp32 tile in memory is folded into
  // the accumulators during the first K-steps.  It travels HBM -> LDS like the operands, NW
  // whole rows (BN * 4 bytes each, one per wave) at a time, into one of NS+1 buffers behind
  // the operand stages: batch b is requested at the end of K-step b, after that K-step's
  // operand copies, and read out of LDS at the wait point of K-step b+NS.  The waits in
  // between leave the youngest requests in flight (vmcnt counts in order), so a batch has
  // NS K-steps to arrive and no K-step waits for HBM on its account; reading whole rows
  // keeps HBM on long bursts where a lane-per-row layout would touch 16 rows at once.  K
  // loops too short for that add the old values in the epilogue, where rows are whole too.
  static_assert(BN * 4 <= 1024, "a row of the fp32 tile is one 64-lane copy");
  constexpr int NBT = BM / NW, C_LDS = NS * (BM + BN) * 128, C_PITCH = 1024 + 16;  // a copy is 1 KB
  const bool stream_c = EPI == JPP_EPI_ACC_F32 && kt_n >= NBT + NS;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  // byte offset, from the start of C, of this lane's 16 bytes of tile row `wave`
  // (lanes past the end of a narrow row repeat its last piece)
  const uint32_t c_off0 =
      (uint32_t)(((m0 + wave) * p.ldc + n0 + min(lane, BN / 4 - 1) * 4) * 4);
  const uint32_t lds0 = lds_address(smem);
  typename TileA::Offsets offa;
  typename TileB::Offsets offb;
  TileA::offsets(offa, p.lda, wave, lane);
  TileB::offsets(offb, p.ldb, wave, lane);
  constexpr int IA = TileA::INSTS, IB = TileB::INSTS;
  const int row_w = wn * (BN / WN), row_x = wm * (BM / 2);

  // Software pipeline over K-steps of 64 with NS LDS stages:
  //   * the HBM -> LDS copy of K-step t+NS is issued inside K-step t, right after the
  //     barrier that retires stage t % NS's readers, so it has NS-1 K-steps to land;
  //   * that barrier sits in front of the last MFMA block of a K-step and the first
  //     fragments of K-step t+1 are read from LDS behind it, under those MFMAs.
  // Block q of a K-step multiplies contraction elements 32 (q / HS) .. + 31 of the stage: the
  // wave's TN fragments of B (read once per HS blocks) with part q % HS of its TM fragments
  // of A, each fragment read while the block before it computes.
  // Waits count requests from the youngest (vmcnt is in order): at the wait point of K-step
  // t the copies of K-steps t+2 .. t+NS-1 and the accumulator rows requested during the last
  // NS-1 K-steps may stay in flight (where a stage's refill is split over two K-steps, see
  // LATE below, its second half is the youngest request and everything is waited for).
  constexpr int OPB = IA + IB;  // operand copies per wave and K-step
  bf16x8 fw[2][TN], fx[2][TMH];
  if (kt_n > 0) {
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const int k = min(s, kt_n - 1);
      if (dma_wave) {
        TileA::template issue<0, IA>(uniform_ptr(a_at(k)), offa, lds0 + s * STAGE, wave);
        TileB::template issue<0, IB>(uniform_ptr(b_at(k)), offb, lds0 + s * STAGE + A_BYTES, wave);
      }
    }
    dma_wait<(NS - 1) * OPB>();  // stage 0 has landed; the others may still be in flight
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < TN; ++j) fw[0][j] = TileB::frag16(smem + A_BYTES, row_w + j * 16, 0, lane);
#pragma unroll
  for (int i = 0; i < TMH; ++i) fx[0][i] = TileA::frag16(smem, row_x + i * 16, 0, lane);

  int st = 0;   // stage of K-step kt: kt % NS
  int cbi = 0;  // accumulator-row buffer of K-step kt: kt % (NS + 1)
  // The refill of a retired stage is 8 wave-level copies per wave, 64 per workgroup, and the
  // CU's path to memory takes one in 16 cycles: issued all behind the barrier, under the last
  // MFMA block, they kept that block waiting on the path (a wave issues in order) for twice
  // the time its MFMAs need.  With two stages the 256 x 256 tile therefore issues LATE of
  // its four parts under the first MFMA block of the next K-step instead (still three blocks
  // ahead of the wait for them): 4 - 6 % per K-step by timestamps inside the loop, 0.2 - 1 %
  // of the Llama-3-8B-shaped step depending on the device.  (3 or 4 parts late: slower again,
  // the copies land too late.)
  constexpr int LATE = (NS == 2 && BM == 256 && BN == 256 && NW == 8) ? 2 : 0;
  constexpr bool SPLIT = LATE > 0;
  const bf16_t* ga_late = nullptr;
  const bf16_t* gb_late = nullptr;
  int st_late = 0;
  for (int kt = 0; kt < kt_n; ++kt) {
    const int nst = st + 1 == NS ? 0 : st + 1;
    const uint8_t* sa = smem + st * STAGE;
    const uint8_t* sb = sa + A_BYTES;
    const uint8_t* na = smem + nst * STAGE;
    // past the end the last K-step is fetched again, unused
    const int kn = min(kt + NS, kt_n - 1);
    const bf16_t* ga = uniform_ptr(a_at(kn));
    const bf16_t* gb = uniform_ptr(b_at(kn));
#pragma unroll
    for (int ks = 0; ks < NB; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1, curw = ks / HS, part = ks % HS;
      if (ks < NB - 1) {
        if ((ks + 1) % HS == 0) {
#pragma unroll
          for (int j = 0; j < TN; ++j) fw[1][j] = TileB::frag16(sb, row_w + j * 16, 1, lane);
        }
#pragma unroll
        for (int i = 0; i < TMH; ++i)
          fx[nxt][i] = TileA::frag16(sa, row_x + ((ks + 1) % HS * TMH + i) * 16, (ks + 1) / HS, lane);
      } else {
        // every fragment of this stage is in registers: once all waves are here (and the
        // next stage has landed) this stage can be refilled
        {
          // accumulator rows requested during K-steps kt+1-NS .. kt-1 that may stay in flight
          int cin = 0;
          if (EPI == JPP_EPI_ACC_F32 && stream_c)
            cin = max(0, min(kt - 1, NBT - 1) - max(0, kt + 1 - NS) + 1);
          if (SPLIT || cin <= 0) dma_wait<(NS - 2) * OPB>();
          else if (cin == 1) dma_wait<(NS - 2) * OPB + 1>();
          else if (cin == 2) dma_wait<(NS - 2) * OPB + 2>();
          else dma_wait<(NS - 2) * OPB + 3>();
          static_assert(NS <= 4, "the wait above distinguishes up to three rows in flight");
        }
        lds_wait_all();
        __syncthreads();
        if constexpr (EPI == JPP_EPI_ACC_F32) {
          if (stream_c && kt >= NS && kt < NBT + NS) {
            // batch kt-NS (tile rows NW (kt-NS) .. + NW-1) is in LDS: the lanes that hold
            // those rows add them in.  Buffers are used round robin over NS+1, so the one
            // read here is written again only behind the next K-step's barrier.
            const int row0 = (kt - NS) * NW, rl = (lane & 15) - (row0 & 15);
            const int fold_buf = cbi + 1 == NS + 1 ? 0 : cbi + 1;  // (kt - NS) % (NS + 1)
            if (wm == row0 / (BM / 2) && rl >= 0 && rl < NW) {
              const uint8_t* src = smem + C_LDS + (fold_buf * NW + rl) * C_PITCH +
                                   (wn * (BN / WN) + (lane >> 4) * 4) * 4;
#pragma unroll
              for (int i = 0; i < TM; ++i)
                if (i == (row0 % (BM / 2)) / 16) {
#pragma unroll
                  for (int j = 0; j < TN; ++j) acc[i][j] += *(const f32x4*)(src + j * 64);
                }
            }
          }
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) fw[0][j] = TileB::frag16(na + A_BYTES, row_w + j * 16, 0, lane);
#pragma unroll
        for (int i = 0; i < TMH; ++i) fx[0][i] = TileA::frag16(na, row_x + i * 16, 0, lane);
      }
      // the refill of the retired stage is spread over this block's MFMAs: a wave that
      // issues its loads back to back waits on the memory pipeline with its MFMAs behind it
      constexpr int PARTS = TMH < IA && TMH < IB ? TMH : (IA < IB ? IA : IB);
      static_assert(IA % PARTS == 0 && IB % PARTS == 0 && TMH % PARTS == 0,
                    "loads per wave must split over the MFMA rows");
      // MFMAs go in 2x2 groups of tiles, walked so that from one MFMA to the next exactly one
      // operand changes: fewer operand bits toggle per issue than row by row, and the clock
      // under load follows the toggling (walks that change both operands at group borders,
      // whole rows, or columns first measured 0.5 - 1.2 % slower on the Llama-3-8B-shaped step)
      static_assert(TMH % 2 == 0 && TN % 2 == 0, "2x2 groups of MFMA tiles");
#pragma unroll
      for (int ib = 0; ib < TMH / 2; ++ib) {
        if (!SPLIT && ks == NB - 1) {
#pragma unroll
          for (int i = 2 * ib; i < 2 * ib + 2; ++i)
            if (i % (TMH / PARTS) == 0 && dma_wave) {
              TileA::template issue_part<IA / PARTS>(i / (TMH / PARTS), ga, offa, lds0 + st * STAGE, wave);
              TileB::template issue_part<IB / PARTS>(i / (TMH / PARTS), gb, offb,
                                                     lds0 + st * STAGE + A_BYTES, wave);
            }
        }
        if constexpr (SPLIT) {
          static_assert(!SPLIT || (PARTS == 4 && TMH == 4 && LATE >= 2 && LATE <= 4),
                        "four parts, at most two of them in the last block (it has two slots)");
          // parts 0 .. 3 - LATE in the last block (spread from its end), the others one per
          // pair of MFMA rows from the start of the next K-step on
          const int slot = ks * 2 + ib;           // pair of MFMA rows within the K-step
          if (ks == NB - 1) {
            const int part = slot - (2 * NB - (4 - LATE));
            if (part >= 0 && dma_wave) {
              TileA::template issue_part<IA / PARTS>(part, ga, offa, lds0 + st * STAGE, wave);
              TileB::template issue_part<IB / PARTS>(part, gb, offb, lds0 + st * STAGE + A_BYTES, wave);
            }
          } else if (slot < LATE && kt > 0 && dma_wave) {
            const int part = 4 - LATE + slot;
            TileA::template issue_part<IA / PARTS>(part, ga_late, offa, lds0 + st_late * STAGE, wave);
            TileB::template issue_part<IB / PARTS>(part, gb_late, offb,
                                                   lds0 + st_late * STAGE + A_BYTES, wave);
          }
        }
        // a walk over the 2 x TN tiles of this pair of rows, the next pair taking the columns in
        // the opposite direction
#pragma unroll
        for (int q = 0; q < TN / 2; ++q) {
          const int jb = ib & 1 ? TN / 2 - 1 - q : q;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            // (row, column) within the 2 x 2 group: 00 01 11 10, the next group 10 11 01 00
            const int ii = (q & 1) ? (e < 2 ? 1 : 0) : (e < 2 ? 0 : 1);
            const int jj = (e == 1 || e == 2) ? 1 : 0;
            const int i = 2 * ib + ii, j = 2 * jb + ((ib & 1) ? 1 - jj : jj);
            acc[part * TMH + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                fw[curw][j], fx[cur][i], acc[part * TMH + i][j], 0, 0, 0);
          }
        }
      }
    }
    if constexpr (EPI == JPP_EPI_ACC_F32) {
      if (stream_c && kt < NBT)
        dma_load16(uniform_ptr((const bf16_t*)p.c), c_off0 + (uint32_t)(kt * NW * p.ldc * 4),
                   lds0 + C_LDS + (cbi * NW + wave) * C_PITCH);
    }
    ga_late = ga; gb_late = gb; st_late = st;
    st = nst;
    cbi = cbi + 1 == NS + 1 ? 0 : cbi + 1;
  }
  dma_wait_all();   // the refetches of the last two K-steps must not outlive the block's LDS

  if constexpr (EPI == JPP_EPI_ACC_F32 || EPI == JPP_EPI_F32) {
    // fp32 outputs leave through LDS as well (see below), a quarter of the tile per pass:
    // 16-byte stores of contiguous rows instead of 32-byte pieces of 32 rows
    constexpr int IPP = TM / 2, RP = IPP * 16, PITCH = BN * 4 + 16, NT = NW * 64;
    constexpr int TPR = BN / 4, RPI = NT / TPR;
#pragma unroll 1
    for (int pass = 0; pass < 2 * (TM / IPP); ++pass) {
      const int half = pass / (TM / IPP), i0 = (pass % (TM / IPP)) * IPP;
      __syncthreads();
      if (wm == half) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
          if (i >= i0 && i < i0 + IPP) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
              *(f32x4*)(smem + ((i - i0) * 16 + (lane & 15)) * PITCH +
                        (wn * (BN / WN) + j * 16 + (lane >> 4) * 4) * 4) = acc[i][j];
          }
      }
      __syncthreads();
      const long mrow0 = m0 + half * (BM / 2) + i0 * 16;
      const int c4 = (tid % TPR) * 4;
      static_assert(RP % RPI == 0, "rows of a pass split evenly over the threads");
      float4 v[RP / RPI];
      if (EPI == JPP_EPI_ACC_F32 && !stream_c) {
        // a K loop too short to stream the old values in: they are read here, by rows, all of
        // a thread's rows before the first is used
        float4 old[RP / RPI];
#pragma unroll
        for (int it = 0; it < RP / RPI; ++it)
          old[it] = *(const float4*)((const float*)p.c + (mrow0 + tid / TPR + it * RPI) * p.ldc +
                                     n0 + c4);
#pragma unroll
        for (int it = 0; it < RP / RPI; ++it) {
          const float4 t = *(const float4*)(smem + (tid / TPR + it * RPI) * PITCH + c4 * 4);
          v[it] = make_float4(old[it].x + t.x, old[it].y + t.y, old[it].z + t.z, old[it].w + t.w);
        }
      } else {
#pragma unroll
        for (int it = 0; it < RP / RPI; ++it)
          v[it] = *(const float4*)(smem + (tid / TPR + it * RPI) * PITCH + c4 * 4);
      }
#pragma unroll
      for (int it = 0; it < RP / RPI; ++it) {
        float* dst = (float*)p.c + (mrow0 + tid / TPR + it * RPI) * p.ldc + n0 + c4;
        // the accumulators are not read again before the next microbatch: stored past the
        // caches they leave L2 to the operand panels (+0.4 % on the Llama-8B-shaped stage)
        if (EPI == JPP_EPI_ACC_F32)
          __builtin_nontemporal_store(f32x4{v[it].x, v[it].y, v[it].z, v[it].w}, (f32x4*)dst);
        else
          *(float4*)dst = v[it];
      }
    }
  } else {
    // bf16 outputs.  An accumulator lane holds one row and 4 consecutive columns, so storing
    // from that layout scatters 8-byte pieces over 32 rows per instruction.  Instead the tile
    // goes through LDS (free after the K loop) half at a time - fp32, [BM/2 rows][BN + 4]
    // - and is taken back out by rows: a thread owns 8 consecutive columns of a row, so
    // every global access of the epilogue (output, residual, pre-activation, gate/up) is a
    // 16-byte piece of a contiguous run, and the arithmetic runs in fp32 exactly as before.
    constexpr int HALF = BM / 2, PITCH = BN * 4 + 16, NT = NW * 64;
    const bf16_t* bias = p.bias;
#pragma unroll 1
    for (int half = 0; half < 2; ++half) {
      __syncthreads();  // fragments of the last K-step / the previous half are out of LDS
      if (wm == half) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            *(f32x4*)(smem + (i * 16 + (lane & 15)) * PITCH +
                      (wn * (BN / WN) + j * 16 + (lane >> 4) * 4) * 4) = acc[i][j];
      }
      __syncthreads();
      const long mrow0 = m0 + half * HALF;
      if constexpr (EPI == JPP_EPI_SWIGLU) {
        // a thread owns 8 features of a row: gate at columns 64q + w, up at 64q + 32 + w
        constexpr int TPR = BN / 16, RPI = NT / TPR;  // threads per row, rows per sweep
        const int fc = tid % TPR, q = fc >> 2, w = (fc & 3) * 8;
        for (int r = tid / TPR; r < HALF; r += RPI) {
          const uint8_t* row = smem + r * PITCH + (q * 64 + w) * 4;
          const float4 g0 = *(const float4*)row, g1 = *(const float4*)(row + 16);
          const float4 u0 = *(const float4*)(row + 128), u1 = *(const float4*)(row + 144);
          const uint4 gp = make_uint4(pack_bf16x2(g0.x, g0.y), pack_bf16x2(g0.z, g0.w),
                                      pack_bf16x2(g1.x, g1.y), pack_bf16x2(g1.z, g1.w));
          const uint4 up = make_uint4(pack_bf16x2(u0.x, u0.y), pack_bf16x2(u0.z, u0.w),
                                      pack_bf16x2(u1.x, u1.y), pack_bf16x2(u1.z, u1.w));
          bf16_t* crow = (bf16_t*)p.c + (mrow0 + r) * p.ldc + n0 + q * 64 + w;
          // gate and up are next read by the backward pass, many tasks later: stored past the
          // caches (their product below is the next GEMM's operand and stays cached)
          __builtin_nontemporal_store(u32x4{gp.x, gp.y, gp.z, gp.w}, (u32x4*)crow);
          __builtin_nontemporal_store(u32x4{up.x, up.y, up.z, up.w}, (u32x4*)(crow + 32));
          // from the rounded values, as a separate kernel would read them back
          float gv[8], uv[8];
          unpack8(gp, gv);
          unpack8(up, uv);
#pragma unroll
          for (int e = 0; e < 8; ++e) gv[e] = swiglu_f(gv[e], uv[e]);
          *(uint4*)((bf16_t*)p.c2 + (mrow0 + r) * p.ldc2 + n0 / 2 + q * 32 + w) = pack8(gv);
        }
      } else if constexpr (EPI == JPP_EPI_DSWIGLU) {
        // the tile holds ds for BN features; gate / up of block q at columns 64q.., 64q+32..
        constexpr int TPR = BN / 8, RPI = NT / TPR;
        const int fc = tid % TPR, q = fc >> 2, w = (fc & 3) * 8;
        for (int r = tid / TPR; r < HALF; r += RPI) {
          const uint8_t* row = smem + r * PITCH + fc * 32;
          const float4 d0 = *(const float4*)row, d1 = *(const float4*)(row + 16);
          const long col = 2 * n0 + q * 64 + w;
          const bf16_t* arow = p.aux + (mrow0 + r) * p.ldaux + col;
          float gv[8], uv[8], dv[8];
          unpack8(*(const uint4*)arow, gv);
          unpack8(*(const uint4*)(arow + 32), uv);
          unpack8(make_uint4(pack_bf16x2(d0.x, d0.y), pack_bf16x2(d0.z, d0.w),
                             pack_bf16x2(d1.x, d1.y), pack_bf16x2(d1.z, d1.w)), dv);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            float dg, du;
            swiglu_grad_f(gv[e], uv[e], dv[e], dg, du);
            gv[e] = dg;
            uv[e] = du;
          }
          bf16_t* crow = (bf16_t*)p.c + (mrow0 + r) * p.ldc + col;
          *(uint4*)crow = pack8(gv);
          *(uint4*)(crow + 32) = pack8(uv);
        }
      } else {
        constexpr int TPR = BN / 8, RPI = NT / TPR;
        const int c8 = (tid % TPR) * 8;
        float bv[8];
        if (bias) unpack8(*(const uint4*)(bias + n0 + c8), bv);
        for (int r = tid / TPR; r < HALF; r += RPI) {
          const uint8_t* row = smem + r * PITCH + c8 * 4;
          const float4 a0 = *(const float4*)row, a1 = *(const float4*)(row + 16);
          float v[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
          const long at = (mrow0 + r) * p.ldc + n0 + c8;
          if (bias) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] += bv[e];
          }
          if constexpr (EPI == JPP_EPI_BF16) {
            if (p.resid) {
              float rv[8];
              unpack8(*(const uint4*)(p.resid + (mrow0 + r) * p.ldresid + n0 + c8), rv);
#pragma unroll
              for (int e = 0; e < 8; ++e) v[e] += rv[e];
            }
            if constexpr (!TA && TB) {
              // rotary embedding of the query / key heads (forward projection): the partner
              // of a column sits half a head away in the same staged row; both are rounded to
              // bf16 first, as a pass of its own would read them back
              if (p.rope_cos && n0 + c8 < p.rope_cols) {
                const int hh = p.rope_hd >> 1, cin = (n0 + c8) & (p.rope_hd - 1);
                const bool lo = cin < hh;
                const uint8_t* prow = row + (lo ? hh : -hh) * 4;
                const float4 b0 = *(const float4*)prow, b1 = *(const float4*)(prow + 16);
                const float w[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
                const long pos = (p.rope_row0 + mrow0 + r) % p.rope_seq;
                const float* ct = p.rope_cos + pos * hh + (cin & (hh - 1));
                const float* st = p.rope_sin + pos * hh + (cin & (hh - 1));
                const float4 c0 = *(const float4*)ct, c1 = *(const float4*)(ct + 4);
                const float4 s0 = *(const float4*)st, s1 = *(const float4*)(st + 4);
                const float cs[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
                const float sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                  const float own = (float)(__bf16)v[e], other = (float)(__bf16)w[e];
                  float o1, o2;
                  rope_rotate(lo ? own : other, lo ? other : own, cs[e], sn[e], o1, o2);
                  v[e] = lo ? o1 : o2;
                }
              }
            }
          } else if constexpr (EPI == JPP_EPI_GELU) {
            float gl[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) gl[e] = gelu_f(v[e], p.gelu_tanh);
            *(uint4*)((bf16_t*)p.c2 + (mrow0 + r) * p.ldc2 + n0 + c8) = pack8(gl);
          } else if constexpr (EPI == JPP_EPI_DGELU) {
            float uv[8];
            unpack8(*(const uint4*)(p.aux + (mrow0 + r) * p.ldaux + n0 + c8), uv);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] *= gelu_grad_f(uv[e], p.gelu_tanh);
          }
          *(uint4*)((bf16_t*)p.c + at) = pack8(v);
        }
      }
    }
  }
}

#undef a_at
#undef b_at

template <int BM, int BN, bool TA, bool TB, int EPI, int NW, int NS>
const char* class_name() {
  // built once per instantiation; the initialisation of a function-local static is
  // thread-safe
  static const std::string name = [] {
    char buf[64];
    const char* lay = TA ? "tn" : (TB ? "nn" : "nt");
    const char* epi = EPI == JPP_EPI_BF16 ? "bf16" : EPI == JPP_EPI_GELU ? "gelu"
                    : EPI == JPP_EPI_DGELU ? "dgelu" : EPI == JPP_EPI_ACC_F32 ? "accf32"
                    : EPI == JPP_EPI_SWIGLU ? "swiglu" : EPI == JPP_EPI_DSWIGLU ? "dswiglu" : "f32";
    snprintf(buf, sizeof(buf), "gemm_%s_%s_%dx%d%s%s", lay, epi, BM, BN, NW == 8 ? "w8" : "",
             NS == 2 ? "" : NS == 3 ? "s3" : "s4");
    return std::string(buf);
  }();
  return name.c_str();
}

template <int BM, int BN, bool TA, bool TB, int EPI, int NW = 4, int NS = 2, bool KP = false>
int launch(hipStream_t stream, GemmParams& p) {
  // two operand stages; the bf16 epilogues stage half a tile in fp32 with padded rows
  constexpr int SMEM_LOOP = NS * (BM + BN) * 128, SMEM_EPI = (BM / 2) * (BN * 4 + 16);
  // + NS+1 buffers of NW rows of the fp32 tile (padded) for C += A B
  constexpr int SMEM = EPI == JPP_EPI_ACC_F32 ? SMEM_LOOP + (NS + 1) * NW * (1024 + 16)
                       : (EPI == JPP_EPI_F32 || SMEM_LOOP > SMEM_EPI) ? SMEM_LOOP : SMEM_EPI;
  if constexpr (!KP) {
    // several operand pairs: only the accumulating weight-gradient kernels on 256-wide tiles
    // are built for that
    if (p.k_parts > 1) {
      if constexpr (TA && TB && EPI == JPP_EPI_ACC_F32 && BN == 256 && NW == 8 && NS == 2)
        return launch<BM, BN, TA, TB, EPI, NW, NS, true>(stream, p);
      else
        return jpp_set_error(JPP_ERR_INVALID, "gemm: several operand pairs are supported for "
                             "accumulated weight gradients (tn, JPP_EPI_ACC_F32) on 256x256 and "
                             "128x256 tiles");
    }
  }
  // algorithmic extent: grouped launches count the non-padding rows when the caller gave them
  const double cb = EPI == JPP_EPI_ACC_F32 || EPI == JPP_EPI_DSWIGLU ? 8
                    : EPI == JPP_EPI_F32 ? 4 : EPI == JPP_EPI_SWIGLU ? 3 : 2;
  double am = p.m, ak = (double)p.k * (p.k_parts > 1 ? p.k_parts : 1), copies = 1;
  if (p.group_mode == JPP_GROUP_M && p.group_rows) am = p.group_rows;
  if (p.group_mode == JPP_GROUP_K) { ak = p.group_rows; copies = p.n_seg; }
  const double b_bytes = 2.0 * p.n * ak * (p.group_mode == JPP_GROUP_M ? p.n_seg : 1);
  // (the small-tile launches of a row-grouped product's last round add their time to the class
  // of its 256x256 launch, which declares the whole product's work)
  const bool tail = p.tail_split >= 2;
  ProbeScope probe(stream, tail ? class_name<256, 256, TA, TB, EPI, 8, 2>()
                                : class_name<BM, BN, TA, TB, EPI, NW, NS>(),
                   tail ? 0.0 : 2.0 * am * p.n * ak,
                   tail ? 0.0 : 2.0 * am * ak + b_bytes + copies * am * p.n * cb);
  auto kern = gemm_kernel<BM, BN, TA, TB, EPI, NW, NS, KP>;
  static_assert(SMEM <= 160 * 1024, "LDS of one CU");
  // the LDS limit of a kernel is sticky: set once per instantiation, by whichever host
  // thread launches it first (the others wait for that call and see its result)
  static std::once_flag configured;
  static hipError_t configure_rc = hipSuccess;
  std::call_once(configured, [&] {
    configure_rc = hipFuncSetAttribute((const void*)kern,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
  });
  JPP_CHECK_HIP(configure_rc);
  p.tiles_m = p.m / BM;
  p.tiles_n = p.n / BN;
  const int blocks = p.tiles_m * p.tiles_n * (p.group_mode == JPP_GROUP_K ? p.n_seg : 1);
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(NW * 64), SMEM, stream, GemmArgs<false>{p});
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

// Several accumulated weight gradients (C_i += sum_j A_ij^T B_ij) as one grid of 256x256
// tiles: problem i's tiles follow problem i-1's, so the half-filled last rounds of the single
// launches (384 or 896 tiles on 256 CUs) close up - the four weight gradients of a
// Llama-3-8B-shaped layer are 13 full rounds together.
int launch_multi(hipStream_t stream, GemmParams* ps, int n) {
  constexpr int BM = 256, BN = 256, NW = 8, NS = 2;
  constexpr int SMEM = NS * (BM + BN) * 128 + (NS + 1) * NW * (1024 + 16);
  GemmArgs<true> args;
  args.p = ps[0];
  int first = 0;
  double flops = 0, bytes = 0;
  for (int i = 0; i < n; ++i) {
    GemmParams& p = ps[i];
    p.tiles_m = p.m / BM;
    p.tiles_n = p.n / BN;
    const double ak = (double)p.k * p.k_parts;
    flops += 2.0 * p.m * p.n * ak;
    bytes += 2.0 * ak * (p.m + p.n) + 8.0 * p.m * p.n;
    if (i > 0) {
      GemmProblem& q = args.more[i - 1];
      q.a[0] = p.a; q.b[0] = p.b;
      for (int j = 0; j < 3; ++j) { q.a[j + 1] = p.a_more[j]; q.b[j + 1] = p.b_more[j]; }
      q.c = p.c; q.lda = p.lda; q.ldb = p.ldb; q.ldc = p.ldc;
      q.tiles_m = p.tiles_m; q.tiles_n = p.tiles_n; q.first = first;
    }
    first += p.tiles_m * p.tiles_n;
  }
  args.p.tiles_m = ps[0].tiles_m;
  args.p.tiles_n = ps[0].tiles_n;
  for (int i = n; i < 4; ++i) {
    memset(&args.more[i - 1], 0, sizeof(GemmProblem));
    args.more[i - 1].first = 0x7fffffff;
  }
  ProbeScope probe(stream, "gemm_tn_accf32_256x256w8_multi", flops, bytes);
  auto kern = gemm_kernel<BM, BN, true, true, JPP_EPI_ACC_F32, NW, NS, true, true>;
  static std::once_flag configured;
  static hipError_t configure_rc = hipSuccess;
  std::call_once(configured, [&] {
    configure_rc = hipFuncSetAttribute((const void*)kern,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
  });
  JPP_CHECK_HIP(configure_rc);
  hipLaunchKernelGGL(kern, dim3(first), dim3(NW * 64), SMEM, stream, args);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

template <bool TA, bool TB, int EPI>
int launch_tiled(hipStream_t stream, GemmParams& p, int tile) {
  switch (tile) {
    case 2:  // 8 waves of 128x32; three stages where the accumulator rows leave room
      return launch<256, 128, TA, TB, EPI, 8, EPI == JPP_EPI_ACC_F32 ? 2 : 3>(stream, p);
    case 3:  // 8 waves of 64x64
      return launch<128, 256, TA, TB, EPI, 8, EPI == JPP_EPI_ACC_F32 ? 2 : 3>(stream, p);
    case 4: return launch<256, 256, TA, TB, EPI, 8>(stream, p);
    default:
      // 128x128: 8 waves (64x32 each); the SwiGLU epilogues, which no measured workload
      // reaches at this tile size, keep the plain 4-wave form.  With more tiles than two per
      // CU, two stages and two workgroups per CU; with fewer (and a K loop long enough to pay
      // for the longer prologue) the one workgroup a CU gets prefetches deeper instead (4
      // stages, 3 where the accumulator rows need room too).
      if constexpr (EPI == JPP_EPI_SWIGLU || EPI == JPP_EPI_DSWIGLU) {
        return launch<128, 128, TA, TB, EPI>(stream, p);
      } else {
        const long tiles = (long)(p.m / 128) * (p.n / 128) *
                           (p.group_mode == JPP_GROUP_K ? p.n_seg : 1);
        if (tiles > 2 * 256 || p.k < 2048) return launch<128, 128, TA, TB, EPI, 8>(stream, p);
        return launch<128, 128, TA, TB, EPI, 8, EPI == JPP_EPI_ACC_F32 ? 3 : 4>(stream, p);
      }
  }
}

// 256 CUs.  The 256x256 tile run by 8 waves (two per SIMD, so one wave's LDS
// reads hide under the other's MFMAs) is the fastest whenever it gives most CUs
// a tile; smaller problems take 128x128 tiles, two workgroups per CU.
int choose_tile(long m, long n) {
  const long t256 = (m % 256 == 0 && n % 256 == 0) ? (m / 256) * (n / 256) : 0;
  return t256 >= 192 ? 4 : 1;
}


// sub-problem whose first row / column is (m_off, n_off) of the full one
void shift_origin(GemmParams& p, bool ta, bool tb, int epi, long m_off, long n_off) {
  p.a += ta ? m_off : m_off * p.lda;
  p.b += tb ? n_off : n_off * p.ldb;
  for (int i = 0; i + 1 < p.k_parts; ++i) {
    p.a_more[i] += ta ? m_off : m_off * p.lda;
    p.b_more[i] += tb ? n_off : n_off * p.ldb;
  }
  const long c_cols = epi == JPP_EPI_DSWIGLU ? 2 * n_off : n_off;  // dSwiGLU writes d gate, d up
  const bool f32 = epi == JPP_EPI_ACC_F32 || epi == JPP_EPI_F32;
  p.c = f32 ? (void*)((float*)p.c + m_off * p.ldc + c_cols)
            : (void*)((bf16_t*)p.c + m_off * p.ldc + c_cols);
  if (p.c2)  // SwiGLU: s has one column per gate/up pair; GELU: as wide as C
    p.c2 = (bf16_t*)p.c2 + m_off * p.ldc2 + (epi == JPP_EPI_SWIGLU ? n_off / 2 : n_off);
  if (p.bias) p.bias += n_off;
  if (p.rope_cos) {  // (n_off is a multiple of 256: whole heads)
    p.rope_row0 += m_off;
    p.rope_cols = (int)(p.rope_cols > n_off ? p.rope_cols - n_off : 0);
  }
  if (p.resid) p.resid += m_off * p.ldresid + n_off;
  if (p.aux) p.aux += m_off * p.ldaux + c_cols;
}

int dispatch(hipStream_t stream, const jpp_gemm_args* a, GemmParams& p, int tile) {
  const int ta = a->trans_a != 0, tb = a->trans_b != 0, e = a->epilogue;
#define JPP_GEMM_CASE(TA_, TB_, E_) \
  if (ta == TA_ && tb == TB_ && e == E_) return launch_tiled<TA_, TB_, E_>(stream, p, tile)
  JPP_GEMM_CASE(0, 1, JPP_EPI_BF16);     // forward
  JPP_GEMM_CASE(0, 1, JPP_EPI_GELU);     // forward + GELU
  JPP_GEMM_CASE(0, 1, JPP_EPI_F32);      // forward, f32 out (router logits)
  JPP_GEMM_CASE(0, 1, JPP_EPI_SWIGLU);   // gate/up projection + SwiGLU
  JPP_GEMM_CASE(0, 1, JPP_EPI_ACC_F32);  // weight gradient from a transposed activation
  JPP_GEMM_CASE(0, 0, JPP_EPI_BF16);     // input gradient
  JPP_GEMM_CASE(0, 0, JPP_EPI_DGELU);    // input gradient through GELU
  JPP_GEMM_CASE(0, 0, JPP_EPI_DSWIGLU);  // input gradient through SwiGLU
  JPP_GEMM_CASE(1, 1, JPP_EPI_ACC_F32);  // weight gradient, accumulated
  JPP_GEMM_CASE(1, 1, JPP_EPI_BF16);     // weight gradient, bf16
  JPP_GEMM_CASE(1, 1, JPP_EPI_F32);      // weight gradient, f32
#undef JPP_GEMM_CASE
  return jpp_set_error(JPP_ERR_INVALID, "gemm: unsupported combination trans_a=%d trans_b=%d epilogue=%d",
                       ta, tb, e);
}

// checks one problem's arguments and fills the kernel's view of it
int prepare(const jpp_gemm_args* a, GemmParams& p) {
  JPP_REQUIRE(a && a->a && a->b && a->c, "gemm: null operand");
  const bool group_k = a->group_mode == JPP_GROUP_K;
  JPP_REQUIRE(a->m > 0 && a->n > 0 && (a->k > 0 || group_k), "gemm: empty problem %ldx%ldx%ld",
              (long)a->m, (long)a->n, (long)a->k);
  JPP_REQUIRE(a->m % 128 == 0 && a->n % 128 == 0 && (a->k % 64 == 0 || group_k),
              "gemm: M,N must be multiples of 128 and K of 64, got %ldx%ldx%ld", (long)a->m,
              (long)a->n, (long)a->k);
  JPP_REQUIRE(a->lda >= (a->trans_a ? a->m : (group_k ? 0 : a->k)) &&
                  a->ldb >= (a->trans_b ? a->n : (group_k ? 0 : a->k)) &&
                  a->ldc >= a->n,
              "gemm: leading dimension too small");
  JPP_REQUIRE(a->lda % 8 == 0 && a->ldb % 8 == 0 && a->ldc % 4 == 0,
              "gemm: leading dimensions must keep 16-byte alignment");
  JPP_REQUIRE(((uintptr_t)a->a | (uintptr_t)a->b | (uintptr_t)a->c) % 16 == 0,
              "gemm: operands must be 16-byte aligned");
  JPP_REQUIRE(a->m < (1L << 31) && a->n < (1L << 31) && a->k < (1L << 31), "gemm: too large");
  p.a = (const bf16_t*)a->a;
  p.b = (const bf16_t*)a->b;
  p.c = a->c;
  p.c2 = a->c2;
  p.bias = (const bf16_t*)a->bias;
  p.resid = (const bf16_t*)a->resid;
  p.aux = (const bf16_t*)a->aux;
  p.m = (int)a->m; p.n = (int)a->n; p.k = (int)a->k;
  p.lda = a->lda; p.ldb = a->ldb; p.ldc = a->ldc;
  p.ldc2 = a->ldc2; p.ldresid = a->ldresid; p.ldaux = a->ldaux;
  p.gelu_tanh = a->gelu_tanh;
  p.seg = a->seg; p.seg_rows = a->seg_rows; p.n_seg = a->n_seg; p.group_mode = a->group_mode;
  p.group_rows = a->group_rows;
  p.tail_split = 0;
  p.stride_b = a->stride_b; p.stride_c = a->stride_c;
  p.k_parts = a->k_parts > 1 ? a->k_parts : 1;
  p.kt_part = (int)(a->k / 64);
  for (int i = 0; i < 3; ++i) {
    p.a_more[i] = (const bf16_t*)a->a_more[i];
    p.b_more[i] = (const bf16_t*)a->b_more[i];
    p.seg_more[i] = a->seg_more[i];
    p.seg_rows_more[i] = a->seg_rows_more[i];
  }
  p.rope_cos = a->rope_cos; p.rope_sin = a->rope_sin;
  p.rope_cols = (int)a->rope_cols; p.rope_seq = a->rope_seq; p.rope_hd = a->rope_head_dim;
  p.rope_row0 = 0;
  if (a->rope_cos || a->rope_sin) {
    JPP_REQUIRE(a->rope_cos && a->rope_sin, "gemm: rope_cos and rope_sin go together");
    JPP_REQUIRE(a->epilogue == JPP_EPI_BF16 && !a->trans_a && a->trans_b && !a->bias &&
                    !a->resid && a->group_mode == JPP_GROUP_NONE,
                "gemm: the rotary epilogue goes with JPP_EPI_BF16, trans_a = 0, trans_b = 1 and "
                "no bias, residual or groups");
    JPP_REQUIRE((a->rope_head_dim == 64 || a->rope_head_dim == 128) && a->rope_seq > 0 &&
                    a->rope_cols >= 0 && a->rope_cols <= a->n &&
                    a->rope_cols % a->rope_head_dim == 0,
                "gemm: rotary epilogue: heads of 64 or 128 elements, rope_cols a multiple of the "
                "head size and at most N, rope_seq positive");
    JPP_REQUIRE(((uintptr_t)a->rope_cos | (uintptr_t)a->rope_sin) % 16 == 0,
                "gemm: rotary tables must be 16-byte aligned");
  }
  if (a->k_parts > 1) {
    JPP_REQUIRE(a->k_parts <= 4 && a->group_mode != JPP_GROUP_M,
                "gemm: at most 4 operand pairs, and not with grouped rows (JPP_GROUP_M)");
    for (int i = 0; i + 1 < a->k_parts; ++i) {
      JPP_REQUIRE(a->a_more[i] && a->b_more[i] &&
                      ((uintptr_t)a->a_more[i] | (uintptr_t)a->b_more[i]) % 16 == 0,
                  "gemm: operand pair %d is null or not 16-byte aligned", i + 1);
      if (group_k)
        JPP_REQUIRE(a->seg_more[i] && !a->seg_rows_more[i] == !a->seg_rows,
                    "gemm: operand pair %d of a grouped contraction needs its row groups "
                    "(seg_more, and seg_rows_more when seg_rows is given)", i + 1);
    }
  }
  if (a->group_mode != JPP_GROUP_NONE) {
    JPP_REQUIRE(a->group_mode == JPP_GROUP_M || a->group_mode == JPP_GROUP_K,
                "gemm: unknown group_mode %d", a->group_mode);
    JPP_REQUIRE(a->seg && a->n_seg > 0 && a->n_seg <= 256, "gemm: grouped problem needs seg[n_seg+1]");
    JPP_REQUIRE((a->m % 256 == 0 && a->n % 256 == 0) || (a->group_mode == JPP_GROUP_K && a->tile),
                "gemm: grouped problems need M, N multiples of 256 (a grouped contraction with "
                "a tile of the caller's choice: of that tile)");
    JPP_REQUIRE(!a->bias && !a->resid, "gemm: grouped problems take no bias / residual");
  }
  if (a->epilogue == JPP_EPI_GELU)
    JPP_REQUIRE(a->c2 && a->ldc2 >= a->n && a->ldc2 % 4 == 0, "gemm: GELU epilogue needs c2");
  if (a->epilogue == JPP_EPI_DGELU)
    JPP_REQUIRE(a->aux && a->ldaux >= a->n && a->ldaux % 4 == 0, "gemm: dGELU epilogue needs aux");
  if (a->epilogue == JPP_EPI_SWIGLU)
    JPP_REQUIRE(a->c2 && a->ldc2 >= a->n / 2 && a->ldc2 % 4 == 0 && !a->bias && !a->resid &&
                    a->group_mode != JPP_GROUP_K,
                "gemm: SwiGLU epilogue needs c2 [M, N/2] and takes no bias / residual");
  if (a->epilogue == JPP_EPI_DSWIGLU)
    JPP_REQUIRE(a->aux && a->ldaux >= 2 * a->n && a->ldaux % 4 == 0 && a->ldc >= 2 * a->n &&
                    !a->bias && !a->resid && a->group_mode != JPP_GROUP_K,
                "gemm: dSwiGLU epilogue needs aux and C of width 2N and takes no bias / residual");
  if (a->epilogue == JPP_EPI_ACC_F32)
    JPP_REQUIRE((double)a->m * a->ldc * 4 < 4294967296.0,
                "gemm: an accumulated output must span less than 4 GiB (32-bit offsets)");
  if (a->resid) JPP_REQUIRE(a->ldresid >= a->n && a->ldresid % 4 == 0, "gemm: bad ldresid");
  return JPP_OK;
}

}  // namespace

extern "C" int jpp_gemm_bf16(void* stream_, const jpp_gemm_args* a) {
  hipStream_t stream = (hipStream_t)stream_;
  GemmParams p;
  if (int rc = prepare(a, p)) return rc;
  int tile = a->tile ? a->tile : choose_tile(a->m, a->n);
  // row groups come in 256-row segments; a contraction split into groups takes any tile
  if (a->group_mode == JPP_GROUP_M || (a->group_mode == JPP_GROUP_K && !a->tile)) tile = 4;
  // several operand pairs exist on the 256-wide tiles only: a tile left to the library goes
  // there whatever the problem's size (N not a multiple of 256 is refused below, with the
  // kernel's message)
  if (a->k_parts > 1 && !a->tile) tile = 4;
  JPP_REQUIRE(tile >= 1 && tile <= 4, "gemm: unknown tile %d", tile);
  if ((tile == 2 || tile == 4) && a->m % 256) tile = a->n % 256 ? 1 : 3;
  if ((tile == 3 || tile == 4) && a->n % 256) tile = a->m % 256 ? 1 : 2;

  // A grid of 256x256 tiles whose last round fills at most half of the 256 CUs runs that
  // round as a separate launch of 128x256 tiles over the last rows or columns: a full round
  // of half-size tiles takes little more than half the time the half-empty round did.
  // (Only when the choice of tile was left to the library.)
  if (tile == 4 && a->tile == 0 && a->group_mode == JPP_GROUP_NONE) {
    const long tm = a->m / 256, tn = a->n / 256, rest = (tm * tn) % 256;
    if (tm * tn > 256 && rest > 0 && rest <= 128) {
      const long rows = rest % tn == 0 ? rest / tn * 256 : 0;             // split along M
      const long cols = !rows && rest % tm == 0 ? rest / tm * 256 : 0;    // split along N
      if (rows || cols) {
        GemmParams head = p, tail = p;
        if (rows) {
          head.m = p.m - (int)rows;
          tail.m = (int)rows;
          shift_origin(tail, a->trans_a != 0, a->trans_b != 0, a->epilogue, head.m, 0);
        } else {
          head.n = p.n - (int)cols;
          tail.n = (int)cols;
          shift_origin(tail, a->trans_a != 0, a->trans_b != 0, a->epilogue, 0, head.n);
        }
        const int rc = dispatch(stream, a, head, 4);
        return rc != JPP_OK ? rc : dispatch(stream, a, tail, 3);
      }
    }
  }
  // Row groups: how many rows are in use is known on the device only, so the same split is
  // made there (group_head_rows) - the launches of small tiles are always enqueued and the
  // workgroups of those that find no rows of theirs leave at once.
  if (tile == 4 && a->tile == 0 && a->group_mode == JPP_GROUP_M && a->epilogue == JPP_EPI_BF16) {
    const long tm = a->m / 256, tn = a->n / 256;
    if (tm * tn > 256 && tn <= 128) {
      GemmParams head = p, small = p, wide = p;
      head.tail_split = 1;
      small.tail_split = 2;
      small.m = (int)std::min<long>(a->m, 64 / tn * 256);    // at most 64 tiles of 256x256
      wide.tail_split = 3;
      wide.m = (int)std::min<long>(a->m, 128 / tn * 256);    // at most 128
      int rc = dispatch(stream, a, head, 4);
      if (rc == JPP_OK && small.m > 0) rc = dispatch(stream, a, small, 1);
      return rc != JPP_OK ? rc : dispatch(stream, a, wide, 3);
    }
  }
  return dispatch(stream, a, p, tile);
}

extern "C" int jpp_gemm_bf16_multi(void* stream_, const jpp_gemm_args* problems, int n_problems) {
  hipStream_t stream = (hipStream_t)stream_;
  JPP_REQUIRE(problems && n_problems >= 1 && n_problems <= 4, "gemm_multi: 1 to 4 problems");
  if (n_problems == 1) return jpp_gemm_bf16(stream_, problems);
  GemmParams ps[4];
  long tiles = 0;
  for (int i = 0; i < n_problems; ++i) {
    const jpp_gemm_args* a = problems + i;
    if (int rc = prepare(a, ps[i])) return rc;
    JPP_REQUIRE(a->trans_a && a->trans_b && a->epilogue == JPP_EPI_ACC_F32 &&
                    a->group_mode == JPP_GROUP_NONE && !a->bias && !a->resid && !a->tile,
                "gemm_multi: problem %d is not a plain accumulated weight gradient (trans_a = "
                "trans_b = 1, JPP_EPI_ACC_F32, no groups, bias, residual or tile choice)", i);
    JPP_REQUIRE(a->m % 256 == 0 && a->n % 256 == 0,
                "gemm_multi: problem %d: M and N must be multiples of 256, got %ldx%ld", i,
                (long)a->m, (long)a->n);
    JPP_REQUIRE(a->k == problems[0].k && ps[i].k_parts == ps[0].k_parts,
                "gemm_multi: problem %d differs from problem 0 in k or k_parts", i);
    tiles += (a->m / 256) * (a->n / 256);
  }
  JPP_REQUIRE(tiles < (1L << 30), "gemm_multi: too many tiles");
  return launch_multi(stream, ps, n_problems);
}
