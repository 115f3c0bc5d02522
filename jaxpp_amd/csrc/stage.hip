// Stage executor: runs the FWD / BWD / BWD_I / BWD_W tasks of one pipeline
// rank on one GPU, in whatever order the schedule's table dictates.
//
// Plays the part of `task_impl` in the reference
// (src/jaxpp/jax_primitives.py:776-859) for the stages one rank owns:
//   * a forward task runs the stage's layers and leaves a residual set
//     ("stash") in a slot of a fixed ring; the slot is released by the task
//     that last reads it - BWD, or BWD_W when the backward is split - which is
//     the lifetime the reference derives with `infer_donation` / `add_deletes`
//     (src/jaxpp/core.py:1732-1890);
//   * with a split backward, BWD_I runs the input-gradient chain plus the
//     small non-matmul parameter gradients (bias column sums, norm scale /
//     shift), and BWD_W runs the weight-gradient GEMMs, exactly the partition
//     `partition_eqns(memory_scarce=True)` makes (src/jaxpp/jaxpr_utils.py:105-169);
//   * gradients are accumulated in fp32 in place: the loop carry of `treduce`
//     with `Add` (src/jaxpp/training.py:112-123).
#include <math.h>
#include <string.h>

#include <algorithm>
#include <map>
#include <string>
#include <utility>
#include <vector>

#include "common.h"

namespace {

struct ParamInfo {
  const char* name;
  int64_t rows, cols;
};

struct Buf {  // a carved piece of a slot / scratch allocation
  size_t off = 0, bytes = 0;
};

struct Carver {
  size_t total = 0;
  Buf take(size_t bytes) {
    Buf b;
    b.off = total;
    b.bytes = bytes;
    total += (bytes + 255) & ~(size_t)255;
    return b;
  }
};

// Residuals of one layer for one microbatch (offsets into a slot).
struct LayerStash {
  // common
  Buf x, qkv, ctx, lse;
  // bert
  Buf a, mean1, rstd1, x1, u, g, c, mean2, rstd2;
  // llama
  Buf n1, h1, n2, gu, s;
  // mixtral: routing tables and token-permuted expert buffers (gu, s reused, [cap, ..])
  Buf ids, gates, row_of, tok_of, gate_of, seg, xp, eo;
  // pre-LN decoder block: x, qkv, ctx, lse, mean1, rstd1, n1, h1, mean2, rstd2, n2, u, g
  // cotangents kept for the weight-gradient task
  Buf dc, du, da, dqkv;   // bert (dqkv shared with the others, du with the decoder block)
  Buf dyin, dgu, dh1;     // llama (dyin, dh1 also the decoder block)
  Buf deo, dlogits;       // mixtral
};

}  // namespace

struct jpp_stage {
  jpp_stage_desc d;
  int64_t T, h, f, qkvw, ctxw, hd, cap = 0;  // cap: rows of the token-permuted buffers
  std::vector<ParamInfo> pinfo;
  std::vector<size_t> poff;        // element offset of parameter i inside a layer block
  size_t layer_elems = 0;
  size_t es = 2;                   // bytes per element of parameters and activations
  uint8_t* params = nullptr;       // [chunk][layer][layer_elems] bf16 or f32
  float* grads = nullptr;          // same shape, f32
  float* opt[3] = {nullptr, nullptr, nullptr};  // f32 weights, m, v of the optimizer (same shape)
  std::vector<LayerStash> lay;     // per layer of a chunk, offsets into a slot
  size_t slot_bytes = 0;
  std::vector<uint8_t*> slots;
  std::vector<int> free_slots;
  std::map<std::pair<int, int>, int> live;  // (chunk, mubatch) -> slot
  std::map<std::pair<int, int>, int> phase; // 1: forward done, 2: BWD_I done
  // scratch shared by all tasks (stream ordered)
  uint8_t* scratch = nullptr;
  size_t scratch_bytes = 0;
  // Cotangent buffers when the backward is not split (else they live in the slot).  With a
  // second stream there are three sets, used by layer index mod 3: the weight gradients of
  // layer l+1 read set (l+1)%3 while layer l's input-gradient chain writes set l%3 and
  // hands its result to layer l-1 in set (l-1)%3.
  LayerStash wsets[3];
  Buf s_dx[2], s_t1, s_t2, s_t3, s_t4, s_partial, s_partial_side, s_delta, s_wg, s_split, s_cos,
      s_sin, s_moework;
  size_t total_bytes = 0;
  // second stream (two_streams): weight gradients trail the input-gradient chain
  hipStream_t side = nullptr;
  hipEvent_t ev_fork = nullptr;          // recorded on the caller's stream, awaited by `side`
  hipEvent_t ev_set[3] = {};             // last weight-gradient reader of a cotangent set
  bool set_pending[3] = {};
  std::vector<hipEvent_t> ev_slot;       // last `side` reader of a slot
  std::vector<char> slot_pending;
  std::vector<hipEvent_t> ev_bwd_i;      // end of a slot's BWD_I task on the caller's stream
  hipEvent_t ev_tail = nullptr;          // last work queued on `side`
  bool tail_pending = false;

  // Weight gradients of up to wg consecutive microbatches (aligned groups mubatch / wg) run as
  // one product per weight: pend[chunk] lists the (microbatch, slot) pairs whose input-
  // gradient half is done and whose weight-gradient half waits for the rest of its group.
  int wg = 1;
  std::vector<std::vector<std::pair<int, int>>> pend;
  bool broken = false;   // a grouped weight-gradient launch failed half way: accumulators unusable

  bool f32() const { return d.dtype == JPP_DTYPE_F32; }
  void* P(int chunk, int layer, int i) {
    return params + (((size_t)chunk * d.layers_per_chunk + layer) * layer_elems + poff[i]) * es;
  }
  float* G(int chunk, int layer, int i) {
    return grads + ((size_t)chunk * d.layers_per_chunk + layer) * layer_elems + poff[i];
  }
  template <class T_ = void>
  T_* S(const Buf& b) { return (T_*)(scratch + b.off); }
};

namespace {

enum BertP { B_Wqkv, B_bqkv, B_Wo, B_bo, B_ln1g, B_ln1b, B_W1, B_b1, B_W2, B_b2, B_ln2g, B_ln2b };
enum LlamaP { L_rms1, L_Wqkv, L_Wo, L_rms2, L_Wgu, L_Wd };
enum MixtralP { X_rms1, X_Wqkv, X_Wo, X_rms2, X_Wr, X_Wgu, X_Wd };

#define RC(expr)            \
  do {                      \
    int rc_ = (expr);       \
    if (rc_) return rc_;    \
  } while (0)

int ggemm(jpp_stage* s, hipStream_t st, int mode, const int* seg, int n_seg, const void* a, int64_t lda, int ta,
          const void* b, int64_t ldb, int tb, int64_t stride_b, void* c, int64_t ldc,
          int64_t stride_c, int64_t m, int64_t n, int64_t k, int epi, int64_t rows,
          const void* aux = nullptr, int64_t ldaux = 0, void* c2 = nullptr, int64_t ldc2 = 0) {
  jpp_gemm_args g;
  memset(&g, 0, sizeof(g));
  g.a = a; g.b = b; g.c = c; g.m = m; g.n = n; g.k = k;
  g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.trans_a = ta; g.trans_b = tb; g.epilogue = epi;
  g.seg = seg; g.n_seg = n_seg; g.group_mode = mode; g.stride_b = stride_b; g.stride_c = stride_c;
  g.group_rows = rows;
  g.seg_rows = seg + n_seg + 1;   // the routing kernels leave the token counts behind the offsets
  g.aux = aux; g.ldaux = ldaux; g.c2 = c2; g.ldc2 = ldc2;
  return s->d.dtype == JPP_DTYPE_F32 ? jpp_gemm_f32(st, &g) : jpp_gemm_bf16(st, &g);
}

void moe_args(jpp_stage* s, jpp_moe_args& m, uint8_t* slot, const LayerStash& L, int chunk,
              int li) {
  memset(&m, 0, sizeof(m));
  m.x = slot + L.n2.off;
  m.wr = s->P(chunk, li, X_Wr);
  m.ids = (int32_t*)(slot + L.ids.off);
  m.gates = (float*)(slot + L.gates.off);
  m.row_of = (int32_t*)(slot + L.row_of.off);
  m.tok_of = (int32_t*)(slot + L.tok_of.off);
  m.gate_of = (float*)(slot + L.gate_of.off);
  m.seg = (int32_t*)(slot + L.seg.off);
  m.work = s->S<>(s->s_moework);
  m.tokens = s->T; m.hidden = s->h; m.n_experts = s->d.n_experts; m.top_k = s->d.top_k;
  m.dtype = s->d.dtype;
}

int gemm(jpp_stage* s, hipStream_t st, const void* a, int64_t lda, int ta, const void* b, int64_t ldb, int tb,
         void* c, int64_t ldc, int64_t m, int64_t n, int64_t k, int epi, const void* bias = nullptr,
         const void* resid = nullptr, int64_t ldr = 0, const void* aux = nullptr,
         int64_t ldaux = 0, void* c2 = nullptr, int64_t ldc2 = 0, int gelu_tanh = 0) {
  jpp_gemm_args g;
  memset(&g, 0, sizeof(g));
  g.a = a; g.b = b; g.c = c; g.c2 = c2; g.bias = bias; g.resid = resid; g.aux = aux;
  g.m = m; g.n = n; g.k = k;
  g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.ldc2 = ldc2; g.ldresid = ldr; g.ldaux = ldaux;
  g.trans_a = ta; g.trans_b = tb; g.epilogue = epi; g.gelu_tanh = gelu_tanh;
  return s->f32() ? jpp_gemm_f32(st, &g) : jpp_gemm_bf16(st, &g);
}

int rope(jpp_stage* s, hipStream_t st, void* x, int inverse) {
  const int heads = s->d.n_heads + s->d.n_kv_heads;
  float* c = s->S<float>(s->s_cos);
  float* sn = s->S<float>(s->s_sin);
  return s->f32() ? jpp_rope_f32(st, (float*)x, s->qkvw, c, sn, s->d.batch, s->d.seq, heads,
                                 (int)s->hd, inverse)
                  : jpp_rope(st, x, s->qkvw, c, sn, s->d.batch, s->d.seq, heads, (int)s->hd, inverse);
}
int attn_f(jpp_stage* s, hipStream_t st, const jpp_attn_args* a) {
  return s->f32() ? jpp_attn_fwd_f32(st, a) : jpp_attn_fwd(st, a);
}
int attn_b(jpp_stage* s, hipStream_t st, const jpp_attn_args* a) {
  return s->f32() ? jpp_attn_bwd_f32(st, a) : jpp_attn_bwd(st, a);
}

// a layer's four bias gradients: column sums of the cotangents, added to the accumulators
int bias_grads4(jpp_stage* s, hipStream_t st, const jpp_colsum_item* items, float* partial) {
  if (!s->f32()) return jpp_colsum_accum_multi(st, 4, items, s->T, partial);
  for (int i = 0; i < 4; ++i)
    RC(jpp_colsum_accum_f32(st, (const float*)items[i].x, items[i].ld, s->T, items[i].cols,
                            items[i].acc));
  return JPP_OK;
}

// dW[rows, cols] (+)= X^T dY, X: [T, rows], dY: [T, cols]
int wgrad(jpp_stage* s, hipStream_t st, const void* x, int64_t ldx, const void* dy, int64_t lddy,
          float* acc, int64_t rows, int64_t cols) {
  if (s->f32()) return gemm(s, st, x, ldx, 1, dy, lddy, 1, acc, cols, rows, cols, s->T, JPP_EPI_ACC_F32);
  if (s->d.fused_wgrad_accum) {
    // A weight matrix of at most 128 tiles of 128x128 leaves half of the CUs without work:
    // the contraction over the tokens is then split over `parts` workgroups per tile, which
    // leave f32 partial products in scratch, and an ordered sum adds them to the accumulator
    // (the order is fixed, so the result does not depend on timing).
    const int64_t tiles = (rows / 128) * (cols / 128);
    int parts = 1;
    while (parts < 8 && tiles * parts * 2 <= 256 && s->T % (parts * 2 * 64) == 0 &&
           s->T / (parts * 2) >= 512)
      parts *= 2;
    if (parts > 1 && (size_t)parts * rows * cols * 4 <= s->s_wg.bytes) {
      float* ws = s->S<float>(s->s_wg);
      jpp_gemm_args g;
      memset(&g, 0, sizeof(g));
      g.a = x; g.b = dy; g.c = ws; g.m = rows; g.n = cols; g.k = 0;
      g.lda = ldx; g.ldb = lddy; g.ldc = cols; g.trans_a = 1; g.trans_b = 1;
      g.epilogue = JPP_EPI_F32; g.tile = 1;
      g.seg = s->S<int32_t>(s->s_split) + 16 * (parts == 2 ? 0 : parts == 4 ? 1 : 2);
      g.n_seg = parts; g.group_mode = JPP_GROUP_K; g.stride_c = rows * cols;
      g.group_rows = s->T;
      RC(jpp_gemm_bf16(st, &g));
      return jpp_sum_accum_f32(st, acc, ws, parts, rows * cols);
    }
    return gemm(s, st, x, ldx, 1, dy, lddy, 1, acc, cols, rows, cols, s->T, JPP_EPI_ACC_F32);
  }
  void* g = s->S<>(s->s_wg);
  RC(gemm(s, st, x, ldx, 1, dy, lddy, 1, g, cols, rows, cols, s->T, JPP_EPI_BF16));
  return jpp_grad_accum_f32(st, acc, g, rows * cols, 0);
}

// dW (+)= sum over n microbatches of X_i^T dY_i: one product over n operand pairs when the
// matrix is large enough to fill the device, else one product per microbatch (in order)
int wgrad_n(jpp_stage* s, hipStream_t st, int n, const void* const* xs, int64_t ldx,
            const void* const* dys, int64_t lddy, float* acc, int64_t rows, int64_t cols) {
  const bool big = rows % 256 == 0 && cols % 256 == 0 && (rows / 256) * (cols / 256) >= 192;
  if (n == 1 || !big || s->f32() || !s->d.fused_wgrad_accum) {
    for (int i = 0; i < n; ++i) RC(wgrad(s, st, xs[i], ldx, dys[i], lddy, acc, rows, cols));
    return JPP_OK;
  }
  jpp_gemm_args g;
  memset(&g, 0, sizeof(g));
  g.a = xs[0]; g.b = dys[0]; g.c = acc; g.m = rows; g.n = cols; g.k = s->T;
  g.lda = ldx; g.ldb = lddy; g.ldc = cols; g.trans_a = 1; g.trans_b = 1;
  g.epilogue = JPP_EPI_ACC_F32;
  g.k_parts = n;
  for (int i = 1; i < n; ++i) { g.a_more[i - 1] = xs[i]; g.b_more[i - 1] = dys[i]; }
  return jpp_gemm_bf16(st, &g);
}

// The dense weight gradients of one layer, gathered so that they can leave as one launch.
struct WgradBatch {
  jpp_gemm_args g[4];
  int n = 0;
  void add(jpp_stage* s, int pairs, const void* const* xs, int64_t ldx, const void* const* dys,
           int64_t lddy, float* acc, int64_t rows, int64_t cols) {
    jpp_gemm_args& q = g[n++];
    memset(&q, 0, sizeof(q));
    q.a = xs[0]; q.b = dys[0]; q.c = acc; q.m = rows; q.n = cols; q.k = s->T;
    q.lda = ldx; q.ldb = lddy; q.ldc = cols; q.trans_a = 1; q.trans_b = 1;
    q.epilogue = JPP_EPI_ACC_F32;
    q.k_parts = pairs;
    for (int i = 1; i < pairs; ++i) { q.a_more[i - 1] = xs[i]; q.b_more[i - 1] = dys[i]; }
  }
  void add1(jpp_stage* s, const void* x, int64_t ldx, const void* dy, int64_t lddy, float* acc,
            int64_t rows, int64_t cols) {
    add(s, 1, &x, ldx, &dy, lddy, acc, rows, cols);
  }
};

// Runs a layer's gathered weight gradients: as one grid of 256x256 tiles when that takes
// fewer rounds of the 256 CUs than the launches one by one (whose last rounds stay partly
// empty: a round of 128x256 tiles for a rest of at most 128 tiles costs about 0.77 of a full
// one), else one by one.  Which way is taken depends on the shapes only.
int run_wgrads(jpp_stage* s, hipStream_t st, WgradBatch& w) {
  bool multi = w.n >= 2 && !s->f32() && s->d.fused_wgrad_accum;
  long total = 0;
  double apart = 0;
  for (int i = 0; i < w.n && multi; ++i) {
    const jpp_gemm_args& q = w.g[i];
    if (q.m % 256 || q.n % 256) { multi = false; break; }
    const long t = (q.m / 256) * (q.n / 256), rest = t % 256;
    total += t;
    apart += (double)(t / 256) + (rest == 0 ? 0.0 : (rest <= 128 && t > 256 ? 0.77 : 1.0));
  }
  // (matrices of fewer than 192 tiles would run one by one on 128x128 tiles, each launch
  // leaving most of the device idle: BERT-large's four are 192 tiles of 256x256 together,
  // one round, -3.3 % step time; below half a round in total the single launches, which
  // split the contraction over workgroups, keep the device busier)
  if (multi && total >= 128 && (double)((total + 255) / 256) < apart - 0.25) {
    // smallest first: measured 1 % faster than largest first at the Llama-3-8B shapes
    jpp_gemm_args order[4];
    for (int i = 0; i < w.n; ++i) order[i] = w.g[i];
    std::stable_sort(order, order + w.n, [](const jpp_gemm_args& a, const jpp_gemm_args& b) {
      return a.m * a.n < b.m * b.n;
    });
    return jpp_gemm_bf16_multi(st, order, w.n);
  }
  for (int i = 0; i < w.n; ++i) {
    const jpp_gemm_args& q = w.g[i];
    const int pairs = q.k_parts > 1 ? q.k_parts : 1;
    const void* xs[4] = {q.a, q.a_more[0], q.a_more[1], q.a_more[2]};
    const void* dys[4] = {q.b, q.b_more[0], q.b_more[1], q.b_more[2]};
    RC(wgrad_n(s, st, pairs, xs, q.lda, dys, q.ldb, (float*)q.c, q.m, q.n));
  }
  return JPP_OK;
}

int norm_f(jpp_stage* s, hipStream_t st, const void* x, const void* gamma, const void* beta,
           void* y, float* mean, float* rstd) {
  jpp_norm_args a;
  memset(&a, 0, sizeof(a));
  a.x = x; a.gamma = gamma; a.beta = beta; a.y = y; a.mean = mean; a.rstd = rstd;
  a.rows = s->T; a.cols = s->h; a.eps = s->d.eps;
  return s->f32() ? jpp_norm_fwd_f32(st, &a) : jpp_norm_fwd(st, &a);
}

int norm_b(jpp_stage* s, hipStream_t st, const void* dy, const void* x, const float* mean,
           const float* rstd, const void* gamma, const void* resid, void* dx, float* dgamma,
           float* dbeta) {
  jpp_norm_args a;
  memset(&a, 0, sizeof(a));
  a.dy = dy; a.x = x; a.mean = (float*)mean; a.rstd = (float*)rstd; a.gamma = gamma;
  a.resid = resid; a.dx = dx; a.dgamma = dgamma; a.dbeta = dbeta;
  a.partial = s->S<float>(s->s_partial);
  a.rows = s->T; a.cols = s->h; a.eps = s->d.eps;
  return s->f32() ? jpp_norm_bwd_f32(st, &a) : jpp_norm_bwd(st, &a);
}

void attn_args(jpp_stage* s, jpp_attn_args& a, uint8_t* slot, const LayerStash& L) {
  memset(&a, 0, sizeof(a));
  uint8_t* qkv = slot + L.qkv.off;
  a.q = qkv;
  a.k = qkv + (int64_t)s->d.n_heads * s->hd * s->es;
  a.v = qkv + (int64_t)(s->d.n_heads + s->d.n_kv_heads) * s->hd * s->es;
  a.ldq = a.ldk = a.ldv = s->qkvw;
  a.o = slot + L.ctx.off;
  a.ldo = s->ctxw;
  a.lse = (float*)(slot + L.lse.off);
  a.batch = s->d.batch; a.seq = s->d.seq; a.n_heads = s->d.n_heads;
  a.n_kv_heads = s->d.n_kv_heads; a.head_dim = (int)s->hd; a.causal = s->d.causal;
}

// ---- one layer, forward ----------------------------------------------------
int layer_fwd(jpp_stage* s, hipStream_t st, int chunk, int li, uint8_t* slot, void* y) {
  const LayerStash& L = s->lay[li];
  const int64_t T = s->T, h = s->h, f = s->f;
  auto at = [&](const Buf& b) { return (void*)(slot + b.off); };
  jpp_attn_args aa;
  if (s->d.family == JPP_FAMILY_BERT) {
    RC(gemm(s, st, at(L.x), h, 0, s->P(chunk, li, B_Wqkv), 3 * h, 1, at(L.qkv), 3 * h, T, 3 * h, h,
            JPP_EPI_BF16, s->P(chunk, li, B_bqkv)));
    attn_args(s, aa, slot, L);
    RC(attn_f(s, st, &aa));
    RC(gemm(s, st, at(L.ctx), h, 0, s->P(chunk, li, B_Wo), h, 1, at(L.a), h, T, h, h, JPP_EPI_BF16,
            s->P(chunk, li, B_bo), at(L.x), h));
    RC(norm_f(s, st, at(L.a), s->P(chunk, li, B_ln1g), s->P(chunk, li, B_ln1b), at(L.x1),
              (float*)at(L.mean1), (float*)at(L.rstd1)));
    RC(gemm(s, st, at(L.x1), h, 0, s->P(chunk, li, B_W1), f, 1, at(L.u), f, T, f, h, JPP_EPI_GELU,
            s->P(chunk, li, B_b1), nullptr, 0, nullptr, 0, at(L.g), f, s->d.gelu_tanh));
    RC(gemm(s, st, at(L.g), f, 0, s->P(chunk, li, B_W2), h, 1, at(L.c), h, T, h, f, JPP_EPI_BF16,
            s->P(chunk, li, B_b2), at(L.x1), h));
    RC(norm_f(s, st, at(L.c), s->P(chunk, li, B_ln2g), s->P(chunk, li, B_ln2b), y,
              (float*)at(L.mean2), (float*)at(L.rstd2)));
    return JPP_OK;
  }
  if (s->d.family == JPP_FAMILY_DECODER) {
    // pre-LN block with biases and a GELU feed-forward; parameters as in the BERT layer
    RC(norm_f(s, st, at(L.x), s->P(chunk, li, B_ln1g), s->P(chunk, li, B_ln1b), at(L.n1),
              (float*)at(L.mean1), (float*)at(L.rstd1)));
    RC(gemm(s, st, at(L.n1), h, 0, s->P(chunk, li, B_Wqkv), 3 * h, 1, at(L.qkv), 3 * h, T, 3 * h, h,
            JPP_EPI_BF16, s->P(chunk, li, B_bqkv)));
    attn_args(s, aa, slot, L);
    RC(attn_f(s, st, &aa));
    RC(gemm(s, st, at(L.ctx), h, 0, s->P(chunk, li, B_Wo), h, 1, at(L.h1), h, T, h, h, JPP_EPI_BF16,
            s->P(chunk, li, B_bo), at(L.x), h));
    RC(norm_f(s, st, at(L.h1), s->P(chunk, li, B_ln2g), s->P(chunk, li, B_ln2b), at(L.n2),
              (float*)at(L.mean2), (float*)at(L.rstd2)));
    RC(gemm(s, st, at(L.n2), h, 0, s->P(chunk, li, B_W1), f, 1, at(L.u), f, T, f, h, JPP_EPI_GELU,
            s->P(chunk, li, B_b1), nullptr, 0, nullptr, 0, at(L.g), f, s->d.gelu_tanh));
    RC(gemm(s, st, at(L.g), f, 0, s->P(chunk, li, B_W2), h, 1, y, h, T, h, f, JPP_EPI_BF16,
            s->P(chunk, li, B_b2), at(L.h1), h));
    return JPP_OK;
  }
  // llama
  RC(norm_f(s, st, at(L.x), s->P(chunk, li, L_rms1), nullptr, at(L.n1), nullptr,
            (float*)at(L.rstd1)));
  if (s->f32()) {
    RC(gemm(s, st, at(L.n1), h, 0, s->P(chunk, li, L_Wqkv), s->qkvw, 1, at(L.qkv), s->qkvw, T,
            s->qkvw, h, JPP_EPI_BF16));
    RC(rope(s, st, at(L.qkv), 0));
  } else {
    // the projection rotates the query and key heads in its epilogue (the same values a pass
    // of jpp_rope over its plain result would leave)
    jpp_gemm_args g;
    memset(&g, 0, sizeof(g));
    g.a = at(L.n1); g.b = s->P(chunk, li, L_Wqkv); g.c = at(L.qkv);
    g.m = T; g.n = s->qkvw; g.k = h;
    g.lda = h; g.ldb = s->qkvw; g.ldc = s->qkvw;
    g.trans_a = 0; g.trans_b = 1; g.epilogue = JPP_EPI_BF16;
    g.rope_cos = s->S<float>(s->s_cos); g.rope_sin = s->S<float>(s->s_sin);
    g.rope_cols = (int64_t)(s->d.n_heads + s->d.n_kv_heads) * s->hd;
    g.rope_seq = s->d.seq; g.rope_head_dim = (int)s->hd;
    RC(jpp_gemm_bf16(st, &g));
  }
  attn_args(s, aa, slot, L);
  RC(attn_f(s, st, &aa));
  RC(gemm(s, st, at(L.ctx), s->ctxw, 0, s->P(chunk, li, L_Wo), h, 1, at(L.h1), h, T, h, s->ctxw,
          JPP_EPI_BF16, nullptr, at(L.x), h));
  RC(norm_f(s, st, at(L.h1), s->P(chunk, li, L_rms2), nullptr, at(L.n2), nullptr,
            (float*)at(L.rstd2)));
  if (s->d.family == JPP_FAMILY_MIXTRAL) {
    jpp_moe_args ma;
    moe_args(s, ma, slot, L, chunk, li);
    const int E = s->d.n_experts;
    const int* seg = ma.seg;
    RC(jpp_moe_route(st, &ma));
    RC(jpp_moe_gather(st, &ma, at(L.n2), at(L.xp)));
    // gate and up columns of each expert's Wgu are interleaved in blocks of 32, as in the
    // dense layer: SwiGLU runs in the epilogue
    RC(ggemm(s, st, JPP_GROUP_M, seg, E, at(L.xp), h, 0, s->P(chunk, li, X_Wgu), 2 * f, 1, h * 2 * f,
             at(L.gu), 2 * f, 0, s->cap, 2 * f, h, JPP_EPI_SWIGLU, s->T * s->d.top_k, nullptr, 0,
             at(L.s), f));
    RC(ggemm(s, st, JPP_GROUP_M, seg, E, at(L.s), f, 0, s->P(chunk, li, X_Wd), h, 1, f * h, at(L.eo), h,
             0, s->cap, h, f, JPP_EPI_BF16, s->T * s->d.top_k));
    RC(jpp_moe_combine_fwd(st, &ma, at(L.eo), at(L.h1), y));
    return JPP_OK;
  }
  // gate and up columns of Wgu are interleaved in blocks of 32: SwiGLU runs in the epilogue
  RC(gemm(s, st, at(L.n2), h, 0, s->P(chunk, li, L_Wgu), 2 * f, 1, at(L.gu), 2 * f, T, 2 * f, h,
          JPP_EPI_SWIGLU, nullptr, nullptr, 0, nullptr, 0, at(L.s), f));
  RC(gemm(s, st, at(L.s), f, 0, s->P(chunk, li, L_Wd), h, 1, y, h, T, h, f, JPP_EPI_BF16, nullptr,
          at(L.h1), h));
  return JPP_OK;
}

// ---- one layer, input-gradient half -------------------------------------------
// `w` holds the cotangents the weight-gradient half will read: the slot itself
// when the backward is split, the shared scratch set otherwise.
int layer_bwd_i(jpp_stage* s, hipStream_t st, int chunk, int li, uint8_t* slot, uint8_t* wbase,
                const LayerStash& W, const void* dy, void* dx) {
  const LayerStash& L = s->lay[li];
  const int64_t T = s->T, h = s->h, f = s->f;
  auto at = [&](const Buf& b) { return (void*)(slot + b.off); };
  auto wt = [&](const Buf& b) { return (void*)(wbase + b.off); };
  float* partial = s->S<float>(s->s_partial);
  jpp_attn_args aa;
  if (s->d.family == JPP_FAMILY_BERT) {
    void* dx1 = s->S<>(s->s_t1);
    void* dctx = s->S<>(s->s_t2);
    RC(norm_b(s, st, dy, at(L.c), (float*)at(L.mean2), (float*)at(L.rstd2),
              s->P(chunk, li, B_ln2g), nullptr, wt(W.dc), s->G(chunk, li, B_ln2g),
              s->G(chunk, li, B_ln2b)));
    RC(gemm(s, st, wt(W.dc), h, 0, s->P(chunk, li, B_W2), h, 0, wt(W.du), f, T, f, h, JPP_EPI_DGELU,
            nullptr, nullptr, 0, at(L.u), f, nullptr, 0, s->d.gelu_tanh));
    RC(gemm(s, st, wt(W.du), f, 0, s->P(chunk, li, B_W1), f, 0, dx1, h, T, h, f, JPP_EPI_BF16, nullptr,
            wt(W.dc), h));
    RC(norm_b(s, st, dx1, at(L.a), (float*)at(L.mean1), (float*)at(L.rstd1),
              s->P(chunk, li, B_ln1g), nullptr, wt(W.da), s->G(chunk, li, B_ln1g),
              s->G(chunk, li, B_ln1b)));
    RC(gemm(s, st, wt(W.da), h, 0, s->P(chunk, li, B_Wo), h, 0, dctx, h, T, h, h, JPP_EPI_BF16));
    attn_args(s, aa, slot, L);
    uint8_t* dqkv = (uint8_t*)wt(W.dqkv);
    aa.d_o = dctx; aa.lddo = h;
    aa.dq = dqkv; aa.dk = dqkv + h * s->es; aa.dv = dqkv + 2 * h * s->es;
    aa.lddq = aa.lddk = aa.lddv = 3 * h;
    aa.delta = s->S<float>(s->s_delta);
    RC(attn_b(s, st, &aa));
    RC(gemm(s, st, dqkv, 3 * h, 0, s->P(chunk, li, B_Wqkv), 3 * h, 0, dx, h, T, h, 3 * h,
            JPP_EPI_BF16, nullptr, wt(W.da), h));
    const jpp_colsum_item bias_grads[4] = {{wt(W.dc), h, h, s->G(chunk, li, B_b2)},
                                           {wt(W.du), f, f, s->G(chunk, li, B_b1)},
                                           {wt(W.da), h, h, s->G(chunk, li, B_bo)},
                                           {dqkv, 3 * h, 3 * h, s->G(chunk, li, B_bqkv)}};
    RC(bias_grads4(s, st, bias_grads, partial));
    return JPP_OK;
  }
  void* dn = s->S<>(s->s_t2);   // dn2, later dn1
  void* dctx = s->S<>(s->s_t3);
  if (s->d.family == JPP_FAMILY_DECODER) {
    RC(gemm(s, st, dy, h, 0, s->P(chunk, li, B_W2), h, 0, wt(W.du), f, T, f, h, JPP_EPI_DGELU,
            nullptr, nullptr, 0, at(L.u), f, nullptr, 0, s->d.gelu_tanh));
    RC(gemm(s, st, wt(W.du), f, 0, s->P(chunk, li, B_W1), f, 0, dn, h, T, h, f, JPP_EPI_BF16));
    RC(norm_b(s, st, dn, at(L.h1), (float*)at(L.mean2), (float*)at(L.rstd2),
              s->P(chunk, li, B_ln2g), dy, wt(W.dh1), s->G(chunk, li, B_ln2g),
              s->G(chunk, li, B_ln2b)));
    RC(gemm(s, st, wt(W.dh1), h, 0, s->P(chunk, li, B_Wo), h, 0, dctx, h, T, h, h, JPP_EPI_BF16));
    attn_args(s, aa, slot, L);
    uint8_t* dqkv = (uint8_t*)wt(W.dqkv);
    aa.d_o = dctx; aa.lddo = h;
    aa.dq = dqkv; aa.dk = dqkv + h * s->es; aa.dv = dqkv + 2 * h * s->es;
    aa.lddq = aa.lddk = aa.lddv = 3 * h;
    aa.delta = s->S<float>(s->s_delta);
    RC(attn_b(s, st, &aa));
    RC(gemm(s, st, dqkv, 3 * h, 0, s->P(chunk, li, B_Wqkv), 3 * h, 0, dn, h, T, h, 3 * h,
            JPP_EPI_BF16));
    RC(norm_b(s, st, dn, at(L.x), (float*)at(L.mean1), (float*)at(L.rstd1),
              s->P(chunk, li, B_ln1g), wt(W.dh1), dx, s->G(chunk, li, B_ln1g),
              s->G(chunk, li, B_ln1b)));
    const jpp_colsum_item bias_grads[4] = {{dy, h, h, s->G(chunk, li, B_b2)},
                                           {wt(W.du), f, f, s->G(chunk, li, B_b1)},
                                           {wt(W.dh1), h, h, s->G(chunk, li, B_bo)},
                                           {dqkv, 3 * h, 3 * h, s->G(chunk, li, B_bqkv)}};
    RC(bias_grads4(s, st, bias_grads, partial));
    return JPP_OK;
  }
  // llama
  if (s->d.family == JPP_FAMILY_MIXTRAL) {
    jpp_moe_args ma;
    moe_args(s, ma, slot, L, chunk, li);
    const int E = s->d.n_experts;
    void* dxp = s->S<>(s->s_t4);
    RC(jpp_moe_bwd_prepare(st, &ma, dy, at(L.eo), (float*)wt(W.dlogits), wt(W.deo)));
    RC(ggemm(s, st, JPP_GROUP_M, ma.seg, E, wt(W.deo), h, 0, s->P(chunk, li, X_Wd), h, 0, f * h,
             wt(W.dgu), 2 * f, 0, s->cap, f, h, JPP_EPI_DSWIGLU, s->T * s->d.top_k, at(L.gu), 2 * f));
    RC(ggemm(s, st, JPP_GROUP_M, ma.seg, E, wt(W.dgu), 2 * f, 0, s->P(chunk, li, X_Wgu), 2 * f, 0,
             h * 2 * f, dxp, h, 0, s->cap, h, 2 * f, JPP_EPI_BF16, s->T * s->d.top_k));
    RC(jpp_moe_combine_bwd(st, &ma, dxp, (const float*)wt(W.dlogits), dn));
  } else {
    RC(gemm(s, st, dy, h, 0, s->P(chunk, li, L_Wd), h, 0, wt(W.dgu), 2 * f, T, f, h, JPP_EPI_DSWIGLU,
            nullptr, nullptr, 0, at(L.gu), 2 * f));
    RC(gemm(s, st, wt(W.dgu), 2 * f, 0, s->P(chunk, li, L_Wgu), 2 * f, 0, dn, h, T, h, 2 * f,
            JPP_EPI_BF16));
  }
  RC(norm_b(s, st, dn, at(L.h1), nullptr, (float*)at(L.rstd2), s->P(chunk, li, L_rms2), dy,
            wt(W.dh1), s->G(chunk, li, L_rms2), nullptr));
  RC(gemm(s, st, wt(W.dh1), h, 0, s->P(chunk, li, L_Wo), h, 0, dctx, s->ctxw, T, s->ctxw, h,
          JPP_EPI_BF16));
  attn_args(s, aa, slot, L);
  uint8_t* dqkv = (uint8_t*)wt(W.dqkv);
  aa.d_o = dctx; aa.lddo = s->ctxw;
  aa.dq = dqkv;
  aa.dk = dqkv + (int64_t)s->d.n_heads * s->hd * s->es;
  aa.dv = dqkv + (int64_t)(s->d.n_heads + s->d.n_kv_heads) * s->hd * s->es;
  aa.lddq = aa.lddk = aa.lddv = s->qkvw;
  aa.delta = s->S<float>(s->s_delta);
  if (s->f32()) {
    RC(attn_b(s, st, &aa));
    RC(rope(s, st, dqkv, 1));
  } else {
    // dq and dk leave the attention backward already rotated back
    aa.rope_cos = s->S<float>(s->s_cos);
    aa.rope_sin = s->S<float>(s->s_sin);
    RC(attn_b(s, st, &aa));
  }
  RC(gemm(s, st, dqkv, s->qkvw, 0, s->P(chunk, li, L_Wqkv), s->qkvw, 0, dn, h, T, h, s->qkvw,
          JPP_EPI_BF16));
  RC(norm_b(s, st, dn, at(L.x), nullptr, (float*)at(L.rstd1), s->P(chunk, li, L_rms1), wt(W.dh1),
            dx, s->G(chunk, li, L_rms1), nullptr));
  return JPP_OK;
}

// ---- one layer, weight-gradient half --------------------------------------------
int layer_bwd_w(jpp_stage* s, hipStream_t st, int chunk, int li, uint8_t* slot, uint8_t* wbase,
                const LayerStash& W, const void* dy) {
  // scratch for partial sums: the second stream has its own
  float* partial = s->S<float>(st == s->side && s->side ? s->s_partial_side : s->s_partial);
  const LayerStash& L = s->lay[li];
  const int64_t h = s->h, f = s->f;
  auto at = [&](const Buf& b) { return (void*)(slot + b.off); };
  auto wt = [&](const Buf& b) { return (void*)(wbase + b.off); };
  WgradBatch wb;
  if (s->d.family == JPP_FAMILY_BERT) {
    wb.add1(s, at(L.g), f, wt(W.dc), h, s->G(chunk, li, B_W2), f, h);
    wb.add1(s, at(L.x1), h, wt(W.du), f, s->G(chunk, li, B_W1), h, f);
    wb.add1(s, at(L.ctx), h, wt(W.da), h, s->G(chunk, li, B_Wo), h, h);
    wb.add1(s, at(L.x), h, wt(W.dqkv), 3 * h, s->G(chunk, li, B_Wqkv), h, 3 * h);
    return run_wgrads(s, st, wb);
  }
  if (s->d.family == JPP_FAMILY_DECODER) {
    wb.add1(s, at(L.g), f, dy, h, s->G(chunk, li, B_W2), f, h);
    wb.add1(s, at(L.n2), h, wt(W.du), f, s->G(chunk, li, B_W1), h, f);
    wb.add1(s, at(L.ctx), h, wt(W.dh1), h, s->G(chunk, li, B_Wo), h, h);
    wb.add1(s, at(L.n1), h, wt(W.dqkv), 3 * h, s->G(chunk, li, B_Wqkv), h, 3 * h);
    return run_wgrads(s, st, wb);
  }
  if (s->d.family == JPP_FAMILY_MIXTRAL) {
    jpp_moe_args ma;
    moe_args(s, ma, slot, L, chunk, li);
    const int E = s->d.n_experts;
    RC(ggemm(s, st, JPP_GROUP_K, ma.seg, E, at(L.s), f, 1, wt(W.deo), h, 1, 0, s->G(chunk, li, X_Wd), h,
             f * h, f, h, 0, JPP_EPI_ACC_F32, s->T * s->d.top_k));
    RC(ggemm(s, st, JPP_GROUP_K, ma.seg, E, at(L.xp), h, 1, wt(W.dgu), 2 * f, 1, 0,
             s->G(chunk, li, X_Wgu), 2 * f, h * 2 * f, h, 2 * f, 0, JPP_EPI_ACC_F32, s->T * s->d.top_k));
    RC(jpp_moe_router_wgrad(st, &ma, at(L.n2), (const float*)wt(W.dlogits), s->G(chunk, li, X_Wr),
                            partial));
    wb.add1(s, at(L.ctx), s->ctxw, wt(W.dh1), h, s->G(chunk, li, X_Wo), s->ctxw, h);
    wb.add1(s, at(L.n1), h, wt(W.dqkv), s->qkvw, s->G(chunk, li, X_Wqkv), h, s->qkvw);
    return run_wgrads(s, st, wb);
  }
  wb.add1(s, at(L.s), f, dy, h, s->G(chunk, li, L_Wd), f, h);
  wb.add1(s, at(L.n2), h, wt(W.dgu), 2 * f, s->G(chunk, li, L_Wgu), h, 2 * f);
  wb.add1(s, at(L.ctx), s->ctxw, wt(W.dh1), h, s->G(chunk, li, L_Wo), s->ctxw, h);
  wb.add1(s, at(L.n1), h, wt(W.dqkv), s->qkvw, s->G(chunk, li, L_Wqkv), h, s->qkvw);
  return run_wgrads(s, st, wb);
}

// Weight-gradient half of layer li for n microbatches of one chunk at once (their residuals
// and cotangents in slots[0..n-1]); the dense products run over all of them together, the
// experts' grouped products and the router's, whose row groups differ from microbatch to
// microbatch, one microbatch after the other.
int layer_bwd_w_group(jpp_stage* s, hipStream_t st, int chunk, int li, int n, uint8_t* const* slots) {
  const LayerStash& L = s->lay[li];
  const int64_t h = s->h, f = s->f;
  const void* xs[4];
  const void* dys[4];
  auto gather = [&](const Buf& x, const Buf& dy) {
    for (int i = 0; i < n; ++i) { xs[i] = slots[i] + x.off; dys[i] = slots[i] + dy.off; }
  };
  WgradBatch wb;
  if (s->d.family == JPP_FAMILY_BERT) {
    gather(L.g, L.dc);   wb.add(s, n, xs, f, dys, h, s->G(chunk, li, B_W2), f, h);
    gather(L.x1, L.du);  wb.add(s, n, xs, h, dys, f, s->G(chunk, li, B_W1), h, f);
    gather(L.ctx, L.da); wb.add(s, n, xs, h, dys, h, s->G(chunk, li, B_Wo), h, h);
    gather(L.x, L.dqkv); wb.add(s, n, xs, h, dys, 3 * h, s->G(chunk, li, B_Wqkv), h, 3 * h);
    return run_wgrads(s, st, wb);
  }
  if (s->d.family == JPP_FAMILY_DECODER) {
    gather(L.g, L.dyin);   wb.add(s, n, xs, f, dys, h, s->G(chunk, li, B_W2), f, h);
    gather(L.n2, L.du);    wb.add(s, n, xs, h, dys, f, s->G(chunk, li, B_W1), h, f);
    gather(L.ctx, L.dh1);  wb.add(s, n, xs, h, dys, h, s->G(chunk, li, B_Wo), h, h);
    gather(L.n1, L.dqkv);  wb.add(s, n, xs, h, dys, 3 * h, s->G(chunk, li, B_Wqkv), h, 3 * h);
    return run_wgrads(s, st, wb);
  }
  if (s->d.family == JPP_FAMILY_MIXTRAL) {
    float* partial = s->S<float>(st == s->side && s->side ? s->s_partial_side : s->s_partial);
    const int E = s->d.n_experts;
    // the experts' weight gradients over all n microbatches at once where the grouped
    // contraction takes several operand pairs (each with its own row groups: the routing
    // differs from microbatch to microbatch), else microbatch by microbatch
    const bool together = n > 1 && !s->f32() && s->d.fused_wgrad_accum;
    if (together) {
      auto experts = [&](const Buf& x, int64_t ldx, const Buf& dy, int64_t lddy, float* acc,
                         int64_t rows, int64_t cols) {
        jpp_gemm_args g;
        memset(&g, 0, sizeof(g));
        g.m = rows; g.n = cols; g.lda = ldx; g.ldb = lddy; g.ldc = cols;
        g.trans_a = 1; g.trans_b = 1; g.epilogue = JPP_EPI_ACC_F32;
        g.group_mode = JPP_GROUP_K; g.n_seg = E; g.stride_c = rows * cols;
        g.group_rows = (int64_t)n * s->T * s->d.top_k;
        g.c = acc; g.k_parts = n;
        for (int i = 0; i < n; ++i) {
          const int32_t* seg = (const int32_t*)(slots[i] + L.seg.off);
          const void* a = slots[i] + x.off;
          const void* b = slots[i] + dy.off;
          if (i == 0) { g.a = a; g.b = b; g.seg = seg; g.seg_rows = seg + E + 1; }
          else { g.a_more[i - 1] = a; g.b_more[i - 1] = b; g.seg_more[i - 1] = seg;
                 g.seg_rows_more[i - 1] = seg + E + 1; }
        }
        return jpp_gemm_bf16(st, &g);
      };
      RC(experts(L.s, f, L.deo, h, s->G(chunk, li, X_Wd), f, h));
      RC(experts(L.xp, h, L.dgu, 2 * f, s->G(chunk, li, X_Wgu), h, 2 * f));
    }
    for (int i = 0; i < n; ++i) {
      uint8_t* slot = slots[i];
      auto at = [&](const Buf& b) { return (void*)(slot + b.off); };
      jpp_moe_args ma;
      moe_args(s, ma, slot, L, chunk, li);
      if (!together) {
        RC(ggemm(s, st, JPP_GROUP_K, ma.seg, E, at(L.s), f, 1, at(L.deo), h, 1, 0, s->G(chunk, li, X_Wd), h,
                 f * h, f, h, 0, JPP_EPI_ACC_F32, s->T * s->d.top_k));
        RC(ggemm(s, st, JPP_GROUP_K, ma.seg, E, at(L.xp), h, 1, at(L.dgu), 2 * f, 1, 0,
                 s->G(chunk, li, X_Wgu), 2 * f, h * 2 * f, h, 2 * f, 0, JPP_EPI_ACC_F32, s->T * s->d.top_k));
      }
      RC(jpp_moe_router_wgrad(st, &ma, at(L.n2), (const float*)at(L.dlogits), s->G(chunk, li, X_Wr),
                              partial));
    }
    gather(L.ctx, L.dh1);  wb.add(s, n, xs, s->ctxw, dys, h, s->G(chunk, li, X_Wo), s->ctxw, h);
    gather(L.n1, L.dqkv);  wb.add(s, n, xs, h, dys, s->qkvw, s->G(chunk, li, X_Wqkv), h, s->qkvw);
    return run_wgrads(s, st, wb);
  }
  gather(L.s, L.dyin);   wb.add(s, n, xs, f, dys, h, s->G(chunk, li, L_Wd), f, h);
  gather(L.n2, L.dgu);   wb.add(s, n, xs, h, dys, 2 * f, s->G(chunk, li, L_Wgu), h, 2 * f);
  gather(L.ctx, L.dh1);  wb.add(s, n, xs, s->ctxw, dys, h, s->G(chunk, li, L_Wo), s->ctxw, h);
  gather(L.n1, L.dqkv);  wb.add(s, n, xs, h, dys, s->qkvw, s->G(chunk, li, L_Wqkv), h, s->qkvw);
  return run_wgrads(s, st, wb);
}

// Runs the pending weight-gradient halves of a chunk (a whole group, or what a flush finds)
// and releases their slots.  The operand pairs go into the product in microbatch order,
// whatever order the tasks arrived in.  If a launch fails, gradients of the layers above it
// have already been accumulated and nothing can take them back: the stage is marked broken
// (every later task and join reports JPP_ERR_STATE) instead of leaving entries pending that
// a later flush would accumulate a second time.
int run_pending_w(jpp_stage* s, hipStream_t st, int chunk) {
  auto& pend = s->pend[chunk];
  if (pend.empty()) return JPP_OK;
  std::sort(pend.begin(), pend.end());
  uint8_t* slots[4];
  const int n = (int)pend.size();
  for (int i = 0; i < n; ++i) slots[i] = s->slots[pend[i].second];
  int rc = JPP_OK;
  hipStream_t ws = st;
  if (s->side) {
    // the group runs on the second stream, behind everything the caller's stream holds so
    // far (the input-gradient halves that wrote the cotangents in the slots)
    JPP_CHECK_HIP(hipEventRecord(s->ev_fork, st));
    JPP_CHECK_HIP(hipStreamWaitEvent(s->side, s->ev_fork, 0));
    ws = s->side;
  }
  for (int li = s->d.layers_per_chunk - 1; li >= 0 && rc == JPP_OK; --li)
    rc = layer_bwd_w_group(s, ws, chunk, li, n, slots);
  if (s->side && rc == JPP_OK) {
    // a forward that takes one of these slots next waits for the group to have read it
    for (auto& e : pend) {
      if (hipEventRecord(s->ev_slot[e.second], s->side) != hipSuccess)
        rc = jpp_set_error(JPP_ERR_HIP, "run_task: hipEventRecord on the second stream failed");
      s->slot_pending[e.second] = 1;
    }
    if (hipEventRecord(s->ev_tail, s->side) != hipSuccess)
      rc = jpp_set_error(JPP_ERR_HIP, "run_task: hipEventRecord on the second stream failed");
    s->tail_pending = true;
  }
  for (auto& e : pend) {
    const auto key = std::make_pair(chunk, e.first);
    s->free_slots.push_back(e.second);
    s->live.erase(key);
    s->phase.erase(key);
  }
  pend.clear();
  if (rc != JPP_OK) s->broken = true;
  return rc;
}

// The input-gradient half of (chunk, mb) is done: its weight-gradient half runs now if it
// completes its group (microbatches mb / G * G .. + G - 1, in any order), else it waits; a
// microbatch of another group arriving first sends what is pending ahead as it is.
int defer_or_run_w(jpp_stage* s, hipStream_t st, int chunk, int mb, int slot_i) {
  auto& pend = s->pend[chunk];
  if (!pend.empty() && pend.front().first / s->wg != mb / s->wg) RC(run_pending_w(s, st, chunk));
  pend.emplace_back(mb, slot_i);
  if ((int)pend.size() == s->wg) RC(run_pending_w(s, st, chunk));
  return JPP_OK;
}

int flush_pending_w(jpp_stage* s, hipStream_t st) {
  for (int c = 0; c < (int)s->pend.size(); ++c) RC(run_pending_w(s, st, c));
  return JPP_OK;
}

void carve_layer(jpp_stage* s, Carver& c, LayerStash& L, bool with_w) {
  const size_t T = s->T, h = s->h, f = s->f, e = s->es;
  const size_t stat = (size_t)s->d.batch * s->d.n_heads * s->d.seq * 4;
  L.x = c.take(T * h * e);
  L.qkv = c.take(T * s->qkvw * e);
  L.ctx = c.take(T * s->ctxw * e);
  L.lse = c.take(stat);
  if (s->d.family == JPP_FAMILY_BERT) {
    L.a = c.take(T * h * e);
    L.mean1 = c.take(T * 4); L.rstd1 = c.take(T * 4);
    L.x1 = c.take(T * h * e);
    L.u = c.take(T * f * e);
    L.g = c.take(T * f * e);
    L.c = c.take(T * h * e);
    L.mean2 = c.take(T * 4); L.rstd2 = c.take(T * 4);
  } else if (s->d.family == JPP_FAMILY_DECODER) {
    L.mean1 = c.take(T * 4); L.rstd1 = c.take(T * 4);
    L.mean2 = c.take(T * 4); L.rstd2 = c.take(T * 4);
    L.n1 = c.take(T * h * e);
    L.h1 = c.take(T * h * e);
    L.n2 = c.take(T * h * e);
    L.u = c.take(T * f * e);
    L.g = c.take(T * f * e);
  } else {
    L.rstd1 = c.take(T * 4); L.rstd2 = c.take(T * 4);
    L.n1 = c.take(T * h * e);
    L.h1 = c.take(T * h * e);
    L.n2 = c.take(T * h * e);
    if (s->d.family == JPP_FAMILY_MIXTRAL) {
      const size_t cap = s->cap;
      L.ids = c.take(T * 2 * 4); L.gates = c.take(T * 2 * 4); L.row_of = c.take(T * 2 * 4);
      L.tok_of = c.take(cap * 4); L.gate_of = c.take(cap * 4); L.seg = c.take(64 * 4);
      L.xp = c.take(cap * h * e);
      L.gu = c.take(cap * 2 * f * e);
      L.s = c.take(cap * f * e);
      L.eo = c.take(cap * h * e);
    } else {
      L.gu = c.take(T * 2 * f * e);
      L.s = c.take(T * f * e);
    }
  }
  if (with_w) {
    // carved by the caller through carve_w
  }
}

void carve_w(jpp_stage* s, Carver& c, LayerStash& L) {
  const size_t T = s->T, h = s->h, f = s->f, e = s->es;
  L.dqkv = c.take(T * s->qkvw * e);
  if (s->d.family == JPP_FAMILY_BERT) {
    L.dc = c.take(T * h * e);
    L.du = c.take(T * f * e);
    L.da = c.take(T * h * e);
  } else if (s->d.family == JPP_FAMILY_DECODER) {
    L.dyin = c.take(T * h * e);
    L.du = c.take(T * f * e);
    L.dh1 = c.take(T * h * e);
  } else if (s->d.family == JPP_FAMILY_MIXTRAL) {
    L.dyin = c.take(T * h * e);
    L.dgu = c.take(s->cap * 2 * f * e);
    L.dh1 = c.take(T * h * e);
    L.deo = c.take(s->cap * h * e);
    L.dlogits = c.take(T * s->d.n_experts * 4);
  } else {
    L.dyin = c.take(T * h * e);
    L.dgu = c.take(T * 2 * f * e);
    L.dh1 = c.take(T * h * e);
  }
}

}  // namespace

extern "C" {

int jpp_stage_create(const jpp_stage_desc* d, jpp_stage** out) {
  JPP_REQUIRE(d && out, "stage_create: null");
  *out = nullptr;
  JPP_REQUIRE(d->family == JPP_FAMILY_BERT || d->family == JPP_FAMILY_LLAMA ||
                  d->family == JPP_FAMILY_MIXTRAL || d->family == JPP_FAMILY_DECODER,
              "stage_create: unknown family %d", d->family);
  if (d->family == JPP_FAMILY_MIXTRAL) {
    JPP_REQUIRE(d->n_experts == 8 && d->top_k == 2,
                "stage_create: the mixture layer is built for 8 experts, top-2");
    JPP_REQUIRE(d->hidden % 256 == 0 && d->ffn % 256 == 0,
                "stage_create: the mixture layer needs hidden and ffn multiples of 256");
    JPP_REQUIRE(d->fused_wgrad_accum, "stage_create: the mixture layer accumulates in the GEMM");
  }
  JPP_REQUIRE(d->hidden > 0 && d->n_heads > 0 && d->ffn > 0 && d->seq > 0 && d->batch > 0,
              "stage_create: bad shape");
  JPP_REQUIRE(d->n_chunks > 0 && d->layers_per_chunk > 0 && d->max_live > 0,
              "stage_create: n_chunks, layers_per_chunk and max_live must be positive");
  const int kvh = d->n_kv_heads > 0 ? d->n_kv_heads : d->n_heads;
  const int hd = d->head_dim > 0 ? d->head_dim : d->hidden / d->n_heads;
  JPP_REQUIRE(hd == 64 || hd == 128, "stage_create: head_dim must be 64 or 128, got %d", hd);
  JPP_REQUIRE(d->n_heads % kvh == 0, "stage_create: n_heads %% n_kv_heads != 0");
  const int64_t T = (int64_t)d->batch * d->seq;
  JPP_REQUIRE(T % 128 == 0 && d->seq % 128 == 0, "stage_create: seq must be a multiple of 128");
  JPP_REQUIRE(d->hidden % 128 == 0 && d->ffn % 128 == 0 && ((d->n_heads + 2 * kvh) * hd) % 128 == 0,
              "stage_create: hidden, ffn and qkv width must be multiples of 128");
  JPP_REQUIRE(d->hidden <= 8192, "stage_create: hidden > 8192 not supported by the norm kernels");
  if (d->family == JPP_FAMILY_BERT)
    JPP_REQUIRE(kvh == d->n_heads && d->n_heads * hd == d->hidden && !d->causal,
                "stage_create: the BERT layer needs n_heads*head_dim == hidden, no GQA, no mask");
  if (d->family == JPP_FAMILY_DECODER)
    JPP_REQUIRE(kvh == d->n_heads && d->n_heads * hd == d->hidden,
                "stage_create: the decoder block needs n_heads*head_dim == hidden and no GQA");

  JPP_REQUIRE(d->dtype == JPP_DTYPE_BF16 || d->dtype == JPP_DTYPE_F32, "stage_create: unknown dtype %d",
              d->dtype);
  if (d->dtype == JPP_DTYPE_F32)
    JPP_REQUIRE(d->fused_wgrad_accum,
                "stage_create: f32 stages accumulate in the weight-gradient GEMM");

  JPP_REQUIRE(d->wgrad_group >= 0 && d->wgrad_group <= 4, "stage_create: wgrad_group must be 0..4");
  if (d->wgrad_group > 1)
    JPP_REQUIRE(d->fused_wgrad_accum && d->dtype == JPP_DTYPE_BF16,
                "stage_create: grouped weight gradients need bf16 and accumulation in the GEMM");

  jpp_stage* s = new jpp_stage();
  s->d = *d;
  s->wg = d->wgrad_group > 1 ? d->wgrad_group : 1;
  s->pend.resize(d->n_chunks);
  s->es = d->dtype == JPP_DTYPE_F32 ? 4 : 2;
  s->d.n_kv_heads = kvh;
  s->d.head_dim = hd;
  s->T = T; s->h = d->hidden; s->f = d->ffn; s->hd = hd;
  s->qkvw = (int64_t)(d->n_heads + 2 * kvh) * hd;
  s->ctxw = (int64_t)d->n_heads * hd;
  const int64_t h = s->h, f = s->f;
  if (d->family == JPP_FAMILY_MIXTRAL) s->cap = jpp_moe_capacity(T, d->n_experts, d->top_k);
  if (d->family == JPP_FAMILY_MIXTRAL)
    s->pinfo = {{"rms1_g", 1, h}, {"Wqkv", h, s->qkvw}, {"Wo", s->ctxw, h}, {"rms2_g", 1, h},
                {"Wr", h, d->n_experts}, {"Wgu", d->n_experts * h, 2 * f},
                {"Wd", d->n_experts * f, h}};
  else if (d->family == JPP_FAMILY_BERT || d->family == JPP_FAMILY_DECODER)
    s->pinfo = {{"Wqkv", h, 3 * h}, {"bqkv", 1, 3 * h}, {"Wo", h, h}, {"bo", 1, h},
                {"ln1_g", 1, h}, {"ln1_b", 1, h}, {"W1", h, f}, {"b1", 1, f},
                {"W2", f, h}, {"b2", 1, h}, {"ln2_g", 1, h}, {"ln2_b", 1, h}};
  else
    s->pinfo = {{"rms1_g", 1, h}, {"Wqkv", h, s->qkvw}, {"Wo", s->ctxw, h},
                {"rms2_g", 1, h}, {"Wgu", h, 2 * f}, {"Wd", f, h}};
  size_t off = 0;
  for (auto& p : s->pinfo) {
    s->poff.push_back(off);
    off += (size_t)((p.rows * p.cols + 127) / 128 * 128);  // keep 256-byte alignment
  }
  s->layer_elems = off;

  // residual slots
  Carver slot;
  s->lay.resize(d->layers_per_chunk);
  // cotangents the weight-gradient half reads live in the slot whenever that half may run
  // in a later task than the input-gradient half
  const bool slot_w = d->split_backward || s->wg > 1;
  for (auto& L : s->lay) {
    carve_layer(s, slot, L, false);
    if (slot_w) carve_w(s, slot, L);
  }
  s->slot_bytes = slot.total;

  // scratch
  Carver sc;
  if (!slot_w)
    for (int i = 0; i < (d->two_streams ? 3 : 1); ++i) carve_w(s, sc, s->wsets[i]);
  const size_t e = s->es;
  s->s_dx[0] = sc.take(T * h * e);
  s->s_dx[1] = sc.take(T * h * e);
  const size_t rows_t = d->family == JPP_FAMILY_MIXTRAL ? (size_t)s->cap : (size_t)T;
  s->s_t1 = sc.take(d->family == JPP_FAMILY_BERT ? rows_t * h * e : 256);  // BERT: dx1
  s->s_t4 = sc.take(d->family == JPP_FAMILY_MIXTRAL ? rows_t * h * e : 256);
  s->s_moework = sc.take(d->family == JPP_FAMILY_MIXTRAL
                             ? (size_t)2 * ((T + 255) / 256) * d->n_experts * 4 + 256 : 256);
  s->s_t2 = sc.take(T * h * e);
  s->s_t3 = sc.take(T * s->ctxw * e);
  const size_t widest = (size_t)std::max<int64_t>(std::max<int64_t>(s->qkvw, 2 * f), h);
  // norm-gradient partial sums (two vectors), the router's, or a layer's four bias gradients
  s->s_partial = sc.take(std::max({(size_t)2 * JPP_NORM_PARTIALS * widest * 4,
                                   (size_t)64 * h * 8 * 4,
                                   (size_t)JPP_NORM_PARTIALS * (size_t)(5 * h + f) * 4}));
  s->s_partial_side = sc.take(d->two_streams ? (size_t)64 * h * 8 * 4 : 256);
  s->s_delta = sc.take((size_t)2 * d->batch * d->n_heads * d->seq * 4);
  size_t max_w = 0;
  for (auto& p : s->pinfo) max_w = std::max(max_w, (size_t)(p.rows * p.cols));
  // unfused path: a bf16 weight gradient; fused path: partial products of a split contraction
  // (at most 256 tiles of 128x128 in all)
  s->s_wg = sc.take(d->fused_wgrad_accum ? (size_t)256 * 128 * 128 * 4 : max_w * e);
  s->s_split = sc.take(3 * 16 * 4);  // token offsets of a contraction split in 2, 4, 8
  s->s_cos = sc.take((size_t)d->seq * (hd / 2) * 4);
  s->s_sin = sc.take((size_t)d->seq * (hd / 2) * 4);
  s->scratch_bytes = sc.total;

  const size_t n_layers = (size_t)d->n_chunks * d->layers_per_chunk;
  hipError_t e1 = hipMalloc((void**)&s->params, n_layers * s->layer_elems * s->es);
  hipError_t e2 = e1 == hipSuccess ? hipMalloc((void**)&s->grads, n_layers * s->layer_elems * 4)
                                   : e1;
  hipError_t e3 = e2 == hipSuccess ? hipMalloc((void**)&s->scratch, s->scratch_bytes) : e2;
  hipError_t e4 = e3;
  if (e3 == hipSuccess) {
    // a chunk may hold G - 1 microbatches back beyond the schedule's own peak
    const int n_slots = d->max_live + d->n_chunks * (s->wg - 1);
    for (int i = 0; i < n_slots; ++i) {
      uint8_t* p = nullptr;
      e4 = hipMalloc((void**)&p, s->slot_bytes);
      if (e4 != hipSuccess) break;
      s->slots.push_back(p);
      s->free_slots.push_back(n_slots - 1 - i);
    }
  }
  if (e4 != hipSuccess) {
    jpp_stage_destroy(s);
    return jpp_set_error(JPP_ERR_HIP, "stage_create: allocation failed: %s",
                         hipGetErrorString(e4));
  }
  s->total_bytes = n_layers * s->layer_elems * (4 + s->es) + s->scratch_bytes +
                   s->slot_bytes * s->slots.size();
  // first failure of the set-up copies below; checked once behind them
  hipError_t e_init = hipSuccess;
  auto keep = [&](hipError_t e) { if (e_init == hipSuccess) e_init = e; };
  keep(hipMemset(s->params, 0, n_layers * s->layer_elems * s->es));
  keep(hipMemset(s->grads, 0, n_layers * s->layer_elems * 4));

  {
    int32_t split[3 * 16] = {};
    for (int k = 0; k < 3; ++k)
      for (int i = 0; i <= (2 << k); ++i) split[16 * k + i] = (int32_t)(T / (2 << k) * i);
    keep(hipMemcpy(s->S<>(s->s_split), split, sizeof(split), hipMemcpyHostToDevice));
  }
  if (d->family == JPP_FAMILY_LLAMA || d->family == JPP_FAMILY_MIXTRAL) {
    // cos/sin of pos * theta^(-2i/d): evaluated in double, stored as f32
    const int half = hd / 2;
    std::vector<float> c((size_t)d->seq * half), sn((size_t)d->seq * half);
    for (int pos = 0; pos < d->seq; ++pos)
      for (int i = 0; i < half; ++i) {
        const double ang = (double)pos * pow((double)d->rope_theta, -2.0 * i / hd);
        c[(size_t)pos * half + i] = (float)cos(ang);
        sn[(size_t)pos * half + i] = (float)sin(ang);
      }
    keep(hipMemcpy(s->S<>(s->s_cos), c.data(), c.size() * 4, hipMemcpyHostToDevice));
    keep(hipMemcpy(s->S<>(s->s_sin), sn.data(), sn.size() * 4, hipMemcpyHostToDevice));
  }
  if (e_init != hipSuccess) {
    jpp_stage_destroy(s);
    return jpp_set_error(JPP_ERR_HIP, "stage_create: clearing or filling the stage's buffers "
                         "failed: %s", hipGetErrorString(e_init));
  }
  hipError_t e5 = hipSuccess;
  if (d->two_streams) {
    // default priority; non-blocking so that it does not serialise against the null stream
    e5 = hipStreamCreateWithFlags(&s->side, hipStreamNonBlocking);
    auto mk = [&](hipEvent_t* ev) {
      if (e5 == hipSuccess) e5 = hipEventCreateWithFlags(ev, hipEventDisableTiming);
    };
    mk(&s->ev_fork);
    mk(&s->ev_tail);
    for (auto& ev : s->ev_set) mk(&ev);
    s->ev_slot.assign(s->slots.size(), nullptr);
    s->ev_bwd_i.assign(s->slots.size(), nullptr);
    s->slot_pending.assign(s->slots.size(), 0);
    for (auto& ev : s->ev_slot) mk(&ev);
    for (auto& ev : s->ev_bwd_i) mk(&ev);
  }
  if (e5 == hipSuccess) e5 = hipDeviceSynchronize();
  if (e5 != hipSuccess) {
    jpp_stage_destroy(s);
    return jpp_set_error(JPP_ERR_HIP, "stage_create: %s", hipGetErrorString(e5));
  }
  *out = s;
  return JPP_OK;
}

int jpp_stage_destroy(jpp_stage* s) {
  if (!s) return JPP_OK;
  hipDeviceSynchronize();
  auto drop = [](hipEvent_t ev) { if (ev) hipEventDestroy(ev); };
  drop(s->ev_fork);
  drop(s->ev_tail);
  for (auto ev : s->ev_set) drop(ev);
  for (auto ev : s->ev_slot) drop(ev);
  for (auto ev : s->ev_bwd_i) drop(ev);
  if (s->side) hipStreamDestroy(s->side);
  for (auto p : s->slots) hipFree(p);
  if (s->scratch) hipFree(s->scratch);
  for (auto p : s->opt)
    if (p) hipFree(p);
  if (s->grads) hipFree(s->grads);
  if (s->params) hipFree(s->params);
  delete s;
  return JPP_OK;
}

int jpp_stage_n_params(const jpp_stage* s) { return s ? (int)s->pinfo.size() : 0; }

int jpp_stage_param_info(const jpp_stage* s, int i, const char** name, int64_t* rows,
                         int64_t* cols) {
  JPP_REQUIRE(s && i >= 0 && i < (int)s->pinfo.size(), "param_info: bad index %d", i);
  if (name) *name = s->pinfo[i].name;
  if (rows) *rows = s->pinfo[i].rows;
  if (cols) *cols = s->pinfo[i].cols;
  return JPP_OK;
}

static int check_pli(const jpp_stage* s, int chunk, int layer, int i) {
  JPP_REQUIRE(s, "stage: null");
  JPP_REQUIRE(chunk >= 0 && chunk < s->d.n_chunks && layer >= 0 && layer < s->d.layers_per_chunk &&
                  i >= 0 && i < (int)s->pinfo.size(),
              "stage: (chunk %d, layer %d, param %d) out of range", chunk, layer, i);
  return JPP_OK;
}

int jpp_stage_param_ptr(jpp_stage* s, int chunk, int layer, int i, void** ptr) {
  RC(check_pli(s, chunk, layer, i));
  *ptr = s->P(chunk, layer, i);
  return JPP_OK;
}

int jpp_stage_grad_ptr(jpp_stage* s, int chunk, int layer, int i, float** ptr) {
  RC(check_pli(s, chunk, layer, i));
  *ptr = s->G(chunk, layer, i);
  return JPP_OK;
}

int jpp_stage_join(jpp_stage* s, void* stream) {
  JPP_REQUIRE(s, "stage: null");
  if (s->broken)
    return jpp_set_error(JPP_ERR_STATE, "stage_join: a grouped weight-gradient launch of this "
                         "stage failed earlier; its accumulators are incomplete");
  RC(flush_pending_w(s, (hipStream_t)stream));   // weight gradients held back for their group
  if (s->tail_pending) JPP_CHECK_HIP(hipStreamWaitEvent((hipStream_t)stream, s->ev_tail, 0));
  return JPP_OK;
}

int jpp_stage_quiesce(jpp_stage* s) {
  JPP_REQUIRE(s, "stage: null");
  for (auto& pend : s->pend)
    if (!pend.empty())
      return jpp_set_error(JPP_ERR_STATE, "stage_quiesce: weight gradients of %d microbatch(es) are "
                           "held back for their group; call jpp_stage_join first", (int)pend.size());
  if (s->side) JPP_CHECK_HIP(hipStreamSynchronize(s->side));
  // nothing of the stage's own stream is in flight: no later task has to wait for it
  std::fill(s->slot_pending.begin(), s->slot_pending.end(), 0);
  for (auto& p : s->set_pending) p = false;
  s->tail_pending = false;
  return JPP_OK;
}

int jpp_stage_zero_grads(jpp_stage* s, void* stream) {
  JPP_REQUIRE(s, "stage: null");
  RC(jpp_stage_join(s, stream));  // weight gradients still in flight accumulate into the old values
  const size_t n = (size_t)s->d.n_chunks * s->d.layers_per_chunk * s->layer_elems;
  return jpp_fill_u32(s->grads, 0u, n, stream);
}

int jpp_stage_optimizer_init(jpp_stage* s, void* stream) {
  JPP_REQUIRE(s, "stage: null");
  const size_t n = (size_t)s->d.n_chunks * s->d.layers_per_chunk * s->layer_elems;
  for (auto& p : s->opt)
    if (!p && !(s->f32() && &p == &s->opt[0])) {   // f32 parameters are their own f32 weights
      if (hipMalloc((void**)&p, n * 4) != hipSuccess) {
        p = nullptr;
        (void)hipGetLastError();
        return jpp_set_error(JPP_ERR_HIP, "optimizer_init: cannot allocate %zu bytes of state", n * 4);
      }
      s->total_bytes += n * 4;
    }
  if (!s->f32()) RC(jpp_cast_bf16_to_f32(stream, s->params, s->opt[0], (int64_t)n));
  RC(jpp_fill_u32(s->opt[1], 0u, n, stream));
  return jpp_fill_u32(s->opt[2], 0u, n, stream);
}

int jpp_stage_opt_ptr(jpp_stage* s, int which, int chunk, int layer, int i, float** ptr) {
  RC(check_pli(s, chunk, layer, i));
  JPP_REQUIRE(which >= 0 && which < 3, "opt_ptr: which = %d, expected 0 (weights), 1 (m) or 2 (v)",
              which);
  JPP_REQUIRE(s->opt[which == 0 && s->f32() ? 1 : which],
              "opt_ptr: jpp_stage_optimizer_init has not run");
  float* base = which == 0 && s->f32() ? (float*)s->params : s->opt[which];
  *ptr = base + (s->G(chunk, layer, i) - s->grads);
  return JPP_OK;
}

int jpp_stage_adam_step(jpp_stage* s, void* stream, int64_t step, double lr, double beta1,
                        double beta2, double eps, double grad_scale) {
  JPP_REQUIRE(s, "stage: null");
  JPP_REQUIRE((s->opt[0] || s->f32()) && s->opt[1] && s->opt[2],
              "adam_step: jpp_stage_optimizer_init has not run");
  RC(jpp_stage_join(s, stream));  // weight gradients may still be running on the second stream
  jpp_adam_args a;
  a.count = (int64_t)s->d.n_chunks * s->d.layers_per_chunk * (int64_t)s->layer_elems;
  a.grad = s->grads;
  a.master = s->f32() ? (float*)s->params : s->opt[0];
  a.param = s->f32() ? nullptr : s->params;
  a.m = s->opt[1];
  a.v = s->opt[2];
  a.step = step;
  a.lr = lr; a.beta1 = beta1; a.beta2 = beta2; a.eps = eps;
  a.grad_scale = grad_scale;
  a.zero_grad = 1;
  return jpp_adam_step(stream, &a);
}

int jpp_stage_routing(jpp_stage* s, int chunk, int mb, int layer, int32_t* ids, float* gates,
                      void* stream) {
  JPP_REQUIRE(s, "stage_routing: null stage");
  JPP_REQUIRE(s->d.family == JPP_FAMILY_MIXTRAL, "stage_routing: not a mixture-of-experts stage");
  JPP_REQUIRE(chunk >= 0 && chunk < s->d.n_chunks && layer >= 0 && layer < s->d.layers_per_chunk,
              "stage_routing: (chunk %d, layer %d) out of range", chunk, layer);
  JPP_REQUIRE(ids || gates, "stage_routing: nothing to copy");
  auto it = s->live.find(std::make_pair(chunk, mb));
  if (it == s->live.end())
    return jpp_set_error(JPP_ERR_STATE, "stage_routing: (chunk %d, mubatch %d) holds no residuals",
                         chunk, mb);
  const uint8_t* slot = s->slots[it->second];
  const LayerStash& L = s->lay[layer];
  const size_t n = (size_t)s->T * s->d.top_k * 4;
  if (ids)
    JPP_CHECK_HIP(hipMemcpyAsync(ids, slot + L.ids.off, n, hipMemcpyDeviceToDevice, (hipStream_t)stream));
  if (gates)
    JPP_CHECK_HIP(hipMemcpyAsync(gates, slot + L.gates.off, n, hipMemcpyDeviceToDevice,
                                 (hipStream_t)stream));
  return JPP_OK;
}

size_t jpp_stage_bytes(const jpp_stage* s) { return s ? s->total_bytes : 0; }
int jpp_stage_live_slots(const jpp_stage* s) { return s ? (int)s->live.size() : 0; }

int jpp_stage_run_task(jpp_stage* s, int kind, int chunk, int mb, const void* in, void* out,
                       void* stream) {
  JPP_REQUIRE(s, "run_task: null stage");
  if (s->broken)
    return jpp_set_error(JPP_ERR_STATE, "run_task: a grouped weight-gradient launch of this stage "
                         "failed earlier; its accumulators are incomplete");
  JPP_REQUIRE(chunk >= 0 && chunk < s->d.n_chunks, "run_task: chunk %d out of range", chunk);
  hipStream_t st = (hipStream_t)stream;
  const int nl = s->d.layers_per_chunk;
  const size_t act = (size_t)s->T * s->h * s->es;
  const auto key = std::make_pair(chunk, mb);

  if (kind == JPP_FWD) {
    JPP_REQUIRE(in && out, "run_task(FWD): needs in and out");
    if (s->live.count(key))
      return jpp_set_error(JPP_ERR_STATE, "run_task(FWD): (chunk %d, mubatch %d) is already live",
                           chunk, mb);
    if (s->free_slots.empty())
      return jpp_set_error(JPP_ERR_STATE,
                           "run_task(FWD): all %d residual slots are live; the schedule needs a "
                           "larger max_live", (int)s->slots.size());
    const int slot_i = s->free_slots.back();
    s->free_slots.pop_back();
    s->live[key] = slot_i;
    s->phase[key] = 1;
    uint8_t* slot = s->slots[slot_i];
    if (s->side && s->slot_pending[slot_i]) {
      // weight gradients of the slot's previous microbatch may still be reading it
      JPP_CHECK_HIP(hipStreamWaitEvent(st, s->ev_slot[slot_i], 0));
      s->slot_pending[slot_i] = 0;
    }
    JPP_CHECK_HIP(hipMemcpyAsync(slot + s->lay[0].x.off, in, act, hipMemcpyDeviceToDevice, st));
    for (int li = 0; li < nl; ++li) {
      void* y = li + 1 < nl ? (void*)(slot + s->lay[li + 1].x.off) : out;
      RC(layer_fwd(s, st, chunk, li, slot, y));
    }
    return JPP_OK;
  }

  auto it = s->live.find(key);
  if (it == s->live.end())
    return jpp_set_error(JPP_ERR_STATE, "run_task: no forward residuals for (chunk %d, mubatch %d)",
                         chunk, mb);
  uint8_t* slot = s->slots[it->second];
  const int ph = s->phase[key];
  const bool split = s->d.split_backward != 0;

  const bool two = s->side != nullptr;
  const int slot_i = it->second;
  // queue `side` behind what the caller's stream holds so far
  auto fork = [&]() -> int {
    JPP_CHECK_HIP(hipEventRecord(s->ev_fork, st));
    JPP_CHECK_HIP(hipStreamWaitEvent(s->side, s->ev_fork, 0));
    return JPP_OK;
  };
  // `side` has read the slot for the last time in this task
  auto side_done_with_slot = [&]() -> int {
    JPP_CHECK_HIP(hipEventRecord(s->ev_slot[slot_i], s->side));
    s->slot_pending[slot_i] = 1;
    JPP_CHECK_HIP(hipEventRecord(s->ev_tail, s->side));
    s->tail_pending = true;
    return JPP_OK;
  };

  if (kind == JPP_BWD || kind == JPP_BWD_I) {
    JPP_REQUIRE(in && out, "run_task(BWD): needs in and out");
    if (ph != 1)
      return jpp_set_error(JPP_ERR_STATE, "run_task: backward of (chunk %d, mubatch %d) ran twice",
                           chunk, mb);
    if (kind == JPP_BWD_I && !split)
      return jpp_set_error(JPP_ERR_STATE,
                           "run_task(BWD_I): stage was created without split_backward");
    const bool bert = s->d.family == JPP_FAMILY_BERT;
    // cotangent set of layer li when they live in scratch
    auto set_of = [&](int li) { return two ? ((li % 3) + 3) % 3 : 0; };
    auto wait_set = [&](int k) -> int {
      if (two && s->set_pending[k]) {
        JPP_CHECK_HIP(hipStreamWaitEvent(st, s->ev_set[k], 0));
        s->set_pending[k] = false;
      }
      return JPP_OK;
    };
    const bool slot_w = split || s->wg > 1;   // cotangents for the weight gradients: in the slot
    const void* dy = in;
    for (int li = nl - 1; li >= 0; --li) {
      uint8_t* wbase = slot_w ? slot : s->scratch;
      const LayerStash& W = slot_w ? s->lay[li] : s->wsets[set_of(li)];
      if (!slot_w) {
        // this layer writes its own set and (its result) the set of the layer below
        RC(wait_set(set_of(li)));
        if (li > 0 && !bert) RC(wait_set(set_of(li - 1)));
      }
      void* dx;
      if (li == 0) dx = out;
      else if (slot_w && !bert) dx = slot + s->lay[li - 1].dyin.off;
      else if (two && !bert) dx = s->scratch + s->wsets[set_of(li - 1)].dyin.off;
      else dx = s->S<>(s->s_dx[li & 1]);
      if (!bert && li == nl - 1 && (slot_w || two)) {
        // the weight gradients read the incoming cotangent later (a BWD_W task, or the
        // second stream after this call has returned): keep a copy
        uint8_t* keep = wbase + W.dyin.off;
        JPP_CHECK_HIP(hipMemcpyAsync(keep, in, act, hipMemcpyDeviceToDevice, st));
        dy = keep;
      }
      RC(layer_bwd_i(s, st, chunk, li, slot, wbase, W, dy, dx));
      if (kind == JPP_BWD && s->wg == 1) {
        if (two) {
          RC(fork());
          RC(layer_bwd_w(s, s->side, chunk, li, slot, wbase, W, dy));
          if (!split) {
            JPP_CHECK_HIP(hipEventRecord(s->ev_set[set_of(li)], s->side));
            s->set_pending[set_of(li)] = true;
          }
        } else {
          RC(layer_bwd_w(s, st, chunk, li, slot, wbase, W, dy));
        }
      }
      dy = dx;
    }
    if (kind == JPP_BWD && s->wg > 1) {
      s->phase[key] = 3;                       // both halves issued or handed to the group
      RC(defer_or_run_w(s, st, chunk, mb, slot_i));
    } else if (kind == JPP_BWD) {
      if (two) RC(side_done_with_slot());
      s->free_slots.push_back(slot_i);
      s->live.erase(it);
      s->phase.erase(key);
    } else {
      if (two) JPP_CHECK_HIP(hipEventRecord(s->ev_bwd_i[slot_i], st));
      s->phase[key] = 2;
    }
    return JPP_OK;
  }

  if (kind == JPP_BWD_W) {
    if (!split)
      return jpp_set_error(JPP_ERR_STATE,
                           "run_task(BWD_W): stage was created without split_backward");
    if (ph != 2)
      return jpp_set_error(JPP_ERR_STATE, "run_task(BWD_W): BWD_I of (chunk %d, mubatch %d) has not run",
                           chunk, mb);
    if (s->wg > 1) {
      s->phase[key] = 3;
      return defer_or_run_w(s, st, chunk, mb, slot_i);
    }
    hipStream_t ws = st;
    if (two) {
      // everything it needs was complete when the BWD_I task ended on the caller's stream
      JPP_CHECK_HIP(hipStreamWaitEvent(s->side, s->ev_bwd_i[slot_i], 0));
      ws = s->side;
    }
    for (int li = nl - 1; li >= 0; --li)
      RC(layer_bwd_w(s, ws, chunk, li, slot, slot, s->lay[li], slot + s->lay[li].dyin.off));
    if (two) RC(side_done_with_slot());
    s->free_slots.push_back(slot_i);
    s->live.erase(it);
    s->phase.erase(key);
    return JPP_OK;
  }
  return jpp_set_error(JPP_ERR_INVALID, "run_task: unknown task kind %d", kind);
}

}  // extern "C"
