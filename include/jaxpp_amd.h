/* jaxpp_amd -- C ABI of the MI355X stage executor and its kernels.
 *
 * The reference (NVIDIA/jaxpp, Python on JAX/XLA) has no native interface for
 * this path; what this library replaces is
 *   - the op seam: the XLA executable a stage task compiles to
 *     (src/jaxpp/jax_primitives.py:704-730, `callable_task` / `apply_task`),
 *     i.e. the GEMM / attention / norm / activation / accumulate kernels; and
 *   - the task seam: `task_impl` dispatching one (stage, kind, microbatch)
 *     task on device buffers (src/jaxpp/jax_primitives.py:776-859).
 * Each entry point below names the reference construct it stands in for.
 *
 * Conventions
 *   - plain C, POD arguments, device pointers owned by the caller unless
 *     stated; nothing here takes or returns framework tensor types;
 *   - every function returns 0 (JPP_OK) or a negative jpp_status and never
 *     throws or aborts; jpp_last_error() returns the thread's last message;
 *   - kernels are enqueued on the given HIP stream and never synchronise;
 *   - `stream` is a hipStream_t passed as void* (NULL = default stream);
 *   - bf16 tensors are raw uint16 bit patterns, row-major, leading dimension
 *     in elements.
 */
#ifndef JAXPP_AMD_H_
#define JAXPP_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  JPP_OK = 0,
  JPP_ERR_INVALID = -1, /* shape / alignment / argument violation, found on host */
  JPP_ERR_HIP = -2,     /* a HIP runtime call or launch failed */
  JPP_ERR_STATE = -3    /* task order violates residual lifetimes */
} jpp_status;

/* TaskType of the reference (src/jaxpp/types.py:79-96); same integer values. */
typedef enum { JPP_FWD = 1, JPP_BWD = 2, JPP_BWD_I = 3, JPP_BWD_W = 4 } jpp_task_kind;

/* Layer families.  BERT: post-LN encoder layer (the README's FlaxBertLayer stack,
 * README.md:46-72); DECODER: the pre-LN causal block with biases and a GELU feed-forward of
 * the reference's example model (examples/basic.py:33-91); LLAMA and MIXTRAL: RMSNorm, RoPE,
 * GQA, SwiGLU / top-2 of 8 experts (the shapes the headline configurations name). */
typedef enum {
  JPP_FAMILY_BERT = 0, JPP_FAMILY_LLAMA = 1, JPP_FAMILY_MIXTRAL = 2, JPP_FAMILY_DECODER = 3
} jpp_family;

const char* jpp_last_error(void);
int jpp_version(void);

/* ---- device plumbing for hosts that have no GPU runtime of their own ------
 * (a ctypes / FFI host; under JAX, XLA owns buffers and streams instead) */
int jpp_device_count(int* count);
int jpp_set_device(int device);
int jpp_malloc(void** ptr, size_t bytes);
int jpp_free(void* ptr);
int jpp_memcpy_h2d(void* dst, const void* src, size_t bytes);
int jpp_memcpy_d2h(void* dst, const void* src, size_t bytes);
int jpp_memcpy_d2d_async(void* dst, const void* src, size_t bytes, void* stream);
int jpp_fill_u32(void* dst, uint32_t value, size_t count, void* stream);
int jpp_stream_create(void** stream);
int jpp_stream_destroy(void* stream);
int jpp_stream_sync(void* stream);
int jpp_device_sync(void);
int jpp_event_create(void** event);
int jpp_event_destroy(void* event);
int jpp_event_record(void* event, void* stream);
int jpp_stream_wait_event(void* stream, void* event); /* later work on stream waits for event */
int jpp_event_sync(void* event);
int jpp_event_elapsed_ms(void* start, void* stop, float* ms);
int jpp_mem_info(size_t* free_bytes, size_t* total_bytes);
/* HIP graphs.  Every entry point of this library only enqueues work on the stream it is
 * given (and, for a stage with two_streams, on a stream forked from and joined to it with
 * events), allocates nothing and clears memory with kernels, so a sequence of calls can be
 * recorded between begin and end and replayed with launch - a rank's whole row of the task
 * table, for instance.  The reference leaves this to XLA (command buffers); a jax.ffi handler
 * over these entry points may be marked command-buffer compatible for the same reason.
 * Record after one eager pass (first launches set kernel attributes) and jpp_stage_quiesce,
 * on a stream created with jpp_stream_create; call jpp_stage_join on the recording stream
 * before end; record whole rows of the table (every forward with its backward); probes
 * (jpp_probe_begin) stay off while recording. */
int jpp_graph_begin(void* stream);
int jpp_graph_end(void* stream, void** graph_exec);
int jpp_graph_launch(void* graph_exec, void* stream);
int jpp_graph_destroy(void* graph_exec);

/* ---- launch probe: per-kernel timings, the counterpart of the reference's
 * collect_task_times_ms (src/jaxpp/jax_primitives.py:742-773) at kernel
 * granularity.  Between begin and end every launch of the named kernel class
 * is bracketed by HIP events on the stream it is launched on; end waits for
 * them and returns the number of launches, their summed duration and the
 * algorithmic FLOPs / HBM bytes the launchers declared.  Class names:
 *   gemm_<nn|nt|tn>_<bf16|gelu|dgelu|accf32|f32>_<BM>x<BN>   (nn: y = x W,
 *       nt: dx = dy W^T, tn: dW = x^T dy)
 *   (+ "w8" for 8-wave tiles, "s3"/"s4" for 3 or 4 LDS stages),
 *   attn_fwd, attn_bwd_dq, attn_bwd_dkv, norm_fwd, norm_bwd, swiglu_fwd,
 *   swiglu_bwd, rope, grad_accum, colsum, adam */
int jpp_probe_begin(const char* kernel_class);
int jpp_probe_end(int64_t* launches, double* total_ms, double* total_flops, double* total_bytes);
/* With jpp_probe_begin("*") every class is bracketed and jpp_probe_end returns the totals over
 * all of them; jpp_probe_class then reads class `index` (0, 1, ... until JPP_ERR_INVALID) of
 * the probe that has just ended: its name (valid until the next jpp_probe_begin) and its own
 * figures.  Further classes: sum_accum, mse, fill, cast, moe_route, moe_gather,
 * moe_combine_fwd, moe_bwd_prepare, moe_combine_bwd, moe_router_wgrad. */
int jpp_probe_class(int index, const char** name, int64_t* launches, double* total_ms,
                    double* total_flops, double* total_bytes);

/* ---- GEMM: stands in for the `dot_general`s of a stage task ----------------
 * C[M,N] = epilogue( sum_k Aop[m,k] * Bop[n,k] ), bf16 operands, fp32 MFMA
 * accumulation.
 *   trans_a = 0: A is [M,K] (lda >= K);  1: A is [K,M] (lda >= M)
 *   trans_b = 0: B is [N,K] (ldb >= K);  1: B is [K,N] (ldb >= N)
 * so  y = x W      -> trans_a 0, trans_b 1   (W stored [in,out])
 *     dx = dy W^T  -> trans_a 0, trans_b 0
 *     dW = x^T dy  -> trans_a 1, trans_b 1
 * M and N must be multiples of 128, K of 64; all pointers 16-byte aligned and
 * leading dimensions multiples of 8. */
typedef enum {
  JPP_EPI_BF16 = 0,    /* C(bf16) = acc [+ bias[n]] [+ resid[m,n]]                     */
  JPP_EPI_GELU = 1,    /* u = acc + bias;  C = u,  C2 = gelu(u)   (both bf16)          */
  JPP_EPI_DGELU = 2,   /* C(bf16) = acc * gelu'(aux[m,n])                              */
  JPP_EPI_ACC_F32 = 3, /* C(f32) += acc      (the `add prev_acc g` of a backward task) */
  JPP_EPI_F32 = 4,     /* C(f32) = acc                                                 */
  /* SwiGLU with gate and up projections interleaved in blocks of 32 columns: column 64q+w of
   * the fused projection is gate feature 32q+w for w < 32 and up feature 32q+w-32 otherwise. */
  JPP_EPI_SWIGLU = 5,  /* C(bf16) = acc (N = 2f, interleaved);
                          C2[m, 32q+w] = silu(C[m, 64q+w]) * C[m, 64q+32+w]   (bf16, [M, f]) */
  JPP_EPI_DSWIGLU = 6  /* acc = ds [M, N = f]; aux = the interleaved gate/up [M, 2f];
                          C (bf16, [M, 2f], interleaved) = d(gate), d(up) of silu(gate)*up      */
} jpp_epilogue;

typedef struct {
  const void* a;
  const void* b;
  void* c;
  void* c2;          /* second output (JPP_EPI_GELU, JPP_EPI_SWIGLU) */
  const void* bias;  /* bf16 [N] or NULL */
  const void* resid; /* bf16 [M,N] or NULL */
  const void* aux;   /* bf16 [M,N] (JPP_EPI_DGELU), [M,2N] (JPP_EPI_DSWIGLU) */
  int64_t m, n, k;
  int64_t lda, ldb, ldc, ldc2, ldresid, ldaux;
  int trans_a, trans_b;
  int epilogue;      /* jpp_epilogue */
  int gelu_tanh;     /* 0: erf form, 1: tanh approximation */
  int tile;          /* 0: choose (may run the last, half-empty round of 256x256 tiles as a second
                        launch of 128x256 tiles); 1: 128x128; 2: 256x128; 3: 128x256; 4: 256x256
                        (8 waves each) */
  /* grouped GEMM over experts (0 = plain).  seg: device int32 [n_seg + 1], row
   * offsets of the expert groups in the token-permuted buffers, multiples of 256.
   *   JPP_GROUP_M: rows of A and C are grouped; group e multiplies b + e * stride_b.
   *                m is the capacity of the permuted buffer; tiles past seg[n_seg] exit.
   *                With tile = 0 and JPP_EPI_BF16 the product is up to three launches: when
   *                the 256x256 tiles of the seg[n_seg] rows in use end in a round that fills
   *                at most half of the CUs, that round's rows are 128x128 or 128x256 tiles
   *                (same bits).
   *   JPP_GROUP_K: (weight gradients) C_e = c + e * stride_c gets the product over the
   *                rows seg[e] .. seg[e+1] (multiples of 64) of A and B; k is ignored.  Also
   *                the way to split one long contraction over workgroups: equal ranges, an
   *                f32 epilogue into scratch, then jpp_sum_accum_f32. */
  const int32_t* seg;
  int n_seg;
  int group_mode;
  int64_t stride_b, stride_c;
  int64_t group_rows; /* non-padding rows over all groups, for the probe's FLOP and byte
                       * accounting only (0: the padded extent is counted) */
  const int32_t* seg_rows; /* device int32 [n_seg] or NULL: rows of each group that hold data;
                            * the rest of a group is zero padding, which JPP_GROUP_K then leaves
                            * out of the contraction (whole 64-row steps of it) */
  /* One product over several operand pairs: with k_parts = 2..4 the contraction runs over
   * (a, b), then (a_more[0], b_more[0]), ... - k elements each, same shapes and leading
   * dimensions - as if the pairs were concatenated along the contraction index.  The
   * weight gradients of several microbatches accumulate this way with one read and one write
   * of the fp32 accumulator instead of one per microbatch.  0 or 1: one pair.  Built for
   * trans_a = trans_b = 1 with JPP_EPI_ACC_F32 on the 256-wide tiles: N a multiple of 256,
   * `tile` 0 (the library then takes 256x256, or 128x256 when M is not a multiple of 256),
   * 3 or 4; anything else is JPP_ERR_INVALID. */
  const void* a_more[3];
  const void* b_more[3];
  int k_parts;
  /* JPP_GROUP_K over several operand pairs: pair i > 0 has its own row groups,
   * seg_more[i-1] (device int32 [n_seg + 1]) and, if seg_rows is given, seg_rows_more[i-1]
   * (device int32 [n_seg]); C_e then gets the products over group e of every pair (the expert
   * weight gradients of several microbatches, whose routing differs). */
  const int32_t* seg_more[3];
  const int32_t* seg_rows_more[3];
  /* Rotary embedding in the epilogue (JPP_EPI_BF16, trans_a = 0, trans_b = 1, no bias, residual
   * or groups; NULL: none): columns [0, rope_cols) of C are heads of rope_head_dim (64 or 128)
   * elements, row r of C is position r % rope_seq, and the tables are f32
   * [rope_seq, rope_head_dim / 2] as for jpp_rope.  The product is rounded to bf16, rotated and
   * rounded again: the very values jpp_rope leaves when run over the plain result. */
  const float* rope_cos;
  const float* rope_sin;
  int64_t rope_cols;
  int rope_seq, rope_head_dim;
} jpp_gemm_args;

enum { JPP_GROUP_NONE = 0, JPP_GROUP_M = 1, JPP_GROUP_K = 2 };

int jpp_gemm_bf16(void* stream, const jpp_gemm_args* args);

/* Up to four independent accumulated weight gradients - every problem with trans_a = trans_b =
 * 1, JPP_EPI_ACC_F32, no groups, M and N multiples of 256, the same k and k_parts - as ONE
 * grid of 256x256 tiles, problem after problem.  Stands where the reference's weight-gradient
 * task holds several independent dot_generals (one per parameter of the layer,
 * src/jaxpp/jaxpr_utils.py:138-167 puts them all into BWD_W): launched one by one, each leaves
 * its last round of tiles partly empty (a 6144 x 4096 gradient is 384 tiles on 256 CUs);
 * together they close up.  Every output element is computed by one workgroup in a fixed order
 * (deterministic), the same order as in a single launch on 256x256 tiles; a single launch that
 * runs its last round on 128x256 tiles adds the old accumulator value at another point of the
 * sum there, so the two agree to fp32 rounding.  n_problems = 1 is jpp_gemm_bf16. */
int jpp_gemm_bf16_multi(void* stream, const jpp_gemm_args* problems, int n_problems);

/* ---- fused attention (softmax(QK^T/sqrt(d)) V), forward and backward -------
 * q: [batch*seq, *] with head h at columns h*head_dim (row stride ldq); k, v
 * likewise with n_kv_heads heads; query head h reads kv head h / (n_heads /
 * n_kv_heads).  lse: f32 [batch, n_heads, seq], natural-log sum-exp of the
 * scaled scores.  head_dim 64 or 128; seq a multiple of 128. */
typedef struct {
  const void* q; const void* k; const void* v;
  void* o;                  /* fwd: out; bwd: in */
  float* lse;               /* fwd: out; bwd: in */
  const void* d_o;          /* bwd */
  void* dq; void* dk; void* dv;
  float* delta;             /* bwd scratch, f32 [batch, n_heads, seq, 2] (JPP_WS_ATTN_DELTA) */
  int64_t ldq, ldk, ldv, ldo, lddo, lddq, lddk, lddv;
  int batch, seq, n_heads, n_kv_heads, head_dim, causal;
  /* Backward only, optional (NULL: off): f32 [seq, head_dim/2] tables of the half-split rotary
   * embedding the caller applied to q and k before the forward.  dq and dk are then written
   * already rotated back (by the negative angle), i.e. as jpp_rope(..., inverse = 1) would
   * leave them: the cotangents of the un-rotated q and k, without a pass of their own. */
  const float* rope_cos;
  const float* rope_sin;
} jpp_attn_args;

int jpp_attn_fwd(void* stream, const jpp_attn_args* args);
int jpp_attn_bwd(void* stream, const jpp_attn_args* args);

/* ---- scratch sizes ---------------------------------------------------------
 * Bytes of the caller-provided scratch buffer an operator needs (under JAX: what the FFI
 * handler asks the scratch allocator for).  d0, d1, d2 per operator; 0 for an unknown one. */
typedef enum {
  JPP_WS_NORM_BWD = 0,         /* jpp_norm_args.partial: d0 = cols */
  JPP_WS_COLSUM = 1,           /* jpp_colsum_accum(_multi) partial: d0 = cols (summed over the tensors) */
  JPP_WS_ATTN_DELTA = 2,       /* jpp_attn_args.delta: d0 = batch, d1 = n_heads, d2 = seq */
  JPP_WS_MSE = 3,              /* jpp_mse_loss partial */
  JPP_WS_MOE_WORK = 4,         /* jpp_moe_args.work: d0 = tokens, d1 = n_experts */
  JPP_WS_MOE_ROUTER_WGRAD = 5, /* jpp_moe_router_wgrad partial: d0 = hidden, d1 = n_experts */
  JPP_WS_SPLIT_WGRAD = 6       /* `parts` of jpp_sum_accum_f32: d0 = n_parts, d1 = rows, d2 = cols */
} jpp_workspace_op;
size_t jpp_workspace_bytes(int op, int64_t d0, int64_t d1, int64_t d2);

/* ---- row-wise norms ---------------------------------------------------------
 * x, y, dy, dx: bf16 [rows, cols]; gamma/beta bf16 [cols]; mean/rstd f32
 * [rows].  The backward adds `resid` (bf16, may be NULL) to dx, and
 * accumulates the parameter gradients into the f32 arrays dgamma / dbeta
 * (`+=`, fixed summation order) using `partial` (f32 [2 * JPP_NORM_PARTIALS *
 * cols]) as scratch.  beta == NULL and mean == NULL select RMSNorm. */
#define JPP_NORM_PARTIALS 256
typedef struct {
  const void* x; const void* gamma; const void* beta;
  void* y; float* mean; float* rstd;
  const void* dy; const void* resid; void* dx;
  float* dgamma; float* dbeta; float* partial;
  int64_t rows, cols;
  float eps;
} jpp_norm_args;

int jpp_norm_fwd(void* stream, const jpp_norm_args* args);
int jpp_norm_bwd(void* stream, const jpp_norm_args* args);
/* No counterpart in the reference.  jpp_norm_bwd for callers that cannot allocate device
 * memory and have no workspace to pass (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): `args->partial` is ignored and the partial sums go to a
 * buffer the library holds itself in static device memory (16 MiB per GPU, for the whole
 * life of the process).  Same kernels, same summation order and bit-identical results as
 * jpp_norm_bwd; cols <= 8192 (more is JPP_ERR_INVALID).  It calls no allocating routine
 * (while a launch probe is active the probe's events are created as for any entry point).
 * The first call on a device looks the buffer's address up (hipGetSymbolAddress): make that
 * call outside a graph capture.  All calls on one GPU share the buffer, so two calls that
 * overlap on one GPU (different streams, or two host threads) race; calls on one stream do
 * not. */
int jpp_norm_bwd_static(void* stream, const jpp_norm_args* args);

/* ---- elementwise ------------------------------------------------------------ */
/* s[t,j] = silu(gate[t,j]) * up[t,j]; backward writes dgu [T,2f] in gu's layout.
 * interleaved = 0: gu = [gate | up] halves; 1: blocks of 32 columns as for JPP_EPI_SWIGLU. */
int jpp_swiglu_fwd(void* stream, const void* gu, void* s, int64_t rows, int64_t f,
                   int interleaved);
int jpp_swiglu_bwd(void* stream, const void* gu, const void* ds, void* dgu, int64_t rows,
                   int64_t f, int interleaved);
/* Half-split rotary embedding applied in place to the first n_rot_heads heads
 * of each row (q and k heads are adjacent in a packed qkv row); cos/sin: f32
 * [seq, head_dim/2]; inverse != 0 rotates by the negative angle (backward). */
int jpp_rope(void* stream, void* x, int64_t ld, const float* cos_tab, const float* sin_tab,
             int batch, int seq, int n_rot_heads, int head_dim, int inverse);
/* acc[i] += g[i]; g is bf16 (g_is_f32 == 0) or f32.  The gradient accumulation
 * of `treduce`'s Add (src/jaxpp/training.py:112-123) as a standalone pass. */
int jpp_grad_accum_f32(void* stream, float* acc, const void* g, int64_t count, int g_is_f32);
/* acc[i] += parts[0][i] + parts[1][i] + ... + parts[n_parts-1][i], summed in that order;
 * parts: f32 [n_parts, count].  Closes a contraction that was split over workgroups
 * (JPP_GROUP_K with an f32 epilogue into `parts`) without making the result depend on timing. */
int jpp_sum_accum_f32(void* stream, float* acc, const float* parts, int n_parts, int64_t count);
/* acc[j] += sum_t x[t,j] (bias gradients); partial: f32 [JPP_NORM_PARTIALS*cols]. */
int jpp_colsum_accum(void* stream, const void* x, int64_t ld, int64_t rows, int64_t cols,
                     float* acc, float* partial);
/* The same for up to 4 tensors of `rows` rows in one pair of launches (the bias gradients of
 * a layer); partial: f32 [JPP_NORM_PARTIALS * sum of cols]. */
typedef struct {
  const void* x;     /* bf16 [rows, cols], leading dimension ld */
  int64_t ld, cols;  /* multiples of 8 */
  float* acc;        /* f32 [cols], added to */
} jpp_colsum_item;
int jpp_colsum_accum_multi(void* stream, int n, const jpp_colsum_item* items, int64_t rows,
                           float* partial);
/* Loss of the last stage as in the reference's examples (README.md:76-78):
 * loss[0] = scale * mean((out - target)^2) over `count` bf16 elements, and its
 * cotangent dout = scale * 2 (out - target) / count (bf16).  partial: f32
 * [JPP_NORM_PARTIALS] scratch; the reduction order is fixed. */
int jpp_mse_loss(void* stream, const void* out, const void* target, int64_t count, float scale,
                 float* loss, void* dout, float* partial);
int jpp_cast_f32_to_bf16(void* stream, const float* src, void* dst, int64_t count);
int jpp_cast_bf16_to_f32(void* stream, const void* src, float* dst, int64_t count);

/* ---- the same operators on f32 tensors -----------------------------------------
 * The full-precision flavour of a stage (jpp_stage_desc.dtype = JPP_DTYPE_F32): the
 * reference's CPU-runnable configuration is float32 end to end (BERT-style stack of
 * hidden 256; tests/test_transformations.py:42-93 also builds its model in float32).
 * Same argument structs, every bf16 tensor replaced by an f32 one; plain fp32 arithmetic
 * in a fixed summation order, sized for small problems (not for the matrix cores).
 * jpp_gemm_f32: M, N multiples of 64, K of 16; every epilogue of jpp_gemm_bf16
 * (JPP_EPI_BF16 = store in the element type, with bias and residual) and both grouped modes
 * (group offsets multiples of 64; a grouped contraction runs over the padded extent).
 * jpp_attn_*_f32: seq a multiple of 64.  jpp_norm_bwd_f32 does not use `partial`. */
int jpp_gemm_f32(void* stream, const jpp_gemm_args* args);
int jpp_attn_fwd_f32(void* stream, const jpp_attn_args* args);
int jpp_attn_bwd_f32(void* stream, const jpp_attn_args* args);
int jpp_norm_fwd_f32(void* stream, const jpp_norm_args* args);
int jpp_norm_bwd_f32(void* stream, const jpp_norm_args* args);
int jpp_rope_f32(void* stream, float* x, int64_t ld, const float* cos_tab, const float* sin_tab,
                 int batch, int seq, int n_rot_heads, int head_dim, int inverse);
int jpp_colsum_accum_f32(void* stream, const float* x, int64_t ld, int64_t rows, int64_t cols,
                         float* acc);
int jpp_mse_loss_f32(void* stream, const float* out, const float* target, int64_t count,
                     float scale, float* loss, float* dout);

/* ---- after the loop: the optimizer on the accumulated gradients --------------
 * The reference's train step applies `optimizer.update(grad, opt_state, pars)` and
 * `optax.apply_updates` to what `treduce` returns (README.md:90-93; examples/basic.py:234
 * builds the optimizer with `optax.adam`).  One fused pass over a flat tensor:
 *   g  = grad_scale * grad
 *   m  = beta1 m + (1 - beta1) g          v = beta2 v + (1 - beta2) g^2
 *   w -= lr (m / (1 - beta1^step)) / (sqrt(v / (1 - beta2^step)) + eps)
 * in f32, then param = bf16(w).  `master` holds the f32 weights; without it the bf16
 * `param` is the only copy (read, updated in f32, rounded back).  With zero_grad the
 * accumulator is cleared in the same pass, ready for the next loop. */
typedef struct {
  int64_t count;
  float* grad;        /* f32 [count]: the loop's gradient accumulator */
  float* master;      /* f32 [count] weights, updated in place; may be NULL */
  void* param;        /* bf16 [count] weights, rewritten; may be NULL when master is given */
  float* m;           /* f32 [count] first moment, updated in place */
  float* v;           /* f32 [count] second moment, updated in place */
  int64_t step;       /* 1 for the first update */
  /* doubles, so that 1 - beta and the bias corrections are formed as the reference's
   * Python floats form them before they meet f32 data */
  double lr, beta1, beta2, eps;
  double grad_scale;  /* e.g. 1 / n_mubatches when the loss is not already divided */
  int zero_grad;
} jpp_adam_args;
int jpp_adam_step(void* stream, const jpp_adam_args* args);

/* ---- top-2 mixture of experts: routing around the grouped GEMMs --------------
 * Tokens are assigned to rows of "permuted" buffers, grouped by expert in token
 * order, each group padded to a multiple of 256 rows (padding rows are zero);
 * jpp_moe_capacity() rows always suffice.  seg[e] is the first row of expert e. */
enum jpp_dtype { JPP_DTYPE_BF16 = 0, JPP_DTYPE_F32 = 1 };

typedef struct {
  const void* x;     /* bf16 [tokens, hidden]: router input (jpp_moe_route only) */
  const void* wr;    /* bf16 [hidden, n_experts] */
  int32_t* ids;      /* [tokens, 2] selected experts, by descending logit (ties: lower id) */
  float* gates;      /* [tokens, 2] softmax over the two selected logits */
  int32_t* row_of;   /* [tokens, 2] row of each assignment */
  int32_t* tok_of;   /* [capacity] token of each row, -1 for padding */
  float* gate_of;    /* [capacity] gate of each row */
  int32_t* seg;      /* [2 n_experts + 1]: first row of each group and the end of the last,
                        then the number of rows of each group that hold tokens */
  void* work;        /* int32 [2 * ceil(tokens / 256) * n_experts] scratch */
  int64_t tokens, hidden;
  int n_experts, top_k; /* 8, 2 */
  int dtype;            /* jpp_dtype of x, wr and of every activation tensor passed beside the
                           struct (bf16 in the comments here and below: f32 when JPP_DTYPE_F32) */
} jpp_moe_args;

int64_t jpp_moe_capacity(int64_t tokens, int n_experts, int top_k);
int jpp_moe_route(void* stream, const jpp_moe_args* args);
/* xp[row] = x[tok_of[row]] */
int jpp_moe_gather(void* stream, const jpp_moe_args* args, const void* x, void* xp);
/* y[t] = resid[t] + sum_k gates[t,k] * eo[row_of[t,k]] */
int jpp_moe_combine_fwd(void* stream, const jpp_moe_args* args, const void* eo, const void* resid,
                        void* y);
/* dlogits f32 [tokens, n_experts]; deo[row] = gate_of[row] * dy[tok_of[row]] */
int jpp_moe_bwd_prepare(void* stream, const jpp_moe_args* args, const void* dy, const void* eo,
                        float* dlogits, void* deo);
/* dx[t] = dxp[row_of[t,0]] + dxp[row_of[t,1]] + dlogits[t] Wr^T */
int jpp_moe_combine_bwd(void* stream, const jpp_moe_args* args, const void* dxp,
                        const float* dlogits, void* dx);
/* acc[hidden, n_experts] += x^T dlogits; partial: f32 [64 * hidden * n_experts] */
int jpp_moe_router_wgrad(void* stream, const jpp_moe_args* args, const void* x,
                         const float* dlogits, float* acc, float* partial);

/* ---- stage executor: stands in for `task_impl` on one pipeline rank ----------
 * A stage object holds this rank's chunks (the stages the schedule places on
 * it), their parameters (bf16, or f32: `dtype`), the f32 gradient accumulators (the loop carry of
 * `treduce`), and a ring of residual slots sized for the schedule's peak
 * number of live microbatches (src/jaxpp/core.py:1732-1890 decides the same
 * lifetimes by donation and explicit deletes). */
typedef struct jpp_stage jpp_stage;

typedef struct {
  int family;            /* jpp_family */
  int hidden, n_heads, n_kv_heads, head_dim, ffn, seq, batch;
  int causal;
  float rope_theta;
  float eps;
  int gelu_tanh;
  int n_experts, top_k;
  int n_chunks;          /* stages held by this rank */
  int layers_per_chunk;
  int max_live;          /* residual slots */
  int split_backward;    /* 1: BWD_I / BWD_W tasks will be issued separately */
  int fused_wgrad_accum; /* 1: accumulate in the weight-gradient GEMM epilogue;
                            0: bf16 gradient then jpp_grad_accum_f32 */
  int two_streams;       /* 1: weight-gradient work (BWD_W tasks, and the weight-gradient half
                            of BWD tasks) runs on a second HIP stream owned by the stage, forked
                            from and ordered against the caller's stream with events; it may
                            still be running when jpp_stage_run_task returns control of the
                            caller's stream - see jpp_stage_join */
  int dtype;             /* jpp_dtype of parameters, activations and boundary tensors.
                            JPP_DTYPE_F32: every family, through the *_f32 operators and the
                            routing kernels' f32 form; gradient accumulators are f32 either way */
  int wgrad_group;       /* 0, 1: each microbatch's weight gradients run in the task the table
                            gives them.  2..4: the weight gradients of the microbatches
                            g * wgrad_group .. + wgrad_group - 1 of a chunk run together, when
                            the last of them is due, as one product per weight over all their
                            tokens - the fp32 accumulator is then read and written once per
                            group instead of once per microbatch.  A microbatch held back keeps
                            its residual slot (the stage allocates wgrad_group - 1 slots per
                            chunk beyond max_live, and jpp_stage_live_slots counts them);
                            jpp_stage_join runs what is still held back, so call it (or
                            jpp_stage_zero_grads / jpp_stage_adam_step, which do) before reading
                            the accumulators.  Groups are fixed by microbatch index and a
                            group's operand pairs enter its product in microbatch order, so
                            the accumulators do not depend on the order in which the members
                            of a group arrive; a member of another group of the same chunk
                            arriving in between sends what is pending ahead as a shorter
                            product (same sums, other rounding).  If a grouped launch fails
                            the stage is unusable: every later task and join returns
                            JPP_ERR_STATE.  bf16 and fused_wgrad_accum only.  With
                            two_streams a group runs on the stage's second stream, behind
                            the input-gradient half of its last member. */
} jpp_stage_desc;


int jpp_stage_create(const jpp_stage_desc* desc, jpp_stage** out);
int jpp_stage_destroy(jpp_stage* stage);
/* Parameters of one layer, in a fixed order per family. */
int jpp_stage_n_params(const jpp_stage* stage);
int jpp_stage_param_info(const jpp_stage* stage, int index, const char** name, int64_t* rows,
                         int64_t* cols);
/* bf16 parameter / f32 accumulator storage of (chunk, layer, index). */
int jpp_stage_param_ptr(jpp_stage* stage, int chunk, int layer, int index, void** ptr);
int jpp_stage_grad_ptr(jpp_stage* stage, int chunk, int layer, int index, float** ptr);
int jpp_stage_zero_grads(jpp_stage* stage, void* stream);
/* Makes `stream` wait for everything the stage has in flight on its own stream (weight
 * gradients, with two_streams).  Call it before reading the accumulators on `stream`;
 * jpp_stage_zero_grads does it by itself.  A no-op without two_streams. */
int jpp_stage_join(jpp_stage* stage, void* stream);
/* Blocks the host until the stage's own stream is idle and forgets the events later tasks
 * would otherwise wait for.  For use before recording a graph: a recording may not depend on
 * work that was queued before it began. */
int jpp_stage_quiesce(jpp_stage* stage);
/* Optimizer state of a stage: f32 weights (cast up from the bf16 parameters as they are
 * now) and zeroed moments, laid out like the parameters; allocated by the first call,
 * reset by later ones (call it again after writing parameters through
 * jpp_stage_param_ptr).  `which` of jpp_stage_opt_ptr: 0 f32 weights, 1 m, 2 v. */
int jpp_stage_optimizer_init(jpp_stage* stage, void* stream);
int jpp_stage_opt_ptr(jpp_stage* stage, int which, int chunk, int layer, int index, float** ptr);
/* jpp_adam_step over every parameter of the stage (one launch), clearing the gradient
 * accumulators; joins the stage's second stream first. */
int jpp_stage_adam_step(jpp_stage* stage, void* stream, int64_t step, double lr, double beta1,
                        double beta2, double eps, double grad_scale);
size_t jpp_stage_bytes(const jpp_stage* stage);
/* One task.  `in` is the incoming boundary activation (FWD) or cotangent
 * (BWD, BWD_I), `out` receives the outgoing activation / cotangent; both are
 * bf16 [batch*seq, hidden] and may be reused by the caller once the call has
 * returned (stream order).  BWD_W takes neither.  A BWD_I that is never
 * followed by BWD_W leaves its slot occupied. */
int jpp_stage_run_task(jpp_stage* stage, int kind, int chunk, int mubatch, const void* in,
                       void* out, void* stream);
int jpp_stage_live_slots(const jpp_stage* stage);
/* Mixture-of-experts stages: the routing a forward task chose for one layer of a live
 * (chunk, microbatch) - between its FWD and the task that releases its residuals - copied on
 * `stream` into caller-owned device buffers: ids int32 [tokens, top_k] (experts by descending
 * logit) and gates f32 [tokens, top_k]; either may be NULL.  The reference leaves routing to
 * the user's model; a host needs it for load statistics and auxiliary losses, and the parity
 * tests to hold the oracle to the device's choice where router logits tie within rounding. */
int jpp_stage_routing(jpp_stage* stage, int chunk, int mubatch, int layer, int32_t* ids,
                      float* gates, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* JAXPP_AMD_H_ */
