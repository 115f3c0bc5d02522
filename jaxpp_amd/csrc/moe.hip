// Top-2 mixture-of-experts routing around the grouped GEMMs: router, stable
// token -> expert-row assignment with 256-row padded groups, gather, combine,
// and their backward.  Everything is deterministic: positions come from
// prefix sums in token order, reductions run in a fixed order.
#include <math.h>

#include <algorithm>

#include "common.h"

namespace {

constexpr int kE = 8;        // experts
constexpr int kPad = 256;    // expert groups start at multiples of the GEMM tile height

// 8 consecutive elements of a bf16 or an f32 tensor
__device__ __forceinline__ void load8(const bf16_t* p, float (&f)[8]) {
  unpack8(*(const uint4*)p, f);
}
__device__ __forceinline__ void load8(const float* p, float (&f)[8]) {
  const float4 a = ((const float4*)p)[0], b = ((const float4*)p)[1];
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w;
  f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}
__device__ __forceinline__ void store8(bf16_t* p, const float (&f)[8]) { *(uint4*)p = pack8(f); }
__device__ __forceinline__ void store8(float* p, const float (&f)[8]) {
  ((float4*)p)[0] = make_float4(f[0], f[1], f[2], f[3]);
  ((float4*)p)[1] = make_float4(f[4], f[5], f[6], f[7]);
}
__device__ __forceinline__ void copy8(const bf16_t* src, bf16_t* dst) { *(uint4*)dst = *(const uint4*)src; }
__device__ __forceinline__ void copy8(const float* src, float* dst) {
  ((float4*)dst)[0] = ((const float4*)src)[0];
  ((float4*)dst)[1] = ((const float4*)src)[1];
}
__device__ __forceinline__ float to_f32(bf16_t v) { return bf16_to_f32(v); }
__device__ __forceinline__ float to_f32(float v) { return v; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// logits = x Wr (fp32), top-2 by value (ties -> lower index), gates = softmax
// over the two selected logits.  One wave per token.
template <typename El>
__global__ __launch_bounds__(256) void router_kernel(const El* __restrict__ x,
                                                     const El* __restrict__ wr, long T, int h,
                                                     int* __restrict__ ids,
                                                     float* __restrict__ gates) {
  const int lane = threadIdx.x & 63;
  const long t = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  float acc[kE];
#pragma unroll
  for (int e = 0; e < kE; ++e) acc[e] = 0.f;
  for (int c = lane; c < h / 8; c += 64) {
    float xv[8];
    load8(x + t * h + c * 8, xv);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float w[8];
      load8(wr + (long)(c * 8 + j) * kE, w);
#pragma unroll
      for (int e = 0; e < kE; ++e) acc[e] += xv[j] * w[e];
    }
  }
#pragma unroll
  for (int e = 0; e < kE; ++e) acc[e] = wave_sum(acc[e]);
  if (lane == 0) {
    int i0 = 0;
    for (int e = 1; e < kE; ++e)
      if (acc[e] > acc[i0]) i0 = e;
    int i1 = i0 == 0 ? 1 : 0;
    for (int e = 0; e < kE; ++e)
      if (e != i0 && acc[e] > acc[i1]) i1 = e;
    const float g0 = 1.0f / (1.0f + expf(acc[i1] - acc[i0]));
    ids[t * 2] = i0; ids[t * 2 + 1] = i1;
    gates[t * 2] = g0; gates[t * 2 + 1] = 1.0f - g0;
  }
}

// per block of 256 tokens: how many assignments each expert receives
__global__ __launch_bounds__(256) void count_kernel(const int* __restrict__ ids, long T,
                                                    int* __restrict__ cnt) {
  __shared__ int hist[kE];
  if (threadIdx.x < kE) hist[threadIdx.x] = 0;
  __syncthreads();
  const long t = (long)blockIdx.x * 256 + threadIdx.x;
  if (t < T) {
    atomicAdd(&hist[ids[t * 2]], 1);
    atomicAdd(&hist[ids[t * 2 + 1]], 1);
  }
  __syncthreads();
  if (threadIdx.x < kE) cnt[blockIdx.x * kE + threadIdx.x] = hist[threadIdx.x];
}

// seg[e]: first row of expert e (multiple of 256), seg[kE + 1 + e]: its number of tokens;
// base[blk][e]: first row of the block's assignments to e.  One thread per expert.
__global__ void scan_kernel(const int* __restrict__ cnt, int nblk, int* __restrict__ seg,
                            int* __restrict__ base) {
  __shared__ int total[kE];
  const int e = threadIdx.x;
  if (e < kE) {
    int s = 0;
    for (int b = 0; b < nblk; ++b) {
      base[b * kE + e] = s;
      s += cnt[b * kE + e];
    }
    total[e] = s;
  }
  __syncthreads();
  if (e == 0) {
    int at = 0;
    for (int i = 0; i < kE; ++i) {
      seg[i] = at;
      at += (total[i] + kPad - 1) / kPad * kPad;
    }
    seg[kE] = at;
    for (int i = 0; i < kE; ++i) seg[kE + 1 + i] = total[i];
  }
  __syncthreads();
  if (e < kE)
    for (int b = 0; b < nblk; ++b) base[b * kE + e] += seg[e];
}

// rows in token order inside each expert group
__global__ __launch_bounds__(256) void assign_kernel(const int* __restrict__ ids,
                                                     const float* __restrict__ gates, long T,
                                                     const int* __restrict__ base,
                                                     int* __restrict__ row_of,
                                                     int* __restrict__ tok_of,
                                                     float* __restrict__ gate_of) {
  __shared__ int wave_cnt[4][kE];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long t = (long)blockIdx.x * 256 + threadIdx.x;
  const int i0 = t < T ? ids[t * 2] : -1, i1 = t < T ? ids[t * 2 + 1] : -1;
  int before[2] = {0, 0};
#pragma unroll
  for (int e = 0; e < kE; ++e) {
    const bool mine = i0 == e || i1 == e;
    const unsigned long long m = __ballot(mine);
    const int prefix = __popcll(m & ((1ull << lane) - 1));
    if (i0 == e) before[0] = prefix;
    if (i1 == e) before[1] = prefix;
    if (lane == 0) wave_cnt[wave][e] = __popcll(m);
  }
  __syncthreads();
  if (t < T) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int e = k ? i1 : i0;
      int row = base[blockIdx.x * kE + e] + before[k];
      for (int w = 0; w < wave; ++w) row += wave_cnt[w][e];
      row_of[t * 2 + k] = row;
      tok_of[row] = (int)t;
      gate_of[row] = gates[t * 2 + k];
    }
  }
}

// xp[row] = x[tok_of[row]] (zero for padding rows)
template <typename El>
__global__ __launch_bounds__(256) void gather_kernel(const El* __restrict__ x,
                                                     const int* __restrict__ tok_of,
                                                     const int* __restrict__ seg, int h,
                                                     El* __restrict__ xp) {
  const int hc = h / 8;
  const long rows = seg[kE];
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < rows * hc; i += (long)gridDim.x * 256) {
    const long row = i / hc;
    const int c = (int)(i - row * hc);
    const int t = tok_of[row];
    if (t >= 0) {
      copy8(x + (long)t * h + c * 8, xp + row * h + c * 8);
    } else {
      const float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      store8(xp + row * h + c * 8, z);
    }
  }
}

// y[t] = resid[t] + sum_k gate[t,k] * eo[row_of[t,k]]
template <typename El>
__global__ __launch_bounds__(256) void combine_fwd_kernel(const El* __restrict__ eo,
                                                          const int* __restrict__ row_of,
                                                          const float* __restrict__ gates,
                                                          const El* __restrict__ resid, long T,
                                                          int h, El* __restrict__ y) {
  const int hc = h / 8;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < T * hc; i += (long)gridDim.x * 256) {
    const long t = i / hc;
    const int c = (int)(i - t * hc);
    float r[8], a[8], b[8];
    load8(resid + t * h + c * 8, r);
    load8(eo + (long)row_of[t * 2] * h + c * 8, a);
    load8(eo + (long)row_of[t * 2 + 1] * h + c * 8, b);
    const float g0 = gates[t * 2], g1 = gates[t * 2 + 1];
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (r[e] + g0 * a[e]) + g1 * b[e];
    store8(y + t * h + c * 8, r);
  }
}

// d(gate) and d(logits): one wave per token
template <typename El>
__global__ __launch_bounds__(256) void gate_bwd_kernel(const El* __restrict__ dy,
                                                       const El* __restrict__ eo,
                                                       const int* __restrict__ row_of,
                                                       const int* __restrict__ ids,
                                                       const float* __restrict__ gates, long T,
                                                       int h, float* __restrict__ dlogits) {
  const int lane = threadIdx.x & 63;
  const long t = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  const El* e0 = eo + (long)row_of[t * 2] * h;
  const El* e1 = eo + (long)row_of[t * 2 + 1] * h;
  float d0 = 0.f, d1 = 0.f;
  for (int c = lane; c < h / 8; c += 64) {
    float g[8], a[8], b[8];
    load8(dy + t * h + c * 8, g);
    load8(e0 + c * 8, a);
    load8(e1 + c * 8, b);
#pragma unroll
    for (int e = 0; e < 8; ++e) { d0 += g[e] * a[e]; d1 += g[e] * b[e]; }
  }
  d0 = wave_sum(d0);
  d1 = wave_sum(d1);
  if (lane < kE) {
    const float g0 = gates[t * 2], g1 = gates[t * 2 + 1];
    const float dot = g0 * d0 + g1 * d1;
    float v = 0.f;
    if (lane == ids[t * 2]) v = g0 * (d0 - dot);
    if (lane == ids[t * 2 + 1]) v = g1 * (d1 - dot);
    dlogits[t * kE + lane] = v;
  }
}

// deo[row] = gate_of[row] * dy[tok_of[row]] (zero for padding rows)
template <typename El>
__global__ __launch_bounds__(256) void scatter_dy_kernel(const El* __restrict__ dy,
                                                         const int* __restrict__ tok_of,
                                                         const float* __restrict__ gate_of,
                                                         const int* __restrict__ seg, int h,
                                                         El* __restrict__ deo) {
  const int hc = h / 8;
  const long rows = seg[kE];
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < rows * hc; i += (long)gridDim.x * 256) {
    const long row = i / hc;
    const int c = (int)(i - row * hc);
    const int t = tok_of[row];
    float f[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (t >= 0) {
      load8(dy + (long)t * h + c * 8, f);
      const float g = gate_of[row];
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] *= g;
    }
    store8(deo + row * h + c * 8, f);
  }
}

// dx[t] = dxp[row_of[t,0]] + dxp[row_of[t,1]] + dlogits[t] Wr^T.  A thread owns 8 columns and
// keeps their 8 x 8 router weights in registers; the workgroup walks tokens together, so a
// token's rows and logit gradients are the same address for every lane (scalar loads) and
// the vector memory path carries the two expert rows and the result only.
template <typename El>
__global__ __launch_bounds__(256) void combine_bwd_kernel(const El* __restrict__ dxp,
                                                          const int* __restrict__ row_of,
                                                          const float* __restrict__ dlogits,
                                                          const El* __restrict__ wr, long T,
                                                          int h, El* __restrict__ dx) {
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= h / 8) return;
  float w[8][kE];
#pragma unroll
  for (int j = 0; j < 8; ++j) load8(wr + (long)(c * 8 + j) * kE, w[j]);
  for (long t = blockIdx.x; t < T; t += gridDim.x) {
    float a[8], b[8], dl[kE];
    load8(dxp + (long)row_of[t * 2] * h + c * 8, a);
    load8(dxp + (long)row_of[t * 2 + 1] * h + c * 8, b);
#pragma unroll
    for (int e = 0; e < kE; ++e) dl[e] = dlogits[t * kE + e];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float r = 0.f;
#pragma unroll
      for (int e = 0; e < kE; ++e) r += dl[e] * w[j][e];
      a[j] = (a[j] + b[j]) + r;
    }
    store8(dx + t * h + c * 8, a);
  }
}

// dWr[j, e] += sum_t x[t, j] * dlogits[t, e]: block (row panel b, column panel)
// writes partial[b][j][e]; wr_reduce sums the panels in order
template <typename El>
__global__ __launch_bounds__(256) void wr_partial_kernel(const El* __restrict__ x,
                                                         const float* __restrict__ dlogits, long T,
                                                         int h, float* __restrict__ partial) {
  // a thread owns 8 columns (one 16-byte piece of a bf16 row per token); a column's terms are
  // added in token order
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= h / 8) return;
  float acc[8][kE];
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int e = 0; e < kE; ++e) acc[j][e] = 0.f;
  // (few workgroups for this much data: 16 row pieces per lane in flight keep memory busy)
#pragma unroll 16
  for (long t = blockIdx.x; t < T; t += gridDim.x) {
    float xv[8], dl[kE];
    load8(x + t * h + c * 8, xv);
#pragma unroll
    for (int e = 0; e < kE; ++e) dl[e] = dlogits[t * kE + e];
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int e = 0; e < kE; ++e) acc[j][e] += xv[j] * dl[e];
  }
  float* dst = partial + ((long)blockIdx.x * h + c * 8) * kE;
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int e = 0; e < kE; ++e) dst[j * kE + e] = acc[j][e];
}
__global__ __launch_bounds__(256) void wr_reduce_kernel(const float* __restrict__ partial, int nb,
                                                        long n, float* __restrict__ acc) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float s = 0.f;
#pragma unroll 16
  for (int b = 0; b < nb; ++b) s += partial[(long)b * n + i];
  acc[i] += s;
}

__global__ __launch_bounds__(256) void fill_i32_kernel(int* dst, int v, long n) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256)
    dst[i] = v;
}

int grid_for(long items, int cap = 8192) {
  long g = (items + 255) / 256;
  return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}

}  // namespace

extern "C" {

int64_t jpp_moe_capacity(int64_t tokens, int n_experts, int top_k) {
  return (tokens * top_k + (int64_t)n_experts * (kPad - 1) + kPad - 1) / kPad * kPad;
}

int jpp_moe_route(void* stream, const jpp_moe_args* a) {
  JPP_REQUIRE(a && a->x && a->wr && a->ids && a->gates && a->row_of && a->tok_of && a->gate_of &&
                  a->seg && a->work,
              "moe_route: null operand");
  JPP_REQUIRE(a->n_experts == kE && a->top_k == 2, "moe_route: built for 8 experts, top-2");
  JPP_REQUIRE(a->tokens > 0 && a->hidden % 8 == 0, "moe_route: bad shape");
  JPP_REQUIRE(a->dtype == JPP_DTYPE_BF16 || a->dtype == JPP_DTYPE_F32, "moe_route: unknown dtype %d",
              a->dtype);
  hipStream_t st = (hipStream_t)stream;
  ProbeScope probe(st, "moe_route", 0, (a->dtype == JPP_DTYPE_F32 ? 4.0 : 2.0) * a->tokens * a->hidden);   // reads x once
  const long T = a->tokens;
  const int nblk = (int)((T + 255) / 256);
  int* cnt = (int*)a->work;
  int* base = cnt + (long)nblk * kE;
  const long cap = jpp_moe_capacity(T, kE, 2);
  if (a->dtype == JPP_DTYPE_F32) {
    hipLaunchKernelGGL(router_kernel<float>, dim3((unsigned)((T + 3) / 4)), dim3(256), 0, st,
                       (const float*)a->x, (const float*)a->wr, T, (int)a->hidden, a->ids, a->gates);
  } else {
    hipLaunchKernelGGL(router_kernel<bf16_t>, dim3((unsigned)((T + 3) / 4)), dim3(256), 0, st,
                       (const bf16_t*)a->x, (const bf16_t*)a->wr, T, (int)a->hidden, a->ids, a->gates);
  }
  hipLaunchKernelGGL(fill_i32_kernel, dim3(grid_for(cap)), dim3(256), 0, st, a->tok_of, -1, cap);
  hipLaunchKernelGGL(count_kernel, dim3(nblk), dim3(256), 0, st, a->ids, T, cnt);
  hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(64), 0, st, cnt, nblk, a->seg, base);
  hipLaunchKernelGGL(assign_kernel, dim3(nblk), dim3(256), 0, st, a->ids, a->gates, T, base,
                     a->row_of, a->tok_of, a->gate_of);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_moe_gather(void* stream, const jpp_moe_args* a, const void* x, void* xp) {
  JPP_REQUIRE(a && x && xp, "moe_gather: null operand");
  const long cap = jpp_moe_capacity(a->tokens, kE, 2);
  ProbeScope probe((hipStream_t)stream, "moe_gather", 0, 2 * (a->dtype == JPP_DTYPE_F32 ? 4.0 : 2.0) * a->tokens * a->top_k * a->hidden);
  if (a->dtype == JPP_DTYPE_F32) {
    hipLaunchKernelGGL(gather_kernel<float>, dim3(grid_for(cap * (a->hidden / 8))), dim3(256), 0,
                       (hipStream_t)stream, (const float*)x, a->tok_of, a->seg, (int)a->hidden,
                       (float*)xp);
  } else {
    hipLaunchKernelGGL(gather_kernel<bf16_t>, dim3(grid_for(cap * (a->hidden / 8))), dim3(256), 0,
                       (hipStream_t)stream, (const bf16_t*)x, a->tok_of, a->seg, (int)a->hidden,
                       (bf16_t*)xp);
  }
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_moe_combine_fwd(void* stream, const jpp_moe_args* a, const void* eo, const void* resid,
                        void* y) {
  JPP_REQUIRE(a && eo && resid && y, "moe_combine_fwd: null operand");
  ProbeScope probe((hipStream_t)stream, "moe_combine_fwd", 0,
                   (a->dtype == JPP_DTYPE_F32 ? 4.0 : 2.0) * a->tokens * a->hidden * (a->top_k + 2));   // top_k rows + residual in, y out
  if (a->dtype == JPP_DTYPE_F32) {
    hipLaunchKernelGGL(combine_fwd_kernel<float>, dim3(grid_for(a->tokens * (a->hidden / 8))), dim3(256), 0,
                       (hipStream_t)stream, (const float*)eo, a->row_of, a->gates,
                       (const float*)resid, (long)a->tokens, (int)a->hidden, (float*)y);
  } else {
    hipLaunchKernelGGL(combine_fwd_kernel<bf16_t>, dim3(grid_for(a->tokens * (a->hidden / 8))), dim3(256), 0,
                       (hipStream_t)stream, (const bf16_t*)eo, a->row_of, a->gates,
                       (const bf16_t*)resid, (long)a->tokens, (int)a->hidden, (bf16_t*)y);
  }
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_moe_bwd_prepare(void* stream, const jpp_moe_args* a, const void* dy, const void* eo,
                        float* dlogits, void* deo) {
  JPP_REQUIRE(a && dy && eo && dlogits && deo, "moe_bwd_prepare: null operand");
  hipStream_t st = (hipStream_t)stream;
  // gate gradients read dy and top_k rows of eo; the scatter reads dy again per copy, writes deo
  ProbeScope probe(st, "moe_bwd_prepare", 0, (a->dtype == JPP_DTYPE_F32 ? 4.0 : 2.0) * a->tokens * a->hidden * (1 + 3 * a->top_k));
  const long cap = jpp_moe_capacity(a->tokens, kE, 2);
  if (a->dtype == JPP_DTYPE_F32) {
    hipLaunchKernelGGL(gate_bwd_kernel<float>, dim3((unsigned)((a->tokens + 3) / 4)), dim3(256), 0, st,
                       (const float*)dy, (const float*)eo, a->row_of, a->ids, a->gates,
                       (long)a->tokens, (int)a->hidden, dlogits);
  } else {
    hipLaunchKernelGGL(gate_bwd_kernel<bf16_t>, dim3((unsigned)((a->tokens + 3) / 4)), dim3(256), 0, st,
                       (const bf16_t*)dy, (const bf16_t*)eo, a->row_of, a->ids, a->gates,
                       (long)a->tokens, (int)a->hidden, dlogits);
  }
  if (a->dtype == JPP_DTYPE_F32) {
    hipLaunchKernelGGL(scatter_dy_kernel<float>, dim3(grid_for(cap * (a->hidden / 8))), dim3(256), 0, st,
                       (const float*)dy, a->tok_of, a->gate_of, a->seg, (int)a->hidden,
                       (float*)deo);
  } else {
    hipLaunchKernelGGL(scatter_dy_kernel<bf16_t>, dim3(grid_for(cap * (a->hidden / 8))), dim3(256), 0, st,
                       (const bf16_t*)dy, a->tok_of, a->gate_of, a->seg, (int)a->hidden,
                       (bf16_t*)deo);
  }
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_moe_combine_bwd(void* stream, const jpp_moe_args* a, const void* dxp,
                        const float* dlogits, void* dx) {
  JPP_REQUIRE(a && dxp && dlogits && dx, "moe_combine_bwd: null operand");
  ProbeScope probe((hipStream_t)stream, "moe_combine_bwd", 0,
                   (a->dtype == JPP_DTYPE_F32 ? 4.0 : 2.0) * a->tokens * a->hidden * (a->top_k + 1));
  // 256 threads cover 2048 columns; about 16 tokens per workgroup
  const dim3 cgrid((unsigned)std::min<long>((a->tokens + 15) / 16, 4096),
                   (unsigned)((a->hidden / 8 + 255) / 256));
  if (a->dtype == JPP_DTYPE_F32) {
    hipLaunchKernelGGL(combine_bwd_kernel<float>, cgrid, dim3(256), 0,
                       (hipStream_t)stream, (const float*)dxp, a->row_of, dlogits,
                       (const float*)a->wr, (long)a->tokens, (int)a->hidden, (float*)dx);
  } else {
    hipLaunchKernelGGL(combine_bwd_kernel<bf16_t>, cgrid, dim3(256), 0,
                       (hipStream_t)stream, (const bf16_t*)dxp, a->row_of, dlogits,
                       (const bf16_t*)a->wr, (long)a->tokens, (int)a->hidden, (bf16_t*)dx);
  }
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_moe_router_wgrad(void* stream, const jpp_moe_args* a, const void* x, const float* dlogits,
                         float* acc, float* partial) {
  JPP_REQUIRE(a && x && dlogits && acc && partial, "moe_router_wgrad: null operand");
  hipStream_t st = (hipStream_t)stream;
  ProbeScope probe(st, "moe_router_wgrad", 0, (a->dtype == JPP_DTYPE_F32 ? 4.0 : 2.0) * a->tokens * a->hidden);
  const int nb = 64;
  if (a->dtype == JPP_DTYPE_F32) {
    hipLaunchKernelGGL(wr_partial_kernel<float>, dim3(nb, (unsigned)((a->hidden / 8 + 255) / 256)), dim3(256), 0,
                       st, (const float*)x, dlogits, (long)a->tokens, (int)a->hidden, partial);
  } else {
    hipLaunchKernelGGL(wr_partial_kernel<bf16_t>, dim3(nb, (unsigned)((a->hidden / 8 + 255) / 256)), dim3(256), 0,
                       st, (const bf16_t*)x, dlogits, (long)a->tokens, (int)a->hidden, partial);
  }
  const long n = (long)a->hidden * kE;
  hipLaunchKernelGGL(wr_reduce_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, partial,
                     nb, n, acc);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

}  // extern "C"
