// The layer's operators on fp32 tensors: the full-precision flavour of a stage, as the
// reference's own CPU-runnable configuration uses it (BERT-style stack of hidden 256 in
// float32, tests/test_transformations.py:42-93 builds its model in float32 too).  Same
// argument structs as the bf16 entry points with every bf16 tensor replaced by an f32 one.
//
// These kernels serve small problems whose results must hold 1e-4 against an fp32 CPU run;
// they are written for plain fp32 arithmetic in a fixed summation order (FMA chains over
// the contraction index, row and column sums in index order), not for the matrix cores.
#include <math.h>

#include "common.h"

namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

__device__ __forceinline__ float gelu32(float u, int tanh_form) {
  if (tanh_form) {
    const float t = tanhf(0.7978845608028654f * (u + 0.044715f * u * u * u));
    return 0.5f * u * (1.0f + t);
  }
  return 0.5f * u * (1.0f + erff(u * 0.7071067811865476f));
}

__device__ __forceinline__ float gelu_grad32(float u, int tanh_form) {
  if (tanh_form) {
    const float t = tanhf(0.7978845608028654f * (u + 0.044715f * u * u * u));
    return 0.5f * (1.0f + t) +
           0.5f * u * (1.0f - t * t) * 0.7978845608028654f * (1.0f + 0.134145f * u * u);
  }
  return 0.5f * (1.0f + erff(u * 0.7071067811865476f)) +
         u * expf(-0.5f * u * u) * 0.3989422804014327f;
}

__device__ __forceinline__ float swiglu32(float g, float u) { return g / (1.0f + expf(-g)) * u; }
__device__ __forceinline__ void swiglu_grad32(float g, float u, float d, float& dg, float& du) {
  const float sg = 1.0f / (1.0f + expf(-g));
  dg = d * u * sg * (1.0f + g * (1.0f - sg));
  du = d * g * sg;
}

// ---------------------------------------------------------------------------
// C[m,n] = epilogue(sum_k Aop[m,k] Bop[n,k]); operand orientations as jpp_gemm_bf16
// ---------------------------------------------------------------------------
struct SgemmParams {
  const float* a;
  const float* b;
  float* c;
  float* c2;
  const float* bias;
  const float* resid;
  const float* aux;
  int m, n, k;
  long lda, ldb, ldc, ldc2, ldresid, ldaux;
  int ta, tb, epi, gelu_tanh;
  // grouped problems, as for the bf16 GEMM: seg[0..n_seg] are row offsets (multiples of 64)
  const int* seg;
  int n_seg, group_mode;
  long stride_b, stride_c;
};

// 64x64 output tile, 16x16 threads of 4x4 outputs each, K in steps of 16 through LDS
__global__ __launch_bounds__(256) void sgemm_kernel(SgemmParams p) {
  __shared__ float As[16][68], Bs[16][68];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const long m0 = (long)blockIdx.y * 64, n0 = (long)blockIdx.x * 64;
  if (p.group_mode == JPP_GROUP_M) {
    // rows of A and C are grouped by expert; each group multiplies its own B
    if (m0 >= p.seg[p.n_seg]) return;
    int e = 0;
    while (p.seg[e + 1] <= m0) ++e;
    p.b += (long)e * p.stride_b;
  } else if (p.group_mode == JPP_GROUP_K) {
    // one output per expert (blockIdx.z); the contraction runs over the expert's rows
    const int e = blockIdx.z;
    const long r0 = p.seg[e];
    p.k = p.seg[e + 1] - p.seg[e];
    p.a += r0 * p.lda;
    p.b += r0 * p.ldb;
    p.c += (long)e * p.stride_c;
  }
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < p.k; k0 += 16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = tid + 256 * i;
      // consecutive threads follow the operand's contiguous index
      if (p.ta) {
        const int mm = e & 63, kk = e >> 6;
        As[kk][mm] = p.a[(long)(k0 + kk) * p.lda + m0 + mm];
      } else {
        const int kk = e & 15, mm = e >> 4;
        As[kk][mm] = p.a[(m0 + mm) * p.lda + k0 + kk];
      }
      if (p.tb) {
        const int nn = e & 63, kk = e >> 6;
        Bs[kk][nn] = p.b[(long)(k0 + kk) * p.ldb + n0 + nn];
      } else {
        const int kk = e & 15, nn = e >> 4;
        Bs[kk][nn] = p.b[(n0 + nn) * p.ldb + k0 + kk];
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      const float4 av = *(const float4*)&As[kk][ty * 4];
      const float4 bv = *(const float4*)&Bs[kk][tx * 4];
      const float a4[4] = {av.x, av.y, av.z, av.w}, b4[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a4[i], b4[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const long row = m0 + ty * 4 + i;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long col = n0 + tx * 4 + j;
      float v = acc[i][j];
      if (p.epi == JPP_EPI_ACC_F32) {
        p.c[row * p.ldc + col] += v;
        continue;
      }
      if (p.epi == JPP_EPI_SWIGLU) {
        // a 64-column tile is one block of the interleaved layout: gate features in its first
        // 32 columns (threads tx < 8), the matching up features 32 columns on (thread tx + 8,
        // lane + 8 of the same wave)
        p.c[row * p.ldc + col] = v;
        const float other = __shfl_xor(v, 8);
        if (tx < 8) p.c2[row * p.ldc2 + n0 / 2 + tx * 4 + j] = swiglu32(v, other);
        continue;
      }
      if (p.epi == JPP_EPI_DSWIGLU) {
        // v = d s of feature `col`; gate / up of that feature sit at 64 q + w and 64 q + 32 + w
        const long q = col >> 5, w = col & 31;
        const float* arow = p.aux + row * p.ldaux + 64 * q + w;
        float dg, du;
        swiglu_grad32(arow[0], arow[32], v, dg, du);
        float* crow = p.c + row * p.ldc + 64 * q + w;
        crow[0] = dg;
        crow[32] = du;
        continue;
      }
      if (p.bias) v += p.bias[col];
      if (p.epi == JPP_EPI_GELU) {
        p.c2[row * p.ldc2 + col] = gelu32(v, p.gelu_tanh);
      } else if (p.epi == JPP_EPI_DGELU) {
        v *= gelu_grad32(p.aux[row * p.ldaux + col], p.gelu_tanh);
      } else if (p.resid) {
        v += p.resid[row * p.ldresid + col];
      }
      p.c[row * p.ldc + col] = v;
    }
  }
}

// ---------------------------------------------------------------------------
// LayerNorm / RMSNorm: one wave per row
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void norm_fwd32_kernel(const float* __restrict__ x,
                                                         const float* __restrict__ gamma,
                                                         const float* __restrict__ beta,
                                                         float* __restrict__ y, float* mean_out,
                                                         float* rstd_out, long rows, int cols,
                                                         float eps) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float* xr = x + row * cols;
  float mean = 0.f;
  if (beta) {
    float s = 0.f;
    for (int c = lane; c < cols; c += 64) s += xr[c];
    mean = wave_sum(s) / cols;
  }
  float q = 0.f;
  for (int c = lane; c < cols; c += 64) {
    const float d = xr[c] - mean;
    q += d * d;
  }
  const float rstd = rsqrtf(wave_sum(q) / cols + eps);
  for (int c = lane; c < cols; c += 64) {
    const float v = (xr[c] - mean) * rstd * gamma[c];
    y[row * cols + c] = beta ? v + beta[c] : v;
  }
  if (lane == 0) {
    if (mean_out) mean_out[row] = mean;
    rstd_out[row] = rstd;
  }
}

__global__ __launch_bounds__(256) void norm_bwd32_kernel(const float* __restrict__ dy,
                                                         const float* __restrict__ x,
                                                         const float* mean_in,
                                                         const float* __restrict__ rstd_in,
                                                         const float* __restrict__ gamma,
                                                         const float* resid, float* __restrict__ dx,
                                                         long rows, int cols) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float rstd = rstd_in[row], mean = mean_in ? mean_in[row] : 0.f;
  const float* xr = x + row * cols;
  const float* dyr = dy + row * cols;
  float s1 = 0.f, s2 = 0.f;
  for (int c = lane; c < cols; c += 64) {
    const float dg = dyr[c] * gamma[c];
    s1 += dg;
    s2 += dg * (xr[c] - mean) * rstd;
  }
  s2 = wave_sum(s2) / cols;
  s1 = mean_in ? wave_sum(s1) / cols : 0.f;
  for (int c = lane; c < cols; c += 64) {
    const float xh = (xr[c] - mean) * rstd;
    float o = (dyr[c] * gamma[c] - s1 - xh * s2) * rstd;
    if (resid) o += resid[row * cols + c];
    dx[row * cols + c] = o;
  }
}

// dgamma[c] += sum_r dy[r,c] xhat[r,c]; dbeta[c] += sum_r dy[r,c]: a thread per column, rows
// in index order
__global__ __launch_bounds__(64) void norm_wgrad32_kernel(const float* __restrict__ dy,
                                                          const float* __restrict__ x,
                                                          const float* mean_in,
                                                          const float* __restrict__ rstd_in,
                                                          float* dgamma, float* dbeta, long rows,
                                                          int cols) {
  const int c = blockIdx.x * 64 + threadIdx.x;
  if (c >= cols) return;
  float g = 0.f, b = 0.f;
  for (long r = 0; r < rows; ++r) {
    const float d = dy[r * cols + c];
    const float mean = mean_in ? mean_in[r] : 0.f;
    g += d * (x[r * cols + c] - mean) * rstd_in[r];
    b += d;
  }
  dgamma[c] += g;
  if (dbeta) dbeta[c] += b;
}

// acc[c] += sum_r x[r,c]
__global__ __launch_bounds__(64) void colsum32_kernel(const float* __restrict__ x, long ld,
                                                      long rows, int cols, float* acc) {
  const int c = blockIdx.x * 64 + threadIdx.x;
  if (c >= cols) return;
  float s = 0.f;
  for (long r = 0; r < rows; ++r) s += x[r * ld + c];
  acc[c] += s;
}

// loss = scale * mean((out - target)^2), dout = scale * 2 (out - target) / count: one
// workgroup, partial sums per thread in index order, then a fixed tree
__global__ __launch_bounds__(256) void mse32_kernel(const float* __restrict__ out,
                                                    const float* __restrict__ target, long count,
                                                    float scale, float* loss, float* dout) {
  __shared__ float red[256];
  float s = 0.f;
  const float k = scale * 2.0f / (float)count;
  for (long i = threadIdx.x; i < count; i += 256) {
    const float d = out[i] - target[i];
    s += d * d;
    if (dout) dout[i] = k * d;
  }
  red[threadIdx.x] = s;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) loss[0] = scale * red[0] / (float)count;
}

// half-split rotary embedding in place on the first `heads` heads of each row
__global__ __launch_bounds__(256) void rope32_kernel(float* __restrict__ x, long ld,
                                                     const float* __restrict__ cos_tab,
                                                     const float* __restrict__ sin_tab, long rows,
                                                     int seq, int heads, int d, int inverse) {
  const int half = d / 2;
  const long total = rows * heads * half;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    const int j = (int)(i % half);
    const long th = i / half;
    const int hh = (int)(th % heads);
    const long t = th / heads;
    const int pos = (int)(t % seq);
    float* p = x + t * ld + hh * d + j;
    const float cs = cos_tab[(long)pos * half + j];
    const float sn = inverse ? -sin_tab[(long)pos * half + j] : sin_tab[(long)pos * half + j];
    const float a = p[0], b = p[half];
    p[0] = a * cs - b * sn;
    p[half] = b * cs + a * sn;
  }
}

// ---------------------------------------------------------------------------
// Attention.  A row (query or key) belongs to a pair of adjacent lanes, each holding half
// of the head dimension; dot products over the head dimension are the sum of the pair's
// halves.  The other side's rows pass through LDS 32 at a time.
// ---------------------------------------------------------------------------
struct Attn32 {
  const float *q, *k, *v, *d_o;
  float *o, *lse, *dq, *dk, *dv, *delta;
  long ldq, ldk, ldv, ldo, lddo, lddq, lddk, lddv;
  int batch, seq, n_heads, n_kv_heads, causal;
  float scale;
};

__device__ __forceinline__ float pair_sum(float v) { return v + __shfl_xor(v, 1); }

template <int D>
__global__ __launch_bounds__(128) void attn_fwd32_kernel(Attn32 p) {
  constexpr int H = D / 2;
  __shared__ float Ks[32][D], Vs[32][D];
  const int tid = threadIdx.x, r = tid >> 1, half = tid & 1;
  const int h = blockIdx.y, b = blockIdx.z, hk = h / (p.n_heads / p.n_kv_heads);
  const int qi = blockIdx.x * 64 + r;
  const long row0 = (long)b * p.seq;
  float q[H], o[H];
#pragma unroll
  for (int d = 0; d < H; ++d) {
    q[d] = p.q[(row0 + qi) * p.ldq + h * D + half * H + d];
    o[d] = 0.f;
  }
  float m = -INFINITY, l = 0.f;
  const int kend = p.causal ? blockIdx.x * 64 + 64 : p.seq;
  for (int k0 = 0; k0 < kend; k0 += 32) {
    __syncthreads();
    for (int e = tid; e < 32 * D; e += 128) {
      const int kr = e / D, d = e % D;
      Ks[kr][d] = p.k[(row0 + k0 + kr) * p.ldk + hk * D + d];
      Vs[kr][d] = p.v[(row0 + k0 + kr) * p.ldv + hk * D + d];
    }
    __syncthreads();
    float s[32];
    float mx = m;
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      float t = 0.f;
#pragma unroll
      for (int d = 0; d < H; ++d) t = fmaf(q[d], Ks[j][half * H + d], t);
      t = pair_sum(t) * p.scale;
      if (p.causal && k0 + j > qi) t = -INFINITY;
      s[j] = t;
      mx = fmaxf(mx, t);
    }
    const float alpha = __expf(m - mx);   // m = -inf on the first tile: alpha = 0, o = l = 0
    l *= alpha;
#pragma unroll
    for (int d = 0; d < H; ++d) o[d] *= alpha;
    m = mx;
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      const float e = expf(s[j] - m);
      l += e;
#pragma unroll
      for (int d = 0; d < H; ++d) o[d] = fmaf(e, Vs[j][half * H + d], o[d]);
    }
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int d = 0; d < H; ++d) p.o[(row0 + qi) * p.ldo + h * D + half * H + d] = o[d] * inv;
  if (half == 0) p.lse[((long)b * p.n_heads + h) * p.seq + qi] = m + logf(l);
}

// dQ (a pair of lanes per query), and delta = rowsum(dO o O) for the dK/dV kernel
template <int D>
__global__ __launch_bounds__(128) void attn_dq32_kernel(Attn32 p) {
  constexpr int H = D / 2;
  __shared__ float Ks[32][D], Vs[32][D];
  const int tid = threadIdx.x, r = tid >> 1, half = tid & 1;
  const int h = blockIdx.y, b = blockIdx.z, hk = h / (p.n_heads / p.n_kv_heads);
  const int qi = blockIdx.x * 64 + r;
  const long row0 = (long)b * p.seq;
  float q[H], g[H], dq[H];
  float dl = 0.f;
#pragma unroll
  for (int d = 0; d < H; ++d) {
    q[d] = p.q[(row0 + qi) * p.ldq + h * D + half * H + d];
    g[d] = p.d_o[(row0 + qi) * p.lddo + h * D + half * H + d];
    dl = fmaf(g[d], p.o[(row0 + qi) * p.ldo + h * D + half * H + d], dl);
    dq[d] = 0.f;
  }
  dl = pair_sum(dl);
  const long stat = ((long)b * p.n_heads + h) * p.seq + qi;
  if (half == 0) p.delta[stat] = dl;
  const float lse = p.lse[stat];
  const int kend = p.causal ? blockIdx.x * 64 + 64 : p.seq;
  for (int k0 = 0; k0 < kend; k0 += 32) {
    __syncthreads();
    for (int e = tid; e < 32 * D; e += 128) {
      const int kr = e / D, d = e % D;
      Ks[kr][d] = p.k[(row0 + k0 + kr) * p.ldk + hk * D + d];
      Vs[kr][d] = p.v[(row0 + k0 + kr) * p.ldv + hk * D + d];
    }
    __syncthreads();
#pragma unroll 1
    for (int j = 0; j < 32; ++j) {
      float t = 0.f, dp = 0.f;
#pragma unroll
      for (int d = 0; d < H; ++d) {
        t = fmaf(q[d], Ks[j][half * H + d], t);
        dp = fmaf(g[d], Vs[j][half * H + d], dp);
      }
      t = pair_sum(t) * p.scale;
      dp = pair_sum(dp);
      const float pr = (p.causal && k0 + j > qi) ? 0.f : expf(t - lse);
      const float ds = pr * (dp - dl) * p.scale;
#pragma unroll
      for (int d = 0; d < H; ++d) dq[d] = fmaf(ds, Ks[j][half * H + d], dq[d]);
    }
  }
#pragma unroll
  for (int d = 0; d < H; ++d) p.dq[(row0 + qi) * p.lddq + h * D + half * H + d] = dq[d];
}

// dK, dV (a pair of lanes per key): the queries of every head of the key's group, in order
template <int D>
__global__ __launch_bounds__(128) void attn_dkv32_kernel(Attn32 p) {
  constexpr int H = D / 2;
  __shared__ float Qs[32][D], Gs[32][D], Ls[32], Ds[32];
  const int tid = threadIdx.x, r = tid >> 1, half = tid & 1;
  const int hk = blockIdx.y, b = blockIdx.z, grp = p.n_heads / p.n_kv_heads;
  const int kj = blockIdx.x * 64 + r;
  const long row0 = (long)b * p.seq;
  float k[H], v[H], dk[H], dv[H];
#pragma unroll
  for (int d = 0; d < H; ++d) {
    k[d] = p.k[(row0 + kj) * p.ldk + hk * D + half * H + d];
    v[d] = p.v[(row0 + kj) * p.ldv + hk * D + half * H + d];
    dk[d] = dv[d] = 0.f;
  }
  const int qbeg = p.causal ? blockIdx.x * 64 : 0;
  for (int h = hk * grp; h < (hk + 1) * grp; ++h) {
    for (int q0 = qbeg; q0 < p.seq; q0 += 32) {
      __syncthreads();
      for (int e = tid; e < 32 * D; e += 128) {
        const int qr = e / D, d = e % D;
        Qs[qr][d] = p.q[(row0 + q0 + qr) * p.ldq + h * D + d];
        Gs[qr][d] = p.d_o[(row0 + q0 + qr) * p.lddo + h * D + d];
      }
      if (tid < 32) {
        const long stat = ((long)b * p.n_heads + h) * p.seq + q0 + tid;
        Ls[tid] = p.lse[stat];
        Ds[tid] = p.delta[stat];
      }
      __syncthreads();
#pragma unroll 1
      for (int i = 0; i < 32; ++i) {
        float t = 0.f, dp = 0.f;
#pragma unroll
        for (int d = 0; d < H; ++d) {
          t = fmaf(Qs[i][half * H + d], k[d], t);
          dp = fmaf(Gs[i][half * H + d], v[d], dp);
        }
        t = pair_sum(t) * p.scale;
        dp = pair_sum(dp);
        const float pr = (p.causal && kj > q0 + i) ? 0.f : expf(t - Ls[i]);
        const float ds = pr * (dp - Ds[i]) * p.scale;
#pragma unroll
        for (int d = 0; d < H; ++d) {
          dv[d] = fmaf(pr, Gs[i][half * H + d], dv[d]);
          dk[d] = fmaf(ds, Qs[i][half * H + d], dk[d]);
        }
      }
    }
  }
#pragma unroll
  for (int d = 0; d < H; ++d) {
    p.dk[(row0 + kj) * p.lddk + hk * D + half * H + d] = dk[d];
    p.dv[(row0 + kj) * p.lddv + hk * D + half * H + d] = dv[d];
  }
}

int attn_check(const jpp_attn_args* a, const char* who, Attn32& p) {
  JPP_REQUIRE(a && a->q && a->k && a->v && a->o && a->lse, "%s: null operand", who);
  JPP_REQUIRE(a->head_dim == 64 || a->head_dim == 128, "%s: head_dim must be 64 or 128", who);
  JPP_REQUIRE(a->batch > 0 && a->seq > 0 && a->seq % 64 == 0, "%s: seq must be a multiple of 64", who);
  JPP_REQUIRE(a->n_heads > 0 && a->n_kv_heads > 0 && a->n_heads % a->n_kv_heads == 0,
              "%s: n_heads must be a multiple of n_kv_heads", who);
  JPP_REQUIRE(a->ldq >= (int64_t)a->n_heads * a->head_dim && a->ldo >= (int64_t)a->n_heads * a->head_dim &&
                  a->ldk >= (int64_t)a->n_kv_heads * a->head_dim &&
                  a->ldv >= (int64_t)a->n_kv_heads * a->head_dim,
              "%s: leading dimension too small", who);
  p.q = (const float*)a->q; p.k = (const float*)a->k; p.v = (const float*)a->v;
  p.o = (float*)a->o; p.lse = a->lse;
  p.d_o = (const float*)a->d_o; p.dq = (float*)a->dq; p.dk = (float*)a->dk; p.dv = (float*)a->dv;
  p.delta = a->delta;
  p.ldq = a->ldq; p.ldk = a->ldk; p.ldv = a->ldv; p.ldo = a->ldo;
  p.lddo = a->lddo; p.lddq = a->lddq; p.lddk = a->lddk; p.lddv = a->lddv;
  p.batch = a->batch; p.seq = a->seq; p.n_heads = a->n_heads; p.n_kv_heads = a->n_kv_heads;
  p.causal = a->causal;
  p.scale = 1.0f / sqrtf((float)a->head_dim);
  return JPP_OK;
}

}  // namespace

extern "C" {

int jpp_gemm_f32(void* stream, const jpp_gemm_args* a) {
  JPP_REQUIRE(!a || a->k_parts <= 1, "gemm_f32: one operand pair per product");
  JPP_REQUIRE(a && a->a && a->b && a->c, "gemm_f32: null operand");
  JPP_REQUIRE(!a->rope_cos && !a->rope_sin,
              "gemm_f32: no rotary epilogue on f32 tensors (jpp_rope_f32 is the pass for them)");
  const bool group_k = a->group_mode == JPP_GROUP_K;
  JPP_REQUIRE(a->m > 0 && a->n > 0 && (a->k > 0 || group_k) && a->m % 64 == 0 && a->n % 64 == 0 &&
                  (a->k % 16 == 0 || group_k),
              "gemm_f32: M, N must be multiples of 64 and K of 16, got %ldx%ldx%ld", (long)a->m,
              (long)a->n, (long)a->k);
  if (a->group_mode != JPP_GROUP_NONE) {
    JPP_REQUIRE(a->group_mode == JPP_GROUP_M || group_k, "gemm_f32: unknown group_mode %d",
                a->group_mode);
    JPP_REQUIRE(a->seg && a->n_seg > 0 && a->n_seg <= 256, "gemm_f32: grouped problem needs seg[n_seg+1]");
    JPP_REQUIRE(!a->bias && !a->resid, "gemm_f32: grouped problems take no bias / residual");
    JPP_REQUIRE(!group_k || (a->trans_a && a->trans_b),
                "gemm_f32: a grouped contraction takes both operands with the rows as the slow index");
  }
  const int e = a->epilogue;
  JPP_REQUIRE(e >= JPP_EPI_BF16 && e <= JPP_EPI_DSWIGLU, "gemm_f32: unsupported epilogue %d", e);
  JPP_REQUIRE(a->lda >= (a->trans_a ? a->m : (group_k ? 0 : a->k)) &&
                  a->ldb >= (a->trans_b ? a->n : (group_k ? 0 : a->k)) && a->ldc >= a->n,
              "gemm_f32: leading dimension too small");
  if (e == JPP_EPI_GELU) JPP_REQUIRE(a->c2 && a->ldc2 >= a->n, "gemm_f32: GELU epilogue needs c2");
  if (e == JPP_EPI_DGELU) JPP_REQUIRE(a->aux && a->ldaux >= a->n, "gemm_f32: dGELU epilogue needs aux");
  if (e == JPP_EPI_SWIGLU)
    JPP_REQUIRE(a->c2 && a->ldc2 >= a->n / 2 && !a->bias && !a->resid,
                "gemm_f32: SwiGLU epilogue needs c2 [M, N/2] and takes no bias / residual");
  if (e == JPP_EPI_DSWIGLU)
    JPP_REQUIRE(a->aux && a->ldaux >= 2 * a->n && a->ldc >= 2 * a->n && !a->bias && !a->resid,
                "gemm_f32: dSwiGLU epilogue needs aux and C of width 2N and takes no bias / residual");
  if (a->resid) JPP_REQUIRE(a->ldresid >= a->n, "gemm_f32: bad ldresid");
  SgemmParams p;
  p.a = (const float*)a->a; p.b = (const float*)a->b; p.c = (float*)a->c; p.c2 = (float*)a->c2;
  p.bias = (const float*)a->bias; p.resid = (const float*)a->resid; p.aux = (const float*)a->aux;
  p.m = (int)a->m; p.n = (int)a->n; p.k = (int)a->k;
  p.lda = a->lda; p.ldb = a->ldb; p.ldc = a->ldc; p.ldc2 = a->ldc2; p.ldresid = a->ldresid;
  p.ldaux = a->ldaux;
  p.ta = a->trans_a != 0; p.tb = a->trans_b != 0; p.epi = e; p.gelu_tanh = a->gelu_tanh;
  p.seg = a->seg; p.n_seg = a->n_seg; p.group_mode = a->group_mode;
  p.stride_b = a->stride_b; p.stride_c = a->stride_c;
  hipLaunchKernelGGL(sgemm_kernel,
                     dim3((unsigned)(a->n / 64), (unsigned)(a->m / 64), group_k ? (unsigned)a->n_seg : 1u),
                     dim3(256), 0, (hipStream_t)stream, p);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_rope_f32(void* stream, float* x, int64_t ld, const float* cos_tab, const float* sin_tab,
                 int batch, int seq, int n_rot_heads, int head_dim, int inverse) {
  JPP_REQUIRE(x && cos_tab && sin_tab, "rope_f32: null operand");
  JPP_REQUIRE(batch > 0 && seq > 0 && n_rot_heads > 0 && head_dim > 0 && head_dim % 2 == 0 &&
                  ld >= (int64_t)n_rot_heads * head_dim,
              "rope_f32: bad shape");
  const long rows = (long)batch * seq, total = rows * n_rot_heads * (head_dim / 2);
  const unsigned grid = (unsigned)((total + 255) / 256 > 65536 ? 65536 : (total + 255) / 256);
  hipLaunchKernelGGL(rope32_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, x, (long)ld,
                     cos_tab, sin_tab, rows, seq, n_rot_heads, head_dim, inverse);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_norm_fwd_f32(void* stream, const jpp_norm_args* a) {
  JPP_REQUIRE(a && a->x && a->gamma && a->y && a->rstd, "norm_fwd_f32: null operand");
  JPP_REQUIRE(a->rows > 0 && a->cols > 0, "norm_fwd_f32: empty");
  JPP_REQUIRE((a->beta == nullptr) == (a->mean == nullptr),
              "norm_fwd_f32: beta and mean are both given (LayerNorm) or both NULL (RMSNorm)");
  hipLaunchKernelGGL(norm_fwd32_kernel, dim3((unsigned)((a->rows + 3) / 4)), dim3(256), 0,
                     (hipStream_t)stream, (const float*)a->x, (const float*)a->gamma,
                     (const float*)a->beta, (float*)a->y, a->mean, a->rstd, (long)a->rows,
                     (int)a->cols, a->eps);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_norm_bwd_f32(void* stream, const jpp_norm_args* a) {
  JPP_REQUIRE(a && a->x && a->gamma && a->dy && a->dx && a->rstd && a->dgamma,
              "norm_bwd_f32: null operand");
  JPP_REQUIRE(a->rows > 0 && a->cols > 0, "norm_bwd_f32: empty");
  JPP_REQUIRE(!a->mean || a->dbeta, "norm_bwd_f32: LayerNorm needs dbeta");
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(norm_bwd32_kernel, dim3((unsigned)((a->rows + 3) / 4)), dim3(256), 0, st,
                     (const float*)a->dy, (const float*)a->x, (const float*)a->mean,
                     (const float*)a->rstd, (const float*)a->gamma, (const float*)a->resid,
                     (float*)a->dx, (long)a->rows, (int)a->cols);
  hipLaunchKernelGGL(norm_wgrad32_kernel, dim3((unsigned)((a->cols + 63) / 64)), dim3(64), 0, st,
                     (const float*)a->dy, (const float*)a->x, (const float*)a->mean,
                     (const float*)a->rstd, a->dgamma, a->mean ? a->dbeta : nullptr, (long)a->rows,
                     (int)a->cols);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_colsum_accum_f32(void* stream, const float* x, int64_t ld, int64_t rows, int64_t cols,
                         float* acc) {
  JPP_REQUIRE(x && acc && rows > 0 && cols > 0 && ld >= cols, "colsum_accum_f32: bad arguments");
  hipLaunchKernelGGL(colsum32_kernel, dim3((unsigned)((cols + 63) / 64)), dim3(64), 0,
                     (hipStream_t)stream, x, (long)ld, (long)rows, (int)cols, acc);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_mse_loss_f32(void* stream, const float* out, const float* target, int64_t count,
                     float scale, float* loss, float* dout) {
  JPP_REQUIRE(out && target && loss && count > 0, "mse_loss_f32: bad arguments");
  hipLaunchKernelGGL(mse32_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, out, target,
                     (long)count, scale, loss, dout);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_attn_fwd_f32(void* stream, const jpp_attn_args* a) {
  Attn32 p;
  if (int rc = attn_check(a, "attn_fwd_f32", p)) return rc;
  const dim3 grid((unsigned)(a->seq / 64), (unsigned)a->n_heads, (unsigned)a->batch);
  if (a->head_dim == 64)
    hipLaunchKernelGGL(attn_fwd32_kernel<64>, grid, dim3(128), 0, (hipStream_t)stream, p);
  else
    hipLaunchKernelGGL(attn_fwd32_kernel<128>, grid, dim3(128), 0, (hipStream_t)stream, p);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_attn_bwd_f32(void* stream, const jpp_attn_args* a) {
  Attn32 p;
  if (int rc = attn_check(a, "attn_bwd_f32", p)) return rc;
  JPP_REQUIRE(a->d_o && a->dq && a->dk && a->dv && a->delta, "attn_bwd_f32: null operand");
  JPP_REQUIRE(a->lddo >= (int64_t)a->n_heads * a->head_dim && a->lddq >= (int64_t)a->n_heads * a->head_dim &&
                  a->lddk >= (int64_t)a->n_kv_heads * a->head_dim &&
                  a->lddv >= (int64_t)a->n_kv_heads * a->head_dim,
              "attn_bwd_f32: leading dimension too small");
  hipStream_t st = (hipStream_t)stream;
  const dim3 gq((unsigned)(a->seq / 64), (unsigned)a->n_heads, (unsigned)a->batch);
  const dim3 gk((unsigned)(a->seq / 64), (unsigned)a->n_kv_heads, (unsigned)a->batch);
  if (a->head_dim == 64) {
    hipLaunchKernelGGL(attn_dq32_kernel<64>, gq, dim3(128), 0, st, p);
    hipLaunchKernelGGL(attn_dkv32_kernel<64>, gk, dim3(128), 0, st, p);
  } else {
    hipLaunchKernelGGL(attn_dq32_kernel<128>, gq, dim3(128), 0, st, p);
    hipLaunchKernelGGL(attn_dkv32_kernel<128>, gk, dim3(128), 0, st, p);
  }
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

}  // extern "C"
