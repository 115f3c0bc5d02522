// HBM-bound kernels of a stage task: LayerNorm / RMSNorm forward and
// backward, SwiGLU, rotary embedding, gradient accumulation, bias-gradient
// column sums and dtype casts.  All move 16 bytes per lane per access and keep
// statistics in fp32.  Parameter gradients are reduced in a fixed order
// (per-block partial sums, then one ordered pass) so results do not depend on
// scheduling.
#include <math.h>

#include <mutex>

#include "common.h"

// Scratch of jpp_norm_bwd_static (the entry point that allocates nothing): the per-block
// partial sums of the scale / shift gradients, 2 x JPP_NORM_PARTIALS rows of at most
// kStaticNormCols columns (16 MiB).  Every GPU the library runs on holds its own copy at its
// own address until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress: the device address comes from static_scratch() below and is what
// kernels are given.
constexpr int kStaticNormCols = 8192;
static __device__ __align__(256) float scratch[2 * JPP_NORM_PARTIALS * kStaticNormCols];

namespace {

constexpr int kMaxChunksPerLane = 16;  // a wave holds one row of <= 8192 columns
static_assert(kStaticNormCols == 8 * 64 * kMaxChunksPerLane, "scratch sized for the widest row");

// Device address of `scratch` on the current device, looked up once per device.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
float* g_scratch_ptr[kMaxDevices] = {};

int static_scratch(float** out) {
  int dev = -1;
  JPP_CHECK_HIP(hipGetDevice(&dev));
  JPP_REQUIRE(dev >= 0 && dev < kMaxDevices, "static scratch: device %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    JPP_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    JPP_REQUIRE(ptr, "static scratch: hipGetSymbolAddress returned a null address");
    g_scratch_ptr[dev] = (float*)ptr;
  }
  *out = g_scratch_ptr[dev];
  return JPP_OK;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}


// ---------------------------------------------------------------------------
// norm forward: one wave per row, the row cached in registers
// ---------------------------------------------------------------------------
template <bool LN, int NCH>
__global__ __launch_bounds__(256) void norm_fwd_kernel(const bf16_t* __restrict__ x,
                                                       const bf16_t* __restrict__ gamma,
                                                       const bf16_t* __restrict__ beta,
                                                       bf16_t* __restrict__ y,
                                                       float* __restrict__ mean_out,
                                                       float* __restrict__ rstd_out, long rows,
                                                       int cols, float eps) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int nchunk = cols >> 3;
  const uint4* xr = (const uint4*)(x + row * cols);
  uint4 v[NCH];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + 64 * i;
    v[i] = c < nchunk ? xr[c] : make_uint4(0, 0, 0, 0);
    float f[8];
    unpack8(v[i], f);
#pragma unroll
    for (int e = 0; e < 8; ++e) s += LN ? f[e] : f[e] * f[e];
  }
  s = wave_sum(s);
  float mean = 0.f, var;
  if (LN) {
    mean = s / cols;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      if (lane + 64 * i < nchunk) {
        float f[8];
        unpack8(v[i], f);
#pragma unroll
        for (int e = 0; e < 8; ++e) q += (f[e] - mean) * (f[e] - mean);
      }
    }
    var = wave_sum(q) / cols;
  } else {
    var = s / cols;
  }
  const float rstd = 1.0f / sqrtf(var + eps);
  if (lane == 0) {
    rstd_out[row] = rstd;
    if (LN) mean_out[row] = mean;
  }
  uint4* yr = (uint4*)(y + row * cols);
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + 64 * i;
    if (c < nchunk) {
      float f[8], g[8], b[8];
      unpack8(v[i], f);
      unpack8(((const uint4*)gamma)[c], g);
      if (LN) unpack8(((const uint4*)beta)[c], b);
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = (f[e] - mean) * rstd * g[e] + (LN ? b[e] : 0.f);
      yr[c] = pack8(f);
    }
  }
}

// ---------------------------------------------------------------------------
// norm backward: dx per row, and per-block partial sums of dgamma / dbeta
// ---------------------------------------------------------------------------
constexpr int kNormBwdWaves = 8;
template <bool LN, int NCH>
__global__ __launch_bounds__(kNormBwdWaves * 64) void norm_bwd_kernel(
    const bf16_t* __restrict__ dy, const bf16_t* __restrict__ x, const float* __restrict__ mean_in,
    const float* __restrict__ rstd_in, const bf16_t* __restrict__ gamma,
    const bf16_t* __restrict__ resid, bf16_t* __restrict__ dx, float* __restrict__ partial,
    long rows, int cols) {
  __shared__ float red[kNormBwdWaves][64 * 8];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nchunk = cols >> 3;
  const long stride = (long)gridDim.x * kNormBwdWaves;
  float pg[NCH][8], pb[LN ? NCH : 1][8];
#pragma unroll
  for (int i = 0; i < NCH; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      pg[i][e] = 0.f;
      if (LN) pb[i][e] = 0.f;
    }
  for (long row = (long)blockIdx.x * kNormBwdWaves + wave; row < rows; row += stride) {
    const float rstd = rstd_in[row];
    const float mean = LN ? mean_in[row] : 0.f;
    const uint4* xr = (const uint4*)(x + row * cols);
    const uint4* dyr = (const uint4*)(dy + row * cols);
    uint4 vx[NCH], vd[NCH];
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = lane + 64 * i;
      if (c < nchunk) {
        vx[i] = xr[c];
        vd[i] = dyr[c];
        float fx[8], fd[8], g[8];
        unpack8(vx[i], fx);
        unpack8(vd[i], fd);
        unpack8(((const uint4*)gamma)[c], g);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float xh = (fx[e] - mean) * rstd;
          const float dg = fd[e] * g[e];
          s1 += dg;
          s2 += dg * xh;
          pg[i][e] += fd[e] * xh;
          if (LN) pb[i][e] += fd[e];
        }
      }
    }
    s2 = wave_sum(s2) / cols;
    s1 = LN ? wave_sum(s1) / cols : 0.f;
    uint4* dxr = (uint4*)(dx + row * cols);
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = lane + 64 * i;
      if (c < nchunk) {
        float fx[8], fd[8], g[8], r[8];
        unpack8(vx[i], fx);
        unpack8(vd[i], fd);
        unpack8(((const uint4*)gamma)[c], g);
        if (resid) unpack8(((const uint4*)(resid + row * cols))[c], r);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float xh = (fx[e] - mean) * rstd;
          float o = (fd[e] * g[e] - s1 - xh * s2) * rstd;
          if (resid) o += r[e];
          fx[e] = o;
        }
        dxr[c] = pack8(fx);
      }
    }
  }
  // combine the waves of the block in a fixed order, one chunk column at a time
  float* pgam = partial + (long)blockIdx.x * cols;
  float* pbet = partial + ((long)gridDim.x + blockIdx.x) * cols;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + 64 * i;
#pragma unroll
    for (int pass = 0; pass < (LN ? 2 : 1); ++pass) {
      __syncthreads();
#pragma unroll
      for (int e = 0; e < 8; ++e) red[wave][lane * 8 + e] = pass ? pb[LN ? i : 0][e] : pg[i][e];
      __syncthreads();
      if (wave == 0 && c < nchunk) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float t = red[0][lane * 8 + e];
#pragma unroll
          for (int w = 1; w < kNormBwdWaves; ++w) t += red[w][lane * 8 + e];
          (pass ? pbet : pgam)[c * 8 + e] = t;
        }
      }
    }
  }
}

// Rows of 4096 or 8192 columns: a row is spread over the 8 waves of a workgroup (a lane owns
// NCHB pieces of 8 columns), R rows at a time.  The wave-per-row kernel above needs the row,
// its gradient and 8 partial sums per piece in registers - 200 to 256 registers and, at 8192
// columns, spills - so few waves fit a CU and each waits out its own loads.  Here a lane holds
// 12 registers per row, the loads of R rows are in flight together, and the price is one
// barrier per R rows for the row sums (wave sums meet in LDS and are added in wave order).
// Every column belongs to one lane of the workgroup, so its partial sums of the scale / shift
// gradients leave without a reduction across waves; summation orders are fixed throughout.
__device__ __forceinline__ void keep_packed(uint4& v) {
  asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w));
}

template <bool LN, int NCHB, int R>
__global__ __launch_bounds__(512) void norm_bwd_wide_kernel(
    const bf16_t* __restrict__ dy, const bf16_t* __restrict__ x, const float* __restrict__ mean_in,
    const float* __restrict__ rstd_in, const bf16_t* __restrict__ gamma,
    const bf16_t* __restrict__ resid, bf16_t* __restrict__ dx, float* __restrict__ partial,
    long rows, int cols) {
  __shared__ float red[2][R][8][2];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float g[NCHB][8], pg[NCHB][8], pb[LN ? NCHB : 1][8];
#pragma unroll
  for (int i = 0; i < NCHB; ++i) {
    unpack8(((const uint4*)gamma)[tid + 512 * i], g[i]);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      pg[i][e] = 0.f;
      if (LN) pb[i][e] = 0.f;
    }
  }
  int par = 0;
  for (long r0 = (long)blockIdx.x * R; r0 < rows; r0 += (long)gridDim.x * R, par ^= 1) {
    uint4 vx[R][NCHB], vd[R][NCHB], vr[R][NCHB];
    float rstd[R], mean[R];
#pragma unroll
    for (int q = 0; q < R; ++q) {
      const long row = min(r0 + q, rows - 1);   // rows past the end repeat the last one, unused
      rstd[q] = rstd_in[row];
      mean[q] = LN ? mean_in[row] : 0.f;
#pragma unroll
      for (int i = 0; i < NCHB; ++i) {
        const long at = row * (cols / 8) + tid + 512 * i;
        vx[q][i] = ((const uint4*)x)[at];
        vd[q][i] = ((const uint4*)dy)[at];
        if (resid) vr[q][i] = ((const uint4*)resid)[at];
      }
    }
#pragma unroll
    for (int q = 0; q < R; ++q) {
      float s1 = 0.f, s2 = 0.f;
#pragma unroll
      for (int i = 0; i < NCHB; ++i) {
        float fx[8], fd[8];
        unpack8(vx[q][i], fx);
        unpack8(vd[q][i], fd);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float dg = fd[e] * g[i][e];
          s1 += dg;
          s2 += dg * ((fx[e] - mean[q]) * rstd[q]);
        }
      }
      s2 = wave_sum(s2);
      if (LN) s1 = wave_sum(s1);
      if (lane == 0) {
        red[par][q][wave][0] = s1;
        red[par][q][wave][1] = s2;
      }
    }
    __syncthreads();
    // the rows stay packed across the barrier: without this the compiler keeps the unpacked
    // f32 values of all R rows alive instead (three times the registers)
#pragma unroll
    for (int q = 0; q < R; ++q)
#pragma unroll
      for (int i = 0; i < NCHB; ++i) {
        keep_packed(vx[q][i]);
        keep_packed(vd[q][i]);
        if (resid) keep_packed(vr[q][i]);
      }
#pragma unroll
    for (int q = 0; q < R; ++q) {
      if (r0 + q >= rows) break;
      float s1 = 0.f, s2 = 0.f;
#pragma unroll
      for (int w = 0; w < 8; ++w) {
        s1 += red[par][q][w][0];
        s2 += red[par][q][w][1];
      }
      s2 /= cols;
      s1 = LN ? s1 / cols : 0.f;
#pragma unroll
      for (int i = 0; i < NCHB; ++i) {
        float fx[8], fd[8], r[8];
        unpack8(vx[q][i], fx);
        unpack8(vd[q][i], fd);
        if (resid) unpack8(vr[q][i], r);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float xh = (fx[e] - mean[q]) * rstd[q];
          pg[i][e] += fd[e] * xh;
          if (LN) pb[i][e] += fd[e];
          float o = (fd[e] * g[i][e] - s1 - xh * s2) * rstd[q];
          if (resid) o += r[e];
          fx[e] = o;
        }
        ((uint4*)dx)[(r0 + q) * (cols / 8) + tid + 512 * i] = pack8(fx);
      }
    }
  }
  float* pgam = partial + (long)blockIdx.x * cols;
  float* pbet = partial + ((long)gridDim.x + blockIdx.x) * cols;
#pragma unroll
  for (int i = 0; i < NCHB; ++i) {
    const int c = (tid + 512 * i) * 8;
    *(float4*)(pgam + c) = make_float4(pg[i][0], pg[i][1], pg[i][2], pg[i][3]);
    *(float4*)(pgam + c + 4) = make_float4(pg[i][4], pg[i][5], pg[i][6], pg[i][7]);
    if (LN) {
      *(float4*)(pbet + c) = make_float4(pb[i][0], pb[i][1], pb[i][2], pb[i][3]);
      *(float4*)(pbet + c + 4) = make_float4(pb[i][4], pb[i][5], pb[i][6], pb[i][7]);
    }
  }
}

// acc[j] += sum_b partial[b][j]: a block owns 32 columns; 32 thread groups sum interleaved
// subsets of the partials (8 independent loads each for 256 partials), then one combines them
// in a fixed order.  blockIdx.y picks one of two reductions (gamma and beta of a LayerNorm
// share a launch): the second one's partials follow the first's, its accumulator is acc2.
__global__ __launch_bounds__(1024) void partial_reduce_kernel(const float* __restrict__ partial,
                                                              int nblocks, int cols,
                                                              float* __restrict__ acc,
                                                              float* __restrict__ acc2) {
  __shared__ float red[32][33];
  const int c = threadIdx.x & 31, g = threadIdx.x >> 5;
  const int j = blockIdx.x * 32 + c;
  if (blockIdx.y) {
    partial += (long)nblocks * cols;
    acc = acc2;
  }
  float s = 0.f;
  if (j < cols) {
#pragma unroll 8
    for (int b = g; b < nblocks; b += 32) s += partial[(long)b * cols + j];
  }
  red[g][c] = s;
  __syncthreads();
  if (g == 0 && j < cols) {
    float t = red[0][c];
#pragma unroll
    for (int w = 1; w < 32; ++w) t += red[w][c];
    acc[j] += t;
  }
}

// ---------------------------------------------------------------------------
// column sums (bias gradients): block b sums rows b, b+nb, ... of a 2048-wide
// column panel
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void colsum_partial_kernel(const bf16_t* __restrict__ x, long ld,
                                                             long rows, int cols,
                                                             float* __restrict__ partial) {
  const int c = blockIdx.y * 256 + threadIdx.x;  // 8-column chunk
  if (c * 8 >= cols) return;
  float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (long row = blockIdx.x; row < rows; row += gridDim.x) {
    float f[8];
    unpack8(*(const uint4*)(x + row * ld + c * 8), f);
#pragma unroll
    for (int e = 0; e < 8; ++e) s[e] += f[e];
  }
  float* dst = partial + (long)blockIdx.x * cols + c * 8;
  *(float4*)dst = make_float4(s[0], s[1], s[2], s[3]);
  *(float4*)(dst + 4) = make_float4(s[4], s[5], s[6], s[7]);
}

// Several column sums in one launch: the tensors' columns are laid side by side in one virtual
// row of `total` columns (each tensor's share a multiple of 8), and so are the partial sums.
struct ColsumBatch {
  const bf16_t* x[4];
  long ld[4];
  float* acc[4];
  int start[5];  // first virtual column of each tensor; start[n] = total
  int n;
};

__global__ __launch_bounds__(256) void colsum_multi_partial_kernel(ColsumBatch b, long rows,
                                                                   float* __restrict__ partial) {
  const int c = (blockIdx.y * 256 + threadIdx.x) * 8;  // virtual column of this thread's chunk
  const int total = b.start[b.n];
  if (c >= total) return;
  int i = 0;
  while (c >= b.start[i + 1]) ++i;
  const bf16_t* x = b.x[i] + (c - b.start[i]);
  const long ld = b.ld[i];
  float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (long row = blockIdx.x; row < rows; row += gridDim.x) {
    float f[8];
    unpack8(*(const uint4*)(x + row * ld), f);
#pragma unroll
    for (int e = 0; e < 8; ++e) s[e] += f[e];
  }
  float* dst = partial + (long)blockIdx.x * total + c;
  *(float4*)dst = make_float4(s[0], s[1], s[2], s[3]);
  *(float4*)(dst + 4) = make_float4(s[4], s[5], s[6], s[7]);
}

// as partial_reduce_kernel, the result scattered to the tensors' accumulators
__global__ __launch_bounds__(1024) void colsum_multi_reduce_kernel(const float* __restrict__ partial,
                                                                   int nblocks, ColsumBatch b) {
  __shared__ float red[32][33];
  const int c = threadIdx.x & 31, g = threadIdx.x >> 5;
  const int j = blockIdx.x * 32 + c, total = b.start[b.n];
  float s = 0.f;
  if (j < total) {
#pragma unroll 8
    for (int k = g; k < nblocks; k += 32) s += partial[(long)k * total + j];
  }
  red[g][c] = s;
  __syncthreads();
  if (g == 0 && j < total) {
    float t = red[0][c];
#pragma unroll
    for (int w = 1; w < 32; ++w) t += red[w][c];
    int i = 0;
    while (j >= b.start[i + 1]) ++i;
    b.acc[i][j - b.start[i]] += t;
  }
}

// ---------------------------------------------------------------------------
// SwiGLU
// ---------------------------------------------------------------------------
// gate and up of 8 features starting at feature 8c of row t: halves layout [gate | up], or
// interleaved in blocks of 32 columns (column 64q+w: gate feature 32q+w for w < 32, else up)
__device__ __forceinline__ long gate_col(int c, int f, int il) {
  return il ? (long)(c >> 2) * 64 + (c & 3) * 8 : (long)c * 8;
}
__device__ __forceinline__ long up_col(int c, int f, int il) {
  return il ? (long)(c >> 2) * 64 + 32 + (c & 3) * 8 : (long)f + (long)c * 8;
}

__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const bf16_t* __restrict__ gu,
                                                         bf16_t* __restrict__ s, long rows,
                                                         int f, int il) {
  const int fc = f >> 3;
  const long total = rows * fc;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    const long t = i / fc;
    const int c = (int)(i - t * fc);
    float a[8], b[8];
    unpack8(*(const uint4*)(gu + t * 2 * f + gate_col(c, f, il)), a);
    unpack8(*(const uint4*)(gu + t * 2 * f + up_col(c, f, il)), b);
#pragma unroll
    for (int e = 0; e < 8; ++e) a[e] = a[e] * __builtin_amdgcn_rcpf(1.0f + __expf(-a[e])) * b[e];  // as the GEMM epilogue's
    *(uint4*)(s + t * f + c * 8) = pack8(a);
  }
}

__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const bf16_t* __restrict__ gu,
                                                         const bf16_t* __restrict__ ds,
                                                         bf16_t* __restrict__ dgu, long rows,
                                                         int f, int il) {
  const int fc = f >> 3;
  const long total = rows * fc;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    const long t = i / fc;
    const int c = (int)(i - t * fc);
    const long gc = gate_col(c, f, il), uc = up_col(c, f, il);
    float a[8], b[8], d[8];
    unpack8(*(const uint4*)(gu + t * 2 * f + gc), a);
    unpack8(*(const uint4*)(gu + t * 2 * f + uc), b);
    unpack8(*(const uint4*)(ds + t * f + c * 8), d);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float sg = __builtin_amdgcn_rcpf(1.0f + __expf(-a[e]));
      const float da = d[e] * b[e] * sg * (1.0f + a[e] * (1.0f - sg));
      const float db = d[e] * a[e] * sg;
      a[e] = da;
      b[e] = db;
    }
    *(uint4*)(dgu + t * 2 * f + gc) = pack8(a);
    *(uint4*)(dgu + t * 2 * f + uc) = pack8(b);
  }
}

// ---------------------------------------------------------------------------
// rotary embedding, half-split layout, in place
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rope_kernel(bf16_t* __restrict__ x, long ld,
                                                   const float* __restrict__ cos_tab,
                                                   const float* __restrict__ sin_tab, long rows,
                                                   int seq, int heads, int d, int inverse) {
  const int hc = d >> 4;  // 8-element chunks in half a head
  const long total = rows * heads * hc;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    const int c = (int)(i % hc);
    const long th = i / hc;
    const int hh = (int)(th % heads);
    const long t = th / heads;
    const int pos = (int)(t % seq);
    bf16_t* p = x + t * ld + hh * d + c * 8;
    float a[8], b[8];
    unpack8(*(const uint4*)p, a);
    unpack8(*(const uint4*)(p + d / 2), b);
    const float* ct = cos_tab + (long)pos * (d / 2) + c * 8;
    const float* st = sin_tab + (long)pos * (d / 2) + c * 8;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float cs = ct[e], sn = inverse ? -st[e] : st[e];
      float o1, o2;
      rope_rotate(a[e], b[e], cs, sn, o1, o2);
      a[e] = o1;
      b[e] = o2;
    }
    *(uint4*)p = pack8(a);
    *(uint4*)(p + d / 2) = pack8(b);
  }
}

// ---------------------------------------------------------------------------
// gradient accumulation and casts
// ---------------------------------------------------------------------------
template <bool G_F32>
__global__ __launch_bounds__(256) void grad_accum_kernel(float* __restrict__ acc,
                                                         const void* __restrict__ g, long n8) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n8; i += (long)gridDim.x * 256) {
    float4 a0 = ((float4*)acc)[2 * i], a1 = ((float4*)acc)[2 * i + 1];
    if (G_F32) {
      const float4 g0 = ((const float4*)g)[2 * i], g1 = ((const float4*)g)[2 * i + 1];
      a0.x += g0.x; a0.y += g0.y; a0.z += g0.z; a0.w += g0.w;
      a1.x += g1.x; a1.y += g1.y; a1.z += g1.z; a1.w += g1.w;
    } else {
      float f[8];
      unpack8(((const uint4*)g)[i], f);
      a0.x += f[0]; a0.y += f[1]; a0.z += f[2]; a0.w += f[3];
      a1.x += f[4]; a1.y += f[5]; a1.z += f[6]; a1.w += f[7];
    }
    ((float4*)acc)[2 * i] = a0;
    ((float4*)acc)[2 * i + 1] = a1;
  }
}

// acc += parts[0] + parts[1] + ... (in that order): the partial products of a contraction
// that was split over workgroups
__global__ __launch_bounds__(256) void sum_accum_kernel(float* __restrict__ acc,
                                                        const float* __restrict__ parts,
                                                        int n_parts, long n4) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n4; i += (long)gridDim.x * 256) {
    float4 s = ((const float4*)parts)[i];
    for (int k = 1; k < n_parts; ++k) {
      const float4 t = ((const float4*)parts)[(long)k * n4 + i];
      s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
    }
    float4 a = ((float4*)acc)[i];
    a.x += s.x; a.y += s.y; a.z += s.z; a.w += s.w;
    ((float4*)acc)[i] = a;
  }
}

template <bool G_F32>
__global__ void grad_accum_tail_kernel(float* acc, const void* g, long start, long count) {
  const long i = start + blockIdx.x * 256 + threadIdx.x;
  if (i < count) acc[i] += G_F32 ? ((const float*)g)[i] : bf16_to_f32(((const bf16_t*)g)[i]);
}

__global__ __launch_bounds__(256) void cast_f32_bf16_kernel(const float* __restrict__ src,
                                                            bf16_t* __restrict__ dst, long n) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256)
    dst[i] = f32_to_bf16(src[i]);
}
__global__ __launch_bounds__(256) void cast_bf16_f32_kernel(const bf16_t* __restrict__ src,
                                                            float* __restrict__ dst, long n) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256)
    dst[i] = bf16_to_f32(src[i]);
}
__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t* dst, uint32_t v, long n) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256)
    dst[i] = v;
}

// loss of the last stage: mean((out - target)^2) * scale, and its cotangent
__global__ __launch_bounds__(256) void mse_partial_kernel(const bf16_t* __restrict__ out,
                                                          const bf16_t* __restrict__ target,
                                                          long n8, float dscale,
                                                          bf16_t* __restrict__ dout,
                                                          float* __restrict__ partial) {
  __shared__ float red[4];
  float s = 0.f;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n8; i += (long)gridDim.x * 256) {
    float a[8], b[8];
    unpack8(((const uint4*)out)[i], a);
    unpack8(((const uint4*)target)[i], b);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float d = a[e] - b[e];
      s += d * d;
      a[e] = d * dscale;
    }
    ((uint4*)dout)[i] = pack8(a);
  }
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) partial[blockIdx.x] = ((red[0] + red[1]) + red[2]) + red[3];
}
__global__ void mse_final_kernel(const float* partial, int n, float scale, float* loss) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    float s = 0.f;
    for (int i = 0; i < n; ++i) s += partial[i];
    loss[0] = s * scale;
  }
}

int grid_for(long items, int per_block = 256, int cap = 256 * 32) {
  long g = (items + per_block - 1) / per_block;
  return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}

template <bool LN>
int launch_norm_fwd(hipStream_t st, const jpp_norm_args* a) {
  const int blocks = (int)((a->rows + 3) / 4);
  const int nch = (int)((a->cols / 8 + 63) / 64);
#define JPP_NF(N)                                                                            \
  hipLaunchKernelGGL((norm_fwd_kernel<LN, N>), dim3(blocks), dim3(256), 0, st,               \
                     (const bf16_t*)a->x, (const bf16_t*)a->gamma, (const bf16_t*)a->beta,   \
                     (bf16_t*)a->y, a->mean, a->rstd, (long)a->rows, (int)a->cols, a->eps)
  if (nch <= 1) JPP_NF(1);
  else if (nch <= 2) JPP_NF(2);
  else if (nch <= 4) JPP_NF(4);
  else if (nch <= 8) JPP_NF(8);
  else JPP_NF(16);
#undef JPP_NF
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

template <bool LN>
int launch_norm_bwd(hipStream_t st, const jpp_norm_args* a) {
  const int nch = (int)((a->cols / 8 + 63) / 64);
  const int blocks = JPP_NORM_PARTIALS;
#define JPP_NB(N)                                                                             \
  hipLaunchKernelGGL((norm_bwd_kernel<LN, N>), dim3(blocks), dim3(kNormBwdWaves * 64), 0, st, \
                     (const bf16_t*)a->dy, (const bf16_t*)a->x, a->mean, a->rstd,             \
                     (const bf16_t*)a->gamma, (const bf16_t*)a->resid, (bf16_t*)a->dx,        \
                     a->partial, (long)a->rows, (int)a->cols)
#define JPP_NBW(N)                                                                            \
  hipLaunchKernelGGL((norm_bwd_wide_kernel<LN, N, 4>), dim3(blocks), dim3(512), 0, st,         \
                     (const bf16_t*)a->dy, (const bf16_t*)a->x, a->mean, a->rstd,             \
                     (const bf16_t*)a->gamma, (const bf16_t*)a->resid, (bf16_t*)a->dx,        \
                     a->partial, (long)a->rows, (int)a->cols)
  if (a->cols == 4096) JPP_NBW(1);
  else if (a->cols == 8192) JPP_NBW(2);
  else if (nch <= 1) JPP_NB(1);
  else if (nch <= 2) JPP_NB(2);
  else if (nch <= 4) JPP_NB(4);
  else if (nch <= 8) JPP_NB(8);
  else JPP_NB(16);
#undef JPP_NB
#undef JPP_NBW
  JPP_LAUNCH_CHECK();
  const int cb = (int)((a->cols + 31) / 32);
  hipLaunchKernelGGL(partial_reduce_kernel, dim3(cb, LN ? 2 : 1), dim3(1024), 0, st, a->partial,
                     blocks, (int)a->cols, a->dgamma, a->dbeta);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

}  // namespace

extern "C" {

int jpp_norm_fwd(void* stream, const jpp_norm_args* a) {
  JPP_REQUIRE(a && a->x && a->gamma && a->y && a->rstd, "norm_fwd: null operand");
  JPP_REQUIRE(a->rows > 0 && a->cols > 0 && a->cols % 8 == 0 &&
                  a->cols <= 8 * 64 * kMaxChunksPerLane,
              "norm_fwd: cols must be a multiple of 8 and at most %d, got %ld",
              8 * 64 * kMaxChunksPerLane, (long)a->cols);
  JPP_REQUIRE((a->beta == nullptr) == (a->mean == nullptr),
              "norm_fwd: beta and mean are both given (LayerNorm) or both NULL (RMSNorm)");
  ProbeScope probe((hipStream_t)stream, "norm_fwd", 0, 4.0 * a->rows * a->cols);
  return a->beta ? launch_norm_fwd<true>((hipStream_t)stream, a)
                 : launch_norm_fwd<false>((hipStream_t)stream, a);
}

int jpp_norm_bwd(void* stream, const jpp_norm_args* a) {
  JPP_REQUIRE(a && a->x && a->gamma && a->dy && a->dx && a->rstd && a->dgamma && a->partial,
              "norm_bwd: null operand");
  JPP_REQUIRE(a->rows > 0 && a->cols > 0 && a->cols % 8 == 0 &&
                  a->cols <= 8 * 64 * kMaxChunksPerLane,
              "norm_bwd: cols must be a multiple of 8 and at most %d, got %ld",
              8 * 64 * kMaxChunksPerLane, (long)a->cols);
  const bool ln = a->mean != nullptr;
  JPP_REQUIRE(!ln || a->dbeta, "norm_bwd: LayerNorm needs dbeta");
  ProbeScope probe((hipStream_t)stream, "norm_bwd", 0, (a->resid ? 8.0 : 6.0) * a->rows * a->cols);
  return ln ? launch_norm_bwd<true>((hipStream_t)stream, a)
            : launch_norm_bwd<false>((hipStream_t)stream, a);
}

int jpp_norm_bwd_static(void* stream, const jpp_norm_args* a) {
  JPP_REQUIRE(a, "norm_bwd_static: null operand");
  JPP_REQUIRE(a->cols > 0 && a->cols <= kStaticNormCols,
              "norm_bwd_static: %ld columns exceed the %d the library's own scratch holds",
              (long)a->cols, kStaticNormCols);
  float* ptr = nullptr;
  if (int rc = static_scratch(&ptr)) return rc;
  // The kernels write rows 0 .. JPP_NORM_PARTIALS-1 (and, for LayerNorm, the same number of
  // rows behind them) of `cols` columns before the reduction reads exactly those, so nothing
  // of an earlier call is read and nothing needs clearing.
  jpp_norm_args b = *a;
  b.partial = ptr;
  return jpp_norm_bwd(stream, &b);
}

int jpp_swiglu_fwd(void* stream, const void* gu, void* s, int64_t rows, int64_t f,
                   int interleaved) {
  JPP_REQUIRE(gu && s && rows > 0 && f > 0 && f % (interleaved ? 32 : 8) == 0,
              "swiglu_fwd: bad arguments");
  ProbeScope probe((hipStream_t)stream, "swiglu_fwd", 0, 6.0 * rows * f);
  hipLaunchKernelGGL(swiglu_fwd_kernel, dim3(grid_for(rows * (f / 8))), dim3(256), 0,
                     (hipStream_t)stream, (const bf16_t*)gu, (bf16_t*)s, (long)rows, (int)f,
                     interleaved);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_swiglu_bwd(void* stream, const void* gu, const void* ds, void* dgu, int64_t rows,
                   int64_t f, int interleaved) {
  JPP_REQUIRE(gu && ds && dgu && rows > 0 && f > 0 && f % (interleaved ? 32 : 8) == 0,
              "swiglu_bwd: bad arguments");
  ProbeScope probe((hipStream_t)stream, "swiglu_bwd", 0, 10.0 * rows * f);
  hipLaunchKernelGGL(swiglu_bwd_kernel, dim3(grid_for(rows * (f / 8))), dim3(256), 0,
                     (hipStream_t)stream, (const bf16_t*)gu, (const bf16_t*)ds, (bf16_t*)dgu,
                     (long)rows, (int)f, interleaved);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_rope(void* stream, void* x, int64_t ld, const float* cos_tab, const float* sin_tab,
             int batch, int seq, int n_rot_heads, int head_dim, int inverse) {
  JPP_REQUIRE(x && cos_tab && sin_tab, "rope: null operand");
  JPP_REQUIRE(batch > 0 && seq > 0 && n_rot_heads > 0 && head_dim % 16 == 0 && ld % 8 == 0 &&
                  ld >= (int64_t)n_rot_heads * head_dim,
              "rope: bad shape");
  const long rows = (long)batch * seq;
  ProbeScope probe((hipStream_t)stream, "rope", 0, 4.0 * rows * n_rot_heads * head_dim);
  hipLaunchKernelGGL(rope_kernel, dim3(grid_for(rows * n_rot_heads * (head_dim / 16))), dim3(256),
                     0, (hipStream_t)stream, (bf16_t*)x, (long)ld, cos_tab, sin_tab, rows, seq,
                     n_rot_heads, head_dim, inverse);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_grad_accum_f32(void* stream, float* acc, const void* g, int64_t count, int g_is_f32) {
  JPP_REQUIRE(acc && g && count >= 0, "grad_accum: bad arguments");
  JPP_REQUIRE((uintptr_t)acc % 16 == 0 && (uintptr_t)g % 16 == 0,
              "grad_accum: operands must be 16-byte aligned");
  if (count == 0) return JPP_OK;
  ProbeScope probe((hipStream_t)stream, "grad_accum", 0, (g_is_f32 ? 12.0 : 10.0) * count);
  const long n8 = count / 8;
  hipStream_t st = (hipStream_t)stream;
  if (n8) {
    if (g_is_f32)
      hipLaunchKernelGGL(grad_accum_kernel<true>, dim3(grid_for(n8)), dim3(256), 0, st, acc, g, n8);
    else
      hipLaunchKernelGGL(grad_accum_kernel<false>, dim3(grid_for(n8)), dim3(256), 0, st, acc, g, n8);
  }
  if (count % 8) {
    if (g_is_f32)
      hipLaunchKernelGGL(grad_accum_tail_kernel<true>, dim3(1), dim3(256), 0, st, acc, g, n8 * 8,
                         (long)count);
    else
      hipLaunchKernelGGL(grad_accum_tail_kernel<false>, dim3(1), dim3(256), 0, st, acc, g, n8 * 8,
                         (long)count);
  }
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_colsum_accum(void* stream, const void* x, int64_t ld, int64_t rows, int64_t cols,
                     float* acc, float* partial) {
  JPP_REQUIRE(x && acc && partial && rows > 0 && cols > 0 && cols % 8 == 0 && ld % 8 == 0 &&
                  ld >= cols,
              "colsum: bad arguments");
  hipStream_t st = (hipStream_t)stream;
  ProbeScope probe(st, "colsum", 0, 2.0 * rows * cols);
  const int nb = (int)(rows < JPP_NORM_PARTIALS ? rows : JPP_NORM_PARTIALS);
  const int panels = (int)((cols / 8 + 255) / 256);
  hipLaunchKernelGGL(colsum_partial_kernel, dim3(nb, panels), dim3(256), 0, st, (const bf16_t*)x,
                     (long)ld, (long)rows, (int)cols, partial);
  hipLaunchKernelGGL(partial_reduce_kernel, dim3((int)((cols + 31) / 32)), dim3(1024), 0, st,
                     partial, nb, (int)cols, acc, (float*)nullptr);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_sum_accum_f32(void* stream, float* acc, const float* parts, int n_parts, int64_t count) {
  JPP_REQUIRE(acc && parts && n_parts >= 1 && count > 0 && count % 4 == 0,
              "sum_accum: bad arguments (count must be a positive multiple of 4)");
  JPP_REQUIRE((uintptr_t)acc % 16 == 0 && (uintptr_t)parts % 16 == 0,
              "sum_accum: operands must be 16-byte aligned");
  ProbeScope probe((hipStream_t)stream, "sum_accum", 0, (4.0 * n_parts + 8.0) * count);
  hipLaunchKernelGGL(sum_accum_kernel, dim3(grid_for(count / 4)), dim3(256), 0, (hipStream_t)stream,
                     acc, parts, n_parts, (long)(count / 4));
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_colsum_accum_multi(void* stream, int n, const jpp_colsum_item* items, int64_t rows,
                           float* partial) {
  JPP_REQUIRE(items && partial && n >= 1 && n <= 4 && rows > 0,
              "colsum_multi: 1 to 4 tensors and a partial-sum buffer are required");
  ColsumBatch b;
  b.n = n;
  int at = 0;
  double bytes = 0;
  for (int i = 0; i < n; ++i) {
    const jpp_colsum_item& it = items[i];
    JPP_REQUIRE(it.x && it.acc && it.cols > 0 && it.cols % 8 == 0 && it.ld % 8 == 0 &&
                    it.ld >= it.cols && (uintptr_t)it.x % 16 == 0,
                "colsum_multi: tensor %d: cols and ld must be multiples of 8, ld >= cols", i);
    b.x[i] = (const bf16_t*)it.x;
    b.ld[i] = it.ld;
    b.acc[i] = it.acc;
    b.start[i] = at;
    at += (int)it.cols;
    bytes += 2.0 * rows * it.cols;
  }
  b.start[n] = at;
  hipStream_t st = (hipStream_t)stream;
  ProbeScope probe(st, "colsum", 0, bytes);
  const int nb = (int)(rows < JPP_NORM_PARTIALS ? rows : JPP_NORM_PARTIALS);
  const int panels = (at / 8 + 255) / 256;
  hipLaunchKernelGGL(colsum_multi_partial_kernel, dim3(nb, panels), dim3(256), 0, st, b, (long)rows,
                     partial);
  hipLaunchKernelGGL(colsum_multi_reduce_kernel, dim3((at + 31) / 32), dim3(1024), 0, st, partial, nb,
                     b);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_mse_loss(void* stream, const void* out, const void* target, int64_t count, float scale,
                 float* loss, void* dout, float* partial) {
  JPP_REQUIRE(out && target && loss && dout && partial && count > 0 && count % 8 == 0,
              "mse_loss: bad arguments (count must be a positive multiple of 8)");
  hipStream_t st = (hipStream_t)stream;
  const long n8 = count / 8;
  const int nb = (int)(n8 < JPP_NORM_PARTIALS ? n8 : JPP_NORM_PARTIALS);
  ProbeScope probe(st, "mse", 0, 6.0 * count);
  hipLaunchKernelGGL(mse_partial_kernel, dim3(nb), dim3(256), 0, st, (const bf16_t*)out,
                     (const bf16_t*)target, n8, 2.0f * scale / (float)count, (bf16_t*)dout, partial);
  hipLaunchKernelGGL(mse_final_kernel, dim3(1), dim3(64), 0, st, partial, nb,
                     scale / (float)count, loss);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_cast_f32_to_bf16(void* stream, const float* src, void* dst, int64_t count) {
  JPP_REQUIRE(src && dst && count > 0, "cast: bad arguments");
  ProbeScope probe((hipStream_t)stream, "cast", 0, 6.0 * count);
  hipLaunchKernelGGL(cast_f32_bf16_kernel, dim3(grid_for(count)), dim3(256), 0,
                     (hipStream_t)stream, src, (bf16_t*)dst, (long)count);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_cast_bf16_to_f32(void* stream, const void* src, float* dst, int64_t count) {
  JPP_REQUIRE(src && dst && count > 0, "cast: bad arguments");
  ProbeScope probe((hipStream_t)stream, "cast", 0, 6.0 * count);
  hipLaunchKernelGGL(cast_bf16_f32_kernel, dim3(grid_for(count)), dim3(256), 0,
                     (hipStream_t)stream, (const bf16_t*)src, dst, (long)count);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

int jpp_fill_u32(void* dst, uint32_t value, size_t count, void* stream) {
  JPP_REQUIRE(dst || count == 0, "fill: null destination");
  if (count == 0) return JPP_OK;
  ProbeScope probe((hipStream_t)stream, "fill", 0, 4.0 * count);
  hipLaunchKernelGGL(fill_u32_kernel, dim3(grid_for((long)count)), dim3(256), 0,
                     (hipStream_t)stream, (uint32_t*)dst, value, (long)count);
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}

}  // extern "C"
