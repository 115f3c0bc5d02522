// The step on the far side of the microbatch loop: Adam on the f32 gradient accumulators
// the loop leaves behind (README.md:90-93 applies `optimizer.update` + `apply_updates` to
// the gradients `treduce` returns; examples/basic.py:234 uses `optax.adam`).  One pass over
// a flat tensor: reads gradient, both moments and the f32 weights, writes moments, weights
// and the bf16 copy the stage computes with, and can clear the accumulator for the next
// loop on the way - 16 bytes read and 18 written per parameter, all of it HBM traffic.
#include <math.h>

#include "common.h"

namespace {

struct AdamParams {
  float* grad;
  float* master;
  bf16_t* param;
  float* m;
  float* v;
  float lr, b1, b2, omb1, omb2, eps, bc1, bc2, gscale;  // omb = 1 - beta, bc = 1 - beta^t
  int zero_grad;
};

// the arithmetic of optax.adam (eps outside the root, eps_root = 0): m and v are the
// exponential averages of g and g^2, each divided by 1 - beta^t before use
__device__ __forceinline__ float adam_one(const AdamParams& p, float g, float w, float& m,
                                          float& v) {
  g *= p.gscale;
  m = p.b1 * m + p.omb1 * g;
  v = p.b2 * v + p.omb2 * g * g;
  const float mh = m / p.bc1, vh = v / p.bc2;
  return w - p.lr * mh / (sqrtf(vh) + p.eps);
}

__device__ __forceinline__ void adam_four(const AdamParams& p, const float4& g, float4& w,
                                          float4& m, float4& v) {
  w.x = adam_one(p, g.x, w.x, m.x, v.x);
  w.y = adam_one(p, g.y, w.y, m.y, v.y);
  w.z = adam_one(p, g.z, w.z, m.z, v.z);
  w.w = adam_one(p, g.w, w.w, m.w, v.w);
}

// 8 parameters per lane and trip: two 16-byte pieces of every f32 tensor, one of the bf16
template <bool MASTER>
__global__ __launch_bounds__(256) void adam_kernel(AdamParams p, long n8) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n8; i += (long)gridDim.x * 256) {
    const float4 g0 = ((const float4*)p.grad)[2 * i], g1 = ((const float4*)p.grad)[2 * i + 1];
    float4 m0 = ((const float4*)p.m)[2 * i], m1 = ((const float4*)p.m)[2 * i + 1];
    float4 v0 = ((const float4*)p.v)[2 * i], v1 = ((const float4*)p.v)[2 * i + 1];
    float4 w0, w1;
    if (MASTER) {
      w0 = ((const float4*)p.master)[2 * i];
      w1 = ((const float4*)p.master)[2 * i + 1];
    } else {
      float f[8];
      unpack8(((const uint4*)p.param)[i], f);
      w0 = make_float4(f[0], f[1], f[2], f[3]);
      w1 = make_float4(f[4], f[5], f[6], f[7]);
    }
    adam_four(p, g0, w0, m0, v0);
    adam_four(p, g1, w1, m1, v1);
    ((float4*)p.m)[2 * i] = m0;
    ((float4*)p.m)[2 * i + 1] = m1;
    ((float4*)p.v)[2 * i] = v0;
    ((float4*)p.v)[2 * i + 1] = v1;
    if (MASTER) {
      ((float4*)p.master)[2 * i] = w0;
      ((float4*)p.master)[2 * i + 1] = w1;
    }
    if (p.param) {
      const float f[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
      ((uint4*)p.param)[i] = pack8(f);
    }
    if (p.zero_grad) {
      ((float4*)p.grad)[2 * i] = make_float4(0.f, 0.f, 0.f, 0.f);
      ((float4*)p.grad)[2 * i + 1] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
}

template <bool MASTER>
__global__ void adam_tail_kernel(AdamParams p, long start, long count) {
  const long i = start + threadIdx.x;
  if (i >= count) return;
  float m = p.m[i], v = p.v[i];
  const float w = adam_one(p, p.grad[i], MASTER ? p.master[i] : bf16_to_f32(p.param[i]), m, v);
  p.m[i] = m;
  p.v[i] = v;
  if (MASTER) p.master[i] = w;
  if (p.param) p.param[i] = f32_to_bf16(w);
  if (p.zero_grad) p.grad[i] = 0.f;
}

}  // namespace

extern "C" int jpp_adam_step(void* stream, const jpp_adam_args* a) {
  JPP_REQUIRE(a && a->grad && a->m && a->v && (a->master || a->param),
              "adam_step: null operand (grad, m, v and one of master / param are required)");
  JPP_REQUIRE(a->count >= 0, "adam_step: negative count");
  JPP_REQUIRE(((uintptr_t)a->grad | (uintptr_t)a->m | (uintptr_t)a->v | (uintptr_t)a->master |
               (uintptr_t)a->param) % 16 == 0,
              "adam_step: operands must be 16-byte aligned");
  JPP_REQUIRE(a->step >= 1, "adam_step: step counts from 1, got %ld", (long)a->step);
  JPP_REQUIRE(a->beta1 >= 0. && a->beta1 < 1. && a->beta2 >= 0. && a->beta2 < 1.,
              "adam_step: beta1, beta2 must lie in [0, 1)");
  if (a->count == 0) return JPP_OK;
  AdamParams p;
  p.grad = a->grad; p.master = a->master; p.param = (bf16_t*)a->param; p.m = a->m; p.v = a->v;
  // every scalar is formed in double and rounded once, as a Python float that meets an f32
  // array is
  p.lr = (float)a->lr; p.b1 = (float)a->beta1; p.b2 = (float)a->beta2; p.eps = (float)a->eps;
  p.omb1 = (float)(1.0 - a->beta1);
  p.omb2 = (float)(1.0 - a->beta2);
  p.bc1 = (float)(1.0 - pow(a->beta1, (double)a->step));
  p.bc2 = (float)(1.0 - pow(a->beta2, (double)a->step));
  p.gscale = (float)a->grad_scale;
  p.zero_grad = a->zero_grad;
  hipStream_t st = (hipStream_t)stream;
  const double bytes = 12.0 + 8.0 + (a->master ? 8.0 : 2.0) + (a->param ? 2.0 : 0.0) +
                       (a->zero_grad ? 4.0 : 0.0);
  ProbeScope probe(st, "adam", 0, bytes * a->count);
  const long n8 = a->count / 8;
  const int grid = (int)(n8 < 1 ? 1 : (n8 + 255) / 256 > 256 * 32 ? 256 * 32 : (n8 + 255) / 256);
  if (n8) {
    if (a->master) hipLaunchKernelGGL(adam_kernel<true>, dim3(grid), dim3(256), 0, st, p, n8);
    else hipLaunchKernelGGL(adam_kernel<false>, dim3(grid), dim3(256), 0, st, p, n8);
  }
  if (a->count % 8) {
    if (a->master)
      hipLaunchKernelGGL(adam_tail_kernel<true>, dim3(1), dim3(8), 0, st, p, n8 * 8, (long)a->count);
    else
      hipLaunchKernelGGL(adam_tail_kernel<false>, dim3(1), dim3(8), 0, st, p, n8 * 8, (long)a->count);
  }
  JPP_LAUNCH_CHECK();
  return JPP_OK;
}
