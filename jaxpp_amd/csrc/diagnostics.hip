// What the matrix cores of this device sustain with nothing else in flight: a register-only
// loop of MFMAs on every SIMD (8 waves per CU, 256 CUs), timed with events.  The GEMM
// kernels are priced against the published peak; this figure says how much of the distance
// to it is the device's (clock under load depends on how many operand bits toggle) and how
// much is the kernels'.
#include "common.h"
#include "../../include/jaxpp_amd_diag.h"

namespace {

__device__ __forceinline__ uint32_t lcg(uint32_t& s) {
  s = s * 1664525u + 1013904223u;
  return s;
}

// SHAPE 32: v_mfma_f32_32x32x16_bf16 on 8 accumulators; 16: v_mfma_f32_16x16x32_bf16 on 32
// (128 accumulator registers either way).
// Operands differ from one MFMA to the next (as in a GEMM) unless they are all zero.
template <int SHAPE>
__global__ __launch_bounds__(512) void mfma_rate_kernel(float* out, int iters, int random_operands) {
  bf16x8 a[8], b[8];
  uint32_t s = threadIdx.x * 7919u + blockIdx.x * 104729u + 12345u;
  for (int i = 0; i < 8; ++i)
    for (int e = 0; e < 8; ++e) {
      const float x = random_operands ? ((int)(lcg(s) >> 8) % 2001 - 1000) * 0.001f : 0.f;
      const float y = random_operands ? ((int)(lcg(s) >> 8) % 2001 - 1000) * 0.00002f : 0.f;
      a[i][e] = (__bf16)x;
      b[i][e] = (__bf16)y;
    }
  float sum = 0.f;
  if constexpr (SHAPE == 16) {
    f32x4 acc[32];
    for (int i = 0; i < 32; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 32; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i & 7], b[(i * 3 + 1) & 7], acc[i], 0, 0, 0);
    }
    for (int i = 0; i < 32; ++i) sum += acc[i][0];
  } else {
    f32x16 acc[8];
    for (int i = 0; i < 8; ++i)
      for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[(i * 3 + 1) & 7], acc[i], 0, 0, 0);
    }
    for (int i = 0; i < 8; ++i) sum += acc[i][0];
  }
  out[blockIdx.x * 512 + threadIdx.x] = sum;
}

}  // namespace

extern "C" int jpp_mfma_rate(int shape, int random_operands, int64_t iters, double* tflops) {
  JPP_REQUIRE(tflops, "mfma_rate: null result");
  JPP_REQUIRE(shape == 16 || shape == 32, "mfma_rate: shape is 16 (16x16x32) or 32 (32x32x16)");
  JPP_REQUIRE(iters > 0 && iters <= (1 << 24), "mfma_rate: iters out of range");
  constexpr int kBlocks = 256;
  float* out = nullptr;
  JPP_CHECK_HIP(hipMalloc((void**)&out, kBlocks * 512 * sizeof(float)));
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipError_t err = hipEventCreate(&e0);
  if (err == hipSuccess) err = hipEventCreate(&e1);
  float ms = 0.f;
  if (err == hipSuccess) {
    for (int rep = 0; rep < 2 && err == hipSuccess; ++rep) {  // the second run is the warm one
      hipEventRecord(e0, nullptr);
      if (shape == 16)
        hipLaunchKernelGGL(mfma_rate_kernel<16>, dim3(kBlocks), dim3(512), 0, nullptr, out,
                           (int)iters, random_operands);
      else
        hipLaunchKernelGGL(mfma_rate_kernel<32>, dim3(kBlocks), dim3(512), 0, nullptr, out,
                           (int)iters, random_operands);
      hipEventRecord(e1, nullptr);
      err = hipEventSynchronize(e1);
      if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
    }
  }
  if (e0) hipEventDestroy(e0);
  if (e1) hipEventDestroy(e1);
  hipFree(out);
  if (err != hipSuccess)
    return jpp_set_error(JPP_ERR_HIP, "mfma_rate: %s", hipGetErrorString(err));
  // per trip and wave: 32 MFMAs of 2*16*16*32 flops or 8 of 2*32*32*16
  const double per_trip = shape == 16 ? 32 * 16384.0 : 8 * 32768.0;
  *tflops = (double)kBlocks * 8 * (double)iters * per_trip / (ms * 1e-3) / 1e12;
  return JPP_OK;
}
