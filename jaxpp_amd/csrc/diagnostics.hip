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

// 8 waves of one workgroup read LDS in a loop, every wave with the same per-lane byte
// offsets; lane 0 of wave 0 reports the shader clocks the loop took.  Eight reads are in
// flight per wave, so the LDS pipeline stays full and the time per read is what the
// pattern costs in LDS cycles (bank conflicts included), not its latency.
typedef int lds_v4i __attribute__((ext_vector_type(4)));
typedef int lds_v2i __attribute__((ext_vector_type(2)));
constexpr int kLdsProbeBytes = 65536;
template <bool TRANSPOSING>
__global__ __launch_bounds__(512) void lds_read_rate_kernel(const uint32_t* offsets, int iters,
                                                            long long* cycles, int* sink) {
  extern __shared__ uint8_t lds[];
  for (int i = threadIdx.x; i < kLdsProbeBytes / 4; i += 512) ((uint32_t*)lds)[i] = i;
  __syncthreads();
  const uint32_t a = lds_address(lds) + offsets[threadIdx.x & 63];
  int acc = 0;
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
    if constexpr (!TRANSPOSING) {
      lds_v4i r0, r1, r2, r3, r4, r5, r6, r7;
      asm volatile(
          "ds_read_b128 %0, %8\n\tds_read_b128 %1, %8\n\tds_read_b128 %2, %8\n\t"
          "ds_read_b128 %3, %8\n\tds_read_b128 %4, %8\n\tds_read_b128 %5, %8\n\t"
          "ds_read_b128 %6, %8\n\tds_read_b128 %7, %8\n\ts_waitcnt lgkmcnt(0)"
          : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3), "=&v"(r4), "=&v"(r5), "=&v"(r6),
            "=&v"(r7)
          : "v"(a)
          : "memory");
      acc += r0.x + r1.y + r2.z + r3.w + r4.x + r5.y + r6.z + r7.w;
    } else {
      lds_v2i r0, r1, r2, r3, r4, r5, r6, r7;
      asm volatile(
          "ds_read_b64_tr_b16 %0, %8\n\tds_read_b64_tr_b16 %1, %8\n\t"
          "ds_read_b64_tr_b16 %2, %8\n\tds_read_b64_tr_b16 %3, %8\n\t"
          "ds_read_b64_tr_b16 %4, %8\n\tds_read_b64_tr_b16 %5, %8\n\t"
          "ds_read_b64_tr_b16 %6, %8\n\tds_read_b64_tr_b16 %7, %8\n\ts_waitcnt lgkmcnt(0)"
          : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3), "=&v"(r4), "=&v"(r5), "=&v"(r6),
            "=&v"(r7)
          : "v"(a)
          : "memory");
      acc += r0.x + r1.y + r2.x + r3.y + r4.x + r5.y + r6.x + r7.y;
    }
  }
  const long long t1 = clock64();
  if (threadIdx.x == 0) *cycles = t1 - t0;
  sink[threadIdx.x & 63] = acc;
}

}  // namespace

extern "C" int jpp_lds_read_rate(const uint32_t* lane_offsets, int transposing,
                                 double* cycles_per_read) {
  JPP_REQUIRE(lane_offsets && cycles_per_read, "lds_read_rate: null argument");
  const uint32_t width = transposing ? 8 : 16;
  for (int l = 0; l < 64; ++l)
    JPP_REQUIRE(lane_offsets[l] % width == 0 && lane_offsets[l] + width <= (uint32_t)kLdsProbeBytes,
                "lds_read_rate: lane %d reads %u bytes at offset %u: not aligned, or beyond the "
                "%d bytes of LDS the probe owns", l, width, lane_offsets[l], kLdsProbeBytes);
  constexpr int kIters = 2000;
  uint32_t* d_off = nullptr;
  long long* d_cycles = nullptr;
  int* d_sink = nullptr;
  hipError_t err = hipMalloc((void**)&d_off, 64 * sizeof(uint32_t));
  if (err == hipSuccess) err = hipMalloc((void**)&d_cycles, sizeof(long long));
  if (err == hipSuccess) err = hipMalloc((void**)&d_sink, 64 * sizeof(int));
  if (err == hipSuccess)
    err = hipMemcpy(d_off, lane_offsets, 64 * sizeof(uint32_t), hipMemcpyHostToDevice);
  auto kern = transposing ? lds_read_rate_kernel<true> : lds_read_rate_kernel<false>;
  if (err == hipSuccess)
    err = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                              kLdsProbeBytes);
  long long cycles = 0;
  for (int rep = 0; rep < 2 && err == hipSuccess; ++rep) {  // the second run is the warm one
    hipLaunchKernelGGL(kern, dim3(1), dim3(512), kLdsProbeBytes, nullptr, d_off, kIters, d_cycles,
                       d_sink);
    err = hipGetLastError();
    if (err == hipSuccess) err = hipDeviceSynchronize();
    if (err == hipSuccess)
      err = hipMemcpy(&cycles, d_cycles, sizeof(cycles), hipMemcpyDeviceToHost);
  }
  if (d_off) hipFree(d_off);
  if (d_cycles) hipFree(d_cycles);
  if (d_sink) hipFree(d_sink);
  if (err != hipSuccess)
    return jpp_set_error(JPP_ERR_HIP, "lds_read_rate: %s", hipGetErrorString(err));
  *cycles_per_read = (double)cycles / (kIters * 8.0 * 8.0);  // 8 waves x 8 reads per trip
  return JPP_OK;
}

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
