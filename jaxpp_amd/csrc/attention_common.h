// Pieces shared by the attention kernels: parameters, fragment helpers, the HBM -> LDS tile
// copy and the per-XCD work order.
#ifndef JAXPP_AMD_ATTENTION_COMMON_H_
#define JAXPP_AMD_ATTENTION_COMMON_H_

#include <math.h>

#include <type_traits>

#include "common.h"

namespace jpp_attn {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct AttnParams {
  const bf16_t* q; const bf16_t* k; const bf16_t* v;
  bf16_t* o; float* lse;
  const bf16_t* d_o;
  bf16_t* dq; bf16_t* dk; bf16_t* dv;
  float* delta;
  long ldq, ldk, ldv, ldo, lddo, lddq, lddk, lddv;
  int batch, seq, n_heads, n_kv_heads;
  float scale;
  const float* rope_cos;  // backward: dq / dk leave rotated back when set
  const float* rope_sin;
};

// Transpose of the half-split rotary embedding on an accumulator row: the lane holds, of
// the row at sequence position `pos`, the head's elements d = 32 i + 8 (r / 4) + 4 (lane /
// 32) + r % 4 in acc[i][r]; element d < D/2 pairs with d + D/2, i.e. acc[i] with
// acc[i + DT/2], same r.  The values are rounded to bf16 first, as a separate pass would
// read them back from memory.
template <int D, int DT>
__device__ __forceinline__ void rope_back(f32x16 (&acc)[DT], const float* cos_tab,
                                          const float* sin_tab, int pos, int lane) {
  static_assert(DT * 32 == D && DT % 2 == 0, "head of D elements in DT tiles of 32");
  const float* ct = cos_tab + (long)pos * (D / 2) + (lane >> 5) * 4;
  const float* st = sin_tab + (long)pos * (D / 2) + (lane >> 5) * 4;
#pragma unroll
  for (int i = 0; i < DT / 2; ++i)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float4 c4 = *(const float4*)(ct + i * 32 + g * 8);
      const float4 s4 = *(const float4*)(st + i * 32 + g * 8);
      const float cs[4] = {c4.x, c4.y, c4.z, c4.w}, sn[4] = {-s4.x, -s4.y, -s4.z, -s4.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float a = (float)(__bf16)acc[i][4 * g + e];
        const float b = (float)(__bf16)acc[i + DT / 2][4 * g + e];
        acc[i][4 * g + e] = a * cs[e] - b * sn[e];
        acc[i + DT / 2][4 * g + e] = b * cs[e] + a * sn[e];
      }
    }
}

// 8 consecutive accumulator registers -> one bf16 MFMA operand (round to nearest even; two
// elements per conversion instruction)
__device__ __forceinline__ bf16x8 acc_to_frag(const f32x16& a, int base) {
  typedef float f32x8 __attribute__((ext_vector_type(8)));
  const f32x8 v = {a[base], a[base + 1], a[base + 2], a[base + 3],
                   a[base + 4], a[base + 5], a[base + 6], a[base + 7]};
  return __builtin_convertvector(v, bf16x8);
}

// row-major operand fragment straight from HBM (lane: row = lane&31, 8
// contraction elements of step ks)
__device__ __forceinline__ bf16x8 global_frag(const bf16_t* base, long ld, int ks, int lane) {
  return *(const bf16x8*)(base + (long)(lane & 31) * ld + ks * 16 + (lane >> 5) * 8);
}

// a [64][D] tile lives in LDS as D/64 slabs of [64][64]
template <int D>
__device__ __forceinline__ bf16x8 slabs_frag(const uint8_t* slabs, int row0, int ks, int lane) {
  return slab_frag(slabs + (ks >> 2) * 8192, row0, ks & 3, lane);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// MFMAs as volatile asm statements, for the kernels that run one wave per SIMD and order
// their own instructions: such statements are emitted where they are written, in the order
// they are written, and LDS reads do not cross them.  The first letter names where the
// accumulator lives, the other two the operands: `a` the accumulation registers (reached by
// MFMAs and loads only), `v` the ordinary ones (where elementwise code can read a result).
// The compiler does not know these statements are MFMAs: a kernel that uses them keeps every
// other access to their results 11 issue slots behind them itself.
#define JPP_MFMA(NAME, ACC, A, B)                                                          \
  __device__ __forceinline__ void NAME(f32x16& acc, const bf16x8& a, const bf16x8& b) {    \
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0"                                 \
                 : "+" ACC(acc) : A(a), B(b) : "memory");                                  \
  }
JPP_MFMA(mfma_avv, "a", "v", "v")
JPP_MFMA(mfma_vaa, "v", "a", "a")
JPP_MFMA(mfma_vva, "v", "v", "a")
JPP_MFMA(mfma_vvv, "v", "v", "v")
#undef JPP_MFMA
// the first product of a chain: the accumulator starts from zero
__device__ __forceinline__ void mfma_vva_first(f32x16& acc, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "a"(b) : "memory");
}
__device__ __forceinline__ void mfma_vvv_first(f32x16& acc, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "v"(b) : "memory");
}
__device__ __forceinline__ void mfma_vaa_first(f32x16& acc, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "a"(a), "a"(b) : "memory");
}
// two floats -> one register of two bf16 (round to nearest even), one instruction
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// A wave's 32 x D result tile leaves through LDS by rows.  In the accumulators a lane holds,
// of row lane & 31, the columns 32 i + 8 g + 4 (lane >> 5) + 0..3 in acc[i][4 g ..]: stored
// from there, one instruction would touch 32 rows with 8 bytes each, and the CU's path to
// memory takes such an instruction line by line.  So the tile is rounded to bf16 into `stage`
// (32 * D * 2 bytes of LDS that only this wave uses; 16-byte units of a row XOR-ed with the
// row index, which spreads a write over the banks) and read back with a lane owning 16
// consecutive bytes of a row, 64 / (D / 8) whole rows per store instruction.  LDS operations
// of one wave execute in order: no barrier.
template <int D, int DT>
__device__ __forceinline__ void store_tile_by_rows(const f32x16 (&acc)[DT], uint32_t stage,
                                                   bf16_t* dst, long ld, int lane) {
  static_assert(DT * 32 == D, "head of D elements in DT tiles of 32");
  constexpr int UNITS = D / 8, RPI = 64 / UNITS;
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) u32x2* lds_u2;
  typedef __attribute__((address_space(3))) const u32x4* lds_u4;
  const int row = lane & 31, hh = lane >> 5;
  const uint32_t wbase = stage + row * (D * 2) + hh * 8;
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int u = i * 4 + g;
      *(lds_u2)(uintptr_t)(wbase + (uint32_t)((u ^ (row & (UNITS - 1))) << 4)) =
          u32x2{pack2(acc[i][4 * g], acc[i][4 * g + 1]), pack2(acc[i][4 * g + 2], acc[i][4 * g + 3])};
    }
  const int r0 = lane / UNITS, U = lane % UNITS;
#pragma unroll
  for (int k = 0; k < 32 / RPI; ++k) {
    const int r = k * RPI + r0;
    const u32x4 v = *(lds_u4)(uintptr_t)(stage + r * (D * 2) + (uint32_t)((U ^ (r & (UNITS - 1))) << 4));
    *(u32x4*)(dst + (long)r * ld + U * 8) = v;
  }
}


// f(integral_constant<int, I>) for I = FROM .. TO - 1
template <int FROM, int TO, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (FROM < TO) {
    f(std::integral_constant<int, FROM>{});
    static_for<FROM + 1, TO>(f);
  }
}

// One wave-level HBM -> LDS load whose LDS address is `lds_base` + IMM (both wave-uniform;
// the add writes M0 itself) and whose source is the wave-uniform address `src` + OFF bytes +
// the lane's `off`.  (The instruction's offset field moves the source and the LDS address
// alike, so M0 is set OFF short of the target.)
template <int IMM, int OFF>
__device__ __forceinline__ void dma_load16_at(uint64_t src, uint32_t off, uint32_t lds_base) {
  static_assert(OFF >= 0 && OFF < 4096 && IMM >= OFF, "offset field of a global load");
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%4"
               :
               : "s"(lds_base), "v"(off), "s"(src), "n"(IMM - OFF), "n"(OFF)
               : "memory", "scc");
}
__device__ __forceinline__ uint64_t uniform_u64(uint64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | lo;
}

// Makes the compiler wait here for the loads that produce these registers.  Without it the
// wait lands at their first use inside the main loop as a vmcnt count, and there it also
// waits for the HBM -> LDS copies of the next tile, which the wave has just issued (vmcnt
// counts every vector memory operation of the wave, in order).
template <int N>
__device__ __forceinline__ void settle(bf16x8 (&f)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+v"(f[i]));
}
__device__ __forceinline__ void settle(float& x) { asm volatile("" : "+v"(x)); }

// HBM -> LDS copy of a [64][D] tile (row stride ld) by the 4 waves of a
// workgroup, as D/64 swizzled slabs; no registers involved.
using Tile64 = DmaTile<64, false>;
template <int D>
__device__ __forceinline__ void dma_tile(const bf16_t* src, const Tile64::Offsets& off,
                                         uint32_t lds, int wave) {
#pragma unroll
  for (int c = 0; c < D / 64; ++c)
    Tile64::issue<0, Tile64::INSTS>(uniform_ptr(src + c * 64), off, lds + c * 8192, wave);
}

// Which (block, head, batch) a workgroup works on.  Workgroups are handed to the 8 XCDs
// round robin in launch order, and each XCD has its own L2: the launch order is rearranged
// so that one XCD sees only 1/8 of the (head, batch) pairs - adjacent heads, which share
// their K/V under grouped-query attention - and its K/V working set stays in its L2.
// Within an XCD blocks still go out in increasing x for all its heads (heavy first).
struct Work { int x, h, b; };
__device__ __forceinline__ Work xcd_work() {
  const int gx = gridDim.x, gy = gridDim.y;
  const int pairs = gy * gridDim.z;
  int x = blockIdx.x, pair = blockIdx.y + gy * blockIdx.z;
  if ((pairs & 7) == 0) {
    const int l = x + gx * pair, per = pairs >> 3;
    const int xcd = l & 7, j = l >> 3;
    x = j / per;
    pair = xcd * per + j % per;
  }
  return {x, pair % gy, pair / gy};
}

// sets the kernel's dynamic LDS limit (sticky per kernel)
template <class K>
int set_smem(K kern, int bytes) {
  JPP_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    bytes));
  return JPP_OK;
}

// dQ and the row statistics the dK/dV kernels read (attention_dq.hip)
int launch_dq(hipStream_t stream, const AttnParams& p, int head_dim, bool causal);
// dK/dV under a causal mask (attention_dkv.hip); grid (seq/128, kv heads, batch)
int launch_dkv_causal(hipStream_t stream, const AttnParams& p, int head_dim, dim3 grid);

}  // namespace jpp_attn

#endif  // JAXPP_AMD_ATTENTION_COMMON_H_
