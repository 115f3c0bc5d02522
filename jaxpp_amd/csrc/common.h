// Shared device/host helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/jaxpp_amd.h"

typedef uint16_t bf16_t;  // raw bfloat16 bits as stored in HBM
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// -- error plumbing ---------------------------------------------------------
// Every entry point returns 0 or a negative jpp_status and leaves a message
// that jpp_last_error() hands back (thread local).
int jpp_set_error(int code, const char* fmt, ...);

#define JPP_CHECK_HIP(expr)                                                     \
  do {                                                                          \
    hipError_t e_ = (expr);                                                     \
    if (e_ != hipSuccess)                                                       \
      return jpp_set_error(JPP_ERR_HIP, "%s failed: %s (%s:%d)", #expr,         \
                           hipGetErrorString(e_), __FILE__, __LINE__);          \
  } while (0)

#define JPP_REQUIRE(cond, ...)                                                  \
  do {                                                                          \
    if (!(cond)) return jpp_set_error(JPP_ERR_INVALID, __VA_ARGS__);            \
  } while (0)

#define JPP_LAUNCH_CHECK()                                                      \
  do {                                                                          \
    hipError_t e_ = hipGetLastError();                                          \
    if (e_ != hipSuccess)                                                       \
      return jpp_set_error(JPP_ERR_HIP, "kernel launch failed: %s (%s:%d)",     \
                           hipGetErrorString(e_), __FILE__, __LINE__);          \
  } while (0)

// -- launch probe -------------------------------------------------------------
// While a probe is active (jpp_probe_begin), every launch whose class name
// matches is bracketed by HIP events on its own stream; jpp_probe_end sums the
// durations and the algorithmic work the launcher declared.
bool jpp_probe_wants(const char* kernel_class);
void jpp_probe_open(hipStream_t stream, const char* kernel_class);
void jpp_probe_close(hipStream_t stream, double flops, double bytes);

struct ProbeScope {
  hipStream_t stream;
  double flops, bytes;
  bool on;
  ProbeScope(hipStream_t s, const char* cls, double fl, double by)
      : stream(s), flops(fl), bytes(by), on(jpp_probe_wants(cls)) {
    if (on) jpp_probe_open(stream, cls);
  }
  ~ProbeScope() {
    if (on) jpp_probe_close(stream, flops, bytes);
  }
};

// -- bf16 <-> f32 -------------------------------------------------------------
__device__ __forceinline__ float bf16_to_f32(bf16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}
__device__ __forceinline__ float bf16lo_to_f32(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t w) {
  return __uint_as_float(w & 0xffff0000u);
}
// round to nearest even
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  __bf16 b = (__bf16)f;
  return __builtin_bit_cast(bf16_t, b);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
}

// 8 bf16 of a 16-byte piece <-> 8 floats
__device__ __forceinline__ void unpack8(const uint4& v, float (&f)[8]) {
  f[0] = bf16lo_to_f32(v.x); f[1] = bf16hi_to_f32(v.x);
  f[2] = bf16lo_to_f32(v.y); f[3] = bf16hi_to_f32(v.y);
  f[4] = bf16lo_to_f32(v.z); f[5] = bf16hi_to_f32(v.z);
  f[6] = bf16lo_to_f32(v.w); f[7] = bf16hi_to_f32(v.w);
}
__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
  return make_uint4(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                    pack_bf16x2(f[6], f[7]));
}

// Rotary embedding of one pair: a and b are elements i and i + d/2 of a head, cs / sn the
// table entries of (position, i).  One definition for the pass of its own and for the GEMM
// epilogue that applies it, so that both round alike.
__device__ __forceinline__ void rope_rotate(float a, float b, float cs, float sn, float& o1,
                                            float& o2) {
  o1 = a * cs - b * sn;
  o2 = b * cs + a * sn;
}

// -- LDS operand slabs ----------------------------------------------------------
// A slab is [rows][64] bf16 (128 B per row, no padding).  The eight 16-byte
// chunks of a row are XOR-swizzled with the row index.  LDS serves 256 bytes a
// cycle from 64 banks, so two consecutive rows span the banks once: the swizzle
// steps once per two rows (16 rows x one chunk, the fragment of a 16x16x32 MFMA,
// then lie on 16 different (row parity, chunk) pairs), and rows two apart also
// differ in the upper half of the chunk index, which is what the transposing
// reads need (16 lanes on 4 rows x 64 bytes).  Found with a read-only loop of 8
// waves over XOR-linear maps of the row bits, in cycles per wave-level read:
// ds_read_b128 4.00 (the floor) for the 16-row and the 32-row fragments - the
// row-wise swizzle (row ^ row >> 3) & 7 used before took 6.00 for the former -
// and ds_read_b64_tr_b16 2.3 for the transposed fragments (the floor; 4.00 with
// any swizzle whose upper bit is the same for rows two apart).
__device__ __forceinline__ int slab_swz(int row) {
  const int h = (row >> 1) & 7;
  return h ^ ((h & 1) * 6);
}
__device__ __forceinline__ int slab_off(int row, int chunk) {
  return row * 128 + ((chunk ^ slab_swz(row)) << 4);
}

// MFMA operand fragment for v_mfma_f32_32x32x16_bf16: lane l supplies the row
// (l & 31) and the 8 contraction elements of chunk 2*kstep + (l >> 5).
__device__ __forceinline__ bf16x8 slab_frag(const uint8_t* slab, int row0, int kstep, int lane) {
  int row = row0 + (lane & 31);
  return *(const bf16x8*)(slab + slab_off(row, kstep * 2 + (lane >> 5)));
}

// ---------------------------------------------------------------------------
// Direct-to-LDS tiles (global_load_lds_dwordx4): no register staging.
// A wave-level load moves 64 x 16 bytes from per-lane global addresses into
// 1 KiB of LDS in lane order, so the LDS image of a tile is its memory image
// with the 16-byte chunks permuted inside each KiB.
//
//   MC = false  memory [ROWS][64..], contraction index contiguous.  LDS image
//               is the swizzled slab read by slab_frag().
//   MC = true   memory [64][ROWS..], contraction index is the slow one.  LDS
//               image keeps that orientation, chunk c of row k stored at
//               c ^ mc_swz(k); fragments come out through the LDS transpose
//               read (ds_read_b64_tr_b16), which hands lane i of a 16-lane
//               group the column i of a 4 x 16 block.
// ---------------------------------------------------------------------------
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
#define JPP_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define JPP_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

// One wave-level direct-to-LDS load: 64 lanes x 16 bytes from `base + off`
// (uniform 64-bit base, per-lane 32-bit byte offset) to LDS bytes
// [lds_addr, lds_addr + 1024) in lane order.  Issued through inline assembly
// so that the compiler does not serialise LDS reads of the *other* stage
// behind it; the caller waits for completion itself (dma_wait_all) before the
// data is read.
__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t*)p;
}
__device__ __forceinline__ const bf16_t* uniform_ptr(const bf16_t* p) {
  const uint64_t v = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const bf16_t*)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ void dma_load16(const bf16_t* base, uint32_t off, uint32_t lds_addr) {
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(off), "s"(base)
               : "memory");
}
__device__ __forceinline__ void dma_wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// waits until at most PENDING of this wave's most recent loads are outstanding
template <int PENDING>
__device__ __forceinline__ void dma_wait() {
  static_assert(PENDING >= 0 && PENDING < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PENDING) : "memory");
}
// waits for this wave's LDS reads, so that what they read may be overwritten
__device__ __forceinline__ void lds_wait_all() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// Chunk permutation of row k of an MC tile.  A transpose read has lanes 0-15 on rows
// k .. k+3 and lanes 16-31 on rows k+8 .. k+11 (8 rows are a multiple of the bank span
// apart): bits 0-1 of k move a chunk by 64 bytes, bit 3 by 32, so those 32 lanes touch
// every bank once.
__device__ __forceinline__ int mc_swz(int k) { return ((k & 3) << 2) ^ (((k >> 3) & 1) << 1); }

template <int ROWS, bool MC, int NW = 4>
struct DmaTile {
  static constexpr int BYTES = ROWS * 128;
  static constexpr int INSTS = ROWS / (8 * NW);  // wave-level loads per wave (NW waves share a tile)
  static_assert(INSTS >= 1, "tile too small for this many waves");
  typedef uint32_t Offsets[INSTS];

  // per-lane byte offsets (from the tile's first element) of this wave's loads;
  // loop invariant
  static __device__ __forceinline__ void offsets(Offsets& off, long ld, int wave, int lane) {
#pragma unroll
    for (int i = 0; i < INSTS; ++i) {
      const int inst = wave * INSTS + i;
      if constexpr (!MC) {
        const int row = inst * 8 + (lane >> 3);
        off[i] = (uint32_t)(((long)row * ld + (((lane & 7) ^ slab_swz(row)) << 3)) * 2);
      } else {
        constexpr int CPR = ROWS / 8, RPI = 64 / CPR;
        const int k = inst * RPI + lane / CPR;
        off[i] = (uint32_t)(((long)k * ld + (((lane % CPR) ^ mc_swz(k)) << 3)) * 2);
      }
    }
  }

  // loads FIRST .. FIRST+COUNT-1 of this wave's share; `tile` = LDS byte address
  template <int FIRST, int COUNT>
  static __device__ __forceinline__ void issue(const bf16_t* src, const Offsets& off,
                                               uint32_t tile, int wave) {
#pragma unroll
    for (int i = FIRST; i < FIRST + COUNT; ++i)
      dma_load16(src, off[i], tile + (wave * INSTS + i) * 1024);
  }

  // loads part*COUNT .. part*COUNT+COUNT-1 (`part` constant after unrolling)
  template <int COUNT>
  static __device__ __forceinline__ void issue_part(int part, const bf16_t* src, const Offsets& off,
                                                    uint32_t tile, int wave) {
#pragma unroll
    for (int i = 0; i < COUNT; ++i)
      dma_load16(src, off[part * COUNT + i], tile + (wave * INSTS + part * COUNT + i) * 1024);
  }

  // Operand fragment for v_mfma_f32_16x16x32_bf16: rows row0 .. row0+15 of the operand and
  // the contraction elements 32 k32 .. 32 k32 + 31 of the tile; lane l supplies row l & 15
  // and the 8 elements of chunk l >> 4.
  static __device__ __forceinline__ bf16x8 frag16(const uint8_t* tile, int row0, int k32, int lane) {
    const int g = lane >> 4, s = lane & 15;
    if constexpr (!MC) {
      return *(const bf16x8*)(tile + slab_off(row0 + s, k32 * 4 + g));
    } else {
      // two transpose reads of 4 contraction rows x 16 operand rows per 16-lane group
      const int n = row0 + ((s & 3) << 2);
      const int k = k32 * 32 + (g << 3) + (s >> 2);
      const uint8_t* p = tile + k * (ROWS * 2) + (((n >> 3) ^ mc_swz(k)) << 4) + ((n & 7) << 1);
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) s16x4*)JPP_LDS_PTR(p));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) s16x4*)JPP_LDS_PTR(p + 4 * ROWS * 2));
      const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(bf16x8, v);
    }
  }
};

// Fragment of a [rows][64 * nslab] tile held as KC slabs, taken the other way
// round: operand rows are the tile's columns col0 .. col0+31, the contraction
// index is the tile's row.  Step `st` covers tile rows 16 st .. 16 st + 15 in
// the order (4 hh + e, 8 + 4 hh + e), e = 0..3, hh = lane / 32: the order in
// which 8 consecutive accumulator registers of a 32x32 MFMA tile enumerate
// their row index, so such registers can be the other operand unchanged.
__device__ __forceinline__ bf16x8 slab_frag_tr(const uint8_t* slabs, int rows_per_slab, int col0,
                                               int st, int lane) {
  const int g = lane >> 4, s = lane & 15;
  const int n = col0 + ((g & 1) << 4) + ((s & 3) << 2);
  const int k = st * 16 + ((g >> 1) << 2) + (s >> 2);
  const uint8_t* slab = slabs + (n >> 6) * rows_per_slab * 128 + ((n & 7) << 1);
  const int c = (n & 63) >> 3;
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) s16x4*)JPP_LDS_PTR(slab + slab_off(k, c)));
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) s16x4*)JPP_LDS_PTR(slab + slab_off(k + 8, c)));
  const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, v);
}
