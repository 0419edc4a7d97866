// Shared device helpers for the gfx950 kernels: 16-bit element traits, MFMA
// wrappers, wave64 shuffles, error plumbing for the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/fsa_hip.h"

namespace fsa {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

constexpr int WAVE = 64;
constexpr float LOG2E = 1.4426950408889634f;

// ---- element traits -------------------------------------------------------
template <typename T> struct Elem;

template <> struct Elem<__bf16> {
  typedef bf16x8 vec8;
  typedef bf16x4 vec4;
  static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

template <> struct Elem<_Float16> {
  typedef f16x8 vec8;
  typedef f16x4 vec4;
  static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

// 16-byte / 8-byte raw moves (global or LDS) reinterpreted as element vectors.
template <typename V> __device__ __forceinline__ V load16(const void* p) {
  uint4 r = *reinterpret_cast<const uint4*>(p);
  return __builtin_bit_cast(V, r);
}
template <typename V> __device__ __forceinline__ void store16(void* p, V v) {
  *reinterpret_cast<uint4*>(p) = __builtin_bit_cast(uint4, v);
}
// The same 16-byte moves for data that is written once and read once by a later kernel (partial rows):
// marked non-temporal so that they do not displace the K / V blocks and query rows that are reused.
template <typename V> __device__ __forceinline__ V load16_stream(const void* p) {
  typedef unsigned int u4_ __attribute__((ext_vector_type(4)));
  u4_ r = __builtin_nontemporal_load(reinterpret_cast<const u4_*>(p));
  return __builtin_bit_cast(V, r);
}
template <typename V> __device__ __forceinline__ void store16_stream(void* p, V v) {
  typedef unsigned int u4_ __attribute__((ext_vector_type(4)));
  __builtin_nontemporal_store(__builtin_bit_cast(u4_, v), reinterpret_cast<u4_*>(p));
}
template <typename V> __device__ __forceinline__ V load8(const void* p) {
  uint2 r = *reinterpret_cast<const uint2*>(p);
  return __builtin_bit_cast(V, r);
}
template <typename V> __device__ __forceinline__ void store8(void* p, V v) {
  *reinterpret_cast<uint2*>(p) = __builtin_bit_cast(uint2, v);
}

// elements p[0..3] and p[16..19] as one 8-element fragment (two 8-byte moves)
template <typename T> __device__ __forceinline__ typename Elem<T>::vec8 load8x2(const T* p) {
  typename Elem<T>::vec4 lo = load8<typename Elem<T>::vec4>(p);
  typename Elem<T>::vec4 hi = load8<typename Elem<T>::vec4>(p + 16);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}
// ---- hand-issued 8-byte LDS reads --------------------------------------------------------------
// An LDS instruction that returns 16 bytes per lane (ds_read_b128, ds_read2_b64) delivers 64 bytes per clock
// on gfx950, an 8-byte one (ds_read_b64) 128.  The compiler fuses neighbouring 8-byte reads into the 16-byte
// forms, so the reads that should stay separate are issued by hand.  The compiler does not know that their
// results are still in flight: lds_wait() has to be placed between such reads and the first use of their
// results, with every result passed through it.
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t lds_addr(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}
// the LDS pointer for a byte address
template <typename T> __device__ __forceinline__ const T* lds_ptr(uint32_t addr) {
  return (const T*)(__attribute__((address_space(3))) const T*)(uintptr_t)addr;
}
template <int OFFSET_BYTES> __device__ __forceinline__ u32x2 lds_read8_raw(uint32_t addr) {
  static_assert(OFFSET_BYTES >= 0 && OFFSET_BYTES < 65536, "ds offset field");
  u32x2 r;
  asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFFSET_BYTES));
  return r;
}
template <int N> __device__ __forceinline__ void lds_wait(u32x2 (&r)[N]);
template <> __device__ __forceinline__ void lds_wait<6>(u32x2 (&r)[6]) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]));
}
template <> __device__ __forceinline__ void lds_wait<8>(u32x2 (&r)[8]) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
}
template <> __device__ __forceinline__ void lds_wait<16>(u32x2 (&r)[16]) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]),
                 "+v"(r[8]), "+v"(r[9]), "+v"(r[10]), "+v"(r[11]), "+v"(r[12]), "+v"(r[13]), "+v"(r[14]),
                 "+v"(r[15]));
}
template <typename T> __device__ __forceinline__ typename Elem<T>::vec8 frag8(u32x2 lo, u32x2 hi) {
  u32x4 x = {lo[0], lo[1], hi[0], hi[1]};
  return __builtin_bit_cast(typename Elem<T>::vec8, x);
}

template <typename T> __device__ __forceinline__ typename Elem<T>::vec8 zero8() {
  uint4 z = make_uint4(0, 0, 0, 0);
  return __builtin_bit_cast(typename Elem<T>::vec8, z);
}

// LDS transposing read (gfx950 ds_read_b64_tr_b16).  Inside every group of 16
// lanes, lane j receives, for e = 0..3, element (j % 4) of the 8-byte word whose
// address was supplied by lane 4*e + j/4 of the group.  With lane s pointing at
// M[r0 + (s%16)/4][c0 + 4*(s%4) ..], lane j therefore gets M[r0 + e][c0 + j],
// e = 0..3: four consecutive rows of one column out of a row-major tile.
template <typename T> __device__ __forceinline__ typename Elem<T>::vec4 lds_read_tr4(const T* p) {
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) s16x4* lds_ptr;
  s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
  return __builtin_bit_cast(typename Elem<T>::vec4, r);
}

// Eight values of one column (two runs of four consecutive rows, 8 rows apart)
// of a row-major LDS tile, as the k-contiguous MFMA operand of a contraction
// over the tile's rows.  `p` is this lane's address for row r0 + (lane%16)/4.
template <typename T>
__device__ __forceinline__ typename Elem<T>::vec8 lds_read_tr8(const T* p, int stride8rows) {
  typename Elem<T>::vec4 lo = lds_read_tr4<T>(p);
  typename Elem<T>::vec4 hi = lds_read_tr4<T>(p + stride8rows);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// 2^x by the hardware instruction alone (1 ulp; results below 2^-126 flush to zero, -inf gives 0): the
// library exp2f adds a denormal-range rescaling that costs several VALU operations per element
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32, 64); }

// Maximum of an unsigned value over the wave, returned to every lane, without going through the LDS crossbar:
// prefix maxima inside each row of 16 lanes with the DPP row shifts (lanes shifted in from outside a row read 0),
// the rows combined with the two DPP row broadcasts, the result read from the last lane.
template <int CTRL, int ROW_MASK, bool ZERO_FILL> __device__ __forceinline__ uint32_t dpp_move(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, ROW_MASK, 0xf, ZERO_FILL);
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t x) {
  x = max(x, dpp_move<0x111, 0xf, true>(x));   // row_shr:1
  x = max(x, dpp_move<0x112, 0xf, true>(x));   // row_shr:2
  x = max(x, dpp_move<0x114, 0xf, true>(x));   // row_shr:4
  x = max(x, dpp_move<0x118, 0xf, true>(x));   // row_shr:8 -> lane 15 of a row holds the maximum of the row
  x = max(x, dpp_move<0x142, 0xa, false>(x));  // row_bcast:15 into rows 1 and 3
  x = max(x, dpp_move<0x143, 0xc, false>(x));  // row_bcast:31 into rows 2 and 3
  return (uint32_t)__builtin_amdgcn_readlane((int)x, 63);
}
// the same for 64-bit keys (hi word compared first)
template <int CTRL, int ROW_MASK, bool ZERO_FILL> __device__ __forceinline__ uint64_t dpp_max_u64(uint64_t x) {
  const uint64_t y = ((uint64_t)dpp_move<CTRL, ROW_MASK, ZERO_FILL>((uint32_t)(x >> 32)) << 32) |
                     dpp_move<CTRL, ROW_MASK, ZERO_FILL>((uint32_t)x);
  return y > x ? y : x;
}
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t x) {
  x = dpp_max_u64<0x111, 0xf, true>(x);
  x = dpp_max_u64<0x112, 0xf, true>(x);
  x = dpp_max_u64<0x114, 0xf, true>(x);
  x = dpp_max_u64<0x118, 0xf, true>(x);
  x = dpp_max_u64<0x142, 0xa, false>(x);
  x = dpp_max_u64<0x143, 0xc, false>(x);
  return ((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)(x >> 32), 63) << 32) |
         (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)x, 63);
}

// r / g for a row index r >= 0 and a GQA group of g heads: a shift where g is a power of two (g_shift =
// log2 g), the division otherwise (g_shift < 0).  The general division costs some forty instructions and sits in
// the address computation of every gathered row.
__device__ __forceinline__ int div_group(int r, int g, int g_shift) { return g_shift >= 0 ? (r >> g_shift) : r / g; }
static inline int group_shift(int g) {
  if (g <= 0 || (g & (g - 1)) != 0) return -1;
  int s = 0;
  while ((1 << s) < g) ++s;
  return s;
}

// largest i in [0, n) with a[i] <= x, for ascending a[0..n) with a[0] <= x
__device__ __forceinline__ int upper_seg(const int32_t* __restrict__ a, int n, int x) {
  int lo = 0, hi = n;  // invariant a[lo] <= x, a[hi] > x (virtual)
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (a[mid] <= x) lo = mid; else hi = mid;
  }
  return lo;
}

// ---- host-side error plumbing --------------------------------------------
void set_error(const char* fmt, ...);

#define FSA_CHECK_ARG(cond, ...)            \
  do {                                      \
    if (!(cond)) {                          \
      fsa::set_error(__VA_ARGS__);          \
      return FSA_ERR_INVALID;               \
    }                                       \
  } while (0)

#define FSA_CHECK_LAUNCH(what)                                               \
  do {                                                                       \
    hipError_t e__ = hipGetLastError();                                      \
    if (e__ != hipSuccess) {                                                 \
      fsa::set_error("%s: %s", what, hipGetErrorString(e__));                \
      return (int)e__;                                                       \
    }                                                                        \
  } while (0)

// Optional per-kernel timing: while fsa_profile_enable(1) is in effect every
// launch wrapped in a ProfScope is bracketed by HIP events on its stream.
struct ProfScope {
  ProfScope(const char* name, hipStream_t stream);
  ~ProfScope();
  int idx_;
  hipStream_t stream_;
};

static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// fsa_build_tiles with an optional tile -> block table [num_kv_heads, max_tiles] (max_tiles >= fsa_max_tiles(...))
int build_tiles(const int32_t* counts, int num_kv_heads, int64_t max_blocks, int group_size, int rows_per_tile,
                int32_t* tile_prefix, int32_t* tile_block, int64_t max_tiles, hipStream_t stream);

}  // namespace fsa
