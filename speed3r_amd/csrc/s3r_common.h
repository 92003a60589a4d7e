// Shared host/device helpers for the gfx950 kernels of the sparse global-attention path.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/speed3r_hip.h"

namespace s3r {

// ---- error reporting (host) -------------------------------------------------------------------
char* last_error_buffer();  // thread-local, 512 bytes

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(S3R_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  return S3R_OK;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int elt_size(int dtype) { return dtype == S3R_F32 ? 4 : 2; }

// ---- element types ----------------------------------------------------------------------------
typedef __bf16 bf16_t;
typedef _Float16 f16_t;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename T> __device__ __forceinline__ float to_f32(T x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f32(float x) { return (T)x; }
// value of x after a round trip through the I/O type (the reference rounds probabilities to
// the value dtype before the PV product).  The empty asm keeps the compiler from folding the
// narrowing conversion away when it tracks the value in fp32.
template <typename T> __device__ __forceinline__ float round_to(float x) {
  T t = (T)x;
  unsigned short u = __builtin_bit_cast(unsigned short, t);
  asm volatile("" : "+v"(u));
  return (float)__builtin_bit_cast(T, u);
}
template <> __device__ __forceinline__ float round_to<float>(float x) { return x; }
// The same value for code that goes on in fp32: a bf16 number IS the upper half of its fp32 pattern, so the packed
// conversion with a zero in the lower half leaves the rounded value ready for use (one instruction per value instead
// of half a conversion and an unpacking shift or mask).
template <typename T> __device__ __forceinline__ float round_keep(float x) { return round_to<T>(x); }
template <> __device__ __forceinline__ float round_keep<bf16_t>(float x) {
  float r;
  asm("v_cvt_pk_bf16_f32 %0, 0, %1" : "=v"(r) : "v"(x));
  return r;
}

// 16-byte non-temporal store, for the memory-bound passes whose waves write whole 128-byte lines of a tensor larger
// than the last-level cache (the rotated q and k of 266 496 tokens: one-pass kernel 0.50 against 0.55 ms).  Not for
// the attention kernels' epilogues: their store instructions cover lines piecewise, and past the L2 that costs the
// selection kernel 8 %.
__device__ __forceinline__ void store16_nt(void* dst, const uint4& v) {
  __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(&v), reinterpret_cast<u32x4*>(dst));
}

// 1 / sqrt(x) for a normal positive x by the hardware's reciprocal square root (1 ulp): one instruction where
// sqrtf and the division, both correctly rounded, take about forty.
__device__ __forceinline__ float inv_sqrt(float x) { return __builtin_amdgcn_rsqf(x); }

// fp32 bit pattern -> order-preserving u32: negative values flip all bits, others the sign bit.
__device__ __forceinline__ uint32_t sortable_key(float s) {
  uint32_t b = __float_as_uint(s);
  return b ^ ((uint32_t)((int32_t)b >> 31) | 0x80000000u);
}

constexpr int kWave = 64;

// LDS layout of a tile whose rows are 128 bytes: the 16-byte chunk c of row r sits at chunk position c ^ k_swizzle(r).
// The LDS of this chip has 64 banks (256 bytes per clock, two rows of a tile; a row's parity picks the bank half).
// * ds_read_b128 with lane = row (MFMA operands from rows) is served sixteen lanes at a time: rows r and r + 8 share
//   their banks, so the map has to send row bits 1..3 to three different chunk bits.  Measured on one CU with eight
//   waves: 4.3 cycles per instruction, 8.0 with the map r & 7, 32 without a map; a single wave does not show it.
// * ds_read_b64_tr_b16 (operands from columns) touches, per pass, four rows r..r+3 and four chunks that differ in chunk
//   bits 0..1: rows r and r + 2 have the same parity, so row bit 1 has to go to chunk bit 2.  (These conflicts cost
//   bank cycles but no time in a loop that issues nothing else to the LDS: the instruction's own rate hides them.)
// Both: row bit 1 -> chunk bit 2, row bit 2 -> chunk bit 0, row bit 3 -> chunk bit 1.  The map is linear over GF(2) in
// the row bits, and row bit 4 and above do not enter: k_swizzle(r + 8) = k_swizzle(r) ^ k_swizzle(8) for r < 8.
__device__ __forceinline__ constexpr int k_swizzle(int row) { return (((row >> 1) & 1) << 2) | ((row >> 2) & 3); }

// Value held by lane ^ MASK.  Masks 1 and 2 stay inside a quad and ride on the DPP operand path of an ordinary move
// (no LDS crossbar); masks up to 16 use the swizzle unit without an address register; larger ones the general permute.
template <int MASK> __device__ __forceinline__ float lane_xor(float x) {
  static_assert(MASK > 0 && MASK < 64 && (MASK & (MASK - 1)) == 0, "one bit of the lane number");
  const int v = __float_as_int(x);
  if constexpr (MASK == 1) return __int_as_float(__builtin_amdgcn_update_dpp(v, v, 0xB1, 0xF, 0xF, false));       // quad_perm [1,0,3,2]
  else if constexpr (MASK == 2) return __int_as_float(__builtin_amdgcn_update_dpp(v, v, 0x4E, 0xF, 0xF, false));  // quad_perm [2,3,0,1]
  else if constexpr (MASK < 32) return __int_as_float(__builtin_amdgcn_ds_swizzle(v, (MASK << 10) | 0x1F));       // bit mode: and 0x1f, xor MASK
  else return __shfl_xor(x, MASK);
}
// sum over the aligned group of N lanes (a power of two) the lane belongs to
template <int N> __device__ __forceinline__ float group_sum(float s) {
  if constexpr (N >= 2) s += lane_xor<1>(s);
  if constexpr (N >= 4) s += lane_xor<2>(s);
  if constexpr (N >= 8) s += lane_xor<4>(s);
  if constexpr (N >= 16) s += lane_xor<8>(s);
  if constexpr (N >= 32) s += lane_xor<16>(s);
  if constexpr (N >= 64) s += lane_xor<32>(s);
  return s;
}

}  // namespace s3r
