// Pieces shared by the selection-attention kernels: MFMA wrappers per I/O dtype, 16-byte fragments,
// exchanges with lane ^ 32, compile-time loops.
#pragma once
#include "s3r_common.h"
#include <type_traits>
#include <utility>

namespace s3r {
namespace sel {

template <typename E> struct Mma;
template <> struct Mma<bf16_t> {
  typedef bf16x8 V8;
  typedef __bf16 V2 __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ float dot_ones(V2 a, float acc) {
    V2 one;
    one[0] = (__bf16)1.0f;
    one[1] = (__bf16)1.0f;
    return __builtin_amdgcn_fdot2_f32_bf16(a, one, acc, false);
  }
};
template <> struct Mma<f16_t> {
  typedef f16x8 V8;
  typedef _Float16 V2 __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ float dot_ones(V2 a, float acc) {
    V2 one;
    one[0] = (_Float16)1.0f;
    one[1] = (_Float16)1.0f;
    return __builtin_amdgcn_fdot2(a, one, acc, false);
  }
};

union Frag {
  uint4 u;
  bf16x8 b;
  f16x8 h;
  s16x4 s[2];
};
template <typename E> __device__ __forceinline__ typename Mma<E>::V8 as_v8(const Frag& f);
template <> __device__ __forceinline__ bf16x8 as_v8<bf16_t>(const Frag& f) { return f.b; }
template <> __device__ __forceinline__ f16x8 as_v8<f16_t>(const Frag& f) { return f.h; }

__device__ __forceinline__ float xh_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xh_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <typename F, int... I> __device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F> __device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

}  // namespace sel
}  // namespace s3r
