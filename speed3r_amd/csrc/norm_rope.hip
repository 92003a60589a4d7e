// qk-LayerNorm + 2-D rotary embedding in one pass over a [B,H,N,D] tensor (D = 64), HBM bound.
//
// Replaces, for one of q / k, the chain LayerNorm(head_dim) -> cast -> RoPE2D of the reference layer
// (pi3/models/layers/sparse_attention.py:103-110,120-124; pi3/models/layers/pos_embed.py:112-159), which in eager
// PyTorch is about ten elementwise passes plus two embedding gathers.  Rounding points are the reference's: the
// normalised row is rounded to the I/O dtype, the cos/sin values come from the caller's tables (built with the
// reference's own formula, angles rounded to the I/O dtype before cos/sin), both products and their sum are rounded
// to the I/O dtype.
//
// One lane owns 16 bytes of a row (8 bf16 / 4 fp32 values), 8 (16) lanes own a row; the row statistics are
// xor-shuffle folds over those lanes.  Element e of a half (y: 0..31, x: 32..63) pairs with e +- 16, which lives two
// (four) lanes away: one shuffle per value.  Reads may be strided (the packed projection), writes are contiguous.
#include "s3r_common.h"

namespace s3r {

constexpr int kRows = 4;  // rows per thread

template <typename T>
__global__ __launch_bounds__(256) void norm_rope_kernel(
    const T* __restrict__ x, T* __restrict__ y, const int32_t* __restrict__ pos, const T* __restrict__ cos_tab,
    const T* __restrict__ sin_tab, int P, const T* __restrict__ ln_w, const T* __restrict__ ln_b, float eps,
    int H, int64_t N, uint32_t chunks, int64_t sxb, int64_t sxh, int64_t sxn, int64_t spb, int64_t spn) {
#pragma clang fp contract(off)
  constexpr int D = 64;
  constexpr int VEC = 16 / sizeof(T);
  constexpr int LPR = D / VEC;        // lanes per row
  constexpr int QL = (D / 4) / VEC;   // lanes per quarter of the head dimension
  // a workgroup takes kRows * 256 / LPR consecutive tokens of one (batch, head): the only divisions are by `chunks`
  // and H, on the workgroup's number
  const uint32_t bh = blockIdx.x / chunks;
  const uint32_t chunk = blockIdx.x - bh * chunks;
  const int64_t b = bh / (uint32_t)H;
  const int h = (int)(bh - (uint32_t)b * (uint32_t)H);
  const int lr = threadIdx.x % LPR;   // lane within the row
  constexpr int RPB = 256 / LPR;      // rows per workgroup-wide step
  const int half = lr / (2 * QL);     // 0: y half, 1: x half
  const int second = (lr / QL) & 1;   // which quarter of the half this lane holds
  const int f0 = (lr % QL) * VEC;     // frequency index of the lane's first value

  // kRows rows per thread, their loads (row and position) issued together: the pass lives on loads in flight
  uint4 raw[kRows];
  int pp[kRows];
  bool live[kRows];
  int64_t nn[kRows];
#pragma unroll
  for (int r = 0; r < kRows; r++) {
    const int64_t tok = ((int64_t)chunk * kRows + r) * RPB + threadIdx.x / LPR;
    live[r] = tok < N;
    nn[r] = live[r] ? tok : N - 1;  // idle lanes shadow the last row: the shuffles stay uniform
    const u32x4 t4 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x + b * sxb + h * sxh + nn[r] * sxn + lr * VEC));
    raw[r] = make_uint4(t4[0], t4[1], t4[2], t4[3]);
    pp[r] = pos != nullptr ? pos[b * spb + nn[r] * spn + half] : 0;
  }
  uint4 wr = make_uint4(0, 0, 0, 0), br = wr;
  if (ln_w != nullptr) {
    wr = *reinterpret_cast<const uint4*>(ln_w + lr * VEC);
    if (ln_b != nullptr) br = *reinterpret_cast<const uint4*>(ln_b + lr * VEC);
  }
  const T* we = reinterpret_cast<const T*>(&wr);
  const T* be = reinterpret_cast<const T*>(&br);
#pragma unroll
  for (int r = 0; r < kRows; r++) {
    const T* e = reinterpret_cast<const T*>(&raw[r]);
    float v[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++) v[i] = to_f32(e[i]);

    if (ln_w != nullptr) {  // LayerNorm over the 64 values of the row, fp32 statistics, result rounded to T
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < VEC; i++) s += v[i];
      s = group_sum<LPR>(s);
      const float mean = s * (1.0f / D);
      float q = 0.f;
#pragma unroll
      for (int i = 0; i < VEC; i++) q += (v[i] - mean) * (v[i] - mean);
      q = group_sum<LPR>(q);
      const float rstd = inv_sqrt(q * (1.0f / D) + eps);
#pragma unroll
      for (int i = 0; i < VEC; i++) v[i] = round_keep<T>((v[i] - mean) * rstd * to_f32(we[i]) + to_f32(be[i]));
    }

    if (pos != nullptr) {  // rotary embedding: the y half turns with pos[...,0], the x half with pos[...,1]
      int pq = pp[r];
      pq = pq < 0 ? 0 : (pq >= P ? P - 1 : pq);
      uint4 cr = *reinterpret_cast<const uint4*>(cos_tab + (int64_t)pq * (D / 4) + f0);
      uint4 sr = *reinterpret_cast<const uint4*>(sin_tab + (int64_t)pq * (D / 4) + f0);
      if constexpr (sizeof(T) == 2) {
        // "rotate half" is (-second quarter, first quarter): the minus sign of a first quarter's lanes is put on the
        // sine, on the packed words (rounding is symmetric: round(-a * s) = round(a * -s), the same bits)
        const uint32_t flip = second ? 0u : 0x80008000u;
        sr.x ^= flip; sr.y ^= flip; sr.z ^= flip; sr.w ^= flip;
      }
      const T* ce = reinterpret_cast<const T*>(&cr);
      const T* se = reinterpret_cast<const T*>(&sr);
#pragma unroll
      for (int i = 0; i < VEC; i++) {
        const float other = lane_xor<QL>(v[i]);                 // the paired value, one quarter away
        const float rot = sizeof(T) == 2 || second ? other : -other;  // (16-bit types: the sign is on the sine)
        const float a = round_keep<T>(v[i] * to_f32(ce[i]));
        const float c2 = round_keep<T>(rot * to_f32(se[i]));
        v[i] = a + c2;
      }
    }

    if (live[r]) {
      uint4 out;
      T* oe = reinterpret_cast<T*>(&out);
#pragma unroll
      for (int i = 0; i < VEC; i++) oe[i] = from_f32<T>(v[i]);
      store16_nt(y + (((int64_t)b * H + h) * N + nn[r]) * D + lr * VEC, out);
    }
  }
}

}  // namespace s3r

using namespace s3r;

extern "C" int s3r_norm_rope(const void* x, void* y, const int32_t* pos, const void* cos_tab, const void* sin_tab, int P,
                             const void* ln_w, const void* ln_b, float eps, int B, int H, int64_t N, int D,
                             int64_t sxb, int64_t sxh, int64_t sxn, int64_t spb, int64_t spn, int dtype, void* stream) {
  if (!x || !y) return fail(S3R_ERR_BAD_ARG, "s3r_norm_rope: null pointer");
  if (B <= 0 || H <= 0 || N <= 0) return fail(S3R_ERR_BAD_ARG, "s3r_norm_rope: non-positive size");
  if (dtype != S3R_F32 && dtype != S3R_BF16 && dtype != S3R_F16) return fail(S3R_ERR_UNSUPPORTED, "s3r_norm_rope: dtype %d", dtype);
  if (D != 64) return fail(S3R_ERR_UNSUPPORTED, "s3r_norm_rope: head_dim %d (built for 64)", D);
  if (pos != nullptr && (!cos_tab || !sin_tab || P <= 0)) return fail(S3R_ERR_BAD_ARG, "s3r_norm_rope: positions without tables");
  const int es = elt_size(dtype);
  if (!aligned16(x) || !aligned16(y) || (sxb * es) % 16 || (sxh * es) % 16 || (sxn * es) % 16 ||
      (cos_tab && !aligned16(cos_tab)) || (sin_tab && !aligned16(sin_tab)) || (ln_w && !aligned16(ln_w)) || (ln_b && !aligned16(ln_b)))
    return fail(S3R_ERR_BAD_ARG, "s3r_norm_rope: pointers and strides must be multiples of 16 bytes");
  const int lpr = 64 / (16 / es);
  const int64_t per_wg = (int64_t)kRows * (256 / lpr);  // tokens per workgroup
  const int64_t chunks = (N + per_wg - 1) / per_wg;          // workgroups per (batch, head)
  const int64_t blocks = chunks * B * H;
  if (blocks > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_norm_rope: tensor too large for one launch");
  const uint32_t nchunks = (uint32_t)chunks;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)blocks), blk(256);
  if (dtype == S3R_F32)
    hipLaunchKernelGGL(norm_rope_kernel<float>, grid, blk, 0, st, (const float*)x, (float*)y, pos, (const float*)cos_tab, (const float*)sin_tab, P, (const float*)ln_w, (const float*)ln_b, eps, H, N, nchunks, sxb, sxh, sxn, spb, spn);
  else if (dtype == S3R_BF16)
    hipLaunchKernelGGL(norm_rope_kernel<bf16_t>, grid, blk, 0, st, (const bf16_t*)x, (bf16_t*)y, pos, (const bf16_t*)cos_tab, (const bf16_t*)sin_tab, P, (const bf16_t*)ln_w, (const bf16_t*)ln_b, eps, H, N, nchunks, sxb, sxh, sxn, spb, spn);
  else
    hipLaunchKernelGGL(norm_rope_kernel<f16_t>, grid, blk, 0, st, (const f16_t*)x, (f16_t*)y, pos, (const f16_t*)cos_tab, (const f16_t*)sin_tab, P, (const f16_t*)ln_w, (const f16_t*)ln_b, eps, H, N, nchunks, sxb, sxh, sxn, spb, spn);
  return check_launch("s3r_norm_rope");
}
