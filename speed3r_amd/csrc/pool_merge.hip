// Block mean-pooling and the gated merge: the two pure HBM-streaming kernels of the path.
//
// Both move 16 bytes per lane per access.  Pooling gives one wavefront to one
// (batch, head, block): the wave's 64 lanes cover 64/LPR token rows per load (LPR = lanes per
// head_dim row), accumulate in fp32 and fold the row groups with xor-shuffles.  The merge
// maps consecutive lanes to consecutive 16-byte chunks of the [B,N,H*D] output so stores
// are fully coalesced, and reads the per-head planes in 128-byte row segments.
#include "s3r_common.h"

namespace s3r {

template <typename T, int U>
__global__ __launch_bounds__(256) void pool_mean_kernel(
    const T* __restrict__ x, T* __restrict__ y, int H, int64_t N, int D, int block, int64_t Nc,
    int64_t total, int64_t sxb, int64_t sxh, int64_t sxn, int64_t syb, int64_t syh, int64_t syn) {
  constexpr int VEC = 16 / sizeof(T);
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= total) return;
  const int64_t j = w % Nc;
  const int64_t bh = w / Nc;
  const int h = (int)(bh % H);
  const int64_t b = bh / H;
  const int lpr = D / VEC;   // lanes per row, a power of two <= 64
  const int rpw = 64 / lpr;  // rows per wave-wide load
  const int r0 = lane / lpr;
  const int dc = lane - r0 * lpr;
  const int64_t t0 = j * block;
  const int nvalid = (int)((N - t0 < block) ? (N - t0) : block);
  const T* base = x + b * sxb + h * sxh + t0 * sxn + dc * VEC;

  float acc[VEC];
#pragma unroll
  for (int i = 0; i < VEC; i++) acc[i] = 0.f;
  // batches of U loads issued back to back (rows beyond the block re-read its last row and are not added),
  // so that up to 8 KB per wave are in flight instead of one load at a time; U = 8 or, for blocks below 8 wave-wide
  // loads, the number that covers the block
  for (int r = r0; r < nvalid; r += U * rpw) {
    uint4 raw[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int rr = r + u * rpw;
      {  // streamed once: a non-temporal load keeps the rows from displacing anything in the caches (5.8 -> 6.6 TB/s)
        const u32x4 t4 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(base + (int64_t)(rr < nvalid ? rr : nvalid - 1) * sxn));
        raw[u] = make_uint4(t4[0], t4[1], t4[2], t4[3]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const T* e = reinterpret_cast<const T*>(&raw[u]);
      const bool keep = r + u * rpw < nvalid;
#pragma unroll
      for (int i = 0; i < VEC; i++) acc[i] += keep ? to_f32(e[i]) : 0.f;
    }
  }
  for (int off = lpr; off < 64; off <<= 1) {
#pragma unroll
    for (int i = 0; i < VEC; i++) acc[i] += __shfl_xor(acc[i], off);
  }
  if (r0 == 0) {
    uint4 raw;
    T* e = reinterpret_cast<T*>(&raw);
    const float cnt = (float)nvalid;
#pragma unroll
    for (int i = 0; i < VEC; i++) e[i] = from_f32<T>(acc[i] / cnt);
    *reinterpret_cast<uint4*>(y + b * syb + h * syh + j * syn + dc * VEC) = raw;
  }
}

// Small blocks (one or two wave-wide loads cover a block): a wave takes G consecutive blocks of a head, G * U = 8
// loads in flight as for the large blocks (with one block per wave only 2 KB per wave are in flight and the kernel
// runs at 5.0 instead of 6.6 TB/s at 16-token blocks).
template <typename T, int U, int G>
__global__ __launch_bounds__(256) void pool_mean_group_kernel(
    const T* __restrict__ x, T* __restrict__ y, int H, int64_t N, int D, int block, int64_t Nc, int64_t ngrp,
    int64_t total, int64_t sxb, int64_t sxh, int64_t sxn, int64_t syb, int64_t syh, int64_t syn) {
  constexpr int VEC = 16 / sizeof(T);
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= total) return;
  const int64_t jg = w % ngrp;
  const int64_t bh = w / ngrp;
  const int h = (int)(bh % H);
  const int64_t b = bh / H;
  const int lpr = D / VEC;
  const int rpw = 64 / lpr;
  const int r0 = lane / lpr;
  const int dc = lane - r0 * lpr;
  const T* base = x + b * sxb + h * sxh + dc * VEC;
  uint4 raw[G][U];
  int nval[G];
#pragma unroll
  for (int g = 0; g < G; g++) {
    const int64_t j = jg * G + g;
    const int64_t t0 = (j < Nc ? j : Nc - 1) * block;  // a block beyond the end re-reads the last one and stores nothing
    nval[g] = j < Nc ? (int)((N - t0 < block) ? (N - t0) : block) : 0;
    const int nclamp = (int)((N - t0 < block) ? (N - t0) : block);
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int rr = r0 + u * rpw;
      const u32x4 t4 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(base + (t0 + (rr < nclamp ? rr : nclamp - 1)) * sxn));
      raw[g][u] = make_uint4(t4[0], t4[1], t4[2], t4[3]);
    }
  }
#pragma unroll
  for (int g = 0; g < G; g++) {
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++) acc[i] = 0.f;
#pragma unroll
    for (int u = 0; u < U; u++) {
      const T* e = reinterpret_cast<const T*>(&raw[g][u]);
      const bool keep = r0 + u * rpw < nval[g];
#pragma unroll
      for (int i = 0; i < VEC; i++) acc[i] += keep ? to_f32(e[i]) : 0.f;
    }
    for (int off = lpr; off < 64; off <<= 1) {
#pragma unroll
      for (int i = 0; i < VEC; i++) acc[i] += __shfl_xor(acc[i], off);
    }
    if (r0 == 0 && nval[g] > 0) {
      uint4 out;
      T* e = reinterpret_cast<T*>(&out);
      const float cnt = (float)nval[g];
#pragma unroll
      for (int i = 0; i < VEC; i++) e[i] = from_f32<T>(acc[i] / cnt);
      *reinterpret_cast<uint4*>(y + b * syb + h * syh + (jg * G + g) * syn + dc * VEC) = out;
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gated_merge_kernel(
    const T* __restrict__ oc, const T* __restrict__ os, const T* __restrict__ gate, T* __restrict__ out,
    int H, int64_t N, int D, int block, uint32_t per_batch,
    int64_t scb, int64_t sch, int64_t scm, int64_t ssb, int64_t ssh, int64_t ssn,
    int64_t sgb, int64_t sgh, int64_t sgn) {
#pragma clang fp contract(off)  // products and sum stay separately rounded operations
  constexpr int VEC = 16 / sizeof(T);
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;  // chunk index within the batch entry
  if (i >= per_batch) return;
  const int64_t b = blockIdx.y;
  const uint32_t lpr = (uint32_t)D / VEC;
  const uint32_t dc = i % lpr;
  const uint32_t t = i / lpr;
  const uint32_t h = t % (uint32_t)H;
  const uint32_t n = t / (uint32_t)H;
  const T* g = gate + b * sgb + h * sgh + (int64_t)n * sgn;
  const float g0 = to_f32(g[0]);
  const float g1 = to_f32(g[1]);
  uint4 rs = *reinterpret_cast<const uint4*>(os + b * ssb + h * ssh + (int64_t)n * ssn + dc * VEC);
  uint4 rc = *reinterpret_cast<const uint4*>(oc + b * scb + h * sch + (int64_t)(n / (uint32_t)block) * scm + dc * VEC);
  const T* es = reinterpret_cast<const T*>(&rs);
  const T* ec = reinterpret_cast<const T*>(&rc);
  uint4 ro;
  T* eo = reinterpret_cast<T*>(&ro);
#pragma unroll
  for (int e = 0; e < VEC; e++) {
    // same rounding points as the eager expression: each product, then the sum
    const float a = round_to<T>(g0 * to_f32(ec[e]));
    const float c = round_to<T>(g1 * to_f32(es[e]));
    eo[e] = from_f32<T>(a + c);
  }
  store16_nt(out + ((int64_t)b * per_batch + i) * VEC, ro);
}

}  // namespace s3r

using namespace s3r;

extern "C" int s3r_pool_mean(const void* x, void* y, int B, int H, int64_t N, int D, int block,
                             int64_t sxb, int64_t sxh, int64_t sxn, int64_t syb, int64_t syh, int64_t syn,
                             int dtype, void* stream) {
  if (!x || !y) return fail(S3R_ERR_BAD_ARG, "s3r_pool_mean: null pointer");
  if (B <= 0 || H <= 0 || N <= 0 || D <= 0 || block <= 0) return fail(S3R_ERR_BAD_ARG, "s3r_pool_mean: non-positive size");
  if (dtype != S3R_F32 && dtype != S3R_BF16 && dtype != S3R_F16) return fail(S3R_ERR_UNSUPPORTED, "s3r_pool_mean: dtype %d", dtype);
  const int es = elt_size(dtype);
  const int vec = 16 / es;
  const int lpr = D / vec;
  if (D % vec != 0 || lpr > 64 || (lpr & (lpr - 1)) != 0)
    return fail(S3R_ERR_UNSUPPORTED, "s3r_pool_mean: head_dim %d (row bytes must be a power-of-two multiple of 16, <= 1024)", D);
  if (!aligned16(x) || !aligned16(y) || (sxb * es) % 16 || (sxh * es) % 16 || (sxn * es) % 16 || (syb * es) % 16 ||
      (syh * es) % 16 || (syn * es) % 16)
    return fail(S3R_ERR_BAD_ARG, "s3r_pool_mean: pointers and strides must be 16-byte aligned");
  const int64_t Nc = (N + block - 1) / block;
  const int64_t total = (int64_t)B * H * Nc;
  const int64_t nwg = (total + 3) / 4;
  if (nwg > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_pool_mean: too many blocks");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)nwg), blk(256);
  const int loads = (block * lpr + 63) / 64;  // wave-wide loads that cover one block
#define S3R_POOL(T, U) hipLaunchKernelGGL((pool_mean_kernel<T, U>), grid, blk, 0, st, (const T*)x, (T*)y, H, N, D, block, Nc, total, sxb, sxh, sxn, syb, syh, syn)
#define S3R_POOL_G(T, U, G)                                                                                                  \
  do {                                                                                                                       \
    const int64_t ngrp = (Nc + G - 1) / G, tot = (int64_t)B * H * ngrp;                                                      \
    hipLaunchKernelGGL((pool_mean_group_kernel<T, U, G>), dim3((unsigned)((tot + 3) / 4)), blk, 0, st, (const T*)x, (T*)y, H, N, D, \
                       block, Nc, ngrp, tot, sxb, sxh, sxn, syb, syh, syn);                                                  \
  } while (0)
#define S3R_POOL_T(T)                                       \
  do {                                                      \
    if (loads <= 1 && block * lpr == 64) S3R_POOL_G(T, 1, 8);      \
    else if (loads <= 1) S3R_POOL(T, 1);                    \
    else if (loads == 2 && block * lpr == 128) S3R_POOL_G(T, 2, 4); \
    else if (loads <= 2) S3R_POOL(T, 2);                    \
    else if (loads <= 4) S3R_POOL(T, 4);                    \
    else S3R_POOL(T, 8);                                    \
  } while (0)
  if (dtype == S3R_F32) S3R_POOL_T(float);
  else if (dtype == S3R_BF16) S3R_POOL_T(bf16_t);
  else S3R_POOL_T(f16_t);
#undef S3R_POOL_T
#undef S3R_POOL_G
#undef S3R_POOL
  return check_launch("s3r_pool_mean");
}

extern "C" int s3r_gated_merge(const void* o_cmp, const void* o_sel, const void* gate, void* out,
                               int B, int H, int64_t N, int D, int block,
                               int64_t scb, int64_t sch, int64_t scm, int64_t ssb, int64_t ssh, int64_t ssn,
                               int64_t sgb, int64_t sgh, int64_t sgn, int dtype, void* stream) {
  if (!o_cmp || !o_sel || !gate || !out) return fail(S3R_ERR_BAD_ARG, "s3r_gated_merge: null pointer");
  if (B <= 0 || H <= 0 || N <= 0 || D <= 0 || block <= 0) return fail(S3R_ERR_BAD_ARG, "s3r_gated_merge: non-positive size");
  if (dtype != S3R_F32 && dtype != S3R_BF16 && dtype != S3R_F16) return fail(S3R_ERR_UNSUPPORTED, "s3r_gated_merge: dtype %d", dtype);
  const int es = elt_size(dtype);
  const int vec = 16 / es;
  if (D % vec != 0) return fail(S3R_ERR_UNSUPPORTED, "s3r_gated_merge: head_dim %d not a multiple of %d", D, vec);
  if (!aligned16(o_cmp) || !aligned16(o_sel) || !aligned16(out) || (scb * es) % 16 || (sch * es) % 16 || (scm * es) % 16 ||
      (ssb * es) % 16 || (ssh * es) % 16 || (ssn * es) % 16)
    return fail(S3R_ERR_BAD_ARG, "s3r_gated_merge: o_cmp/o_sel/out pointers and strides must be 16-byte aligned");
  const int64_t per_batch = N * H * (D / vec);
  if (per_batch > 0xffffff00LL || B > 65535) return fail(S3R_ERR_UNSUPPORTED, "s3r_gated_merge: tensor too large for one launch");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)((per_batch + 255) / 256), (unsigned)B), blk(256);
  if (dtype == S3R_F32)
    hipLaunchKernelGGL(gated_merge_kernel<float>, grid, blk, 0, st, (const float*)o_cmp, (const float*)o_sel, (const float*)gate, (float*)out, H, N, D, block, (uint32_t)per_batch, scb, sch, scm, ssb, ssh, ssn, sgb, sgh, sgn);
  else if (dtype == S3R_BF16)
    hipLaunchKernelGGL(gated_merge_kernel<bf16_t>, grid, blk, 0, st, (const bf16_t*)o_cmp, (const bf16_t*)o_sel, (const bf16_t*)gate, (bf16_t*)out, H, N, D, block, (uint32_t)per_batch, scb, sch, scm, ssb, ssh, ssn, sgb, sgh, sgn);
  else
    hipLaunchKernelGGL(gated_merge_kernel<f16_t>, grid, blk, 0, st, (const f16_t*)o_cmp, (const f16_t*)o_sel, (const f16_t*)gate, (f16_t*)out, H, N, D, block, (uint32_t)per_batch, scb, sch, scm, ssb, ssh, ssn, sgb, sgh, sgn);
  return check_launch("s3r_gated_merge");
}
