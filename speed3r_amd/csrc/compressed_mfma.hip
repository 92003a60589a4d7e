// Compressed-branch attention on the gfx950 matrix cores (bf16 / fp16 I/O, head_dim 64):
// dense non-causal flash attention over the pooled tokens, with the raw score tile
// optionally written out for the block selection.
//
// A 256-thread workgroup owns 128 query rows of one head, 32 per wavefront, and walks all
// key tiles of 64 pooled tokens.  K and V tiles are staged once per workgroup in LDS
// (global -> registers one tile ahead -> LDS) and shared by the four waves.  Per wave and
// tile: S^T = K Q^T with v_mfma_f32_32x32x16 (one query per lane, see select_mfma.hip for
// the layout argument), base-2 online softmax in fp32, P rounded to the I/O dtype,
// O^T += V^T P^T with V^T fragments read through ds_read_b64_tr_b16.
#include "s3r_common.h"
#include "attn_params.h"

namespace s3r {

template <typename E> struct MfmaC;
template <> struct MfmaC<bf16_t> {
  typedef bf16x8 V8;
  static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <> struct MfmaC<f16_t> {
  typedef f16x8 V8;
  static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};

union FragC {
  uint4 u;
  bf16x8 b;
  f16x8 h;
  s16x4 s[2];
};
template <typename E> __device__ __forceinline__ typename MfmaC<E>::V8 fragc_as(const FragC& f);
template <> __device__ __forceinline__ bf16x8 fragc_as<bf16_t>(const FragC& f) { return f.b; }
template <> __device__ __forceinline__ f16x8 fragc_as<f16_t>(const FragC& f) { return f.h; }

__device__ __forceinline__ float xh_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xh_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

constexpr int kCLd = 72;  // LDS row stride in elements (144 bytes)

template <typename E>
__global__ __launch_bounds__(256) void compressed_mfma_kernel(AttnParams p) {
  typedef typename MfmaC<E>::V8 V8;
  __shared__ __attribute__((aligned(16))) E Ks[64 * kCLd];
  __shared__ __attribute__((aligned(16))) E Vs[64 * kCLd];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int hh = lane >> 5;
  const int c = lane & 31;
  const int b = blockIdx.y / p.H;
  const int h = blockIdx.y - b * p.H;
  const int64_t Lq = p.Lq, Lk = p.Lk;
  const int64_t q0 = (int64_t)blockIdx.x * 128 + wave * 32;

  const E* qp = (const E*)p.q + (int64_t)b * p.sqb + (int64_t)h * p.sqh;
  const E* kp = (const E*)p.k + (int64_t)b * p.skb + (int64_t)h * p.skh;
  const E* vp = (const E*)p.v + (int64_t)b * p.svb + (int64_t)h * p.svh;

  const int64_t qrow = q0 + c;
  const bool qvalid = qrow < Lq;
  V8 bq[4];
#pragma unroll
  for (int ks = 0; ks < 4; ks++) {
    FragC f;
    f.u = make_uint4(0, 0, 0, 0);
    if (qvalid) f.u = *reinterpret_cast<const uint4*>(qp + qrow * p.sqm + ks * 16 + hh * 8);
    bq[ks] = fragc_as<E>(f);
  }

  f32x16 ot[2];
#pragma unroll
  for (int dt = 0; dt < 2; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) ot[dt][r] = 0.f;
  float m_i = -INFINITY, l_i = 0.f;
  const float sl2 = p.scale * 1.4426950408889634f;

  const int tr_row = 4 * hh + ((lane & 15) >> 2);
  const int tr_col = ((lane >> 4) & 1) * 16 + (lane & 3) * 4;

  // cooperative tile staging: thread owns 16-byte chunks e = tid and tid + 256 of each 64x64 tile
  const int ld_row0 = tid >> 3, ld_dch = tid & 7;  // second chunk: row + 32
  uint4 kr[2], vr[2];
  auto prefetch = [&](int64_t start) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int64_t row = start + ld_row0 + 32 * i;
      kr[i] = make_uint4(0, 0, 0, 0);
      vr[i] = make_uint4(0, 0, 0, 0);
      if (row < Lk) {
        kr[i] = *reinterpret_cast<const uint4*>(kp + row * p.skn + ld_dch * 8);
        vr[i] = *reinterpret_cast<const uint4*>(vp + row * p.svn + ld_dch * 8);
      }
    }
  };

  const int ntiles = (int)((Lk + 63) / 64);
  prefetch(0);
  for (int t = 0; t < ntiles; t++) {
    const int64_t start = (int64_t)t * 64;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 2; i++) {
      *reinterpret_cast<uint4*>(Ks + (ld_row0 + 32 * i) * kCLd + ld_dch * 8) = kr[i];
      *reinterpret_cast<uint4*>(Vs + (ld_row0 + 32 * i) * kCLd + ld_dch * 8) = vr[i];
    }
    __syncthreads();
    if (t + 1 < ntiles) prefetch(start + 64);
    const bool partial = start + 64 > Lk;

    f32x16 st[2];
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
#pragma unroll
      for (int r = 0; r < 16; r++) st[kt][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        FragC f;
        f.u = *reinterpret_cast<const uint4*>(Ks + (kt * 32 + c) * kCLd + ks * 16 + hh * 8);
        st[kt] = MfmaC<E>::mma(fragc_as<E>(f), bq[ks], st[kt]);
      }
    }

    if (p.scores != nullptr && qvalid) {
      float* srow = p.scores + (((int64_t)b * p.H + h) * Lq + qrow) * Lk + start;
      const bool vec = ((Lk & 3) == 0) && !partial && ((reinterpret_cast<uintptr_t>(p.scores) & 15u) == 0);
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          const int col = kt * 32 + 4 * hh + 8 * g4;
          if (vec) {
            *reinterpret_cast<float4*>(srow + col) = make_float4(st[kt][4 * g4], st[kt][4 * g4 + 1], st[kt][4 * g4 + 2], st[kt][4 * g4 + 3]);
          } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
              if (start + col + e < Lk) srow[col + e] = st[kt][4 * g4 + e];
          }
        }
    }

    if (partial) {
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int64_t key = start + kt * 32 + hh * 4 + 8 * (r >> 2) + (r & 3);
          if (key >= Lk) st[kt][r] = -INFINITY;
        }
    }
    float mx = st[0][0];
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int r = 0; r < 16; r++) mx = fmaxf(mx, st[kt][r]);
    mx = xh_max(mx);
    const float m_new = fmaxf(m_i, mx * sl2);
    const float alpha = __builtin_amdgcn_exp2f(m_i - m_new);
    float rowsum = 0.f;
    V8 pf[2][2];
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int jj = 0; jj < 2; jj++) {
        V8 pk;
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const float pv = __builtin_amdgcn_exp2f(fmaf(st[kt][8 * jj + e], sl2, -m_new));
          rowsum += pv;
          pk[e] = (E)pv;
        }
        pf[kt][jj] = pk;
      }
    l_i = l_i * alpha + rowsum;
    m_i = m_new;
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
      for (int r = 0; r < 16; r++) ot[dt][r] *= alpha;

#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int jj = 0; jj < 2; jj++)
#pragma unroll
        for (int dt = 0; dt < 2; dt++) {
          const E* a0 = Vs + (kt * 32 + jj * 16 + tr_row) * kCLd + dt * 32 + tr_col;
          FragC f;
          f.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
          f.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0 + 8 * kCLd));
          ot[dt] = MfmaC<E>::mma(fragc_as<E>(f), pf[kt][jj], ot[dt]);
        }
  }

  const float l = xh_sum(l_i);
  if (qvalid) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    E* op = (E*)p.o + (int64_t)b * p.sob + (int64_t)h * p.soh + qrow * p.som;
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        union { E e[4]; uint2 u; } pk;
#pragma unroll
        for (int e = 0; e < 4; e++) pk.e[e] = (E)(ot[dt][4 * g4 + e] * inv);
        *reinterpret_cast<uint2*>(op + dt * 32 + 4 * hh + 8 * g4) = pk.u;
      }
    if (p.lse != nullptr && hh == 0)
      p.lse[((int64_t)b * p.H + h) * Lq + qrow] = l > 0.f ? (m_i + __builtin_amdgcn_logf(l)) * 0.6931471805599453f : -INFINITY;
  }
}

int launch_compressed_mfma(const AttnParams& p, int dtype, void* stream) {
  if (p.topk_idx != nullptr && p.scores == nullptr)
    return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk: fused selection not built; pass a scores buffer");
  const int64_t nqg = (p.Lq + 127) / 128;
  if (nqg > 0x7fffffffLL || (int64_t)p.B * p.H > 65535) return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk: grid too large");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)nqg, (unsigned)(p.B * p.H)), blk(256);
  if (dtype == S3R_BF16)
    hipLaunchKernelGGL(compressed_mfma_kernel<bf16_t>, grid, blk, 0, st, p);
  else
    hipLaunchKernelGGL(compressed_mfma_kernel<f16_t>, grid, blk, 0, st, p);
  int rc = check_launch("compressed_mfma_kernel");
  if (rc != S3R_OK) return rc;
  if (p.topk_idx != nullptr)
    rc = s3r_topk_rows(p.scores, p.topk_idx, (int64_t)p.B * p.H * p.Lq, (int)p.Lk, p.Lk, p.K, stream);
  return rc;
}

}  // namespace s3r
