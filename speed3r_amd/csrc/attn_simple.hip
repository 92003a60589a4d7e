// Generic (any I/O dtype, head_dim <= 64) attention kernel for both branches.
//
// This is the fp32-I/O instance of the path and the fallback for shapes the MFMA kernels do
// not cover (block < 64, head_dim < 64).  One 256-thread workgroup owns one query block
// (64 rows for the compressed branch, `block` rows for the selection branch) of one head.
// Thread (r, g) owns query row r and a quarter of the columns: key columns g, g+4, ... of the
// score tile and head_dim slice [16g, 16g+16) of the output.  The query row lives in
// registers; K, V and the probability tile go through LDS as fp32.  All arithmetic is fp32
// FMA; probabilities are rounded to the I/O dtype before the PV product as the reference's
// kernels do (a no-op for fp32 I/O).
//
// Causal variant of the compressed branch (p.causal; flash_attention_topk.py:71,93): a 64-row query block walks the
// key tiles below end_n = min((block + 1) * 64, Lk) only, and key j > query i gets the score -inf, in the softmax
// and in the stored score (the reference ranks such keys, below every finite score, lowest column first).
#include "s3r_common.h"
#include "attn_params.h"

namespace s3r {

constexpr int kLd = 68;  // LDS row stride in floats: float4-aligned, rows 4 banks apart

template <typename T, bool SELECT>
__global__ __launch_bounds__(256) void attn_simple_kernel(AttnParams p) {
  __shared__ float Ks[64 * kLd];
  __shared__ float Vs[64 * kLd];
  __shared__ float Ps[64 * kLd];

  const int tid = threadIdx.x;
  const int r = tid >> 2;
  const int g = tid & 3;
  const int BM = SELECT ? p.block : 64;  // query rows per workgroup == key columns per tile
  const int64_t mblk = blockIdx.x;
  const int b = blockIdx.y / p.H;
  const int h = blockIdx.y - b * p.H;
  const int D = p.D;
  const int64_t qrow = mblk * BM + r;
  const bool qvalid = (r < BM) && (qrow < p.Lq);

  const T* qp = (const T*)p.q + (int64_t)b * p.sqb + (int64_t)h * p.sqh;
  const T* kp = (const T*)p.k + (int64_t)b * p.skb + (int64_t)h * p.skh;
  const T* vp = (const T*)p.v + (int64_t)b * p.svb + (int64_t)h * p.svh;

  float qreg[64];
#pragma unroll
  for (int d = 0; d < 64; d++) qreg[d] = (qvalid && d < D) ? to_f32(qp[qrow * p.sqm + d]) : 0.f;

  float m_i = -INFINITY, l_i = 0.f;
  float acc[16];
#pragma unroll
  for (int i = 0; i < 16; i++) acc[i] = 0.f;

  const bool causal = !SELECT && p.causal != 0;
  const int64_t end_n = causal ? ((mblk + 1) * 64 < p.Lk ? (mblk + 1) * 64 : p.Lk) : p.Lk;
  const int ntiles = SELECT ? p.K : (int)((end_n + 63) / 64);
  const int32_t* idx_row = SELECT ? p.idx + (int64_t)b * p.sib + (int64_t)h * p.sih + mblk * p.sim : nullptr;

  for (int t = 0; t < ntiles; t++) {
    int64_t start;
    if (SELECT) {
      const int32_t j = idx_row[t];
      start = (int64_t)j * p.block;
      if (j < 0 || start >= p.Lk) continue;  // uniform over the workgroup
    } else {
      start = (int64_t)t * 64;
    }
    const int nvalid = (int)((p.Lk - start < BM) ? (p.Lk - start) : BM);

    __syncthreads();
#pragma unroll 4
    for (int i = 0; i < 16; i++) {
      const int e = tid + 256 * i;
      const int row = e >> 6, d = e & 63;
      const bool ok = row < nvalid && d < D;
      Ks[row * kLd + d] = ok ? to_f32(kp[(start + row) * p.skn + d]) : 0.f;
      Vs[row * kLd + d] = ok ? to_f32(vp[(start + row) * p.svn + d]) : 0.f;
    }
    __syncthreads();

    float s[16];
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int c = g + 4 * i;
      const float4* kr = reinterpret_cast<const float4*>(&Ks[c * kLd]);
      float a = 0.f;
#pragma unroll
      for (int d4 = 0; d4 < 16; d4++) {
        const float4 kv = kr[d4];
        a = fmaf(qreg[4 * d4 + 0], kv.x, a);
        a = fmaf(qreg[4 * d4 + 1], kv.y, a);
        a = fmaf(qreg[4 * d4 + 2], kv.z, a);
        a = fmaf(qreg[4 * d4 + 3], kv.w, a);
      }
      s[i] = (causal && start + c > qrow) ? -INFINITY : a;
    }
    if (!SELECT && p.scores != nullptr && qvalid) {
      float* srow = p.scores + (((int64_t)b * p.H + h) * p.Lq + qrow) * p.Lk + start;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int c = g + 4 * i;
        if (c < nvalid) srow[c] = s[i];
      }
    }

    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int c = g + 4 * i;
      s[i] = (c < nvalid && s[i] != -INFINITY) ? s[i] * p.scale : -INFINITY;  // (-inf * a non-positive scale)
      mx = fmaxf(mx, s[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 1));
    mx = fmaxf(mx, __shfl_xor(mx, 2));
    const float m_new = fmaxf(m_i, mx);
    const float alpha = (m_i == -INFINITY) ? 0.f : expf(m_i - m_new);
    float rowsum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int c = g + 4 * i;
      const float pv = (c < nvalid && s[i] != -INFINITY) ? expf(s[i] - m_new) : 0.f;
      rowsum += pv;
      Ps[r * kLd + c] = round_to<T>(pv);
    }
    l_i = l_i * alpha + rowsum;
    m_i = m_new;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] *= alpha;
    __syncthreads();

    for (int c = 0; c < nvalid; c++) {
      const float pc = Ps[r * kLd + c];
      const float4* vr = reinterpret_cast<const float4*>(&Vs[c * kLd + g * 16]);
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const float4 vv = vr[i4];
        acc[4 * i4 + 0] = fmaf(pc, vv.x, acc[4 * i4 + 0]);
        acc[4 * i4 + 1] = fmaf(pc, vv.y, acc[4 * i4 + 1]);
        acc[4 * i4 + 2] = fmaf(pc, vv.z, acc[4 * i4 + 2]);
        acc[4 * i4 + 3] = fmaf(pc, vv.w, acc[4 * i4 + 3]);
      }
    }
  }

  float l = l_i;
  l += __shfl_xor(l, 1);
  l += __shfl_xor(l, 2);
  if (qvalid) {
    T* op = (T*)p.o + (int64_t)b * p.sob + (int64_t)h * p.soh + qrow * p.som;
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int d = g * 16 + i;
      if (d < D) op[d] = from_f32<T>(acc[i] * inv);
    }
    if (p.lse != nullptr && g == 0) p.lse[((int64_t)b * p.H + h) * p.Lq + qrow] = l > 0.f ? m_i + logf(l) : -INFINITY;
  }
}

template <typename T>
static int launch_t(const AttnParams& p, bool select, hipStream_t st) {
  const int BM = select ? p.block : 64;
  const int64_t nblk = (p.Lq + BM - 1) / BM;
  if (nblk > 0x7fffffffLL || (int64_t)p.B * p.H > 65535) return fail(S3R_ERR_UNSUPPORTED, "attention: grid too large");
  dim3 grid((unsigned)nblk, (unsigned)(p.B * p.H)), blk(256);
  if (select)
    hipLaunchKernelGGL((attn_simple_kernel<T, true>), grid, blk, 0, st, p);
  else
    hipLaunchKernelGGL((attn_simple_kernel<T, false>), grid, blk, 0, st, p);
  return check_launch("attn_simple_kernel");
}

int launch_attn_simple(const AttnParams& p, int dtype, bool select, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (dtype == S3R_F32) return launch_t<float>(p, select, st);
  if (dtype == S3R_BF16) return launch_t<bf16_t>(p, select, st);
  return launch_t<f16_t>(p, select, st);
}

}  // namespace s3r
