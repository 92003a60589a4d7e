// Selection-branch attention on the gfx950 matrix cores (bf16 / fp16 I/O, block 64, head_dim 64).
//
// One wavefront owns one 64-row query block of one head and walks that block's selected key
// blocks; the four waves of a workgroup take four consecutive query blocks and never
// synchronise with each other (each has a private LDS region).
//
// Data flow per selected key block (64 keys x 64 head_dim):
//   * the K tile goes global -> registers directly in the MFMA A-operand layout
//     (lane = key row, 8 consecutive head_dim values = one 16-byte load); the loads of the
//     next tile are issued as soon as the S^T MFMAs of the current one have consumed the
//     registers, so they fly during the softmax and PV phases;
//   * S^T = K Q^T with v_mfma_f32_32x32x16: the accumulator layout then puts one QUERY per
//     lane (column = lane & 31) and 16 keys per 32x32 tile in its registers, so row max / row
//     sum are in-lane loops plus one exchange with lane ^ 32, and the online-softmax rescale
//     factor is lane-local;
//   * P is rounded to the I/O dtype in registers; the accumulator layout of S^T is already the
//     B-operand layout of O^T = V^T P^T (contraction index = key), with a fixed permutation of
//     keys inside each group of 16 that the V operand simply follows;
//   * the V tile goes global -> LDS without passing through registers (global_load_lds, 16
//     bytes per lane, issued right after the previous tile's PV phase has read the buffer, so
//     it flies during the next S^T and softmax phases) and comes back through
//     ds_read_b64_tr_b16, which hands each lane 4 consecutive KEYS of one head_dim column: the
//     A operand V^T without any explicit transpose.  Rows are 128 bytes; the 16-byte chunks
//     of rows 2,3 (mod 4) are stored with their halves swapped so that the four rows one
//     transposed read touches fall into four disjoint bank groups.
// The softmax runs in base 2 on logits pre-multiplied by scale*log2(e); statistics are fp32.
// The running maximum is only raised when it grows by more than 8 (a factor 256), so the
// accumulator rescale is skipped for most tiles; the final normalisation makes this exact.
//
// Workgroup -> work mapping is XCD-aware: hardware deals workgroups round-robin over the 8
// XCDs, so workgroup w is given work item (w % 8) * per_xcd + w / 8: each XCD then walks a
// contiguous range of query blocks of one head at a time and its L2 sees one head's K/V.
#include "s3r_common.h"
#include "attn_params.h"

namespace s3r {

template <typename E> struct MfmaT;
template <> struct MfmaT<bf16_t> {
  typedef bf16x8 V8;
  static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <> struct MfmaT<f16_t> {
  typedef f16x8 V8;
  static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};

union Frag16B {  // 16 bytes seen as a global-load unit or as an MFMA operand
  uint4 u;
  bf16x8 b;
  f16x8 h;
  s16x4 s[2];
};
template <typename E> __device__ __forceinline__ typename MfmaT<E>::V8 frag_as(const Frag16B& f);
template <> __device__ __forceinline__ bf16x8 frag_as<bf16_t>(const Frag16B& f) { return f.b; }
template <> __device__ __forceinline__ f16x8 frag_as<f16_t>(const Frag16B& f) { return f.h; }

__device__ __forceinline__ float xhalf_max(float x) {  // max of x over lanes l and l^32
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xhalf_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

constexpr float kRescaleSlack = 8.0f;  // log2 units the running max may lag behind before a rescale
constexpr int kVTile = 64 * 64;        // elements of one V tile in LDS (rows of 128 bytes, no padding)

template <typename E>
__global__ __launch_bounds__(256, 2) void select_mfma_kernel(AttnParams p, int nqb, int nqg, int total_wg) {
  typedef typename MfmaT<E>::V8 V8;
  __shared__ __attribute__((aligned(1024))) E vlds_all[4][kVTile];

  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int hh = lane >> 5;  // which half of the wave
  const int c = lane & 31;   // row/column inside a 32-wide MFMA tile

  // XCD-aware remap of the linear workgroup id
  const int w = blockIdx.x;
  const int xcd = w & 7, slot = w >> 3;
  const int per = total_wg >> 3, rem = total_wg & 7;
  const int vid = xcd * per + (xcd < rem ? xcd : rem) + slot;
  const int bh = vid / nqg;
  const int qg = vid - bh * nqg;
  const int b = bh / p.H;
  const int h = bh - b * p.H;
  const int qb = qg * 4 + wave;
  if (qb >= nqb) return;  // no workgroup-level barrier is used anywhere below

  const int64_t N = p.Lq;
  const int64_t q0 = (int64_t)qb * 64;
  const E* qp = (const E*)p.q + (int64_t)b * p.sqb + (int64_t)h * p.sqh;
  const E* kp = (const E*)p.k + (int64_t)b * p.skb + (int64_t)h * p.skh;
  const E* vp = (const E*)p.v + (int64_t)b * p.svb + (int64_t)h * p.svh;
  E* op = (E*)p.o + (int64_t)b * p.sob + (int64_t)h * p.soh;
  const int32_t* idx_row = p.idx + (int64_t)b * p.sib + (int64_t)h * p.sih + (int64_t)qb * p.sim;
  E* vl = &vlds_all[wave][0];

  // The block's index list, one entry per lane (K <= 64), compacted to the valid entries in order.
  const int32_t my_idx = lane < p.K ? idx_row[lane] : -1;
  uint64_t todo = __ballot(my_idx >= 0 && (int64_t)my_idx * 64 < N);
  int remaining = __popcll(todo);
  if (remaining == 0) {  // nothing to attend to: zeros
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
      const int64_t row = q0 + qt * 32 + c;
      if (row < N) {
#pragma unroll
        for (int i = 0; i < 4; i++) *reinterpret_cast<uint4*>(op + row * p.som + hh * 32 + i * 8) = make_uint4(0, 0, 0, 0);
        if (p.lse != nullptr && hh == 0) p.lse[((int64_t)b * p.H + h) * N + row] = -INFINITY;
      }
    }
    return;
  }
  auto next_start = [&]() -> int64_t {
    const int t = __ffsll((unsigned long long)todo) - 1;
    todo &= todo - 1;
    return (int64_t)__builtin_amdgcn_readlane(my_idx, t) * 64;
  };

  // Q block as the B operand of S^T = K Q^T: lane holds Q[q0 + qt*32 + c][ks*16 + hh*8 .. +8]
  V8 bq[2][4];
#pragma unroll
  for (int qt = 0; qt < 2; qt++) {
    const int64_t row = q0 + qt * 32 + c;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      Frag16B f;
      f.u = make_uint4(0, 0, 0, 0);
      if (row < N) f.u = *reinterpret_cast<const uint4*>(qp + row * p.sqm + ks * 16 + hh * 8);
      bq[qt][ks] = frag_as<E>(f);
    }
  }

  f32x16 ot[2][2];  // O^T accumulators [dt][qt]: lane holds query qt*32+c, head_dim rows dt*32 + 4hh + 8(r/4) + r%4
#pragma unroll
  for (int dt = 0; dt < 2; dt++)
#pragma unroll
    for (int qt = 0; qt < 2; qt++)
#pragma unroll
      for (int r = 0; r < 16; r++) ot[dt][qt][r] = 0.f;
  float m_i[2] = {-INFINITY, -INFINITY};  // reference maximum in use (base-2 scaled logits)
  float l_i[2] = {0.f, 0.f};              // per-lane partial row sums (this half's keys)
  const float sl2 = p.scale * 1.4426950408889634f;

  // K tile: A operand, lane holds K[start + kt*32 + c][ks*16 + hh*8 .. +8].  Addresses are a wave-uniform
  // 64-bit tile base plus a 32-bit per-lane offset.  Rows beyond N (ragged last block) re-read row N-1: their
  // scores are masked, and their V rows are zeroed in LDS before use.
  const uint32_t koff0 = (uint32_t)c * (uint32_t)p.skn + hh * 8;
  const uint32_t koff1 = (uint32_t)(32 + c) * (uint32_t)p.skn + hh * 8;
  auto load_k = [&](V8 (&ak)[2][4], int64_t start) {
    const E* kb = kp + start * p.skn;
    uint32_t off[2] = {koff0, koff1};
    if (start + 64 > N) {
      const uint32_t last = (uint32_t)(N - 1 - start);
      off[0] = (c < last ? c : last) * (uint32_t)p.skn + hh * 8;
      off[1] = (32 + c < last ? 32 + c : last) * (uint32_t)p.skn + hh * 8;
    }
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        Frag16B f;
        f.u = *reinterpret_cast<const uint4*>(kb + off[kt] + ks * 16);
        ak[kt][ks] = frag_as<E>(f);
      }
    }
  };
  // V tile: global -> LDS, instruction i fills rows 8i..8i+7 (lane -> row 8i + lane/8, chunk position lane%8);
  // position cp of row r holds source chunk cp ^ (4 * ((r >> 1) & 1)).
  const int ldv_row = lane >> 3;
  const int ldv_chunk = (lane & 7) ^ (((ldv_row >> 1) & 1) << 2);
  const uint32_t voff = (uint32_t)ldv_row * (uint32_t)p.svn + ldv_chunk * 8;
  auto load_v = [&](int64_t start) {
    const bool partial = start + 64 > N;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const E* vb = vp + (start + i * 8) * p.svn;  // wave-uniform
      uint32_t off = voff;
      if (partial) {
        const int64_t last = N - 1 - start - i * 8;  // may be negative: whole group beyond N
        const int64_t r = ldv_row < last ? ldv_row : last;
        off = (uint32_t)(int32_t)(r * p.svn) + ldv_chunk * 8;
      }
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(vb + (int32_t)off),
                                       (__attribute__((address_space(3))) void*)(vl + i * 512), 16, 0, 0);
    }
  };
  // per-lane byte offset of the transposed V read inside a 16-key group, for head_dim half dt = 0 (dt = 1: ^ 64)
  const int i16 = lane & 15;
  const int tr_row = 4 * hh + (i16 >> 2);
  const int tr_chunk = (((lane >> 4) & 1) * 2 + ((i16 & 3) >> 1)) ^ (((tr_row >> 1) & 1) << 2);
  const int tr_off = tr_row * 128 + tr_chunk * 16 + (i16 & 1) * 8;

  // One tile: S^T and softmax per query half; the next tile's K loads are issued into the same registers as soon
  // as the second half's S^T MFMAs have consumed them; PV from the LDS tile; then the next tile's V load into the
  // same LDS buffer.  `next` < 0: no further tile.
  V8 ak[2][4];
  auto tile = [&](int64_t start, int64_t next) {
    const bool partial = start + 64 > N;
    V8 pf[2][2][2];  // P^T operands [qt][kt][jj]
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
      f32x16 st[2];  // [kt]
#pragma unroll
      for (int kt = 0; kt < 2; kt++) {
#pragma unroll
        for (int r = 0; r < 16; r++) st[kt][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) st[kt] = MfmaT<E>::mma(ak[kt][ks], bq[qt][ks], st[kt]);
      }
      if (qt == 1 && next >= 0) load_k(ak, next);
      if (partial) {  // keys at or beyond N: register r of tile kt holds key kt*32 + 4hh + 8(r/4) + r%4
        const int lim = (int)(N - start) - 4 * hh;
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
          for (int r = 0; r < 16; r++)
            if (kt * 32 + 8 * (r >> 2) + (r & 3) >= lim) st[kt][r] = -INFINITY;
      }
      float mx = st[0][0];
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++) mx = fmaxf(mx, st[kt][r]);
      mx = xhalf_max(mx) * sl2;
      const bool grow = mx > m_i[qt] + kRescaleSlack;  // true on the first tile (m_i = -inf)
      if (__any(grow)) {
        const float m_new = grow ? mx : m_i[qt];
        const float alpha = __builtin_amdgcn_exp2f(m_i[qt] - m_new);  // 1 where the maximum stays
        m_i[qt] = m_new;
        l_i[qt] *= alpha;
#pragma unroll
        for (int dt = 0; dt < 2; dt++)
#pragma unroll
          for (int r = 0; r < 16; r++) ot[dt][qt][r] *= alpha;
      }
      const float m_use = m_i[qt];
      float rowsum = 0.f;
#pragma unroll
      for (int kt = 0; kt < 2; kt++) {
#pragma unroll
        for (int jj = 0; jj < 2; jj++) {
          V8 pk;
#pragma unroll
          for (int e = 0; e < 8; e++) {
            const float pv = __builtin_amdgcn_exp2f(fmaf(st[kt][8 * jj + e], sl2, -m_use));
            rowsum += pv;
            pk[e] = (E)pv;
          }
          pf[qt][kt][jj] = pk;
        }
      }
      l_i[qt] += rowsum;
    }

    if (partial) {  // last, ragged key block: wait for the tile, then clear the rows beyond N
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      const int nvalid = (int)(N - start);
#pragma unroll
      for (int i = 0; i < 8; i++)
        if (i * 8 + ldv_row >= nvalid) *reinterpret_cast<uint4*>(vl + i * 512 + lane * 8) = make_uint4(0, 0, 0, 0);
    }

    // O^T += V^T P^T.  k-step (kt,jj) contracts keys kt*32 + 16jj + {4hh..4hh+3, 8+4hh..8+4hh+3}.
    const char* vbase = reinterpret_cast<const char*>(vl);
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
#pragma unroll
      for (int jj = 0; jj < 2; jj++) {
#pragma unroll
        for (int dt = 0; dt < 2; dt++) {
          const char* a0 = vbase + (tr_off ^ (dt * 64)) + (kt * 32 + jj * 16) * 128;
          Frag16B f;
          f.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
          f.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0 + 8 * 128));
          const V8 vf = frag_as<E>(f);
#pragma unroll
          for (int qt = 0; qt < 2; qt++) ot[dt][qt] = MfmaT<E>::mma(vf, pf[qt][kt][jj], ot[dt][qt]);
        }
      }
    }
    if (next >= 0) load_v(next);
  };

  int64_t start = next_start();
  load_k(ak, start);
  load_v(start);
  while (remaining > 0) {
    remaining--;
    const int64_t next = remaining > 0 ? next_start() : -1;
    tile(start, next);
    start = next;
  }

  // epilogue
#pragma unroll
  for (int qt = 0; qt < 2; qt++) {
    const float l = xhalf_sum(l_i[qt]);
    const float inv = l > 0.f ? 1.f / l : 0.f;
    const int64_t row = q0 + qt * 32 + c;
    if (row < N) {
#pragma unroll
      for (int dt = 0; dt < 2; dt++) {
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          union { E e[4]; uint2 u; } pk;
#pragma unroll
          for (int e = 0; e < 4; e++) pk.e[e] = (E)(ot[dt][qt][4 * g4 + e] * inv);
          *reinterpret_cast<uint2*>(op + row * p.som + dt * 32 + 4 * hh + 8 * g4) = pk.u;
        }
      }
      if (p.lse != nullptr && hh == 0)
        p.lse[((int64_t)b * p.H + h) * N + row] = l > 0.f ? (m_i[qt] + __builtin_amdgcn_logf(l)) * 0.6931471805599453f : -INFINITY;
    }
  }
}

int launch_select_mfma(const AttnParams& p, int dtype, void* stream) {
  const int64_t nqb = (p.Lq + 63) / 64;
  const int64_t nqg = (nqb + 3) / 4;
  const int64_t total = nqg * p.B * p.H;
  if (total > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_select_attn: grid too large");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)total), blk(256);
  if (dtype == S3R_BF16)
    hipLaunchKernelGGL(select_mfma_kernel<bf16_t>, grid, blk, 0, st, p, (int)nqb, (int)nqg, (int)total);
  else
    hipLaunchKernelGGL(select_mfma_kernel<f16_t>, grid, blk, 0, st, p, (int)nqb, (int)nqg, (int)total);
  return check_launch("select_mfma_kernel");
}

}  // namespace s3r
