// One pass over the layer's packed q/k/v projection (head_dim 64), HBM bound: every token row of q and k is read once,
// normalised (LayerNorm over the head dimension), rotated (2-D rotary embedding) and written contiguous for the
// selection kernel, and in the same pass the RAW rows of q, k and v are summed into the block means of the compressed
// branch.  v itself is not rewritten: the attention kernels read it in place through its strides.
//
// Replaces, in pi3/models/layers/sparse_attention.py, the pooling of the raw projection (:97-99) together with the three
// .contiguous() copies, q_norm / k_norm, the casts and the two rope calls on the full tokens (:115-124): there each of
// q and k is read three times (pooling, norm, rope) and written twice; here 3*N*C elements are read and 2*N*C written.
//
// One wavefront per (batch, head, block).  A lane owns 16 bytes of a row (8 bf16 / 4 fp32 values), 8 (16) lanes own a
// row, the wave covers 8 (4) token rows per step; row statistics are xor-shuffle folds over the lanes of a row, the
// rotation partner (element +-16 inside a half) lives two (four) lanes away.  Rounding points are those of the
// separate kernels (s3r_pool_mean, s3r_norm_rope), and the order of the additions is the pooling kernel's, so both
// results are the same bits as theirs.
#include "s3r_common.h"

namespace s3r {

// One wave-wide step (8 or 4 token rows of q, k and v: five 16-byte loads per lane with the table rows) is in flight
// at a time and q's temporaries are dead before k's are born: the kernel lives on many resident waves (128 registers,
// four per SIMD), not on deep batches per wave -- with two steps in flight the register file held half as many waves
// and the pass took 2.4 times as long.
// ALL: LayerNorm with bias and positions are all there (the layer's own call): their run-time tests, and the default
// values of the paths not taken, are then not compiled in.
template <typename T, bool ALL>
__global__ __launch_bounds__(256, 4) void qkv_prepass_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, T* __restrict__ q_out, T* __restrict__ k_out,
    T* __restrict__ qc, T* __restrict__ kc, T* __restrict__ vc, const int32_t* __restrict__ pos, const T* __restrict__ cos_tab,
    const T* __restrict__ sin_tab, int P, const T* __restrict__ qn_w, const T* __restrict__ qn_b, const T* __restrict__ kn_w,
    const T* __restrict__ kn_b, float eps, int H, int64_t N, int block, int64_t Nc, int64_t total, int64_t sxb, int64_t sxh,
    int64_t sxn, int64_t spb, int64_t spn) {
#pragma clang fp contract(off)
  constexpr int D = 64;
  constexpr int VEC = 16 / sizeof(T);
  constexpr int LPR = D / VEC;       // lanes per row
  constexpr int RPW = 64 / LPR;      // rows per wave-wide step
  constexpr int QL = (D / 4) / VEC;  // lanes per quarter of the head dimension
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= total) return;
  // heads fastest: the waves that run side by side read neighbouring 128-byte pieces of the same token rows of the
  // packed projection (one head each), not rows 3*H*128 bytes apart
  const int h = (int)(w % H);
  const int64_t bj = w / H;
  const int64_t j = bj % Nc;
  const int64_t b = bj / Nc;
  const int r0 = lane / LPR;
  const int lr = lane - r0 * LPR;
  const int64_t t0 = j * block;
  const int nvalid = (int)((N - t0 < block) ? (N - t0) : block);
  const int64_t in_off = b * sxb + h * sxh + lr * VEC;
  T* const qo = q_out + ((b * H + h) * N) * D + lr * VEC;
  T* const ko = k_out + ((b * H + h) * N) * D + lr * VEC;
  const int half = lr / (2 * QL);    // 0: y half, 1: x half
  const int second = (lr / QL) & 1;  // which quarter of the half this lane holds
  const int f0 = (lr % QL) * VEC;    // frequency index of the lane's first value

  // LayerNorm parameters of the lane's 16 bytes (q_norm and k_norm are different modules): fetched in every step from
  // the vector cache rather than held, their 16 registers are worth more as room for one more resident wave
  const bool norm = ALL || qn_w != nullptr;
  const bool rotate = ALL || pos != nullptr;
  // The block's positions, fetched with two coalesced loads per 64 tokens (lane l holds values l and 64 + l of the
  // (y, x) pairs) and handed out by shuffles: the table rows of a step then need no load of their own position first.
  int pos_lo = 0, pos_hi = 0;
  auto fetch_positions = [&](int first) {  // tokens first .. first + 63 of the block
    const int ta = first + (lane >> 1), tb = first + 32 + (lane >> 1);
    const int64_t na = t0 + (ta < nvalid ? ta : nvalid - 1), nb = t0 + (tb < nvalid ? tb : nvalid - 1);
    pos_lo = pos[b * spb + na * spn + (lane & 1)];
    pos_hi = pos[b * spb + nb * spn + (lane & 1)];
  };

  float aq[VEC], ak[VEC], av[VEC];
#pragma unroll
  for (int i = 0; i < VEC; i++) aq[i] = ak[i] = av[i] = 0.f;

  // one wave-wide step; WHOLE: all its rows are inside the block (no row to keep out of the sums and the stores)
  auto step = [&](int rbase, auto whole_tag) {
    constexpr bool WHOLE = decltype(whole_tag)::value;
    const int rr = rbase + r0;
    const bool keep = WHOLE || rr < nvalid;
    const int rcl = keep ? rr : nvalid - 1;  // rows beyond the block shadow its last row (not added, not stored)
    if (rotate && (rbase & 63) == 0) fetch_positions(rbase);
    const int64_t off = in_off + (t0 + rcl) * sxn;
    const u32x4 lq = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(q + off));
    const u32x4 lk = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(k + off));
    const u32x4 lv = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(v + off));
    uint4 rc = make_uint4(0, 0, 0, 0), rs = rc;
    if (rotate) {
      const int slot = 2 * (rcl & 63) + half;  // index of (token, y or x) among the fetched 128
      const int from_lo = __shfl(pos_lo, slot & 63), from_hi = __shfl(pos_hi, slot & 63);
      int pp = slot < 64 ? from_lo : from_hi;
      pp = pp < 0 ? 0 : (pp >= P ? P - 1 : pp);
      rc = *reinterpret_cast<const uint4*>(cos_tab + (int64_t)pp * (D / 4) + f0);
      rs = *reinterpret_cast<const uint4*>(sin_tab + (int64_t)pp * (D / 4) + f0);
      if constexpr (sizeof(T) == 2) {
        // "rotate half" is (-second quarter, first quarter): the lanes of a first quarter take their partner's value
        // with a minus sign, which is put on the sine instead, on the packed words (rounding is symmetric:
        // round(-a * s) = round(a * -s), the same bits)
        const uint32_t flip = second ? 0u : 0x80008000u;
        rs.x ^= flip; rs.y ^= flip; rs.z ^= flip; rs.w ^= flip;
      }
    }
    const T* ce = reinterpret_cast<const T*>(&rc);
    const T* se = reinterpret_cast<const T*>(&rs);
#pragma unroll
    for (int i = 0; i < VEC; i++) av[i] += keep ? to_f32(reinterpret_cast<const T*>(&lv)[i]) : 0.f;
    auto one = [&](const u32x4& raw, float (&acc)[VEC], const T* __restrict__ ln_w, const T* __restrict__ ln_b, T* dst) {
      uint4 wgt_raw = make_uint4(0, 0, 0, 0), bias_raw = wgt_raw;
      if (norm) {
        wgt_raw = *reinterpret_cast<const uint4*>(ln_w + lr * VEC);
        if (ALL || ln_b != nullptr) bias_raw = *reinterpret_cast<const uint4*>(ln_b + lr * VEC);
      }
      const T* wgt = reinterpret_cast<const T*>(&wgt_raw);
      const T* bias = reinterpret_cast<const T*>(&bias_raw);
      float x[VEC];
#pragma unroll
      for (int i = 0; i < VEC; i++) {
        x[i] = to_f32(reinterpret_cast<const T*>(&raw)[i]);
        acc[i] += keep ? x[i] : 0.f;
      }
      if (norm) {  // fp32 statistics over the 64 values of the row, result rounded to T
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < VEC; i++) s += x[i];
        s = group_sum<LPR>(s);
        const float mean = s * (1.0f / D);
        float var = 0.f;
#pragma unroll
        for (int i = 0; i < VEC; i++) var += (x[i] - mean) * (x[i] - mean);
        var = group_sum<LPR>(var);
        const float rstd = 1.0f / sqrtf(var * (1.0f / D) + eps);
#pragma unroll
        for (int i = 0; i < VEC; i++) x[i] = round_to<T>((x[i] - mean) * rstd * to_f32(wgt[i]) + to_f32(bias[i]));
      }
      if (rotate) {
#pragma unroll
        for (int i = 0; i < VEC; i++) {
          const float other = lane_xor<QL>(x[i]);     // the paired value, one quarter away
          const float rot = sizeof(T) == 2 || second ? other : -other;  // (16-bit types: the sign is on the sine)
          const float a = round_to<T>(x[i] * to_f32(ce[i]));
          const float c2 = round_to<T>(rot * to_f32(se[i]));
          x[i] = a + c2;
        }
      }
      if (keep) {
        uint4 o;
#pragma unroll
        for (int i = 0; i < VEC; i++) reinterpret_cast<T*>(&o)[i] = from_f32<T>(x[i]);
        *reinterpret_cast<uint4*>(dst + (t0 + rr) * D) = o;
      }
    };
    one(lq, aq, qn_w, qn_b, qo);
    __builtin_amdgcn_sched_barrier(0);  // q's temporaries are dead before k's are born
    one(lk, ak, kn_w, kn_b, ko);
  };
  for (int rbase = 0; rbase < nvalid; rbase += RPW) {  // wave-uniform trip count: the position shuffles span the wave
    if (rbase + RPW <= nvalid) step(rbase, std::true_type{});
    else step(rbase, std::false_type{});
  }
  // block means: fold the row groups, divide by the number of valid tokens
  for (int off = LPR; off < 64; off <<= 1) {
#pragma unroll
    for (int i = 0; i < VEC; i++) {
      aq[i] += __shfl_xor(aq[i], off);
      ak[i] += __shfl_xor(ak[i], off);
      av[i] += __shfl_xor(av[i], off);
    }
  }
  if (r0 == 0) {
    const float cnt = (float)nvalid;
    uint4 oq, ok, ov;
#pragma unroll
    for (int i = 0; i < VEC; i++) {
      reinterpret_cast<T*>(&oq)[i] = from_f32<T>(aq[i] / cnt);
      reinterpret_cast<T*>(&ok)[i] = from_f32<T>(ak[i] / cnt);
      reinterpret_cast<T*>(&ov)[i] = from_f32<T>(av[i] / cnt);
    }
    const int64_t o = ((b * H + h) * Nc + j) * D + lr * VEC;
    *reinterpret_cast<uint4*>(qc + o) = oq;
    *reinterpret_cast<uint4*>(kc + o) = ok;
    *reinterpret_cast<uint4*>(vc + o) = ov;
  }
}

}  // namespace s3r

using namespace s3r;

extern "C" int s3r_qkv_prepass(const void* q, const void* k, const void* v, void* q_out, void* k_out, void* qc, void* kc, void* vc,
                               const int32_t* pos, const void* cos_tab, const void* sin_tab, int P, const void* qn_w,
                               const void* qn_b, const void* kn_w, const void* kn_b, float eps, int B, int H, int64_t N, int D,
                               int block, int64_t sxb, int64_t sxh, int64_t sxn, int64_t spb, int64_t spn, int dtype, void* stream) {
  if (!q || !k || !v || !q_out || !k_out || !qc || !kc || !vc) return fail(S3R_ERR_BAD_ARG, "s3r_qkv_prepass: null pointer");
  if (B <= 0 || H <= 0 || N <= 0 || block <= 0) return fail(S3R_ERR_BAD_ARG, "s3r_qkv_prepass: non-positive size");
  if (dtype != S3R_F32 && dtype != S3R_BF16 && dtype != S3R_F16) return fail(S3R_ERR_UNSUPPORTED, "s3r_qkv_prepass: dtype %d", dtype);
  if (D != 64) return fail(S3R_ERR_UNSUPPORTED, "s3r_qkv_prepass: head_dim %d (built for 64)", D);
  if (pos != nullptr && (!cos_tab || !sin_tab || P <= 0)) return fail(S3R_ERR_BAD_ARG, "s3r_qkv_prepass: positions without tables");
  if ((qn_w == nullptr) != (kn_w == nullptr)) return fail(S3R_ERR_BAD_ARG, "s3r_qkv_prepass: q and k are normalised together or not at all");
  const int es = elt_size(dtype);
  const void* ptrs[] = {q, k, v, q_out, k_out, qc, kc, vc, cos_tab, sin_tab, qn_w, qn_b, kn_w, kn_b};
  for (const void* ptr : ptrs)
    if (ptr != nullptr && !aligned16(ptr)) return fail(S3R_ERR_BAD_ARG, "s3r_qkv_prepass: pointers must be multiples of 16 bytes");
  if ((sxb * es) % 16 || (sxh * es) % 16 || (sxn * es) % 16) return fail(S3R_ERR_BAD_ARG, "s3r_qkv_prepass: strides must be multiples of 16 bytes");
  const int64_t Nc = (N + block - 1) / block;
  const int64_t total = (int64_t)B * H * Nc;
  const int64_t blocks = (total + 3) / 4;
  if (blocks > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_qkv_prepass: tensor too large for one launch");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)blocks), blk(256);
  const bool all = pos != nullptr && qn_w != nullptr && qn_b != nullptr && kn_b != nullptr;
#define S3R_PREPASS_ARGS(T)                                                                                                       \
  grid, blk, 0, st, (const T*)q, (const T*)k, (const T*)v, (T*)q_out, (T*)k_out, (T*)qc, (T*)kc, (T*)vc, pos, (const T*)cos_tab,  \
      (const T*)sin_tab, P, (const T*)qn_w, (const T*)qn_b, (const T*)kn_w, (const T*)kn_b, eps, H, N, block, Nc, total, sxb, sxh, \
      sxn, spb, spn
#define S3R_PREPASS(T)                                                                   \
  do {                                                                                   \
    if (all) hipLaunchKernelGGL((qkv_prepass_kernel<T, true>), S3R_PREPASS_ARGS(T));     \
    else hipLaunchKernelGGL((qkv_prepass_kernel<T, false>), S3R_PREPASS_ARGS(T));        \
  } while (0)
  if (dtype == S3R_F32) S3R_PREPASS(float);
  else if (dtype == S3R_BF16) S3R_PREPASS(bf16_t);
  else S3R_PREPASS(f16_t);
#undef S3R_PREPASS
#undef S3R_PREPASS_ARGS
  return check_launch("s3r_qkv_prepass");
}
