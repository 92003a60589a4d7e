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

// A wave works on one wave-wide step (8 or 4 token rows of q, k and v) while the rows of the next one are on their
// way, and q's temporaries are dead before k's are born: the kernel lives on many resident waves (at most 128
// registers, four per SIMD), not on deep batches per wave -- with two steps computed together the register file held
// half as many waves and the pass took 2.4 times as long.
// ALL: LayerNorm with bias and positions are all there (the layer's own call): their run-time tests, and the default
// values of the paths not taken, are then not compiled in.
// STAGED (with ALL): the workgroup first spreads the rotation tables (cosine, sine and minus sine) and the four
// LayerNorm parameter rows as fp32 over LDS, so that a step reads ready operands instead of unpacking 16-bit table and
// parameter values again for every row (a fifth of a step's vector instructions); the launcher takes it while the
// tables fit the LDS share of four resident workgroups.
template <typename T, bool ALL, bool STAGED>
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
  static_assert(!STAGED || ALL, "the staged tables serve the instance with norm, biases and positions");
  extern __shared__ __align__(16) float staged[];  // [cos | sin | -sin][P][16], then q_norm w, b, k_norm w, b [64] each
  const int lane = threadIdx.x & 63;
  if constexpr (STAGED) {
    const int rows16 = P * (D / 4);
    for (int i = threadIdx.x * VEC; i < rows16; i += 256 * VEC) {  // table rows are 16 values: whole 16-byte pieces
      const uint4 c = *reinterpret_cast<const uint4*>(cos_tab + i);
      const uint4 s = *reinterpret_cast<const uint4*>(sin_tab + i);
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        const float sv = to_f32(reinterpret_cast<const T*>(&s)[e]);
        staged[i + e] = to_f32(reinterpret_cast<const T*>(&c)[e]);
        staged[rows16 + i + e] = sv;
        staged[2 * rows16 + i + e] = -sv;
      }
    }
    const int which = threadIdx.x >> 6;
    const T* const src = which == 0 ? qn_w : which == 1 ? qn_b : which == 2 ? kn_w : kn_b;
    staged[3 * rows16 + threadIdx.x] = to_f32(src[lane]);
    __syncthreads();
  }
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

  // the rows of a step (q, k and v: three 16-byte loads per lane) are requested one step ahead where the registers
  // allow it (the staged instance; the others would pay for the twelve registers with spills)
  constexpr bool AHEAD = STAGED;
  u32x4 nq, nk, nv;
  auto request = [&](int rbase) {
    const int rr = rbase + r0;
    const int64_t off = in_off + (t0 + (rr < nvalid ? rr : nvalid - 1)) * sxn;
    nq = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(q + off));
    nk = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(k + off));
    nv = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(v + off));
  };
  if constexpr (AHEAD) request(0);
  // one wave-wide step; WHOLE: all its rows are inside the block (no row to keep out of the sums and the stores)
  auto step = [&](int rbase, auto whole_tag) {
    constexpr bool WHOLE = decltype(whole_tag)::value;
    const int rr = rbase + r0;
    const bool keep = WHOLE || rr < nvalid;
    const int rcl = keep ? rr : nvalid - 1;  // rows beyond the block shadow its last row (not added, not stored)
    if (rotate && (rbase & 63) == 0) fetch_positions(rbase);
    if constexpr (!AHEAD) request(rbase);
    const u32x4 lq = nq, lk = nk, lv = nv;
    if constexpr (AHEAD) {
      if (rbase + RPW < nvalid) request(rbase + RPW);
    }
    uint4 rc = make_uint4(0, 0, 0, 0), rs = rc;
    const float* tab_c = nullptr;  // STAGED: the lane's piece of its position's table rows in LDS
    const float* tab_s = nullptr;
    if (rotate) {
      const int slot = 2 * (rcl & 63) + half;  // index of (token, y or x) among the fetched 128
      const int from_lo = __shfl(pos_lo, slot & 63), from_hi = __shfl(pos_hi, slot & 63);
      int pp = slot < 64 ? from_lo : from_hi;
      pp = pp < 0 ? 0 : (pp >= P ? P - 1 : pp);
      if constexpr (STAGED) {
        // "rotate half" is (-second quarter, first quarter): the lanes of a first quarter take their partner's value
        // with a minus sign, which is put on the sine instead (rounding is symmetric: round(-a * s) = round(a * -s))
        tab_c = staged + pp * (D / 4) + f0;
        tab_s = tab_c + (second ? 1 : 2) * P * (D / 4);
      } else {
        rc = *reinterpret_cast<const uint4*>(cos_tab + (int64_t)pp * (D / 4) + f0);
        rs = *reinterpret_cast<const uint4*>(sin_tab + (int64_t)pp * (D / 4) + f0);
        if constexpr (sizeof(T) == 2) {  // the same sign trick on the packed words
          const uint32_t flip = second ? 0u : 0x80008000u;
          rs.x ^= flip; rs.y ^= flip; rs.z ^= flip; rs.w ^= flip;
        }
      }
    }
    const T* ce = reinterpret_cast<const T*>(&rc);
    const T* se = reinterpret_cast<const T*>(&rs);
#pragma unroll
    for (int i = 0; i < VEC; i++) av[i] += keep ? to_f32(reinterpret_cast<const T*>(&lv)[i]) : 0.f;
    auto one = [&](const u32x4& raw, float (&acc)[VEC], const T* __restrict__ ln_w, const T* __restrict__ ln_b, int ln_row, T* dst) {
      float wgt[VEC], bias[VEC];
      if constexpr (STAGED) {
        const float* lw = staged + 3 * P * (D / 4) + ln_row * D + lr * VEC;
#pragma unroll
        for (int i = 0; i < VEC; i += 4) {
          *reinterpret_cast<float4*>(&wgt[i]) = *reinterpret_cast<const float4*>(lw + i);
          *reinterpret_cast<float4*>(&bias[i]) = *reinterpret_cast<const float4*>(lw + D + i);
        }
      } else {
        uint4 wgt_raw = make_uint4(0, 0, 0, 0), bias_raw = wgt_raw;
        if (norm) {
          wgt_raw = *reinterpret_cast<const uint4*>(ln_w + lr * VEC);
          if (ALL || ln_b != nullptr) bias_raw = *reinterpret_cast<const uint4*>(ln_b + lr * VEC);
        }
#pragma unroll
        for (int i = 0; i < VEC; i++) {
          wgt[i] = to_f32(reinterpret_cast<const T*>(&wgt_raw)[i]);
          bias[i] = to_f32(reinterpret_cast<const T*>(&bias_raw)[i]);
        }
      }
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
        const float rstd = inv_sqrt(var * (1.0f / D) + eps);
#pragma unroll
        for (int i = 0; i < VEC; i++) x[i] = round_keep<T>((x[i] - mean) * rstd * wgt[i] + bias[i]);
      }
      if (rotate) {
        float cs[VEC], sn[VEC];
        if constexpr (STAGED) {
#pragma unroll
          for (int i = 0; i < VEC; i += 4) {
            *reinterpret_cast<float4*>(&cs[i]) = *reinterpret_cast<const float4*>(tab_c + i);
            *reinterpret_cast<float4*>(&sn[i]) = *reinterpret_cast<const float4*>(tab_s + i);
          }
        } else {
#pragma unroll
          for (int i = 0; i < VEC; i++) {
            cs[i] = to_f32(ce[i]);
            sn[i] = to_f32(se[i]);
          }
        }
#pragma unroll
        for (int i = 0; i < VEC; i++) {
          const float other = lane_xor<QL>(x[i]);     // the paired value, one quarter away
          const float rot = STAGED || sizeof(T) == 2 || second ? other : -other;  // (else the sign is on the sine)
          const float a = round_keep<T>(x[i] * cs[i]);
          const float c2 = round_keep<T>(rot * sn[i]);
          x[i] = a + c2;
        }
      }
      if (keep) {
        uint4 o;
#pragma unroll
        for (int i = 0; i < VEC; i++) reinterpret_cast<T*>(&o)[i] = from_f32<T>(x[i]);
        // non-temporal like the loads: nothing of this pass is read again before the attention kernels (0.50 against
        // 0.55 ms at 266 496 tokens x 16 heads)
        store16_nt(dst + (t0 + rr) * D, o);
      }
    };
    one(lq, aq, qn_w, qn_b, 0, qo);
    __builtin_amdgcn_sched_barrier(0);  // q's temporaries are dead before k's are born
    one(lk, ak, kn_w, kn_b, 2, ko);
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
  // three fp32 tables of P rows of 16 values and four parameter rows; four workgroups share a CU's 160 KB
  const size_t staged_bytes = ((size_t)3 * P * 16 + 4 * 64) * sizeof(float);
  const bool staged = all && staged_bytes <= 32 * 1024;
  const unsigned lds = staged ? (unsigned)staged_bytes : 0u;
#define S3R_PREPASS_ARGS(T)                                                                                                       \
  grid, blk, lds, st, (const T*)q, (const T*)k, (const T*)v, (T*)q_out, (T*)k_out, (T*)qc, (T*)kc, (T*)vc, pos, (const T*)cos_tab,  \
      (const T*)sin_tab, P, (const T*)qn_w, (const T*)qn_b, (const T*)kn_w, (const T*)kn_b, eps, H, N, block, Nc, total, sxb, sxh, \
      sxn, spb, spn
#define S3R_PREPASS(T)                                                                            \
  do {                                                                                            \
    if (staged) hipLaunchKernelGGL((qkv_prepass_kernel<T, true, true>), S3R_PREPASS_ARGS(T));     \
    else if (all) hipLaunchKernelGGL((qkv_prepass_kernel<T, true, false>), S3R_PREPASS_ARGS(T));  \
    else hipLaunchKernelGGL((qkv_prepass_kernel<T, false, false>), S3R_PREPASS_ARGS(T));          \
  } while (0)
  if (dtype == S3R_F32) S3R_PREPASS(float);
  else if (dtype == S3R_BF16) S3R_PREPASS(bf16_t);
  else S3R_PREPASS(f16_t);
#undef S3R_PREPASS
#undef S3R_PREPASS_ARGS
  return check_launch("s3r_qkv_prepass");
}
