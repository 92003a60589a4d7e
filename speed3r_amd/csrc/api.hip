// C-ABI entry points of the two attention operators: argument validation and kernel choice.
#include "s3r_common.h"
#include "attn_params.h"
#include "attn_bwd.h"
#include <stdlib.h>
#include <string.h>
#include <mutex>

namespace s3r {

char* last_error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

static bool dtype_ok(int dtype) { return dtype == S3R_F32 || dtype == S3R_BF16 || dtype == S3R_F16; }

// 16-byte vector access along head_dim needs aligned bases and row strides
static bool vec_ok(const void* p, int es, int64_t s0, int64_t s1, int64_t s2) {
  return aligned16(p) && (s0 * es) % 16 == 0 && (s1 * es) % 16 == 0 && (s2 * es) % 16 == 0;
}

}  // namespace s3r

using namespace s3r;

extern "C" const char* s3r_version(void) { return "speed3r_hip 0.1 gfx950"; }

extern "C" const char* s3r_last_error(void) { return last_error_buffer(); }

extern "C" int s3r_capabilities(void) { return S3R_CAP_FUSED_TOPK; }

extern "C" int s3r_compressed_attn_topk(const void* q, const void* k, const void* v, void* o, float* lse, int32_t* topk_idx,
                                        float* scores, int B, int H, int Lq, int Lk, int D, int K,
                                        int64_t sqb, int64_t sqh, int64_t sqm, int64_t skb, int64_t skh, int64_t skn,
                                        int64_t svb, int64_t svh, int64_t svn, int64_t sob, int64_t soh, int64_t som,
                                        float softmax_scale, int dtype, void* stream) {
  if (!q || !k || (!o && !topk_idx) || (o && !v)) return fail(S3R_ERR_BAD_ARG, "s3r_compressed_attn_topk: null pointer");
  if (B <= 0 || H <= 0 || Lq <= 0 || Lk <= 0 || D <= 0) return fail(S3R_ERR_BAD_ARG, "s3r_compressed_attn_topk: non-positive size");
  if (!dtype_ok(dtype)) return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk: dtype %d", dtype);
  if (D > 64) return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk: head_dim %d > 64", D);
  if (topk_idx != nullptr && (K < 1 || K > 64 || (K & (K - 1)) != 0))
    return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk: top-k %d must be a power of two <= 64", K);

  AttnParams p = {};
  p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse; p.scores = scores; p.idx = nullptr; p.topk_idx = topk_idx;
  p.B = B; p.H = H; p.Lq = Lq; p.Lk = Lk; p.D = D; p.block = 64; p.K = K;
  p.sqb = sqb; p.sqh = sqh; p.sqm = sqm; p.skb = skb; p.skh = skh; p.skn = skn;
  p.svb = svb; p.svh = svh; p.svn = svn; p.sob = sob; p.soh = soh; p.som = som;
  p.scale = softmax_scale;

  const int es = elt_size(dtype);
  const bool mfma_ok = dtype != S3R_F32 && D == 64 && softmax_scale > 0.f && vec_ok(q, es, sqb, sqh, sqm) &&
                       vec_ok(k, es, skb, skh, skn) && (!o || (vec_ok(v, es, svb, svh, svn) && vec_ok(o, es, sob, soh, som)));
  if (mfma_ok) return launch_compressed_mfma(p, dtype, stream);
  if (topk_idx != nullptr && scores == nullptr)
    return fail(S3R_ERR_UNSUPPORTED,
                "s3r_compressed_attn_topk: fused selection needs bf16/fp16, head_dim 64, 16-byte aligned tensors; "
                "pass a scores buffer for other shapes");
  if (!o) return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk: indices without the attention output need the MFMA path");
  int rc = launch_attn_simple(p, dtype, /*select=*/false, stream);
  if (rc != S3R_OK) return rc;
  if (topk_idx != nullptr) rc = s3r_topk_rows(scores, topk_idx, (int64_t)B * H * Lq, Lk, Lk, K, stream);
  return rc;
}

extern "C" int s3r_compressed_attn_topk_causal(const void* q, const void* k, const void* v, void* o, float* lse, int32_t* topk_idx,
                                               float* scores, int B, int H, int Lq, int Lk, int D, int K,
                                               int64_t sqb, int64_t sqh, int64_t sqm, int64_t skb, int64_t skh, int64_t skn,
                                               int64_t svb, int64_t svh, int64_t svn, int64_t sob, int64_t soh, int64_t som,
                                               float softmax_scale, int dtype, void* stream) {
  if (!q || !k || !v || !o) return fail(S3R_ERR_BAD_ARG, "s3r_compressed_attn_topk_causal: null pointer");
  if (B <= 0 || H <= 0 || Lq <= 0 || Lk <= 0 || D <= 0) return fail(S3R_ERR_BAD_ARG, "s3r_compressed_attn_topk_causal: non-positive size");
  if (!dtype_ok(dtype)) return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk_causal: dtype %d", dtype);
  if (D > 64) return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk_causal: head_dim %d > 64", D);
  if (topk_idx != nullptr && (K < 1 || K > 64 || (K & (K - 1)) != 0))
    return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk_causal: top-k %d must be a power of two <= 64", K);
  if (topk_idx != nullptr && scores == nullptr)
    return fail(S3R_ERR_BAD_ARG, "s3r_compressed_attn_topk_causal: the indices are selected from a score buffer; pass one");
  AttnParams p = {};
  p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse; p.scores = scores; p.idx = nullptr; p.topk_idx = topk_idx;
  p.B = B; p.H = H; p.Lq = Lq; p.Lk = Lk; p.D = D; p.block = 64; p.K = K; p.causal = 1;
  p.sqb = sqb; p.sqh = sqh; p.sqm = sqm; p.skb = skb; p.skh = skh; p.skn = skn;
  p.svb = svb; p.svh = svh; p.svn = svn; p.sob = sob; p.soh = soh; p.som = som;
  p.scale = softmax_scale;
  int rc = launch_attn_simple(p, dtype, /*select=*/false, stream);
  if (rc != S3R_OK) return rc;
  if (topk_idx != nullptr) rc = launch_topk_rows(scores, topk_idx, (int64_t)B * H * Lq, Lk, Lk, K, Lq, stream);
  return rc;
}

// ---- the entry point that allocates nothing --------------------------------------------------
// Score buffer of s3r_compressed_attn_topk_static: device memory owned by the code object, one copy per GPU at
// its own address, held until the process ends.  The name below is only a handle for hipGetSymbolAddress; host
// code uses the looked-up address.
static __device__ __align__(256) float scratch[S3R_STATIC_SCORES_MAX];

namespace s3r {

static constexpr int kMaxDevices = 64;
static float* g_scratch_ptr[kMaxDevices] = {};   // per device, filled on the first call there
static std::mutex g_scratch_mutex;

// Address of the current device's copy of `scratch`; looked up once per device.
static int static_scores(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(S3R_ERR_HIP, "s3r_compressed_attn_topk_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk_static: device %d", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    float* ptr = nullptr;
    e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      return fail(S3R_ERR_HIP, "s3r_compressed_attn_topk_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return S3R_OK;
}

}  // namespace s3r

extern "C" int s3r_compressed_attn_topk_static(const void* q, const void* k, const void* v, void* o, float* lse, int32_t* topk_idx,
                                               int B, int H, int Lq, int Lk, int D, int K,
                                               int64_t sqb, int64_t sqh, int64_t sqm, int64_t skb, int64_t skh, int64_t skn,
                                               int64_t svb, int64_t svh, int64_t svn, int64_t sob, int64_t soh, int64_t som,
                                               float softmax_scale, int dtype, void* stream) {
  if (!o || !topk_idx) return fail(S3R_ERR_BAD_ARG, "s3r_compressed_attn_topk_static: null pointer");
  if (B <= 0 || H <= 0 || Lq <= 0 || Lk <= 0) return fail(S3R_ERR_BAD_ARG, "s3r_compressed_attn_topk_static: non-positive size");
  const unsigned long long need = (unsigned long long)B * H * Lq * (unsigned long long)Lk;
  if (need > S3R_STATIC_SCORES_MAX)
    return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk_static: B*H*Lq*Lk = %llu scores exceed the built-in buffer of %u "
                                     "(use s3r_compressed_attn_topk)", need, (unsigned)S3R_STATIC_SCORES_MAX);
  float* scores = nullptr;
  int rc = static_scores(&scores);
  if (rc != S3R_OK) return rc;
  // every score of the B*H*Lq*Lk the selection reads is written by the attention kernel first: nothing to clear
  return s3r_compressed_attn_topk(q, k, v, o, lse, topk_idx, scores, B, H, Lq, Lk, D, K, sqb, sqh, sqm, skb, skh, skn,
                                  svb, svh, svn, sob, soh, som, softmax_scale, dtype, stream);
}

namespace s3r {

// merge arguments of the fused variant; out == nullptr: plain selection attention
struct MergeArgs {
  const void* o_cmp;
  const void* gate;
  void* out;
  int64_t scb, sch, scm, sgb, sgh, sgn;
};

static int select_attn_impl(const char* who, const void* q, const void* k, const void* v, const int32_t* idx, void* o, float* lse,
                            int B, int H, int64_t N, int D, int block, int K,
                            int64_t sqb, int64_t sqh, int64_t sqn, int64_t skb, int64_t skh, int64_t skn,
                            int64_t svb, int64_t svh, int64_t svn, int64_t sob, int64_t soh, int64_t son,
                            int64_t sib, int64_t sih, int64_t sim, float softmax_scale, int dtype, const MergeArgs& m,
                            void* stream) {
  const bool merge = m.out != nullptr;
  if (!q || !k || !v || !idx || (!merge && !o)) return fail(S3R_ERR_BAD_ARG, "%s: null pointer", who);
  if (merge && (!m.o_cmp || !m.gate)) return fail(S3R_ERR_BAD_ARG, "%s: null pointer", who);
  if (B <= 0 || H <= 0 || N <= 0 || D <= 0 || K <= 0) return fail(S3R_ERR_BAD_ARG, "%s: non-positive size", who);
  if (!dtype_ok(dtype)) return fail(S3R_ERR_UNSUPPORTED, "%s: dtype %d", who, dtype);
  if (D > 64) return fail(S3R_ERR_UNSUPPORTED, "%s: head_dim %d > 64", who, D);
  if (block != 4 && block != 16 && block != 32 && block != 64)
    return fail(S3R_ERR_UNSUPPORTED, "%s: block %d not in {4,16,32,64}", who, block);

  AttnParams p = {};
  p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse; p.scores = nullptr; p.idx = idx; p.topk_idx = nullptr;
  p.B = B; p.H = H; p.Lq = N; p.Lk = N; p.D = D; p.block = block; p.K = K;
  p.sqb = sqb; p.sqh = sqh; p.sqm = sqn; p.skb = skb; p.skh = skh; p.skn = skn;
  p.svb = svb; p.svh = svh; p.svn = svn; p.sob = sob; p.soh = soh; p.som = son;
  p.sib = sib; p.sih = sih; p.sim = sim;
  p.scale = softmax_scale;
  p.merge_oc = m.o_cmp; p.merge_gate = m.gate; p.merge_out = m.out;
  p.scb = m.scb; p.sch = m.sch; p.scm = m.scm; p.sgb = m.sgb; p.sgh = m.sgh; p.sgn = m.sgn;

  const int es = elt_size(dtype);
  // (row strides of q, k, v positive and below 2^20 elements: the transfers use 32-bit byte offsets inside a 64-row tile)
  const bool mfma_ok = dtype != S3R_F32 && D == 64 && block == 64 && K <= 64 && softmax_scale > 0.f &&
                       skn > 0 && svn > 0 && sqn > 0 && skn < (1 << 20) && svn < (1 << 20) && sqn < (1 << 20) &&
                       vec_ok(q, es, sqb, sqh, sqn) && vec_ok(k, es, skb, skh, skn) && vec_ok(v, es, svb, svh, svn) &&
                       (merge ? (vec_ok(m.o_cmp, es, m.scb, m.sch, m.scm) && aligned16(m.out)) : vec_ok(o, es, sob, soh, son));
  // 16-token blocks (the reference layer's own setting): MFMA kernel that pairs query blocks
  const bool b16_ok = dtype != S3R_F32 && D == 64 && block == 16 && K <= 64 && softmax_scale > 0.f &&
                      skn > 0 && svn > 0 && sqn > 0 && skn < (1 << 20) && svn < (1 << 20) && sqn < (1 << 20) &&
                      vec_ok(q, es, sqb, sqh, sqn) && vec_ok(k, es, skb, skh, skn) && vec_ok(v, es, svb, svh, svn) &&
                      (merge ? (vec_ok(m.o_cmp, es, m.scb, m.sch, m.scm) && aligned16(m.out)) : vec_ok(o, es, sob, soh, son));
  if (merge) {
    if (b16_ok) return launch_select_b16(p, dtype, stream);
    if (!mfma_ok)
      return fail(S3R_ERR_UNSUPPORTED, "%s: the fused merge needs an MFMA kernel (bf16/fp16, head_dim 64, block 64 or 16, "
                                       "16-byte aligned tensors); run s3r_select_attn and s3r_gated_merge instead", who);
    return launch_select_pipe(p, dtype, stream);
  }
  if (mfma_ok) return launch_select_pipe(p, dtype, stream);
  if (b16_ok) return launch_select_b16(p, dtype, stream);
  return launch_attn_simple(p, dtype, /*select=*/true, stream);
}

}  // namespace s3r

extern "C" int s3r_select_attn(const void* q, const void* k, const void* v, const int32_t* idx, void* o, float* lse,
                               int B, int H, int64_t N, int D, int block, int K,
                               int64_t sqb, int64_t sqh, int64_t sqn, int64_t skb, int64_t skh, int64_t skn,
                               int64_t svb, int64_t svh, int64_t svn, int64_t sob, int64_t soh, int64_t son,
                               int64_t sib, int64_t sih, int64_t sim, float softmax_scale, int dtype, void* stream) {
  const MergeArgs none = {};
  return select_attn_impl("s3r_select_attn", q, k, v, idx, o, lse, B, H, N, D, block, K, sqb, sqh, sqn, skb, skh, skn,
                          svb, svh, svn, sob, soh, son, sib, sih, sim, softmax_scale, dtype, none, stream);
}

extern "C" int s3r_select_attn_merge(const void* q, const void* k, const void* v, const int32_t* idx,
                                     const void* o_cmp, const void* gate, void* out,
                                     int B, int H, int64_t N, int D, int block, int K,
                                     int64_t sqb, int64_t sqh, int64_t sqn, int64_t skb, int64_t skh, int64_t skn,
                                     int64_t svb, int64_t svh, int64_t svn, int64_t sib, int64_t sih, int64_t sim,
                                     int64_t scb, int64_t sch, int64_t scm, int64_t sgb, int64_t sgh, int64_t sgn,
                                     float softmax_scale, int dtype, void* stream) {
  if (!out) return fail(S3R_ERR_BAD_ARG, "s3r_select_attn_merge: null pointer");
  const MergeArgs m = {o_cmp, gate, out, scb, sch, scm, sgb, sgh, sgn};
  return select_attn_impl("s3r_select_attn_merge", q, k, v, idx, nullptr, nullptr, B, H, N, D, block, K, sqb, sqh, sqn,
                          skb, skh, skn, svb, svh, svn, 0, 0, 0, sib, sih, sim, softmax_scale, dtype, m, stream);
}

extern "C" int s3r_attn_bwd_delta(const void* o, const void* dout, float* delta, int B, int H, int64_t N, int D,
                                  int64_t sob, int64_t soh, int64_t son, int64_t sdb, int64_t sdh, int64_t sdn,
                                  int dtype, void* stream) {
  if (!o || !dout || !delta) return fail(S3R_ERR_BAD_ARG, "s3r_attn_bwd_delta: null pointer");
  if (B <= 0 || H <= 0 || N <= 0) return fail(S3R_ERR_BAD_ARG, "s3r_attn_bwd_delta: non-positive size");
  if ((dtype != S3R_BF16 && dtype != S3R_F16) || D != 64)
    return fail(S3R_ERR_UNSUPPORTED, "s3r_attn_bwd_delta: built for bf16/fp16, head_dim 64");
  if (!vec_ok(o, 2, sob, soh, son) || !vec_ok(dout, 2, sdb, sdh, sdn))
    return fail(S3R_ERR_BAD_ARG, "s3r_attn_bwd_delta: pointers and strides must be multiples of 16 bytes");
  return launch_bwd_delta(o, dout, delta, B, H, N, sob, soh, son, sdb, sdh, sdn, dtype, stream);
}

extern "C" int s3r_key_block_lists(const int32_t* idx, int32_t* kq_list, int32_t* kq_off, int B, int H, int64_t nqb, int K, int64_t nkb,
                                   int64_t sib, int64_t sih, int64_t sim, int64_t list_stride, void* stream) {
  if (!idx || !kq_list || !kq_off) return fail(S3R_ERR_BAD_ARG, "s3r_key_block_lists: null pointer");
  if (B <= 0 || H <= 0 || nqb <= 0 || K <= 0 || nkb <= 0) return fail(S3R_ERR_BAD_ARG, "s3r_key_block_lists: non-positive size");
  if (nqb * K > 0x7fffffffLL || nkb >= 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_key_block_lists: more than 2^31 entries per head");
  if (list_stride < nqb * K) return fail(S3R_ERR_BAD_ARG, "s3r_key_block_lists: list_stride below nqb * K");
  return launch_key_block_lists(idx, kq_list, kq_off, B, H, nqb, K, nkb, sib, sih, sim, list_stride, stream);
}

extern "C" int s3r_attn_bwd(const void* q, const void* k, const void* v, const void* dout, const float* lse, const float* delta,
                            const int32_t* idx, const int32_t* kq_list, const int32_t* kq_off, int64_t list_stride,
                            void* dq, void* dk, void* dv,
                            int B, int H, int64_t Lq, int64_t Lk, int D, int block, int K,
                            int64_t sqb, int64_t sqh, int64_t sqm, int64_t skb, int64_t skh, int64_t skn,
                            int64_t svb, int64_t svh, int64_t svn, int64_t sgb, int64_t sgh, int64_t sgm,
                            int64_t sdqb, int64_t sdqh, int64_t sdqm, int64_t sdkb, int64_t sdkh, int64_t sdkn,
                            int64_t sdvb, int64_t sdvh, int64_t sdvn, int64_t sib, int64_t sih, int64_t sim,
                            float softmax_scale, int dtype, void* stream) {
  if (!q || !k || !v || !dout || !lse || !delta) return fail(S3R_ERR_BAD_ARG, "s3r_attn_bwd: null pointer");
  if (!dq && !dk && !dv) return fail(S3R_ERR_BAD_ARG, "s3r_attn_bwd: no gradient requested");
  if ((dk == nullptr) != (dv == nullptr)) return fail(S3R_ERR_BAD_ARG, "s3r_attn_bwd: dk and dv come together");
  if (idx != nullptr && dk != nullptr && (!kq_list || !kq_off)) return fail(S3R_ERR_BAD_ARG, "s3r_attn_bwd: dk/dv of the selection branch need the key-centric lists");
  if (B <= 0 || H <= 0 || Lq <= 0 || Lk <= 0 || (idx != nullptr && K <= 0)) return fail(S3R_ERR_BAD_ARG, "s3r_attn_bwd: non-positive size");
  if ((dtype != S3R_BF16 && dtype != S3R_F16) || D != 64 || (idx != nullptr && block != 64 && block != 16) || K > 64 || !(softmax_scale > 0.f))
    return fail(S3R_ERR_UNSUPPORTED, "s3r_attn_bwd: built for bf16/fp16, head_dim 64, block 64 or 16, top-k <= 64, positive scale");
  const int64_t lim = 1 << 20;
  if (sqm <= 0 || skn <= 0 || svn <= 0 || sgm <= 0 || sqm >= lim || skn >= lim || svn >= lim || sgm >= lim)
    return fail(S3R_ERR_UNSUPPORTED, "s3r_attn_bwd: row strides must be positive and below 2^20 elements");
  if (!vec_ok(q, 2, sqb, sqh, sqm) || !vec_ok(k, 2, skb, skh, skn) || !vec_ok(v, 2, svb, svh, svn) || !vec_ok(dout, 2, sgb, sgh, sgm) ||
      (dq && !vec_ok(dq, 2, sdqb, sdqh, sdqm)) || (dk && (!vec_ok(dk, 2, sdkb, sdkh, sdkn) || !vec_ok(dv, 2, sdvb, sdvh, sdvn))))
    return fail(S3R_ERR_BAD_ARG, "s3r_attn_bwd: pointers and strides must be multiples of 16 bytes");
  BwdParams p = {};
  p.q = q; p.k = k; p.v = v; p.dout = dout; p.lse = lse; p.delta = delta; p.dq = dq; p.dk = dk; p.dv = dv;
  p.idx = idx; p.kq_list = kq_list; p.kq_off = kq_off; p.list_stride = list_stride;
  p.B = B; p.H = H; p.Lq = Lq; p.Lk = Lk; p.K = K; p.block = idx != nullptr ? block : 64;
  p.sqb = sqb; p.sqh = sqh; p.sqm = sqm; p.skb = skb; p.skh = skh; p.skn = skn; p.svb = svb; p.svh = svh; p.svn = svn;
  p.sgb = sgb; p.sgh = sgh; p.sgm = sgm; p.sdqb = sdqb; p.sdqh = sdqh; p.sdqm = sdqm; p.sdkb = sdkb; p.sdkh = sdkh; p.sdkn = sdkn;
  p.sdvb = sdvb; p.sdvh = sdvh; p.sdvn = sdvn; p.sib = sib; p.sih = sih; p.sim = sim;
  p.scale = softmax_scale;
  return launch_attn_bwd(p, dtype, stream);
}
