// Exact row-wise top-k of materialised fp32 scores: one wavefront per row, HBM-streaming.
//
// The wave reads its row 256 columns at a time (16 bytes per lane, two loads in flight).  Lane p
// keeps the p-th largest 64-bit key seen so far, key = sortable(bits(score)) << 32 | (cols-1-col),
// so the lanes together hold a descending sorted list and lane K-1 holds the admission
// threshold.  Each score is first compared, as a float, against the threshold's score (one
// VALU compare; the test is conservative: ties, signed zeros and NaNs pass); only if some lane
// of the wave has a candidate are exact keys formed, and candidates beating the threshold key
// are inserted one at a time with a single-lane shift of the list.  Keys are unique per row,
// so the result is the unique top-k under the reference's order: descending score, equal
// scores lowest column first, +0.0 above -0.0, NaNs by bit pattern.  Unfilled slots keep key
// 0, which decodes to column cols-1, the reference's filler when cols < K.
#include "s3r_common.h"

namespace s3r {

__device__ __forceinline__ uint64_t readlane_u64(uint64_t v, int src) {
  uint32_t lo = __builtin_amdgcn_readlane((uint32_t)v, src);
  uint32_t hi = __builtin_amdgcn_readlane((uint32_t)(v >> 32), src);
  return ((uint64_t)hi << 32) | lo;
}

struct RowTopK {
  uint64_t mine;  // lane p: p-th largest key so far (0 = empty)
  uint64_t thr;   // key in lane K-1 (wave-uniform)
  float thr_f;    // its score; a NaN while the list is not full, so that "s < thr_f" is false for every s
  int K, lane;

  __device__ __forceinline__ void init(int k, int l) {
    mine = 0;
    thr = 0;
    thr_f = __uint_as_float(0xFFFFFFFFu);
    K = k;
    lane = l;
  }
  // value of x held by lane-1 (lane 0 receives its own): one DPP move per 32-bit half, no LDS crossbar
  static __device__ __forceinline__ uint64_t from_lane_below(uint64_t x) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp((int)(uint32_t)x, (int)(uint32_t)x, 0x138 /* wave_shr:1 */, 0xf, 0xf, false);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp((int)(uint32_t)(x >> 32), (int)(uint32_t)(x >> 32), 0x138, 0xf, 0xf, false);
    return ((uint64_t)hi << 32) | lo;
  }
  // candidates of the wave: lanes with cand set offer key `comp`; those that beat the threshold are inserted.
  // All 64 lanes hold list entries, so an insertion below position K-1 is harmless and needs no re-check.
  __device__ __forceinline__ void offer(bool cand, uint64_t comp) {
    uint64_t mask = __ballot(cand && comp > thr);
    while (mask) {
      const int src = __ffsll((unsigned long long)mask) - 1;
      mask &= mask - 1;
      const uint64_t c = readlane_u64(comp, src);
      const uint64_t up = from_lane_below(mine);
      if (mine < c) mine = (lane > 0 && up < c) ? up : c;
    }
    thr = readlane_u64(mine, K - 1);
    const uint32_t k32 = (uint32_t)(thr >> 32);
    thr_f = __uint_as_float(k32 ^ ((k32 & 0x80000000u) ? 0x80000000u : 0xFFFFFFFFu));
  }
};

__global__ __launch_bounds__(256) void topk_rows_kernel(const float* __restrict__ scores, int32_t* __restrict__ idx,
                                                        int64_t rows, int cols_all, int64_t row_stride, int K, int vec_ok,
                                                        int64_t causal_lq) {
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= rows) return;
  int cols = cols_all;
  if (causal_lq > 0) {  // the causal kernel's 64-row query block stops at end_n (flash_attention_topk.py:71)
    const int64_t end_n = ((w % causal_lq) / 64 + 1) * 64;
    if (end_n < cols) cols = (int)end_n;
  }
  const float* row = scores + w * row_stride;
  RowTopK st;
  st.init(K, lane);
  const uint32_t last = (uint32_t)(cols - 1);

  int c0 = 0;
  if (vec_ok) {
    // Segments of 4096 columns held in registers (16 x 16 bytes per lane, all loads in flight at once).
    // Before any exact work the segment yields a lower bound on the row's K-th largest score: the K-th largest
    // of the 64 per-lane maxima (64 distinct elements of the row), found by a ballot binary search on the
    // sortable keys.  Only scores at or above max(bound, list threshold) are offered to the list.
    constexpr int SEG = 16;
    for (; c0 < cols; c0 += SEG * 256) {
      float4 seg[SEG];
#pragma unroll
      for (int i = 0; i < SEG; i++) {
        const int col = c0 + (i * 64 + lane) * 4;
        seg[i] = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        if (col < cols) seg[i] = *reinterpret_cast<const float4*>(row + col);
      }
      // 256 groups (lane, component): group maxima over valid columns.  Neighbouring columns fall into different
      // groups, so a run of adjacent large scores still raises the bound.  fmaxf ignores NaNs and a group without
      // a valid finite entry reports -inf: the bound can only get lower, never wrong.
      float mx[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
      for (int i = 0; i < SEG; i++) {
        const int col = c0 + (i * 64 + lane) * 4;
        mx[0] = fmaxf(mx[0], seg[i].x);
        mx[1] = fmaxf(mx[1], col + 1 < cols ? seg[i].y : -INFINITY);
        mx[2] = fmaxf(mx[2], col + 2 < cols ? seg[i].z : -INFINITY);
        mx[3] = fmaxf(mx[3], col + 3 < cols ? seg[i].w : -INFINITY);
      }
      const uint32_t mk[4] = {sortable_key(mx[0]), sortable_key(mx[1]), sortable_key(mx[2]), sortable_key(mx[3])};
      uint32_t t = 0;  // K-th largest of the 256 group-maximum keys, by binary search on the key bits
      for (int bit = 31; bit >= 0; bit--) {
        const uint32_t cand = t | (1u << bit);
        const int cnt = __popcll(__ballot(mk[0] >= cand)) + __popcll(__ballot(mk[1] >= cand)) +
                        __popcll(__ballot(mk[2] >= cand)) + __popcll(__ballot(mk[3] >= cand));
        if (cnt >= K) t = cand;
      }
      const uint32_t tk = (uint32_t)(st.thr >> 32);
      const uint32_t fk = t > tk ? t : tk;  // filter key: never above the row's true K-th largest key
      float filt = __uint_as_float(fk ^ ((fk & 0x80000000u) ? 0x80000000u : 0xFFFFFFFFu));
      if (fk == 0) filt = __uint_as_float(0xFFFFFFFFu);
#pragma unroll
      for (int i = 0; i < SEG; i++) {
        const float v[4] = {seg[i].x, seg[i].y, seg[i].z, seg[i].w};
        const bool any = !(v[0] < filt) || !(v[1] < filt) || !(v[2] < filt) || !(v[3] < filt);
        if (__any(any)) {
          const int col = c0 + (i * 64 + lane) * 4;
#pragma unroll
          for (int j = 0; j < 4; j++) {
            const bool cand = !(v[j] < filt) && (col + j < cols);
            if (__any(cand)) st.offer(cand, ((uint64_t)sortable_key(v[j]) << 32) | (last - (uint32_t)(col + j)));
          }
        }
      }
    }
  }
  for (; c0 < cols; c0 += 64) {  // tail, or rows that cannot be read 16 bytes at a time
    const int col = c0 + lane;
    const bool valid = col < cols;
    const float s = valid ? row[col] : 0.f;
    const bool cand = valid && !(s < st.thr_f);
    if (__any(cand)) st.offer(cand, ((uint64_t)sortable_key(s) << 32) | (last - (uint32_t)col));
  }
  if (lane < K) idx[w * K + lane] = (int32_t)(last - (uint32_t)(st.mine & 0xffffffffu));
}

}  // namespace s3r

using namespace s3r;

namespace s3r {
int launch_topk_rows(const float* scores, int32_t* idx, int64_t rows, int cols, int64_t row_stride, int K, int64_t causal_lq,
                     void* stream) {
  if (!scores || !idx) return fail(S3R_ERR_BAD_ARG, "s3r_topk_rows: null pointer");
  if (rows <= 0 || cols <= 0 || row_stride < cols) return fail(S3R_ERR_BAD_ARG, "s3r_topk_rows: bad rows/cols/stride");
  if (K < 1 || K > 64) return fail(S3R_ERR_UNSUPPORTED, "s3r_topk_rows: K=%d outside [1,64]", K);
  const int64_t nwg = (rows + 3) / 4;
  if (nwg > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_topk_rows: too many rows");
  const int vec_ok = aligned16(scores) && (row_stride % 4 == 0);
  hipLaunchKernelGGL(topk_rows_kernel, dim3((unsigned)nwg), dim3(256), 0, (hipStream_t)stream, scores, idx, rows, cols,
                     row_stride, K, vec_ok, causal_lq);
  return check_launch("s3r_topk_rows");
}
}  // namespace s3r

extern "C" int s3r_topk_rows(const float* scores, int32_t* idx, int64_t rows, int cols, int64_t row_stride, int K,
                             void* stream) {
  return launch_topk_rows(scores, idx, rows, cols, row_stride, K, 0, stream);
}
