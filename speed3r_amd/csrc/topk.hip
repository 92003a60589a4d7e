// Exact row-wise top-k of materialised fp32 scores: one wavefront per row.
//
// The wave streams its row 64 columns at a time.  Lane p keeps the p-th largest 64-bit key
// seen so far, key = sortable(bits(score)) << 32 | (cols-1-col), so the lanes together hold a
// descending sorted list and lane K-1 holds the admission threshold.  A column enters only
// if its key beats the threshold (one ballot per 64 columns); survivors are inserted one at
// a time with a single-lane shift of the list.  Keys are unique per row, so the result is
// the unique top-k under the reference's order: descending score, equal scores lowest
// column first, +0.0 above -0.0, NaNs by bit pattern.  Unfilled slots keep key 0, which
// decodes to column cols-1, the reference's filler when cols < K.
#include "s3r_common.h"

namespace s3r {

__device__ __forceinline__ uint64_t readlane_u64(uint64_t v, int src) {
  uint32_t lo = __builtin_amdgcn_readlane((uint32_t)v, src);
  uint32_t hi = __builtin_amdgcn_readlane((uint32_t)(v >> 32), src);
  return ((uint64_t)hi << 32) | lo;
}

// Insert key c (wave-uniform) into the descending list held one entry per lane.
__device__ __forceinline__ void list_insert(uint64_t& mine, uint64_t c, int lane) {
  const uint64_t up = __shfl_up(mine, 1);
  if (mine < c) mine = (lane > 0 && up < c) ? up : c;
}

__global__ __launch_bounds__(256) void topk_rows_kernel(const float* __restrict__ scores, int32_t* __restrict__ idx,
                                                        int64_t rows, int cols, int64_t row_stride, int K) {
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= rows) return;
  const float* row = scores + w * row_stride;
  uint64_t mine = 0;
  uint64_t thr = 0;
  for (int c0 = 0; c0 < cols; c0 += 64) {
    const int col = c0 + lane;
    uint64_t comp = 0;
    if (col < cols) comp = ((uint64_t)sortable_key(row[col]) << 32) | (uint32_t)(cols - 1 - col);
    uint64_t mask = __ballot(comp > thr);
    while (mask) {
      const int src = __ffsll((unsigned long long)mask) - 1;
      mask &= mask - 1;
      const uint64_t c = readlane_u64(comp, src);
      if (c > thr) {
        list_insert(mine, c, lane);
        thr = readlane_u64(mine, K - 1);
      }
    }
  }
  if (lane < K) idx[w * K + lane] = (int32_t)((uint32_t)(cols - 1) - (uint32_t)(mine & 0xffffffffu));
}

}  // namespace s3r

using namespace s3r;

extern "C" int s3r_topk_rows(const float* scores, int32_t* idx, int64_t rows, int cols, int64_t row_stride, int K,
                             void* stream) {
  if (!scores || !idx) return fail(S3R_ERR_BAD_ARG, "s3r_topk_rows: null pointer");
  if (rows <= 0 || cols <= 0 || row_stride < cols) return fail(S3R_ERR_BAD_ARG, "s3r_topk_rows: bad rows/cols/stride");
  if (K < 1 || K > 64) return fail(S3R_ERR_UNSUPPORTED, "s3r_topk_rows: K=%d outside [1,64]", K);
  const int64_t nwg = (rows + 3) / 4;
  if (nwg > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_topk_rows: too many rows");
  hipLaunchKernelGGL(topk_rows_kernel, dim3((unsigned)nwg), dim3(256), 0, (hipStream_t)stream, scores, idx, rows, cols,
                     row_stride, K);
  return check_launch("s3r_topk_rows");
}
