// Key-centric lists of the selection branch's index tensor, for the dK/dV kernel of the backward.
//
// Reference: count_query_fixedlen and reorder_topk_idx_fixedlen with the stable argsort between them
// (pi3/models/sparse_attn/topk_blocksparse_attention.py:423-554).  For every (b, h) and key block j the list
// holds the ids of the query blocks whose index row names j, one entry per occurrence, ascending; off[j] .. off[j+1]
// delimit it.  Entries of idx that are < 0 or >= nkb appear in no list.
//
// Five small kernels, no workspace besides the two outputs:
//   zero     off[*] = 0
//   count    histogram of the index entries, block j counted at off[j + 2] (pre-aggregated per workgroup in LDS)
//   scan     inclusive prefix sum per (b, h): off[j + 1] = first position of block j's list
//   fill     every entry takes a position with an atomic increment of off[j + 1], which thereby ends up at the END of
//            block j's list = the start of block j+1's: exactly the offsets array, off[0] = 0 included
//   sort     the atomic order is arbitrary, so each list is then sorted ascending, which makes the result unique
//            (equal ids are indistinguishable): lists of up to 512 entries by one wavefront in registers (rank by
//            counting), longer ones by one workgroup with Batcher's merge exchange, in LDS (up to 8192 entries) or
//            in place in global memory.
#include "s3r_common.h"

namespace s3r {
namespace kl {

constexpr int kLdsCap = 8192;

__global__ __launch_bounds__(256) void zero_kernel(int32_t* __restrict__ off, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) off[i] = 0;
}

// count and fill share one kernel body.  Neighbouring query blocks name mostly the same key blocks, and atomics on
// one address serialise in memory, so a workgroup first gathers its 1024 index entries in an LDS hash table (key
// block -> occurrences), every entry taking its rank among the workgroup's occurrences of its key block with an LDS
// atomic; one global atomic per DISTINCT key block then adds the count (count pass: at off[j + 2]) or reserves the
// positions (fill pass: at off[j + 1]), and in the fill pass every entry writes its query block at base + rank.
// A workgroup stays inside one (b, h): grid.y = B*H, grid.x = chunks of 1024 entries.
constexpr int kHashSlots = 2048;

template <bool FILL>
__global__ __launch_bounds__(1024) void gather_kernel(const int32_t* __restrict__ idx, int32_t* __restrict__ off, int32_t* __restrict__ list, int H,
                                                      int64_t nqb, int K, int64_t nkb, int64_t sib, int64_t sih, int64_t sim, int64_t list_stride) {
  __shared__ int32_t keys[kHashSlots];
  __shared__ int32_t cnt[kHashSlots];
  __shared__ int32_t base[kHashSlots];
  const int t = threadIdx.x;
  for (int i = t; i < kHashSlots; i += 1024) {
    keys[i] = -1;
    cnt[i] = 0;
  }
  __syncthreads();
  const int64_t bh = blockIdx.y;
  const int64_t hh = bh % H, bb = bh / H;
  const int64_t e = (int64_t)blockIdx.x * 1024 + t;  // entry within this (b, h)
  int32_t j = -1, m = 0;
  if (e < nqb * K) {
    m = (int32_t)(e / K);
    j = idx[bb * sib + hh * sih + (int64_t)m * sim + (e - (int64_t)m * K)];
    if (j < 0 || j >= nkb) j = -1;
  }
  int slot = 0, rank = 0;
  if (j >= 0) {
    slot = (int)(((uint32_t)j * 2654435761u) >> 21);  // 11 bits
    while (true) {
      const int32_t old = atomicCAS(&keys[slot], -1, j);
      if (old == -1 || old == j) break;
      slot = (slot + 1) & (kHashSlots - 1);  // at most 1024 keys in 2048 slots: a free slot exists
    }
    rank = atomicAdd(&cnt[slot], 1);
  }
  __syncthreads();
  for (int i = t; i < kHashSlots; i += 1024) {
    const int32_t kj = keys[i];
    if (kj >= 0) {
      if (FILL) base[i] = atomicAdd(off + bh * (nkb + 1) + kj + 1, cnt[i]);
      else if ((int64_t)kj + 2 <= nkb) atomicAdd(off + bh * (nkb + 1) + kj + 2, cnt[i]);  // the last block's count is not needed
    }
  }
  if (FILL) {
    __syncthreads();
    if (j >= 0) list[bh * list_stride + base[slot] + rank] = m;
  }
}

// one workgroup of 1024 per (b, h): in-place inclusive scan of n values
__global__ __launch_bounds__(1024) void scan_kernel(int32_t* __restrict__ off, int64_t n) {
  __shared__ int32_t part[1024];
  int32_t* a = off + (int64_t)blockIdx.x * n;
  const int t = threadIdx.x;
  const int64_t per = (n + 1023) / 1024;
  const int64_t lo = t * per, hi = lo + per < n ? lo + per : n;
  int32_t s = 0;
  for (int64_t i = lo; i < hi; i++) s += a[i];
  part[t] = s;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {  // Hillis-Steele over the 1024 partial sums
    const int32_t v = t >= d ? part[t - d] : 0;
    __syncthreads();
    part[t] += v;
    __syncthreads();
  }
  int32_t run = t > 0 ? part[t - 1] : 0;
  for (int64_t i = lo; i < hi; i++) {
    run += a[i];
    a[i] = run;
  }
}

// lists of 2 .. 64*M entries: one wavefront each, M entries per lane in registers; rank of an entry = entries below it
// + equal entries at lower positions.  Every entry is in a register before the first one is written back.
template <int M>
__device__ __forceinline__ void wave_rank_sort(int32_t* a, int n, int lane) {
  int32_t x[M];
  int rank[M];
#pragma unroll
  for (int r = 0; r < M; r++) {
    x[r] = 64 * r + lane < n ? a[64 * r + lane] : 0x7fffffff;
    rank[r] = 0;
  }
#pragma unroll
  for (int s = 0; s < M; s++) {
    const int cnt = n - 64 * s < 64 ? n - 64 * s : 64;  // entries held in register s
    for (int i = 0; i < cnt; i++) {
      const int32_t xi = __builtin_amdgcn_readlane(x[s], i);
#pragma unroll
      for (int r = 0; r < M; r++) rank[r] += (xi < x[r] || (xi == x[r] && 64 * s + i < 64 * r + lane)) ? 1 : 0;
    }
  }
#pragma unroll
  for (int r = 0; r < M; r++)
    if (64 * r + lane < n) a[rank[r]] = x[r];
}

constexpr int kWaveSortCap = 512;

__global__ __launch_bounds__(256) void sort_short_kernel(int32_t* __restrict__ list, const int32_t* __restrict__ off, int64_t nkb,
                                                         int64_t list_stride, int64_t nseg) {
  const int64_t seg = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 6;
  const int lane = threadIdx.x & 63;
  if (seg >= nseg) return;
  const int64_t bh = seg / nkb, j = seg - bh * nkb;
  const int32_t lo = off[bh * (nkb + 1) + j], hi = off[bh * (nkb + 1) + j + 1];
  const int n = __builtin_amdgcn_readfirstlane(hi - lo);
  if (n < 2 || n > kWaveSortCap) return;
  int32_t* a = list + bh * list_stride + lo;
  if (n <= 64) wave_rank_sort<1>(a, n, lane);
  else if (n <= 128) wave_rank_sort<2>(a, n, lane);
  else if (n <= 256) wave_rank_sort<4>(a, n, lane);
  else wave_rank_sort<8>(a, n, lane);
}

// Batcher's merge exchange (Knuth, TAOCP 3, algorithm 5.2.2M) on n entries, any n: per stage (p, k) the comparators
// (a, a + k) with (a - k mod p) mod 2k < k and a, a+k in the same block of 2p are disjoint; 256 threads share them.
template <typename P>
__device__ __forceinline__ void merge_exchange(P a, int n) {
  for (int lp = 0; (1 << lp) < n; lp++)  // p = 2^lp
    for (int lk = lp; lk >= 0; lk--) {   // k = 2^lk
      const int k = 1 << lk;
      const int kp = lk == lp ? 0 : k;  // k mod p
      for (int i = threadIdx.x; i < n - k; i += 256) {
        const int r = i - kp;
        if (r >= 0 && (r & (2 * k - 1)) < k && (i >> (lp + 1)) == ((i + k) >> (lp + 1))) {
          const int32_t u = a[i], v = a[i + k];
          if (u > v) {
            a[i] = v;
            a[i + k] = u;
          }
        }
      }
      __syncthreads();
    }
}

// lists beyond the wave sort: workgroup w looks at lists w, w + G, w + 2G, ... (long lists come in runs of
// neighbouring key blocks; the stride spreads a run over many workgroups) and sorts the long ones
__global__ __launch_bounds__(256) void sort_long_kernel(int32_t* __restrict__ list, const int32_t* __restrict__ off, int64_t nkb,
                                                        int64_t list_stride, int64_t nseg) {
  __shared__ int32_t stage[kLdsCap];
  __shared__ int64_t found[256];
  __shared__ int nfound;
  const int64_t G = gridDim.x;
  for (int64_t base = blockIdx.x; base < nseg; base += 256 * G) {
    if (threadIdx.x == 0) nfound = 0;
    __syncthreads();
    const int64_t seg = base + (int64_t)threadIdx.x * G;
    if (seg < nseg) {
      const int64_t bh = seg / nkb, j = seg - bh * nkb;
      if (off[bh * (nkb + 1) + j + 1] - off[bh * (nkb + 1) + j] > kWaveSortCap) found[atomicAdd(&nfound, 1)] = seg;
    }
    __syncthreads();
    const int nf = nfound;
    for (int f = 0; f < nf; f++) {
      const int64_t sg = found[f];
      const int64_t bh = sg / nkb, j = sg - bh * nkb;
      const int32_t lo = off[bh * (nkb + 1) + j];
      const int n = off[bh * (nkb + 1) + j + 1] - lo;
      int32_t* a = list + bh * list_stride + lo;
      if (n <= kLdsCap) {
        for (int i = threadIdx.x; i < n; i += 256) stage[i] = a[i];
        __syncthreads();
        merge_exchange(stage, n);
        for (int i = threadIdx.x; i < n; i += 256) a[i] = stage[i];
        __syncthreads();
      } else {
        merge_exchange(a, n);  // in place in global memory: __syncthreads orders the workgroup's accesses
      }
    }
    __syncthreads();
  }
}

}  // namespace kl

int launch_key_block_lists(const int32_t* idx, int32_t* kq_list, int32_t* kq_off, int B, int H, int64_t nqb, int K, int64_t nkb,
                           int64_t sib, int64_t sih, int64_t sim, int64_t list_stride, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  const int64_t bh = (int64_t)B * H;
  const int64_t noff = bh * (nkb + 1), total = bh * nqb * K, nseg = bh * nkb;
  const int64_t g_off = (noff + 255) / 256, g_ent = (total + 255) / 256, g_short = (nseg * 64 + 255) / 256;
  if (g_off > 0x7fffffffLL || g_ent > 0x7fffffffLL || g_short > 0x7fffffffLL || bh > 65535)
    return fail(S3R_ERR_UNSUPPORTED, "s3r_key_block_lists: tensor too large for one launch");
  hipLaunchKernelGGL(kl::zero_kernel, dim3((unsigned)g_off), dim3(256), 0, st, kq_off, noff);
  const dim3 g_gather((unsigned)((nqb * K + 1023) / 1024), (unsigned)bh);
  hipLaunchKernelGGL(kl::gather_kernel<false>, g_gather, dim3(1024), 0, st, idx, kq_off, kq_list, H, nqb, K, nkb, sib, sih, sim, list_stride);
  hipLaunchKernelGGL(kl::scan_kernel, dim3((unsigned)bh), dim3(1024), 0, st, kq_off, nkb + 1);
  hipLaunchKernelGGL(kl::gather_kernel<true>, g_gather, dim3(1024), 0, st, idx, kq_off, kq_list, H, nqb, K, nkb, sib, sih, sim, list_stride);
  hipLaunchKernelGGL(kl::sort_short_kernel, dim3((unsigned)g_short), dim3(256), 0, st, kq_list, kq_off, nkb, list_stride, nseg);
  const int64_t g_long = nseg < 4096 ? nseg : 4096;
  hipLaunchKernelGGL(kl::sort_long_kernel, dim3((unsigned)g_long), dim3(256), 0, st, kq_list, kq_off, nkb, list_stride, nseg);
  return check_launch("s3r_key_block_lists");
}

}  // namespace s3r
