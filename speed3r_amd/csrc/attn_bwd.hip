// Backward of the two attention operators on the gfx950 matrix cores (bf16 / fp16 I/O, block 64, head_dim 64).
//
// Reference: _topk_blocksparse_attention_bwd with backward_sum_o_do, backward_dkdv, backward_dq
// (pi3/models/sparse_attn/topk_blocksparse_attention.py:132-170,558-712,722-850,907-1038) for the selection
// branch and _flash_attn_backward (pi3/models/sparse_attn/flash_attention_topk.py:204-630) for the compressed
// branch, which is the same computation over ALL key tiles (DENSE below).  With P = exp(scale*S - lse) recomputed
// from the forward's log-sum-exp and delta = rowsum(dO * O):
//   dV = P^T dO          dP = dO V^T          dS = scale * P * (dP - delta)          dQ = dS K          dK = dS^T Q
// P (for dV) and dS (for dQ, dK) are rounded to the I/O dtype before the products, accumulation is fp32
// (reference :683-690, :826-838).
//
// Three kernels:
//   * bwd_delta_kernel: delta[b,h,n] = sum_d o * dO in fp32 (HBM bound).
//   * bwd_dq_kernel: one wavefront per 64-row query block, four independent waves per workgroup; walks the block's
//     selected key tiles (or all of them).  Everything is computed transposed, as in the forward kernels:
//     S^T = K Q^T and dP^T = V dO^T put one QUERY per lane, so lse and delta are per-lane scalars;
//     dQ^T += K^T dS^T takes K^T fragments from ds_read_b64_tr_b16.  K and V half tiles (32 keys) go global -> LDS
//     by direct transfers, double buffered (16 KB per wave).  The K half is staged once, in a layout that serves
//     the transposed reads and the row reads (A operand of S^T) without bank conflicts.
//   * bwd_dkdv_kernel: one workgroup of two waves per 64-key block, each wave owns 32 keys (one KEY per lane:
//     S = Q K^T, dP = dO V^T with K, V fragments in registers as B operands) and walks the query blocks that
//     selected the key block (key-centric lists built by the host from the index tensor, reference :423-554).
//     Q and dO tiles (64 queries) and the matching lse / delta values go global -> LDS, shared by the two waves,
//     double buffered (the next tile's transfers fly during a whole tile of work), one barrier per tile;
//     dV^T += dO^T P and dK^T += Q^T dS read their A operands transposed from the same buffers.
// Query rows beyond Lq have lse = +inf (P = 0), keys beyond Lk are masked (P = 0); rows past the end of a tensor are
// never read (transfers re-read the last valid row).
//
// 16-token blocks (BLK = 16, the reference layer's own block size) run through the same kernels: a 32-row half tile
// is then two 16-row blocks, and neighbouring blocks name mostly the same partners, so both kernels walk UNIONS of
// lists (distinct blocks from a 512-slot hash table in LDS, with a count byte per list: how often that list names the
// block; a product's quadrant whose count is 0 gets P = 0, one listed twice counts twice).  dQ kernel: the union of
// the index rows of the wave's four query blocks, two distinct key blocks per half tile against all 64 queries.
// dK/dV kernel: the workgroup's 64 keys are four neighbouring key blocks; it walks the union of their four
// query-block lists, four entries per 64-row tile, with the tile code of the 64-token blocks; the union is built a
// chunk of the (ascending) lists at a time.
#include "select_common.h"
#include "attn_bwd.h"

namespace s3r {
namespace bwd {
using namespace sel;

constexpr int kHalfBytes = 32 * 128;  // one half tile: 32 rows of 64 two-byte values
// dK/dV at 16-token blocks: list entries per chunk of the union of four neighbouring key blocks' lists (a quarter from
// each list; the union's hash table has 512 slots)
constexpr int kMergeMax = 384;
constexpr float kLog2e = 1.4426950408889634f;

typedef std::integral_constant<int, 0> H0;
typedef std::integral_constant<int, 1> H1;

// ---- delta ---------------------------------------------------------------------------------------------------
template <typename E>
__global__ __launch_bounds__(256) void bwd_delta_kernel(const E* __restrict__ o, const E* __restrict__ dout, float* __restrict__ delta,
                                                         int H, int64_t N, int64_t rows, int64_t sob, int64_t soh, int64_t son,
                                                         int64_t sdb, int64_t sdh, int64_t sdn) {
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = gid >> 3;  // 8 lanes of 16 bytes per 64-value row
  const int part = (int)(gid & 7);
  const bool live = row < rows;
  const int64_t rr = live ? row : rows - 1;
  const int64_t n = rr % N, bh = rr / N;
  const int h = (int)(bh % H);
  const int64_t b = bh / H;
  // both tensors are streamed once: non-temporal loads
  const u32x4 a = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(o + b * sob + h * soh + n * son + part * 8));
  const u32x4 g = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(dout + b * sdb + h * sdh + n * sdn + part * 8));
  const E* ae = reinterpret_cast<const E*>(&a);
  const E* ge = reinterpret_cast<const E*>(&g);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) s += (float)ae[i] * (float)ge[i];
#pragma unroll
  for (int off = 1; off < 8; off <<= 1) s += __shfl_xor(s, off);
  if (live && part == 0) delta[rr] = s;
}

// ---- shared pieces of the two MFMA kernels -----------------------------------------------------------------------
// Transfer of rows [8*i0*.., ...) of a 32-row half tile: instruction i moves rows 8i .. 8i+7 (16 bytes per lane).
// LDS chunk (row, c') holds head_dim chunk c' ^ k_swizzle(row) in every tile: 16-byte row reads and
// ds_read_b64_tr_b16 reads both run without bank conflicts with it.  (VSW marks the tiles that are also read
// transposed; the map is the same.)  Rows are clamped to `last` (relative to `base`'s row 0).
template <typename E, bool VSW>
__device__ __forceinline__ void dma_rows(const E* base, uint32_t rowbytes, int first_row, int last, char* lds_half, int lane, int i_begin, int i_end) {
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, 0x7fffffff, 0x00020000);
  const int lr = lane >> 3;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    if (i >= i_begin && i < i_end) {
      const int ldsrow = 8 * i + lr;
      int row = first_row + ldsrow;
      row = row < last ? row : last;
      const int chunk = (lane & 7) ^ k_swizzle(ldsrow);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)(lds_half + i * 1024), 16,
                                               (uint32_t)row * rowbytes + (uint32_t)(chunk * 16), 0, 0, 0);
    }
  }
}

// The same for a half tile made of two 16-row blocks: instructions 0, 1 move block A, 2, 3 block B; rows are clamped
// to last_a / last_b (relative to the block's first row).
template <typename E, bool VSW>
__device__ __forceinline__ void dma_rows16(const E* base_a, const E* base_b, uint32_t rowbytes, int last_a, int last_b, char* lds_half, int lane) {
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)base_a, 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void*)base_b, 0, 0x7fffffff, 0x00020000);
  const int lr = lane >> 3;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int ldsrow = 8 * i + lr;
    const int last = i < 2 ? last_a : last_b;
    int row = ldsrow & 15;
    row = row < last ? row : last;
    const int chunk = (lane & 7) ^ k_swizzle(ldsrow);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(i < 2 ? ra : rb, (__attribute__((address_space(3))) void*)(lds_half + i * 1024), 16,
                                             (uint32_t)row * rowbytes + (uint32_t)(chunk * 16), 0, 0, 0);
  }
}

// A operand from row reads of a half tile: lane = row c, k-step ks: head_dim chunk 2ks + hh.
template <typename E, bool VSW>
__device__ __forceinline__ void read_rows(const char* half, int c, int hh, typename Mma<E>::V8 (&dst)[4]) {
  const int sw = k_swizzle(c);
#pragma unroll
  for (int ks = 0; ks < 4; ks++) {
    Frag f;
    f.u = *reinterpret_cast<const uint4*>(half + c * 128 + (((2 * ks + hh) ^ sw) << 4));
    dst[ks] = as_v8<E>(f);
  }
}

template <typename E, bool VSW>
__device__ __forceinline__ typename Mma<E>::V8 read_row_frag(const char* half, int c, int hh, int ks) {
  const int sw = k_swizzle(c);
  Frag f;
  f.u = *reinterpret_cast<const uint4*>(half + c * 128 + (((2 * ks + hh) ^ sw) << 4));
  return as_v8<E>(f);
}

// A operand X^T from transposed reads of a half tile staged with VSW: fragment [jj][dt] holds, for head_dim row
// dt*32 + c, the 8 rows 16jj + {4hh..4hh+3, 8+4hh..8+4hh+3} of the half: the order in which a 32x32 accumulator
// with one column per lane hands over its registers 8jj .. 8jj+7.
template <typename E>
__device__ __forceinline__ void read_transposed(const char* half, int tr_off, typename Mma<E>::V8 (&dst)[2][2]) {
#pragma unroll
  for (int jj = 0; jj < 2; jj++)
#pragma unroll
    for (int dt = 0; dt < 2; dt++) {
      const char* a0 = half + (tr_off ^ (dt * 64)) + (jj * 16) * 128;
      const char* a8 = half + (tr_off ^ (dt * 64) ^ (k_swizzle(8) << 4)) + (jj * 16 + 8) * 128;  // rows 8 further down: chunk map ^ k_swizzle(8)
      Frag f;
      f.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
      f.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a8));
      dst[jj][dt] = as_v8<E>(f);
    }
}

template <typename E>
__device__ __forceinline__ typename Mma<E>::V8 read_transposed_frag(const char* half, int tr_off, int jj, int dt) {
  const char* a0 = half + (tr_off ^ (dt * 64)) + (jj * 16) * 128;
  const char* a8 = half + (tr_off ^ (dt * 64) ^ (k_swizzle(8) << 4)) + (jj * 16 + 8) * 128;
  Frag f;
  f.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
  f.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a8));
  return as_v8<E>(f);
}

// The same reads written by hand, each group one asm statement that ends with its own wait: the compiler neither sees an
// LDS access nor adds a wait of its own, and no register of an outstanding read is left to the register allocator.  A
// compiler-visible LDS read that follows direct transfers into LDS makes the compiler wait for every transfer that it
// cannot tell apart from the buffer being read, here also those of the NEXT half tile, which have just been issued.
// Row fragments of two half tiles (K and V, or Q and dO): lane = row c, k-step ks: head_dim chunk 2ks + hh.
__device__ __forceinline__ void read_rows2_sync(const char* half_a, const char* half_b, int c, int hh, u32x4 (&a)[4], u32x4 (&b)[4]) {
  // one address per tile: row and the chunk of k-step 0; the k-step flips chunk bits 1..2 (tiles are 1 KB aligned).
  // The empty asm keeps the eight addresses from being computed ahead of the loop and held in registers.
  const uint32_t off = (uint32_t)(c * 128 + ((hh ^ k_swizzle(c)) << 4));
  uint32_t a0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)half_a + off;
  uint32_t b0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)half_b + off;
  asm volatile("" : "+v"(a0), "+v"(b0));
  asm volatile(
      "ds_read_b128 %0, %8\n\tds_read_b128 %1, %9\n\tds_read_b128 %2, %10\n\tds_read_b128 %3, %11\n\t"
      "ds_read_b128 %4, %12\n\tds_read_b128 %5, %13\n\tds_read_b128 %6, %14\n\tds_read_b128 %7, %15\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(a[0]), "=&v"(a[1]), "=&v"(a[2]), "=&v"(a[3]), "=&v"(b[0]), "=&v"(b[1]), "=&v"(b[2]), "=&v"(b[3])
      : "v"(a0), "v"(a0 ^ 32u), "v"(a0 ^ 64u), "v"(a0 ^ 96u), "v"(b0), "v"(b0 ^ 32u), "v"(b0 ^ 64u), "v"(b0 ^ 96u)
      : "memory");
}
// Transposed fragments of one half tile: dst[jj][dt][rows 0-7 | 8-15 of the 16-row group jj].
__device__ __forceinline__ void read_transposed_sync(const char* half, int tr_off, u32x2 (&dst)[2][2][2]) {
  uint32_t t0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)half + (uint32_t)tr_off;
  asm volatile("" : "+v"(t0));
  const uint32_t t8 = t0 ^ (uint32_t)(k_swizzle(8) << 4);  // rows 8 further down: chunk map ^ k_swizzle(8)
  asm volatile(
      "ds_read_b64_tr_b16 %0, %8\n\tds_read_b64_tr_b16 %1, %10 offset:1024\n\t"
      "ds_read_b64_tr_b16 %2, %9\n\tds_read_b64_tr_b16 %3, %11 offset:1024\n\t"
      "ds_read_b64_tr_b16 %4, %8 offset:2048\n\tds_read_b64_tr_b16 %5, %10 offset:3072\n\t"
      "ds_read_b64_tr_b16 %6, %9 offset:2048\n\tds_read_b64_tr_b16 %7, %11 offset:3072\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(dst[0][0][0]), "=&v"(dst[0][0][1]), "=&v"(dst[0][1][0]), "=&v"(dst[0][1][1]), "=&v"(dst[1][0][0]), "=&v"(dst[1][0][1]),
        "=&v"(dst[1][1][0]), "=&v"(dst[1][1][1])
      : "v"(t0), "v"(t0 ^ 64u), "v"(t8), "v"(t8 ^ 64u)
      : "memory");
}
template <typename E> __device__ __forceinline__ typename Mma<E>::V8 frag_of(u32x4 w) {
  Frag f;
  f.u = make_uint4(w[0], w[1], w[2], w[3]);
  return as_v8<E>(f);
}
template <typename E> __device__ __forceinline__ typename Mma<E>::V8 frag_of(u32x2 lo, u32x2 hi) {
  Frag f;
  f.u = make_uint4(lo[0], lo[1], hi[0], hi[1]);
  return as_v8<E>(f);
}

__device__ __forceinline__ int tr_offset(int lane) {
  const int hh = lane >> 5;
  const int i16 = lane & 15;
  const int tr_row = 4 * hh + (i16 >> 2);
  const int tr_chunk = (((lane >> 4) & 1) * 2 + ((i16 & 3) >> 1)) ^ k_swizzle(tr_row);
  return tr_row * 128 + tr_chunk * 16 + (i16 & 1) * 8;
}

// Store of a transposed 64 x 64 accumulator pair acc[dt] (lane = row of the output, registers = head_dim values
// dt*32 + 8*(r/4) + 4*hh + r%4): one exchange with lane ^ 32 per packed word gives every lane 8 consecutive values.
template <typename E>
__device__ __forceinline__ void store_rows(const f32x16 (&acc)[2], E* rowptr, bool live, int hh) {
#pragma unroll
  for (int dt = 0; dt < 2; dt++)
#pragma unroll
    for (int gp = 0; gp < 2; gp++) {
      union { E e[8]; uint32_t w[4]; uint4 u; } pc;
      union { E e[2]; uint32_t w; } t;
#pragma unroll
      for (int wi = 0; wi < 2; wi++) {
        t.e[0] = (E)acc[dt][8 * gp + 2 * wi];
        t.e[1] = (E)acc[dt][8 * gp + 2 * wi + 1];
        const uint32_t a = t.w;
        t.e[0] = (E)acc[dt][8 * gp + 4 + 2 * wi];
        t.e[1] = (E)acc[dt][8 * gp + 4 + 2 * wi + 1];
        const uint32_t bw = t.w;
        const auto r = __builtin_amdgcn_permlane32_swap(a, bw, false, false);
        pc.w[wi] = r[0];
        pc.w[2 + wi] = r[1];
      }
      if (live) *reinterpret_cast<uint4*>(rowptr + dt * 32 + 8 * (2 * gp + hh)) = pc.u;
    }
}

// ---- dQ ----------------------------------------------------------------------------------------------------------
template <typename E, bool DENSE, int BLK>
__global__ __launch_bounds__(256, 2) void bwd_dq_kernel(BwdParams p, int nqb, int nqg, int total_wg) {
  typedef typename Mma<E>::V8 V8;
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[4 * kHalfBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[4 * kHalfBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[4 * kHalfBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v1[4 * kHalfBytes];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int hh = lane >> 5;
  const int c = lane & 31;

  const int w = blockIdx.x;  // workgroup w -> work item: each XCD walks a contiguous range of query blocks of one head
  const int xcd = w & 7, slot = w >> 3;
  const int per = total_wg >> 3, rem = total_wg & 7;
  const int vid = xcd * per + (xcd < rem ? xcd : rem) + slot;
  const int bh = vid / nqg;
  const int qg = vid - bh * nqg;
  const int b = bh / p.H;
  const int h = bh - b * p.H;
  const int qb = qg * 4 + wave;
  if (qb >= nqb) return;

  const int64_t Lq = p.Lq, Lk = p.Lk;
  const int64_t q0 = (int64_t)qb * 64;
  const E* qp = (const E*)p.q + (int64_t)b * p.sqb + (int64_t)h * p.sqh;
  const E* kp = (const E*)p.k + (int64_t)b * p.skb + (int64_t)h * p.skh;
  const E* vp = (const E*)p.v + (int64_t)b * p.svb + (int64_t)h * p.svh;
  const E* gp = (const E*)p.dout + (int64_t)b * p.sgb + (int64_t)h * p.sgh;
  const float* lsep = p.lse + ((int64_t)b * p.H + h) * Lq;
  const float* dlp = p.delta + ((int64_t)b * p.H + h) * Lq;

  char* k_buf[2] = {reinterpret_cast<char*>(lds_k0) + wave * kHalfBytes, reinterpret_cast<char*>(lds_k1) + wave * kHalfBytes};
  char* v_buf[2] = {reinterpret_cast<char*>(lds_v0) + wave * kHalfBytes, reinterpret_cast<char*>(lds_v1) + wave * kHalfBytes};

  // B operands Q and dO (lane = query row, head_dim chunk hh + 2 ks), per-query lse (base 2) and delta
  V8 bq[2][4], bg[2][4];
  float lse2[2], dlts[2];  // log-sum-exp in base 2, delta times the softmax scale
#pragma unroll
  for (int qt = 0; qt < 2; qt++) {
    const int64_t row = q0 + qt * 32 + c;
    const bool live = row < Lq;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      Frag f, g;
      f.u = make_uint4(0, 0, 0, 0);
      g.u = make_uint4(0, 0, 0, 0);
      if (live) {
        f.u = *reinterpret_cast<const uint4*>(qp + row * p.sqm + ks * 16 + hh * 8);
        g.u = *reinterpret_cast<const uint4*>(gp + row * p.sgm + ks * 16 + hh * 8);
      }
      bq[qt][ks] = as_v8<E>(f);
      bg[qt][ks] = as_v8<E>(g);
    }
    lse2[qt] = live ? lsep[row] * kLog2e : INFINITY;
    dlts[qt] = live ? dlp[row] * p.scale : 0.f;
  }
  f32x16 dqt[2][2];  // dQ^T accumulators [qt][dt]: lane = query, registers = head_dim
#pragma unroll
  for (int qt = 0; qt < 2; qt++)
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
      for (int r = 0; r < 16; r++) dqt[qt][dt][r] = 0.f;

  // key tiles of this query block
  static_assert(BLK == 64 || (BLK == 16 && !DENSE), "blocks of 64 tokens, or of 16 with an index list");
  int32_t my_idx = -1;
  uint64_t todo = 0;
  int ntiles;
  int dense_next = 0;
  // BLK 16: the wave's 64 queries are four query blocks with a list each; neighbouring lists name mostly the same key
  // blocks, so the wave walks the UNION of the four lists.  Entry n of the walk list (LDS) is a distinct key block and
  // four count bytes (how often query block j lists it; 0: not at all, above 1: a duplicated entry, which weighs the
  // block that often, as the forward pass does).  A tile is four entries: two per 32-key half.
  __shared__ __attribute__((aligned(16))) int2 lds_walk[BLK == 16 ? 4 : 1][BLK == 16 ? 264 : 1];
  int2* const walk = lds_walk[BLK == 16 ? wave : 0];
  int n_union = 0;
  bool dup = false;  // some list names a block more than once (wave-uniform)
  if constexpr (DENSE) {
    ntiles = (int)((Lk + 63) >> 6);
  } else if constexpr (BLK == 64) {
    const int32_t* idx_row = p.idx + (int64_t)b * p.sib + (int64_t)h * p.sih + (int64_t)qb * p.sim;
    my_idx = lane < p.K ? idx_row[lane] : -1;
    todo = __ballot(my_idx >= 0 && (int64_t)my_idx * 64 < Lk);
    ntiles = __popcll(todo);
  } else {
    const int64_t nqb16 = (Lq + 15) >> 4;
    int32_t my16[4] = {-1, -1, -1, -1};  // entry `lane` of the four lists
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const int64_t qb16 = (int64_t)qb * 4 + s;
      if (qb16 < nqb16 && lane < p.K) {
        const int32_t v = (p.idx + (int64_t)b * p.sib + (int64_t)h * p.sih + qb16 * p.sim)[lane];
        my16[s] = (v >= 0 && (int64_t)v * 16 < Lk) ? v : -1;
      }
    }
    // Distinct blocks and their counts through a hash table in LDS (512 slots in this wave's first K buffer, which no
    // transfer touches before the list is complete): every lane inserts its entry of list j with a compare-and-swap on
    // the key (linear probing; at most 4 x 64 distinct blocks) and adds 1 << 8j to the slot's count; the occupied
    // slots are then compacted into the list, eight slots per lane, positions from ballots.
    int32_t* const hkey = reinterpret_cast<int32_t*>(k_buf[0]);          // [512]
    uint32_t* const hcnt = reinterpret_cast<uint32_t*>(k_buf[0] + 2048);  // [512]
    reinterpret_cast<int4*>(hkey)[lane] = make_int4(-1, -1, -1, -1);
    reinterpret_cast<int4*>(hkey)[lane + 64] = make_int4(-1, -1, -1, -1);
    reinterpret_cast<int4*>(hcnt)[lane] = make_int4(0, 0, 0, 0);
    reinterpret_cast<int4*>(hcnt)[lane + 64] = make_int4(0, 0, 0, 0);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int32_t e = my16[j];
      bool active = e >= 0;
      uint32_t slot = ((uint32_t)e * 0x9E3779B1u) >> 23;
      while (active) {
        const int32_t old = atomicCAS(hkey + slot, -1, e);
        if (old == -1 || old == e) {
          atomicAdd(hcnt + slot, 1u << (8 * j));
          active = false;
        } else {
          slot = (slot + 1) & 511u;
        }
      }
    }
    const int4 k0 = reinterpret_cast<const int4*>(hkey)[2 * lane], k1 = reinterpret_cast<const int4*>(hkey)[2 * lane + 1];
    const int4 c0 = reinterpret_cast<const int4*>(hcnt)[2 * lane], c1 = reinterpret_cast<const int4*>(hcnt)[2 * lane + 1];
    const int32_t ks8[8] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};
    const int32_t cs8[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
    uint32_t pos = 0;  // occupied slots of the lanes below
    uint32_t cnt_bits = 0;
#pragma unroll
    for (int s8 = 0; s8 < 8; s8++) {
      const uint64_t m = __ballot(ks8[s8] >= 0);
      pos = __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, pos));
      n_union += __popcll(m);
      cnt_bits |= (uint32_t)cs8[s8];
    }
#pragma unroll
    for (int s8 = 0; s8 < 8; s8++)
      if (ks8[s8] >= 0) walk[pos++] = make_int2(ks8[s8], cs8[s8]);
    if (lane < 4) walk[n_union + lane] = make_int2(-1, 0);  // the last tile's missing entries
    dup = __any((cnt_bits & 0xfefefefeu) != 0);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the table is read and the list written before the first transfer
    ntiles = (n_union + 3) >> 2;
  }
  auto pop = [&]() -> int64_t {  // start row of the next tile, BLK 16: its list position (callers pop exactly ntiles times)
    if constexpr (DENSE) {
      return (int64_t)(dense_next++) * 64;
    } else if constexpr (BLK == 64) {
      const int t = __ffsll((unsigned long long)todo) - 1;
      todo &= todo - 1;
      return (int64_t)__builtin_amdgcn_readlane(my_idx, t) * 64;
    } else {
      return (int64_t)(dense_next++);
    }
  };
  // BLK 16: the four entries (key block, four count bytes; -1: none) of the tile being computed and of the tile whose
  // first half is fetched meanwhile, read from the walk list once per tile (a hand-written read, like the fragments')
  // and kept in scalar registers
  struct Entries16 { int32_t blk[4] = {-1, -1, -1, -1}; uint32_t cnt[4] = {0, 0, 0, 0}; };
  struct NoEntries {};
  typedef std::conditional_t<BLK == 16, Entries16, NoEntries> TileEntries;
  TileEntries ent_cur, ent_nxt;
  auto read_entries = [&](int64_t t, Entries16& e) {
    const uint32_t a = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)reinterpret_cast<const char*>(walk + 4 * t);
    u32x4 v0, v1;
    asm volatile("ds_read_b128 %0, %2\n\tds_read_b128 %1, %2 offset:16\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v0), "=&v"(v1) : "v"(a));
    e.blk[0] = __builtin_amdgcn_readfirstlane((int32_t)v0[0]); e.cnt[0] = (uint32_t)__builtin_amdgcn_readfirstlane((int32_t)v0[1]);
    e.blk[1] = __builtin_amdgcn_readfirstlane((int32_t)v0[2]); e.cnt[1] = (uint32_t)__builtin_amdgcn_readfirstlane((int32_t)v0[3]);
    e.blk[2] = __builtin_amdgcn_readfirstlane((int32_t)v1[0]); e.cnt[2] = (uint32_t)__builtin_amdgcn_readfirstlane((int32_t)v1[1]);
    e.blk[3] = __builtin_amdgcn_readfirstlane((int32_t)v1[2]); e.cnt[3] = (uint32_t)__builtin_amdgcn_readfirstlane((int32_t)v1[3]);
  };
  // first key row, number of valid rows and the count bytes of entry `s` (0..3) of a tile (none: row 0, no counts)
  auto sub_block = [&](const Entries16& e, int s, int64_t& start, int& nv, uint32_t& counts) {
    const int32_t blk = e.blk[s];
    counts = e.cnt[s];
    start = blk >= 0 ? (int64_t)blk * 16 : 0;
    nv = blk >= 0 ? (int)(Lk - start < 16 ? Lk - start : 16) : 0;
  };

  const float scale = p.scale;
  const float sl2 = scale * kLog2e;
  const uint32_t krow = (uint32_t)p.skn * (uint32_t)sizeof(E), vrow = (uint32_t)p.svn * (uint32_t)sizeof(E);
  const int tr_off = tr_offset(lane);

  auto fetch = [&](int64_t start, auto hf, int buf, const TileEntries& ent) {  // half HF of the tile at `start` -> buffers `buf`
    constexpr int HF = decltype(hf)::value;
    if constexpr (BLK == 64) {
      const int last = (int)((Lk - start < 64 ? Lk - start : 64) - 1);
      dma_rows<E, true>(kp + start * p.skn, krow, 32 * HF, last, k_buf[buf], lane, 0, 4);
      dma_rows<E, false>(vp + start * p.svn, vrow, 32 * HF, last, v_buf[buf], lane, 0, 4);
    } else {
      int64_t sa, sb;
      int na, nb;
      uint32_t ca, cb;
      sub_block(ent, 2 * HF, sa, na, ca);
      sub_block(ent, 2 * HF + 1, sb, nb, cb);
      const int la = na > 0 ? na - 1 : 0, lb = nb > 0 ? nb - 1 : 0;
      dma_rows16<E, true>(kp + sa * p.skn, kp + sb * p.skn, krow, la, lb, k_buf[buf], lane);
      dma_rows16<E, false>(vp + sa * p.svn, vp + sb * p.svn, vrow, la, lb, v_buf[buf], lane);
    }
  };
  auto compute = [&](int64_t start, auto hf, int buf, const TileEntries& ent) {
    constexpr int HF = decltype(hf)::value;
    int nvalid = 64;
    int na = 16, nb = 16;      // BLK 16: valid keys of the half's two blocks A (rows 0..15) and B (16..31)
    uint32_t ca = 0, cb = 0;   // and how often each of the four query blocks lists them
    if constexpr (BLK == 64) {
      nvalid = (int)(Lk - start < 64 ? Lk - start : 64);
    } else {
      int64_t sa, sb;
      sub_block(ent, 2 * HF, sa, na, ca);
      sub_block(ent, 2 * HF + 1, sb, nb, cb);
    }
    const bool ragged = nvalid < 64;
    V8 ak[4], av[4];
    {
      u32x4 kw[4], vw[4];
      read_rows2_sync(k_buf[buf], v_buf[buf], c, hh, kw, vw);
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        ak[ks] = frag_of<E>(kw[ks]);
        av[ks] = frag_of<E>(vw[ks]);
      }
    }
    V8 ds[2][2];  // dS^T as B operand [qt][jj]
    constexpr int QT0 = 0, QT1 = 2;
#pragma unroll
    for (int qt = QT0; qt < QT1; qt++) {
      f32x16 st, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) { st[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < 4; ks++) st = Mma<E>::mma(ak[ks], bq[qt][ks], st);
#pragma unroll
      for (int ks = 0; ks < 4; ks++) dp = Mma<E>::mma(av[ks], bg[qt][ks], dp);
      if constexpr (BLK == 64) {
#pragma unroll
        for (int r = 0; r < 16; r++) st[r] = __builtin_amdgcn_exp2f(fmaf(st[r], sl2, -lse2[qt]));  // P^T
        if (ragged) {  // keys beyond Lk carry no probability
#pragma unroll
          for (int r = 0; r < 16; r++)
            if (32 * HF + 4 * hh + 8 * (r >> 2) + (r & 3) >= nvalid) st[r] = 0.f;
        }
      } else {
        // registers 0..7 are keys of block A, 8..15 of block B; this lane's query block lists each 0, 1 or more times,
        // and a probability counts that often: the count goes into the exponent (lse - log2(count); 0 times: +inf),
        // two values per lane instead of a test per score
        const int sh = 8 * (2 * qt + (c >> 4));
        const uint32_t wa = (ca >> sh) & 0xffu, wb = (cb >> sh) & 0xffu;
        float la = wa != 0 ? lse2[qt] : INFINITY, lb = wb != 0 ? lse2[qt] : INFINITY;
        if (dup) {
          la -= __builtin_amdgcn_logf((float)(wa > 1 ? wa : 1));
          lb -= __builtin_amdgcn_logf((float)(wb > 1 ? wb : 1));
        }
#pragma unroll
        for (int r = 0; r < 16; r++) st[r] = __builtin_amdgcn_exp2f(fmaf(st[r], sl2, -(r < 8 ? la : lb)));  // P^T
        if (na < 16 || nb < 16) {  // (wave-uniform) a block cut short by the end of the sequence, or none
#pragma unroll
          for (int r = 0; r < 16; r++)
            if (4 * hh + 8 * ((r >> 2) & 1) + (r & 3) >= (r < 8 ? na : nb)) st[r] = 0.f;
        }
      }
#pragma unroll
      for (int r = 0; r < 16; r++) ds[qt][r >> 3][r & 7] = (E)(st[r] * fmaf(dp[r], scale, -dlts[qt]));  // scale * P * (dP - delta)
    }
    V8 kt[2][2];
    {
      u32x2 tw[2][2][2];
      read_transposed_sync(k_buf[buf], tr_off, tw);
#pragma unroll
      for (int jj = 0; jj < 2; jj++)
#pragma unroll
        for (int dt = 0; dt < 2; dt++) kt[jj][dt] = frag_of<E>(tw[jj][dt][0], tw[jj][dt][1]);
    }
#pragma unroll
    for (int jj = 0; jj < 2; jj++)
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int qt = QT0; qt < QT1; qt++) dqt[qt][dt] = Mma<E>::mma(kt[jj][dt], ds[qt][jj], dqt[qt][dt]);
  };

  if (ntiles > 0) {
    int64_t cur = pop();
    if constexpr (BLK == 16) read_entries(cur, ent_cur);
    fetch(cur, H0{}, 0, ent_cur);
    for (int t = 0; t < ntiles; t++) {
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the reads of buffer 1 (previous tile) are done
      fetch(cur, H1{}, 1, ent_cur);
      __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): half 0 has landed
      compute(cur, H0{}, 0, ent_cur);
      const bool more = t + 1 < ntiles;
      const int64_t nxt = more ? pop() : cur;
      if constexpr (BLK == 16) {
        if (more) read_entries(nxt, ent_nxt);
      }
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the reads of buffer 0 are done
      if (more) {
        fetch(nxt, H0{}, 0, ent_nxt);
        __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): half 1 has landed
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      }
      compute(cur, H1{}, 1, ent_cur);
      cur = nxt;
      ent_cur = ent_nxt;
    }
  }

  E* dqp = (E*)p.dq + (int64_t)b * p.sdqb + (int64_t)h * p.sdqh;
#pragma unroll
  for (int qt = 0; qt < 2; qt++) {
    const int64_t row = q0 + qt * 32 + c;
    store_rows<E>(dqt[qt], dqp + row * p.sdqm, row < Lq, hh);
  }
}

// ---- dK, dV ------------------------------------------------------------------------------------------------------
template <typename E, bool DENSE, int BLK>
__global__ __launch_bounds__(128, 2) void bwd_dkdv_kernel(BwdParams p, int nkb, int nqb_all, int total_wg) {
  typedef typename Mma<E>::V8 V8;
  constexpr int kTileBytes = 2 * kHalfBytes;  // a 64-row query tile
  __shared__ __attribute__((aligned(1024))) unsigned char lds_q0[kTileBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_q1[kTileBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_g0[kTileBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_g1[kTileBytes];
  // per-query scalars of a tile: [0,64) lse, [64,128) delta.  BLK 16: four such pairs kVar floats apart, one per key
  // block of the workgroup, each with its own variant of lse (delta is repeated, so that a lane finds both values of
  // a query at a fixed distance and reads them with one instruction)
  constexpr int kVar = 136;
  constexpr int kDeltaAt = 64;
  __shared__ __attribute__((aligned(256))) float lds_s0[BLK == 16 ? 4 * kVar : 128];
  __shared__ __attribute__((aligned(256))) float lds_s1[BLK == 16 ? 4 * kVar : 128];
  __shared__ __attribute__((aligned(16))) int2 lds_union[BLK == 16 ? kMergeMax + 8 : 1];  // BLK 16: the current chunk's union of the four lists

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int hh = lane >> 5;
  const int c = lane & 31;

  // With lists the grid has two passes over the key blocks: the first (workgroups [0, total_wg)) takes the blocks whose
  // lists are long, the second the others, so the longest lists of a skewed index tensor start first instead of
  // wherever their key block falls in the launch order.
  const bool long_pass = DENSE || (int)blockIdx.x < total_wg;
  const int w = (int)blockIdx.x < total_wg ? (int)blockIdx.x : (int)blockIdx.x - total_wg;
  const int xcd = w & 7, slot = w >> 3;
  const int per = total_wg >> 3, rem = total_wg & 7;
  const int vid = xcd * per + (xcd < rem ? xcd : rem) + slot;
  const int bh = vid / nkb;
  const int kb = vid - bh * nkb;
  const int b = bh / p.H;
  const int h = bh - b * p.H;

  const int64_t Lq = p.Lq, Lk = p.Lk;
  if constexpr (!DENSE) {
    const int64_t nkbl = (Lk + BLK - 1) / BLK;
    const int32_t* off = p.kq_off + ((int64_t)b * p.H + h) * (nkbl + 1);
    int len;
    if constexpr (BLK == 64) {
      len = off[kb + 1] - off[kb];
    } else {  // the workgroup walks the lists of its four key blocks one after the other, four entries per step
      const int64_t ka = (int64_t)kb * 4;
      const int64_t kz = ka + 4 < nkbl ? ka + 4 : nkbl;
      len = (off[kz] - off[ka]) / 4;
    }
    len = __builtin_amdgcn_readfirstlane(len);
    if ((len > 4 * p.K) != long_pass) return;
  }
  const E* qp = (const E*)p.q + (int64_t)b * p.sqb + (int64_t)h * p.sqh;
  const E* kp = (const E*)p.k + (int64_t)b * p.skb + (int64_t)h * p.skh;
  const E* vp = (const E*)p.v + (int64_t)b * p.svb + (int64_t)h * p.svh;
  const E* gp = (const E*)p.dout + (int64_t)b * p.sgb + (int64_t)h * p.sgh;
  const float* lsep = p.lse + ((int64_t)b * p.H + h) * Lq;
  const float* dlp = p.delta + ((int64_t)b * p.H + h) * Lq;

  // B operands K and V of this wave's 32 keys (lane = key, head_dim chunk hh + 2 ks).  BLK 16: these are two
  // neighbouring key blocks, the workgroup's 64 keys four.
  const int64_t key = (int64_t)kb * 64 + wave * 32 + c;
  V8 bk[4], bv[4];
  f32x16 dkt[2], dvt[2];  // dK^T, dV^T [dt]: lane = key, registers = head_dim
  auto load_keys = [&]() {
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      Frag f, g;
      f.u = make_uint4(0, 0, 0, 0);
      g.u = make_uint4(0, 0, 0, 0);
      if (key < Lk) {
        f.u = *reinterpret_cast<const uint4*>(kp + key * p.skn + ks * 16 + hh * 8);
        g.u = *reinterpret_cast<const uint4*>(vp + key * p.svn + ks * 16 + hh * 8);
      }
      bk[ks] = as_v8<E>(f);
      bv[ks] = as_v8<E>(g);
    }
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
      for (int r = 0; r < 16; r++) { dkt[dt][r] = 0.f; dvt[dt][r] = 0.f; }
  };
  load_keys();

  // query blocks that attend to this key block
  static_assert(BLK == 64 || (BLK == 16 && !DENSE), "blocks of 64 tokens, or of 16 with key-centric lists");
  int n_lists;
  const int32_t* list = nullptr;
  const int32_t* off16 = nullptr;  // BLK 16: the list offsets of this (b, h); `list` then points at the head's whole list array
  if constexpr (DENSE) {
    n_lists = nqb_all;
  } else if constexpr (BLK == 64) {
    const int32_t* off = p.kq_off + ((int64_t)b * p.H + h) * (nkb + 1);
    const int32_t lo = off[kb], hi = off[kb + 1];
    n_lists = hi - lo;
    list = p.kq_list + ((int64_t)b * p.H + h) * p.list_stride + lo;
  } else {
    const int64_t nkb16 = (Lk + 15) >> 4;
    const int32_t* off = p.kq_off + ((int64_t)b * p.H + h) * (nkb16 + 1);
    n_lists = 0;  // set per key block below
    list = p.kq_list + ((int64_t)b * p.H + h) * p.list_stride;
    off16 = off;
  }
  // BLK 16: how often each of the workgroup's four key blocks lists the two query blocks this wave fetches for the
  // tile in flight (a byte per key block), set by block_of for the fetch that follows it
  uint32_t ent_cnt_a = 0, ent_cnt_b = 0;
  // List entries come 64 at a time (lane l holds entry base + l), so the latency of the list read is paid once per
  // 64 tiles and not in front of every tile's transfers.  The lists are walked front to back.
  int32_t held_a = -1;
  int base_a = -64;
  auto entry = [&](const int32_t* lst, int len, int32_t& held, int& base, int i) -> int32_t {
    if (i >= base + 64) {
      base = i & ~63;
      held = base + lane < len ? lst[base + lane] : -1;
    }
    return __builtin_amdgcn_readlane(held, i - base);
  };
  auto block_of = [&](int i) -> int64_t {
    if constexpr (DENSE) {
      return (int64_t)i;
    } else if constexpr (BLK == 64) {
      return (int64_t)entry(list, n_lists, held_a, base_a, i);
    } else {  // tile i of the chunk: entries 4i .. 4i+3 of the union, this wave fetches 4i + 2 wave and the next one
      const int4 v = *reinterpret_cast<const int4*>(lds_union + 4 * i + 2 * wave);
      const int32_t q0 = __builtin_amdgcn_readfirstlane(v.x), q1 = __builtin_amdgcn_readfirstlane(v.z);
      ent_cnt_a = (uint32_t)__builtin_amdgcn_readfirstlane(v.y);
      ent_cnt_b = (uint32_t)__builtin_amdgcn_readfirstlane(v.w);
      return (int64_t)(uint32_t)q0 | ((int64_t)q1 << 32);  // packed for `fetch`; -1: none
    }
  };

  const float scale = p.scale;
  const float sl2 = scale * kLog2e;
  // The per-query terms ride in the accumulators instead of in the vector slots.  The accumulator of S starts at
  // -lse / scale (16-token blocks: the variant of the lane's key block, its count folded in), so P = exp2(scale * log2(e) *
  // accumulator); the accumulator of dP starts at -delta, so dS / scale = P * accumulator.  No slot then begins with an
  // LDS read of per-query values in front of the arithmetic that needs them: the start values come with four
  // ds_read_b128 per accumulator ahead of the half's products (those of the second half's dP a quarter per slot, next
  // to the fragments of its products: the 16-token instance has no register to spare for all of them at once).  bf16
  // also puts the softmax scale onto dK once at the end (the rounding of dS to the I/O type is relative and
  // does not care for the factor): per score a multiplication, an exponential and a multiplication instead of two fused
  // multiply-adds, an exponential and a multiplication; fp16, with its narrow range, scales every dS.  bf16, 266 496
  // tokens: 64-token blocks, top-16: 2.88 -> 2.79 (delta) -> 2.62 ms (lse); 16-token blocks, top-32: 3.74 -> 3.67 ms.
  const float inv_scale = 1.0f / scale;
  constexpr bool FOLD = true;  // (kept as a switch: the other form reads lse and delta from LDS inside the vector slots)
  constexpr bool LATE_SCALE = std::is_same<E, bf16_t>::value;  // the softmax scale goes onto dK at the end
  const uint32_t qrow = (uint32_t)p.sqm * (uint32_t)sizeof(E), grow = (uint32_t)p.sgm * (uint32_t)sizeof(E);
  const int tr_off = tr_offset(lane);
  const int lse_at = BLK == 16 ? (2 * wave + (c >> 4)) * kVar : 0;
  // (one per parity of the instruction inside its half tile: the chunk map of rows 8..15 differs from that of rows 0..7)
  const uint32_t q_voff[2] = {(uint32_t)(lane >> 3) * qrow + (uint32_t)(((lane & 7) ^ k_swizzle(lane >> 3)) * 16),
                              (uint32_t)(lane >> 3) * qrow + (uint32_t)(((lane & 7) ^ k_swizzle((lane >> 3) + 8)) * 16)};
  const uint32_t g_voff[2] = {(uint32_t)(lane >> 3) * grow + (uint32_t)(((lane & 7) ^ k_swizzle(lane >> 3)) * 16),
                              (uint32_t)(lane >> 3) * grow + (uint32_t)(((lane & 7) ^ k_swizzle((lane >> 3) + 8)) * 16)};

  float staged = 0.f;          // this lane's lse or delta value of the tile in flight, as loaded (BLK 64: wave 0 lse,
                               // wave 1 delta; BLK 16: lanes 0..31 lse, 32..63 delta of the wave's 32 queries)
  bool staged_inf = false;     // rows past the end of the tensor or of a block publish lse = +inf
  uint32_t staged_cnt = 0;     // BLK 16: the count bytes of the row's query block
  int staged_buf = -1;         // (wave-uniform) the buffer it goes to; -1: nothing staged
  // One query tile (64 rows of Q and dO, 64 lse and delta values) -> buffer BUF; each wave moves half of every
  // operand (instructions 2*wave, 2*wave+1 of both 32-row halves), wave 0 the lse values, wave 1 delta.
  auto fetch = [&](int64_t qblk, auto bufc) {
    constexpr int BUF = decltype(bufc)::value;
    char* qb = reinterpret_cast<char*>(BUF == 0 ? lds_q0 : lds_q1);
    char* gb = reinterpret_cast<char*>(BUF == 0 ? lds_g0 : lds_g1);
    if constexpr (BLK == 64) {
      const int64_t start = qblk * 64;
      const int last = (int)((Lq - start < 64 ? Lq - start : 64) - 1);
      if (last >= 63) {
        // (wave-uniform) a full tile: per-lane offsets (row lane/8 and its chunk) that do not depend on the tile, the
        // instruction's rows ride in the scalar offset
        const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc((void*)(qp + start * p.sqm), 0, 0x7fffffff, 0x00020000);
        const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc((void*)(gp + start * p.sgm), 0, 0x7fffffff, 0x00020000);
#pragma unroll
        for (int hf = 0; hf < 2; hf++)
#pragma unroll
          for (int ii = 0; ii < 2; ii++) {
            const int i = 2 * wave + ii;
            const uint32_t rows = (uint32_t)(32 * hf + 8 * i);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rq, (__attribute__((address_space(3))) void*)(qb + hf * kHalfBytes + i * 1024), 16,
                                                     q_voff[ii], rows * qrow, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rg, (__attribute__((address_space(3))) void*)(gb + hf * kHalfBytes + i * 1024), 16,
                                                     g_voff[ii], rows * grow, 0, 0);
          }
      } else {
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
          dma_rows<E, true>(qp + start * p.sqm, qrow, 32 * hf, last, qb + hf * kHalfBytes, lane, 2 * wave, 2 * wave + 2);
          dma_rows<E, true>(gp + start * p.sgm, grow, 32 * hf, last, gb + hf * kHalfBytes, lane, 2 * wave, 2 * wave + 2);
        }
      }
      // per-query scalars pass through a register and are stored to LDS by `publish` before the barrier that opens
      // the tile
      const int r = lane < last ? lane : last;
      staged = ((wave == 0 ? lsep : dlp) + start)[r];
      staged_inf = wave == 0 && lane > last;  // query rows beyond Lq: lse = +inf, no probability
      staged_buf = BUF;
    } else {
      // this wave's half of the tile: the 16 queries of each of the step's two query blocks (none: any rows,
      // lse = +inf); lanes 0..31 fetch the 32 lse values, lanes 32..63 the delta values
      const int32_t ea = (int32_t)(qblk & 0xffffffffLL), eb = (int32_t)(qblk >> 32);  // the step's two query blocks (-1: none)
      const int64_t sa = ea >= 0 ? (int64_t)ea * 16 : 0, sbk = eb >= 0 ? (int64_t)eb * 16 : 0;
      const int na = ea >= 0 ? (int)(Lq - sa < 16 ? Lq - sa : 16) : 0;
      const int nb = eb >= 0 ? (int)(Lq - sbk < 16 ? Lq - sbk : 16) : 0;
      const int la = na > 0 ? na - 1 : 0, lb = nb > 0 ? nb - 1 : 0;
      dma_rows16<E, true>(qp + sa * p.sqm, qp + sbk * p.sqm, qrow, la, lb, qb + wave * kHalfBytes, lane);
      dma_rows16<E, true>(gp + sa * p.sgm, gp + sbk * p.sgm, grow, la, lb, gb + wave * kHalfBytes, lane);
      const int j = lane & 31, j16 = j & 15;
      const bool second = (j >> 4) != 0;
      const int nmine = second ? nb : na;
      const int64_t row = (second ? sbk : sa) + (j16 < nmine ? j16 : 0);
      staged = (hh == 0 ? lsep : dlp)[row];
      staged_inf = hh == 0 && j16 >= nmine;
      staged_cnt = second ? ent_cnt_b : ent_cnt_a;
      staged_buf = BUF;
    }
  };
  // The loaded value is first touched here, a whole tile of work after its load: any arithmetic on it inside `fetch`
  // would make the wave wait for the load there, and with it (the counter is in order) for the tile transfers issued
  // just before, which is the tile that should be in flight during the current tile's work.
  auto publish = [&]() {
    if (staged_buf < 0) return;
    float* const sb = staged_buf == 0 ? lds_s0 : lds_s1;
    if constexpr (BLK == 64) {
      // scaled once here (lse to base 2, delta by the softmax scale) instead of once per score
      if constexpr (FOLD) sb[64 * wave + lane] = staged_inf ? -INFINITY : wave == 0 ? -staged * inv_scale : -staged;
      else sb[64 * wave + lane] = staged_inf ? INFINITY : staged * (wave == 0 ? kLog2e : scale);
    } else {
      // P of (query, key) counts as often as the key's block lists the query's block: the count goes into the
      // exponent (lse - log2(count); 0 times: lse = +inf), one variant of the query's value per key block
      const bool is_lse = hh == 0;
      const float base = FOLD ? (staged_inf ? -INFINITY : is_lse ? -staged * inv_scale : -staged)
                              : (staged_inf ? INFINITY : staged * (is_lse ? kLog2e : scale));
      const bool plain = __ballot(is_lse && (staged_cnt & 0xfefefefeu) != 0) == 0;  // (wave-uniform) no block listed twice
      float* const to = sb + (is_lse ? 0 : kDeltaAt) + 32 * wave + (lane & 31);
#pragma unroll
      for (int kk = 0; kk < 4; kk++) {
        const uint32_t wgt = (staged_cnt >> (8 * kk)) & 0xffu;
        float vkk;
        if constexpr (FOLD) {  // start value of the S accumulator: -(lse - ln(count)) / scale
          vkk = is_lse && wgt == 0 ? -INFINITY : base;
          if (!plain && is_lse) vkk += __builtin_amdgcn_logf((float)(wgt > 1 ? wgt : 1)) * (1.0f / sl2);
        } else {
          vkk = is_lse && wgt == 0 ? INFINITY : base;
          if (!plain && is_lse) vkk -= __builtin_amdgcn_logf((float)(wgt > 1 ? wgt : 1));
        }
        to[kk * kVar] = vkk;
      }
    }
    staged_buf = -1;
  };
  // One tile in three stages per 32-query half (A = row reads + S, dP; B = P and dS from the per-query scalars; C =
  // transposed reads + dV^T, dK^T) with every instruction placed by hand, as in the forward kernel.  The vector work of
  // a 32-query half (16 scores per lane: P, dS, their roundings) is cut into eight slots of two scores; each slot also
  // issues one matrix product of another stage: the scores of half 1 run under the vector work of half 0, the dV / dK
  // products of half 0 under the vector work of half 1.  Only the scores of half 0 and the products of half 1 have no
  // vector work to hide behind.  Query rows beyond Lq need no masks: their lse is +inf.
  auto tile64 = [&](auto bufc) {
    constexpr int BUF = decltype(bufc)::value;
    const char* qb = reinterpret_cast<const char*>(BUF == 0 ? lds_q0 : lds_q1);
    const char* gb = reinterpret_cast<const char*>(BUF == 0 ? lds_g0 : lds_g1);
    const float* sb = BUF == 0 ? lds_s0 : lds_s1;
    const float* sl = sb + lse_at;  // BLK 16: the lse variant of this lane's key block
    f32x16 sc[2], dpv[2];   // S and dP of the two halves
    V8 pbv[2][2], dbv[2][2];  // P and dS as B operands [half][jj]
    V8 aq[4], ag[4];          // row fragments of Q, dO (A operands of the scores)
    V8 gt[2][2], qt[2][2];    // transposed fragments of dO, Q (A operands of dV^T, dK^T)
    auto mma_a = [&](auto hf_tag, auto i_tag) {  // product i of 8 of a half's scores: 0-3 S, 4-7 dP
      constexpr int HF = decltype(hf_tag)::value, i = decltype(i_tag)::value, ks = i & 3;
      f32x16 z;
#pragma unroll
      for (int r = 0; r < 16; r++) z[r] = 0.f;
      if constexpr (i < 4) sc[HF] = Mma<E>::mma(aq[ks], bk[ks], ks == 0 && !FOLD ? z : sc[HF]);
      else dpv[HF] = Mma<E>::mma(ag[ks], bv[ks], ks == 0 && !FOLD ? z : dpv[HF]);
    };
    // FOLD: the accumulator of a half's dP starts at minus delta of its queries (registers 4g .. 4g+3 hold the queries
    // 4hh + 8g .. + 3 of the half)
    auto lse_init = [&](auto hf_tag) {
      constexpr int HF = decltype(hf_tag)::value;
      if constexpr (FOLD) {
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          const float4 l4 = *reinterpret_cast<const float4*>(sl + 32 * HF + 4 * hh + 8 * g4);
          sc[HF][4 * g4] = l4.x;
          sc[HF][4 * g4 + 1] = l4.y;
          sc[HF][4 * g4 + 2] = l4.z;
          sc[HF][4 * g4 + 3] = l4.w;
        }
      }
    };
    auto delta_init_piece = [&](auto hf_tag, auto g_tag) {  // registers 4g .. 4g+3 of the half's dP accumulator
      constexpr int HF = decltype(hf_tag)::value, g4 = decltype(g_tag)::value;
      if constexpr (FOLD) {
        const float4 d4 = *reinterpret_cast<const float4*>(sl + kDeltaAt + 32 * HF + 4 * hh + 8 * g4);
        dpv[HF][4 * g4] = d4.x;
        dpv[HF][4 * g4 + 1] = d4.y;
        dpv[HF][4 * g4 + 2] = d4.z;
        dpv[HF][4 * g4 + 3] = d4.w;
      }
    };
    auto delta_init = [&](auto hf_tag) {
      lse_init(hf_tag);
      static_for<4>([&](auto g_tag) { delta_init_piece(hf_tag, g_tag); });
    };
    auto mma_c = [&](auto hf_tag, auto i_tag) {  // product i of 8 of a half's dV^T / dK^T updates
      constexpr int HF = decltype(hf_tag)::value, i = decltype(i_tag)::value, jj = (i >> 1) & 1, dt = i & 1;
      if constexpr (i < 4) dvt[dt] = Mma<E>::mma(gt[jj][dt], pbv[HF][jj], dvt[dt]);
      else dkt[dt] = Mma<E>::mma(qt[jj][dt], dbv[HF][jj], dkt[dt]);
    };
    auto vec = [&](auto hf_tag, auto j_tag) {  // scores 2j, 2j+1 of the half: P, dS, both rounded
      constexpr int HF = decltype(hf_tag)::value, j = decltype(j_tag)::value, r = 2 * j;
      // queries 4hh + 8(j/2) + 2(j%2) + {0, 1} of the half
      f32x16& sh = sc[HF];
      f32x16& dh = dpv[HF];
      float p0, p1, e0, e1;
      if constexpr (FOLD) {
        p0 = __builtin_amdgcn_exp2f(sh[r] * sl2);
        p1 = __builtin_amdgcn_exp2f(sh[r + 1] * sl2);
        e0 = LATE_SCALE ? p0 * dh[r] : p0 * (dh[r] * scale);
        e1 = LATE_SCALE ? p1 * dh[r + 1] : p1 * (dh[r + 1] * scale);
      } else {
        const float2 l2 = *reinterpret_cast<const float2*>(sl + 32 * HF + 4 * hh + 8 * (j >> 1) + 2 * (j & 1));
        p0 = __builtin_amdgcn_exp2f(fmaf(sh[r], sl2, -l2.x));
        p1 = __builtin_amdgcn_exp2f(fmaf(sh[r + 1], sl2, -l2.y));
        const float2 d2 = *reinterpret_cast<const float2*>(sl + kDeltaAt + 32 * HF + 4 * hh + 8 * (j >> 1) + 2 * (j & 1));
        e0 = p0 * fmaf(dh[r], scale, -d2.x);
        e1 = p1 * fmaf(dh[r + 1], scale, -d2.y);
      }
      V8& pv = pbv[HF][r >> 3];
      V8& dv = dbv[HF][r >> 3];
      pv[r & 7] = (E)p0;
      pv[(r & 7) + 1] = (E)p1;
      dv[r & 7] = (E)e0;
      dv[(r & 7) + 1] = (E)e1;
    };
    if constexpr (BLK == 64) {
      read_rows<E, true>(qb, c, hh, aq);
      read_rows<E, true>(gb, c, hh, ag);
    } else {  // all eight fragments requested at once and waited for by hand: left to itself the compiler, short of
      // registers further down the tile, reads them one at a time in this instance, each in front of its product
      u32x4 qw[4], gw[4];
      read_rows2_sync(qb, gb, c, hh, qw, gw);
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        aq[ks] = frag_of<E>(qw[ks]);
        ag[ks] = frag_of<E>(gw[ks]);
      }
    }
    delta_init(H0{});
    static_for<8>([&](auto i_tag) { mma_a(H0{}, i_tag); });
    __builtin_amdgcn_sched_barrier(0);
    // the fragments of a region's second four products are requested four slots ahead, one per slot, so that at most
    // five fragments are in registers at a time
    read_rows<E, true>(qb + kHalfBytes, c, hh, aq);
    lse_init(H1{});
    static_for<8>([&](auto j_tag) {
      constexpr int j = decltype(j_tag)::value;
      if constexpr (j < 4) ag[j] = read_row_frag<E, true>(gb + kHalfBytes, c, hh, j);
      if constexpr (j < 4) delta_init_piece(H1{}, j_tag);  // (a quarter per slot: needed from the fifth product on)
      mma_a(H1{}, j_tag);
      vec(H0{}, j_tag);
      __builtin_amdgcn_sched_barrier(0);
    });
    read_transposed<E>(gb, tr_off, gt);
    static_for<8>([&](auto j_tag) {
      constexpr int j = decltype(j_tag)::value;
      if constexpr (j < 4) qt[(j >> 1) & 1][j & 1] = read_transposed_frag<E>(qb, tr_off, (j >> 1) & 1, j & 1);
      mma_c(H0{}, j_tag);
      vec(H1{}, j_tag);
      __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (BLK == 64) {
      read_transposed<E>(gb + kHalfBytes, tr_off, gt);
      read_transposed<E>(qb + kHalfBytes, tr_off, qt);
      static_for<8>([&](auto i_tag) { mma_c(H1{}, i_tag); });
    } else {
      u32x2 gw[2][2][2], qw[2][2][2];
      read_transposed_sync(gb + kHalfBytes, tr_off, gw);
#pragma unroll
      for (int jj = 0; jj < 2; jj++)
#pragma unroll
        for (int dt = 0; dt < 2; dt++) gt[jj][dt] = frag_of<E>(gw[jj][dt][0], gw[jj][dt][1]);
      static_for<4>([&](auto i_tag) { mma_c(H1{}, i_tag); });
      read_transposed_sync(qb + kHalfBytes, tr_off, qw);
#pragma unroll
      for (int jj = 0; jj < 2; jj++)
#pragma unroll
        for (int dt = 0; dt < 2; dt++) qt[jj][dt] = frag_of<E>(qw[jj][dt][0], qw[jj][dt][1]);
      static_for<4>([&](auto i_tag) { mma_c(H1{}, std::integral_constant<int, decltype(i_tag)::value + 4>{}); });
    }
  };
  // this wave's part of the tile has landed, its reads of the other buffer are done; after the barrier both hold
  // for both waves
  auto sync = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    publish();
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
  };

  auto walk = [&]() {  // all tiles of the current list, double buffered
    if (n_lists > 0) {
      int64_t cur = block_of(0);
      fetch(cur, H0{});
      for (int t = 0; t < n_lists; t += 2) {
        sync();
        const bool more1 = t + 1 < n_lists;
        const int64_t nxt1 = more1 ? block_of(t + 1) : cur;
        if (more1) fetch(nxt1, H1{});
        tile64(H0{});
        if (!more1) break;
        sync();
        const bool more2 = t + 2 < n_lists;
        cur = more2 ? block_of(t + 2) : nxt1;
        if (more2) fetch(cur, H0{});
        tile64(H1{});
      }
    }
  };
  E* dkp = (E*)p.dk + (int64_t)b * p.sdkb + (int64_t)h * p.sdkh;
  E* dvp = (E*)p.dv + (int64_t)b * p.sdvb + (int64_t)h * p.sdvh;
  if constexpr (BLK == 64) {
    walk();
    if constexpr (LATE_SCALE) {
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) dkt[dt][r] *= scale;
    }
    store_rows<E>(dkt, dkp + key * p.sdkn, key < Lk, hh);
    store_rows<E>(dvt, dvp + key * p.sdvn, key < Lk, hh);
  } else {
    // The workgroup's 64 keys are FOUR neighbouring key blocks, whose lists name mostly the same query blocks (at
    // 266 496 tokens, top-32, the union of the four lists is half as long as the lists together), and the workgroup walks
    // that union, four distinct query blocks per 64-row tile, with the 64-token kernel's tile code: a probability counts
    // as often as its key block's list names its query block (`publish`).  The union is built a chunk at a time from
    // the (ascending) lists: every list offers a window of its next kWin entries; tau = the smallest value that follows
    // a window; the chunk takes the window entries below tau (the list that sets tau gives its whole window, so the
    // walk advances; entries at or above tau may have partners in other lists that are not in their windows yet).
    // Each wave inserts two of the lists into a 512-slot hash table in an idle tile buffer: compare-and-swap on the query
    // block, linear probing, 1 added to the list's byte of the slot's count; wave 0 then compacts the occupied slots into
    // lds_union, eight slots per lane, positions from ballots.  Tiles come in the table's order (fp32 summation order
    // only).  Every list entry is in exactly one chunk, so whatever the chunks' borders, every (query block, key block)
    // pair is counted as often as listed.
    constexpr int kWin = kMergeMax / 4;
    static_assert(kWin > 64 && kWin <= 128, "a window is read with two loads per lane; a query block repeats at most 64 times in a list");
    const int64_t nkb16 = (Lk + 15) >> 4;
    const int32_t* lp[4];
    int llen[4], lpos[4];
#pragma unroll
    for (int i4 = 0; i4 < 4; i4++) {
      const int64_t kblk = (int64_t)kb * 4 + i4;
      const bool there = kblk < nkb16;
      const int32_t o0 = there ? __builtin_amdgcn_readfirstlane(off16[kblk]) : 0;
      const int32_t o1 = there ? __builtin_amdgcn_readfirstlane(off16[kblk + 1]) : 0;
      lp[i4] = list + o0;
      llen[i4] = o1 - o0;
      lpos[i4] = 0;
    }
    int32_t* const hkey = reinterpret_cast<int32_t*>(lds_q0);          // [512]
    uint32_t* const hcnt = reinterpret_cast<uint32_t*>(lds_q0 + 2048);  // [512]
    auto insert = [&](bool active, int32_t e, uint32_t one) {
      uint32_t slot = ((uint32_t)e * 0x9E3779B1u) >> 23;
      while (active) {
        const int32_t old = atomicCAS(hkey + slot, -1, e);
        if (old == -1 || old == e) {
          atomicAdd(hcnt + slot, one);
          active = false;
        } else {
          slot = (slot + 1) & 511u;
        }
      }
    };
    auto build_chunk = [&]() -> bool {  // false: the lists are exhausted.  Both waves take the same decisions.
      // all eight loads in one round trip: lane kWin - 64 of a list's second load fetches the value after the window
      int32_t ev[4][2];
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const int i0 = lpos[i4] + lane, i1 = lpos[i4] + 64 + lane;
        ev[i4][0] = i0 < llen[i4] ? lp[i4][i0] : 0x7fffffff;
        ev[i4][1] = lane <= kWin - 64 && i1 < llen[i4] ? lp[i4][i1] : 0x7fffffff;
      }
      int32_t tau = 0x7fffffff;
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const int32_t nextv = __builtin_amdgcn_readlane(ev[i4][1], kWin - 64);
        tau = nextv < tau ? nextv : tau;
        if (lane == kWin - 64) ev[i4][1] = 0x7fffffff;  // not part of the window
      }
      int taken[4], total = 0;
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        taken[i4] = __popcll(__ballot(ev[i4][0] < tau)) + __popcll(__ballot(ev[i4][1] < tau));  // a prefix: the list is ascending
        total += taken[i4];
      }
      if (total == 0) return false;
      __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0), lgkmcnt(0): this wave is through the previous chunk's tiles
      __syncthreads();                      // ... and so is the other one: the table's buffer and the list are free
      reinterpret_cast<int4*>(hkey)[threadIdx.x] = make_int4(-1, -1, -1, -1);
      reinterpret_cast<int4*>(hcnt)[threadIdx.x] = make_int4(0, 0, 0, 0);
      __syncthreads();
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        if ((i4 >> 1) == wave) {  // (wave-uniform) this wave's two lists
          insert(ev[i4][0] < tau, ev[i4][0], 1u << (8 * i4));
          insert(ev[i4][1] < tau, ev[i4][1], 1u << (8 * i4));
        }
        lpos[i4] += taken[i4];
      }
      __syncthreads();
      if (wave == 0) {
        const int4 k0 = reinterpret_cast<const int4*>(hkey)[2 * lane], k1 = reinterpret_cast<const int4*>(hkey)[2 * lane + 1];
        const int4 c0 = reinterpret_cast<const int4*>(hcnt)[2 * lane], c1 = reinterpret_cast<const int4*>(hcnt)[2 * lane + 1];
        const int32_t ks8[8] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};
        const int32_t cs8[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
        uint32_t at = 0;  // occupied slots of the lanes below
        int n_union = 0;
#pragma unroll
        for (int s8 = 0; s8 < 8; s8++) {
          const uint64_t m = __ballot(ks8[s8] >= 0);
          at = __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, at));
          n_union += __popcll(m);
        }
#pragma unroll
        for (int s8 = 0; s8 < 8; s8++)
          if (ks8[s8] >= 0) lds_union[at++] = make_int2(ks8[s8], cs8[s8]);
        if (lane < 4) lds_union[n_union + lane] = make_int2(-1, 0);  // the last tile's missing entries
        if (lane == 0) lds_union[kMergeMax + 7] = make_int2(n_union, 0);
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the table is read before the first transfer lands on it
      }
      __syncthreads();
      n_lists = (__builtin_amdgcn_readfirstlane(lds_union[kMergeMax + 7].x) + 3) >> 2;  // tiles of this chunk
      return true;
    };
    while (build_chunk()) walk();
    if constexpr (LATE_SCALE) {
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) dkt[dt][r] *= scale;
    }
    store_rows<E>(dkt, dkp + key * p.sdkn, key < Lk, hh);
    store_rows<E>(dvt, dvp + key * p.sdvn, key < Lk, hh);
  }
}

}  // namespace bwd

int launch_attn_bwd(const BwdParams& p, int dtype, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  const bool dense = p.idx == nullptr;
  const int64_t nqb = (p.Lq + 63) / 64, nkb = (p.Lk + 63) / 64;
  const int64_t nqg = (nqb + 3) / 4;
  const int64_t total_q = nqg * p.B * p.H, total_k = nkb * p.B * p.H;
  if (total_q > 0x7fffffffLL || total_k > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "attention backward: grid too large");
  if (!dense && 2 * total_k > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "attention backward: grid too large");
  dim3 gq((unsigned)total_q), bq(256), gk((unsigned)(dense ? total_k : 2 * total_k)), bk(128);
#define S3R_BWD_LAUNCH(E)                                                                                                       \
  do {                                                                                                                          \
    if (p.dq != nullptr) {                                                                                                      \
      if (dense) hipLaunchKernelGGL((bwd::bwd_dq_kernel<E, true, 64>), gq, bq, 0, st, p, (int)nqb, (int)nqg, (int)total_q);     \
      else if (p.block == 16) hipLaunchKernelGGL((bwd::bwd_dq_kernel<E, false, 16>), gq, bq, 0, st, p, (int)nqb, (int)nqg, (int)total_q); \
      else hipLaunchKernelGGL((bwd::bwd_dq_kernel<E, false, 64>), gq, bq, 0, st, p, (int)nqb, (int)nqg, (int)total_q);          \
    }                                                                                                                           \
    if (p.dk != nullptr) {                                                                                                      \
      if (dense) hipLaunchKernelGGL((bwd::bwd_dkdv_kernel<E, true, 64>), gk, bk, 0, st, p, (int)nkb, (int)nqb, (int)total_k);   \
      else if (p.block == 16) hipLaunchKernelGGL((bwd::bwd_dkdv_kernel<E, false, 16>), gk, bk, 0, st, p, (int)nkb, (int)nqb, (int)total_k); \
      else hipLaunchKernelGGL((bwd::bwd_dkdv_kernel<E, false, 64>), gk, bk, 0, st, p, (int)nkb, (int)nqb, (int)total_k);        \
    }                                                                                                                           \
  } while (0)
  if (dtype == S3R_BF16) S3R_BWD_LAUNCH(bf16_t);
  else S3R_BWD_LAUNCH(f16_t);
#undef S3R_BWD_LAUNCH
  return check_launch("attention backward");
}

int launch_bwd_delta(const void* o, const void* dout, float* delta, int B, int H, int64_t N, int64_t sob, int64_t soh, int64_t son,
                     int64_t sdb, int64_t sdh, int64_t sdn, int dtype, void* stream) {
  const int64_t rows = (int64_t)B * H * N;
  const int64_t blocks = (rows * 8 + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_attn_bwd_delta: tensor too large for one launch");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)blocks), blk(256);
  if (dtype == S3R_BF16)
    hipLaunchKernelGGL(bwd::bwd_delta_kernel<bf16_t>, grid, blk, 0, st, (const bf16_t*)o, (const bf16_t*)dout, delta, H, N, rows, sob, soh, son, sdb, sdh, sdn);
  else
    hipLaunchKernelGGL(bwd::bwd_delta_kernel<f16_t>, grid, blk, 0, st, (const f16_t*)o, (const f16_t*)dout, delta, H, N, rows, sob, soh, son, sdb, sdh, sdn);
  return check_launch("bwd_delta_kernel");
}

}  // namespace s3r
