// Compressed-branch attention on the gfx950 matrix cores (bf16 / fp16 I/O, head_dim 64):
// dense non-causal flash attention over the pooled tokens, plus the exact top-k block
// selection, either fused into the same pass or from a score matrix written to HBM.
//
// A workgroup of four wavefronts (the top-k-only kernel also: two) owns 32 query rows of one head per wavefront and walks all key
// tiles of 64 pooled tokens.  K and V tiles are staged once per workgroup in LDS (global ->
// registers two tiles ahead -> LDS one tile ahead, two LDS buffers, one barrier per tile) and
// shared by the four waves.  Rows are 128 bytes without padding; 16-byte chunks are stored
// XOR-swizzled (K: chunk ^ k_swizzle(row) for the 16-byte operand reads, V: halves swapped on rows
// 2,3 mod 4 for the transposed reads) so that LDS reads are bank-conflict free.
// Per wave and tile: S^T = K Q^T with v_mfma_f32_32x32x16 (one query per lane and its partner
// lane ^ 32, 32 of the tile's 64 keys in each lane's registers), base-2 online softmax in
// fp32, P rounded to the I/O dtype, O^T += V^T P^T with V^T fragments from ds_read_b64_tr_b16.
//
// Selection without a score buffer (the top-k-only instance, KTOP > 0): two sweeps over the key tiles, K tiles by
// direct transfers into an LDS ring.  Sweep 1 keeps, per lane, the K largest of its half-tile maxima; the K-th
// largest of the two lanes' lists is a lower bound of the row's K-th largest score.  Sweep 2 recomputes the scores
// and appends every score >= that threshold to a small per-lane queue in LDS (no branch).  Every lane keeps the
// exact top-K of the keys IT sees (half of each tile): a descending sorted list of K keys,
// key = (sortable(bits(score)), Lk-1-col) in lexicographic order, in registers.  When some lane's queue is nearly
// full, all lanes merge their queues into their lists with a register-resident bitonic network (no divergence:
// every lane runs the same network on its own data) and raise their thresholds to their lists' last entries.  At
// the end the two lanes of a query merge their lists and lane < 32 writes the K indices in descending key order.
// The filter is conservative (anything that could enter passes), the network compares full keys, so the result is
// the same unique top-K as a sort of the whole row.
#include "s3r_common.h"
#include "attn_params.h"
#include <type_traits>
#include <utility>

namespace s3r {
namespace cmp {

template <typename E> struct Mma;
template <> struct Mma<bf16_t> {
  typedef bf16x8 V8;
  static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Mma<f16_t> {
  typedef f16x8 V8;
  static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
union Frag {
  uint4 u;
  u32x4 w;
  bf16x8 b;
  f16x8 h;
  s16x4 s[2];
};
template <typename E> __device__ __forceinline__ typename Mma<E>::V8 as_v8(const Frag& f);
template <> __device__ __forceinline__ bf16x8 as_v8<bf16_t>(const Frag& f) { return f.b; }
template <> __device__ __forceinline__ f16x8 as_v8<f16_t>(const Frag& f) { return f.h; }

__device__ __forceinline__ uint32_t xh_swap(uint32_t x) {  // value held by lane ^ 32
  auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
  return (threadIdx.x & 32) ? r[0] : r[1];
}
__device__ __forceinline__ float xh_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xh_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// ---- register-resident bitonic networks (descending order) ----
// A key is the pair (sortable bits of the score, Lk-1-col) held as ONE double, sortable * 2^21 + (Lk-1-col): exact for
// Lk <= 2^21 (53 bits), ordered like the 64-bit integer key, and a compare-exchange is one v_max_f64 and one
// v_min_f64 instead of a 64-bit compare and four selects.  0.0 is the filler (it decodes to column Lk-1).
typedef double key_t;
constexpr double kKeyScale = 2097152.0;  // 2^21
__device__ __forceinline__ key_t make_key(uint32_t score_bits, uint32_t rev_col) {
  return __builtin_fma((double)sortable_key(__uint_as_float(score_bits)), kKeyScale, (double)rev_col);
}
__device__ __forceinline__ uint32_t key_sortable(key_t k) { return (uint32_t)(k * (1.0 / kKeyScale)); }  // truncation
__device__ __forceinline__ uint32_t key_rev_col(key_t k) {
  const double hi = __builtin_trunc(k * (1.0 / kKeyScale));
  return (uint32_t)__builtin_fma(hi, -kKeyScale, k);
}
__device__ __forceinline__ void cex_desc(key_t& a, key_t& b) {  // a = max, b = min
  const key_t hi = __builtin_fmax(a, b);
  const key_t lo = __builtin_fmin(a, b);
  a = hi;
  b = lo;
}
template <int N> __device__ __forceinline__ void bitonic_merge_desc(key_t (&x)[N]) {  // x bitonic -> descending
#pragma unroll
  for (int d = N / 2; d >= 1; d >>= 1)
#pragma unroll
    for (int i = 0; i < N; i++)
      if ((i & d) == 0) cex_desc(x[i], x[i | d]);
}
// top-N of (descending a) U (descending b) -> a, descending; the last NF entries of b are fillers (key 0, below
// every real key), so the first NF entries of a meet nothing
template <int N, int NF = 0> __device__ __forceinline__ void merge_top_desc(key_t (&a)[N], const key_t (&b)[N]) {
#pragma unroll
  for (int i = NF; i < N; i++) a[i] = __builtin_fmax(a[i], b[N - 1 - i]);  // half-cleaner: a is now bitonic
  bitonic_merge_desc<N>(a);
}
// Sorting network for the 13 entries a lane's queue can hold (descending, entries 0..12 of x): Batcher's odd-even
// merge sort for 16 inputs without the comparators that touch inputs 13..15, 48 compare-exchanges against the 80
// of the bitonic network for 16 (checked on all 2^13 zero-one inputs by tests/test_sort_network.py).
constexpr int kSortNet13Size = 48;
constexpr signed char kSortNet13[kSortNet13Size][2] = {
    {0, 1}, {2, 3}, {0, 2}, {1, 3}, {1, 2}, {4, 5}, {6, 7}, {4, 6}, {5, 7}, {5, 6}, {0, 4}, {2, 6},
    {2, 4}, {1, 5}, {3, 7}, {3, 5}, {1, 2}, {3, 4}, {5, 6}, {8, 9}, {10, 11}, {8, 10}, {9, 11}, {9, 10},
    {8, 12}, {10, 12}, {9, 10}, {11, 12}, {0, 8}, {4, 12}, {4, 8}, {2, 10}, {6, 10}, {2, 4}, {6, 8}, {10, 12},
    {1, 9}, {5, 9}, {3, 11}, {7, 11}, {3, 5}, {7, 9}, {1, 2}, {3, 4}, {5, 6}, {7, 8}, {9, 10}, {11, 12}};
template <int N> __device__ __forceinline__ void sort13_desc(key_t (&x)[N]) {
  static_assert(N >= 13, "the network sorts entries 0..12");
#pragma unroll
  for (int i = 0; i < kSortNet13Size; i++) cex_desc(x[kSortNet13[i][0]], x[kSortNet13[i][1]]);
}

constexpr int kTile = 64 * 64;  // elements per LDS tile
// Scores appended between two checks of the queues' fill.  A check every 4 scores lets a queue fill to 9 of its 13 entries
// before the lists are merged (8 scores: to 5), and the merges are the expensive part: 0.186 -> 0.165 ms at 4164 pooled
// tokens, top-16; 0.316 -> 0.260 ms for top-32.
constexpr int kGroup = 4;
constexpr int kQCap = 16;       // width of the merge network that folds a lane's queue into its list
// Top-k-only kernel: LDS queue slots per lane (the last one is the dump slot of non-survivors) and K tiles in the
// LDS ring: 28 KB of queues + 24 KB of tiles, three workgroups per compute unit for every list length (the top-32
// kernel reaches the 168 registers of that occupancy with 24 dwords spilled inside the queue drain, its rare path).
template <int KTOP> struct TopkCfg {
  static constexpr int kQSlots = 14;
  static constexpr int kRing = 3;
};
template <> struct TopkCfg<0> {
  static constexpr int kQSlots = 1;
  static constexpr int kRing = 2;
};

// The eight K fragments of a 64-key tile, rows c (f[0]) and c + 32 (f[1]), k-steps 0..3 (chunk bits 1..2 of the address),
// read by hand: the compiler neither knows that this reads LDS nor when it lands, so it adds no wait for transfers into
// other LDS buffers that are still in flight.  Reads and wait are one statement: between a hand-written read and its
// wait the compiler must not get a chance to move or spill a register whose value has not arrived.
__device__ __forceinline__ void lds_read_kfrags(uint32_t kb, u32x4 (&f)[2][4]) {
  asm volatile(
      "ds_read_b128 %0, %8\n\tds_read_b128 %4, %8 offset:4096\n\tds_read_b128 %1, %9\n\tds_read_b128 %5, %9 offset:4096\n\t"
      "ds_read_b128 %2, %10\n\tds_read_b128 %6, %10 offset:4096\n\tds_read_b128 %3, %11\n\tds_read_b128 %7, %11 offset:4096\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(f[0][0]), "=&v"(f[0][1]), "=&v"(f[0][2]), "=&v"(f[0][3]), "=&v"(f[1][0]), "=&v"(f[1][1]), "=&v"(f[1][2]), "=&v"(f[1][3])
      : "v"(kb), "v"(kb ^ 32u), "v"(kb ^ 64u), "v"(kb ^ 96u)
      : "memory");
}
// The 13 slots of a lane's queue (64 x 8 bytes apart) in one statement, reads and wait together: between a hand-written
// read and its wait the compiler must not get a chance to move or spill a register whose value has not arrived.
__device__ __forceinline__ void lds_read_queue13(uint32_t addr, u32x2 (&r)[13]) {
  asm volatile(
      "ds_read_b64 %0, %13\n\tds_read_b64 %1, %13 offset:512\n\tds_read_b64 %2, %13 offset:1024\n\t"
      "ds_read_b64 %3, %13 offset:1536\n\tds_read_b64 %4, %13 offset:2048\n\tds_read_b64 %5, %13 offset:2560\n\t"
      "ds_read_b64 %6, %13 offset:3072\n\tds_read_b64 %7, %13 offset:3584\n\tds_read_b64 %8, %13 offset:4096\n\t"
      "ds_read_b64 %9, %13 offset:4608\n\tds_read_b64 %10, %13 offset:5120\n\tds_read_b64 %11, %13 offset:5632\n\t"
      "ds_read_b64 %12, %13 offset:6144\n\ts_waitcnt lgkmcnt(0)"
      : "=&v"(r[0]), "=&v"(r[1]), "=&v"(r[2]), "=&v"(r[3]), "=&v"(r[4]), "=&v"(r[5]), "=&v"(r[6]), "=&v"(r[7]), "=&v"(r[8]),
        "=&v"(r[9]), "=&v"(r[10]), "=&v"(r[11]), "=&v"(r[12])
      : "v"(addr)
      : "memory");
}

// WAVES: wavefronts (of 32 query rows) per workgroup.  The top-k-only kernel also comes with two: its waves meet at a
// barrier per tile, so whatever one wave does beyond the common path (a fold of its queues) holds up its whole
// workgroup; with few workgroups (one round, nothing else on the SIMD to fill the gap) pairs lose less than quads.
// Two waves per workgroup double the K tile transfers per query row and use a ring of two tiles (30 KB of LDS with the
// queues, five workgroups per CU).
template <typename E, int KTOP /* 0: attention (+ scores); > 0: top-k only */, int WAVES>
__global__ __launch_bounds__(256, KTOP > 0 ? 3 : 2) void compressed_mfma_kernel(AttnParams p) {
  typedef typename Mma<E>::V8 V8;
  constexpr bool FUSED = KTOP > 0;
  static_assert(WAVES == 4 || (WAVES == 2 && FUSED), "two waves per workgroup: top-k-only kernel");
  constexpr int KL = FUSED ? KTOP : 1;  // list length per lane
  constexpr int kQSlots = TopkCfg<KTOP>::kQSlots;
  constexpr int NB = WAVES == 2 ? 2 : TopkCfg<KTOP>::kRing;
  constexpr int NI = 8 / WAVES;  // transfer instructions (8 rows each) per wave and tile
  __shared__ __attribute__((aligned(1024))) E Ks[NB][kTile];
  __shared__ __attribute__((aligned(1024))) E Vs[FUSED ? 1 : 2][FUSED ? 8 : kTile];  // the top-k-only kernel stages K tiles alone
  __shared__ __attribute__((aligned(16))) uint2 queue[FUSED ? WAVES : 1][kQSlots][64];
  __shared__ __attribute__((aligned(16))) float sstage[FUSED ? 1 : 4][FUSED ? 4 : 32 * 64];  // score-store staging (unfused launches)

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int hh = lane >> 5;
  const int c = lane & 31;
  const int b = blockIdx.y / p.H;
  const int h = blockIdx.y - b * p.H;
  const int64_t Lq = p.Lq, Lk = p.Lk;
  const int64_t q0 = (int64_t)blockIdx.x * (32 * WAVES) + wave * 32;

  const E* qp = (const E*)p.q + (int64_t)b * p.sqb + (int64_t)h * p.sqh;
  const E* kp = (const E*)p.k + (int64_t)b * p.skb + (int64_t)h * p.skh;
  const E* vp = (const E*)p.v + (int64_t)b * p.svb + (int64_t)h * p.svh;

  const int64_t qrow = q0 + c;
  const bool qvalid = qrow < Lq;
  V8 bq[4];
#pragma unroll
  for (int ks = 0; ks < 4; ks++) {
    Frag f;
    f.u = make_uint4(0, 0, 0, 0);
    if (qvalid) f.u = *reinterpret_cast<const uint4*>(qp + qrow * p.sqm + ks * 16 + hh * 8);
    bq[ks] = as_v8<E>(f);
  }

  f32x16 ot[2];
#pragma unroll
  for (int dt = 0; dt < 2; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) ot[dt][r] = 0.f;
  float m_i = -INFINITY, l_i = 0.f;
  const float sl2 = p.scale * 1.4426950408889634f;

  // ---- tile staging: thread owns chunk rows ld_row, ld_row+32 at chunk position ld_pos of both tiles ----
  const int ld_row = tid >> 3, ld_pos = tid & 7;
  uint4 kr[2], vr[2];
  auto fetch = [&](int64_t start) {  // global -> registers; rows beyond Lk re-read the last row (they are masked)
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int r = ld_row + 32 * i;
      int64_t row = start + r;
      row = row < Lk ? row : Lk - 1;
      kr[i] = *reinterpret_cast<const uint4*>(kp + row * p.skn + ((ld_pos ^ k_swizzle(r)) * 8));
      vr[i] = *reinterpret_cast<const uint4*>(vp + row * p.svn + ((ld_pos ^ (((r >> 1) & 1) << 2)) * 8));
    }
  };
  auto stash = [&](int buf) {  // registers -> LDS
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int r = ld_row + 32 * i;
      *reinterpret_cast<uint4*>(&Ks[buf][r * 64 + ld_pos * 8]) = kr[i];
      *reinterpret_cast<uint4*>(&Vs[buf][r * 64 + ld_pos * 8]) = vr[i];
    }
  };
  // per-lane LDS read offsets (bytes)
  const int i16 = lane & 15;
  const int tr_row = 4 * hh + (i16 >> 2);
  const int tr_chunk = (((lane >> 4) & 1) * 2 + ((i16 & 3) >> 1)) ^ (((tr_row >> 1) & 1) << 2);
  const int tr_off = tr_row * 128 + tr_chunk * 16 + (i16 & 1) * 8;

  // ---- fused selection state ----
  key_t list[KL];  // descending
#pragma unroll
  for (int i = 0; i < KL; i++) list[i] = 0;
  float thr = -INFINITY;   // survivors are the scores >= thr
  float thr0 = -INFINITY;  // the row's threshold from the group maxima; thr never drops below it
  int qn = 0;
  uint2* qlane = FUSED ? &queue[wave][0][lane] : nullptr;  // entry e at qlane[e * 64]
  const uint32_t lkm1 = (uint32_t)(Lk - 1);

  auto drain = [&]() {  // merge this lane's queue into its list; every lane runs the same network
    // All queue slots are fetched at once and waited for once (hand-written reads: left to the compiler, each read
    // lands inside the `e < qn` branch of its entry with a wait of its own, thirteen LDS round trips in a row;
    // top-16 at 4 164 keys 0.148 -> 0.140 ms).
    u32x2 raw[13];
    if constexpr (FUSED) {  // (the attention instance has no queue and never folds)
      static_assert(!FUSED || kQSlots - 1 == 13, "the fold reads 13 queue slots");
      lds_read_queue13((uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)reinterpret_cast<char*>(qlane), raw);
    }
    key_t cand[kQCap];
#pragma unroll
    for (int e = 0; e < kQCap; e++) {
      cand[e] = 0;
      if (e < kQSlots - 1) {
        cand[e] = e < qn ? make_key(raw[e][0], lkm1 - raw[e][1]) : 0.0;
      }
    }
    // the queue's 13 entries through their own network; cand[13..15] stay fillers
    static_assert(!FUSED || (kQSlots - 1 == 13 && kQCap == 16), "the fold is built for 13 queue entries in a 16-wide merge");
    constexpr int kFill = kQCap - 13;
    sort13_desc(cand);
    if constexpr (KL == kQCap) {
      merge_top_desc<KL, kFill>(list, cand);
    } else if constexpr (KL < kQCap) {  // the KL best of list U cand are among the list and the KL best candidates
      key_t best[KL];
#pragma unroll
      for (int i = 0; i < KL; i++) best[i] = cand[i];
      merge_top_desc<KL>(list, best);
    } else {  // KL == 2 * kQCap: the half-cleaner of a 32-wide merge only reaches the lower half of the list (the
      // candidates, padded to the list's length with fillers, meet entries kQCap .. KL-1), in place; the list is then
      // bitonic and holds the KL best of list U cand
      static_assert(KL == 2 * kQCap, "list lengths above the queue width are built for exactly twice that width");
#pragma unroll
      for (int i = kFill; i < kQCap; i++) list[kQCap + i] = __builtin_fmax(list[kQCap + i], cand[kQCap - 1 - i]);
      bitonic_merge_desc<KL>(list);
    }
    qn = 0;
    // threshold = score of the list's last entry (key 0, a filler, maps to a NaN, which fmaxf drops: thr0 remains)
    const uint32_t k32 = key_sortable(list[KL - 1]);
    thr = fmaxf(__uint_as_float(k32 ^ ((k32 & 0x80000000u) ? 0x80000000u : 0xFFFFFFFFu)), thr0);  // fmaxf drops the NaN
    // the partner lane's bound holds for this lane too: K keys of the same query row score at least that much
    thr = fmaxf(thr, __uint_as_float(xh_swap(__float_as_uint(thr))));
  };

  const int ntiles = (int)((Lk + 63) / 64);
  // Fused selection, first sweep: per lane the K largest half-tile maxima, descending
  float top[KL];
#pragma unroll
  for (int i = 0; i < KL; i++) top[i] = -INFINITY;
  if constexpr (!FUSED) {
  fetch(0);
  stash(0);
  if (ntiles > 1) fetch(64);

  for (int t = 0; t < ntiles; t++) {
    const int buf = t & 1;
    const int64_t start = (int64_t)t * 64;
    __syncthreads();  // tile t visible in LDS; everyone is done with buffer buf^1
    if (t + 1 < ntiles) stash(buf ^ 1);
    if (t + 2 < ntiles) fetch(start + 128);
    const bool partial = start + 64 > Lk;

    f32x16 st[2];
    const char* kbase = reinterpret_cast<const char*>(&Ks[buf][0]);
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
#pragma unroll
      for (int r = 0; r < 16; r++) st[kt][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        Frag f;
        f.u = *reinterpret_cast<const uint4*>(kbase + (kt * 32 + c) * 128 + (((ks * 2 + hh) ^ k_swizzle(c)) * 16));
        st[kt] = Mma<E>::mma(as_v8<E>(f), bq[ks], st[kt]);
      }
    }

    if (p.scores != nullptr) {
      float* sbase = p.scores + (((int64_t)b * p.H + h) * Lq + q0) * Lk + start;  // row 0 of this wave, column 0 of the tile
      const bool vec = ((Lk & 3) == 0) && !partial && ((reinterpret_cast<uintptr_t>(p.scores) & 15u) == 0);
      if (vec) {
        // transpose the 32 x 64 score tile through a wave-private LDS stage so that every store instruction
        // writes four full 256-byte row segments (16-byte chunk ch of row r sits at chunk ch ^ (r & 15))
        float* stg = &sstage[wave][0];
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
          for (int g4 = 0; g4 < 4; g4++) {
            const int ch = kt * 8 + 2 * g4 + hh;
            *reinterpret_cast<float4*>(stg + c * 64 + ((ch ^ (c & 15)) * 4)) =
                make_float4(st[kt][4 * g4], st[kt][4 * g4 + 1], st[kt][4 * g4 + 2], st[kt][4 * g4 + 3]);
          }
#pragma unroll
        for (int i = 0; i < 8; i++) {
          const int r = i * 4 + (lane >> 4), ch = lane & 15;
          const float4 v4 = *reinterpret_cast<const float4*>(stg + r * 64 + ((ch ^ (r & 15)) * 4));
          if (q0 + r < Lq) *reinterpret_cast<float4*>(sbase + (int64_t)r * Lk + ch * 4) = v4;
        }
      } else if (qvalid) {
        float* srow = sbase + (int64_t)c * Lk;
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int col = kt * 32 + 4 * hh + 8 * (r >> 2) + (r & 3);
            if (start + col < Lk) srow[col] = st[kt][r];
          }
      }
    }

    const int lim = (int)(Lk - start) - 4 * hh;  // register r of tile kt holds key kt*32 + 4hh + 8(r/4) + r%4
    if (partial) {
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

    const char* vbase = reinterpret_cast<const char*>(&Vs[buf][0]);
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int jj = 0; jj < 2; jj++)
#pragma unroll
        for (int dt = 0; dt < 2; dt++) {
          const char* a0 = vbase + (tr_off ^ (dt * 64)) + (kt * 32 + jj * 16) * 128;
          Frag f;
          f.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
          f.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0 + 8 * 128));
          ot[dt] = Mma<E>::mma(as_v8<E>(f), pf[kt][jj], ot[dt]);
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
  }  // !FUSED

  if constexpr (FUSED) {
    // One sweep over the key tiles: S^T by MFMA, then either the group maxima (first sweep) or the candidate filter
    // (second sweep).  K tiles go global -> LDS by direct transfers into a ring of NB buffers, NB - 1 tiles ahead of
    // the tile being read; wave w moves rows 8 NI w .. 8 NI (w + 1) - 1 of a tile (NI instructions of 8 rows).  LDS chunk
    // (row, c') holds head_dim chunk c' ^ k_swizzle(row).  Rows beyond Lk re-read the last row (they are masked).
    const uint32_t krow_bytes = (uint32_t)p.skn * (uint32_t)sizeof(E);
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);  // the LDS destination of a transfer is a scalar (M0)
    const int dl_row = wave_u * (8 * NI) + (lane >> 3);
    // (the chunk map repeats every 16 rows: instructions of equal parity share it)
    const uint32_t dl_chunk[2] = {(uint32_t)(((lane & 7) ^ k_swizzle(lane >> 3)) * 16), (uint32_t)(((lane & 7) ^ k_swizzle((lane >> 3) + 8)) * 16)};
    uint32_t dl_off[4] = {0, 0, 0, 0};  // NI of them are used
#pragma unroll
    for (int i = 0; i < NI; i++) dl_off[i] = (uint32_t)(dl_row + 8 * i) * krow_bytes + dl_chunk[i & 1];
    auto dma_tile = [&](int t, int buf) {  // tiles past the end repeat the last one (never read)
      const int tt = t < ntiles ? t : ntiles - 1;
      const int64_t start = (int64_t)tt * 64;
      const int rem = (int)(Lk - 1 - start);
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(kp + start * p.skn), 0, 0x7fffffff, 0x00020000);
      char* dst = reinterpret_cast<char*>(&Ks[buf][0]) + wave_u * (NI * 1024);
      uint32_t off[4] = {0, 0, 0, 0};  // the per-lane offsets of a full tile never change
#pragma unroll
      for (int i = 0; i < NI; i++) off[i] = dl_off[i];
      if (__builtin_expect(rem < 63, 0)) {       // ragged last tile: rows beyond the end re-read the last row
#pragma unroll
        for (int i = 0; i < NI; i++) {
          int r = dl_row + 8 * i;
          r = r < rem ? r : rem;
          off[i] = (uint32_t)r * krow_bytes + dl_chunk[i & 1];
          asm volatile("" : "+v"(off[i]));       // stays inside this branch
        }
      }
#pragma unroll
      for (int i = 0; i < NI; i++)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)(dst + i * 1024), 16, off[i], 0, 0, 0);
    };
    const uint32_t lds_k = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)reinterpret_cast<char*>(&Ks[0][0]);
    const uint32_t kr_off = lds_k + (uint32_t)(c * 128 + ((hh ^ k_swizzle(c)) << 4));  // A operand: lane = key row, chunk hh + 2 ks
    auto sweep = [&](auto filter_tag, const int stride) {  // tiles 0, stride, 2 stride, ...
      constexpr bool FILTER = decltype(filter_tag)::value;
      const int nsteps = (ntiles + stride - 1) / stride;
      for (int i = 0; i < NB - 1; i++) dma_tile(i * stride, i);
      int buf = 0, fill = NB - 1;  // ring positions of step i's tile and of step i + NB - 1's
      for (int i = 0; i < nsteps; i++) {
        const int t = i * stride;
        // this wave's share of tile t has landed (transfers complete in order, NI per tile, NB - 2 tiles younger) ...
        __builtin_amdgcn_s_waitcnt(0x0F70 | (NI * (NB - 2)));
        __builtin_amdgcn_s_barrier();  // ... and everybody's; all waves are done with tile t - 1, whose buffer is refilled now
        dma_tile((i + NB - 1) * stride, fill);
        {
          const int64_t start = (int64_t)t * 64;
          const bool partial = start + 64 > Lk;
          u32x4 kf[2][4];
          const uint32_t kb = kr_off + (uint32_t)buf * (kTile * (uint32_t)sizeof(E));
          lds_read_kfrags(kb, kf);
          f32x16 st[2];
#pragma unroll
          for (int kt = 0; kt < 2; kt++) {
#pragma unroll
            for (int r = 0; r < 16; r++) st[kt][r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
              Frag f;
              f.w = kf[kt][ks];
              st[kt] = Mma<E>::mma(as_v8<E>(f), bq[ks], st[kt]);
            }
          }
          buf = buf + 1 == NB ? 0 : buf + 1;
          fill = fill + 1 == NB ? 0 : fill + 1;
          if (partial) {  // last tile only: keys beyond Lk get a score that neither raises a maximum nor passes the filter
            const int lim = (int)(Lk - start) - 4 * hh;  // register r of tile kt holds key kt*32 + 4hh + 8(r/4) + r%4
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
              for (int r = 0; r < 16; r++)
                if (kt * 32 + 8 * (r >> 2) + (r & 3) >= lim) st[kt][r] = FILTER ? __uint_as_float(0x7FC00000u) : -INFINITY;
          }
          if constexpr (!FILTER) {
            float mx = st[0][0];
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
              for (int r = 0; r < 16; r++) mx = fmaxf(mx, st[kt][r]);
            // this lane's maximum over its 32 keys of the tile goes into its descending list of the K largest such
            // maxima (NaN never enters: fmaxf/fminf drop it)
#pragma unroll
            for (int i = 0; i < KL; i++) {
              const float hi = fmaxf(top[i], mx);
              mx = fminf(top[i], mx);
              top[i] = hi;
            }
          } else {
            const uint32_t col0 = (uint32_t)start + 4 * hh;
            const uint32_t qbase = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)reinterpret_cast<char*>(qlane);
            // One test for the whole tile first: the largest of the lane's 32 scores (two chains of three-way maxima, no
            // branch between them; a masked key's NaN loses either way) against the threshold.  Six tiles in seven hold no
            // survivor for any row of the wave at 16 266 keys, and end here instead of after eight group tests with a
            // branch each (top-16: 0.754 -> 0.710 ms; 16 656 keys, top-32: 0.887 -> 0.828 ms).
            bool tile_hit;
            {
              // ordinary VALU reads of both accumulators first: the compiler pads the distance from the MFMAs that
              // wrote them for these instructions, not for inline assembly
              const float s0 = fmaxf(st[0][0], st[0][15]), s1 = fmaxf(st[1][0], st[1][15]);
              asm volatile("" ::"v"(s0), "v"(s1));
              float ma, mb, mt;
              asm("v_max3_f32 %0, %1, %2, %3\n\tv_max3_f32 %0, %0, %4, %5\n\tv_max3_f32 %0, %0, %6, %7\n\tv_max3_f32 %0, %0, %8, %9\n\t"
                  "v_max3_f32 %0, %0, %10, %11\n\tv_max3_f32 %0, %0, %12, %13\n\tv_max3_f32 %0, %0, %14, %15\n\tv_max_f32 %0, %0, %16"
                  : "=&v"(ma)
                  : "v"(st[0][0]), "v"(st[0][1]), "v"(st[0][2]), "v"(st[0][3]), "v"(st[0][4]), "v"(st[0][5]), "v"(st[0][6]), "v"(st[0][7]),
                    "v"(st[0][8]), "v"(st[0][9]), "v"(st[0][10]), "v"(st[0][11]), "v"(st[0][12]), "v"(st[0][13]), "v"(st[0][14]), "v"(st[0][15]));
              asm("v_max3_f32 %0, %1, %2, %3\n\tv_max3_f32 %0, %0, %4, %5\n\tv_max3_f32 %0, %0, %6, %7\n\tv_max3_f32 %0, %0, %8, %9\n\t"
                  "v_max3_f32 %0, %0, %10, %11\n\tv_max3_f32 %0, %0, %12, %13\n\tv_max3_f32 %0, %0, %14, %15\n\tv_max_f32 %0, %0, %16"
                  : "=&v"(mb)
                  : "v"(st[1][0]), "v"(st[1][1]), "v"(st[1][2]), "v"(st[1][3]), "v"(st[1][4]), "v"(st[1][5]), "v"(st[1][6]), "v"(st[1][7]),
                    "v"(st[1][8]), "v"(st[1][9]), "v"(st[1][10]), "v"(st[1][11]), "v"(st[1][12]), "v"(st[1][13]), "v"(st[1][14]), "v"(st[1][15]));
              asm("v_max_f32 %0, %1, %2" : "=v"(mt) : "v"(ma), "v"(mb));
              tile_hit = __builtin_amdgcn_ballot_w64(mt >= thr) != 0;
            }
            if (tile_hit)
#pragma unroll
            for (int g = 0; g < 32 / kGroup; g++) {  // a group of scores, then a drain check
              if ((g % (16 / kGroup)) == 0) {
                // an ordinary VALU read of the accumulator before the hand-written block below: the compiler pads
                // the distance from the MFMA that wrote it for this instruction, not for inline assembly
                const float settled = fmaxf(st[g / (16 / kGroup)][0], st[g / (16 / kGroup)][15]);
                asm volatile("" ::"v"(settled));
              }
              {  // No survivor among the group's 4 x 64 scores (NaNs of masked keys drop out of the maxima): next group, for
                 // two maxima, one compare and one branch instead of four of each.  With K wanted out of several thousand keys,
                 // three groups in four end here (16 266 keys, top-16: 1.11 -> 0.92 ms; 4 164 keys: 0.166 -> 0.152 ms); a
                 // second test over eight registers in front of this one gains 2 % more and is not worth its code.
                const int kt = g / (16 / kGroup), r = (g % (16 / kGroup)) * kGroup;
                float m4;  // two instructions by hand: the compiler's fmaxf quiets every operand first (a NaN loses either way)
                asm("v_max3_f32 %0, %1, %2, %3\n\tv_max_f32 %0, %0, %4"
                    : "=&v"(m4) : "v"(st[kt][r]), "v"(st[kt][r + 1]), "v"(st[kt][r + 2]), "v"(st[kt][r + 3]));
                if (__builtin_amdgcn_ballot_w64(m4 >= thr) == 0) continue;
              }
#pragma unroll
              for (int e8 = 0; e8 < kGroup; e8++) {
                const int kt = g / (16 / kGroup), r = (g % (16 / kGroup)) * kGroup + e8;
                const int koff = kt * 32 + 8 * (r >> 2) + (r & 3);
                // Branch-free append, five VALU instructions: survivors (score >= thr; thr is never a NaN, a masked
                // key's NaN fails) go to queue slot qn, the others to the dump slot; every lane writes (score, column).
                uint32_t slot, col;
                // survivors are a fraction of a percent of the scores: most of the time none of the 64 lanes has one at
                // this register, and the whole append is skipped for one compare and a scalar branch
                if (__builtin_expect(__builtin_amdgcn_ballot_w64(st[kt][r] >= thr) == 0, 1)) continue;
                asm volatile(
                    "v_cmp_ge_f32 vcc, %[s], %[thr]\n\t"
                    "v_cndmask_b32 %[slot], %[dump], %[qn], vcc\n\t"
                    "v_addc_co_u32 %[qn], vcc, 0, %[qn], vcc\n\t"
                    "v_add_u32 %[col], %[koff], %[col0]\n\t"
                    "v_lshl_add_u32 %[slot], %[slot], 9, %[qbase]\n\t"
                    "ds_write2_b32 %[slot], %[s], %[col] offset1:1"
                    : [slot] "=&v"(slot), [col] "=&v"(col), [qn] "+v"(qn)
                    : [s] "v"(st[kt][r]), [thr] "v"(thr), [dump] "n"(kQSlots - 1), [koff] "n"(koff), [col0] "v"(col0), [qbase] "v"(qbase)
                    : "vcc", "memory");
              }
              if (__any(qn > kQSlots - 1 - kGroup)) drain();  // at most kQSlots-1-group queued before a group, at most kQSlots-1 after
            }
          }
        }
      }
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the transfers issued past the last tile are done too
    };
    // First sweep: every lane keeps the K largest of its half-tile maxima (maxima over 32 different keys each).
    // A sample of the tiles is enough: the K-th largest maximum over any subset of the keys is still a lower bound.
    // With fewer sampled tiles the bound is looser (more survivors in the second sweep) but the sweep shorter;
    // about 20 sampled tiles balance the two (measured at 66 and 261 tiles; 16 to 22 are within 1 % of each other, 32
    // and 12 are 2-3 % slower for lists of 16).
    const int stride1 = ntiles >= 64 ? (ntiles / 20 < 12 ? ntiles / 20 : 12) : 1;
    sweep(std::false_type{}, stride1);
    // Threshold: the K-th largest of the row's half-tile maxima, i.e. of the union of the two lanes' lists.  K
    // different scores (one per half tile) are at least that large, so a score below it is not among the K
    // largest, whatever the tie-break.  With fewer than K half tiles it stays -inf and every score is a candidate.
    // The K-th largest of two descending lists a, b is the largest min(a[i-1], b[K-i-1]) over the splits i.
    {
      float tau = fmaxf(top[KL - 1], __uint_as_float(xh_swap(__float_as_uint(top[KL - 1]))));  // splits i = K and i = 0
#pragma unroll
      for (int i = 1; i < KL; i++) {
        const float bi = __uint_as_float(xh_swap(__float_as_uint(top[KL - i - 1])));
        tau = fmaxf(tau, fminf(top[i - 1], bi));
      }
      thr0 = qvalid ? tau : INFINITY;  // rows beyond Lq (all-zero scores) must not flood the queue
      thr = thr0;
    }
    // Second sweep: the scores again (same MFMA sequence, same bits), filtered against the threshold; survivors go
    // through the lane's queue into its exact list.
    __syncthreads();  // every wave is done with the tile buffers of the first sweep
    sweep(std::true_type{}, 1);
    drain();
    // the K best of this lane's list and the partner lane's, descending: max of entry i with the partner's entry
    // K-1-i (a bitonic sequence), two entries at a time so that no second copy of the list is held, then one merge
    auto partner = [&](key_t x) {
      const uint64_t bits = (uint64_t)__double_as_longlong(x);
      const uint32_t lo = xh_swap((uint32_t)bits);
      const uint32_t hi = xh_swap((uint32_t)(bits >> 32));
      return __longlong_as_double((long long)(((uint64_t)hi << 32) | lo));
    };
    if constexpr (KL == 1) {
      list[0] = __builtin_fmax(list[0], partner(list[0]));
    } else {
#pragma unroll
      for (int i = 0; i < KL / 2; i++) {
        const key_t a = list[i], b = list[KL - 1 - i];
        const key_t pa = partner(a), pb = partner(b);
        list[i] = __builtin_fmax(a, pb);
        list[KL - 1 - i] = __builtin_fmax(b, pa);
      }
      bitonic_merge_desc<KL>(list);
    }
    if (qvalid && hh == 0) {
      int32_t* irow = p.topk_idx + (((int64_t)b * p.H + h) * Lq + qrow) * KL;
#pragma unroll
      for (int i = 0; i < KL; i++) irow[i] = (int32_t)(lkm1 - key_rev_col(list[i]));
    }
  }
}

template <typename E>
static int launch_e(const AttnParams& p, bool fused, hipStream_t st) {
  if ((int64_t)p.B * p.H > 65535) return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk: grid too large");
  if (!fused) {
    const int64_t nqg = (p.Lq + 127) / 128;
    if (nqg > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk: grid too large");
    dim3 grid((unsigned)nqg, (unsigned)(p.B * p.H)), blk(256);
    hipLaunchKernelGGL((compressed_mfma_kernel<E, 0, 4>), grid, blk, 0, st, p);
    return check_launch("compressed_mfma_kernel");
  }
  // Workgroups of two waves where those of four would leave the chip one round with idle slots (more than one and a
  // half per CU, at most three) and the pairs still fit it at once (five per CU): 4 164 pooled tokens x 16 heads are 528
  // quads or 1056 pairs, top-16 0.125 -> 0.115 ms, top-32 0.200 -> 0.175 ms.  With more rows the quads' shared tiles win
  // (16 266 tokens: pairs +7 %), with fewer the transfers' latency does (1 041 tokens: pairs +2 .. 15 %).
  const int64_t pairs = ((p.Lq + 63) / 64) * (int64_t)p.B * p.H;
  const bool two = pairs > 3 * 256 && pairs <= 5 * 256;
  const int waves = two ? 2 : 4;
  const int64_t nqg = (p.Lq + 32 * waves - 1) / (32 * waves);
  if (nqg > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk: grid too large");
  dim3 grid((unsigned)nqg, (unsigned)(p.B * p.H)), blk(64 * waves);
#define S3R_LAUNCH_TOPK(K)                                                              \
  case K:                                                                               \
    if (two) hipLaunchKernelGGL((compressed_mfma_kernel<E, K, 2>), grid, blk, 0, st, p); \
    else hipLaunchKernelGGL((compressed_mfma_kernel<E, K, 4>), grid, blk, 0, st, p);     \
    break;
  switch (p.K) {
    S3R_LAUNCH_TOPK(1)
    S3R_LAUNCH_TOPK(2)
    S3R_LAUNCH_TOPK(4)
    S3R_LAUNCH_TOPK(8)
    S3R_LAUNCH_TOPK(16)
    S3R_LAUNCH_TOPK(32)
    default: return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk: fused selection is built for top-k in {1,2,4,8,16,32}");
  }
#undef S3R_LAUNCH_TOPK
  return check_launch("compressed_mfma_kernel");
}

}  // namespace cmp

bool compressed_fused_topk_available(int K) { return K == 1 || K == 2 || K == 4 || K == 8 || K == 16 || K == 32; }

int launch_compressed_mfma(const AttnParams& p, int dtype, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  // With a score buffer: one kernel writes the attention output and the raw scores, the row-wise kernel selects
  // from exactly those values.  Without one: the attention runs as a dense sweep of the selection kernel (its
  // pipelined loop is the fastest attention loop of this library) and the indices come from the top-k-only kernel
  // (two sweeps over S, scores never leave the chip).
  if (p.scores != nullptr) {
    int rc = dtype == S3R_BF16 ? cmp::launch_e<bf16_t>(p, false, st) : cmp::launch_e<f16_t>(p, false, st);
    if (rc != S3R_OK) return rc;
    if (p.topk_idx != nullptr)
      rc = s3r_topk_rows(p.scores, p.topk_idx, (int64_t)p.B * p.H * p.Lq, (int)p.Lk, p.Lk, p.K, stream);
    return rc;
  }
  if (p.topk_idx != nullptr && !compressed_fused_topk_available(p.K))
    return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk: fused selection is built for top-k in {1,2,4,8,16,32}; pass a scores buffer");
  if (p.topk_idx != nullptr && (p.Lk > (1 << 21) || p.skn >= (1 << 24)))
    return fail(S3R_ERR_UNSUPPORTED, "s3r_compressed_attn_topk: fused selection is built for Lk <= 2^21 and key strides < 2^24; pass a scores buffer");
  if (p.o != nullptr) {
    int rc;
    if (p.Lq == p.Lk && p.sqm > 0 && p.skn > 0 && p.svn > 0 && p.sqm < (1 << 20) && p.skn < (1 << 20) && p.svn < (1 << 20)) {
      AttnParams d = p;
      d.idx = nullptr;  // dense sweep
      d.topk_idx = nullptr;
      d.block = 64;
      d.merge_out = nullptr;
      rc = launch_select_pipe(d, dtype, stream);
    } else {
      AttnParams a = p;
      a.topk_idx = nullptr;
      rc = dtype == S3R_BF16 ? cmp::launch_e<bf16_t>(a, false, st) : cmp::launch_e<f16_t>(a, false, st);
    }
    if (rc != S3R_OK) return rc;
  }
  if (p.topk_idx != nullptr) return dtype == S3R_BF16 ? cmp::launch_e<bf16_t>(p, true, st) : cmp::launch_e<f16_t>(p, true, st);
  return S3R_OK;
}

}  // namespace s3r
