// Selection-branch attention for 16-token blocks on the gfx950 matrix cores (bf16 / fp16 I/O, head_dim 64):
// the reference layer's own setting, block_size**2 = 16 with 32 blocks per query block
// (pi3/models/layers/sparse_attention.py:73,98,125; kernel topk_blocksparse_attention.py:35-128).
//
// One wavefront owns four consecutive query blocks (64 queries) of one head; one wave per workgroup.
// The 32x32x16 MFMA wants 32 keys and 32 queries per tile, a query block has only 16 of each per list entry, so a
// tile pairs TWO query blocks with ONE list entry of each: rows 0-15 of the key half tile hold the block the first
// query block lists at position i, rows 16-31 the block the second one lists at position i.  S^T = K Q^T then has
// two useful 16x16 quadrants (first block's keys x first block's queries, second x second); the other two are
// masked to probability zero.  Half of the matrix work is thrown away, which is affordable: this shape is bound by
// the texture path (a 2 KB key block serves 16 queries, a quarter of the reuse of the 64-token case), not by MFMA.
// Everything else follows the 64-token kernels: one query per lane (S^T accumulator), P rounded to the I/O dtype,
// O^T += V^T P^T with V^T fragments from ds_read_b64_tr_b16, K/V half tiles by direct transfers with explicit waits,
// double buffered (the two query-block pairs of the wave alternate, so pair 1's tiles fly while pair 0 computes).
// The softmax is online (running maximum per query, accumulators rescaled only when some maximum moved).
// Entries < 0 or starting at or beyond N are skipped, keys beyond N in the ragged last block are masked, a query
// block with no valid entry gives zeros; up to 64 entries per query block.
#include "select_common.h"
#include "attn_params.h"
#include <stdlib.h>
#include <string.h>

namespace s3r {
namespace b16 {
using namespace sel;

constexpr int kHalfBytes = 32 * 128;
#ifndef S3R_B16_WAVES
#define S3R_B16_WAVES 1
#endif
// wavefronts (groups of four query blocks) per workgroup; the waves do not interact.  One: the unions differ in size
// (cfg-3-like lists: 32 to 127 distinct blocks), and a workgroup keeps its slots until its slowest wave is done
// (4 waves: 1.71 ms, 2: 1.50 ms, 1: 1.42 ms at 266 496 tokens, top-32).
constexpr int kWaves = S3R_B16_WAVES;
constexpr float kLog2e = 1.4426950408889634f;
typedef std::integral_constant<int, 0> H0;
typedef std::integral_constant<int, 1> H1;

// UNION: the wave walks the union of its four lists, see below (default); otherwise pairs of list entries.
template <typename E, bool UNION>
__global__ __launch_bounds__(64 * kWaves, 2) void select_b16_kernel(AttnParams p, int nqb, int ngrp, int nwg_per_bh, int total_wg) {
  typedef typename Mma<E>::V8 V8;
  typedef typename Mma<E>::V2 V2;
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[kWaves * kHalfBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[kWaves * kHalfBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[kWaves * kHalfBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v1[kWaves * kHalfBytes];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int hh = lane >> 5;
  const int c = lane & 31;

  const int w = blockIdx.x;  // XCD-aware: each XCD walks a contiguous range of query groups of one head
  const int xcd = w & 7, slot = w >> 3;
  const int per = total_wg >> 3, rem = total_wg & 7;
  const int vid = xcd * per + (xcd < rem ? xcd : rem) + slot;
  const int bh = vid / nwg_per_bh;
  const int wg = vid - bh * nwg_per_bh;
  const int b = bh / p.H;
  const int h = bh - b * p.H;
  const int grp = wg * kWaves + wave;  // group of four query blocks = 64 queries
  if (grp >= ngrp) return;

  const int64_t N = p.Lq;
  const int64_t q0 = (int64_t)grp * 64;
  const E* qp = (const E*)p.q + (int64_t)b * p.sqb + (int64_t)h * p.sqh;
  const E* kp = (const E*)p.k + (int64_t)b * p.skb + (int64_t)h * p.skh;
  const E* vp = (const E*)p.v + (int64_t)b * p.svb + (int64_t)h * p.svh;
  E* op = (E*)p.o + (int64_t)b * p.sob + (int64_t)h * p.soh;

  char* k_buf[2] = {reinterpret_cast<char*>(lds_k0) + wave * kHalfBytes, reinterpret_cast<char*>(lds_k1) + wave * kHalfBytes};
  char* v_buf[2] = {reinterpret_cast<char*>(lds_v0) + wave * kHalfBytes, reinterpret_cast<char*>(lds_v1) + wave * kHalfBytes};

  // B operand Q: lane = query row, head_dim chunk hh + 2 ks
  V8 bq[2][4];
#pragma unroll
  for (int qt = 0; qt < 2; qt++) {
    const int64_t row = q0 + qt * 32 + c;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      Frag f;
      f.u = make_uint4(0, 0, 0, 0);
      if (row < N) f.u = *reinterpret_cast<const uint4*>(qp + row * p.sqm + ks * 16 + hh * 8);
      bq[qt][ks] = as_v8<E>(f);
    }
  }
  // the four index rows of the group, one entry per lane
  int32_t my_idx[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int qb = grp * 4 + j;
    my_idx[j] = -1;
    if (qb < nqb && lane < p.K) my_idx[j] = p.idx[(int64_t)b * p.sib + (int64_t)h * p.sih + (int64_t)qb * p.sim + lane];
    if (my_idx[j] < 0 || (int64_t)my_idx[j] * 16 >= N) my_idx[j] = -1;
  }

  f32x16 ot[2][2];  // O^T [dt][qt]
#pragma unroll
  for (int dt = 0; dt < 2; dt++)
#pragma unroll
    for (int qt = 0; qt < 2; qt++)
#pragma unroll
      for (int r = 0; r < 16; r++) ot[dt][qt][r] = 0.f;
  float m_i[2] = {-INFINITY, -INFINITY}, l_i[2] = {0.f, 0.f};
  const float sl2 = p.scale * kLog2e;
  const uint32_t krow = (uint32_t)p.skn * (uint32_t)sizeof(E), vrow = (uint32_t)p.svn * (uint32_t)sizeof(E);

  // per-lane pieces of the transfers and reads
  const int lr = lane >> 3;
  const int i16 = lane & 15;
  const int tr_row = 4 * hh + (i16 >> 2);
  const int tr_chunk = (((lane >> 4) & 1) * 2 + ((i16 & 3) >> 1)) ^ (((tr_row >> 1) & 1) << 2);
  const int tr_off = tr_row * 128 + tr_chunk * 16 + (i16 & 1) * 8;
  const int kr_off = c * 128 + ((hh ^ (c & 7)) << 4);

  // Unit (i, QT): list position i of query blocks 2 QT and 2 QT + 1.  blk[0], blk[1]: their key blocks (-1: skip).
  auto entry = [&](int i, auto qt_tag, int32_t (&blk)[2]) {
    constexpr int QT = decltype(qt_tag)::value;
    blk[0] = __builtin_amdgcn_readlane(my_idx[2 * QT], i);
    blk[1] = __builtin_amdgcn_readlane(my_idx[2 * QT + 1], i);
  };
  auto fetch = [&](int i, auto qt_tag) {  // the unit's K and V half tiles -> buffers QT (skipped blocks re-read block 0)
    constexpr int QT = decltype(qt_tag)::value;
    int32_t blk[2];
    entry(i, qt_tag, blk);
#pragma unroll
    for (int s = 0; s < 2; s++) {
      const int64_t start = (int64_t)(blk[s] < 0 ? 0 : blk[s]) * 16;
      const int last = (int)((N - start < 16 ? N - start : 16) - 1);
      const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc((void*)(kp + start * p.skn), 0, 0x7fffffff, 0x00020000);
      const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc((void*)(vp + start * p.svn), 0, 0x7fffffff, 0x00020000);
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const int ldsrow = 16 * s + 8 * t + lr;   // row of the 32-row half tile
        int row = 8 * t + lr;                     // row of the 16-token block
        row = row < last ? row : last;
        const uint32_t kc = (uint32_t)(((lane & 7) ^ (ldsrow & 7)) * 16);
        const uint32_t vc = (uint32_t)(((lane & 7) ^ (((ldsrow >> 1) & 1) << 2)) * 16);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (__attribute__((address_space(3))) void*)(k_buf[QT] + (2 * s + t) * 1024), 16,
                                                 (uint32_t)row * krow + kc, 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (__attribute__((address_space(3))) void*)(v_buf[QT] + (2 * s + t) * 1024), 16,
                                                 (uint32_t)row * vrow + vc, 0, 0, 0);
      }
    }
  };
  auto compute = [&](int i, auto qt_tag) {
    constexpr int QT = decltype(qt_tag)::value;
    int32_t blk[2];
    entry(i, qt_tag, blk);
    // this lane's query belongs to block `mine` of the pair; only that block's 16 keys count for it
    const int mine = c >> 4;
    const int32_t myblk = mine == 0 ? blk[0] : blk[1];
    const int nkeys = myblk < 0 ? 0 : (int)(N - (int64_t)myblk * 16 < 16 ? N - (int64_t)myblk * 16 : 16);
    V8 ak[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      Frag f;
      f.u = *reinterpret_cast<const uint4*>(k_buf[QT] + (kr_off ^ (ks << 5)));
      ak[ks] = as_v8<E>(f);
    }
    f32x16 st;
#pragma unroll
    for (int r = 0; r < 16; r++) st[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) st = Mma<E>::mma(ak[ks], bq[QT][ks], st);
    // register r holds key row 4hh + 8(r/4) + r%4 of the half tile: rows 0-15 (r < 8) are block 0's keys, 16-31 block
    // 1's.  Only the 8 registers of this lane's own block are scores of its query: they are picked first, and the
    // softmax runs on 8 values instead of 16.
    const uint32_t m0 = mine == 0 ? 0xFFFFFFFFu : 0u;  // bit masks instead of per-value selects on a condition register
    const uint32_t own_sel = mine == 0 ? 0x07060504u : 0x03020100u;  // v_perm_b32 selector: all four bytes of the first / second source
    float su[8];
#pragma unroll
    for (int j = 0; j < 8; j++) su[j] = __uint_as_float(__builtin_amdgcn_perm(__float_as_uint(st[j]), __float_as_uint(st[8 + j]), own_sel));
    if (__any(nkeys < 16)) {  // a ragged last block or a skipped entry somewhere in the wave
#pragma unroll
      for (int j = 0; j < 8; j++)
        if (4 * hh + 8 * (j >> 2) + (j & 3) >= nkeys) su[j] = -INFINITY;
    }
    float mx = su[0];
#pragma unroll
    for (int j = 1; j < 8; j++) mx = fmaxf(mx, su[j]);
    mx = xh_max(mx) * sl2;  // sl2 > 0: the maximum of the scaled scores
    const float m_new = fmaxf(m_i[QT], mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;   // nothing valid so far: every probability is exp2(-inf) = 0
    const float alpha = __builtin_amdgcn_exp2f(m_i[QT] - m_use);  // 0 while m_i is -inf
    if (__any(m_new != m_i[QT])) {
      l_i[QT] *= alpha;
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) ot[dt][QT][r] *= alpha;
    }
    m_i[QT] = m_new;
    // probabilities of the own block, then the B operand of the PV product: the own block's k-group carries them,
    // the other block's k-group zeros
    union { V8 v; uint32_t w[4]; } pown, pf[2];
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
      V2 pk;
      pk[0] = (E)__builtin_amdgcn_exp2f(fmaf(su[e], sl2, -m_use));
      pk[1] = (E)__builtin_amdgcn_exp2f(fmaf(su[e + 1], sl2, -m_use));
      pown.v[e] = pk[0];
      pown.v[e + 1] = pk[1];
      l_i[QT] = Mma<E>::dot_ones(pk, l_i[QT]);
    }
#pragma unroll
    for (int wi = 0; wi < 4; wi++) {
      pf[0].w[wi] = pown.w[wi] & m0;
      pf[1].w[wi] = pown.w[wi] & ~m0;
    }
    V8 vfr[2][2];
#pragma unroll
    for (int jj = 0; jj < 2; jj++)
#pragma unroll
      for (int dt = 0; dt < 2; dt++) {
        const char* a0 = v_buf[QT] + (tr_off ^ (dt * 64)) + (jj * 16) * 128;
        Frag f;
        f.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
        f.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0 + 8 * 128));
        vfr[jj][dt] = as_v8<E>(f);
      }
#pragma unroll
    for (int jj = 0; jj < 2; jj++)
#pragma unroll
      for (int dt = 0; dt < 2; dt++) ot[dt][QT] = Mma<E>::mma(vfr[jj][dt], pf[jj].v, ot[dt][QT]);
  };

  if constexpr (UNION) {
    // Neighbouring query blocks list mostly the same key blocks.  The wave therefore walks the UNION of its four
    // lists: a tile is two distinct key blocks A, B (rows 0-15, 16-31), fetched once, and every one of the 64 queries
    // whose block lists A (B) uses its 16 scores against A (B); cnt bytes say how often query block j lists the
    // block (0: not at all, its scores are masked; above 1: a duplicated entry, the probabilities count that often).
    // The visiting order differs from the lists' order, which changes fp32 summation order only.
    uint64_t rem[4];
    bool exact = false;  // second walk: running maximum
    auto pop = [&](int32_t& blk, uint32_t& cnts) {  // next distinct key block and its four multiplicities, or -1
      blk = -1;
      cnts = 0;
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (blk < 0 && rem[j] != 0) blk = __builtin_amdgcn_readlane(my_idx[j], __ffsll((unsigned long long)rem[j]) - 1);
      if (blk >= 0) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const uint64_t hit = __ballot(my_idx[j] == blk) & rem[j];
          rem[j] &= ~hit;
          cnts |= (uint32_t)__popcll(hit) << (8 * j);
        }
      }
    };
    auto fetch_u = [&](int buf, int32_t ba, int32_t bb) {  // K and V rows of blocks A, B -> buffers buf (no B: block 0 again)
      char* kb = buf ? k_buf[1] : k_buf[0];
      char* vb = buf ? v_buf[1] : v_buf[0];
#pragma unroll
      for (int s = 0; s < 2; s++) {
        const int32_t blk = s == 0 ? ba : bb;
        const int64_t start = (int64_t)(blk < 0 ? 0 : blk) * 16;
        const int last = (int)((N - start < 16 ? N - start : 16) - 1);
        const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc((void*)(kp + start * p.skn), 0, 0x7fffffff, 0x00020000);
        const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc((void*)(vp + start * p.svn), 0, 0x7fffffff, 0x00020000);
#pragma unroll
        for (int t = 0; t < 2; t++) {
          const int ldsrow = 16 * s + 8 * t + lr;
          int row = 8 * t + lr;
          row = row < last ? row : last;
          const uint32_t kc = (uint32_t)(((lane & 7) ^ (ldsrow & 7)) * 16);
          const uint32_t vc = (uint32_t)(((lane & 7) ^ (((ldsrow >> 1) & 1) << 2)) * 16);
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (__attribute__((address_space(3))) void*)(kb + (2 * s + t) * 1024), 16,
                                                   (uint32_t)row * krow + kc, 0, 0, 0);
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (__attribute__((address_space(3))) void*)(vb + (2 * s + t) * 1024), 16,
                                                   (uint32_t)row * vrow + vc, 0, 0, 0);
        }
      }
    };
    V8 ak[4];       // K fragments of the current tile
    V8 vfr[2][2];   // V^T fragments of the current tile [jj][dt]
    auto load_frags = [&](int buf) {
      const char* kb = buf ? k_buf[1] : k_buf[0];
      const char* vb = buf ? v_buf[1] : v_buf[0];
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        Frag f;
        f.u = *reinterpret_cast<const uint4*>(kb + (kr_off ^ (ks << 5)));
        ak[ks] = as_v8<E>(f);
      }
#pragma unroll
      for (int jj = 0; jj < 2; jj++)
#pragma unroll
        for (int dt = 0; dt < 2; dt++) {
          const char* a0 = vb + (tr_off ^ (dt * 64)) + (jj * 16) * 128;
          Frag f;
          f.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
          f.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0 + 8 * 128));
          vfr[jj][dt] = as_v8<E>(f);
        }
    };
    auto compute_u = [&](int32_t ba, uint32_t ca, int32_t bb, uint32_t cb) {  // on the fragments in registers
      const int nka = (int)(N - (int64_t)ba * 16 < 16 ? N - (int64_t)ba * 16 : 16);
      const int nkb = bb < 0 ? 0 : (int)(N - (int64_t)bb * 16 < 16 ? N - (int64_t)bb * 16 : 16);
      const int mine = c >> 4;
      // The three stages of a 32-query half (one half after the other: interleaving the two halves' stages was slower).
      f32x16 st[2];
      union { V8 v; } pf[2][2];
      auto scores = [&](auto qt_tag) {
        constexpr int QT = decltype(qt_tag)::value;
#pragma unroll
        for (int r = 0; r < 16; r++) st[QT][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) st[QT] = Mma<E>::mma(ak[ks], bq[QT][ks], st[QT]);
      };
      auto softmax = [&](auto qt_tag) {
        constexpr int QT = decltype(qt_tag)::value;
        const uint32_t pa = (ca >> (16 * QT)) & 0xffffu, pb = (cb >> (16 * QT)) & 0xffffu;  // the half's two query blocks
        const int wa = (int)(mine ? pa >> 8 : pa & 0xffu), wb = (int)(mine ? pb >> 8 : pb & 0xffu);
        // register r: key row 4hh + 8((r%8)/4) + r%4 of block A (r < 8) or B (r >= 8).  A block that the lane's query
        // block does not list is left out through two per-lane constants (its maximum is dropped and its exponent gets
        // -inf added); only the ragged last block needs per-register masks.
        if (__any((wa && nka < 16) || (wb && nkb < 16))) {
#pragma unroll
          for (int j = 0; j < 8; j++) {
            const int row = 4 * hh + 8 * (j >> 2) + (j & 3);
            if (row >= nka) st[QT][j] = -INFINITY;
            if (row >= nkb) st[QT][8 + j] = -INFINITY;
          }
        }
        // Softmax reference.  First walk (exact == false): a query's reference is the maximum over the first tile that
        // holds a block of its list and then stays (softmax is shift invariant), so later tiles need no maximum, no
        // comparison and no pass over the accumulators; probabilities may exceed 1, and a row sum that ends up huge or
        // not finite sends the group through a second walk with the running maximum (exact == true).
        const bool unset = m_i[QT] == -INFINITY && (wa | wb) != 0;
        if (exact || __any(unset)) {
          float mxa = st[QT][0], mxb = st[QT][8];
#pragma unroll
          for (int r = 1; r < 8; r++) {
            mxa = fmaxf(mxa, st[QT][r]);
            mxb = fmaxf(mxb, st[QT][8 + r]);
          }
          float mx = fmaxf(wa ? mxa : -INFINITY, wb ? mxb : -INFINITY);
          mx = xh_max(mx) * sl2;
          const float m_new = (exact || unset) ? fmaxf(m_i[QT], mx) : m_i[QT];
          if (__any(m_new != m_i[QT])) {
            const float alpha = __builtin_amdgcn_exp2f(m_i[QT] - (m_new == -INFINITY ? 0.f : m_new));  // 0 while m_i is -inf
            l_i[QT] *= alpha;
#pragma unroll
            for (int dt = 0; dt < 2; dt++)
#pragma unroll
              for (int r = 0; r < 16; r++) ot[dt][QT][r] *= alpha;
          }
          m_i[QT] = m_new;
        }
        const float m_use = m_i[QT] == -INFINITY ? 0.f : m_i[QT];
        const float nega = wa ? -m_use : -INFINITY, negb = wb ? -m_use : -INFINITY;  // -inf: every probability 0
        const bool dup = __any(wa > 1 || wb > 1);
        const float fa = (float)wa, fb = (float)wb;
#pragma unroll
        for (int jj = 0; jj < 2; jj++)
#pragma unroll
          for (int e = 0; e < 8; e += 2) {
            float x0 = __builtin_amdgcn_exp2f(fmaf(st[QT][8 * jj + e], sl2, jj == 0 ? nega : negb));
            float x1 = __builtin_amdgcn_exp2f(fmaf(st[QT][8 * jj + e + 1], sl2, jj == 0 ? nega : negb));
            if (dup) {  // a list that names the block more than once attends it that often
              x0 *= jj == 0 ? fa : fb;
              x1 *= jj == 0 ? fa : fb;
            }
            V2 pk;
            pk[0] = (E)x0;
            pk[1] = (E)x1;
            pf[QT][jj].v[e] = pk[0];
            pf[QT][jj].v[e + 1] = pk[1];
            l_i[QT] = Mma<E>::dot_ones(pk, l_i[QT]);
          }
      };
      auto values = [&](auto qt_tag) {
        constexpr int QT = decltype(qt_tag)::value;
#pragma unroll
        for (int jj = 0; jj < 2; jj++)
#pragma unroll
          for (int dt = 0; dt < 2; dt++) ot[dt][QT] = Mma<E>::mma(vfr[jj][dt], pf[QT][jj].v, ot[dt][QT]);
      };
      // (wave-uniform) does some query of the half list A or B?
      const bool act0 = ((ca | cb) & 0xffffu) != 0, act1 = ((ca | cb) >> 16) != 0;
      if (act0) {
        scores(H0{});
        softmax(H0{});
        values(H0{});
      }
      if (act1) {
        scores(H1{});
        softmax(H1{});
        values(H1{});
      }
    };
    for (int pass = 0; pass < 2; pass++) {
      exact = pass == 1;
#pragma unroll
      for (int j = 0; j < 4; j++) rem[j] = __ballot(my_idx[j] >= 0);
      int32_t a0, b0;
      uint32_t ca0, cb0;
      pop(a0, ca0);
      pop(b0, cb0);
      if (a0 >= 0) {
        int buf = 0;
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): (second walk) the first walk's last reads are done
        // Two tiles in flight: a tile's fragments go to registers in one go, which frees its buffers for the tile
        // after the next before any arithmetic starts.
        fetch_u(0, a0, b0);
        int32_t a1, b1;
        uint32_t ca1, cb1;
        pop(a1, ca1);
        pop(b1, cb1);
        if (a1 >= 0) fetch_u(1, a1, b1);
        while (true) {
          if (a1 >= 0) __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): the current tile has landed (the next one may be in flight)
          else __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0)
          load_frags(buf);
          __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the fragments are in registers, the buffers are free
          int32_t a2, b2;
          uint32_t ca2, cb2;
          pop(a2, ca2);
          pop(b2, cb2);
          if (a2 >= 0) fetch_u(buf, a2, b2);
          compute_u(a0, ca0, b0, cb0);
          if (a1 < 0) break;
          a0 = a1; ca0 = ca1; b0 = b1; cb0 = cb1;
          a1 = a2; ca1 = ca2; b1 = b2; cb1 = cb2;
          buf ^= 1;
        }
      }
      const float big = 1.2676506e30f;  // 2^100
      if (exact || !__any(!(l_i[0] < big) || !(l_i[1] < big))) break;
      // rare: some reference was far too low; start over with the running maximum
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int qt = 0; qt < 2; qt++)
#pragma unroll
          for (int r = 0; r < 16; r++) ot[dt][qt][r] = 0.f;
      m_i[0] = m_i[1] = -INFINITY;
      l_i[0] = l_i[1] = 0.f;
    }
  } else {
  const int nsteps = p.K;
    if (nsteps > 0) {
      fetch(0, H0{});
      for (int i = 0; i < nsteps; i++) {
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the reads of buffers 1 (previous step) are done
        fetch(i, H1{});
        __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): unit (i, 0) has landed
        compute(i, H0{});
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the reads of buffers 0 are done
        if (i + 1 < nsteps) {
          fetch(i + 1, H0{});
          __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): unit (i, 1) has landed
        } else {
          __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        }
        compute(i, H1{});
      }
    }
  
}

  // output: as in the 64-token kernels (one exchange with lane ^ 32 per packed word, 16-byte stores).  With merge
  // operands the gated merge runs here (gate pair of the row, the compressed output of the row's 16-token block; the
  // three roundings of the eager expression kept) and the result goes to the [B, N, H*D] tensor.
  const bool merge = p.merge_out != nullptr;
#pragma unroll
  for (int qt = 0; qt < 2; qt++) {
    const float l = xh_sum(l_i[qt]);
    const float inv = l > 0.f ? 1.f / l : 0.f;
    const int64_t row = q0 + qt * 32 + c;
    const bool live = row < N;
    float g0 = 0.f, g1 = 0.f;
    const E* ocp = nullptr;
    if (merge && live) {
      const E* gp = (const E*)p.merge_gate + (int64_t)b * p.sgb + (int64_t)h * p.sgh + row * p.sgn;
      g0 = (float)gp[0];
      g1 = (float)gp[1];
      ocp = (const E*)p.merge_oc + (int64_t)b * p.scb + (int64_t)h * p.sch + (row >> 4) * p.scm;
    }
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
      for (int gp = 0; gp < 2; gp++) {
        union { E e[8]; uint32_t w[4]; uint4 u; } pc;
        union { E e[2]; uint32_t w; } t;
#pragma unroll
        for (int wi = 0; wi < 2; wi++) {
          t.e[0] = (E)(ot[dt][qt][8 * gp + 2 * wi] * inv);
          t.e[1] = (E)(ot[dt][qt][8 * gp + 2 * wi + 1] * inv);
          const uint32_t a = t.w;
          t.e[0] = (E)(ot[dt][qt][8 * gp + 4 + 2 * wi] * inv);
          t.e[1] = (E)(ot[dt][qt][8 * gp + 4 + 2 * wi + 1] * inv);
          const uint32_t bw = t.w;
          const auto r = __builtin_amdgcn_permlane32_swap(a, bw, false, false);
          pc.w[wi] = r[0];
          pc.w[2 + wi] = r[1];
        }
        const int d0 = dt * 32 + 8 * (2 * gp + hh);
        if (live) {
          if (!merge) {
            *reinterpret_cast<uint4*>(op + row * p.som + d0) = pc.u;
          } else {
            union { E e[8]; uint4 u; } oc, res;
            oc.u = *reinterpret_cast<const uint4*>(ocp + d0);
#pragma unroll
            for (int e = 0; e < 8; e++) {
              const float x = round_to<E>(g0 * (float)oc.e[e]);
              const float y = round_to<E>(g1 * (float)pc.e[e]);
              res.e[e] = (E)(x + y);
            }
            *reinterpret_cast<uint4*>((E*)p.merge_out + (((int64_t)b * N + row) * p.H + h) * 64 + d0) = res.u;
          }
        }
      }
    if (live && p.lse != nullptr && hh == 0)
      p.lse[((int64_t)b * p.H + h) * N + row] = l > 0.f ? (m_i[qt] + __builtin_amdgcn_logf(l)) * 0.6931471805599453f : -INFINITY;
  }
}

}  // namespace b16

int launch_select_b16(const AttnParams& p, int dtype, void* stream) {
  const int64_t nqb = (p.Lq + 15) / 16;
  const int64_t ngrp = (nqb + 3) / 4;
  const int64_t nwg = (ngrp + b16::kWaves - 1) / b16::kWaves;
  const int64_t total = nwg * p.B * p.H;
  if (total > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_select_attn: grid too large");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)total), blk(64 * b16::kWaves);
  // default: the union walk; S3R_B16_KERNEL=pairs picks the walk over pairs of list entries (kept as a cross-check)
  static const bool pairs = [] {
    const char* e = getenv("S3R_B16_KERNEL");
    return e != nullptr && strcmp(e, "pairs") == 0;
  }();
#define S3R_B16(E, U) hipLaunchKernelGGL((b16::select_b16_kernel<E, U>), grid, blk, 0, st, p, (int)nqb, (int)ngrp, (int)nwg, (int)total)
  if (dtype == S3R_BF16) {
    if (pairs) S3R_B16(bf16_t, false); else S3R_B16(bf16_t, true);
  } else {
    if (pairs) S3R_B16(f16_t, false); else S3R_B16(f16_t, true);
  }
#undef S3R_B16
  return check_launch("select_b16_kernel");
}

}  // namespace s3r
