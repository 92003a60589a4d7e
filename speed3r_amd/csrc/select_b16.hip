// Selection-branch attention for 16-token blocks on the gfx950 matrix cores (bf16 / fp16 I/O, head_dim 64):
// the reference layer's own setting, block_size**2 = 16 with 32 blocks per query block
// (pi3/models/layers/sparse_attention.py:73,98,125; kernel topk_blocksparse_attention.py:35-128).
//
// One wavefront owns four consecutive query blocks (64 queries) of one head; one wave per workgroup.
// The 32x32x16 MFMA wants 32 keys and 32 queries per tile, a list entry offers 16 keys for 16 queries.  Two walks:
//  * union walk (default): the wave walks the UNION of its four lists, two distinct key blocks per tile, all 64
//    queries scored against both (neighbouring query blocks list mostly the same blocks, so most quadrants are
//    useful); walk list built first, then a software pipeline over (tile, query half) units, see the kernel body;
//  * pair walk (S3R_B16_KERNEL=pairs, cross-check, and tensors beyond 4 GB per head): a tile pairs TWO query blocks
//    with ONE list entry of each, rows 0-15 of the key half tile hold the block the first query block lists at
//    position i, rows 16-31 the block the second one lists at position i; S^T = K Q^T then has two useful 16x16
//    quadrants, the other two are masked to probability zero; online softmax on the 8 own registers.
// Everything else follows the 64-token kernels: one query per lane (S^T accumulator), P rounded to the I/O dtype,
// O^T += V^T P^T with V^T fragments from ds_read_b64_tr_b16, K/V half tiles by direct transfers with explicit waits.
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
// (measured on the walk before the pipeline: 4 waves 1.71 ms, 2: 1.50 ms, 1: 1.42 ms at 266 496 tokens, top-32).
constexpr int kWaves = S3R_B16_WAVES;
constexpr float kLog2e = 1.4426950408889634f;
typedef std::integral_constant<int, 0> H0;
typedef std::integral_constant<int, 1> H1;

// UNION: the wave walks the union of its four lists, see below (default); otherwise pairs of list entries.
// WIDE (union walk): K or V rows lie 4 GiB or more behind the tensor's first row (beyond a 32-bit byte offset).
template <typename E, bool UNION, bool WIDE>
__global__ __launch_bounds__(64 * kWaves, 2) void select_b16_kernel(AttnParams p, int nqb, int ngrp, int nwg_per_bh, int total_wg) {
  typedef typename Mma<E>::V8 V8;
  typedef typename Mma<E>::V2 V2;
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[kWaves * kHalfBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[kWaves * kHalfBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[kWaves * kHalfBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v1[kWaves * kHalfBytes];

  const int wave = kWaves == 1 ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
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

  // The four index rows of the group, one entry per lane.  They head the longest dependency chain of the start-up
  // (rows -> walk list -> first tiles): their loads go first, ahead of the Q rows in the memory queue.
  int32_t my_idx[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int qb = grp * 4 + j;
    my_idx[j] = -1;
    if (qb < nqb && lane < p.K) my_idx[j] = __builtin_nontemporal_load(p.idx + ((int64_t)b * p.sib + (int64_t)h * p.sih + (int64_t)qb * p.sim + lane));
  }
  __builtin_amdgcn_sched_barrier(0);
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
#pragma unroll
  for (int j = 0; j < 4; j++)
    if (my_idx[j] < 0 || (int64_t)my_idx[j] * 16 >= N) my_idx[j] = -1;

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
  const int kr_off = c * 128 + ((hh ^ k_swizzle(c)) << 4);

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
        const uint32_t kc = (uint32_t)(((lane & 7) ^ k_swizzle(ldsrow)) * 16);
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
    // whose block lists A (B) uses its 16 scores against A (B).  The visiting order differs from the lists' order,
    // which changes fp32 summation order only.
    //
    // 1. The walk list is built first, in LDS: entry n holds a distinct block and four count bytes (how often query
    //    block j lists it; 0: not at all, above 1: a duplicated entry, which attends the block that often).
    // 2. A software pipeline over units (tile t, half h of the 64 queries) then walks the list.  While the
    //    exponentials of unit u run on the VALU, the matrix pipe takes the scores of unit u + 1 and the PV product of
    //    unit u - 1, one MFMA per two exponentials.  K and V tiles come by direct transfers into two half buffers
    //    each, 1.5 tile times ahead of their use; all buffer choices are static (the loop is written for even and odd
    //    tiles), so that the only waits for transfers are the explicit ones.
    uint64_t lanes_any[2];  // lanes (queries) of each half whose query block has at least one valid entry
#pragma unroll
    for (int qt = 0; qt < 2; qt++)
      lanes_any[qt] = (__ballot(my_idx[2 * qt] >= 0) ? 0x0000FFFF0000FFFFull : 0ull) | (__ballot(my_idx[2 * qt + 1] >= 0) ? 0xFFFF0000FFFF0000ull : 0ull);
    __shared__ __attribute__((aligned(16))) int2 lds_walk[kWaves][264];  // up to 4 x 64 entries and the end mark
    int2* const walk = lds_walk[wave];
    const int32_t ragged_blk = (N & 15) ? (int32_t)(N >> 4) : -2;  // the block that ends before its 16th row ...
    const int ragged_last = (int)(N & 15) - 1;
    uint32_t ragged_cnts = 0;  // ... stays out of the list: it gets a step of its own after the pipeline
    // The distinct blocks and their counts come from a hash table in LDS (512 slots in the first K buffer, which
    // the pipeline does not touch before the list is complete): every lane inserts its entry of list j with a
    // compare-and-swap on the key (linear probing; at most 256 distinct blocks) and adds 1 << 8j to the slot's count;
    // then the occupied slots are compacted into the list, eight slots per lane, positions from ballots.  The list's
    // order is the table's, which is as good as any.
    int n_union = 0;
    uint32_t cnt_bits = 0;
    {
      int32_t* const hkey = reinterpret_cast<int32_t*>(k_buf[0]);          // [512]
      uint32_t* const hcnt = reinterpret_cast<uint32_t*>(k_buf[0] + 2048);  // [512]
      reinterpret_cast<int4*>(hkey)[lane] = make_int4(-1, -1, -1, -1);
      reinterpret_cast<int4*>(hkey)[lane + 64] = make_int4(-1, -1, -1, -1);
      reinterpret_cast<int4*>(hcnt)[lane] = make_int4(0, 0, 0, 0);
      reinterpret_cast<int4*>(hcnt)[lane + 64] = make_int4(0, 0, 0, 0);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int32_t e = my_idx[j];
        ragged_cnts |= (uint32_t)__popcll(__ballot(e == ragged_blk)) << (8 * j);
        bool active = e >= 0 && e != ragged_blk;
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
      if (lane == 0) walk[n_union] = make_int2(-1, 0);
      cnt_bits = __any((cnt_bits & 0xfefefefeu) != 0) ? 2u : 0u;
      cnt_bits |= ragged_cnts;
    }
    const bool dup = (cnt_bits & 0xfefefefeu) != 0;  // some list names a block more than once (wave-uniform)
    // tile tau = entries 2 tau, 2 tau + 1 of the walk list (-1 / no counts beyond its end): the read is issued early
    // and its result taken where it is needed
    auto lookup_issue = [&](int tau) -> int4 {
      const int e = 2 * tau;
      int4 v = make_int4(-1, 0, -1, 0);
      if (e < n_union) v = *reinterpret_cast<const int4*>(walk + e);
      return v;
    };
    auto lookup_take = [&](const int4& v, int32_t& a, uint32_t& ca, int32_t& b2, uint32_t& cb) {
      a = __builtin_amdgcn_readfirstlane(v.x);
      ca = (uint32_t)__builtin_amdgcn_readfirstlane(v.y);
      b2 = __builtin_amdgcn_readfirstlane(v.z);
      cb = (uint32_t)__builtin_amdgcn_readfirstlane(v.w);
    };

    // ---- transfers: one descriptor per block, based at the block's first row (a 64-bit address: byte offsets inside
    // the instruction stay below 16 rows, whatever the row stride and the sequence length) ----
    // (the K swizzle of a block's rows 8..15 differs from that of its rows 0..7: one offset per instruction of a block)
    const uint32_t koff = (uint32_t)lr * krow + (uint32_t)(((lane & 7) ^ k_swizzle(lr)) * 16);
    const uint32_t koff8 = (uint32_t)lr * krow + (uint32_t)(((lane & 7) ^ k_swizzle(lr + 8)) * 16);
    const uint32_t voff = (uint32_t)lr * vrow + (uint32_t)(((lane & 7) ^ (((lr >> 1) & 1) << 2)) * 16);
    typedef __attribute__((address_space(3))) char* LdsPtr;  // arithmetic stays in the LDS address space (no null checks)
    const LdsPtr k_lds[2] = {(LdsPtr)lds_k0 + wave * kHalfBytes, (LdsPtr)lds_k1 + wave * kHalfBytes};
    const LdsPtr v_lds[2] = {(LdsPtr)lds_v0 + wave * kHalfBytes, (LdsPtr)lds_v1 + wave * kHalfBytes};
    // 16 rows of one block -> 2 KB at dst.  The instruction's immediate offset moves the LDS side and the global side
    // alike; the scalar offset makes up the difference (row strides are at least 128 bytes).
    // WIDE (a tensor whose last row lies 4 GiB or more behind its first): the descriptor is based at the block itself,
    // a 64-bit address; otherwise at the tensor, and the block's byte offset rides in the 32-bit scalar offset (a
    // multiplication less per block)
    auto dma_block = [&](const E* base, int64_t row_elems, int32_t rec, LdsPtr dst, uint32_t off0, uint32_t off8, uint32_t rowb, int32_t blk) {
      const int64_t far = WIDE ? (int64_t)blk * 16 * row_elems : 0;
      const uint32_t so = WIDE ? 0u : (uint32_t)blk * 16u * rowb;
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(base + far), 0, rec, 0x00020000);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, off0, so, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, off8, so + (8u * rowb - 1024u), 1024, 0);
    };
    auto dma_ragged = [&](const E* base, int64_t row_elems, LdsPtr dst, uint32_t off0, uint32_t off8, uint32_t rowb) {  // rows beyond the sequence re-read its last row
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(base + (int64_t)ragged_blk * 16 * row_elems), 0, -1, 0x00020000);
      const int r0 = lr < ragged_last ? lr : ragged_last, r1 = 8 + lr < ragged_last ? 8 + lr : ragged_last;
      const uint32_t col0 = off0 - (uint32_t)lr * rowb, col8 = off8 - (uint32_t)lr * rowb;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, (uint32_t)r0 * rowb + col0, 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst + 1024, 16, (uint32_t)r1 * rowb + col8, 0, 0, 0);
    };
    // A tile beyond the end of the list (a < 0) is requested all the same, through a descriptor of zero records:
    // every lane is out of range, nothing is fetched, and the count of outstanding transfers does not depend on the
    // list (the waits below are constants).  No second block: the first one again (finite scores).
    auto records = [](int32_t a) -> int32_t {  // -1 (no limit) for a block, 0 for none; scalar instructions by hand: the
      int32_t r;                               // compiler's own select lands in a vector register and the descriptor with it
      asm("s_ashr_i32 %0, %1, 31\n\ts_not_b32 %0, %0" : "=s"(r) : "s"(a) : "scc");
      return r;
    };
    auto dma_k = [&](auto par_tag, int32_t a, int32_t b2) {
      constexpr int P = decltype(par_tag)::value;
      const int32_t rec = records(a);
      dma_block(kp, p.skn, rec, k_lds[P], koff, koff8, krow, a);
      dma_block(kp, p.skn, rec, k_lds[P] + 2048, koff, koff8, krow, b2 < 0 ? a : b2);
    };
    auto dma_v = [&](auto par_tag, int32_t a, int32_t b2) {
      constexpr int P = decltype(par_tag)::value;
      const int32_t rec = records(a);
      dma_block(vp, p.svn, rec, v_lds[P], voff, voff, vrow, a);
      dma_block(vp, p.svn, rec, v_lds[P] + 2048, voff, voff, vrow, b2 < 0 ? a : b2);
    };
    V8 ak[4];       // K fragments of one tile
    V8 vfr[2][2];   // V^T fragments of one tile [jj][dt]
    auto load_k = [&](auto par_tag) {
      constexpr int P = decltype(par_tag)::value;
      const char* kb = P ? k_buf[1] : k_buf[0];
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        Frag f;
        f.u = *reinterpret_cast<const uint4*>(kb + (kr_off ^ (ks << 5)));
        ak[ks] = as_v8<E>(f);
      }
    };
    auto load_v = [&](auto par_tag) {
      constexpr int P = decltype(par_tag)::value;
      const char* vb = P ? v_buf[1] : v_buf[0];
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

    // ---- the arithmetic of a unit ----
    f32x16 st[2];     // scores of the two halves (unit (t, 1) and unit (t, 0) or (t + 1, 0))
    V8 pf[2][2];      // probabilities [half][jj: block A, B]
    float nega[2], negb[2];  // what is added in the exponent for block A / B: minus the reference, or -inf if not listed
    float negm[2] = {0.f, 0.f};  // minus the reference (0 while there is none)
    bool settled[2];             // (wave-uniform) every query of the half that has a list has its reference
    bool exact = false;      // second walk: running maximum
    const int mine = c >> 4;  // the lane's query block within the half
    // Register r of st[QT]: key row 4hh + 8((r%8)/4) + r%4 of block A (r < 8) or B (r >= 8).
    // Softmax reference.  First walk (exact == false): a query's reference is the maximum over the first tile that
    // holds a block of its list and then stays (softmax is shift invariant), so later tiles need no maximum, no
    // comparison and no pass over the accumulators; probabilities may exceed 1, and a row sum that ends up huge or
    // not finite sends the group through a second walk with the running maximum (exact == true).
    auto pre = [&](auto qt_tag, uint32_t ca, uint32_t cb) {
      constexpr int QT = decltype(qt_tag)::value;
      const uint32_t pa = (ca >> (16 * QT)) & 0xffffu, pb = (cb >> (16 * QT)) & 0xffffu;  // the half's two query blocks
      const int wa = (int)(mine ? pa >> 8 : pa & 0xffu), wb = (int)(mine ? pb >> 8 : pb & 0xffu);
      if (exact || !settled[QT]) {  // (wave-uniform) once every query with a list has its reference, none of this runs
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
          negm[QT] = m_new == -INFINITY ? 0.f : -m_new;
        }
        settled[QT] = (__ballot(m_i[QT] != -INFINITY) & lanes_any[QT]) == lanes_any[QT];
      }
      if (dup) {  // a list that names the block w times attends it w times: w exp2(x) = exp2(x + log2 w), log2 0 = -inf
        nega[QT] = __builtin_amdgcn_logf((float)wa) + negm[QT];
        negb[QT] = __builtin_amdgcn_logf((float)wb) + negm[QT];
      } else {
        nega[QT] = wa ? negm[QT] : -INFINITY;
        negb[QT] = wb ? negm[QT] : -INFINITY;
      }
    };
    // Two of the unit's 16 exponentials per slot (8 slots).  A slot computes its pair and rounds / sums the pair of the
    // slot before, so that no instruction waits on an exponential just issued.  Row sums over the unrounded
    // probabilities (two additions; the dot product of the rounded pair with ones is the slower instruction here).
    float px0 = 0.f, px1 = 0.f;  // the pair in flight
    auto exps_finish = [&](auto qt_tag, auto j_tag) {
      constexpr int QT = decltype(qt_tag)::value;
      constexpr int r = 2 * decltype(j_tag)::value, jj = r >> 3, e8 = r & 7;
      V2 pk;
      pk[0] = (E)px0;
      pk[1] = (E)px1;
      pf[QT][jj][e8] = pk[0];
      pf[QT][jj][e8 + 1] = pk[1];
      l_i[QT] += px0 + px1;
    };
    auto exps = [&](auto qt_tag, auto j_tag) {
      constexpr int QT = decltype(qt_tag)::value;
      constexpr int j = decltype(j_tag)::value, r = 2 * j, jj = r >> 3;
      asm volatile("" : "+v"(st[QT]));
      if constexpr (j > 0) exps_finish(qt_tag, std::integral_constant<int, j - 1>{});
      const float ng = jj ? negb[QT] : nega[QT];
      px0 = __builtin_amdgcn_exp2f(fmaf(st[QT][r], sl2, ng));
      px1 = __builtin_amdgcn_exp2f(fmaf(st[QT][r + 1], sl2, ng));
      V8& pa = pf[QT][0];
      V8& pb = pf[QT][1];
      float& li = l_i[QT];
      asm volatile("" : "+v"(pa), "+v"(pb), "+v"(li), "+v"(px0), "+v"(px1));
    };
    auto exps_tail = [&](auto qt_tag) { exps_finish(qt_tag, std::integral_constant<int, 7>{}); };
    auto mma_s = [&](auto qt_tag, auto ks_tag) {  // scores of a half from the K fragments in registers
      constexpr int QT = decltype(qt_tag)::value, ks = decltype(ks_tag)::value;
      if constexpr (ks == 0) {
        f32x16 z;
#pragma unroll
        for (int r = 0; r < 16; r++) z[r] = 0.f;
        st[QT] = Mma<E>::mma(ak[0], bq[QT][0], z);
      } else {
        st[QT] = Mma<E>::mma(ak[ks], bq[QT][ks], st[QT]);
      }
    };
    auto mma_pv = [&](auto qt_tag, auto i_tag) {  // O^T += V^T P^T of a half, V^T fragments in registers
      constexpr int QT = decltype(qt_tag)::value, i = decltype(i_tag)::value, jj = i >> 1, dt = i & 1;
      ot[dt][QT] = Mma<E>::mma(vfr[jj][dt], pf[QT][jj], ot[dt][QT]);
    };
    // Tile t, parity P.  On entry: st[0] = scores of unit (t, 0); ak = K(t); vfr = V(t-1); pf[1] = probabilities of
    // unit (t-1, 1); in flight or landed: K(t+1), V(t) (older group), K(t+2), V(t+1) (newer group).
    // ca, cb: the counts of the tile's blocks; (av, bv): tile t+2, whose V rows are requested here; nx: the pending
    // read of tile t+3's entries, taken here into (a3, ca3, b3, cb3), whose K rows are requested here.
    auto tile = [&](auto par_tag, uint32_t ca, uint32_t cb, int32_t av, int32_t bv, const int4& nx,
                    int32_t& a3, uint32_t& ca3, int32_t& b3, uint32_t& cb3) {
      constexpr int P = decltype(par_tag)::value;
      typedef std::integral_constant<int, P ^ 1> Q;
      pre(H0{}, ca, cb);
      static_for<8>([&](auto j_tag) {  // exponentials of (t, 0); scores of (t, 1); PV of (t-1, 1)
        constexpr int j = decltype(j_tag)::value;
        if constexpr (j == 4) {
          __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): the older group has landed
          load_k(Q{});                                   // K(t+1)
        }
        if constexpr (j < 4) mma_s(H1{}, j_tag);
        else mma_pv(H1{}, std::integral_constant<int, j - 4>{});
        exps(H0{}, j_tag);
        __builtin_amdgcn_sched_barrier(0);
      });
      exps_tail(H0{});
      load_v(par_tag);  // V(t)
      pre(H1{}, ca, cb);
      static_for<8>([&](auto j_tag) {  // exponentials of (t, 1); scores of (t+1, 0); PV of (t, 0)
        constexpr int j = decltype(j_tag)::value;
        if constexpr (j == 2) {
          __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the fragments of K(t+1) and V(t) are in registers
          lookup_take(nx, a3, ca3, b3, cb3);
          dma_k(Q{}, a3, b3);        // K(t+3) over K(t+1)
          dma_v(par_tag, av, bv);    // V(t+2) over V(t)
        }
        if constexpr (j < 4) mma_s(H0{}, j_tag);
        else mma_pv(H0{}, std::integral_constant<int, j - 4>{});
        exps(H1{}, j_tag);
        __builtin_amdgcn_sched_barrier(0);
      });
      exps_tail(H1{});
    };

    const int ntiles = (n_union + 1) >> 1;
    for (int pass = 0; pass < 2; pass++) {
      exact = pass == 1;
      settled[0] = lanes_any[0] == 0;
      settled[1] = lanes_any[1] == 0;
      if (ntiles > 0) {
        int32_t a0, b0, a1, b1, a2, b2, a3, b3;  // blocks and counts of tiles t .. t+3
        uint32_t ca0, cb0, ca1, cb1, ca2, cb2, ca3, cb3;
        lookup_take(lookup_issue(0), a0, ca0, b0, cb0);
        lookup_take(lookup_issue(1), a1, ca1, b1, cb1);
        lookup_take(lookup_issue(2), a2, ca2, b2, cb2);
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): (second walk) the first walk's last reads are done
        dma_k(H0{}, a0, b0);
        dma_k(H1{}, a1, b1);
        dma_v(H0{}, a0, b0);
        __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): K(0) has landed
        load_k(H0{});
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
        dma_k(H0{}, a2, b2);
        dma_v(H1{}, a1, b1);
        static_for<4>([&](auto ks_tag) { mma_s(H0{}, ks_tag); });
#pragma unroll
        for (int jj = 0; jj < 2; jj++) {  // nothing before unit (0, 0): its PV slot adds zero
#pragma unroll
          for (int e = 0; e < 8; e++) pf[1][jj][e] = (E)0.f;
#pragma unroll
          for (int dt = 0; dt < 2; dt++)
#pragma unroll
            for (int e = 0; e < 8; e++) vfr[jj][dt][e] = (E)0.f;
        }
        int t = 0;
        for (; t + 1 < ntiles; t += 2) {
          int4 nx = lookup_issue(t + 3);
          tile(H0{}, ca0, cb0, a2, b2, nx, a3, ca3, b3, cb3);
          ca0 = ca1; cb0 = cb1;
          ca1 = ca2; cb1 = cb2;
          a2 = a3; b2 = b3; ca2 = ca3; cb2 = cb3;
          nx = lookup_issue(t + 4);
          tile(H1{}, ca0, cb0, a2, b2, nx, a3, ca3, b3, cb3);
          ca0 = ca1; cb0 = cb1;
          ca1 = ca2; cb1 = cb2;
          a2 = a3; b2 = b3; ca2 = ca3; cb2 = cb3;
        }
        if (t < ntiles) {  // an odd number of tiles: the last one (nothing left to request)
          const int4 none = make_int4(-1, 0, -1, 0);
          tile(H0{}, ca0, cb0, -1, -1, none, a3, ca3, b3, cb3);
        }
        static_for<4>([&](auto i_tag) { mma_pv(H1{}, i_tag); });  // PV of the last unit
      }
      if (ragged_cnts != 0) {  // the block that ends the sequence early: one unpipelined step with the running maximum
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): earlier reads of the buffers are done
        dma_ragged(kp, p.skn, k_lds[0], koff, koff8, krow);
        dma_ragged(kp, p.skn, k_lds[0] + 2048, koff, koff8, krow);  // the tile's second block: the same rows again (finite values)
        dma_ragged(vp, p.svn, v_lds[0], voff, voff, vrow);
        dma_ragged(vp, p.svn, v_lds[0] + 2048, voff, voff, vrow);
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        load_k(H0{});
        load_v(H0{});
        const bool was_exact = exact;
        exact = true;
        static_for<2>([&](auto qt_tag) {
          constexpr int QT = decltype(qt_tag)::value;
          static_for<4>([&](auto ks_tag) { mma_s(qt_tag, ks_tag); });
#pragma unroll
          for (int j = 0; j < 8; j++)
            if (4 * hh + 8 * (j >> 2) + (j & 3) > ragged_last) st[QT][j] = -INFINITY;
          pre(qt_tag, ragged_cnts, 0u);
          static_for<8>([&](auto j_tag) { exps(qt_tag, j_tag); });
          exps_tail(qt_tag);
          static_for<4>([&](auto i_tag) { mma_pv(qt_tag, i_tag); });
        });
        exact = was_exact;
      }
      // the sums add the unrounded fp32 probabilities (all >= 0): a sum below the bound proves that every probability
      // was below it when it was rounded; fp16 ends at 65504, bf16 has fp32's range (2^100 leaves room for the products)
      const float big = std::is_same<E, f16_t>::value ? 65504.f : 1.2676506e30f;
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
      negm[0] = negm[1] = 0.f;
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
  static const bool pairs_env = [] {
    const char* e = getenv("S3R_B16_KERNEL");
    return e != nullptr && strcmp(e, "pairs") == 0;
  }();
  // 32-bit byte offsets inside a transfer instruction span 16 rows of a block
  if (16 * p.skn * 2 + 128 > 0xffffffffLL || 16 * p.svn * 2 + 128 > 0xffffffffLL)
    return fail(S3R_ERR_UNSUPPORTED, "s3r_select_attn, 16-token blocks: row stride too large");
  const bool pairs = pairs_env;
  const int64_t es = 2;
  const int wide = (p.Lq - 1) * p.skn * es + 128 > 0xffffffffLL || (p.Lq - 1) * p.svn * es + 128 > 0xffffffffLL;
#define S3R_B16(E, U, W) hipLaunchKernelGGL((b16::select_b16_kernel<E, U, W>), grid, blk, 0, st, p, (int)nqb, (int)ngrp, (int)nwg, (int)total)
  if (dtype == S3R_BF16) {
    if (pairs) S3R_B16(bf16_t, false, false); else if (wide) S3R_B16(bf16_t, true, true); else S3R_B16(bf16_t, true, false);
  } else {
    if (pairs) S3R_B16(f16_t, false, false); else if (wide) S3R_B16(f16_t, true, true); else S3R_B16(f16_t, true, false);
  }
#undef S3R_B16
  return check_launch("select_b16_kernel");
}

}  // namespace s3r
