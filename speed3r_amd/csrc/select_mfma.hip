// Selection-branch attention on the gfx950 matrix cores (bf16 / fp16 I/O, block 64, head_dim 64),
// two-waves-per-SIMD variant without software pipelining inside the wave (the default; the
// one-wave-per-SIMD pipelined variant lives in select_pipe.hip).
//
// One wavefront owns one 64-row query block of one head and walks that block's selected key
// blocks; the four waves of a workgroup take four consecutive query blocks and never
// synchronise with each other (each has a private LDS region).
//
// Data flow per selected key block (64 keys x 64 head_dim):
//   * the K tile goes global -> registers directly in the MFMA A-operand layout
//     (lane = key row, 8 consecutive head_dim values = one 16-byte load); the loads of the
//     next tile are issued as soon as the S^T MFMAs of the current one have consumed the
//     registers, so they fly during the softmax and PV phases;
//   * S^T = K Q^T with v_mfma_f32_32x32x16: the accumulator layout then puts one QUERY per
//     lane (column = lane & 31) and 16 keys per 32x32 tile in its registers, so row max / row
//     sum are in-lane loops plus one exchange with lane ^ 32;
//   * P is rounded to the I/O dtype in registers; the accumulator layout of S^T is already the
//     B-operand layout of O^T = V^T P^T (contraction index = key), with a fixed permutation of
//     keys inside each group of 16 that the V operand simply follows;
//   * the V tile goes global -> LDS without passing through registers (global_load_lds, 16
//     bytes per lane, into the wave's other LDS buffer, issued together with the next K tile)
//     and comes back through ds_read_b64_tr_b16, which hands each lane 4 consecutive KEYS of
//     one head_dim column: the A operand V^T without any explicit transpose.  Rows are 128
//     bytes; the 16-byte chunks of rows 2,3 (mod 4) are stored with their halves swapped so
//     that the four rows one transposed read touches fall into four disjoint bank groups.
// The softmax runs in base 2 on logits pre-multiplied by scale*log2(e); statistics are fp32.
// Softmax is shift invariant: the loop uses ONE reference value per query row, the row
// maximum of the first tile, and never rescales the accumulators; if a row sum ends above
// 2^100 or is not finite the query block is recomputed with a true online softmax, which also
// handles every occurrence of the ragged last key block.  Row sums are taken over the
// probabilities after their rounding to the I/O dtype (v_dot2c with a vector of ones).
//
// Workgroup -> work mapping is XCD-aware: hardware deals workgroups round-robin over the 8
// XCDs, so workgroup w is given work item (w % 8) * per_xcd + w / 8: each XCD then walks a
// contiguous range of query blocks of one head at a time and its L2 sees one head's K/V.
#include "select_common.h"
#include "attn_params.h"

namespace s3r {
namespace basic {
using namespace sel;

constexpr int kTile = 64 * 64;  // elements per LDS tile buffer (one K and one V buffer per wave)

template <typename E>
__global__ __launch_bounds__(256, 2) void select_mfma_kernel(AttnParams p, int nqb, int nqg, int total_wg) {
  typedef typename Mma<E>::V8 V8;
  typedef typename Mma<E>::V2 V2;
  // two separate arrays: the compiler then tells the K and V transfers apart when it counts outstanding loads
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k[4 * kTile * 2];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v[4 * kTile * 2];

  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int hh = lane >> 5;
  const int c = lane & 31;

  const int w = blockIdx.x;
  const int xcd = w & 7, slot = w >> 3;
  const int per = total_wg >> 3, rem = total_wg & 7;
  const int vid = xcd * per + (xcd < rem ? xcd : rem) + slot;
  const int bh = vid / nqg;
  const int qg = vid - bh * nqg;
  const int b = bh / p.H;
  const int h = bh - b * p.H;
  const int qb = qg * 4 + wave;
  if (qb >= nqb) return;

  const int64_t N = p.Lq;
  const int64_t q0 = (int64_t)qb * 64;
  const E* qp = (const E*)p.q + (int64_t)b * p.sqb + (int64_t)h * p.sqh;
  const E* kp = (const E*)p.k + (int64_t)b * p.skb + (int64_t)h * p.skh;
  const E* vp = (const E*)p.v + (int64_t)b * p.svb + (int64_t)h * p.svh;
  E* op = (E*)p.o + (int64_t)b * p.sob + (int64_t)h * p.soh;
  const int32_t* idx_row = p.idx + (int64_t)b * p.sib + (int64_t)h * p.sih + (int64_t)qb * p.sim;
  E* kl = reinterpret_cast<E*>(lds_k) + wave * kTile;
  E* vl = reinterpret_cast<E*>(lds_v) + wave * kTile;

  // index list: full tiles go through the pipeline, occurrences of the ragged last block come after it
  const int32_t my_idx = lane < p.K ? idx_row[lane] : -1;
  const int32_t ragged_blk = (N & 63) ? (int32_t)(N >> 6) : -1;
  const bool my_valid = my_idx >= 0 && (int64_t)my_idx * 64 < N;
  uint64_t todo = __ballot(my_valid && my_idx != ragged_blk);
  int n_ragged = __popcll(__ballot(my_valid && my_idx == ragged_blk));
  const int n_full = __popcll(todo);
  if (n_full + n_ragged == 0) {
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
      const int64_t row = q0 + qt * 32 + c;
      if (row < N) {
#pragma unroll
        for (int i = 0; i < 4; i++) *reinterpret_cast<uint4*>(op + row * p.som + hh * 32 + i * 8) = make_uint4(0, 0, 0, 0);
        if (p.lse != nullptr && hh == 0) p.lse[((int64_t)b * p.H + h) * N + row] = -INFINITY;
      }
    }
    return;
  }
  auto pop_start = [&]() -> int64_t {  // next full tile's first key row, or -1
    if (todo == 0) return -1;
    const int t = __ffsll((unsigned long long)todo) - 1;
    todo &= todo - 1;
    return (int64_t)__builtin_amdgcn_readlane(my_idx, t) * 64;
  };

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

  f32x16 ot[2][2];  // [dt][qt]
#pragma unroll
  for (int dt = 0; dt < 2; dt++)
#pragma unroll
    for (int qt = 0; qt < 2; qt++)
#pragma unroll
      for (int r = 0; r < 16; r++) ot[dt][qt][r] = 0.f;
  float m_i[2] = {-INFINITY, -INFINITY};
  float l_i[2] = {0.f, 0.f};
  const float sl2 = p.scale * 1.4426950408889634f;

  f32x16 st[1][2][2];  // score tile [.][qt][kt]
  V8 pf[1][2][2][2];   // probability tile [.][qt][kt][jj]
  V8 ak[1][2][4];      // K tile [.][kt][ks]

  const uint32_t koff0 = (uint32_t)c * (uint32_t)p.skn + hh * 8;
  const uint32_t koff1 = (uint32_t)(32 + c) * (uint32_t)p.skn + hh * 8;
  auto load_k = [&](V8 (&dst)[2][4], int64_t start) {
    const E* kb = kp + start * p.skn;
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        Frag f;
        f.u = *reinterpret_cast<const uint4*>(kb + (kt ? koff1 : koff0) + ks * 16);
        dst[kt][ks] = as_v8<E>(f);
      }
  };
  // K tile global -> LDS: LDS chunk (row, c') holds head_dim chunk c' ^ (row & 7); a lane quad stays inside one 64-byte
  // half row on the global side, and the A-operand reads below (32 rows x one chunk) spread over all banks
  const int ldv_row = lane >> 3;
  // (buffer loads rather than global loads: the compiler then counts the outstanding transfers per LDS array)
  const uint32_t klds_off = ((uint32_t)ldv_row * (uint32_t)p.skn + (((lane & 7) ^ (ldv_row & 7)) * 8)) * (uint32_t)sizeof(E);
  const uint32_t k_step = 8u * (uint32_t)p.skn * (uint32_t)sizeof(E);  // 8 rows per transfer instruction
  auto load_k_lds = [&](int64_t start) {
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(kp + start * p.skn), 0, 0x7fffffff, 0x00020000);
#pragma unroll
    for (int i = 0; i < 8; i++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)(kl + i * 512), 16, klds_off, i * k_step, 0, 0);
  };
  // Every read of a tile buffer is preceded by an explicit wait for its transfer (the compiler's own bookkeeping of
  // transfers into LDS is not relied on): vmcnt counts in issue order and K and V transfers alternate, 8 instructions each.
  auto wait_transfer = [&]() { __builtin_amdgcn_s_waitcnt(0x0F78); };  // vmcnt(8)
  const int kr_off = c * 128 + ((hh ^ (c & 7)) << 4);
  auto read_k = [&](V8 (&dst)[2][4]) {
    const char* kbase = reinterpret_cast<const char*>(kl);
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        Frag f;
        f.u = *reinterpret_cast<const uint4*>(kbase + kt * 4096 + (kr_off ^ (ks << 5)));
        dst[kt][ks] = as_v8<E>(f);
      }
  };
  const int ldv_chunk = (lane & 7) ^ (((ldv_row >> 1) & 1) << 2);
  const uint32_t voff = ((uint32_t)ldv_row * (uint32_t)p.svn + ldv_chunk * 8) * (uint32_t)sizeof(E);
  const uint32_t v_step = 8u * (uint32_t)p.svn * (uint32_t)sizeof(E);
  auto load_v = [&](int64_t start) {
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(vp + start * p.svn), 0, 0x7fffffff, 0x00020000);
#pragma unroll
    for (int i = 0; i < 8; i++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)(vl + i * 512), 16, voff, i * v_step, 0, 0);
  };
  const int i16 = lane & 15;
  const int tr_row = 4 * hh + (i16 >> 2);
  const int tr_chunk = (((lane >> 4) & 1) * 2 + ((i16 & 3) >> 1)) ^ (((tr_row >> 1) & 1) << 2);
  const int tr_off = tr_row * 128 + tr_chunk * 16 + (i16 & 1) * 8;
  // all V^T fragments of one tile: [kt][jj][dt], k-step (kt,jj) = keys kt*32 + 16jj + {4hh.., 8+4hh..}
  auto read_v = [&](V8 (&vfr)[2][2][2]) {
    const char* vbase = reinterpret_cast<const char*>(vl);
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
          vfr[kt][jj][dt] = as_v8<E>(f);
        }
  };
  auto row_max = [&](const f32x16 (&s)[2]) -> float {  // over this lane's 32 keys and its partner's
    float mx = s[0][0];
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[kt][r]);
    return xh_max(mx) * sl2;
  };

  // PV of a finished probability tile without anything to overlap it with
  auto pv_only = [&](const V8 (&pp)[2][2][2]) {
    V8 vfr[2][2][2];
    read_v(vfr);
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int jj = 0; jj < 2; jj++)
#pragma unroll
        for (int dt = 0; dt < 2; dt++)
#pragma unroll
          for (int qt = 0; qt < 2; qt++) ot[dt][qt] = Mma<E>::mma(vfr[kt][jj][dt], pp[qt][kt][jj], ot[dt][qt]);
  };
  auto scores_only = [&](f32x16 (&s)[2][2], const V8 (&kk)[2][4]) {
#pragma unroll
    for (int qt = 0; qt < 2; qt++)
#pragma unroll
      for (int kt = 0; kt < 2; kt++) {
#pragma unroll
        for (int r = 0; r < 16; r++) s[qt][kt][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) s[qt][kt] = Mma<E>::mma(kk[kt][ks], bq[qt][ks], s[qt][kt]);
      }
  };
  // One tile of the fast loop: K from LDS into registers, S^T and exponentials per query half, PV from the V buffer.
  // The transfer of the next K tile starts once the first S^T MFMAs have consumed this tile's K registers (the K
  // buffer is free from then on) and that of the next V tile after the PV reads: each has about one tile of time.
  auto fast_tile = [&](int64_t next) {
    const float mneg[2] = {-m_i[0], -m_i[1]};
    wait_transfer();
    read_k(ak[0]);
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
#pragma unroll
      for (int kt = 0; kt < 2; kt++) {
#pragma unroll
        for (int r = 0; r < 16; r++) st[0][qt][kt][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) st[0][qt][kt] = Mma<E>::mma(ak[0][kt][ks], bq[qt][ks], st[0][qt][kt]);
      }
      if (qt == 0) {
        __builtin_amdgcn_sched_barrier(0);
        load_k_lds(next);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int jj = 0; jj < 2; jj++)
#pragma unroll
          for (int e = 0; e < 8; e += 2) {
            V2 pk;
            pk[0] = (E)__builtin_amdgcn_exp2f(fmaf(st[0][qt][kt][8 * jj + e], sl2, mneg[qt]));
            pk[1] = (E)__builtin_amdgcn_exp2f(fmaf(st[0][qt][kt][8 * jj + e + 1], sl2, mneg[qt]));
            pf[0][qt][kt][jj][e] = pk[0];
            pf[0][qt][kt][jj][e + 1] = pk[1];
            l_i[qt] = Mma<E>::dot_ones(pk, l_i[qt]);
          }
    }
    __builtin_amdgcn_sched_barrier(0);
    wait_transfer();
    pv_only(pf[0]);
    __builtin_amdgcn_sched_barrier(0);  // the refill is issued after the MFMAs that consumed the old contents
    load_v(next);
  };
  // Unpipelined stage with a true online softmax: one key tile (possibly ragged) from global memory.
  auto robust_tile = [&](int64_t start) {
    const int nvalid = (int)((N - start < 64) ? (N - start) : 64);
    const E* kb = kp + start * p.skn;
    const uint32_t last = (uint32_t)(nvalid - 1);
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
      const uint32_t r = (uint32_t)(kt * 32 + c);
      const uint32_t off = (r < last ? r : last) * (uint32_t)p.skn + hh * 8;  // rows beyond N: re-read the last row
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        Frag f;
        f.u = *reinterpret_cast<const uint4*>(kb + off + ks * 16);
        ak[0][kt][ks] = as_v8<E>(f);
      }
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): earlier reads of the V buffer are done
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int row = i * 8 + ldv_row;
      uint4 raw = make_uint4(0, 0, 0, 0);  // V rows beyond N are zero
      if (row < nvalid) raw = *reinterpret_cast<const uint4*>(vp + (start + row) * p.svn + ldv_chunk * 8);
      *reinterpret_cast<uint4*>(vl + i * 512 + lane * 8) = raw;
    }
    scores_only(st[0], ak[0]);
    const int lim = nvalid - 4 * hh;
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++)
          if (kt * 32 + 8 * (r >> 2) + (r & 3) >= lim) st[0][qt][kt][r] = -INFINITY;
      const float mx = row_max(st[0][qt]);
      const float m_new = fmaxf(m_i[qt], mx);
      const float alpha = __builtin_amdgcn_exp2f(m_i[qt] - m_new);  // 0 on the first tile (m_i = -inf)
      m_i[qt] = m_new;
      l_i[qt] *= alpha;
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) ot[dt][qt][r] *= alpha;
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int jj = 0; jj < 2; jj++)
#pragma unroll
          for (int e = 0; e < 8; e += 2) {
            V2 pk;
            pk[0] = (E)__builtin_amdgcn_exp2f(fmaf(st[0][qt][kt][8 * jj + e], sl2, -m_new));
            pk[1] = (E)__builtin_amdgcn_exp2f(fmaf(st[0][qt][kt][8 * jj + e + 1], sl2, -m_new));
            pf[0][qt][kt][jj][e] = pk[0];
            pf[0][qt][kt][jj][e + 1] = pk[1];
            l_i[qt] = Mma<E>::dot_ones(pk, l_i[qt]);
          }
    }
    pv_only(pf[0]);
  };
  auto reset_state = [&]() {
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
      for (int qt = 0; qt < 2; qt++)
#pragma unroll
        for (int r = 0; r < 16; r++) ot[dt][qt][r] = 0.f;
    m_i[0] = m_i[1] = -INFINITY;
    l_i[0] = l_i[1] = 0.f;
  };

  bool redo = false;
  if (n_full > 0) {
    // first tile: its row maxima become the softmax reference
    const int64_t s0 = pop_start();
    load_k_lds(s0);
    load_v(s0);
    int64_t last_start = s0;
    auto pop_or_last = [&]() -> int64_t {  // branch-free: next full tile, or the last one again
      const bool any = todo != 0;
      const int t = any ? __ffsll((unsigned long long)todo) - 1 : 0;
      const int64_t s = (int64_t)__builtin_amdgcn_readlane(my_idx, t) * 64;
      todo &= todo - 1;  // stays 0 once empty
      last_start = any ? s : last_start;
      return last_start;
    };
    wait_transfer();
    read_k(ak[0]);
    scores_only(st[0], ak[0]);
    m_i[0] = row_max(st[0][0]);
    m_i[1] = row_max(st[0][1]);
    for (int i = n_full; i > 0; i--)  // past the end of the list the prefetch re-reads the last tile
      fast_tile(pop_or_last());
    // a reference that was too low shows up as a huge or non-finite row sum
    const float big = 1.2676506e30f;  // 2^100
    redo = __any(!(l_i[0] < big) || !(l_i[1] < big));
  }

  if (redo) {  // rare: recompute the query block with the online softmax
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): no prefetch is still writing LDS
    reset_state();
    uint64_t again = __ballot(my_valid && my_idx != ragged_blk);
    while (again) {
      const int t = __ffsll((unsigned long long)again) - 1;
      again &= again - 1;
      robust_tile((int64_t)__builtin_amdgcn_readlane(my_idx, t) * 64);
    }
  }
  if (n_ragged > 0) {
    __builtin_amdgcn_s_waitcnt(0x0F70);
    for (; n_ragged > 0; n_ragged--) robust_tile((int64_t)ragged_blk * 64);
  }

#pragma unroll
  for (int qt = 0; qt < 2; qt++) {
    const float l = xh_sum(l_i[qt]);
    const float inv = l > 0.f ? 1.f / l : 0.f;
    const int64_t row = q0 + qt * 32 + c;
    if (row < N) {
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          union { E e[4]; uint2 u; } pk;
#pragma unroll
          for (int e = 0; e < 4; e++) pk.e[e] = (E)(ot[dt][qt][4 * g4 + e] * inv);
          *reinterpret_cast<uint2*>(op + row * p.som + dt * 32 + 4 * hh + 8 * g4) = pk.u;
        }
      if (p.lse != nullptr && hh == 0)
        p.lse[((int64_t)b * p.H + h) * N + row] = l > 0.f ? (m_i[qt] + __builtin_amdgcn_logf(l)) * 0.6931471805599453f : -INFINITY;
    }
  }
}

}  // namespace basic

int launch_select_mfma(const AttnParams& p, int dtype, void* stream) {
  const int64_t nqb = (p.Lq + 63) / 64;
  const int64_t nqg = (nqb + 3) / 4;
  const int64_t total = nqg * p.B * p.H;
  if (total > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_select_attn: grid too large");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)total), blk(256);
  if (dtype == S3R_BF16)
    hipLaunchKernelGGL(basic::select_mfma_kernel<bf16_t>, grid, blk, 0, st, p, (int)nqb, (int)nqg, (int)total);
  else
    hipLaunchKernelGGL(basic::select_mfma_kernel<f16_t>, grid, blk, 0, st, p, (int)nqb, (int)nqg, (int)total);
  return check_launch("select_mfma_kernel");
}

}  // namespace s3r
