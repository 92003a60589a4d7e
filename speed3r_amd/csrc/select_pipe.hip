// Selection-branch attention on the gfx950 matrix cores (bf16 / fp16 I/O, block 64, head_dim 64), software-pipelined
// inside the wave.
//
// One wavefront owns one 64-row query block of one head and walks that block's selected key blocks; the waves of a
// workgroup take consecutive query blocks and never synchronise with each other (each has a private LDS region); two
// waves per SIMD.
//   * S^T = K Q^T with v_mfma_f32_32x32x16: the accumulator layout puts one QUERY per lane (column = lane & 31) and 16
//     keys per 32x32 tile in its registers, so row maxima and row sums are in-lane loops plus one exchange with
//     lane ^ 32.
//   * P is rounded to the I/O dtype in registers; the accumulator layout of S^T is already the B-operand layout of
//     O^T = V^T P^T (contraction index = key), with a fixed permutation of keys inside each group of 16 that the V
//     operand simply follows.
//   * K and V tiles go global -> LDS without passing through registers (buffer_load ... lds, 16 bytes per lane).  K
//     fragments come back with ds_read_b128 (lane = key row; the 16-byte chunks of a row are stored XOR-swizzled by
//     the row number so that the reads are conflict free), V^T fragments with ds_read_b64_tr_b16, which hands each
//     lane 4 consecutive KEYS of one head_dim column: the A operand V^T without an explicit transpose (rows are 128
//     bytes; the chunks of rows 2,3 (mod 4) are stored with their halves swapped so that the four rows one transposed
//     read touches fall into four disjoint bank groups).
//   * The softmax runs in base 2 on logits pre-multiplied by scale*log2(e); statistics are fp32.  Softmax is shift
//     invariant: the loop uses ONE reference value per query row, the row maximum of the first half tile, and never
//     rescales the accumulators; if a row sum ends above 2^100 or is not finite the query block is recomputed by an
//     unpipelined stage with a true online softmax, which also handles every occurrence of the ragged last key block.
//   * Workgroup -> work mapping is XCD-aware: hardware deals workgroups round-robin over the 8 XCDs, so workgroup w is
//     given work item (w % 8) * per_xcd + w / 8: each XCD then walks a contiguous range of query blocks of one head at
//     a time and its L2 sees one head's K/V.
//
// The unit of the pipeline is HALF a key tile (32 keys x 64 queries): its S^T is 8 MFMAs, its PV is 8
// MFMAs, its softmax is 32 exponentials per lane.  In one phase the wave issues
//
//     PV MFMAs of unit u-1,  S^T MFMAs of unit u+1      16 MFMAs, one per slot
//     the exponentials / rounding / row sums of unit u   VALU work spread over the same 16 slots
//
// so neither MFMA group depends on the VALU work issued around it: the matrix pipe (32 cycles per
// MFMA) and the vector ALU (about as many cycles of exp/convert work per slot) run side by side in
// the same wave instead of relying on the two waves of a SIMD being out of step.  A K half tile and a
// V half tile are each used by exactly one unit, so their fragments are read from LDS just in time
// (16 registers each) and every LDS byte is read once.
//
// LDS per wave: two K half buffers and two V half buffers (4 KB each), in four separate arrays (the
// compiler then knows that a read of one does not depend on a transfer into another).  A half
// buffer is refilled (buffer_load ... lds, 16 bytes per lane) right after its fragments have been read,
// two phases before it is needed again.
#include "select_common.h"
#include "attn_params.h"

namespace s3r {
namespace pipe {
using namespace sel;

constexpr int kHalf = 32 * 64;  // elements per half tile
#ifndef S3R_PIPE_WAVES
#define S3R_PIPE_WAVES 4
#endif
constexpr int kWaves = S3R_PIPE_WAVES;  // wavefronts (= query blocks) per workgroup; the waves do not interact

// DENSE: no index list, every query block attends to all key tiles in order (the compressed branch's attention over
// the pooled tokens runs through this instance).
// SPLIT (with DENSE, for sweeps with too few query blocks to fill the chip): two waves share a query block, each
// sweeps half of the key tiles, and the first one folds the second one's accumulators into its own through LDS.
template <typename E, bool DENSE, bool SPLIT = false>
__global__ __launch_bounds__(64 * kWaves, 2) void select_pipe_kernel(AttnParams p, int nqb, int nqg, int total_wg) {
  static_assert(!SPLIT || DENSE, "the split sweep is a variant of the dense one");
  typedef typename Mma<E>::V8 V8;
  typedef typename Mma<E>::V2 V2;
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[kWaves * kHalf * 2];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[kWaves * kHalf * 2];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[kWaves * kHalf * 2];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v1[kWaves * kHalf * 2];
  __shared__ float lds_ml[SPLIT ? kWaves * 4 * 64 : 1];  // SPLIT: per wave and lane the two references and the two row sums

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: addresses derived from it stay scalar
  const int lane = threadIdx.x & 63;
  const int hh = lane >> 5;
  const int c = lane & 31;

  // everything the index row's address and the Q transfers need, fetched from the argument block in ONE round trip
  // (the compiler would otherwise fetch each argument where it is first used: three dependent trips before the row)
  if constexpr (!DENSE)
    asm volatile("" ::"s"(p.H), "s"(nqg), "s"(nqb), "s"(total_wg), "s"(p.idx), "s"(p.sib), "s"(p.sih), "s"(p.sim), "s"(p.K), "s"(p.q),
                 "s"(p.sqb), "s"(p.sqh), "s"(p.sqm), "s"(p.Lq));
  const int w = blockIdx.x;
  const int xcd = w & 7, slot = w >> 3;
  const int per = total_wg >> 3, rem = total_wg & 7;
  const int vid = xcd * per + (xcd < rem ? xcd : rem) + slot;
  const int bh = vid / nqg;
  const int qg = vid - bh * nqg;
  const int b = bh / p.H;
  const int h = bh - b * p.H;
  const int split = SPLIT ? (wave & 1) : 0;  // which half of the key tiles
  int qb = SPLIT ? qg * (kWaves / 2) + (wave >> 1) : qg * kWaves + wave;
  // SPLIT: every wave of the workgroup has to reach the barrier of the hand-over, so a pair past the last query block
  // repeats the last block's work and stores nothing
  const bool ghost = SPLIT && qb >= nqb;
  if (SPLIT) qb = qb < nqb ? qb : nqb - 1;
  if (qb >= nqb) return;

  const int64_t N = p.Lq;
  const int64_t q0 = (int64_t)qb * 64;
  const E* qp = (const E*)p.q + (int64_t)b * p.sqb + (int64_t)h * p.sqh;
  const E* kp = (const E*)p.k + (int64_t)b * p.skb + (int64_t)h * p.skh;
  const E* vp = (const E*)p.v + (int64_t)b * p.svb + (int64_t)h * p.svh;
  E* op = (E*)p.o + (int64_t)b * p.sob + (int64_t)h * p.soh;
  const int32_t* idx_row = DENSE ? nullptr : p.idx + (int64_t)b * p.sib + (int64_t)h * p.sih + (int64_t)qb * p.sim;
  // The index row is the head of the longest dependency chain of the start-up (row -> first K tile -> first scores):
  // its load is the wave's first memory instruction, ahead of the Q transfers in the vector memory queue, one entry
  // per lane; the scheduling barrier keeps the compiler from sinking it to its first use.
  int32_t my_idx = -1;
  if constexpr (!DENSE) {
    if (lane < p.K) my_idx = __builtin_nontemporal_load(idx_row + lane);
    __builtin_amdgcn_sched_barrier(0);
  }

  auto k_half = [&](auto hf) -> E* {
    if constexpr (decltype(hf)::value == 0) return reinterpret_cast<E*>(lds_k0) + wave * kHalf;
    else return reinterpret_cast<E*>(lds_k1) + wave * kHalf;
  };
  auto v_half = [&](auto hf) -> E* {
    if constexpr (decltype(hf)::value == 0) return reinterpret_cast<E*>(lds_v0) + wave * kHalf;
    else return reinterpret_cast<E*>(lds_v1) + wave * kHalf;
  };
  typedef std::integral_constant<int, 0> H0;
  typedef std::integral_constant<int, 1> H1;

  // Q block -> LDS by direct transfers (the two V half buffers hold it until the first V tile is fetched), in the
  // layout of a K tile, so that the B operands are read like K fragments.  Lane-linear transfers cost the texture
  // path a quarter of what operand-pattern global loads cost.  Rows beyond N re-read the last row (never stored).
  {
    const int qr = lane >> 3;
    const uint32_t q_rowbytes = (uint32_t)p.sqm * (uint32_t)sizeof(E);
    const int q_last = (int)((N - q0 < 64 ? N - q0 : 64) - 1);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(qp + q0 * p.sqm), 0, 0x7fffffff, 0x00020000);
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
      char* dst = reinterpret_cast<char*>(qt == 0 ? v_half(H0{}) : v_half(H1{}));
#pragma unroll
      for (int i = 0; i < 4; i++) {
        int row = 32 * qt + 8 * i + qr;
        row = row < q_last ? row : q_last;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)(dst + i * 1024), 16,
                                                 (uint32_t)row * q_rowbytes + (uint32_t)(((lane & 7) ^ k_swizzle(8 * i + qr)) * 16), 0, 0,
                                                 2 /* nt: the Q block is read once */);
      }
    }
  }

  // index list: full tiles go through the pipeline, occurrences of the ragged last block come after it
  const int32_t ragged_blk = (N & 63) ? (int32_t)(N >> 6) : -1;
  bool my_valid = false;
  uint64_t todo = 0;
  int n_ragged, n_full;
  int dense_next = 0;  // DENSE: the next tile of the sweep and the end of this wave's range
  int dense_begin = 0, dense_end = 0;
  if constexpr (DENSE) {
    n_full = (int)(N >> 6);
    n_ragged = (N & 63) ? 1 : 0;
    if constexpr (SPLIT) {  // first wave: tiles [0, h0); second wave: [h0, n_full) and the ragged tile
      const int h0 = (n_full + 1) >> 1;
      dense_begin = split ? h0 : 0;
      n_full = split ? n_full - h0 : h0;
      n_ragged = split ? n_ragged : 0;
    }
    dense_next = dense_begin;
    dense_end = dense_begin + n_full;
  } else {
    my_valid = my_idx >= 0 && (int64_t)my_idx * 64 < N;
    todo = __ballot(my_valid && my_idx != ragged_blk);
    n_ragged = __popcll(__ballot(my_valid && my_idx == ragged_blk));
    n_full = __popcll(todo);
  }
  if (!SPLIT && n_full + n_ragged == 0 && p.merge_out == nullptr) {  // nothing to attend to: zeros (the merge path goes on and merges zeros)
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): no transfer may still write LDS when the wave ends
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

  V8 bq[2][4];

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

  f32x16 st[2][2];  // scores [qt][kt]
  V8 pf[2][2][2];   // probabilities [qt][kt][jj]
  V8 ak[4];         // K fragments of one half tile [ks]
  V8 vfr[2][2];     // V^T fragments of one half tile [jj][dt]

  // ---- transfers global -> LDS (8 rows of 128 bytes per instruction, 16 bytes per lane) ----
  // K: LDS chunk (row, c') holds head_dim chunk c' ^ k_swizzle(row), which differs between the rows of an even and of an
  // odd instruction of a tile; V: chunks of rows 2,3 (mod 4) have their halves swapped
  const int ld_row = lane >> 3;
  const uint32_t k_voff[2] = {((uint32_t)ld_row * (uint32_t)p.skn + (((lane & 7) ^ k_swizzle(ld_row)) * 8)) * (uint32_t)sizeof(E),
                              ((uint32_t)ld_row * (uint32_t)p.skn + (((lane & 7) ^ k_swizzle(ld_row + 8)) * 8)) * (uint32_t)sizeof(E)};
  const uint32_t v_voff = ((uint32_t)ld_row * (uint32_t)p.svn + (((lane & 7) ^ (((ld_row >> 1) & 1) << 2)) * 8)) * (uint32_t)sizeof(E);
  // the instruction's immediate offset moves the LDS side AND the global side by i KB: the scalar offset makes up the rest
  const uint32_t k_step = 8u * (uint32_t)p.skn * (uint32_t)sizeof(E) - 1024u;
  const uint32_t v_step = 8u * (uint32_t)p.svn * (uint32_t)sizeof(E) - 1024u;
  auto dma_k = [&](auto hf, int64_t start) {  // keys start + 32*hf .. +31
    constexpr int HF = decltype(hf)::value;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(kp + (start + 32 * HF) * p.skn), 0, 0x7fffffff, 0x00020000);
    __attribute__((address_space(3))) void* dst = (__attribute__((address_space(3))) void*)k_half(hf);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, k_voff[0], 0, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, k_voff[1], k_step, 1024, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, k_voff[0], 2 * k_step, 2048, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, k_voff[1], 3 * k_step, 3072, 0);
  };
  auto dma_v = [&](auto hf, int64_t start) {
    constexpr int HF = decltype(hf)::value;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(vp + (start + 32 * HF) * p.svn), 0, 0x7fffffff, 0x00020000);
    __attribute__((address_space(3))) void* dst = (__attribute__((address_space(3))) void*)v_half(hf);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, v_voff, 0, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, v_voff, v_step, 1024, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, v_voff, 2 * v_step, 2048, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, v_voff, 3 * v_step, 3072, 0);
  };
  // Every read of a half buffer is preceded by an explicit wait for its transfer (the compiler's own bookkeeping of
  // transfers into LDS is not relied on).  vmcnt counts in issue order; in the loop, and in the start-up sequence,
  // which issues in the same rotation K1, V0, K0, V1, exactly 12 transfer instructions are issued between a half
  // buffer's refill and its next read.
  auto wait_transfer = [&]() { __builtin_amdgcn_s_waitcnt(0x0F7C); };  // vmcnt(12)
  // ... and every refill by a wait for the LDS reads of the old contents (a transfer that hits in the vector cache
  // can otherwise overtake a read still queued in the LDS pipeline)
  auto reads_done = [&]() { __builtin_amdgcn_s_waitcnt(0xC07F); };  // lgkmcnt(0)
  // ---- LDS -> registers ----
  const int kr_off = c * 128 + ((hh ^ k_swizzle(c)) << 4);
  auto read_k = [&](auto hf, V8 (&dst)[4]) {  // A operand: lane = key row, head_dim chunk hh + 2*ks
    const char* kbase = reinterpret_cast<const char*>(k_half(hf));
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      Frag f;
      f.u = *reinterpret_cast<const uint4*>(kbase + (kr_off ^ (ks << 5)));
      dst[ks] = as_v8<E>(f);
    }
  };
  const int i16 = lane & 15;
  const int tr_row = 4 * hh + (i16 >> 2);
  const int tr_chunk = (((lane >> 4) & 1) * 2 + ((i16 & 3) >> 1)) ^ (((tr_row >> 1) & 1) << 2);
  const int tr_off = tr_row * 128 + tr_chunk * 16 + (i16 & 1) * 8;
  auto read_v = [&](auto hf, V8 (&dst)[2][2]) {  // V^T fragments [jj][dt]: keys 16jj + {4hh.., 8+4hh..} of the half
    const char* vbase = reinterpret_cast<const char*>(v_half(hf));
#pragma unroll
    for (int jj = 0; jj < 2; jj++)
#pragma unroll
      for (int dt = 0; dt < 2; dt++) {
        const char* a0 = vbase + (tr_off ^ (dt * 64)) + (jj * 16) * 128;
        Frag f;
        f.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
        f.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0 + 8 * 128));
        dst[jj][dt] = as_v8<E>(f);
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
  auto half_max = [&](const f32x16& sc) -> float {  // over this lane's 16 keys of a half tile and its partner's
    float mx = sc[0];
#pragma unroll
    for (int r = 1; r < 16; r++) mx = fmaxf(mx, sc[r]);
    return xh_max(mx) * sl2;
  };
  auto scores_half = [&](auto hf) {  // st[.][hf] from the K half in LDS
    constexpr int HF = decltype(hf)::value;
    read_k(hf, ak);
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
#pragma unroll
      for (int r = 0; r < 16; r++) st[qt][HF][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 4; ks++) st[qt][HF] = Mma<E>::mma(ak[ks], bq[qt][ks], st[qt][HF]);
    }
  };
  auto pv_half = [&](auto hf) {  // ot += V^T P^T for the half whose fragments are in vfr
    constexpr int HF = decltype(hf)::value;
#pragma unroll
    for (int jj = 0; jj < 2; jj++)
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int qt = 0; qt < 2; qt++) ot[dt][qt] = Mma<E>::mma(vfr[jj][dt], pf[qt][HF][jj], ot[dt][qt]);
  };

  // ---- one phase of the pipeline, unit u = (tile, KT) ----
  //   MFMA slots 0..7 : PV of unit u-1 (probabilities pf[.][KT^1], fragments already in vfr)
  //   MFMA slots 8..15: S^T of unit u+1 into st[.][KT^1] (K half KT^1 read at slot 0)
  //   VALU, all slots : exponentials of unit u, st[.][KT] -> pf[.][KT], two elements per slot
  // After its fragments are read, K half KT^1 is refilled from tile k_next and V half KT from tile v_next.
  // Empty volatile asm statements on the score tuple before and on the probability tuple after pin the VALU
  // instructions of a slot; the scheduling barrier after every slot keeps the MFMAs where they are written.
  float mneg[2];
  auto phase = [&](auto kt_tag, int64_t k_next, int64_t v_next) {
    constexpr int KT = decltype(kt_tag)::value;
    constexpr int OT = KT ^ 1;
    typedef std::integral_constant<int, OT> HO;
    static_for<16>([&](auto j_tag) {
      constexpr int j = decltype(j_tag)::value;
      // a half buffer is refilled two slots after its fragments were requested, once they have arrived
      if constexpr (j == 0) {
        wait_transfer();
        read_k(HO{}, ak);
      }
      if constexpr (j == 2) {
        reads_done();
        dma_k(HO{}, k_next);
      }
      if constexpr (j == 8) {
        wait_transfer();
        read_v(kt_tag, vfr);
      }
      if constexpr (j == 10) {
        reads_done();
        dma_v(kt_tag, v_next);
      }
      if constexpr (j < 8) {
        constexpr int jj = j >> 2, dt = (j >> 1) & 1, qt = j & 1;
        ot[dt][qt] = Mma<E>::mma(vfr[jj][dt], pf[qt][OT][jj], ot[dt][qt]);
      } else {
        constexpr int i = j - 8, qt = i >> 2, ks = i & 3;
        if constexpr (ks == 0) {
          f32x16 z;
#pragma unroll
          for (int r = 0; r < 16; r++) z[r] = 0.f;
          st[qt][OT] = Mma<E>::mma(ak[ks], bq[qt][ks], z);
        } else {
          st[qt][OT] = Mma<E>::mma(ak[ks], bq[qt][ks], st[qt][OT]);
        }
      }
      {
        constexpr int e = 2 * j;
        constexpr int qt = e >> 4, r = e & 15, jj = r >> 3, e8 = r & 7;
        asm volatile("" : "+v"(st[qt][KT]));
        const float x0 = __builtin_amdgcn_exp2f(fmaf(st[qt][KT][r], sl2, mneg[qt]));
        const float x1 = __builtin_amdgcn_exp2f(fmaf(st[qt][KT][r + 1], sl2, mneg[qt]));
        V2 pk;
        pk[0] = (E)x0;
        pk[1] = (E)x1;
        pf[qt][KT][jj][e8] = pk[0];
        pf[qt][KT][jj][e8 + 1] = pk[1];
        // row sums over the unrounded probabilities, as the reference's tl.sum(p) before p.to(v.dtype); the pair is
        // added first: two additions chained on the sum stall the second one behind the exponential's result
        l_i[qt] += x0 + x1;
        asm volatile("" : "+v"(pf[qt][KT][jj]), "+v"(l_i[qt]));
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // Unpipelined stage with a true online softmax: one key tile (possibly ragged) from global memory.
  auto robust_tile = [&](int64_t start) {
    const int nvalid = (int)((N - start < 64) ? (N - start) : 64);
    const E* kb = kp + start * p.skn;
    const uint32_t last = (uint32_t)(nvalid - 1);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): earlier reads of the V buffers are done
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int row = i * 8 + ld_row;
      uint4 raw = make_uint4(0, 0, 0, 0);  // V rows beyond N are zero
      if (row < nvalid) raw = *reinterpret_cast<const uint4*>(vp + (start + row) * p.svn + ((lane & 7) ^ (((ld_row >> 1) & 1) << 2)) * 8);
      E* dst = i < 4 ? v_half(H0{}) + i * 512 : v_half(H1{}) + (i - 4) * 512;
      *reinterpret_cast<uint4*>(dst + lane * 8) = raw;
    }
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
      const uint32_t r = (uint32_t)(kt * 32 + c);
      const uint32_t off = (r < last ? r : last) * (uint32_t)p.skn + hh * 8;  // rows beyond N: re-read the last row
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        Frag f;
        f.u = *reinterpret_cast<const uint4*>(kb + off + ks * 16);
        ak[ks] = as_v8<E>(f);
      }
#pragma unroll
      for (int qt = 0; qt < 2; qt++) {
#pragma unroll
        for (int r2 = 0; r2 < 16; r2++) st[qt][kt][r2] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) st[qt][kt] = Mma<E>::mma(ak[ks], bq[qt][ks], st[qt][kt]);
      }
    }
    const int lim = nvalid - 4 * hh;
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++)
          if (kt * 32 + 8 * (r >> 2) + (r & 3) >= lim) st[qt][kt][r] = -INFINITY;
      const float mx = row_max(st[qt]);
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
            const float x0 = __builtin_amdgcn_exp2f(fmaf(st[qt][kt][8 * jj + e], sl2, -m_new));
            const float x1 = __builtin_amdgcn_exp2f(fmaf(st[qt][kt][8 * jj + e + 1], sl2, -m_new));
            pf[qt][kt][jj][e] = (E)x0;
            pf[qt][kt][jj][e + 1] = (E)x1;
            l_i[qt] += x0 + x1;
          }
    }
    read_v(H0{}, vfr);
    pv_half(H0{});
    read_v(H1{}, vfr);
    pv_half(H1{});
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
  // Operands of the gated merge (epilogue): gate pair per query row, the query block's row of the compressed output
  // in this lane's store layout.  Issued right after the main loop, so that their latency passes behind the last PV
  // stage instead of in front of the stores.
  const bool merge = p.merge_out != nullptr;
  uint32_t g_raw[2] = {0, 0};  // gate pair per query row, bits of the I/O type
  uint4 oc_raw[2][2];  // [dt][gp]
  bool merge_loaded = false;
  auto load_merge_operands = [&]() {
    if (merge) {
#pragma unroll
      for (int qt = 0; qt < 2; qt++) {
        const int64_t row = q0 + qt * 32 + c;
        if (row < N) {  // the pair as raw bits: converting it here would wait for the load, and for every transfer before it
          const E* gp = (const E*)p.merge_gate + (int64_t)b * p.sgb + (int64_t)h * p.sgh + row * p.sgn;
          __builtin_memcpy(&g_raw[qt], gp, 4);
        }
      }
      const E* ocp = (const E*)p.merge_oc + (int64_t)b * p.scb + (int64_t)h * p.sch + (int64_t)qb * p.scm;
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int gp = 0; gp < 2; gp++) oc_raw[dt][gp] = *reinterpret_cast<const uint4*>(ocp + dt * 32 + 8 * (2 * gp + hh));
    }
    merge_loaded = true;
  };

  auto read_q = [&]() {  // B operands from the staged Q block: lane = query row, head_dim chunk hh + 2*ks
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
      const char* qbase = reinterpret_cast<const char*>(qt == 0 ? v_half(H0{}) : v_half(H1{}));
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        Frag f;
        f.u = *reinterpret_cast<const uint4*>(qbase + (kr_off ^ (ks << 5)));
        bq[qt][ks] = as_v8<E>(f);
      }
    }
    reads_done();  // before the V buffers are refilled
  };
  if (n_full == 0) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the Q transfers have landed
    read_q();
  }
  if (n_full > 0) {
    int64_t last_start = 0;
    auto pop_or_last = [&]() -> int64_t {  // branch-free: next full tile, or the last one again
      if constexpr (DENSE) {
        last_start = (int64_t)(dense_next < dense_end ? dense_next : dense_end - 1) * 64;
        dense_next++;
        return last_start;
      }
      const bool any = todo != 0;
      const int t = any ? __ffsll((unsigned long long)todo) - 1 : 0;
      const int64_t s = (int64_t)__builtin_amdgcn_readlane(my_idx, t) * 64;
      todo &= todo - 1;  // stays 0 once empty
      last_start = any ? s : last_start;
      return last_start;
    };
    const int64_t s0 = pop_or_last();
    // transfers in the rotation of the loop (K1, V0, K0, V1), so that the loop's waits hold from the first phase on
    dma_k(H0{}, s0);
    dma_k(H1{}, s0);
    __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): the Q transfers, issued before these eight, have landed
    read_q();
    dma_v(H0{}, s0);
    int64_t s1 = pop_or_last(), s2 = pop_or_last();
    // the row maxima over the first half tile become the softmax reference; st[.][0] stays for the first phase
    __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): the first K half
    scores_half(H0{});
    reads_done();
    dma_k(H0{}, s1);  // the K half the second phase reads

    dma_v(H1{}, s0);
    m_i[0] = half_max(st[0][0]);
    m_i[1] = half_max(st[1][0]);
    mneg[0] = -m_i[0];
    mneg[1] = -m_i[1];
#pragma unroll
    for (int qt = 0; qt < 2; qt++)  // the first phase's PV stage adds nothing
#pragma unroll
      for (int jj = 0; jj < 2; jj++)
#pragma unroll
        for (int e = 0; e < 8; e++) pf[qt][1][jj][e] = (E)0.f;
#pragma unroll
    for (int jj = 0; jj < 2; jj++)
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int e = 0; e < 8; e++) vfr[jj][dt][e] = (E)0.f;
    for (int i = n_full; i > 0; i--) {  // past the end of the list the transfers re-read the last tile
      phase(H0{}, s1, s1);
      phase(H1{}, s2, s1);
      s1 = s2;
      s2 = pop_or_last();
    }
    load_merge_operands();
    pv_half(H1{});  // PV of the last unit
    // a reference that was too low shows up as a huge or non-finite row sum
    const float big = 1.2676506e30f;  // 2^100
    redo = __any(!(l_i[0] < big) || !(l_i[1] < big));
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): no transfer is still writing LDS

  if (redo) {  // rare: recompute the query block with the online softmax
    reset_state();
    if constexpr (DENSE) {
      for (int t = dense_begin; t < dense_end; t++) robust_tile((int64_t)t * 64);
    } else {
      uint64_t again = __ballot(my_valid && my_idx != ragged_blk);
      while (again) {
        const int t = __ffsll((unsigned long long)again) - 1;
        again &= again - 1;
        robust_tile((int64_t)__builtin_amdgcn_readlane(my_idx, t) * 64);
      }
    }
  }
  for (; n_ragged > 0; n_ragged--) robust_tile((int64_t)ragged_blk * 64);

  // Output: lane (c, hh) holds for query c + 32*qt the head_dim values dt*32 + 8*g4 + 4*hh + {0..3}.  One exchange with
  // lane ^ 32 per packed word hands every lane eight consecutive head_dim values (hh = 0: group g4 = 2*gp, hh = 1:
  // group 2*gp + 1), so a row receives 32 contiguous bytes per store instruction.
  if constexpr (SPLIT) {
    // the second wave of a pair hands its state over: accumulators [dt][qt] into its four (now idle) 4 KB buffers,
    // register r of lane l at float r*64 + l, references and row sums into lds_ml; the first wave folds them in
    auto xo = [&](int w, int dt, int qt) -> float* {
      unsigned char* a = dt == 0 ? (qt == 0 ? lds_k0 : lds_k1) : (qt == 0 ? lds_v0 : lds_v1);
      return reinterpret_cast<float*>(a + w * (kHalf * 2));
    };
    if (split == 1) {
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int qt = 0; qt < 2; qt++)
#pragma unroll
          for (int r = 0; r < 16; r++) xo(wave, dt, qt)[r * 64 + lane] = ot[dt][qt][r];
#pragma unroll
      for (int qt = 0; qt < 2; qt++) {
        lds_ml[(wave * 4 + qt) * 64 + lane] = m_i[qt];
        lds_ml[(wave * 4 + 2 + qt) * 64 + lane] = l_i[qt];
      }
    }
    __syncthreads();
    if (split == 1 || ghost) return;
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
      const float m1 = lds_ml[((wave + 1) * 4 + qt) * 64 + lane];
      const float l1 = lds_ml[((wave + 1) * 4 + 2 + qt) * 64 + lane];
      const float mt = fmaxf(m_i[qt], m1);
      const float a0 = mt == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_i[qt] - mt);  // exp2(-inf) = 0 for an empty half
      const float a1 = mt == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m1 - mt);
      l_i[qt] = l_i[qt] * a0 + l1 * a1;
      m_i[qt] = mt;
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) ot[dt][qt][r] = ot[dt][qt][r] * a0 + xo(wave + 1, dt, qt)[r * 64 + lane] * a1;
    }
  }
  if (!merge_loaded) load_merge_operands();
  float g0[2], g1[2];
#pragma unroll
  for (int qt = 0; qt < 2; qt++) {
    asm volatile("" : "+v"(g_raw[qt]));  // first use of the pair: the wait for its load falls here, behind the last PV stage
    union { uint16_t u; E e; } lo, hi;
    lo.u = (uint16_t)g_raw[qt];
    hi.u = (uint16_t)(g_raw[qt] >> 16);
    g0[qt] = (float)lo.e;
    g1[qt] = (float)hi.e;
  }
#pragma unroll
  for (int qt = 0; qt < 2; qt++) {
#pragma clang fp contract(off)  // the merge rounds each product and the sum separately, like the eager expression
    const float l = xh_sum(l_i[qt]);
    const float inv = l > 0.f ? 1.f / l : 0.f;
    const int64_t row = q0 + qt * 32 + c;
    const bool live = row < N;
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
      for (int gp = 0; gp < 2; gp++) {
        // two values per conversion instruction, words handled as vectors of two (a union of scalars would convert
        // and mask every value on its own)
        auto pack2 = [](float x, float y) -> uint32_t {
          V2 v;
          v[0] = (E)x;
          v[1] = (E)y;
          return __builtin_bit_cast(uint32_t, v);
        };
        union { uint32_t w[4]; uint4 u; } pc;
#pragma unroll
        for (int wi = 0; wi < 2; wi++) {
          const uint32_t a = pack2(ot[dt][qt][8 * gp + 2 * wi] * inv, ot[dt][qt][8 * gp + 2 * wi + 1] * inv);
          const uint32_t bw = pack2(ot[dt][qt][8 * gp + 4 + 2 * wi] * inv, ot[dt][qt][8 * gp + 4 + 2 * wi + 1] * inv);
          const auto r = __builtin_amdgcn_permlane32_swap(a, bw, false, false);
          pc.w[wi] = r[0];
          pc.w[2 + wi] = r[1];
        }
        const int d0 = dt * 32 + 8 * (2 * gp + hh);
        if (live) {
          if (!merge) {
            *reinterpret_cast<uint4*>(op + row * p.som + d0) = pc.u;
          } else {
            union { uint32_t w[4]; uint4 u; } oc, res;
            oc.u = oc_raw[dt][gp];
#pragma unroll
            for (int wi = 0; wi < 4; wi++) {  // products and sum each rounded to the I/O type, as the eager expression does
              const V2 o2 = __builtin_bit_cast(V2, oc.w[wi]);
              const V2 s2 = __builtin_bit_cast(V2, pc.w[wi]);
              const V2 x2 = __builtin_bit_cast(V2, pack2(g0[qt] * (float)o2[0], g0[qt] * (float)o2[1]));
              const V2 y2 = __builtin_bit_cast(V2, pack2(g1[qt] * (float)s2[0], g1[qt] * (float)s2[1]));
              res.w[wi] = pack2((float)x2[0] + (float)y2[0], (float)x2[1] + (float)y2[1]);
            }
            *reinterpret_cast<uint4*>((E*)p.merge_out + (((int64_t)b * N + row) * p.H + h) * 64 + d0) = res.u;
          }
        }
      }
    if (live && p.lse != nullptr && hh == 0)
      p.lse[((int64_t)b * p.H + h) * N + row] = l > 0.f ? (m_i[qt] + __builtin_amdgcn_logf(l)) * 0.6931471805599453f : -INFINITY;
  }
}

}  // namespace pipe

int launch_select_pipe(const AttnParams& p, int dtype, void* stream) {
  const int64_t nqb = (p.Lq + 63) / 64;
  const bool dense = p.idx == nullptr;  // no index list: every query block sweeps all key tiles
  if (dense && p.Lq != p.Lk) return fail(S3R_ERR_UNSUPPORTED, "dense sweep: Lq %lld != Lk %lld", (long long)p.Lq, (long long)p.Lk);
  // A dense sweep runs with two waves per query block where it has fewer waves than 1.5 per SIMD of the chip (256 CUs x
  // 4), and where its waves fill the chip's 2048 places (two per SIMD) a whole number of times plus a small rest: the
  // rest runs as a round of its own, and with half the key tiles per wave that round is half as long (16 656 pooled
  // tokens x 16 heads = 4176 waves: 1.27 -> 1.21 ms; without such a rest the split costs 2 %).
  const int64_t sweeps = nqb * p.B * p.H;
  const bool split = dense && (sweeps < 1536 || (sweeps > 2048 && sweeps % 2048 != 0 && (sweeps % 2048) * 5 < 2048));
  const int per_wg = split ? pipe::kWaves / 2 : pipe::kWaves;
  const int64_t nqg = (nqb + per_wg - 1) / per_wg;
  const int64_t total = nqg * p.B * p.H;
  if (total > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_select_attn: grid too large");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)total), blk(64 * pipe::kWaves);
#define S3R_PIPE_LAUNCH(E)                                                                                                       \
  do {                                                                                                                           \
    if (split) hipLaunchKernelGGL((pipe::select_pipe_kernel<E, true, true>), grid, blk, 0, st, p, (int)nqb, (int)nqg, (int)total); \
    else if (dense) hipLaunchKernelGGL((pipe::select_pipe_kernel<E, true>), grid, blk, 0, st, p, (int)nqb, (int)nqg, (int)total);  \
    else hipLaunchKernelGGL((pipe::select_pipe_kernel<E, false>), grid, blk, 0, st, p, (int)nqb, (int)nqg, (int)total);            \
  } while (0)
  if (dtype == S3R_BF16) S3R_PIPE_LAUNCH(bf16_t);
  else S3R_PIPE_LAUNCH(f16_t);
#undef S3R_PIPE_LAUNCH
  return check_launch("select_pipe_kernel");
}

}  // namespace s3r
