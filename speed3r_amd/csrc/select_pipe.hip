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
//
// Shared tiles.  A CU's vector-cache -> LDS path moves 64 bytes per cycle; with private tiles a wave needs 8 KB per
// 16 MFMAs (512 matrix cycles), the four SIMDs together exactly those 64 bytes per cycle: the transfers, not the matrix
// pipe, set the pace.  Where the four query blocks of a workgroup walk the same key tiles -- always in a dense sweep,
// and in the list instance whenever the four lists hold the same blocks (neighbouring query blocks mostly do) -- the
// workgroup fetches every half tile ONCE: each wave transfers a quarter of it (one instruction of 1 KB) into a ring of
// four K halves and four V halves shared by the workgroup, and all four waves read their fragments from there.  One
// workgroup barrier per phase: behind it every wave's quarter of the halves read in this phase has landed and every
// wave has finished reading the halves of the phase before, which are the ones refilled in this phase (three phases
// ahead of their use).
//
// The queries are multiplied by scale * log2(e) once, in registers, and rounded back to the I/O type: the scores leave
// the matrix pipe as exponents of two and the loop spends no instruction on scaling them.  bf16 has fp32's exponent
// range, so its instance uses no softmax reference at all in the loop (exp2 of the score itself; row sums outside
// [2^-80, 2^100] send the query block to the online-softmax stage); fp16 subtracts the first half tile's row maximum.
#include "select_common.h"
#include "attn_params.h"

namespace s3r {
namespace pipe {
using namespace sel;

constexpr int kHalf = 32 * 64;  // elements per half tile
constexpr int kWaves = 4;  // wavefronts (= query blocks) per workgroup

// DENSE: no index list, every query block attends to all key tiles in order (the compressed branch's attention over
// the pooled tokens runs through this instance).
// SPLIT (with DENSE, for sweeps with too few query blocks to fill the chip): two waves share a query block, each
// sweeps half of the key tiles, and the first one folds the second one's accumulators into its own through LDS.
// EXACT (chosen when the caller asks for the log-sum-exp, i.e. for a backward pass that recomputes the probabilities from
// it): the queries stay as they are in memory and every fp32 score is scaled in the loop, as the reference kernel does.
template <typename E, bool DENSE, bool SPLIT, bool EXACT>
__global__ __launch_bounds__(64 * kWaves, 2) void select_pipe_kernel(AttnParams p, int nqb, int nqg, int total_wg) {
  static_assert(!SPLIT || DENSE, "the split sweep is a variant of the dense one");
  constexpr bool ALWAYS_SHARED = DENSE && !SPLIT;            // every query block of a dense sweep walks the same tiles
  constexpr bool NOREF = std::is_same<E, bf16_t>::value && !EXACT;  // no softmax reference inside the loop
  typedef typename Mma<E>::V8 V8;
  typedef typename Mma<E>::V2 V2;
  // Separate arrays: the compiler then knows that a read of one does not depend on a transfer into another.
  // Private tiles: four arrays of 16 KB, a wave's K half 0 / K half 1 / V half 0 / V half 1 buffer is its 4 KB of
  // k0a / k1a / v0a / v1a.  Shared tiles: eight arrays of 8 KB, ring slot j of K is the first 4 KB of the j-th k array,
  // ring slot j of V the first 4 KB of the j-th v array; a wave's own 4 KB (staged Q block, unpipelined stage) are
  // waves 0,1 in the a arrays, waves 2,3 in the b arrays.
  constexpr int kArrA = ALWAYS_SHARED ? 2 * kHalf * 2 : kWaves * kHalf * 2;
  constexpr int kArrB = ALWAYS_SHARED ? 2 * kHalf * 2 : 16;
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k0a[kArrA];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k0b[kArrB];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k1a[kArrA];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k1b[kArrB];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v0a[kArrA];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v0b[kArrB];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v1a[kArrA];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v1b[kArrB];
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
  // Every wave of the workgroup has to reach the workgroup's barriers (the hand-over of a split sweep, the phases of
  // shared tiles, the vote of the list instance), so a wave past the last query block repeats the last block's work
  // and stores nothing; in the list instance it leaves after the vote.
  const bool ghost = qb >= nqb;
  qb = qb < nqb ? qb : nqb - 1;

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

  auto region = [&](unsigned char* a, unsigned char* b, int w) -> E* {  // wave w's 4 KB of an array (pair)
    if constexpr (ALWAYS_SHARED) return reinterpret_cast<E*>((w >> 1) ? b : a) + (w & 1) * kHalf;
    else return reinterpret_cast<E*>(a) + w * kHalf;
  };
  auto k_half = [&](auto hf) -> E* {
    if constexpr (decltype(hf)::value == 0) return region(lds_k0a, lds_k0b, wave);
    else return region(lds_k1a, lds_k1b, wave);
  };
  auto v_half = [&](auto hf) -> E* {
    if constexpr (decltype(hf)::value == 0) return region(lds_v0a, lds_v0b, wave);
    else return region(lds_v1a, lds_v1b, wave);
  };
  // the private-tile loop names its buffers through ONE array each (a pointer that may point into either array of a
  // pair would make the compiler wait for every transfer in flight)
  auto k_half_of = [&](auto hf, auto) -> E* {
    static_assert(!ALWAYS_SHARED, "private tiles only");
    return reinterpret_cast<E*>(decltype(hf)::value == 0 ? lds_k0a : lds_k1a) + wave * kHalf;
  };
  auto v_half_of = [&](auto hf, auto) -> E* {
    static_assert(!ALWAYS_SHARED, "private tiles only");
    return reinterpret_cast<E*>(decltype(hf)::value == 0 ? lds_v0a : lds_v1a) + wave * kHalf;
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
  if (!SPLIT && !ALWAYS_SHARED && ghost) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): no transfer may still write LDS when the wave ends
    return;
  }
  if (!SPLIT && !ALWAYS_SHARED && n_full + n_ragged == 0 && p.merge_out == nullptr) {  // nothing to attend to: zeros (the merge path goes on and merges zeros)
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
  auto dma_k = [&](auto hf, auto ab, int64_t start) {  // keys start + 32*hf .. +31
    constexpr int HF = decltype(hf)::value;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(kp + (start + 32 * HF) * p.skn), 0, 0x7fffffff, 0x00020000);
    __attribute__((address_space(3))) void* dst = (__attribute__((address_space(3))) void*)k_half_of(hf, ab);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, k_voff[0], 0, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, k_voff[1], k_step, 1024, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, k_voff[0], 2 * k_step, 2048, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, k_voff[1], 3 * k_step, 3072, 0);
  };
  auto dma_v = [&](auto hf, auto ab, int64_t start) {
    constexpr int HF = decltype(hf)::value;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(vp + (start + 32 * HF) * p.svn), 0, 0x7fffffff, 0x00020000);
    __attribute__((address_space(3))) void* dst = (__attribute__((address_space(3))) void*)v_half_of(hf, ab);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, v_voff, 0, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, v_voff, v_step, 1024, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, v_voff, 2 * v_step, 2048, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, v_voff, 3 * v_step, 3072, 0);
  };
  // Shared tiles: ring slots (the V slots overlap the staged Q blocks of waves 0 and 2, so the first V transfers wait
  // for a barrier behind everybody's read of Q).  A wave moves rows 8*wave .. 8*wave+7 of a half: what instruction
  // number `wave` of dma_k / dma_v moves.
  auto k_ring = [&](auto r) -> E* {
    constexpr int R = decltype(r)::value;
    return reinterpret_cast<E*>(R == 0 ? lds_k0a : R == 1 ? lds_k0b : R == 2 ? lds_k1a : lds_k1b);
  };
  auto v_ring = [&](auto r) -> E* {
    constexpr int R = decltype(r)::value;
    return reinterpret_cast<E*>(R == 0 ? lds_v0a : R == 1 ? lds_v0b : R == 2 ? lds_v1a : lds_v1b);
  };
  const uint32_t k_voff_w = (wave & 1) ? k_voff[1] : k_voff[0];
  const uint32_t k_soff_w = (uint32_t)wave * 8u * (uint32_t)p.skn * (uint32_t)sizeof(E);
  const uint32_t v_soff_w = (uint32_t)wave * 8u * (uint32_t)p.svn * (uint32_t)sizeof(E);
  auto dma_k_piece = [&](auto r, int64_t first_key) {  // this wave's quarter of keys first_key .. +31 into ring slot r
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(kp + first_key * p.skn), 0, 0x7fffffff, 0x00020000);
    __attribute__((address_space(3))) void* dst = (__attribute__((address_space(3))) void*)(reinterpret_cast<char*>(k_ring(r)) + wave * 1024);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, k_voff_w, k_soff_w, 0, 0);
  };
  auto dma_v_piece = [&](auto r, int64_t first_key) {
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(vp + first_key * p.svn), 0, 0x7fffffff, 0x00020000);
    __attribute__((address_space(3))) void* dst = (__attribute__((address_space(3))) void*)(reinterpret_cast<char*>(v_ring(r)) + wave * 1024);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, dst, 16, v_voff, v_soff_w, 0, 0);
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
  auto read_k_at = [&](const E* buf, V8 (&dst)[4]) {  // A operand: lane = key row, head_dim chunk hh + 2*ks
    const char* kbase = reinterpret_cast<const char*>(buf);
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
  auto read_v_at = [&](const E* buf, V8 (&dst)[2][2]) {  // V^T fragments [jj][dt]: keys 16jj + {4hh.., 8+4hh..} of the half
    const char* vbase = reinterpret_cast<const char*>(buf);
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
  auto read_v = [&](auto hf, V8 (&dst)[2][2]) { read_v_at(v_half(hf), dst); };
  auto row_max = [&](const f32x16 (&s)[2]) -> float {  // over this lane's 32 keys and its partner's
    float mx = s[0][0];
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[kt][r]);
    return xh_max(mx) * (EXACT ? sl2 : 1.f);
  };
  auto half_max = [&](const f32x16& sc) -> float {  // over this lane's 16 keys of a half tile and its partner's
    float mx = sc[0];
#pragma unroll
    for (int r = 1; r < 16; r++) mx = fmaxf(mx, sc[r]);
    return xh_max(mx) * (EXACT ? sl2 : 1.f);
  };
  auto scores_half_at = [&](const E* buf) {  // st[.][0] from a K half in LDS
    constexpr int HF = 0;
    read_k_at(buf, ak);
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
  // Private tiles (ring_tag < 0): after its fragments are read, K half KT^1 is refilled from tile k_next and V half KT
  // from tile v_next.
  // Shared tiles (ring_tag = unit number mod 4): K half of unit u+1 from ring slot (u+1)%4, V half of unit u from slot
  // u%4; this wave's quarter of the K half of unit u+4 (first key k_next) goes into slot u%4 and of the V half of unit
  // u+3 (first key v_next) into slot (u+3)%4, both read in the phase before.  The wait in front of the barrier covers
  // this wave's quarters of the two halves read here: transfers complete in order, two per phase, and the four issued
  // since (units u+2, u+3 of K and u+1, u+2 of V) may stay in flight.
  // Empty volatile asm statements on the score tuple before and on the probability tuple after pin the VALU
  // instructions of a slot; the scheduling barrier after every slot keeps the MFMAs where they are written.
  float mneg[2];
  float px[2] = {0.f, 0.f};  // the exponentials of the slot before
  auto phase = [&](auto kt_tag, auto ring_tag, int64_t k_next, int64_t v_next) {
    constexpr int KT = decltype(kt_tag)::value;
    constexpr int OT = KT ^ 1;
    constexpr int U = decltype(ring_tag)::value;
    constexpr bool SH = U >= 0;
    typedef std::integral_constant<int, OT> HO;
    typedef std::integral_constant<int, SH ? 0 : -1 - U> AB;  // private tiles: ring_tag -1 = a arrays, -2 = b arrays
    static_for<16>([&](auto j_tag) {
      constexpr int j = decltype(j_tag)::value;
      if constexpr (SH) {
        if constexpr (j == 0) {
          __builtin_amdgcn_s_waitcnt(0x0074);  // vmcnt(4), lgkmcnt(0)
          __builtin_amdgcn_s_barrier();
          read_k_at(k_ring(std::integral_constant<int, (U + 1) & 3>{}), ak);
        }
        if constexpr (j == 2) dma_k_piece(std::integral_constant<int, U & 3>{}, k_next);
        if constexpr (j == 8) read_v_at(v_ring(std::integral_constant<int, U & 3>{}), vfr);
        if constexpr (j == 10) dma_v_piece(std::integral_constant<int, (U + 3) & 3>{}, v_next);
      } else {
        // a half buffer is refilled two slots after its fragments were requested, once they have arrived
        if constexpr (j == 0) {
          wait_transfer();
          read_k_at(k_half_of(HO{}, AB{}), ak);
        }
        if constexpr (j == 2) {
          reads_done();
          dma_k(HO{}, AB{}, k_next);
        }
        if constexpr (j == 8) {
          wait_transfer();
          read_v_at(v_half_of(kt_tag, AB{}), vfr);
        }
        if constexpr (j == 10) {
          reads_done();
          dma_v(kt_tag, AB{}, v_next);
        }
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
        // The slot starts the two exponentials of its own pair of scores and rounds and sums the pair of the slot
        // BEFORE it (the first slot: the last pair of the unit before, whose probabilities the PV stage needs from
        // its sixth slot on): nothing in a slot waits for an exponential started in the same slot.
        constexpr int e = 2 * j;
        constexpr int qt = e >> 4, r = e & 15;
        constexpr int pe = (e + 30) & 31, PT = j == 0 ? OT : KT;
        constexpr int pqt = pe >> 4, pjj = (pe & 15) >> 3, pe8 = pe & 7;
        asm volatile("" : "+v"(st[qt][KT]));
        const float x0 = __builtin_amdgcn_exp2f(EXACT ? fmaf(st[qt][KT][r], sl2, mneg[qt]) : NOREF ? st[qt][KT][r] : st[qt][KT][r] + mneg[qt]);
        const float x1 = __builtin_amdgcn_exp2f(EXACT ? fmaf(st[qt][KT][r + 1], sl2, mneg[qt]) : NOREF ? st[qt][KT][r + 1] : st[qt][KT][r + 1] + mneg[qt]);
        V2 pk;
        pk[0] = (E)px[0];
        pk[1] = (E)px[1];
        pf[pqt][PT][pjj][pe8] = pk[0];
        pf[pqt][PT][pjj][pe8 + 1] = pk[1];
        // row sums over the unrounded probabilities, as the reference's tl.sum(p) before p.to(v.dtype); the pair is
        // added first: two additions chained on the sum stall the second one
        l_i[pqt] += px[0] + px[1];
        px[0] = x0;
        px[1] = x1;
        asm volatile("" : "+v"(pf[pqt][PT][pjj]), "+v"(l_i[pqt]), "+v"(px[0]), "+v"(px[1]));
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // Unpipelined stage with a true online softmax: one key tile (possibly ragged) from global memory.
  float qs = EXACT ? sl2 : 1.f;  // what a score of the unpipelined stage is still to be multiplied by: 1 while the queries carry the scale
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
      const float mx = row_max(st[qt]) * (EXACT ? 1.f : qs);
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
            const float x0 = __builtin_amdgcn_exp2f(fmaf(st[qt][kt][8 * jj + e], qs, -m_new));
            const float x1 = __builtin_amdgcn_exp2f(fmaf(st[qt][kt][8 * jj + e + 1], qs, -m_new));
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
    // ... and the queries as they are in memory: the recomputation scales the fp32 scores, like the reference kernel
    if constexpr (EXACT) return;
    const int q_last = (int)((N - q0 < 64 ? N - q0 : 64) - 1);
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
      const int row = 32 * qt + c < q_last ? 32 * qt + c : q_last;
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        Frag f;
        f.u = *reinterpret_cast<const uint4*>(qp + (q0 + row) * p.sqm + (hh + 2 * ks) * 8);
        bq[qt][ks] = as_v8<E>(f);
      }
    }
    qs = sl2;
  };

  bool redo = false;
  // Operands of the gated merge (epilogue): gate pair per query row, the query block's row of the compressed output
  // in the layout of this lane's accumulators.  Issued right after the main loop, so that their latency passes behind the last PV
  // stage instead of in front of the stores.
  const bool merge = p.merge_out != nullptr;
  uint32_t g_raw[2] = {0, 0};  // gate pair per query row, bits of the I/O type
  uint2 oc_raw[2][4];  // [dt][g4]: this lane's four head_dim values of group g4, the accumulators' own layout
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
        for (int g4 = 0; g4 < 4; g4++) oc_raw[dt][g4] = *reinterpret_cast<const uint2*>(ocp + dt * 32 + 8 * g4 + 4 * hh);
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
    // the queries carry the softmax scale and the change of base from here on (one rounding to the I/O type)
    if constexpr (!EXACT)
#pragma unroll
    for (int qt = 0; qt < 2; qt++)
#pragma unroll
      for (int ks = 0; ks < 4; ks++)
#pragma unroll
        for (int e = 0; e < 8; e++) bq[qt][ks][e] = (E)((float)bq[qt][ks][e] * sl2);
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
    // the first half tile's scores are in st[.][0]: softmax reference (fp16 only: its row maxima), nothing for the first
    // phase's PV stage to add
    auto first_unit_done = [&]() {
      if constexpr (NOREF) {
        m_i[0] = m_i[1] = 0.f;
      } else {
        m_i[0] = half_max(st[0][0]);
        m_i[1] = half_max(st[1][0]);
      }
      mneg[0] = -m_i[0];
      mneg[1] = -m_i[1];
#pragma unroll
      for (int qt = 0; qt < 2; qt++)
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
    };
    typedef std::integral_constant<int, 0> U0;
    typedef std::integral_constant<int, 1> U1;
    typedef std::integral_constant<int, 2> U2;
    typedef std::integral_constant<int, 3> U3;
    if constexpr (ALWAYS_SHARED) {
      // Units 0..3 of K and 0..2 of V, in the order the loop goes on with (K of unit u+4, V of unit u+3 in phase u).
      int64_t sa = pop_or_last(), sb = pop_or_last();
      dma_k_piece(U0{}, sa);
      dma_k_piece(U1{}, sa + 32);
      dma_k_piece(U2{}, sb);
      dma_k_piece(U3{}, sb + 32);
      __builtin_amdgcn_s_waitcnt(0x0F74);  // vmcnt(4): the Q transfers, issued before these four, have landed
      read_q();                            // (ends with lgkmcnt(0))
      __builtin_amdgcn_s_barrier();        // every wave has read its Q block: the V slots are free
      dma_v_piece(U0{}, sa);
      dma_v_piece(U1{}, sa + 32);
      dma_v_piece(U2{}, sb);
      __builtin_amdgcn_s_waitcnt(0x0F76);  // vmcnt(6): this wave's quarter of the first K half ...
      __builtin_amdgcn_s_barrier();        // ... and the other three
      scores_half_at(k_ring(U0{}));
      first_unit_done();
      // The loop's wait (four transfers may stay in flight) assumes its own issue order, K of unit u+4 and V of unit
      // u+3 in phase u; the start-up sent K ahead of V, so everything sent so far has to land before the first phase.
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      for (int i = n_full >> 1; i > 0; i--) {  // two tiles per round; past the end of the list the transfers re-read the last tile
        const int64_t sc = pop_or_last(), sd = pop_or_last();
        phase(H0{}, U0{}, sc, sb + 32);
        phase(H1{}, U1{}, sc + 32, sc);
        phase(H0{}, U2{}, sd, sc + 32);
        phase(H1{}, U3{}, sd + 32, sd);
        sb = sd;
      }
      if (n_full & 1) {  // the ring is back at slot 0 after every round
        const int64_t sc = pop_or_last();
        phase(H0{}, U0{}, sc, sb + 32);
        phase(H1{}, U1{}, sc + 32, sc);
      }
    } else {
      auto run_private = [&](auto ab) {  // ab = 0: this wave's buffers are in the a arrays, 1: in the b arrays
        typedef std::integral_constant<int, -1 - decltype(ab)::value> Priv;
        const int64_t s0 = pop_or_last();
        // transfers in the rotation of the loop (K1, V0, K0, V1), so that the loop's waits hold from the first phase on
        dma_k(H0{}, ab, s0);
        dma_k(H1{}, ab, s0);
        __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): the Q transfers, issued before these eight, have landed
        read_q();
        dma_v(H0{}, ab, s0);
        int64_t s1 = pop_or_last(), s2 = pop_or_last();
        __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): the first K half
        scores_half_at(k_half_of(H0{}, ab));
        reads_done();
        dma_k(H0{}, ab, s1);  // the K half the second phase reads

        dma_v(H1{}, ab, s0);
        first_unit_done();
        for (int i = n_full; i > 0; i--) {  // past the end of the list the transfers re-read the last tile
          phase(H0{}, Priv{}, s1, s1);
          phase(H1{}, Priv{}, s2, s1);
          s1 = s2;
          s2 = pop_or_last();
        }
      };
      run_private(std::integral_constant<int, 0>{});
    }
    if constexpr (ALWAYS_SHARED) {
      // the later stages write the V slots' memory (every wave its own 4 KB): nobody may still read a slot, and no
      // transfer (the last ones re-read the last tile) may still be on its way into one
      __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0), lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
    }
    load_merge_operands();
    {  // the last pair of the last unit
      V2 pk;
      pk[0] = (E)px[0];
      pk[1] = (E)px[1];
      pf[1][1][1][6] = pk[0];
      pf[1][1][1][7] = pk[1];
      l_i[1] += px[0] + px[1];
    }
    pv_half(H1{});  // PV of the last unit
    // The row sums tell whether the loop's shortcuts held.  They add the unrounded fp32 probabilities, all of them
    // >= 0, so a lane's sum is at least as large as each of its probabilities.
    //  * fp16: a sum below 65504 proves that no probability left fp16's range when it was rounded (the reference, the
    //    first half tile's row maximum, may lie below later scores).
    //  * bf16 (no reference, exp2 of the score itself): a sum below 2^20 proves that every score (times scale*log2(e))
    //    was below 20, a row total above 2^-20 that its largest one was above -20.  Inside that band the rounding of
    //    the scaled queries to bf16 (2^-9 of each product) moves a score by about a thousandth of the band's width or
    //    less; outside it the query block is recomputed from the queries as they are in memory.
    //  * EXACT, bf16: the reference is the first half tile's row maximum, a later score may exceed it by 100.
    const float big = NOREF ? 1048576.f : std::is_same<E, f16_t>::value ? 65504.f : 1.2676506e30f;
    redo = __any(!(l_i[0] < big) || !(l_i[1] < big));
    if constexpr (NOREF) redo = redo || __any(!(xh_sum(l_i[0]) > 9.5367e-7f) || !(xh_sum(l_i[1]) > 9.5367e-7f));
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
      return reinterpret_cast<float*>(dt == 0 ? (qt == 0 ? region(lds_k0a, lds_k0b, w) : region(lds_k1a, lds_k1b, w))
                                              : (qt == 0 ? region(lds_v0a, lds_v0b, w) : region(lds_v1a, lds_v1b, w)));
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
  // With the merge the stored value is gate0 * o_cmp + gate1 * (accumulator / row sum), evaluated in fp32 and rounded
  // ONCE: the selection output is never rounded on its own, nor are the two products (the eager expression rounds all
  // three and the sum: at most two rounding steps of the I/O type away, on the side of the exact value).
  float ocf[2][16];
  if (merge) {
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const V2 lo2 = __builtin_bit_cast(V2, oc_raw[dt][g4].x), hi2 = __builtin_bit_cast(V2, oc_raw[dt][g4].y);
        ocf[dt][4 * g4] = (float)lo2[0];
        ocf[dt][4 * g4 + 1] = (float)lo2[1];
        ocf[dt][4 * g4 + 2] = (float)hi2[0];
        ocf[dt][4 * g4 + 3] = (float)hi2[1];
      }
  }
#pragma unroll
  for (int qt = 0; qt < 2; qt++) {
    const float l = xh_sum(l_i[qt]);
    const float inv = l > 0.f ? 1.f / l : 0.f;
    const float ginv = g1[qt] * inv;
    const int64_t row = q0 + qt * 32 + c;
    const bool live = row < N && !(ALWAYS_SHARED && ghost);
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
        auto value = [&](int r) -> float {
          return merge ? fmaf(ot[dt][qt][r], ginv, g0[qt] * ocf[dt][r]) : ot[dt][qt][r] * inv;
        };
        union { uint32_t w[4]; uint4 u; } pc;
#pragma unroll
        for (int wi = 0; wi < 2; wi++) {
          const uint32_t a = pack2(value(8 * gp + 2 * wi), value(8 * gp + 2 * wi + 1));
          const uint32_t bw = pack2(value(8 * gp + 4 + 2 * wi), value(8 * gp + 4 + 2 * wi + 1));
          const auto r = __builtin_amdgcn_permlane32_swap(a, bw, false, false);
          pc.w[wi] = r[0];
          pc.w[2 + wi] = r[1];
        }
        const int d0 = dt * 32 + 8 * (2 * gp + hh);
        if (live) {
          if (!merge) *reinterpret_cast<uint4*>(op + row * p.som + d0) = pc.u;
          else *reinterpret_cast<uint4*>((E*)p.merge_out + (((int64_t)b * N + row) * p.H + h) * 64 + d0) = pc.u;
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
#define S3R_PIPE_LAUNCH(E, X)                                                                                                      \
  do {                                                                                                                           \
    if (split) hipLaunchKernelGGL((pipe::select_pipe_kernel<E, true, true, X>), grid, blk, 0, st, p, (int)nqb, (int)nqg, (int)total);       \
    else if (dense) hipLaunchKernelGGL((pipe::select_pipe_kernel<E, true, false, X>), grid, blk, 0, st, p, (int)nqb, (int)nqg, (int)total); \
    else hipLaunchKernelGGL((pipe::select_pipe_kernel<E, false, false, X>), grid, blk, 0, st, p, (int)nqb, (int)nqg, (int)total);           \
  } while (0)
  const bool exact = p.lse != nullptr;  // a caller that wants the log-sum-exp wants it to the reference's precision
  if (dtype == S3R_BF16) {
    if (exact) S3R_PIPE_LAUNCH(bf16_t, true);
    else S3R_PIPE_LAUNCH(bf16_t, false);
  } else {
    if (exact) S3R_PIPE_LAUNCH(f16_t, true);
    else S3R_PIPE_LAUNCH(f16_t, false);
  }
#undef S3R_PIPE_LAUNCH
  return check_launch("select_pipe_kernel");
}

}  // namespace s3r
