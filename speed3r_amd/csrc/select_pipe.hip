// Selection-branch attention, software-pipelined variant (bf16 / fp16 I/O, block 64, head_dim 64).
//
// Same data flow and register layouts as select_mfma.hip (one wavefront per 64-row query block,
// S^T = K Q^T and O^T += V^T P^T on v_mfma_f32_32x32x16, V through LDS and transposed reads), but
// the three stages of consecutive key tiles overlap inside ONE wavefront:
//
//     iteration i :   A(i+1)  S^T MFMAs of the next tile          \  32 MFMAs, issued one per slot
//                     C(i-1)  PV MFMAs of the previous tile       /
//                     B(i)    softmax of the current tile            VALU work spread over the 32 slots
//
// An MFMA occupies the matrix pipe for 32 cycles but the wave's issue port for only a few, so
// the exp/convert work of B(i) runs in the shadow of the MFMAs of the neighbouring tiles.  The
// kernel runs one wave per SIMD (about 400 registers: two score tiles, two probability tiles, two
// K tiles, the output accumulators and the V fragments of one tile are live at once); latency
// is covered by distance instead of occupancy: K tiles are loaded two iterations ahead
// (global -> registers), V tiles one to two iterations ahead (global_load_lds into a ring of
// four LDS buffers per wave), and all transposed V reads of an iteration are issued at its top.
//
// The first iteration pairs B(0) with a C stage on an all-zero probability tile and the last one
// pairs B(n-1) with an A stage whose result is never read, so the loop body is uniform and free of
// branches (two iterations per trip, so that the register roles alternate without copies); the
// PV stage of the last tile runs after the loop.  Row sums are taken over the probabilities after
// their rounding to the I/O dtype (v_dot2c with a vector of ones).
//
// Softmax reference: softmax is shift invariant, so the pipelined loop uses ONE reference value
// per query row, the row maximum of the first tile, and never rescales the accumulators.  Later
// tiles may exceed the reference; exp2 of the excess is exact as long as it stays in fp32
// range.  If a row sum ends above 2^100 (or is not finite) the whole query block is recomputed
// by the unpipelined online-softmax stage, which also handles every occurrence of the ragged
// last key block.
#include "s3r_common.h"
#include "attn_params.h"
#include <type_traits>
#include <utility>

namespace s3r {
namespace pipe {

template <typename E> struct Mma;
template <> struct Mma<bf16_t> {
  typedef bf16x8 V8;
  typedef __bf16 V2 __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
  // position-fixed forms: accumulator in VGPRs with operands from AGPRs, and the other way round.  The compiler
  // does not see an MFMA in the asm statement, so the wait states a preceding VALU/AGPR write of an operand
  // needs are supplied here.
  static __device__ __forceinline__ void mma_v(f32x16& acc, V8 a, V8 b) { asm volatile("s_nop 3\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "a"(a), "a"(b)); }
  static __device__ __forceinline__ void mma_v_first(f32x16& acc, V8 a, V8 b) { asm volatile("s_nop 3\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=v"(acc) : "a"(a), "a"(b)); }
  static __device__ __forceinline__ void mma_a(f32x16& acc, V8 a, V8 b) { asm volatile("s_nop 3\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b)); }
  static __device__ __forceinline__ float dot_ones(V2 a, float acc) {
    V2 one;
    one[0] = (__bf16)1.0f;
    one[1] = (__bf16)1.0f;
    return __builtin_amdgcn_fdot2_f32_bf16(a, one, acc, false);
  }
};
template <> struct Mma<f16_t> {
  typedef f16x8 V8;
  typedef _Float16 V2 __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ f32x16 mma(V8 a, V8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ void mma_v(f32x16& acc, V8 a, V8 b) { asm volatile("s_nop 3\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "a"(a), "a"(b)); }
  static __device__ __forceinline__ void mma_v_first(f32x16& acc, V8 a, V8 b) { asm volatile("s_nop 3\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=v"(acc) : "a"(a), "a"(b)); }
  static __device__ __forceinline__ void mma_a(f32x16& acc, V8 a, V8 b) { asm volatile("s_nop 3\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b)); }
  static __device__ __forceinline__ float dot_ones(V2 a, float acc) {
    V2 one;
    one[0] = (_Float16)1.0f;
    one[1] = (_Float16)1.0f;
    return __builtin_amdgcn_fdot2(a, one, acc, false);
  }
};

union Frag {
  uint4 u;
  bf16x8 b;
  f16x8 h;
  s16x4 s[2];
};
template <typename E> __device__ __forceinline__ typename Mma<E>::V8 as_v8(const Frag& f);
template <> __device__ __forceinline__ bf16x8 as_v8<bf16_t>(const Frag& f) { return f.b; }
template <> __device__ __forceinline__ f16x8 as_v8<f16_t>(const Frag& f) { return f.h; }

__device__ __forceinline__ float xh_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xh_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <typename F, int... I> __device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F> __device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

constexpr float kSlack = 8.0f;
constexpr int kVTile = 64 * 64;  // elements per LDS V buffer
constexpr int kVBufs = 4;        // LDS V buffers per wave

template <typename E>
__global__ __launch_bounds__(256, 1) void select_pipe_kernel(AttnParams p, int nqb, int nqg, int total_wg) {
  typedef typename Mma<E>::V8 V8;
  typedef typename Mma<E>::V2 V2;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];

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
  E* vl = reinterpret_cast<E*>(lds_raw) + wave * (kVBufs * kVTile);

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

  f32x16 st[2][2][2];  // score tiles [parity][qt][kt]
  V8 pf[2][2][2][2];   // probability tiles [parity][qt][kt][jj]
  V8 ak[2][2][4];      // K tiles [parity][kt][ks]

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
  const int ldv_row = lane >> 3;
  const int ldv_chunk = (lane & 7) ^ (((ldv_row >> 1) & 1) << 2);
  const uint32_t voff = (uint32_t)ldv_row * (uint32_t)p.svn + ldv_chunk * 8;
  auto load_v = [&](int buf, int64_t start) {
    E* dst = vl + buf * kVTile;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const E* vb = vp + (start + i * 8) * p.svn;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(vb + voff),
                                       (__attribute__((address_space(3))) void*)(dst + i * 512), 16, 0, 0);
    }
  };
  const int i16 = lane & 15;
  const int tr_row = 4 * hh + (i16 >> 2);
  const int tr_chunk = (((lane >> 4) & 1) * 2 + ((i16 & 3) >> 1)) ^ (((tr_row >> 1) & 1) << 2);
  const int tr_off = tr_row * 128 + tr_chunk * 16 + (i16 & 1) * 8;
  // all V^T fragments of one tile: [kt][jj][dt], k-step (kt,jj) = keys kt*32 + 16jj + {4hh.., 8+4hh..}
  auto read_v = [&](V8 (&vfr)[2][2][2], int buf) {
    const char* vbase = reinterpret_cast<const char*>(vl + buf * kVTile);
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

  // ---- one pipelined iteration; PAR = parity of the tile whose softmax runs here ----
  // cbuf: LDS buffer of the previous tile (C stage); k_start -> ak[PAR]; v_start -> LDS buffer vbuf.
  auto iteration = [&](auto par_tag, int cbuf, int64_t k_start, int64_t v_start, int vbuf) {
    constexpr int PAR = decltype(par_tag)::value;
    constexpr int OTH = PAR ^ 1;
    V8 vfr[2][2][2];
    read_v(vfr, cbuf);
    load_k(ak[PAR], k_start);
    load_v(vbuf, v_start);
    const float mneg[2] = {-m_i[0], -m_i[1]};

    // 32 slots, each: one MFMA, then the exponentials of two scores of the current tile.  Empty volatile asm
    // statements on the score tuple before and on the probability tuple after pin the VALU instructions of the
    // slot; a scheduling barrier after every slot keeps the MFMAs where they are written.
    static_for<32>([&](auto s_tag) {
      constexpr int s = decltype(s_tag)::value;
      constexpr int j = s >> 1;
      if constexpr ((s & 1) == 0) {  // A(i+1): S^T of the next tile, accumulators (VGPRs) taken round-robin
        constexpr int ks = j >> 2, qt = (j >> 1) & 1, kt = j & 1;
        if constexpr (ks == 0) {
          f32x16 z;
#pragma unroll
          for (int r = 0; r < 16; r++) z[r] = 0.f;
          st[OTH][qt][kt] = Mma<E>::mma(ak[OTH][kt][ks], bq[qt][ks], z);
        } else {
          st[OTH][qt][kt] = Mma<E>::mma(ak[OTH][kt][ks], bq[qt][ks], st[OTH][qt][kt]);
        }
      } else {  // C(i-1): PV of the previous tile into the AGPR accumulators
        constexpr int kj = j >> 2, dt = (j >> 1) & 1, qt = j & 1;
        constexpr int kt = kj >> 1, jj = kj & 1;
        ot[dt][qt] = Mma<E>::mma(vfr[kt][jj][dt], pf[OTH][qt][kt][jj], ot[dt][qt]);
      }
      {  // B(i): element pair e, e+1 of the current tile
        constexpr int e = 2 * s;
        constexpr int qt = e >> 5, kt = (e >> 4) & 1, r = e & 15, jj = r >> 3, e8 = r & 7;
        asm volatile("" : "+v"(st[PAR][qt][kt]));
        const float x0 = __builtin_amdgcn_exp2f(fmaf(st[PAR][qt][kt][r], sl2, mneg[qt]));
        const float x1 = __builtin_amdgcn_exp2f(fmaf(st[PAR][qt][kt][r + 1], sl2, mneg[qt]));
        V2 pk;
        pk[0] = (E)x0;
        pk[1] = (E)x1;
        pf[PAR][qt][kt][jj][e8] = pk[0];
        pf[PAR][qt][kt][jj][e8 + 1] = pk[1];
        l_i[qt] = Mma<E>::dot_ones(pk, l_i[qt]);
        asm volatile("" : "+v"(pf[PAR][qt][kt][jj]), "+v"(l_i[qt]));
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  // PV of a finished probability tile without anything to overlap it with
  auto pv_only = [&](const V8 (&pp)[2][2][2], int buf) {
    V8 vfr[2][2][2];
    read_v(vfr, buf);
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
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): earlier reads of LDS buffer 0 are done
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
    pv_only(pf[0], 0);
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
    // prologue: tiles 0 and 1 in flight, S^T of tile 0 and its row maxima (the softmax reference), an all-zero
    // probability tile for the first C stage.  Past the end of the list the prefetches re-read the last tile.
    const int64_t s0 = pop_start();
    load_k(ak[0], s0);
    load_v(0, s0);
    int64_t last_start = s0;
    auto pop_or_last = [&]() -> int64_t {  // branch-free: next full tile, or the last one again
      const bool any = todo != 0;
      const int t = any ? __ffsll((unsigned long long)todo) - 1 : 0;
      const int64_t s = (int64_t)__builtin_amdgcn_readlane(my_idx, t) * 64;
      todo &= todo - 1;  // stays 0 once empty
      last_start = any ? s : last_start;
      return last_start;
    };
    int64_t v_next = pop_or_last();  // tile i+1
    load_k(ak[1], v_next);
    int64_t k_next = pop_or_last();  // tile i+2
    scores_only(st[0], ak[0]);
    m_i[0] = row_max(st[0][0]);
    m_i[1] = row_max(st[0][1]);
#pragma unroll
    for (int qt = 0; qt < 2; qt++)
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int jj = 0; jj < 2; jj++)
#pragma unroll
          for (int e = 0; e < 8; e++) pf[1][qt][kt][jj][e] = (E)0.f;

    int i = 0;
    for (int pr = n_full >> 1; pr > 0; pr--) {  // two iterations per trip, no branch inside
      iteration(std::integral_constant<int, 0>{}, i == 0 ? 0 : (i - 1) & 3, k_next, v_next, (i + 1) & 3);
      v_next = k_next;
      k_next = pop_or_last();
      i++;
      iteration(std::integral_constant<int, 1>{}, (i - 1) & 3, k_next, v_next, (i + 1) & 3);
      v_next = k_next;
      k_next = pop_or_last();
      i++;
    }
    if (n_full & 1) {
      iteration(std::integral_constant<int, 0>{}, i == 0 ? 0 : (i - 1) & 3, k_next, v_next, (i + 1) & 3);
      asm volatile("s_nop 15\n\ts_nop 15");  // the asm MFMAs' results settle before compiler-scheduled code reads them
      pv_only(pf[0], (n_full - 1) & 3);
    } else {
      asm volatile("s_nop 15\n\ts_nop 15");
      pv_only(pf[1], (n_full - 1) & 3);
    }
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

}  // namespace pipe

int launch_select_pipe(const AttnParams& p, int dtype, void* stream) {
  const int64_t nqb = (p.Lq + 63) / 64;
  const int64_t nqg = (nqb + 3) / 4;
  const int64_t total = nqg * p.B * p.H;
  if (total > 0x7fffffffLL) return fail(S3R_ERR_UNSUPPORTED, "s3r_select_attn: grid too large");
  const size_t lds = (size_t)4 * pipe::kVBufs * pipe::kVTile * 2;  // 128 KB of dynamic LDS
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)total), blk(256);
  hipError_t e;
  if (dtype == S3R_BF16) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&pipe::select_pipe_kernel<bf16_t>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail(S3R_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    hipLaunchKernelGGL(pipe::select_pipe_kernel<bf16_t>, grid, blk, lds, st, p, (int)nqb, (int)nqg, (int)total);
  } else {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&pipe::select_pipe_kernel<f16_t>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail(S3R_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    hipLaunchKernelGGL(pipe::select_pipe_kernel<f16_t>, grid, blk, lds, st, p, (int)nqb, (int)nqg, (int)total);
  }
  return check_launch("select_pipe_kernel");
}

}  // namespace s3r
