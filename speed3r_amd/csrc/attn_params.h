// Argument block shared by the attention kernels (compressed branch and selection branch).
#pragma once
#include <stdint.h>

namespace s3r {

struct AttnParams {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  float* lse;          // optional [B,H,Lq]
  float* scores;       // optional [B,H,Lq,Lk], compressed branch only
  const int32_t* idx;  // selection branch: [B,H,ceil(Lq/block),K]
  int32_t* topk_idx;   // compressed branch, fused selection: [B,H,Lq,K]
  int B, H;
  int64_t Lq, Lk;
  int D, block, K;
  int causal;          // compressed branch, generic kernel: key j counts for query i only if j <= i, see attn_simple.hip
  int64_t sqb, sqh, sqm;
  int64_t skb, skh, skn;
  int64_t svb, svh, svn;
  int64_t sob, soh, som;
  int64_t sib, sih, sim;
  float scale;
  // selection branch with fused gated merge (merge_out != nullptr): instead of o the kernel writes
  // merge_out[b,n,h*D+d] = gate[b,h,n,0]*o_cmp[b,h,n/block,d] + gate[b,h,n,1]*o_sel[b,h,n,d]  (contiguous [B,Lq,H*D])
  const void* merge_oc;
  const void* merge_gate;
  void* merge_out;
  int64_t scb, sch, scm;
  int64_t sgb, sgh, sgn;
};

// launchers implemented in the .hip files; each returns S3R_OK or an error code
// row-wise top-k; causal_lq > 0: row r (query r % causal_lq) ranks only its first min((q/64 + 1) * 64, cols) columns
int launch_topk_rows(const float* scores, int32_t* idx, int64_t rows, int cols, int64_t row_stride, int K, int64_t causal_lq, void* stream);
int launch_attn_simple(const AttnParams& p, int dtype, bool select, void* stream);
int launch_select_pipe(const AttnParams& p, int dtype, void* stream);
int launch_select_b16(const AttnParams& p, int dtype, void* stream);  // block 16
int launch_compressed_mfma(const AttnParams& p, int dtype, void* stream);

}  // namespace s3r
