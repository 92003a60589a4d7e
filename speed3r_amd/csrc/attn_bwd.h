// Argument block of the attention backward kernels (selection branch and, without an index tensor, the dense
// compressed branch).
#pragma once
#include <stdint.h>

namespace s3r {

struct BwdParams {
  const void* q;
  const void* k;
  const void* v;
  const void* dout;        // gradient of the attention output, layout of q
  const float* lse;        // [B,H,Lq] natural-log log-sum-exp of the scaled scores (forward output)
  const float* delta;      // [B,H,Lq] rowsum(dout * out)
  void* dq;                // nullptr: skip the dQ kernel
  void* dk;                // nullptr: skip the dK/dV kernel
  void* dv;
  const int32_t* idx;      // [B,H,ceil(Lq/block),K] block indices of the forward, nullptr: every key tile (dense)
  const int32_t* kq_list;  // key-centric lists: query-block ids grouped by key block, [B,H,list_stride]
  const int32_t* kq_off;   // [B,H,ceil(Lk/block)+1] offsets of each key block's list
  int64_t list_stride;
  int B, H;
  int64_t Lq, Lk;
  int K;
  int block;               // tokens per block of the selection branch: 64 or 16 (ignored without idx)
  int64_t sqb, sqh, sqm;
  int64_t skb, skh, skn;
  int64_t svb, svh, svn;
  int64_t sgb, sgh, sgm;   // dout
  int64_t sdqb, sdqh, sdqm;
  int64_t sdkb, sdkh, sdkn;
  int64_t sdvb, sdvh, sdvn;
  int64_t sib, sih, sim;
  float scale;
};

int launch_attn_bwd(const BwdParams& p, int dtype, void* stream);
int launch_key_block_lists(const int32_t* idx, int32_t* kq_list, int32_t* kq_off, int B, int H, int64_t nqb, int K, int64_t nkb,
                           int64_t sib, int64_t sih, int64_t sim, int64_t list_stride, void* stream);
int launch_bwd_delta(const void* o, const void* dout, float* delta, int B, int H, int64_t N, int64_t sob, int64_t soh, int64_t son,
                     int64_t sdb, int64_t sdh, int64_t sdn, int dtype, void* stream);

}  // namespace s3r
