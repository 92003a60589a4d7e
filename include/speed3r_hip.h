/*
 * speed3r_hip.h -- C ABI of the MI355X (gfx950) implementation of Speed3R's global
 * top-k block-sparse attention path.
 *
 * The reference implements this path in Python + Triton and has no FFI of its own; each
 * entry point below replaces the Python-level call named in its comment (paths relative to
 * the reference root).  All tensors are device pointers; strides are in ELEMENTS; the last
 * (head_dim) stride of every q/k/v/o tensor is 1.  Launches are asynchronous on `stream`
 * (a hipStream_t passed as void*; NULL = the default stream).  Every function returns
 * S3R_OK or a negative error code and never throws; s3r_last_error() gives the message of
 * the calling thread's last failure.  No entry point allocates memory.  State kept between calls: the
 * S3R_B16_KERNEL environment switch (read once, on first use) and the built-in score buffer of
 * s3r_compressed_attn_topk_static; nothing else.
 */
#ifndef SPEED3R_HIP_H
#define SPEED3R_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of q/k/v/o/gate tensors ("I/O dtype") */
#define S3R_F32 0
#define S3R_BF16 1
#define S3R_F16 2

#define S3R_OK 0
#define S3R_ERR_BAD_ARG (-1)     /* null pointer, non-positive size, misaligned pointer/stride */
#define S3R_ERR_UNSUPPORTED (-2) /* shape/dtype outside what the kernels are built for */
#define S3R_ERR_HIP (-3)         /* a HIP runtime call or launch failed */

/* Library identification, e.g. "speed3r_hip 0.1 gfx950". */
const char* s3r_version(void);
/* Message of the calling thread's most recent failing call ("" if none). */
const char* s3r_last_error(void);
/* Bit set of optional features built into this library. */
#define S3R_CAP_FUSED_TOPK 1 /* s3r_compressed_attn_topk selects without a scores buffer */
int s3r_capabilities(void);

/*
 * Block mean-pooling: y[b,h,j,:] = mean over tokens [j*block, min((j+1)*block, N)) of x[b,h,t,:].
 * Replaces F.avg_pool1d(kernel=stride=block) in pi3/models/layers/sparse_attention.py:97-99
 * (applied there to the packed qkv; pass H = 3*heads with the packed strides to pool all
 * three at once).  fp32 accumulation, result rounded to `dtype`.  y is [B,H,ceil(N/block),D]
 * with its own strides.  A ragged tail block is a mean over its valid tokens.
 * Requires D*sizeof(elt) to be a power-of-two multiple of 16 bytes up to 1024, and 16-byte
 * aligned pointers/strides.
 */
int s3r_pool_mean(const void* x, void* y, int B, int H, int64_t N, int D, int block,
                  int64_t sxb, int64_t sxh, int64_t sxn,
                  int64_t syb, int64_t syh, int64_t syn,
                  int dtype, void* stream);

/*
 * Compressed-branch attention with top-k block selection.
 * Replaces flash_attn_topk_func / forward_with_topk / _fwd_kernel_with_topk
 * (pi3/models/sparse_attn/flash_attention_topk.py:22-200,633-668), non-causal, no bias.
 *   o[b,h,i,:]   = softmax_j(scale * q[i].k[j]) v[j]          (I/O dtype)
 *   lse[b,h,i]   = log sum_j exp(scale * q[i].k[j])           (fp32, optional, [B,H,Lq] contiguous)
 *   topk_idx[b,h,i,0..K-1] = columns of the K largest raw UNSCALED fp32 q[i].k[j], ordered by
 *       descending 64-bit key (sortable(bits(s)) << 32 | Lk-1-j): descending score, equal
 *       scores lowest column first; if Lk < K the trailing slots hold Lk-1.
 *       (int32, optional, [B,H,Lq,K] contiguous)
 *   scores[b,h,i,j] = raw fp32 q[i].k[j]                      (optional, [B,H,Lq,Lk] contiguous)
 * When `scores` is given the indices are computed from exactly those stored values, so
 * s3r_topk_rows() on `scores` reproduces `topk_idx` bit for bit.  When `scores` is NULL the
 * scores never reach HBM: the attention output comes from a dense sweep of the selection
 * kernel and the indices from a top-k-only kernel that recomputes the scores on chip
 * (bf16/fp16, D == 64, K in {1,2,4,8,16,32}, Lk <= 2^21; two launches on `stream`).  `o` (and then `v`)
 * may be NULL when only the indices are wanted (MFMA path), `topk_idx` may be NULL when only the
 * attention is: a caller with two streams runs the two halves side by side.
 * Requires D <= 64 (D == 64 for the MFMA path), K a power of two <= 64.
 */
int s3r_compressed_attn_topk(const void* q, const void* k, const void* v,
                             void* o, float* lse, int32_t* topk_idx, float* scores,
                             int B, int H, int Lq, int Lk, int D, int K,
                             int64_t sqb, int64_t sqh, int64_t sqm,
                             int64_t skb, int64_t skh, int64_t skn,
                             int64_t svb, int64_t svh, int64_t svn,
                             int64_t sob, int64_t soh, int64_t som,
                             float softmax_scale, int dtype, void* stream);

/*
 * The causal variant of s3r_compressed_attn_topk: the IS_CAUSAL branches of _fwd_kernel_with_topk
 * (flash_attention_topk.py:71,93), which the reference layer never takes (it calls with causal=False).
 * Query i (row i of its 64-row block m = i / 64) sees the keys below end_n = min((m + 1) * 64, Lk) only:
 *   o, lse:   softmax over the keys j <= i;
 *   topk_idx: the K largest of the keys j < end_n, where a key j > i has the score -inf (it ranks below every finite
 *             score, lowest column first, as the reference's integer keys order it); if end_n < K the trailing slots
 *             hold end_n - 1;
 *   scores:   [B,H,Lq,Lk] fp32 work buffer, required with `topk_idx` (row i: raw scores of the keys j < end_n with
 *             -inf for j > i; columns from end_n on are not written).
 * Any I/O dtype, D <= 64, K a power of two <= 64; runs the generic (non-MFMA) kernels.  The reference's backward
 * ignores `causal` (flash_attention_topk.py:653-666 calls _flash_attn_backward without it), so s3r_attn_bwd on the
 * lse of this call reproduces the reference's gradients as they are.
 */
int s3r_compressed_attn_topk_causal(const void* q, const void* k, const void* v,
                                    void* o, float* lse, int32_t* topk_idx, float* scores,
                                    int B, int H, int Lq, int Lk, int D, int K,
                                    int64_t sqb, int64_t sqh, int64_t sqm,
                                    int64_t skb, int64_t skh, int64_t skn,
                                    int64_t svb, int64_t svh, int64_t svn,
                                    int64_t sob, int64_t soh, int64_t som,
                                    float softmax_scale, int dtype, void* stream);

/*
 * s3r_compressed_attn_topk with its score buffer built into the library: allocates nothing.
 * No counterpart in the reference.  For callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It is the `scores != NULL` path of
 * s3r_compressed_attn_topk (any I/O dtype, any K a power of two <= 64; indices selected from exactly the stored
 * fp32 scores, so results equal that call bit for bit) with the B*H*Lq*Lk scores held in a file-scope device array
 * of S3R_STATIC_SCORES_MAX floats (96 MiB per GPU the library runs on, kept until the process ends).  Larger
 * problems return S3R_ERR_UNSUPPORTED.  `o` and `topk_idx` are both required.  The first call on a device looks up
 * that device's copy of the array (no allocation; make it outside a graph capture).  All calls on one GPU share
 * the array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not.
 */
#define S3R_STATIC_SCORES_MAX (24u * 1024u * 1024u)
int s3r_compressed_attn_topk_static(const void* q, const void* k, const void* v,
                                    void* o, float* lse, int32_t* topk_idx,
                                    int B, int H, int Lq, int Lk, int D, int K,
                                    int64_t sqb, int64_t sqh, int64_t sqm,
                                    int64_t skb, int64_t skh, int64_t skn,
                                    int64_t svb, int64_t svh, int64_t svn,
                                    int64_t sob, int64_t soh, int64_t som,
                                    float softmax_scale, int dtype, void* stream);

/*
 * Row-wise exact top-k of a materialised fp32 score matrix (same ordering rule as above).
 * Stands for the streaming bitonic top-k inside _fwd_kernel_with_topk
 * (flash_attention_topk.py:112-132,145-152; topk_utils.py:11-23,438-501).
 * scores: `rows` rows of `cols` floats, row r at scores + r*row_stride; idx: [rows, K] int32.
 * 1 <= K <= 64.
 */
int s3r_topk_rows(const float* scores, int32_t* idx, int64_t rows, int cols, int64_t row_stride,
                  int K, void* stream);

/*
 * Selection-branch attention: every `block`-row query block attends to the K key blocks its
 * index row lists, in list order.
 * Replaces topk_blocksparse_attention / _topk_blocksparse_attention_fwd /
 * block_sparse_forward_kernel (pi3/models/sparse_attn/topk_blocksparse_attention.py:35-128,
 * 852-904,1093-1121).
 *   idx: int32 [B,H,ceil(N/block),K] (strides sib,sih,sim; last stride 1), block units;
 *        entries < 0 or with idx*block >= N are skipped; duplicates are attended twice.
 *   o:   I/O dtype [B,H,N,D];  lse: optional fp32 [B,H,N] contiguous.
 * Keys beyond N in a partial last block are masked out; a query block with no valid entry
 * gives zeros.  block in {4,16,32,64}, D <= 64 (MFMA paths: block 64 or 16, D == 64, bf16/fp16, K <= 64).
 * Rounding points of the 64-token MFMA kernel: with lse == NULL the queries are multiplied by
 * softmax_scale * log2(e) once and rounded to the I/O dtype, and the fp32 scores of those queries are exponents of two
 * (the reference scales each fp32 score, :100); a query block whose scaled scores leave [-20, 20] (bf16) is recomputed
 * with the reference's per-score scaling.  With lse != NULL (a forward whose backward will recompute the probabilities
 * from lse) every score is scaled in fp32 as in the reference.
 * The reference's larger blocks (128, 256; topk_blocksparse_attention.py:862) are the caller's to rewrite, as the
 * Python operator does: the list of a query block serves each of its 64-row parts, a listed key block j becomes the
 * entries r*j .. r*j+r-1 (r = block/64), and the call is made with block 64 and K*r entries per row.
 */
int s3r_select_attn(const void* q, const void* k, const void* v, const int32_t* idx,
                    void* o, float* lse,
                    int B, int H, int64_t N, int D, int block, int K,
                    int64_t sqb, int64_t sqh, int64_t sqn,
                    int64_t skb, int64_t skh, int64_t skn,
                    int64_t svb, int64_t svh, int64_t svn,
                    int64_t sob, int64_t soh, int64_t son,
                    int64_t sib, int64_t sih, int64_t sim,
                    float softmax_scale, int dtype, void* stream);

/*
 * Selection-branch attention with the gated merge in its epilogue: the selection output never
 * goes to memory; the kernel writes
 *   out[b,n,h*D+d] = gate[b,h,n,0]*o_cmp[b,h,n/block,d] + gate[b,h,n,1]*o_sel[b,h,n,d]
 * 16-token blocks: with the rounding points of s3r_gated_merge (o_sel, each product and the sum rounded to the I/O
 * dtype), so the result equals s3r_select_attn followed by s3r_gated_merge bit for bit.  64-token blocks: the expression
 * is evaluated in fp32 on the unrounded selection output and rounded ONCE (at most four rounding steps of the I/O dtype,
 * taken on |gate0 o_cmp| + |gate1 o_sel|, away from the two-call result, on the side of the exact value).
 * Replaces topk_blocksparse_attention (pi3/models/sparse_attn/topk_blocksparse_attention.py:1093-1121)
 * together with the merge expression of pi3/models/layers/sparse_attention.py:127-136.
 * Arguments as in s3r_select_attn and s3r_gated_merge; out is contiguous [B,N,H*D].
 * Only for the MFMA paths (bf16/fp16, D == 64, block == 64 or 16, 16-byte aligned tensors); other
 * shapes return S3R_ERR_UNSUPPORTED and the caller runs the two operators one after the other.
 */
int s3r_select_attn_merge(const void* q, const void* k, const void* v, const int32_t* idx,
                          const void* o_cmp, const void* gate, void* out,
                          int B, int H, int64_t N, int D, int block, int K,
                          int64_t sqb, int64_t sqh, int64_t sqn,
                          int64_t skb, int64_t skh, int64_t skn,
                          int64_t svb, int64_t svh, int64_t svn,
                          int64_t sib, int64_t sih, int64_t sim,
                          int64_t scb, int64_t sch, int64_t scm,
                          int64_t sgb, int64_t sgh, int64_t sgn,
                          float softmax_scale, int dtype, void* stream);

/*
 * qk-LayerNorm and 2-D rotary embedding of one [B,H,N,64] tensor (q or k) in one pass:
 *   y = RoPE2D(LayerNorm(x) rounded to the I/O dtype, pos)
 * Replaces self.q_norm / self.k_norm, the cast and self.rope of the reference layer
 * (pi3/models/layers/sparse_attention.py:103-110,120-124) and RoPE2D.forward
 * (pi3/models/layers/pos_embed.py:112-159).
 *   x: strides sxb,sxh,sxn (last stride 1; the packed projection can be passed as a view); y: contiguous.
 *   pos: int32 (y,x) per token, strides spb,spn (pair contiguous), or NULL for no rotation.
 *   cos_tab, sin_tab: I/O dtype [P,16], row p = cos/sin of the angles p * base^(-2i/32), i = 0..15, with the
 *     angles rounded to the I/O dtype first (the reference's table); positions are clamped to [0,P-1].
 *   ln_w, ln_b: I/O dtype [64] LayerNorm weight and bias, ln_w NULL for no normalisation (ln_b optional).
 * Products and sum of the rotation are rounded to the I/O dtype like the reference's eager expression.  The row
 * statistics are fp32; 1/sqrt(var + eps) comes from the hardware's reciprocal square root (1 ulp), so for 16-bit I/O
 * a value may land on the neighbouring representable number of the eager result (as it may from the order of the sums).
 */
int s3r_norm_rope(const void* x, void* y, const int32_t* pos, const void* cos_tab, const void* sin_tab, int P,
                  const void* ln_w, const void* ln_b, float eps,
                  int B, int H, int64_t N, int D,
                  int64_t sxb, int64_t sxh, int64_t sxn, int64_t spb, int64_t spn,
                  int dtype, void* stream);

/*
 * The layer's pre-pass over the packed q/k/v projection in ONE kernel: block means of the raw q, k, v rows (the
 * compressed branch's inputs) and qk-LayerNorm + 2-D rotary embedding of the full-token q and k, each input row read once.
 * Replaces F.avg_pool1d on the raw projection, the three .contiguous() copies, q_norm / k_norm with their casts and
 * the two rope calls on the full tokens (pi3/models/layers/sparse_attention.py:97-99,115-124).  Same bits as
 * s3r_pool_mean on q, k, v followed by s3r_norm_rope on q and k.
 *   q, k, v: [B,H,N,64] views with common strides sxb,sxh,sxn (last stride 1), e.g. the three sections of the packed
 *     [B,N,3*H*64] projection; v is only read (the attention kernels take it in place).
 *   q_out, k_out: contiguous [B,H,N,64];  qc, kc, vc: contiguous [B,H,ceil(N/block),64] (a ragged last block is a mean
 *     over its valid tokens).
 *   pos, cos_tab, sin_tab, P, eps and the LayerNorm parameters (qn_* for q, kn_* for k; both NULL for no norm) as in
 *     s3r_norm_rope.
 */
int s3r_qkv_prepass(const void* q, const void* k, const void* v, void* q_out, void* k_out, void* qc, void* kc, void* vc,
                    const int32_t* pos, const void* cos_tab, const void* sin_tab, int P,
                    const void* qn_w, const void* qn_b, const void* kn_w, const void* kn_b, float eps,
                    int B, int H, int64_t N, int D, int block,
                    int64_t sxb, int64_t sxh, int64_t sxn, int64_t spb, int64_t spn, int dtype, void* stream);

/*
 * LayerNorm over the channels of token rows:  y[r,:] = (x[r,:] - mean_r) * rstd_r * w + b, fp32 statistics, one
 * rounding to the I/O dtype.  Replaces, for inference, the nn.LayerNorm modules in front of the attention layers and
 * the MLPs (norm1 / norm2, pi3/models/layers/block.py:281,296,312,315).
 *   x, y: [rows, C] in the I/O dtype with row strides sx, sy (elements; multiples of 16 bytes); w, b: [C] (b may be
 *   NULL).  C: a multiple of 16 bytes worth of elements, at most 4096 (two-byte types) or 2048 (fp32).
 */
int s3r_layer_norm(const void* x, void* y, const void* w, const void* b, float eps, int64_t rows, int C,
                   int64_t sx, int64_t sy, int dtype, void* stream);

/*
 * Gated merge of the two branches, written in the [B,N,H*D] layout the output projection
 * reads:  out[b,n,h*D+d] = gate[b,h,n,0]*o_cmp[b,h,n/block,d] + gate[b,h,n,1]*o_sel[b,h,n,d].
 * Replaces the einops/broadcast expression in pi3/models/layers/sparse_attention.py:127-136.
 * Each product and the sum are rounded to the I/O dtype, like the eager expression.
 * gate strides sgb,sgh,sgn address the pair (last stride 1); out is contiguous.
 */
int s3r_gated_merge(const void* o_cmp, const void* o_sel, const void* gate, void* out,
                    int B, int H, int64_t N, int D, int block,
                    int64_t scb, int64_t sch, int64_t scm,
                    int64_t ssb, int64_t ssh, int64_t ssn,
                    int64_t sgb, int64_t sgh, int64_t sgn,
                    int dtype, void* stream);

/*
 * Backward of the two attention operators (bf16/fp16, head_dim 64; selection blocks of 64 or 16 tokens, `block`
 * is ignored when idx == NULL).
 * Replaces _topk_blocksparse_attention_bwd (pi3/models/sparse_attn/topk_blocksparse_attention.py:907-1038, kernels
 * backward_sum_o_do :132-170, backward_dkdv :558-712, backward_dq :722-850) and, with idx == NULL (every key tile),
 * _flash_attn_backward (pi3/models/sparse_attn/flash_attention_topk.py:204-630).
 *
 * s3r_attn_bwd_delta:  delta[b,h,n] = sum_d o[b,h,n,d] * dout[b,h,n,d]  (fp32, contiguous [B,H,N]).
 * s3r_attn_bwd: with P = exp(scale * q k^T - lse) over the keys the forward attended to,
 *   dv = P^T dout,  dS = scale * P * (dout v^T - delta),  dq = dS k,  dk = dS^T q;
 *   P and dS are rounded to the I/O dtype before the products, accumulation is fp32 (for dk in bf16 with 64-token
 *   blocks the rounded factor is dS / scale and the scale multiplies the fp32 sum: the same relative rounding).
 *   lse: the forward's optional output (natural log, scaled scores), fp32 [B,H,Lq] contiguous.
 *   idx: the forward's block indices [B,H,ceil(Lq/block),K] (strides sib,sih,sim), or NULL for dense attention.
 *   kq_list, kq_off (needed for dk/dv when idx is given): for every (b,h) the query-block ids that list key block j,
 *     one entry per occurrence, ascending, are kq_list[(b*H+h)*list_stride + kq_off[(b*H+h)*(nkb+1) + j] ...
 *     kq_off[... + j+1]), nkb = ceil(Lk/block); entries of idx that are < 0 or >= nkb appear in no list
 *     (reference count_query_fixedlen / reorder_topk_idx_fixedlen, :423-554).  With block 16 the dk/dv kernel merges
 *     neighbouring lists and relies on every list being ascending, as s3r_key_block_lists leaves it.
 *   dq (layout strides sdq*), dk, dv (sdk*, sdv*): I/O dtype; dq == NULL or dk == dv == NULL skips that kernel.
 *   Every row of dq, dk, dv inside the tensors is written (zeros where nothing attends).
 */
/*
 * Key-centric lists for s3r_attn_bwd from the forward's index tensor.
 * Replaces count_query_fixedlen, the stable argsort and reorder_topk_idx_fixedlen of the reference's backward
 * (pi3/models/sparse_attn/topk_blocksparse_attention.py:423-554).
 *   idx: [B,H,nqb,K] int32 (strides sib,sih,sim, last dimension contiguous); nkb: number of key blocks.
 *   kq_off: [B,H,nkb+1] int32, contiguous; kq_list: [B,H,list_stride] int32, list_stride >= nqb*K.
 * Block j's list of (b,h) = kq_list[(b*H+h)*list_stride + kq_off[..j] ... kq_off[..j+1]): the query-block ids whose
 * index row names j, one entry per occurrence, ascending.  Entries of idx < 0 or >= nkb appear in no list; the part
 * of kq_list behind kq_off[..nkb] is left as it was.  No workspace; the result does not depend on the run.
 */
int s3r_key_block_lists(const int32_t* idx, int32_t* kq_list, int32_t* kq_off, int B, int H, int64_t nqb, int K, int64_t nkb,
                        int64_t sib, int64_t sih, int64_t sim, int64_t list_stride, void* stream);
int s3r_attn_bwd_delta(const void* o, const void* dout, float* delta, int B, int H, int64_t N, int D,
                       int64_t sob, int64_t soh, int64_t son, int64_t sdb, int64_t sdh, int64_t sdn,
                       int dtype, void* stream);
int s3r_attn_bwd(const void* q, const void* k, const void* v, const void* dout, const float* lse, const float* delta,
                 const int32_t* idx, const int32_t* kq_list, const int32_t* kq_off, int64_t list_stride,
                 void* dq, void* dk, void* dv,
                 int B, int H, int64_t Lq, int64_t Lk, int D, int block, int K,
                 int64_t sqb, int64_t sqh, int64_t sqm, int64_t skb, int64_t skh, int64_t skn,
                 int64_t svb, int64_t svh, int64_t svn, int64_t sgb, int64_t sgh, int64_t sgm,
                 int64_t sdqb, int64_t sdqh, int64_t sdqm, int64_t sdkb, int64_t sdkh, int64_t sdkn,
                 int64_t sdvb, int64_t sdvh, int64_t sdvn, int64_t sib, int64_t sih, int64_t sim,
                 float softmax_scale, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SPEED3R_HIP_H */
