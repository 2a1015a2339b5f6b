/*
 * fa_bwd.h — C ABI of the MI355X (gfx950) flash-attention backward launcher (same library as fa_fwd.h).
 *
 * Replaces the vendor calls torch_mlu's backward launcher `mha_varlen_bwd` makes
 * (torch_mlu/csrc/aten/operators/cnnl/internal/FlashAttention_internal.cpp:269-483):
 *
 *   cnnlSetFlashAttentionBackwardDescriptor + tensor descriptors (:368-447)  -> fa_bwd_params
 *   cnnlGetFlashAttentionBackwardWorkspaceSize (:430-447)                    -> fa_bwd_workspace_bytes
 *   cnnlFlashAttentionBackward (:449-480)                                    -> fa_bwd_launch
 *
 * Given the forward's inputs, its output and its logsumexp, and the gradient of the output, computes
 *     P   = exp(scale * Q K^T + mask - LSE)                (recomputed, never stored)
 *     dV  = P^T dO
 *     dP  = dO V^T,   delta = rowsum(dO o O),   dS = P o (dP - delta)
 *     dQ  = scale * dS K,   dK = scale * dS^T Q
 * (with dropout: dV = (P o M)^T dO / keep and dP = M o (dO V^T) / keep, M regenerated from the forward's seed/offset,
 * keep = the mask's keep probability as defined at fa_fwd_params.dropout_p)
 * with the forward's masking (the FA_MASK_* modes of fa_fwd.h) and head grouping (dK, dV of a kv head sum over the
 * query heads that read it).  Same rules as fa_fwd.h: plain C, device pointers, element strides, no allocation,
 * no synchronisation, work is only enqueued on the caller's stream.
 *
 * The same launcher serves the mem-efficient backward `mem_eff_bwd` (FlashAttention_internal.cpp:692-906, vendor call
 * cnnlFlashAttentionBackward_v2 at :861-903): an additive bias enters the recomputed scores (scale * Q K^T + bias),
 * the causal mask may be aligned to the top-left corner (custom_mask_type 1, :776-779,803-807), and the gradient of
 * the bias, dBias = dS, can be written out.  (The reference allocates that gradient but never hands it to the vendor
 * call, :836,861-903 — it comes back uninitialised there; here it is computed.)
 */
#ifndef FA_BWD_H_
#define FA_BWD_H_

#include <stddef.h>
#include <stdint.h>

#include "fa_fwd.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Addressing as in fa_fwd_params: row (b,s,h) of X at X + b*x_stride_b + s*x_stride_s + h*x_stride_h (elements),
 * head_dim elements contiguous; packed mode (cu_seqlens_q != NULL) ignores *_stride_b and addresses rows by their
 * packed index.  q, dq, out, dout have heads_q heads; k, v, dk, dv have heads_k heads.  lse is the forward's
 * logsumexp (natural log), read through the same three strides the forward wrote it with.
 * The sequence strides of q, k, v and dout must stay below 32 MiB in bytes (a tile's rows are addressed with a
 * 32-bit offset; FA_ERR_UNSUPPORTED otherwise).
 */
typedef struct fa_bwd_params {
  const void* q;
  const void* k;
  const void* v;
  const void* out;
  const void* dout;
  const float* lse;
  void* dq;
  void* dk;
  void* dv;
  const int32_t* cu_seqlens_q; /* device int32[batch+1] or NULL */
  const int32_t* cu_seqlens_k;

  int64_t q_stride_b, q_stride_s, q_stride_h;
  int64_t k_stride_b, k_stride_s, k_stride_h;
  int64_t v_stride_b, v_stride_s, v_stride_h;
  int64_t o_stride_b, o_stride_s, o_stride_h;
  int64_t do_stride_b, do_stride_s, do_stride_h;
  int64_t dq_stride_b, dq_stride_s, dq_stride_h;
  int64_t dk_stride_b, dk_stride_s, dk_stride_h;
  int64_t dv_stride_b, dv_stride_s, dv_stride_h;
  int64_t lse_stride_b, lse_stride_h, lse_stride_s;

  int32_t batch;
  int32_t heads_q;
  int32_t heads_k;
  int32_t seqlen_q;  /* dense: rows per sequence; packed: max over sequences */
  int32_t seqlen_k;
  int32_t head_dim;  /* multiple of 8, 8..256 (FlashAttention_internal.cpp:355-357) */
  int64_t total_q;   /* packed: rows of q (sizes the delta scratch); dense: ignored */

  float scale;
  int32_t dtype;     /* FA_DTYPE_* */
  int32_t is_causal; /* FA_MASK_NONE / FA_MASK_CAUSAL_BOTTOM_RIGHT (= 1) / FA_MASK_CAUSAL_TOP_LEFT, as the forward */
  int32_t reserved;  /* must be 0 */

  /* dropout: same p as the forward and the two numbers it stored (device pointers, read by the kernels, so that no
     host synchronisation is needed); ignored when dropout_p == 0 */
  float dropout_p;
  int32_t reserved2; /* must be 0 */
  const int64_t* philox_seed;
  const int64_t* philox_offset;

  /* optional additive bias of the forward (same dtype as q; NULL = none):
     element (b, h, row, col) at bias + b*bias_stride_b + h*bias_stride_h + row*bias_stride_q + col, h a query head;
     in packed mode b is the sequence and row, col count from the sequence's first row / key.
     Strides may be 0 (broadcast) and must be multiples of 4; the pointer must be 8-byte aligned (as in the forward).
     Values: finite numbers and -inf (a masked position; a row that is -inf throughout gets zero gradients).  +inf and
     NaN entries are outside the contract of this backward: the dK / dV kernels bring the bias into the score layout
     through a matrix product with the identity, where an infinity or NaN spreads over its query row of the 32 x 32
     block, so the gradients of that row are then undefined (other rows are unaffected).  The reference hands any
     bias to the vendor call unchecked (FlashAttention_internal.cpp:836-903) and defines nothing for them either. */
  const void* bias;
  int64_t bias_stride_b, bias_stride_h, bias_stride_q;
  /* optional output (needs bias): the gradient of the bias, [batch, heads_q, seqlen_q, seqlen_k] in q's dtype,
     addressed like bias but never broadcast (every element of it is written, masked positions with 0) */
  void* dbias;
  int64_t dbias_stride_b, dbias_stride_h, dbias_stride_q;
} fa_bwd_params;

/* Host-only validation: FA_OK or a negative code (FA_ERR_UNSUPPORTED for head_dim > 256). */
FA_API int fa_bwd_validate(const fa_bwd_params* p);

/* Bytes of device scratch fa_bwd_launch needs (-rowsum(dO o O) and LSE log2(e), two fp32 per query row and head);
   0 if invalid. */
FA_API size_t fa_bwd_workspace_bytes(const fa_bwd_params* p);

/* Enqueue the backward pass on `stream`; `workspace` must hold fa_bwd_workspace_bytes(p) bytes, 16-byte aligned. */
FA_API int fa_bwd_launch(const fa_bwd_params* p, void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FA_BWD_H_ */
