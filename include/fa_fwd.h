/*
 * fa_fwd.h — C ABI of the MI355X (gfx950) flash-attention forward launcher.
 *
 * This is the boundary a host framework binds to.  It replaces, for the forward path only,
 * the vendor calls that torch_mlu's launcher `mha_varlen_fwd` makes
 * (/root/reference path: torch_mlu/csrc/aten/operators/cnnl/internal/FlashAttention_internal.cpp:57-267):
 *
 *   cnnlCreate/SetFlashAttentionDescriptor + CnnlTensorDescriptor::set x8 (:131-180)  -> fa_fwd_params (one POD struct)
 *   cnnlGetFlashAttentionForwardWorkspaceSize_v2 (:215-228)                         -> fa_fwd_workspace_bytes
 *   cnnlFlashAttentionForward_v2 (:231-258)                                         -> fa_fwd_launch
 *   cnnlGetFlashAttentionGeneratedRandomNumbers (:181-197)                          -> not needed: one (seed, offset) pair per call
 *
 * Plain C: pointers, sizes and strides only.  No torch types, no exceptions, no allocation, no
 * host/device synchronisation, no global mutable state: the library may be dlopen()ed from any
 * language and called from any host thread.  All work is enqueued on the caller's HIP stream.
 */
#ifndef FA_FWD_H_
#define FA_FWD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FA_FWD_ABI_VERSION 9

/* The library is built with hidden visibility; the entry points declared here and in fa_bwd.h are its whole export
   list. */
#ifndef FA_API
#define FA_API __attribute__((visibility("default")))
#endif

/* element types accepted for q/k/v/out (FlashAttention_internal.cpp:73-80 allows exactly these two) */
#define FA_DTYPE_FP16 0
#define FA_DTYPE_BF16 1

/* return codes */
#define FA_OK 0
#define FA_ERR_BAD_ARG (-1)     /* null pointer, non-positive size, misaligned pointer/stride, short workspace */
#define FA_ERR_UNSUPPORTED (-2) /* shape or dtype outside the supported envelope */
#define FA_ERR_LAUNCH (-3)      /* the HIP runtime refused the launch (hipGetLastError != hipSuccess) */
#define FA_ERR_WORKSPACE (-4)   /* fa_fwd_launch_static only: the plan needs more than FA_STATIC_WORKSPACE_BYTES */

/* is_causal values */
#define FA_MASK_NONE 0
#define FA_MASK_CAUSAL_BOTTOM_RIGHT 1 /* col <= row + Lk - Lq: the flash entry points (reference oracle, construct_local_mask) */
#define FA_MASK_CAUSAL_TOP_LEFT 2     /* col <= row: the mem-efficient entry points (CustomMaskType::CausalFromTopLeft,
                                         attention.cpp:368-370) */

/* kernel selection */
#define FA_KERNEL_AUTO 0     /* split-KV kernel when seqlen_q * (heads_q/heads_k) <= 16 (decode, a few speculative
                                tokens; packed mode: seqlen_q is the longest sequence), else the tile kernel */
#define FA_KERNEL_TILE 1     /* MFMA tile (prefill) kernel: 128 query rows per workgroup, two workgroups per CU */
#define FA_KERNEL_SPLITKV 2  /* HBM-bound split-KV kernel (+ merge): query rows x group heads share one pass over K/V */

/*
 * One attention-forward problem:  for every sequence b and query head h
 *     S   = scale * Q[b,h] K[b,h/(heads_q/heads_k)]^T      (fp32 accumulate)
 *     S  += bias[b,h]                                      (optional additive bias, mem-efficient entry points)
 *     S   = -inf where is_causal and col > row + Lk_b - Lq_b (bottom-right aligned; FA_MASK_CAUSAL_TOP_LEFT: col > row)
 *     LSE = ln sum_j exp(S[:,j]),   out = softmax_row(S) V      (dropout_p > 0: out = (softmax_row(S) o M) V / keep
 *                                                          with a keep-mask M of keep probability `keep`, see
 *                                                          dropout_p; LSE is that of the undropped S)
 * which is what cnnlFlashAttentionForward_v2 is asked to compute (FlashAttention_internal.cpp:147-161,231-258; with
 * the bias descriptor of the mem-efficient launcher, :585-590,659-686).
 *
 * Addressing (all strides are in ELEMENTS, row (b,s,h) of X starts at X + b*x_stride_b + s*x_stride_s + h*x_stride_h,
 * the head_dim elements of a row are contiguous — the "contiguous last dimension" the reference demands at :101-108):
 *   dense  (cu_seqlens_q == NULL): every sequence has seqlen_q / seqlen_k rows.
 *   packed (cu_seqlens_q != NULL): sequence b owns rows [cu[b], cu[b+1]) of the packed [total, heads, head_dim]
 *          tensors; *_stride_b is ignored; seqlen_q / seqlen_k are upper bounds (max_seqlen) used to size the grid.
 *          cu_seqlens are int32 device arrays of batch+1 non-decreasing entries starting at 0 (:81-84,125-127) and
 *          are only ever read on the device.  A sequence longer than seqlen_q / seqlen_k says is not an error the
 *          launcher can see: its rows beyond seqlen_q are left unwritten (never written elsewhere).
 * The sequence strides (x_stride_s) of K and V must stay below 32 MiB in bytes: the kernels address the rows of a tile
 * with a 32-bit offset (FA_ERR_UNSUPPORTED otherwise).
 * LSE element (b,h,s) is written at lse + b*lse_stride_b + h*lse_stride_h + s*lse_stride_s; in packed mode s is the
 * packed row index and lse_stride_b is ignored (the reference's kernel-side buffer is [heads_q, total_q], :129).
 * Rows with no visible key (is_causal and Lk < Lq, Lk == 0, or a bias row that is -inf throughout) get out = 0 and
 * LSE = +inf.
 * bias (optional, same dtype as q): element (b,h,row,col) at bias + b*bias_stride_b + h*bias_stride_h
 * + row*bias_stride_q + col (packed mode: b = the sequence, row and col counted from its first row / key); columns
 * contiguous; stride 0 broadcasts over batch or heads (or rows); the base pointer and all three strides must keep
 * 4-element groups 8-byte aligned (multiples of 4 elements).  A problem with a bias always runs the tile kernel; when
 * the base pointer and the strides are multiples of 8 elements and seqlen_k is a multiple of 8 (dense mode), the kernel
 * prefetches bias tiles through LDS, which is faster and gives the same bits.
 */
typedef struct fa_fwd_params {
  const void* q;   /* device, 16-byte aligned */
  const void* k;
  const void* v;
  void* out;
  float* lse;
  const int32_t* cu_seqlens_q; /* device int32[batch+1] or NULL */
  const int32_t* cu_seqlens_k; /* device int32[batch+1] or NULL (both or neither) */

  int64_t q_stride_b, q_stride_s, q_stride_h;
  int64_t k_stride_b, k_stride_s, k_stride_h;
  int64_t v_stride_b, v_stride_s, v_stride_h;
  int64_t o_stride_b, o_stride_s, o_stride_h;
  int64_t lse_stride_b, lse_stride_h, lse_stride_s;

  int32_t batch;     /* > 0 */
  int32_t heads_q;   /* > 0, multiple of heads_k (:122-124) */
  int32_t heads_k;   /* > 0 */
  int32_t seqlen_q;  /* dense: rows per sequence; packed: max over sequences */
  int32_t seqlen_k;
  int32_t head_dim;  /* multiple of 8, 8..256 (:119-121) */

  float scale;       /* softmax scale, already resolved (attention.cpp:174-175 passes it as float) */
  int32_t dtype;     /* FA_DTYPE_* */
  int32_t is_causal; /* FA_MASK_* (0 / 1 keep their old meaning) */
  int32_t kernel;    /* FA_KERNEL_* */
  int32_t num_splits; /* slices of the key range: 0 = choose, else 1..FA_MAX_SPLITS (split-KV kernel; tile kernel, where
                         each query block's tiles are cut into slices) */
  int32_t reserved;  /* must be 0 */

  const void* bias;  /* device or NULL */
  int64_t bias_stride_b, bias_stride_h, bias_stride_q;

  /* dropout on the softmax probabilities (0 = off; both forward kernels).  The mask is a pure function of
     (philox_seed, philox_offset, sequence, query head, row, col), so the backward regenerates it from the two numbers
     and the tile and split-KV kernels drop the same elements. */
  float dropout_p;         /* 0 <= p < 1.  An element is kept iff one byte of a hash word is <= floor((1 - p) 255), i.e.
                              with probability keep = (floor((1 - p) 255) + 1) / 256 (1 - p rounded to a multiple of
                              1 / 256), and kept elements are scaled by 1 / keep — the reference's oracle scales by
                              1 / (1 - p) with a mask that keeps with probability 1 - p — so that the expectation of
                              the output over masks is the undropped output; the backward uses the same factor */
  int32_t reserved2;       /* must be 0 */
  uint64_t philox_seed;
  uint64_t philox_offset;
  int64_t* rng_seed_out;   /* device int64 or NULL: the launch stores philox_seed there (the op's philox_seed slot) */
  int64_t* rng_offset_out; /* device int64 or NULL */
  void* dropout_mask;      /* device or NULL: debug output, dense [batch][heads_q][seqlen_q][seqlen_k] elements of
                              `dtype`, +1 kept / -1 dropped, positions outside a sequence or masked left untouched
                              (packed mode: seqlen_q / seqlen_k are the maxima, rows and keys count from each
                              sequence's start, as FlashAttention_internal.cpp:141-146 shapes it).  Written by the
                              tile kernel only: a call that wants it is planned onto the tile kernel, and with
                              kernel = FA_KERNEL_SPLITKV or a page table it is FA_ERR_UNSUPPORTED */
  /* optional (NULL = all of them): device int32[batch]; only the first min(seqused_k[b], its length) keys of sequence b
     exist — a KV cache that is allocated to seqlen_k rows but filled to a per-sequence length (the `seqused_k` of
     aten::_flash_attention_forward, the `seqlen_k` of aten::_efficient_attention_forward).  The causal mask aligns to
     the used length.  Forward only: the backward has no such argument. */
  const int32_t* seqused_k;
  /* optional (NULL = philox_seed / philox_offset above are the numbers): device int64 each.  When given, the kernel
     reads the seed from *philox_seed_ptr and adds *philox_offset_ptr to philox_offset when it RUNS, so a launch
     recorded into a HIP graph draws a new mask on every replay from a generator state the host advances between
     replays (the capture-aware generator of the reference, framework/generator/generator_impl.cpp:264-292).
     rng_seed_out / rng_offset_out receive the resolved numbers. */
  const int64_t* philox_seed_ptr;
  const int64_t* philox_offset_ptr;
  /* optional paged KV cache (NULL = k / v are per-sequence tensors as above).  Dense mode, no bias, no dropout_mask,
     not top-left causal (anything else: FA_ERR_UNSUPPORTED).  Decode-shaped calls (seqlen_q x heads_q / heads_k <= 16)
     run on the split-KV kernel; longer query chunks (a chunk of a chunked prefill against the cache) on the tile
     kernel, which takes no dropout with a page table.
     k and v then point at pools of pages, [page][row in page][kv head][head_dim]: k_stride_b / v_stride_b are the
     element strides between pages, k_stride_s / v_stride_s between the rows of a page.  Key row r of sequence b lives
     in page block_table[b * block_table_stride + r / page_size] at row r % page_size.  seqlen_k is the longest
     sequence's key count (block_table_stride * page_size at most); seqused_k gives each sequence's own.  page_size
     must be a multiple of 32.  (No counterpart in the reference, whose ops take whole tensors; this is the block
     table of serving engines.) */
  const int32_t* block_table; /* device int32 [batch][block_table_stride] */
  int64_t block_table_stride;
  int32_t page_size;
  int32_t reserved3;          /* must be 0 */
} fa_fwd_params;

#define FA_MAX_SPLITS 64

/* ABI version of the loaded library (== FA_FWD_ABI_VERSION it was built with). */
FA_API int fa_fwd_version(void);

/* Static text for a return code. */
FA_API const char* fa_fwd_error_string(int rc);

/*
 * Validate `p` without touching the GPU.  Returns FA_OK or a negative code; the same checks run inside
 * fa_fwd_workspace_bytes / fa_fwd_launch.  Host-only, so callable on a machine with no device.
 */
FA_API int fa_fwd_validate(const fa_fwd_params* p);

/*
 * Bytes of device scratch fa_fwd_launch needs for `p`: partial (m, l, o) per slice — per (sequence, query head, query row) for both
 * kernels (packed mode: seqlen_q rows per sequence); 0 when nothing is sliced.  Mirrors cnnlGetFlashAttentionForwardWorkspaceSize_v2.  Returns 0 also when `p` is invalid.
 */
FA_API size_t fa_fwd_workspace_bytes(const fa_fwd_params* p);

/*
 * Enqueue the forward pass on `stream` (a hipStream_t passed as void*; NULL = the null stream).
 * `workspace` must hold at least fa_fwd_workspace_bytes(p) bytes (may be NULL when that is 0) and must stay
 * alive until the enqueued work has run; stream-ordered allocators satisfy this.  Never allocates, never
 * synchronises, never throws.  Returns FA_OK or a negative code (nothing is enqueued on error).
 */
FA_API int fa_fwd_launch(const fa_fwd_params* p, void* workspace, size_t workspace_bytes, void* stream);

/*
 * fa_fwd_launch for callers that cannot allocate device memory or pass a workspace (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same kernels and results
 * as fa_fwd_launch; the per-slice partials go to a fixed array of FA_STATIC_WORKSPACE_BYTES bytes of device memory
 * that is part of the library's code object, so each device the library runs on holds that much until the process
 * ends.  Calls no allocating routine.  The first call on a device that needs scratch looks the array's device address
 * up (make that call outside graph capture).  Returns FA_ERR_WORKSPACE, with nothing enqueued, when
 * fa_fwd_workspace_bytes(p) exceeds FA_STATIC_WORKSPACE_BYTES.  All calls on one device share the one array: two
 * launches that both need scratch must not overlap on that device (issue them on one stream, or order the streams
 * with events); calls whose fa_fwd_workspace_bytes(p) is 0 never touch it.  Nothing in the array needs clearing
 * between calls: every slot a launch reads it has written first.
 */
#define FA_STATIC_WORKSPACE_BYTES (64u << 20)
FA_API int fa_fwd_launch_static(const fa_fwd_params* p, void* stream);

/*
 * Which kernel fa_fwd_launch would run for `p` (FA_KERNEL_TILE / FA_KERNEL_SPLITKV) and with how many splits;
 * negative code when `p` is invalid.  Host-only.
 */
FA_API int fa_fwd_plan(const fa_fwd_params* p, int32_t* kernel, int32_t* num_splits);

#ifdef __cplusplus
}
#endif
#endif /* FA_FWD_H_ */
