// Host-only half of the launchers of include/fa_fwd.h and include/fa_bwd.h: argument validation, kernel choice and
// workspace sizes.  Plain C++ without any HIP construct, so that a CPU build with sanitizers can exercise it
// (tests/test_cabi_host.py); fa_fwd_kernels.hip and fa_bwd_kernels.hip include it.  The checks restate those of
// torch_mlu's launchers (torch_mlu/csrc/aten/operators/cnnl/internal/FlashAttention_internal.cpp:73-127 forward,
// :288-366 backward) at the level of raw pointers and strides.
#ifndef FA_HOST_H_
#define FA_HOST_H_

#include <math.h>
#include <stddef.h>
#include <stdint.h>

#include "fa_bwd.h"
#include "fa_fwd.h"

namespace fa {
namespace host {

// ---- forward ------------------------------------------------------------------------------------------------
inline int padded_dim(int d) { return d <= 64 ? 64 : (d <= 128 ? 128 : 256); }
constexpr int64_t kMaxRowStrideBytes = 0xffffffffLL / 128;  // 128 rows x stride must fit an unsigned 32-bit offset
constexpr int32_t kMaxSeqlen = 1 << 29;                      // rows / keys per sequence

inline int validate(const fa_fwd_params* p) {
  if (!p) return FA_ERR_BAD_ARG;
  if (!p->q || !p->k || !p->v || !p->out || !p->lse) return FA_ERR_BAD_ARG;
  if ((p->cu_seqlens_q == nullptr) != (p->cu_seqlens_k == nullptr)) return FA_ERR_BAD_ARG;
  if (p->batch <= 0 || p->heads_q <= 0 || p->heads_k <= 0) return FA_ERR_BAD_ARG;
  if (p->seqlen_q < 0 || p->seqlen_k < 0 || p->head_dim <= 0) return FA_ERR_BAD_ARG;
  if (p->reserved != 0) return FA_ERR_BAD_ARG;
  if (p->dtype != FA_DTYPE_FP16 && p->dtype != FA_DTYPE_BF16) return FA_ERR_UNSUPPORTED;
  if (p->head_dim > 256 || (p->head_dim & 7)) return FA_ERR_UNSUPPORTED;
  if (p->heads_q % p->heads_k) return FA_ERR_UNSUPPORTED;
  // lengths and (sequence, head) counts that keep the kernels' 32-bit row / block arithmetic (row + Lk - Lq, grid
  // sizes) and the 64-bit products below from overflowing
  if (p->seqlen_q > kMaxSeqlen || p->seqlen_k > kMaxSeqlen) return FA_ERR_UNSUPPORTED;
  if ((int64_t)p->batch * p->heads_q > 0x7fffffffLL) return FA_ERR_UNSUPPORTED;
  if (p->kernel < FA_KERNEL_AUTO || p->kernel > FA_KERNEL_SPLITKV) return FA_ERR_BAD_ARG;
  if (p->num_splits < 0 || p->num_splits > FA_MAX_SPLITS) return FA_ERR_BAD_ARG;
  // 16-byte vector access on every row: base pointers and row strides must be multiples of 8 elements
  const uintptr_t al = (uintptr_t)p->q | (uintptr_t)p->k | (uintptr_t)p->v | (uintptr_t)p->out;
  if (al & 15) return FA_ERR_BAD_ARG;
  if ((uintptr_t)p->lse & 3) return FA_ERR_BAD_ARG;
  const int64_t st[] = {p->q_stride_s, p->q_stride_h, p->k_stride_s, p->k_stride_h, p->v_stride_s, p->v_stride_h,
                        p->o_stride_s, p->o_stride_h};
  for (int64_t s : st)
    if (s < 0 || (s & 7)) return FA_ERR_BAD_ARG;
  if (!p->cu_seqlens_q) {
    const int64_t sb[] = {p->q_stride_b, p->k_stride_b, p->v_stride_b, p->o_stride_b};
    for (int64_t s : sb)
      if (s < 0 || (s & 7)) return FA_ERR_BAD_ARG;
    if (p->lse_stride_b < 0) return FA_ERR_BAD_ARG;
  }
  if (p->lse_stride_h < 0 || p->lse_stride_s < 0) return FA_ERR_BAD_ARG;
  // the kernels form per-lane byte offsets inside a tile (up to 128 rows) as 32-bit row x 32-bit stride
  if (p->k_stride_s > kMaxRowStrideBytes / 2 || p->v_stride_s > kMaxRowStrideBytes / 2 ||
      p->q_stride_s > kMaxRowStrideBytes / 2)
    return FA_ERR_UNSUPPORTED;
  if (p->is_causal < FA_MASK_NONE || p->is_causal > FA_MASK_CAUSAL_TOP_LEFT) return FA_ERR_BAD_ARG;
  if (p->reserved2 != 0 || !(p->dropout_p >= 0.f && p->dropout_p < 1.f)) return FA_ERR_BAD_ARG;
  if (p->dropout_p > 0.f) {
    if (p->kernel == FA_KERNEL_SPLITKV && p->dropout_mask) return FA_ERR_UNSUPPORTED;  // only the tile kernel writes the debug mask
    if (p->dropout_mask && ((uintptr_t)p->dropout_mask & 3)) return FA_ERR_BAD_ARG;
    if (((uintptr_t)p->rng_seed_out | (uintptr_t)p->rng_offset_out) & 7) return FA_ERR_BAD_ARG;
    if (((uintptr_t)p->philox_seed_ptr | (uintptr_t)p->philox_offset_ptr) & 7) return FA_ERR_BAD_ARG;
    if (!p->philox_seed_ptr != !p->philox_offset_ptr) return FA_ERR_BAD_ARG;  // both or neither
  }
  if ((uintptr_t)p->seqused_k & 3) return FA_ERR_BAD_ARG;
  if (p->reserved3 != 0) return FA_ERR_BAD_ARG;
  if (p->block_table) {
    // paged K/V: dense mode, pages of whole 32-row blocks, a table wide enough.  Decode-shaped calls (what the
    // split-KV kernel takes) may use dropout; a prefill chunk (the tile kernel) may not.
    if ((uintptr_t)p->block_table & 3) return FA_ERR_BAD_ARG;
    if (p->page_size <= 0 || p->block_table_stride < 0) return FA_ERR_BAD_ARG;
    if (p->page_size % 32) return FA_ERR_UNSUPPORTED;
    if (p->block_table_stride < ((int64_t)p->seqlen_k + p->page_size - 1) / p->page_size) return FA_ERR_BAD_ARG;
    if (p->cu_seqlens_q || p->bias || (p->dropout_p > 0.f && p->dropout_mask) || p->is_causal == FA_MASK_CAUSAL_TOP_LEFT)
      return FA_ERR_UNSUPPORTED;
    if (p->seqlen_q < 1) return FA_ERR_UNSUPPORTED;
    const bool decode_shaped = (int64_t)p->seqlen_q * (p->heads_q / p->heads_k) <= 16;
    if (p->kernel == FA_KERNEL_SPLITKV && !decode_shaped) return FA_ERR_UNSUPPORTED;
    if ((p->kernel == FA_KERNEL_TILE || !decode_shaped) && p->dropout_p > 0.f) return FA_ERR_UNSUPPORTED;
    // the pools' pages are addressed as 64-bit page x stride; rows inside a page as 32-bit row x stride
    if (p->k_stride_b < 0 || p->v_stride_b < 0) return FA_ERR_BAD_ARG;
  }
  if (p->bias) {
    if (((uintptr_t)p->bias & 7) || p->bias_stride_b < 0 || p->bias_stride_h < 0 || p->bias_stride_q < 0 ||
        ((p->bias_stride_b | p->bias_stride_h | p->bias_stride_q) & 3))
      return FA_ERR_BAD_ARG;
    if (p->kernel == FA_KERNEL_SPLITKV) return FA_ERR_UNSUPPORTED;
  }
  if (p->kernel == FA_KERNEL_SPLITKV) {
    // the query rows x the heads of a GQA group are the 16 columns of its MFMA; packed mode: one row per sequence
    if (p->seqlen_q < 1 || (int64_t)p->seqlen_q * (p->heads_q / p->heads_k) > 16) return FA_ERR_UNSUPPORTED;
    if (p->is_causal == FA_MASK_CAUSAL_TOP_LEFT) return FA_ERR_UNSUPPORTED;  // the single query row would see key 0 only
  }
  return FA_OK;
}

inline void plan(const fa_fwd_params* p, int* kernel, int* splits) {
  int kern = p->kernel;
  const int group = p->heads_q / p->heads_k;
  // a page table: decode-shaped calls go to the split-KV kernel, a prefill chunk to the tile kernel's paged variant
  if (p->block_table && kern == FA_KERNEL_AUTO)
    kern = ((int64_t)p->seqlen_q * group <= 16) ? FA_KERNEL_SPLITKV : FA_KERNEL_TILE;
  if (kern == FA_KERNEL_AUTO)
    kern = (p->seqlen_q >= 1 && (int64_t)p->seqlen_q * group <= 16 && p->seqlen_k >= 256 && !p->bias && p->is_causal != FA_MASK_CAUSAL_TOP_LEFT && !(p->dropout_p > 0.f && p->dropout_mask))
               ? FA_KERNEL_SPLITKV
               : FA_KERNEL_TILE;
  int ns = 1;
  if (kern == FA_KERNEL_SPLITKV) {
    ns = p->num_splits;
    if (ns == 0) {
      // A workgroup costs 10-20 us to start and to merge, whatever the length of its slice, so slices are as long as
      // they can be: split only until every CU has one workgroup (256 CUs), give slices of 2048 rows and more
      // precedence over the last doubling while 128 workgroups remain, and never cut below 512 rows.  Measured on
      // B x 8 kv heads x {2k ... 128k} rows: within 8 % of the best power of two everywhere (the former rule, 2048
      // workgroups of at least 512 rows, was up to 1.7 x slower at batch 4-16).
      constexpr int64_t kCUs = 256;
      const int64_t units = (int64_t)p->batch * p->heads_k;
      ns = 1;
      while (ns * 2 <= FA_MAX_SPLITS && units * ns * 2 <= kCUs) ns *= 2;
      while (ns > 1 && p->seqlen_k / ns < 2048 && units * (ns / 2) >= kCUs / 2) ns /= 2;
      while (ns > 1 && p->seqlen_k / ns < 512) ns /= 2;
    }
    const int nblk = (p->seqlen_k + 31) / 32;
    if (ns > nblk) ns = nblk > 0 ? nblk : 1;
  } else if (p->seqlen_q > 0) {
    // Tile kernel (dense or packed; an additive bias, either causal alignment and dropout — whose mask is a function
    // of the row and the key, not of the slice — are fine): with few query blocks against a long K/V (chunked prefill, speculative decoding, a
    // GQA group too wide for the split-KV kernel) the key range of each block is cut into slices so that the CUs
    // have two workgroups each; a slice keeps at least 32 tiles (2048 keys), or 16 where the chunk is much shorter
    // than the cache, so that a causal mask leaves every slice equally full.  Partials go through the workspace.
    const int64_t wgs = (int64_t)p->batch * p->heads_q * ((p->seqlen_q + 127) / 128);
    const int ntiles = (p->seqlen_k + 63) / 64;
    const int min_tiles = ((int64_t)p->seqlen_q * 4 <= p->seqlen_k) ? 16 : 32;
    ns = p->num_splits;
    if (ns == 0) {
      ns = 1;
      while (ns * 2 <= FA_MAX_SPLITS && wgs * ns * 2 <= 512 && ntiles / (ns * 2) >= min_tiles) ns *= 2;
    }
    if (ns > ntiles) ns = ntiles > 0 ? ntiles : 1;
    // keep the partials (fp32, one slot per query row and slice) within 1 GiB
    const int64_t rows = (int64_t)p->batch * p->heads_q * p->seqlen_q;  // <= 2^60
    while (ns > 1 && rows > (1LL << 30) / ((int64_t)ns * (p->head_dim * 4 + 8))) ns /= 2;
  }
  *kernel = kern;
  *splits = ns;
}

// partial slots: one per (sequence, query head, query row, slice) for both kernels (packed mode: seqlen_q rows per
// sequence, the longest one's)
inline size_t partial_slots(const fa_fwd_params* p, int kern, int ns) {
  (void)kern;
  return (size_t)p->batch * p->heads_q * ns * (size_t)p->seqlen_q;
}

inline size_t workspace_bytes(const fa_fwd_params* p, int kern, int ns) {
  if (ns <= 1) return 0;
  const size_t slots = partial_slots(p, kern, ns);
  return slots * (size_t)p->head_dim * 4 + slots * 8;
}

// ---- backward -----------------------------------------------------------------------------------------------

inline int bwd_validate(const fa_bwd_params* p) {
  if (!p) return FA_ERR_BAD_ARG;
  if (!p->q || !p->k || !p->v || !p->out || !p->dout || !p->lse || !p->dq || !p->dk || !p->dv) return FA_ERR_BAD_ARG;
  if ((p->cu_seqlens_q == nullptr) != (p->cu_seqlens_k == nullptr)) return FA_ERR_BAD_ARG;
  if (p->batch <= 0 || p->heads_q <= 0 || p->heads_k <= 0) return FA_ERR_BAD_ARG;
  if (p->seqlen_q < 0 || p->seqlen_k < 0 || p->head_dim <= 0) return FA_ERR_BAD_ARG;
  if (p->reserved != 0 || p->reserved2 != 0) return FA_ERR_BAD_ARG;
  if (!(p->dropout_p >= 0.f && p->dropout_p < 1.f)) return FA_ERR_BAD_ARG;
  if (p->dropout_p > 0.f && (!p->philox_seed || !p->philox_offset ||
                             (((uintptr_t)p->philox_seed | (uintptr_t)p->philox_offset) & 7)))
    return FA_ERR_BAD_ARG;
  if (p->cu_seqlens_q && p->total_q < 0) return FA_ERR_BAD_ARG;
  if (p->is_causal != FA_MASK_NONE && p->is_causal != FA_MASK_CAUSAL_BOTTOM_RIGHT && p->is_causal != FA_MASK_CAUSAL_TOP_LEFT)
    return FA_ERR_BAD_ARG;
  if (p->dbias && !p->bias) return FA_ERR_BAD_ARG;
  if (p->bias) {
    if (((uintptr_t)p->bias & 7) || p->bias_stride_b < 0 || p->bias_stride_h < 0 || p->bias_stride_q < 0 ||
        ((p->bias_stride_b | p->bias_stride_h | p->bias_stride_q) & 3))
      return FA_ERR_BAD_ARG;
  }
  if (p->dbias) {  // an output: aligned like the bias and not broadcast
    if (((uintptr_t)p->dbias & 7) || ((p->dbias_stride_b | p->dbias_stride_h | p->dbias_stride_q) & 3)) return FA_ERR_BAD_ARG;
    if (p->dbias_stride_q < p->seqlen_k || (p->seqlen_q > 1 && p->dbias_stride_q <= 0) ||
        (p->heads_q > 1 && p->dbias_stride_h <= 0) || (p->batch > 1 && p->dbias_stride_b <= 0))
      return FA_ERR_BAD_ARG;
  }
  if (p->dtype != FA_DTYPE_FP16 && p->dtype != FA_DTYPE_BF16) return FA_ERR_UNSUPPORTED;
  if (p->head_dim > 256 || (p->head_dim & 7)) return FA_ERR_UNSUPPORTED;
  if (p->heads_q % p->heads_k) return FA_ERR_UNSUPPORTED;
  if (p->seqlen_q > kMaxSeqlen || p->seqlen_k > kMaxSeqlen) return FA_ERR_UNSUPPORTED;
  if ((int64_t)p->batch * p->heads_q > 0x7fffffffLL) return FA_ERR_UNSUPPORTED;
  const uintptr_t al = (uintptr_t)p->q | (uintptr_t)p->k | (uintptr_t)p->v | (uintptr_t)p->out | (uintptr_t)p->dout |
                       (uintptr_t)p->dq | (uintptr_t)p->dk | (uintptr_t)p->dv;
  if (al & 15) return FA_ERR_BAD_ARG;
  if ((uintptr_t)p->lse & 3) return FA_ERR_BAD_ARG;
  const int64_t st[] = {p->q_stride_s,  p->q_stride_h,  p->k_stride_s,  p->k_stride_h,  p->v_stride_s,  p->v_stride_h,
                        p->o_stride_s,  p->o_stride_h,  p->do_stride_s, p->do_stride_h, p->dq_stride_s, p->dq_stride_h,
                        p->dk_stride_s, p->dk_stride_h, p->dv_stride_s, p->dv_stride_h};
  for (int64_t s : st)
    if (s < 0 || (s & 7)) return FA_ERR_BAD_ARG;
  if (!p->cu_seqlens_q) {
    const int64_t sb[] = {p->q_stride_b,  p->k_stride_b,  p->v_stride_b,  p->o_stride_b,
                          p->do_stride_b, p->dq_stride_b, p->dk_stride_b, p->dv_stride_b};
    for (int64_t s : sb)
      if (s < 0 || (s & 7)) return FA_ERR_BAD_ARG;
  }
  if (p->lse_stride_h < 0 || p->lse_stride_s < 0) return FA_ERR_BAD_ARG;
  // per-lane byte offsets inside a tile (up to 128 rows) are 32-bit row x 32-bit stride
  if (p->k_stride_s > kMaxRowStrideBytes / 2 || p->v_stride_s > kMaxRowStrideBytes / 2 ||
      p->q_stride_s > kMaxRowStrideBytes / 2 || p->do_stride_s > kMaxRowStrideBytes / 2)
    return FA_ERR_UNSUPPORTED;
  return FA_OK;
}

// two fp32 planes per (row, head): -delta and LSE log2(e)
inline size_t bwd_ws_plane(const fa_bwd_params* p) {
  const size_t rows = p->cu_seqlens_q ? (size_t)p->total_q : (size_t)p->batch * p->seqlen_q;
  return (rows * p->heads_q * 4 + 15) & ~(size_t)15;
}
inline size_t bwd_ws_bytes(const fa_bwd_params* p) { return 2 * bwd_ws_plane(p); }

}  // namespace host
}  // namespace fa

#endif  // FA_HOST_H_
