// Kernel-argument block and LDS layout helpers shared by the forward kernels' translation units (gfx950 only).
#ifndef FA_FWD_COMMON_H_
#define FA_FWD_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fa_device.h"

namespace fa {

// Kernel arguments: fa_fwd_params plus what the host derives once.
struct KArgs {
  const unsigned char* q;
  const unsigned char* k;
  const unsigned char* v;
  unsigned char* out;
  float* lse;
  const int32_t* cu_q;
  const int32_t* cu_k;
  int64_t q_sb, q_ss, q_sh;  // byte strides
  int64_t k_sb, k_ss, k_sh;
  int64_t v_sb, v_ss, v_sh;
  int64_t o_sb, o_ss, o_sh;
  int64_t lse_sb, lse_sh, lse_ss;  // element strides
  int32_t batch, heads_q, heads_k, group;
  int32_t seqlen_q, seqlen_k, head_dim;
  int32_t n_mblk;     // tile kernels: workgroups per (sequence, head)
  int32_t pair;       // tile kernel: a workgroup owns query blocks p and n-1-p of its sequence
  int32_t hgroup;     // tile kernel with a bias that is shared by all heads: heads whose workgroups are interleaved
  int32_t n_splits;   // split-KV kernel; tile kernel: slices of the key range per query block (1 = none)
  int32_t is_causal;
  int32_t neg_scale;  // scale < 0: Q is negated on load and |scale| is used, so that max() tracks the true row max
  float scale_log2;   // |scale| * log2(e)
  float scale_abs;    // |scale| (bias path)
  int32_t causal_tl;  // causal mask aligned to the top-left corner (col <= row) instead of the bottom-right one
  const int32_t* seqused_k;   // optional: keys of sequence b beyond seqused_k[b] do not exist
  const int32_t* block_table; // optional (split-KV kernel): paged K/V, page of key row r = table[b * bt_stride + r / page_size]
  int64_t bt_stride;
  int32_t page_size;
  const unsigned char* bias;  // optional additive bias, dense mode: [b][h][row][col] through byte strides
  int64_t bias_sb, bias_sh, bias_sq;
  uint32_t drop_thr;  // dropout: an element is kept iff its byte <= drop_thr
  float drop_rp;      // 256 / (drop_thr + 1): one over the realised keep probability
  uint64_t seed, offset;
  const int64_t* seed_ptr;    // optional: the seed is *seed_ptr and *offset_ptr is added to offset (graph capture)
  const int64_t* offset_ptr;
  int64_t* rng_seed_out;
  int64_t* rng_offset_out;
  unsigned char* dmask;  // debug mask [batch][heads_q][seqlen_q][seqlen_k] elements, or null
  float* ws_o;        // split-KV partials: [batch*heads_q*n_splits][head_dim] fp32, unnormalised
  float* ws_ml;       // [batch*heads_q*n_splits][2]: m (log2 domain), l
                      // (sliced tile kernel: the same per query row, [batch*heads_q*seqlen_q*n_splits])
};

// LDS layouts (rows of DP elements = CPR chunks of 16 bytes; a tile is 64 rows):
//   K tile: physical chunk = logical chunk ^ swzK(row) so that the 16 lanes of a ds_read_b128 (16 different rows,
//           same logical chunk) hit 16 different 16-byte bank groups.
//   V tile: physical chunk = logical chunk ^ swzV(row) so that the 4 rows x 64 bytes a half-wave reads with
//           ds_read_b64_tr_b16 cover all 64 banks once.
template <int DP>
__device__ __forceinline__ int swzK(int row) {
  if constexpr (DP == 64) return (row >> 1) & 7;
  return row & 15;
}
template <int DP>
__device__ __forceinline__ int swzV(int row) {
  if constexpr (DP == 64) return ((row >> 1) & 1) << 2;
  return (row & 3) << 2;
}

// A new row maximum only forces a rescale of the accumulators when it exceeds the one in use by more than this
// many powers of two; until then probabilities are formed against the older maximum and may reach 2^kLazyLog2,
// which fp32 sums and fp16/bf16 P operands hold without loss.  The final out = O / l and LSE = m c + log2 l do not
// depend on which maximum was in use.
constexpr float kLazyLog2 = 8.0f;


}  // namespace fa

#endif  // FA_FWD_COMMON_H_
