// Flash-attention backward for MI355X (gfx950): HIP kernels and the C-ABI launcher declared in include/fa_bwd.h.
//
// Replaces the vendor call cnnlFlashAttentionBackward that torch_mlu's launcher makes
// (torch_mlu/csrc/aten/operators/cnnl/internal/FlashAttention_internal.cpp:449-480) and its descriptor / workspace
// plumbing (:368-447).
//
// Two kernels, no atomics, deterministic:
//   fa_bwd_dq_kernel   — one workgroup = 128 query rows of one (sequence, head), loops over K/V tiles of 64 rows.
//                        Per lane one query row (as in the forward): S^T = K Q^T, dP^T = V dO^T,
//                        P^T = exp2(S^T c - LSE), dS^T = P^T o (dP^T - delta), dQ^T += K^T dS^T.
//                        Also computes delta = rowsum(dO o O) for its rows and stores -delta and LSE log2(e) for the
//                        second kernel (which then starts its dP accumulators from -delta and needs no rescaling of LSE).
//   fa_bwd_dkv_kernel  — one workgroup = 128 key rows of one (sequence, kv head), loops over the query heads of the
//                        GQA group and over Q/dO tiles of 64 rows.  Per lane one key row: S = Q K^T, dP = dO V^T,
//                        P, dS as above, dV^T += dO^T P, dK^T += Q^T dS.
// Both stream their tiles through LDS by global->LDS DMA with one XOR swizzle that is conflict-free for row reads
// (ds_read_b128, MFMA A operand) and for transposed reads (ds_read_b64_tr_b16) of the same tile.
// S and dP are recomputed in each kernel (7 matrix products per tile pair instead of 5) in exchange for not needing
// fp32 atomics on dQ.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "fa_bwd.h"
#include "fa_device.h"
#include "fa_host.h"

// ring depths of the two operand prefetch loops of the dQ kernel
#ifndef FA_RQ
#define FA_RQ 2
#endif
#ifndef FA_RA
#define FA_RA 2
#endif
// ring depths of the two operand prefetch loops of the dK/dV kernel, by what the instantiation computes
#ifndef FA_RS
#define FA_RS(DO_K, DO_V) ((DO_K) ? 2 : 4)
#endif
#ifndef FA_RT
#define FA_RT(DO_K, DO_V) ((DO_K) && (DO_V) ? 2 : 4)
#endif
// heads whose workgroups are interleaved when a bias is broadcast over heads
#ifndef FA_HGROUP
#define FA_HGROUP 4
#endif
// dV-only kernel: all 64 query rows of a tile in one pass (needs 16 more registers)
#ifndef FA_WIDE
#define FA_WIDE(DO_K, DO_V, DP, BIAS) (!(DO_K) && (DP) == 128 && !(BIAS))
#endif
namespace {

using namespace fa;

struct BArgs {
  const unsigned char* q;
  const unsigned char* k;
  const unsigned char* v;
  const unsigned char* o;
  const unsigned char* dout;
  const float* lse;
  unsigned char* dq;
  unsigned char* dk;
  unsigned char* dv;
  float* delta;  // workspace, dense [B][Hq][Sq], packed [Hq][total_q]: -rowsum(dO o O), written by the dQ kernel
  float* lse2;   // workspace, same shape: LSE * log2(e)
  const int32_t* cu_q;
  const int32_t* cu_k;
  int64_t q_sb, q_ss, q_sh;  // byte strides
  int64_t k_sb, k_ss, k_sh;
  int64_t v_sb, v_ss, v_sh;
  int64_t o_sb, o_ss, o_sh;
  int64_t do_sb, do_ss, do_sh;
  int64_t dq_sb, dq_ss, dq_sh;
  int64_t dk_sb, dk_ss, dk_sh;
  int64_t dv_sb, dv_ss, dv_sh;
  int64_t lse_sb, lse_sh, lse_ss;  // element strides
  int64_t dl_sb, dl_sh;            // delta strides (elements); row stride is 1
  int32_t batch, heads_q, heads_k, group;
  int32_t seqlen_q, seqlen_k, head_dim;
  int32_t n_qslot, n_kslot;  // workgroups per (sequence, head) of the dQ kernel / per (sequence, kv head) of the dK/dV kernel
  int32_t is_causal;
  // causal problems with few workgroups per CU: heads of an XCD's range interleaved, heaviest block index first
  // (better balance); otherwise head after head (better L2 reuse)
  int32_t blockmajor_q, blockmajor_k;
  int32_t hgroup_q, hgroup_k;  // a bias shared by all heads: (kv) heads whose workgroups are interleaved (1 = none)
  float scale;       // signed softmax scale
  float scale_log2;  // scale * log2(e), signed
  uint32_t drop_thr;  // dropout: an element was kept iff its byte <= drop_thr
  float drop_rp;      // 256 / (drop_thr + 1): one over the realised keep probability
  const int64_t* seed_ptr;    // the forward's philox_seed / philox_offset slots (device)
  const int64_t* offset_ptr;
  int32_t causal_tl;          // causal mask aligned to the top-left corner (col <= row) instead of the bottom-right one
  const unsigned char* bias;  // optional additive bias [b][h][row][col] through byte strides (dense mode only)
  int64_t bias_sb, bias_sh, bias_sq;
  unsigned char* dbias;       // optional gradient of the bias, same addressing
  int64_t dbias_sb, dbias_sh, dbias_sq;
};

// One swizzle for tiles that are read both by rows (16 lanes = 16 consecutive rows, same logical chunk) and
// transposed (a half-wave = 4 consecutive rows x 4 consecutive chunks): physical chunk = logical ^ swzU(row).
template <int DP>
__device__ __forceinline__ int swzU(int row) {
  if constexpr (DP == 64) return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
  return ((row & 3) << 2) | ((row >> 2) & 3);
}

template <typename T, int DP>
struct TileIO {
  static constexpr int CPR = DP / 8;
  static constexpr int ROWB = DP * 2;
  static constexpr int TILE = 64 * ROWB;
  static constexpr int NI = TILE / 1024 / 4;
  static constexpr int RPI = 64 / CPR;
  static constexpr int KS = DP / 16;
  static constexpr int MB = DP / 32;
  // consecutive DMA instructions of a wavefront are 4 RPI rows apart; the swizzle repeats every 16 rows, so at
  // head_dim 256 (8 rows apart) even and odd instructions need their own chunk index
  static constexpr int NV = (4 * RPI) % 16 == 0 ? 1 : 2;
};

// ---------------------------------------------------------------------------------------------------------
// dQ kernel
// ---------------------------------------------------------------------------------------------------------
// BIAS: the additive bias of this lane's query row is read straight from global memory into the score layout (8 bytes
// = 4 consecutive keys per load, as in the forward); dS of the tile, already packed for the dQ product, is also what
// the gradient of the bias is, and is stored from here (tiles the causal mask skips are stored as zeros).
// BIAS = 2: the bias tile comes through LDS instead, fetched by DMA most of a tile ahead in 16-byte pieces (rows must be
// 16-byte aligned and seqlen_k a multiple of 8): the direct loads are issued only 32 MFMAs before their use.
template <typename T, int DP, bool DROP, int BIAS>
__global__ void __launch_bounds__(256, DP > 128 ? 1 : 2) fa_bwd_dq_kernel(const BArgs a) {
  using IO = TileIO<T, DP>;
  constexpr int CPR = IO::CPR, ROWB = IO::ROWB, TILE = IO::TILE, NI = IO::NI, RPI = IO::RPI, KS = IO::KS, MB = IO::MB;
  constexpr int NV = IO::NV;
  constexpr int BM = 128, BN = 64;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];  // K0 K1 V0 V1

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, c32 = lane & 31;

  // Workgroups are dealt round-robin to the 8 XCDs and dispatched in order: dense problems give each XCD a contiguous
  // range of logical ids (all query blocks of a head share one L2, and no XCD gets only the heavy blocks); packed
  // problems go block-major, heaviest block index first, and sequences shorter than that exit at once.
  int lid = blockIdx.x;
  int pslot, bh;
  if (a.cu_q) {
    const int nbh = a.batch * a.heads_q;
    pslot = lid / nbh;
    bh = lid % nbh;
  } else {
    const int per = gridDim.x >> 3;
    const int nh = per / a.n_qslot;  // whole heads per XCD range
    if (a.blockmajor_q && lid < (per << 3) && nh * a.n_qslot == per) {
      // within an XCD's range run the heaviest block index of all its heads first (longest first)
      const int idx = lid >> 3;
      pslot = idx / nh;
      bh = (lid & 7) * nh + idx % nh;
    } else {
      if (lid < (per << 3)) lid = (lid & 7) * per + (lid >> 3);
      if (BIAS && a.hgroup_q > 1) {
        // a bias broadcast over heads: the same query block of hgroup_q heads runs side by side, so that one fetch
        // of a bias tile serves all of them from L2
        const int span = a.hgroup_q * a.n_qslot;
        const int r = lid % span;
        pslot = r / a.hgroup_q;
        bh = (lid / span) * a.hgroup_q + r % a.hgroup_q;
      } else {
        pslot = lid % a.n_qslot;
        bh = lid / a.n_qslot;
      }
    }
  }
  const int h = bh % a.heads_q, b = bh / a.heads_q;
  const int hk = h / a.group;

  int q0 = 0, k0 = 0, Lq = a.seqlen_q, Lk = a.seqlen_k;
  int64_t qb = (int64_t)b * a.q_sb, kb = (int64_t)b * a.k_sb, vb = (int64_t)b * a.v_sb, ob = (int64_t)b * a.o_sb;
  int64_t dob = (int64_t)b * a.do_sb, dqb = (int64_t)b * a.dq_sb;
  int64_t lb = (int64_t)b * a.lse_sb, dlb = (int64_t)b * a.dl_sb;
  if (a.cu_q) {
    q0 = a.cu_q[b];
    Lq = a.cu_q[b + 1] - q0;
    k0 = a.cu_k[b];
    Lk = a.cu_k[b + 1] - k0;
    qb = kb = vb = ob = dob = dqb = 0;
    lb = dlb = 0;
  }
  // heaviest (last) query block first; packed: counted down from the longest possible sequence
  const int nblk = (Lq + BM - 1) / BM;
  const int blk_first = (a.cu_q ? a.n_qslot : nblk) - 1 - pslot;
  if (blk_first < 0 || blk_first >= nblk) return;
  const int off = a.causal_tl ? 0 : Lk - Lq;
  const int D = a.head_dim;
  const int last_k = Lk - 1;

  const unsigned char* kp = a.k + kb + (int64_t)k0 * a.k_ss + (int64_t)hk * a.k_sh;
  const unsigned char* vp = a.v + vb + (int64_t)k0 * a.v_ss + (int64_t)hk * a.v_sh;

  // ---- DMA: rows clamped to the last valid one, logical chunk un-swizzled on the global side ----
  const int dma_r = wave * RPI + lane / CPR;
  int lcv[NV];  // logical chunk this lane fetches, per instruction parity (see TileIO::NV)
#pragma unroll
  for (int n = 0; n < NV; ++n) {
    lcv[n] = (lane % CPR) ^ swzU<DP>(dma_r + n * 4 * RPI);
    if (lcv[n] * 8 >= D) lcv[n] = 0;
  }
  const unsigned k_ss = (unsigned)a.k_ss, v_ss = (unsigned)a.v_ss;
  const unsigned lds0 = (unsigned)(uintptr_t)(LDS_AS unsigned char*)smem + wave * 1024;
  // per-lane byte offsets of a full tile's first DMA block; the later blocks only move the scalar base
  unsigned koff0[NV], voff0[NV];
#pragma unroll
  for (int n = 0; n < NV; ++n) {
    koff0[n] = (unsigned)dma_r * k_ss + lcv[n] * 16;
    voff0[n] = (unsigned)dma_r * v_ss + lcv[n] * 16;
  }
  auto issue_tile = [&](int j, int buf) {
    const int rmax = last_k - j * BN;
    const unsigned char* kt = kp + (uint64_t)(unsigned)(j * BN) * k_ss;
    const unsigned char* vt = vp + (uint64_t)(unsigned)(j * BN) * v_ss;
    // the whole tile lies inside the sequence: scalar address arithmetic only (not in the bias variants, which have no
    // registers to spare for the two offsets)
    if (!BIAS && rmax >= BN - 1) {
#pragma unroll
      for (int i = 0; i < NI; ++i)
        dma16s(kt + (uint64_t)(unsigned)(i * 4 * RPI) * k_ss, koff0[i % NV], lds0 + buf * TILE + i * 4096);
#pragma unroll
      for (int i = 0; i < NI; ++i)
        dma16s(vt + (uint64_t)(unsigned)(i * 4 * RPI) * v_ss, voff0[i % NV], lds0 + 2 * TILE + buf * TILE + i * 4096);
      return;
    }
#pragma unroll
    for (int i = 0; i < NI; ++i)
      dma16s(kt, (unsigned)min(dma_r + i * 4 * RPI, rmax) * k_ss + lcv[i % NV] * 16, lds0 + buf * TILE + i * 4096);
#pragma unroll
    for (int i = 0; i < NI; ++i)
      dma16s(vt, (unsigned)min(dma_r + i * 4 * RPI, rmax) * v_ss + lcv[i % NV] * 16, lds0 + 2 * TILE + buf * TILE + i * 4096);
  };

  const float c = a.scale_log2;
  int kaddr[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) kaddr[ks] = c32 * ROWB + (((2 * ks + g) ^ swzU<DP>(c32)) * 16);
  const int L = lane & 15, G = lane >> 4;
  const int t_row = 4 * g + (L >> 2);
  int taddr[2][MB];  // transposed-fragment addresses, [half][mb]: rows t_row (+8)
#pragma unroll
  for (int hf = 0; hf < 2; ++hf)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      taddr[hf][mb] = (t_row + 8 * hf) * ROWB + (L & 1) * 8 +
                      (((4 * mb + 2 * (G & 1) + ((L & 3) >> 1)) ^ swzU<DP>(t_row + 8 * hf)) * 16);

  const int m0 = blk_first * BM;
  int n_end = Lk;
  if (a.is_causal) n_end = min(Lk, m0 + BM + off);
  if (n_end < 0) n_end = 0;
  const int ntiles = (n_end + BN - 1) / BN;
  const int row = m0 + 32 * wave + c32;
  const int wave_row_lo = m0 + 32 * wave, wave_row_hi = wave_row_lo + 31;
  if (ntiles > 0) issue_tile(0, 0);

  // ---- per-row operands: Q and dO fragments (B operands), delta, LSE ----
  s16x8 qf[KS], dof[KS];
  float delta = 0.f;
  {
    const int qr = min(row, Lq - 1);
    const unsigned char* qrow = a.q + qb + (int64_t)(q0 + qr) * a.q_ss + (int64_t)h * a.q_sh;
    const unsigned char* dorow = a.dout + dob + (int64_t)(q0 + qr) * a.do_ss + (int64_t)h * a.do_sh;
    const unsigned char* orow = a.o + ob + (int64_t)(q0 + qr) * a.o_ss + (int64_t)h * a.o_sh;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int ch = 2 * ks + g;
      u32x4 x = {0, 0, 0, 0}, y = {0, 0, 0, 0}, z = {0, 0, 0, 0};
      if (ch * 8 < D) {
        x = *(const u32x4*)(qrow + ch * 16);
        y = *(const u32x4*)(dorow + ch * 16);
        z = *(const u32x4*)(orow + ch * 16);
      }
      qf[ks] = __builtin_bit_cast(s16x8, x);
      dof[ks] = __builtin_bit_cast(s16x8, y);
      typedef T T8 __attribute__((ext_vector_type(8)));
      const T8 dv8 = __builtin_bit_cast(T8, y), ov8 = __builtin_bit_cast(T8, z);
#pragma unroll
      for (int e = 0; e < 8; ++e) delta += (float)dv8[e] * (float)ov8[e];
    }
    delta = pair_sum32(delta);
  }
  const float lse2 =
      (row < Lq) ? a.lse[lb + (int64_t)h * a.lse_sh + (int64_t)(q0 + row) * a.lse_ss] * kLog2e : INFINITY;
  if (row < Lq && g == 0) {
    a.delta[dlb + (int64_t)h * a.dl_sh + (q0 + row)] = -delta;
    a.lse2[dlb + (int64_t)h * a.dl_sh + (q0 + row)] = lse2;
  }

  f32x16 acc[MB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
  if constexpr (DP == 256) {
    // One wavefront per SIMD, 512 registers: of those only 256 are vector registers proper.  The operands that
    // nothing but MFMAs touch (the Q and dO fragments, the dQ accumulators: 256 registers) are sent to the
    // accumulation half here, which leaves the vector half to the scores.
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      asm volatile("" : "+a"(qf[ks]));
      asm volatile("" : "+a"(dof[ks]));
    }
#pragma unroll
    for (int i = 0; i < MB; ++i) asm volatile("" : "+a"(acc[i]));
  }
  const int causal_row_lim = a.is_causal ? row + off : 0x7fffffff;
  // dropout: the forward's mask, regenerated (same patch words, same lane layout as the forward's scores)
  uint32_t drop_row = 0, drop_key2 = 0;
  if constexpr (DROP) {
    const DropKeys dk = drop_head_keys((uint64_t)*a.seed_ptr, (uint64_t)*a.offset_ptr, (uint32_t)bh);
    drop_row = dk.k1 ^ drop_row_term((uint32_t)row >> 1);
    drop_key2 = dk.k2;
  }
  const int drop_sh = 16 * (row & 1);
  // bias / dBias of this lane's row, at its first key group (4 g)
  const unsigned char* brow = nullptr;
  unsigned char* dbrow = nullptr;
  if constexpr (BIAS) {
    const int64_t r = min(row, Lq - 1);
    brow = a.bias + (int64_t)b * a.bias_sb + (int64_t)h * a.bias_sh + r * a.bias_sq + 8 * g;
    if (a.dbias && row < Lq) dbrow = a.dbias + (int64_t)b * a.dbias_sb + (int64_t)h * a.dbias_sh + r * a.dbias_sq + 8 * g;
  }
  // BIAS == 2: this wavefront's 32 rows x 64 keys of the bias tile (4 KiB) go through a private LDS area.  DMA
  // instruction i brings rows 8 i .. 8 i + 7; lane l fetches 16 bytes (8 keys): row 8 i + l / 8, key chunk
  // (l % 8) ^ (l / 8), so that row r keeps chunk ch at r * 128 + ((ch ^ (r & 7)) * 16).
  const unsigned char* bbase = nullptr;  // wavefront-uniform: this block's first bias row
  unsigned boff[BIAS == 2 ? 4 : 1];      // per-lane byte offsets of the four DMA instructions
  const int bchunk = (lane & 7) ^ (lane >> 3);
  const unsigned blds = lds0 - wave * 1024 + 4 * TILE + wave * 4096;
  int baddr = 0;  // per-lane LDS read offset of key chunk 0; chunk ch is at baddr ^ (ch * 16)
  if constexpr (BIAS == 2) {
    bbase = a.bias + (int64_t)b * a.bias_sb + (int64_t)h * a.bias_sh + (int64_t)m0 * a.bias_sq;
    const int rmax = Lq - 1 - m0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      boff[i] = (unsigned)min(32 * wave + 8 * i + (lane >> 3), rmax) * (unsigned)a.bias_sq + bchunk * 16;
    baddr = 4 * TILE + wave * 4096 + c32 * 128 + (c32 & 7) * 16 + 8 * g;
  }
  // chunks that start at or beyond Lk (last, partial tile) are pointed at the tile's chunk 0: their scores are masked
  auto issue_bias = [&](int j) {
    const unsigned char* bt = bbase + (int64_t)j * (BN * 2);
    const unsigned adj = (j * BN + bchunk * 8 >= Lk) ? bchunk * 16 : 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) dma16s(bt, boff[i] - adj, blds + i * 1024);
  };
  if constexpr (BIAS == 2)
    if (ntiles > 0) issue_bias(0);
  // chunk t of tile j holds dS of keys j BN + 32 (t >> 1) + 16 (t & 1) + 4 g + {0..3, 8..11} of this lane's row
  auto store_dbias = [&](int j, int t, u32x4 w) {
    if (!dbrow) return;
    const int col = j * BN + 32 * (t >> 1) + 16 * (t & 1);
    unsigned char* d = dbrow + col * 2;
    if (j * BN + BN <= Lk) {
      *(u32x2*)d = u32x2{w[0], w[1]};
      *(u32x2*)(d + 16) = u32x2{w[2], w[3]};
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int e = 8 * (i >> 2) + (i & 3);
        const uint32_t word = w[i >> 1];
        if (col + 4 * g + e < Lk) *(unsigned short*)(d + e * 2) = (unsigned short)((i & 1) ? (word >> 16) : (word & 0xffffu));
      }
    }
  };

  for (int j = 0; j < ntiles; ++j) {
    const int buf = j & 1;
    WAIT_VMCNT(0);
    __syncthreads();
    if (j + 1 < ntiles) issue_tile(j + 1, buf ^ 1);
    if (a.is_causal && j * BN > wave_row_hi + off) {  // fully masked for this wavefront
      if constexpr (BIAS) {
#pragma unroll
        for (int t = 0; t < 4; ++t) store_dbias(j, t, u32x4{0, 0, 0, 0});
      }
      continue;
    }

    const unsigned char* kt = smem + buf * TILE;
    const unsigned char* vt = smem + 2 * TILE + buf * TILE;
    // bias of this tile: 8 loads of 4 keys each (a partial last tile: element-wise, columns clamped to the last valid
    // one, masked below anyway), issued now and consumed after the S / dP MFMAs
    const bool full_tile = j * BN + BN <= Lk;
    u32x2 braw[BIAS ? 8 : 1];
    if constexpr (BIAS == 1) {
      if (full_tile) {
        const unsigned char* bt = brow + (int64_t)j * (BN * 2);
#pragma unroll
        for (int i = 0; i < 8; ++i) braw[i] = *(const u32x2*)(bt + (32 * (i >> 2) + 8 * (i & 3)) * 2);
      } else {
        const unsigned short* be = (const unsigned short*)(brow + (int64_t)j * (BN * 2));
        const int cmax = last_k - j * BN - 4 * g;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int e = 32 * (i >> 2) + 8 * (i & 3);
          braw[i][0] = (uint32_t)be[min(e, cmax)] | ((uint32_t)be[min(e + 1, cmax)] << 16);
          braw[i][1] = (uint32_t)be[min(e + 2, cmax)] | ((uint32_t)be[min(e + 3, cmax)] << 16);
        }
      }
    }
    f32x16 s0, s1, p0, p1;
#pragma unroll
    for (int v = 0; v < 16; ++v) { s0[v] = 0.f; s1[v] = 0.f; p0[v] = 0.f; p1[v] = 0.f; }
    {
      // K and V fragments are fetched RQ - 1 k-steps ahead of the MFMAs that consume them (a ring of RQ slots)
      constexpr int RQ = FA_RQ;
      s16x8 fr[RQ][4];
      auto load_fr = [&](int ks) {
        fr[ks % RQ][0] = *(const s16x8*)(kt + kaddr[ks]);
        fr[ks % RQ][1] = *(const s16x8*)(kt + kaddr[ks] + 32 * ROWB);
        fr[ks % RQ][2] = *(const s16x8*)(vt + kaddr[ks]);
        fr[ks % RQ][3] = *(const s16x8*)(vt + kaddr[ks] + 32 * ROWB);
      };
#pragma unroll
      for (int ks = 0; ks < RQ - 1; ++ks) load_fr(ks);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks + RQ - 1 < KS) load_fr(ks + RQ - 1);
        s0 = Mma<T>::m32(fr[ks % RQ][0], qf[ks], s0);
        s1 = Mma<T>::m32(fr[ks % RQ][1], qf[ks], s1);
        p0 = Mma<T>::m32(fr[ks % RQ][2], dof[ks], p0);
        p1 = Mma<T>::m32(fr[ks % RQ][3], dof[ks], p1);
        __builtin_amdgcn_sched_barrier(0);  // keep the loads of the later steps ahead of these MFMAs
      }
    }
    // P^T = exp2(S^T c - LSE), dS^T = P^T (dP^T - delta); masked positions contribute nothing
    // masked positions (beyond the sequence, above the causal diagonal) get a score whose exponential is 0; only the
    // diagonal and tail tiles run this
    // (the variant that reads the bias directly, short of registers, selects per element in the loop below instead)
    const bool need_mask = (j * BN + BN > Lk) || (a.is_causal && j * BN + BN - 1 > wave_row_lo + off);
    const int lim = need_mask ? min(last_k, causal_row_lim) - j * BN - 4 * g : 0x7fffffff;  // element e visible iff e <= lim
    if (BIAS != 1 && need_mask) {
      const float gone = (c < 0.f) ? INFINITY : -INFINITY;           // times c: -inf (c is never 0)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int e = 8 * (v >> 2) + (v & 3);
        if (e > lim) s0[v] = gone;
        if (32 + e > lim) s1[v] = gone;
      }
    }
    const uint32_t drop_tile = DROP ? (drop_row ^ drop_col_term((uint32_t)(j * (BN / 2) + 2 * g))) : 0u;
    s16x8 dsb[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      if constexpr (BIAS == 2) {  // the two 4-key groups of chunk t
        braw[4 * (t >> 1) + 2 * (t & 1)] = *(const u32x2*)(smem + (baddr ^ ((4 * (t >> 1) + 2 * (t & 1)) * 16)));
        braw[4 * (t >> 1) + 2 * (t & 1) + 1] = *(const u32x2*)(smem + (baddr ^ ((4 * (t >> 1) + 2 * (t & 1) + 1) * 16)));
      }
      u32x4 w;
#pragma unroll
      for (int e2 = 0; e2 < 4; ++e2) {
        float ds[2];
        uint32_t word = 0;
        if constexpr (DROP) {
          const int v0 = 8 * (t & 1) + 2 * e2;
          word = drop_word(drop_tile ^ (uint32_t)(16 * (t >> 1) + 4 * (v0 >> 2) + ((v0 & 3) >> 1)), drop_key2) >> drop_sh;
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int v = 8 * (t & 1) + 2 * e2 + u;
          const float sv = (t < 2) ? s0[v] : s1[v];
          float dpv = (t < 2) ? p0[v] : p1[v];
          float xl = lse2;  // what is subtracted in the exponent: LSE - bias, in log2 units
          if constexpr (BIAS) {
            const uint32_t bw = braw[4 * (t >> 1) + (v >> 2)][(v & 3) >> 1];
            xl = lse2 - Mma<T>::to_float((unsigned short)((v & 1) ? (bw >> 16) : (bw & 0xffffu))) * kLog2e;
          }
          float p = fast_exp2(sv * c - xl);
          if constexpr (BIAS == 1) p = (32 * (t >> 1) + 8 * (v >> 2) + (v & 3) <= lim) ? p : 0.f;
          if constexpr (DROP) dpv = (((word >> (8 * u)) & 0xffu) <= a.drop_thr) ? dpv * a.drop_rp : 0.f;
          ds[u] = p * (dpv - delta);
        }
        w[e2] = Mma<T>::pack2(ds[0], ds[1]);
      }
      dsb[t] = __builtin_bit_cast(s16x8, w);
      if constexpr (BIAS) store_dbias(j, t, w);
    }
    if constexpr (BIAS == 2) {
      // the next tile's bias may overwrite this one now: every dS depends on the values that were read
      asm volatile("" : : "v"(dsb[0]), "v"(dsb[1]), "v"(dsb[2]), "v"(dsb[3]) : "memory");
      if (j + 1 < ntiles) issue_bias(j + 1);
    }
    // dQ^T += K^T dS^T; the transposed K fragments of chunk t + 1 are fetched while chunk t's MFMAs run
    {
      auto kfrag = [&](int mb, int t) {
        const s16x4 lo = lds_read_tr(kt + taddr[0][mb] + (16 * t) * ROWB);
        const s16x4 hi = lds_read_tr(kt + taddr[1][mb] + (16 * t) * ROWB);
        return s16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      };
      constexpr int RA = FA_RA;
      s16x8 ka[RA][MB];
#pragma unroll
      for (int t = 0; t < RA - 1; ++t)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) ka[t][mb] = kfrag(mb, t);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        if (t + RA - 1 < 4) {
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) ka[(t + RA - 1) % RA][mb] = kfrag(mb, t + RA - 1);
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[mb] = Mma<T>::m32(ka[t % RA][mb], dsb[t], acc[mb]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  if constexpr (BIAS) {  // key tiles beyond the causal bound of this block: dBias = 0
    const int nall = (Lk + BN - 1) / BN;
    for (int j = ntiles; j < nall; ++j)
#pragma unroll
      for (int t = 0; t < 4; ++t) store_dbias(j, t, u32x4{0, 0, 0, 0});
  }

  // dQ goes out through LDS, as O does in the forward kernel: staged per wavefront (32 rows, row stride padded by
  // 16 bytes) and stored as whole rows instead of 8-byte pieces of 32 rows per instruction.
  __syncthreads();  // every wavefront is done with the K/V buffers of the last tile
  {
    constexpr int OSTR = ROWB + 16;
    unsigned char* stage = smem + wave * (32 * OSTR);
    const float sc = a.scale;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int v4 = 0; v4 < 4; ++v4) {
        u32x2 w;
        w[0] = Mma<T>::pack2(acc[mb][4 * v4 + 0] * sc, acc[mb][4 * v4 + 1] * sc);
        w[1] = Mma<T>::pack2(acc[mb][4 * v4 + 2] * sc, acc[mb][4 * v4 + 3] * sc);
        *(u32x2*)(stage + c32 * OSTR + (32 * mb + 8 * v4 + 4 * g) * 2) = w;
      }
    constexpr int RPS = 64 / CPR;  // rows per store instruction
    unsigned char* oblk = a.dq + dqb + (int64_t)(q0 + m0 + 32 * wave) * a.dq_ss + (int64_t)h * a.dq_sh;
    const int sr = lane / CPR, sch = lane % CPR;
    const int rows_left = Lq - (m0 + 32 * wave);
#pragma unroll
    for (int i = 0; i < 32 / RPS; ++i) {
      const int r = i * RPS + sr;
      const u32x4 x = *(const u32x4*)(stage + r * OSTR + sch * 16);
      if (r < rows_left && sch * 8 < D) *(u32x4*)(oblk + (int64_t)r * a.dq_ss + sch * 16) = x;
    }
  }
}

// ---------------------------------------------------------------------------------------------------------
// dK / dV kernel
// ---------------------------------------------------------------------------------------------------------
// WHAT selects the outputs: kDK (S, dP, dS, dK), kDV (S, P, dV) or both.  With head_dim 128 both accumulators do not
// fit the 256 registers that two wavefronts per SIMD leave, so dK and dV run as two launches (S is recomputed once
// more); with head_dim <= 64 one launch produces both.
constexpr int kDK = 1, kDV = 2;

// BIAS: here a lane owns a key column and its registers run over query rows, while the bias is contiguous along keys.
// A 32 x 32 block of it is therefore loaded as an MFMA A operand (a lane = one query row, 8 consecutive keys per
// k-step: 8-byte loads) and multiplied by the identity: the product is the same block in the score layout, exact
// (every output is one input times 1.0 plus zeros).  -inf entries are lowered to the most negative finite value
// first, since -inf * 0 would turn the whole row into NaN; the exponential of either is 0.  A block's loads are issued
// ahead of its S / dP MFMAs and consumed after them.
template <typename T, int DP, int WHAT, bool DROP, bool BIAS>
__global__ void __launch_bounds__(256, DP > 128 ? 1 : 2) fa_bwd_dkv_kernel(const BArgs a) {
  constexpr bool DO_K = (WHAT & kDK) != 0, DO_V = (WHAT & kDV) != 0;
  using IO = TileIO<T, DP>;
  constexpr int CPR = IO::CPR, ROWB = IO::ROWB, TILE = IO::TILE, NI = IO::NI, RPI = IO::RPI, KS = IO::KS, MB = IO::MB;
  constexpr int NV = IO::NV;
  constexpr int BKV = 128, BQ = 64;
  constexpr int VEC = 4 * TILE;  // Q0 Q1 dO0 dO1 | lse[2][64] delta[2][64]
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, c32 = lane & 31;

  // Same dispatch-order reasoning as the dQ kernel.  Causal: the first key blocks are the heavy ones (every query
  // row sees them) and they come first.
  int lid = blockIdx.x;
  int pslot, bhk;
  if (a.cu_q) {
    const int nbh = a.batch * a.heads_k;
    pslot = lid / nbh;
    bhk = lid % nbh;
  } else {
    const int per = gridDim.x >> 3;
    const int nh = per / a.n_kslot;
    if (a.blockmajor_k && lid < (per << 3) && nh * a.n_kslot == per) {
      const int idx = lid >> 3;
      pslot = idx / nh;
      bhk = (lid & 7) * nh + idx % nh;
    } else {
      if (lid < (per << 3)) lid = (lid & 7) * per + (lid >> 3);
      if (BIAS && a.hgroup_k > 1) {  // as in the dQ kernel: the same key block of hgroup_k kv heads side by side
        const int span = a.hgroup_k * a.n_kslot;
        const int r = lid % span;
        pslot = r / a.hgroup_k;
        bhk = (lid / span) * a.hgroup_k + r % a.hgroup_k;
      } else {
        pslot = lid % a.n_kslot;
        bhk = lid / a.n_kslot;
      }
    }
  }
  const int hk = bhk % a.heads_k, b = bhk / a.heads_k;

  int q0 = 0, k0 = 0, Lq = a.seqlen_q, Lk = a.seqlen_k;
  int64_t qb = (int64_t)b * a.q_sb, kb = (int64_t)b * a.k_sb, vb = (int64_t)b * a.v_sb, dob = (int64_t)b * a.do_sb;
  int64_t dkb = (int64_t)b * a.dk_sb, dvb = (int64_t)b * a.dv_sb;
  int64_t dlb = (int64_t)b * a.dl_sb;
  if (a.cu_q) {
    q0 = a.cu_q[b];
    Lq = a.cu_q[b + 1] - q0;
    k0 = a.cu_k[b];
    Lk = a.cu_k[b + 1] - k0;
    qb = kb = vb = dob = dkb = dvb = 0;
    dlb = 0;
  }
  if (pslot * BKV >= Lk) return;
  const int off = a.causal_tl ? 0 : Lk - Lq;
  const int D = a.head_dim;

  const int dma_r = wave * RPI + lane / CPR;
  int lcv[NV];
#pragma unroll
  for (int n = 0; n < NV; ++n) {
    lcv[n] = (lane % CPR) ^ swzU<DP>(dma_r + n * 4 * RPI);
    if (lcv[n] * 8 >= D) lcv[n] = 0;
  }
  const unsigned q_ss = (unsigned)a.q_ss, do_ss = (unsigned)a.do_ss;
  const unsigned lds0 = (unsigned)(uintptr_t)(LDS_AS unsigned char*)smem + wave * 1024;
  const unsigned ldsv = (unsigned)(uintptr_t)(LDS_AS unsigned char*)smem + VEC;
  const float c = a.scale_log2;

  int kaddr[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) kaddr[ks] = c32 * ROWB + (((2 * ks + g) ^ swzU<DP>(c32)) * 16);
  const int L = lane & 15, G = lane >> 4;
  const int t_row = 4 * g + (L >> 2);
  int taddr[2][MB];
#pragma unroll
  for (int hf = 0; hf < 2; ++hf)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      taddr[hf][mb] = (t_row + 8 * hf) * ROWB + (L & 1) * 8 +
                      (((4 * mb + 2 * (G & 1) + ((L & 3) >> 1)) ^ swzU<DP>(t_row + 8 * hf)) * 16);

  const int n0 = pslot * BKV;
  const int kvrow = n0 + 32 * wave + c32;  // this lane's key row
  // dropout: column term of this lane's key, and which byte pair of a patch word belongs to it
  const uint32_t drop_col = DROP ? drop_col_term((uint32_t)kvrow >> 1) : 0u;
  const int drop_sh = 8 * (kvrow & 1);
  uint64_t drop_seed = 0, drop_offset = 0;
  if constexpr (DROP) {
    drop_seed = (uint64_t)*a.seed_ptr;
    drop_offset = (uint64_t)*a.offset_ptr;
  }
  const int wave_kv_lo = n0 + 32 * wave;
  // query tiles that can see this key block: rows q with q + off >= n0
  int jq_begin = 0;
  if (a.is_causal) jq_begin = max(0, n0 - off) / BQ;
  const int jq_end = (Lq + BQ - 1) / BQ;
  const int nq = max(0, jq_end - jq_begin);
  const int niter = nq * a.group;  // flattened (query head of the group, query tile)

  // ---- K and V fragments of my key row (B operands) ----
  s16x8 kf[KS], vf[KS];
  {
    const int kr = min(kvrow, Lk - 1);
    const unsigned char* krow = a.k + kb + (int64_t)(k0 + kr) * a.k_ss + (int64_t)hk * a.k_sh;
    const unsigned char* vrow = a.v + vb + (int64_t)(k0 + kr) * a.v_ss + (int64_t)hk * a.v_sh;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int ch = 2 * ks + g;
      u32x4 x = {0, 0, 0, 0}, y = {0, 0, 0, 0};
      if (ch * 8 < D) {
        x = *(const u32x4*)(krow + ch * 16);
        if constexpr (DO_K) y = *(const u32x4*)(vrow + ch * 16);
      }
      kf[ks] = __builtin_bit_cast(s16x8, x);
      vf[ks] = __builtin_bit_cast(s16x8, y);
    }
  }

  // per-lane byte offsets of a full tile's first DMA block; the later blocks only move the scalar base
  unsigned qoff0[NV], dooff0[NV];
#pragma unroll
  for (int n = 0; n < NV; ++n) {
    qoff0[n] = (unsigned)dma_r * q_ss + lcv[n] * 16;
    dooff0[n] = (unsigned)dma_r * do_ss + lcv[n] * 16;
  }
  // ---- DMA of a (query head, query tile): Q rows, dO rows, LSE and delta of the 64 rows ----
  auto issue_iter = [&](int it, int buf) {
    const int hq = hk * a.group + it / nq;
    const int jq = jq_begin + it % nq;
    const int rmax = Lq - 1 - jq * BQ;
    const unsigned char* qt = a.q + qb + (int64_t)(q0 + jq * BQ) * a.q_ss + (int64_t)hq * a.q_sh;
    const unsigned char* dt = a.dout + dob + (int64_t)(q0 + jq * BQ) * a.do_ss + (int64_t)hq * a.do_sh;
    if (!BIAS && rmax >= BQ - 1) {  // the whole tile lies inside the sequence: scalar address arithmetic only
#pragma unroll
      for (int i = 0; i < NI; ++i)
        dma16s(qt + (uint64_t)(unsigned)(i * 4 * RPI) * q_ss, qoff0[i % NV], lds0 + buf * TILE + i * 4096);
#pragma unroll
      for (int i = 0; i < NI; ++i)
        dma16s(dt + (uint64_t)(unsigned)(i * 4 * RPI) * do_ss, dooff0[i % NV], lds0 + 2 * TILE + buf * TILE + i * 4096);
    } else {
#pragma unroll
      for (int i = 0; i < NI; ++i)
        dma16s(qt, (unsigned)min(dma_r + i * 4 * RPI, rmax) * q_ss + lcv[i % NV] * 16, lds0 + buf * TILE + i * 4096);
#pragma unroll
      for (int i = 0; i < NI; ++i)
        dma16s(dt, (unsigned)min(dma_r + i * 4 * RPI, rmax) * do_ss + lcv[i % NV] * 16,
               lds0 + 2 * TILE + buf * TILE + i * 4096);
    }
    if (wave < (DO_K ? 2 : 1)) {  // wavefront 0: LSE log2(e) of the 64 rows, wavefront 1: -delta (4 bytes per lane)
      const int r = min(lane, rmax);
      const float* src = ((wave == 0) ? a.lse2 : a.delta) + dlb + (int64_t)hq * a.dl_sh + (q0 + jq * BQ + r);
      const unsigned dst = ldsv + (wave * 2 + buf) * 256;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(dst), "v"(src) : "m0");
    }
  };
  if (niter > 0) issue_iter(0, 0);
  // The fragments above come from ordinary loads, and the compiler waits for a load at its first use: inside the tile
  // loop that wait (it can only be "every outstanding load") would also cover the next tile's DMA, issued just before,
  // and every tile would start by waiting for its successor.  Using the fragments here puts the wait in front of the
  // loop, where the first tile has to arrive anyway.  (Measured: head_dim 128 gains 1-5 %; head_dim 64 is no faster
  // for it, and at head_dim 256 pinning the fragments here costs the register allocator more than the wait did.)
  if constexpr (DP == 128) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      asm volatile("" : : "v"(kf[ks]));
      if constexpr (DO_K) asm volatile("" : : "v"(vf[ks]));
    }
  }

  // ---- one 32 x 32 bias block (block qbk of iteration it) as A operands: [k-step of 16 keys] ----
  typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));
  auto load_bias = [&](int it, int qbk, u32x4 (&dst)[2]) {
    const int hq = hk * a.group + it / nq;
    const int jq = jq_begin + it % nq;
    const int64_t qr = min(jq * BQ + 32 * qbk + c32, Lq - 1);
    const unsigned char* src0 = a.bias + (int64_t)b * a.bias_sb + (int64_t)hq * a.bias_sh + qr * a.bias_sq;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int kvc = n0 + 32 * wave + 16 * ks + 8 * g;
      const unsigned char* src = src0 + (int64_t)kvc * 2;
      if (kvc + 8 <= Lk) {
        const u32x2 lo = *(const u32x2*)src, hi = *(const u32x2*)(src + 8);
        dst[ks] = u32x4{lo[0], lo[1], hi[0], hi[1]};
      } else {
        u32x4 w = {0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (kvc + e < Lk) w[e >> 1] |= (uint32_t)((const unsigned short*)src)[e] << (16 * (e & 1));
        dst[ks] = w;
      }
    }
  };
  s16x8 ident[2];  // B operand: rows 16 ks + 8 g + e of the 32 x 32 identity, column c32
  if constexpr (BIAS) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int e = 0; e < 8; ++e) ident[ks][e] = (c32 == 16 * ks + 8 * g + e) ? (short)Mma<T>::kOne : (short)0;
  }

  f32x16 dk[MB], dv[MB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) { dk[i][v] = 0.f; dv[i][v] = 0.f; }
  if constexpr (DP == 256 && DO_K) {
    // as in the dQ kernel: the K and V fragments and the dK accumulators (256 registers that only MFMAs touch) go to
    // the accumulation half of the 512 registers a lone wavefront per SIMD has
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      asm volatile("" : "+a"(kf[ks]));
      asm volatile("" : "+a"(vf[ks]));
    }
#pragma unroll
    for (int i = 0; i < MB; ++i) asm volatile("" : "+a"(dk[i]));
  }

  for (int it = 0; it < niter; ++it) {
    const int buf = it & 1;
    WAIT_VMCNT(0);
    __syncthreads();
    if (it + 1 < niter) issue_iter(it + 1, buf ^ 1);
    const int jq = jq_begin + it % nq;
    const int qlo = jq * BQ;
    // every (q, kv) of this tile masked for this wavefront: q + off < kv for all pairs
    if (a.is_causal && qlo + BQ - 1 + off < wave_kv_lo) continue;
    // dropout: key of this iteration's query head ^ column term ^ row term of the tile's first row pair (+ 2 g);
    // the row pair of registers (v, v + 1) adds a compile-time constant with disjoint bits
    uint32_t drop_tile = 0, drop_key2 = 0;
    if constexpr (DROP) {
      const DropKeys dk = drop_head_keys(drop_seed, drop_offset, (uint32_t)(b * a.heads_q + hk * a.group + it / nq));
      drop_tile = dk.k1 ^ drop_col ^ drop_row_term((uint32_t)(qlo / 2 + 2 * g));
      drop_key2 = dk.k2;
    }

    const unsigned char* qt = smem + buf * TILE;
    const unsigned char* dt = smem + 2 * TILE + buf * TILE;
    const float* lse_t = (const float*)(smem + VEC + (0 * 2 + buf) * 256);
    const float* del_t = (const float*)(smem + VEC + (1 * 2 + buf) * 256);
    // Which query rows of this tile may this lane's key see?  Rows ql (relative to the tile) with lo <= ql < hi:
    // hi cuts the rows beyond the sequence, lo is the causal bound kv - off (or "none" for a key beyond the sequence).
    const bool need_mask =
        (qlo + BQ > Lq) || (a.is_causal && qlo + off < wave_kv_lo + 31) || (wave_kv_lo + 32 > Lk);
    const int m_lo = (kvrow < Lk) ? (a.is_causal ? kvrow - off - qlo : -0x40000000) : 0x40000000;
    const unsigned m_span = (unsigned)max(Lq - qlo - m_lo, 0);  // visible iff (unsigned)(ql - m_lo) < m_span
    const int m_base = m_lo - 4 * g;

    // dV alone (head_dim > 64, no bias): the registers allow the scores of all 64 query rows at once, as in the forward
    // kernel: two independent accumulator chains in the S product, one pass of exponentials, 16 dV MFMAs in a row.
    // With 32 rows per pass a wavefront changes between matrix and vector work twice as often, and a SIMD's two
    // wavefronts cover each other's changes less well.
    constexpr bool WIDE = FA_WIDE(DO_K, DO_V, DP, BIAS);
    if constexpr (WIDE) {
      f32x16 s2[2];
#pragma unroll
      for (int v = 0; v < 16; ++v) { s2[0][v] = 0.f; s2[1][v] = 0.f; }
      f32x4 lv[2][4];
      {
        s16x8 qa[2][2];  // [slot][block]: fetched two k-steps ahead
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          qa[ks][0] = *(const s16x8*)(qt + kaddr[ks]);
          qa[ks][1] = *(const s16x8*)(qt + kaddr[ks] + 32 * ROWB);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          s2[0] = Mma<T>::m32(qa[ks & 1][0], kf[ks], s2[0]);
          s2[1] = Mma<T>::m32(qa[ks & 1][1], kf[ks], s2[1]);
          if (ks + 2 < KS) {
            qa[ks & 1][0] = *(const s16x8*)(qt + kaddr[ks + 2]);
            qa[ks & 1][1] = *(const s16x8*)(qt + kaddr[ks + 2] + 32 * ROWB);
          }
          if (ks == KS / 2) {  // LSE of this lane's 32 rows, in time for the exponentials
#pragma unroll
            for (int qbk = 0; qbk < 2; ++qbk)
#pragma unroll
              for (int q4 = 0; q4 < 4; ++q4) lv[qbk][q4] = *(const f32x4*)(lse_t + 32 * qbk + 8 * q4 + 4 * g);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (need_mask) {
        const float gone = (c < 0.f) ? INFINITY : -INFINITY;  // times c: -inf (c is never 0)
#pragma unroll
        for (int qbk = 0; qbk < 2; ++qbk)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int qc = 32 * qbk + 8 * (v >> 2) + (v & 3);  // ql - 4 g
            if (!((unsigned)(qc - m_base) < m_span)) s2[qbk][v] = gone;
          }
      }
      // transposed dO fragments: step i = (chunk tt of 16 query rows, mb), fetched RT - 1 steps ahead
      auto tfrag = [&](int i) {
        const int ro = (16 * (i / MB)) * ROWB;
        const s16x4 lo = lds_read_tr(dt + taddr[0][i % MB] + ro);
        const s16x4 hi = lds_read_tr(dt + taddr[1][i % MB] + ro);
        return s16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      };
      constexpr int RT = 4;
      s16x8 dav[RT];
#pragma unroll
      for (int i = 0; i < RT - 1; ++i) dav[i] = tfrag(i);
      s16x8 pb[4];
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {  // chunk tt: rows 16 tt .. 16 tt + 15 = block tt / 2, half tt % 2
        u32x4 wp;
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
          const int qbk = tt >> 1, v = 8 * (tt & 1) + 2 * e2;
          const float l0 = lv[qbk][v >> 2][v & 3], l1 = lv[qbk][v >> 2][(v & 3) + 1];
          float p0 = fast_exp2(s2[qbk][v] * c - l0), p1 = fast_exp2(s2[qbk][v + 1] * c - l1);
          if constexpr (DROP) {
            const uint32_t rp_const = 16 * qbk + 4 * (v >> 2) + ((v & 3) >> 1);
            const uint32_t word = drop_word(drop_tile ^ (rp_const << 16), drop_key2) >> drop_sh;
            p0 = ((word & 0xffu) <= a.drop_thr) ? p0 * a.drop_rp : 0.f;
            p1 = (((word >> 16) & 0xffu) <= a.drop_thr) ? p1 * a.drop_rp : 0.f;
          }
          wp[e2] = Mma<T>::pack2(p0, p1);
        }
        pb[tt] = __builtin_bit_cast(s16x8, wp);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 4 * MB; ++i) {
        if (i + RT - 1 < 4 * MB) dav[(i + RT - 1) % RT] = tfrag(i + RT - 1);
        dv[i % MB] = Mma<T>::m32(dav[i % RT], pb[i / MB], dv[i % MB]);
        __builtin_amdgcn_sched_barrier(0);
      }
      continue;
    }
#pragma unroll
    for (int qbk = 0; qbk < 2; ++qbk) {  // two blocks of 32 query rows
      // LSE and delta of this lane's 16 rows (register v <-> row 32 qbk + 8 (v >> 2) + 4 g + (v & 3)), fetched ahead
      // of the MFMAs that hide their latency
      // (with a bias the registers are needed elsewhere and the two vectors are read after the MFMAs; in halves
      // where the dK accumulators of head_dim 128 leave no room)
      constexpr bool HALVES = BIAS && DO_K && DP > 64;
      // without dropout the dP accumulators start from -delta of their rows, so that the MFMAs deliver dP - delta
      constexpr bool DELTA_INIT = DO_K && !DROP;
      f32x4 lv[4], dl[4];
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        if constexpr (!BIAS) lv[q4] = *(const f32x4*)(lse_t + 32 * qbk + 8 * q4 + 4 * g);
        if constexpr (DO_K && (!BIAS || DELTA_INIT)) dl[q4] = *(const f32x4*)(del_t + 32 * qbk + 8 * q4 + 4 * g);
      }
      f32x16 s, dp, bacc;
#pragma unroll
      for (int v = 0; v < 16; ++v) { s[v] = 0.f; dp[v] = DELTA_INIT ? dl[v >> 2][v & 3] : 0.f; bacc[v] = 0.f; }
      u32x4 braw[2];  // this block's bias, requested now, used after the S / dP MFMAs
      if constexpr (BIAS) load_bias(it, qbk, braw);
      {
        // Q (and dO) row fragments are fetched RS k-steps ahead of the MFMAs that consume them (a ring of RS slots)
        constexpr int RS = FA_RS(DO_K, DO_V) < KS ? FA_RS(DO_K, DO_V) : KS;
        s16x8 qa[RS], da[RS];
#pragma unroll
        for (int ks = 0; ks < RS; ++ks) {
          qa[ks] = *(const s16x8*)(qt + kaddr[ks] + qbk * 32 * ROWB);
          if constexpr (DO_K) da[ks] = *(const s16x8*)(dt + kaddr[ks] + qbk * 32 * ROWB);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          s = Mma<T>::m32(qa[ks % RS], kf[ks], s);
          if constexpr (DO_K) dp = Mma<T>::m32(da[ks % RS], vf[ks], dp);
          if (ks + RS < KS) {
            qa[ks % RS] = *(const s16x8*)(qt + kaddr[ks + RS] + qbk * 32 * ROWB);
            if constexpr (DO_K) da[ks % RS] = *(const s16x8*)(dt + kaddr[ks + RS] + qbk * 32 * ROWB);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if constexpr (BIAS) {
        // the bias through the matrix unit into the score layout
        s16x8 bcur[2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          const u16x8 x = __builtin_bit_cast(u16x8, braw[ks]);
          const u16x8 lim8 = {Mma<T>::kNegMax, Mma<T>::kNegMax, Mma<T>::kNegMax, Mma<T>::kNegMax,
                              Mma<T>::kNegMax, Mma<T>::kNegMax, Mma<T>::kNegMax, Mma<T>::kNegMax};
          bcur[ks] = __builtin_bit_cast(s16x8, __builtin_elementwise_min(x, lim8));
        }
        bacc = Mma<T>::m32(bcur[0], ident[0], bacc);
        bacc = Mma<T>::m32(bcur[1], ident[1], bacc);
        if constexpr (!HALVES) {
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            lv[q4] = *(const f32x4*)(lse_t + 32 * qbk + 8 * q4 + 4 * g);
            if constexpr (DO_K && !DELTA_INIT) dl[q4] = *(const f32x4*)(del_t + 32 * qbk + 8 * q4 + 4 * g);
          }
        }
      }
      // masked positions get a score whose exponential is 0; only diagonal and tail tiles run this
      if (need_mask) {
        const float gone = (c < 0.f) ? INFINITY : -INFINITY;  // times c: -inf (c is never 0)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int qc = 32 * qbk + 8 * (v >> 2) + (v & 3);  // ql - 4 g
          if (!((unsigned)(qc - m_base) < m_span)) s[v] = gone;
        }
      }
      s16x8 pb[2], dsb[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        u32x4 wp, wd;
        if constexpr (HALVES) {  // LSE and delta of this half's 8 rows only, to keep the register count down
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int q4 = 2 * t; q4 < 2 * t + 2; ++q4) {
            lv[q4] = *(const f32x4*)(lse_t + 32 * qbk + 8 * q4 + 4 * g);
            if constexpr (DO_K && !DELTA_INIT) dl[q4] = *(const f32x4*)(del_t + 32 * qbk + 8 * q4 + 4 * g);
          }
        }
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
          const int v = 8 * t + 2 * e2;  // v, v + 1: consecutive query rows
          float l0 = lv[v >> 2][v & 3], l1 = lv[v >> 2][(v & 3) + 1];
          if constexpr (BIAS) {
            l0 -= bacc[v] * kLog2e;
            l1 -= bacc[v + 1] * kLog2e;
          }
          // minus delta of the two rows (already inside dp when the accumulators started from it)
          const float d0 = (DO_K && !DELTA_INIT) ? dl[v >> 2][v & 3] : 0.f;
          const float d1 = (DO_K && !DELTA_INIT) ? dl[v >> 2][(v & 3) + 1] : 0.f;
          float p0 = fast_exp2(s[v] * c - l0), p1 = fast_exp2(s[v + 1] * c - l1);
          float dp0 = DO_K ? dp[v] : 0.f, dp1 = DO_K ? dp[v + 1] : 0.f;
          float pv0 = p0, pv1 = p1;  // what multiplies dO in dV: P o M / keep
          if constexpr (DROP) {
            const uint32_t rp_const = 16 * qbk + 4 * (v >> 2) + ((v & 3) >> 1);
            const uint32_t word = drop_word(drop_tile ^ (rp_const << 16), drop_key2) >> drop_sh;
            const bool k0 = (word & 0xffu) <= a.drop_thr, k1 = ((word >> 16) & 0xffu) <= a.drop_thr;
            pv0 = k0 ? p0 * a.drop_rp : 0.f;
            pv1 = k1 ? p1 * a.drop_rp : 0.f;
            dp0 = k0 ? dp0 * a.drop_rp : 0.f;
            dp1 = k1 ? dp1 * a.drop_rp : 0.f;
          }
          if constexpr (DO_V) wp[e2] = Mma<T>::pack2(pv0, pv1);
          if constexpr (DO_K) {
            if constexpr (DELTA_INIT) wd[e2] = Mma<T>::pack2(p0 * dp0, p1 * dp1);
            else wd[e2] = Mma<T>::pack2(p0 * (dp0 + d0), p1 * (dp1 + d1));
          }
        }
        pb[t] = __builtin_bit_cast(s16x8, wp);
        dsb[t] = __builtin_bit_cast(s16x8, wd);
      }
      // dV^T += dO^T P,  dK^T += Q^T dS   (contraction over the 32 query rows of this block)
      {
        // transposed dO / Q fragments are fetched RT - 1 steps ahead of their MFMAs (a ring of RT slots; step = (t, mb))
        auto tfrag = [&](const unsigned char* tile, int i) {
          const int ro = (32 * qbk + 16 * (i / MB)) * ROWB;
          const s16x4 lo = lds_read_tr(tile + taddr[0][i % MB] + ro);
          const s16x4 hi = lds_read_tr(tile + taddr[1][i % MB] + ro);
          return s16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        };
        constexpr int RT = FA_RT(DO_K, DO_V) < 2 * MB ? FA_RT(DO_K, DO_V) : 2 * MB;
        s16x8 dav[RT], qav[RT];
#pragma unroll
        for (int i = 0; i < RT - 1; ++i) {
          if constexpr (DO_V) dav[i] = tfrag(dt, i);
          if constexpr (DO_K) qav[i] = tfrag(qt, i);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 2 * MB; ++i) {
          if (i + RT - 1 < 2 * MB) {
            if constexpr (DO_V) dav[(i + RT - 1) % RT] = tfrag(dt, i + RT - 1);
            if constexpr (DO_K) qav[(i + RT - 1) % RT] = tfrag(qt, i + RT - 1);
          }
          if constexpr (DO_V) dv[i % MB] = Mma<T>::m32(dav[i % RT], pb[i / MB], dv[i % MB]);
          if constexpr (DO_K) dk[i % MB] = Mma<T>::m32(qav[i % RT], dsb[i / MB], dk[i % MB]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  }

  // dK and dV go out through LDS like the forward's O: staged per wavefront (its 32 key rows, row stride padded by 16
  // bytes), then stored as whole rows.  One staging area per wavefront serves dK, then dV (LDS operations of a
  // wavefront run in order).
  __syncthreads();  // every wavefront is done with the Q / dO buffers of the last tile
  {
    constexpr int OSTR = ROWB + 16;
    unsigned char* stage = smem + wave * (32 * OSTR);
    constexpr int RPS = 64 / CPR;  // rows per store instruction
    const int sr = lane / CPR, sch = lane % CPR;
    const int rows_left = Lk - (n0 + 32 * wave);
    const float sc = a.scale;
    auto flush = [&](unsigned char* base, int64_t row_stride) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < 32 / RPS; ++i) {
        const int r = i * RPS + sr;
        const u32x4 x = *(const u32x4*)(stage + r * OSTR + sch * 16);
        if (r < rows_left && sch * 8 < D) *(u32x4*)(base + (int64_t)r * row_stride + sch * 16) = x;
      }
    };
    if constexpr (DO_K) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) {
          u32x2 w;
          w[0] = Mma<T>::pack2(dk[mb][4 * v4 + 0] * sc, dk[mb][4 * v4 + 1] * sc);
          w[1] = Mma<T>::pack2(dk[mb][4 * v4 + 2] * sc, dk[mb][4 * v4 + 3] * sc);
          *(u32x2*)(stage + c32 * OSTR + (32 * mb + 8 * v4 + 4 * g) * 2) = w;
        }
      flush(a.dk + dkb + (int64_t)(k0 + n0 + 32 * wave) * a.dk_ss + (int64_t)hk * a.dk_sh, a.dk_ss);
    }
    if constexpr (DO_V) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) {
          u32x2 w;
          w[0] = Mma<T>::pack2(dv[mb][4 * v4 + 0], dv[mb][4 * v4 + 1]);
          w[1] = Mma<T>::pack2(dv[mb][4 * v4 + 2], dv[mb][4 * v4 + 3]);
          *(u32x2*)(stage + c32 * OSTR + (32 * mb + 8 * v4 + 4 * g) * 2) = w;
        }
      flush(a.dv + dvb + (int64_t)(k0 + n0 + 32 * wave) * a.dv_ss + (int64_t)hk * a.dv_sh, a.dv_ss);
    }
  }
}

// ---------------------------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------------------------
constexpr int64_t kMaxRowStrideBytes = fa::host::kMaxRowStrideBytes;
using fa::host::bwd_validate;
using fa::host::bwd_ws_bytes;
using fa::host::bwd_ws_plane;

template <typename T, int DP, bool DROP, bool BIAS>
int bwd_launch(const BArgs& a, hipStream_t st) {
  constexpr int lds_dq = 4 * 64 * DP * 2;
  constexpr int lds_dkv = 4 * 64 * DP * 2 + 4 * 256;
  constexpr bool split = DP > 64;  // head_dim 128: dK and dV as two launches
  constexpr auto kq = fa_bwd_dq_kernel<T, DP, DROP, BIAS ? 1 : 0>;
  // the dQ kernel can fetch 16-byte pieces of bias rows by DMA when every row starts 16-byte aligned and no piece
  // straddles the end of a row
  constexpr bool can_stage = BIAS && !DROP && DP <= 128;
  constexpr auto kq2 = fa_bwd_dq_kernel<T, DP, DROP, can_stage ? 2 : (BIAS ? 1 : 0)>;
  constexpr int lds_dq2 = lds_dq + 4 * 4096;
  const bool staged = can_stage && !a.cu_q && a.seqlen_k % 8 == 0 && (uintptr_t)a.bias % 16 == 0 && a.bias_sb % 16 == 0 &&
                      a.bias_sh % 16 == 0 && a.bias_sq % 16 == 0 && a.bias_sq <= kMaxRowStrideBytes;
  if (staged && !ensure_dynamic_lds<kq2>(lds_dq2)) return FA_ERR_LAUNCH;
  constexpr auto kkv = fa_bwd_dkv_kernel<T, DP, split ? kDK : (kDK | kDV), DROP, BIAS>;
  constexpr auto kv2 = fa_bwd_dkv_kernel<T, DP, kDV, DROP, BIAS>;
  if (!ensure_dynamic_lds<kq>(lds_dq) || !ensure_dynamic_lds<kkv>(lds_dkv) || (split && !ensure_dynamic_lds<kv2>(lds_dkv)))
    return FA_ERR_LAUNCH;
  const int64_t gq = (int64_t)a.batch * a.heads_q * a.n_qslot;
  const int64_t gk = (int64_t)a.batch * a.heads_k * a.n_kslot;
  if (gq > 0x7fffffffLL || gk > 0x7fffffffLL) return FA_ERR_UNSUPPORTED;
  if (gq > 0) {
    if (staged) hipLaunchKernelGGL(kq2, dim3((unsigned)gq), dim3(256), lds_dq2, st, a);
    else hipLaunchKernelGGL(kq, dim3((unsigned)gq), dim3(256), lds_dq, st, a);
    if (hipGetLastError() != hipSuccess) return FA_ERR_LAUNCH;
  }
  if (gk > 0) {
    hipLaunchKernelGGL(kkv, dim3((unsigned)gk), dim3(256), lds_dkv, st, a);
    if (hipGetLastError() != hipSuccess) return FA_ERR_LAUNCH;
    if (split) {
      hipLaunchKernelGGL(kv2, dim3((unsigned)gk), dim3(256), lds_dkv, st, a);
      if (hipGetLastError() != hipSuccess) return FA_ERR_LAUNCH;
    }
  }
  return FA_OK;
}

template <typename T, int DP>
int bwd_dispatch_dp(const BArgs& a, hipStream_t st, bool drop, bool bias) {
  if (drop && bias) return bwd_launch<T, DP, true, true>(a, st);
  if (drop) return bwd_launch<T, DP, true, false>(a, st);
  if (bias) return bwd_launch<T, DP, false, true>(a, st);
  return bwd_launch<T, DP, false, false>(a, st);
}

template <typename T>
int bwd_dispatch(const BArgs& a, hipStream_t st, int dp, bool drop, bool bias) {
  if (dp == 64) return bwd_dispatch_dp<T, 64>(a, st, drop, bias);
  if (dp == 128) return bwd_dispatch_dp<T, 128>(a, st, drop, bias);
  return bwd_dispatch_dp<T, 256>(a, st, drop, bias);
}

}  // namespace

extern "C" {

int fa_bwd_validate(const fa_bwd_params* p) { return bwd_validate(p); }

size_t fa_bwd_workspace_bytes(const fa_bwd_params* p) {
  if (bwd_validate(p) != FA_OK) return 0;
  return bwd_ws_bytes(p);
}

int fa_bwd_launch(const fa_bwd_params* p, void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = bwd_validate(p);
  if (rc != FA_OK) return rc;
  const size_t need = bwd_ws_bytes(p);
  if (need > 0 && (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 15))) return FA_ERR_BAD_ARG;
  BArgs a;
  a.q = (const unsigned char*)p->q; a.k = (const unsigned char*)p->k; a.v = (const unsigned char*)p->v;
  a.o = (const unsigned char*)p->out; a.dout = (const unsigned char*)p->dout; a.lse = p->lse;
  a.dq = (unsigned char*)p->dq; a.dk = (unsigned char*)p->dk; a.dv = (unsigned char*)p->dv;
  a.delta = (float*)workspace;
  a.lse2 = (float*)((unsigned char*)workspace + bwd_ws_plane(p));
  a.cu_q = p->cu_seqlens_q; a.cu_k = p->cu_seqlens_k;
  a.q_sb = p->q_stride_b * 2; a.q_ss = p->q_stride_s * 2; a.q_sh = p->q_stride_h * 2;
  a.k_sb = p->k_stride_b * 2; a.k_ss = p->k_stride_s * 2; a.k_sh = p->k_stride_h * 2;
  a.v_sb = p->v_stride_b * 2; a.v_ss = p->v_stride_s * 2; a.v_sh = p->v_stride_h * 2;
  a.o_sb = p->o_stride_b * 2; a.o_ss = p->o_stride_s * 2; a.o_sh = p->o_stride_h * 2;
  a.do_sb = p->do_stride_b * 2; a.do_ss = p->do_stride_s * 2; a.do_sh = p->do_stride_h * 2;
  a.dq_sb = p->dq_stride_b * 2; a.dq_ss = p->dq_stride_s * 2; a.dq_sh = p->dq_stride_h * 2;
  a.dk_sb = p->dk_stride_b * 2; a.dk_ss = p->dk_stride_s * 2; a.dk_sh = p->dk_stride_h * 2;
  a.dv_sb = p->dv_stride_b * 2; a.dv_ss = p->dv_stride_s * 2; a.dv_sh = p->dv_stride_h * 2;
  a.lse_sb = p->lse_stride_b; a.lse_sh = p->lse_stride_h; a.lse_ss = p->lse_stride_s;
  if (p->cu_seqlens_q) {
    a.dl_sb = 0; a.dl_sh = p->total_q;
  } else {
    a.dl_sb = (int64_t)p->heads_q * p->seqlen_q; a.dl_sh = p->seqlen_q;
  }
  a.batch = p->batch; a.heads_q = p->heads_q; a.heads_k = p->heads_k; a.group = p->heads_q / p->heads_k;
  a.seqlen_q = p->seqlen_q; a.seqlen_k = p->seqlen_k; a.head_dim = p->head_dim;
  a.is_causal = p->is_causal != FA_MASK_NONE ? 1 : 0;
  a.causal_tl = p->is_causal == FA_MASK_CAUSAL_TOP_LEFT ? 1 : 0;
  a.bias = (const unsigned char*)p->bias;
  a.bias_sb = p->bias_stride_b * 2; a.bias_sh = p->bias_stride_h * 2; a.bias_sq = p->bias_stride_q * 2;
  a.dbias = (unsigned char*)p->dbias;
  a.dbias_sb = p->dbias_stride_b * 2; a.dbias_sh = p->dbias_stride_h * 2; a.dbias_sq = p->dbias_stride_q * 2;
  a.n_qslot = (p->seqlen_q + 127) / 128;
  a.n_kslot = (p->seqlen_k + 127) / 128;
  a.blockmajor_q = a.is_causal && (int64_t)p->batch * p->heads_q * a.n_qslot < 8 * 256;
  a.blockmajor_k = a.is_causal && (int64_t)p->batch * p->heads_k * a.n_kslot < 8 * 256;
  a.hgroup_q = a.hgroup_k = 1;
  if (p->bias && !p->cu_seqlens_q && p->bias_stride_h == 0) {
    for (int gsz = FA_HGROUP; gsz > 1 && a.hgroup_q == 1; gsz >>= 1)
      if (p->heads_q % gsz == 0) a.hgroup_q = gsz;
    for (int gsz = FA_HGROUP; gsz > 1 && a.hgroup_k == 1; gsz >>= 1)
      if (p->heads_k % gsz == 0) a.hgroup_k = gsz;
  }
  a.scale = p->scale;
  a.scale_log2 = p->scale * kLog2e;
  if (a.scale_log2 == 0.f) a.scale_log2 = 1e-30f;  // scale 0: uniform probabilities, and -inf * c stays -inf
  const float p_keep = 1.f - p->dropout_p;
  a.drop_thr = (uint32_t)floorf(p_keep * 255.f);
  a.drop_rp = 256.f / (float)(a.drop_thr + 1u);  // the reciprocal of the keep probability the mask realises
  a.seed_ptr = p->philox_seed;
  a.offset_ptr = p->philox_offset;
  hipStream_t st = (hipStream_t)stream;
  const int dp = p->head_dim <= 64 ? 64 : (p->head_dim <= 128 ? 128 : 256);
  const bool drop = p->dropout_p > 0.f, bias = p->bias != nullptr;
  if (p->dtype == FA_DTYPE_BF16) return bwd_dispatch<__bf16>(a, st, dp, drop, bias);
  return bwd_dispatch<_Float16>(a, st, dp, drop, bias);
}

}  // extern "C"
