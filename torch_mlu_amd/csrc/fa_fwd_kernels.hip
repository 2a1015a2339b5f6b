// Flash-attention forward for MI355X (gfx950): HIP kernels and the C-ABI launcher declared in include/fa_fwd.h.
//
// Replaces the single vendor call cnnlFlashAttentionForward_v2 that torch_mlu's launcher makes
// (torch_mlu/csrc/aten/operators/cnnl/internal/FlashAttention_internal.cpp:231-258) together with its
// descriptor / workspace plumbing (:131-230).
//
// Two kernels:
//   fa_tile_kernel     — MFMA-bound.  One workgroup (4 wavefronts) owns 128 query rows of one (sequence, head);
//                        each wavefront keeps its 32 query rows in registers as the B operand of
//                        v_mfma_f32_32x32x16 and computes S^T = K Q^T, so one lane owns one query row's scores
//                        (row max / row sum need a single cross-lane exchange) and P^T is already in B-operand
//                        layout for O^T += V^T P^T.  K/V tiles of 64 rows are double-buffered in LDS by
//                        global->LDS DMA (16 bytes per lane, no staging registers); V^T fragments come from
//                        ds_read_b64_tr_b16.  Causal and ragged (cu_seqlens) work is handled by the tile
//                        scheduler: heavy tiles first, fully masked tiles skipped, partially masked tiles masked.
//   fa_splitkv_kernel  — HBM-bound single-query (decode) shape.  One workgroup owns a contiguous slice of one
//                        (sequence, kv head); every wavefront streams its own 32-row K/V blocks through a private
//                        two-stage LDS ring by global->LDS DMA (no workgroup barriers in the loop), serves all
//                        query heads of the GQA group from one pass over K/V with v_mfma_f32_16x16x32, and the
//                        partial (m, l, o) triples are merged in LDS and, across slices, by fa_merge_rows_kernel.
//
// All arithmetic is bf16/fp16 inputs, fp32 accumulate and fp32 softmax in the exp2 domain
// (the reference asks the vendor kernel for compute_dtype = FLOAT, HIGH_PRECISION: :147-148).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "fa_device.h"
#include "fa_fwd.h"
#include "fa_fwd_common.h"
#include "fa_host.h"

#ifndef FA_HGROUP
#define FA_HGROUP 4
#endif
namespace {

using namespace fa;

// ---------------------------------------------------------------------------------------------------------
// Tile kernel
// ---------------------------------------------------------------------------------------------------------
// BIAS = 1: an additive bias tile is read straight from global memory into the score layout (one lane = one query
// row, groups of 4 consecutive keys = 8 bytes) and the softmax then runs on scores already in the log2 domain.
// BIAS = 2: the same, but the tile is fetched by DMA into LDS one tile ahead (16-byte pieces, so rows must be 16-byte
// aligned and seqlen_k a multiple of 8) and read from there: the loads of mode 1 are issued only 16 MFMAs before
// their use, which leaves most of an L2 miss exposed.
// DROP: dropout on the probabilities.  The row sums (and LSE) are those of the undropped probabilities; dropped
// entries are zeroed in the P operand of the PV product and 1 / (keep probability) is folded into the final normalisation.
// DMASK (with DROP): also write the keep-mask out for tests; a variant of its own because the extra stores cost
// registers (30 spilled at head_dim 128) that the plain dropout kernel does not have to pay.
// PAGED: K and V are pools of pages [page][row][kv head][D] (dense mode; a.k_sb / a.v_sb are the page strides) and key
// row r of sequence b lives in page block_table[b][r / page_size]: a prefill chunk against a paged KV cache.  A DMA
// instruction covers at most 32 consecutive rows that start at a multiple of its length and page_size is a multiple
// of 32, so the rows of one instruction lie inside one page.
template <typename T, int DP, int MINB, int BIAS, bool DROP = false, bool DMASK = false, bool PAGED = false>
__global__ void __launch_bounds__(256, MINB) fa_tile_kernel(const KArgs a) {
  constexpr int CPR = DP / 8;          // 16-byte chunks per row
  constexpr int ROWB = DP * 2;         // bytes per LDS row
  constexpr int BM = 128, BN = 64;
  constexpr int TILE = BN * ROWB;      // bytes per K (or V) tile
  constexpr int NI = TILE / 1024 / 4;  // DMA instructions per wavefront per tile
  constexpr int RPI = 64 / CPR;        // rows covered by one DMA instruction
  constexpr int KS = DP / 16;          // MFMA k-steps over the head dim
  constexpr int MB = DP / 32;          // 32-row blocks of O^T
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];  // K0 K1 V0 V1

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, c32 = lane & 31;

  // ---- which (sequence, head, query block): XCD-aware, heavy blocks first -------------------------------
  // Dense: workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous range of logical ids so that
  // all query blocks of one (sequence, kv head) share that XCD's L2.  Packed (ragged lengths, known only on the
  // device): causal calls that can pair blocks search their pair below; the others go block-major, i.e. the last
  // (heaviest) blocks of all sequences first and sequences shorter than that exit at once.
  int lid = blockIdx.x;
  int pslot, bh;
  // Sliced mode (few query blocks against a long K/V: chunked prefill, speculative decoding): workgroup
  // `split` of n_splits takes a contiguous range of a block's tiles and leaves unnormalised partials (m, l, O) in
  // the workspace, which fa_merge_rows_kernel combines.
  int split = 0;
  int pk_blk = -1;  // packed, paired: the heavy block of this workgroup's pair
  if (a.cu_q && a.pair) {
    // Packed and causal, lengths known only here: every workgroup finds its own work.  A sequence of n blocks is cut
    // into (n + 1) / 2 pairs (n-1-p, p), which all cost the same, about n + 1 tiles.  The sequences are taken longest
    // first (so the short ones fill the end of the launch), and within a sequence the pairs of 8 kv heads (all query
    // heads of their groups) form one run of consecutive workgroups, kv head fastest: consecutive workgroups go to
    // the 8 XCDs in turn, so everything that reads one (sequence, kv head) lands on one XCD at about the same time
    // and shares its L2 for K and V.  One lane per sequence
    // (at most 64, checked by the launcher) works out its rank and where its run of workgroups starts; the
    // workgroups beyond the last pair are the last ones of the grid and exit.
    int nb = 0;
    if (lane < a.batch) nb = (a.cu_q[lane + 1] - a.cu_q[lane] + BM - 1) / BM;
    const int np = (nb + 1) >> 1;  // pairs of this lane's sequence
    int start = 0;                 // pairs of the sequences that come before it
    for (int o = 0; o < a.batch; ++o) {
      const int nbo = __builtin_amdgcn_readlane(nb, o);
      const bool first = nbo > nb || (nbo == nb && o < lane);
      start += first ? (nbo + 1) >> 1 : 0;
    }
    const int H = a.heads_q;
    const bool mine = lane < a.batch && lid >= start * H && lid < (start + np) * H;
    const uint64_t sel = __builtin_amdgcn_ballot_w64(mine);
    bh = -1;
    if (sel != 0) {
      const int sb = __builtin_ctzll(sel);
      const int np_b = __builtin_amdgcn_readlane(np, sb);
      const int r = lid - __builtin_amdgcn_readlane(start, sb) * H;
      int hh, pp;
      if ((a.heads_k & 7) == 0) {
        const int run = 8 * a.group * np_b;  // workgroups of 8 kv heads: (pair, head of the group) x 8 kv heads
        const int t = (r % run) >> 3;
        hh = ((r / run) * 8 + (r & 7)) * a.group + t % a.group;
        pp = t / a.group;
      } else {
        hh = r % H;
        pp = r / H;
      }
      bh = sb * H + hh;
      pk_blk = __builtin_amdgcn_readlane(nb, sb) - 1 - pp;
    }
    if (bh < 0) return;
    pslot = 0;
  } else if (a.cu_q) {
    if (a.n_splits > 1) {
      split = lid % a.n_splits;
      lid /= a.n_splits;
    }
    const int nbh = a.batch * a.heads_q;
    pslot = lid / nbh;
    bh = lid % nbh;
  } else {
    const int total = gridDim.x, per = total >> 3;
    if (lid < (per << 3)) lid = (lid & 7) * per + (lid >> 3);
    if (a.n_splits > 1) {
      split = lid % a.n_splits;
      lid /= a.n_splits;
    }
    if (BIAS && a.hgroup > 1) {
      // a bias broadcast over heads: the same query block of hgroup heads runs side by side, so that one fetch of a
      // bias tile serves all of them from L2 (at the price of fewer query blocks of a head sharing its K/V)
      const int span = a.hgroup * a.n_mblk;
      const int r = lid % span;
      pslot = r / a.hgroup;
      bh = (lid / span) * a.hgroup + r % a.hgroup;
    } else {
      pslot = lid % a.n_mblk;  // a.n_mblk: workgroups per (sequence, head)
      bh = lid / a.n_mblk;
    }
  }
  const int h = bh % a.heads_q, b = bh / a.heads_q;
  const int hk = h / a.group;
  uint32_t drop_key = 0, drop_key2 = 0;
  if constexpr (DROP) {
    // the two numbers of the mask: by value, or (a launch recorded into a graph) read now from the generator's state
    const uint64_t seed = a.seed_ptr ? (uint64_t)*a.seed_ptr : a.seed;
    const uint64_t offset = a.offset_ptr ? (uint64_t)*a.offset_ptr + a.offset : a.offset;
    const DropKeys dk = drop_head_keys(seed, offset, (uint32_t)bh);
    drop_key = dk.k1;
    drop_key2 = dk.k2;
    if (blockIdx.x == 0 && tid == 0) {
      if (a.rng_seed_out) *a.rng_seed_out = (int64_t)seed;
      if (a.rng_offset_out) *a.rng_offset_out = (int64_t)offset;
    }
  }

  int q0 = 0, k0 = 0, Lq = a.seqlen_q, Lk = a.seqlen_k;
  int64_t qb = (int64_t)b * a.q_sb, kb = (int64_t)b * a.k_sb, vb = (int64_t)b * a.v_sb, ob = (int64_t)b * a.o_sb;
  int64_t lb = (int64_t)b * a.lse_sb;
  if (a.cu_q) {
    q0 = a.cu_q[b];
    Lq = a.cu_q[b + 1] - q0;
    k0 = a.cu_k[b];
    Lk = a.cu_k[b + 1] - k0;
    qb = kb = vb = ob = 0;
    lb = 0;
  }
  if (a.seqused_k) Lk = min(Lk, max(a.seqused_k[b], 0));
  // query blocks owned by this workgroup: paired (causal, dense) -> the heavy block nblk-1-p and the light block p,
  // so that every workgroup of a sequence has the same number of tiles; unpaired -> one block, heavy blocks first
  // (packed: counted down from the longest possible sequence so that equal slots mean equal block indices)
  const int nblk = (Lq + BM - 1) / BM;
  const int blk_first = pk_blk >= 0 ? pk_blk : (a.cu_q ? a.n_mblk : nblk) - 1 - pslot;
  const int blk_second = pk_blk >= 0 ? nblk - 1 - pk_blk : pslot;
  if (pk_blk < 0 && (a.pair ? (2 * pslot >= nblk) : (blk_first < 0 || blk_first >= nblk))) return;
  const int n_own = (DP != 256 && a.pair && blk_first != blk_second) ? 2 : 1;  // head_dim 256 never pairs (registers)
  const int off = a.causal_tl ? 0 : Lk - Lq;  // causal: col visible iff col <= row + off

  const unsigned char* qp = a.q + qb + (int64_t)q0 * a.q_ss + (int64_t)h * a.q_sh;
  // (PAGED: the pools' first page, this kv head; the page is added per DMA instruction)
  const unsigned char* kp = a.k + (PAGED ? 0 : kb + (int64_t)k0 * a.k_ss) + (int64_t)hk * a.k_sh;
  const unsigned char* vp = a.v + (PAGED ? 0 : vb + (int64_t)k0 * a.v_ss) + (int64_t)hk * a.v_sh;
  const int D = a.head_dim;

  // ---- DMA bookkeeping ---------------------------------------------------------------------------------
  // DMA instruction i of this wavefront fills LDS rows dma_r + 4 RPI i (one 1 KiB block).  The global address is
  // a wavefront-uniform base (tile start + 4 RPI i rows, scalar registers) plus a per-lane byte offset that does
  // not change from tile to tile, so a full tile costs no vector ALU work; only the last, partial tile clamps
  // rows per lane.  head_dim < DP: pad chunks are pointed at chunk 0 (valid memory); they meet zeros of Q / are
  // never stored.  The swizzles only use row bits that the per-instruction row step leaves alone, except swzK at
  // DP == 256 where odd instructions toggle bit 3.
  const int dma_r = wave * RPI + lane / CPR;
  const int dma_pc = lane % CPR;
  int lck = dma_pc ^ swzK<DP>(dma_r);
  int lck_odd = (DP == 256) ? (lck ^ 8) : lck;
  int lcv = dma_pc ^ swzV<DP>(dma_r);
  if (lck * 8 >= D) lck = 0;
  if (lck_odd * 8 >= D) lck_odd = 0;
  if (lcv * 8 >= D) lcv = 0;
  const unsigned k_ss = (unsigned)a.k_ss, v_ss = (unsigned)a.v_ss;
  const unsigned koff = (unsigned)dma_r * k_ss + lck * 16;
  const unsigned koff_odd = (unsigned)dma_r * k_ss + lck_odd * 16;
  const unsigned voff = (unsigned)dma_r * v_ss + lcv * 16;
  const int last_k = Lk - 1;
  const unsigned lds0 = (unsigned)(uintptr_t)(LDS_AS unsigned char*)smem + wave * 1024;

  // PAGED: the pages of a tile's two 32-row halves and the halves' first rows inside their pages.  The table entries
  // are scalar loads; they are requested two tiles ahead of the DMA that needs them (page_next: tile j + 1 while tile
  // j is computed, page_after: tile j + 2), walking the table with a running (entry, row) pair instead of a division.
  struct PageRef {
    int pg0, pg1, ro0, ro1;
  };
  const int32_t* tbl = nullptr;
  int psz = 32, lk_idx = 0, lk_ro = 0, lk_max = 0;
  if constexpr (PAGED) {
    tbl = a.block_table + (int64_t)b * a.bt_stride;
    psz = a.page_size;
    lk_max = max(last_k, 0) / psz;  // the last entry that belongs to this sequence's keys
  }
  auto lookup_seek = [&](int j) {  // the next lookup is tile j's
    lk_idx = (j * BN) / psz;
    lk_ro = j * BN - lk_idx * psz;
  };
  auto lookup_next = [&]() -> PageRef {
    int i1 = lk_idx, o1 = lk_ro + 32;
    if (o1 >= psz) {
      o1 -= psz;
      ++i1;
    }
    // (wavefront-uniform by construction; said so, since the DMA's base address must live in scalar registers)
    const PageRef r{__builtin_amdgcn_readfirstlane(tbl[min(lk_idx, lk_max)]),
                    __builtin_amdgcn_readfirstlane(tbl[min(i1, lk_max)]), __builtin_amdgcn_readfirstlane(lk_ro),
                    __builtin_amdgcn_readfirstlane(o1)};
    lk_ro += BN;
    while (lk_ro >= psz) {
      lk_ro -= psz;
      ++lk_idx;
    }
    return r;
  };
  PageRef page_next{0, 0, 0, 0}, page_after{0, 0, 0, 0};
  // One DMA instruction of a tile that lies fully inside the sequence: `which` = 0 (K) or 1 (V), block i of tile j
  // into buffer buf.  Only scalar address arithmetic.  These are issued one at a time between MFMAs so that a
  // wavefront never sits in the (narrow, CU-shared) vector-memory issue queue with nothing else to do.
  auto issue_one = [&](int j, int buf, int which, int i, const PageRef& pr) {
    const unsigned dst = lds0 + (which ? 2 * TILE : 0) + buf * TILE + i * 4096;
    const unsigned ss = which ? v_ss : k_ss;
    const unsigned char* base;
    if constexpr (PAGED) {
      const bool hi = i * 4 * RPI >= 32;  // which half of the tile this instruction's rows are in
      const int64_t sb = which ? a.v_sb : a.k_sb;
      base = (which ? vp : kp) + (int64_t)(hi ? pr.pg1 : pr.pg0) * sb +
             (uint64_t)(unsigned)((hi ? pr.ro1 : pr.ro0) + (i * 4 * RPI) % 32) * ss;
    } else {
      base = (which ? vp : kp) + (uint64_t)(unsigned)(j * BN + i * 4 * RPI) * ss;
    }
    dma16s(base, which ? voff : ((DP == 256 && (i & 1)) ? koff_odd : koff), dst);
  };
  // A whole tile at once, rows clamped to the last valid one (first tile, and the partial tile at the end of K).
  auto issue_tile = [&](int j, int buf) {
    if constexpr (PAGED) {
      // per lane: its (clamped) row's page from the table, then a 64-bit address
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int r = min(j * BN + dma_r + i * 4 * RPI, last_k);
        const int e = r / psz;
        const int64_t pg = tbl[e];
        const unsigned ro = (unsigned)(r - e * psz);
        dma16v(kp + pg * a.k_sb + (uint64_t)ro * k_ss + ((DP == 256 && (i & 1)) ? lck_odd : lck) * 16, lds0 + buf * TILE + i * 4096);
        dma16v(vp + pg * a.v_sb + (uint64_t)ro * v_ss + lcv * 16, lds0 + 2 * TILE + buf * TILE + i * 4096);
      }
      return;
    }
    const int rmax = last_k - j * BN;  // >= 0: the tile exists
    const unsigned char* kt = kp + (uint64_t)(unsigned)(j * BN) * k_ss;
    const unsigned char* vt = vp + (uint64_t)(unsigned)(j * BN) * v_ss;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const unsigned r = (unsigned)min(dma_r + i * 4 * RPI, rmax);
      dma16s(kt, r * k_ss + ((DP == 256 && (i & 1)) ? lck_odd : lck) * 16, lds0 + buf * TILE + i * 4096);
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const unsigned r = (unsigned)min(dma_r + i * 4 * RPI, rmax);
      dma16s(vt, r * v_ss + lcv * 16, lds0 + 2 * TILE + buf * TILE + i * 4096);
    }
  };

  // ---- per-lane LDS read offsets (bytes from the start of a K / V tile), fixed for the whole kernel ----------
  // K fragment for k-step ks: rows c32 and 32 + c32 (same swizzle), logical chunk 2 ks + g
  int kaddr[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) kaddr[ks] = c32 * ROWB + (((2 * ks + g) ^ swzK<DP>(c32)) * 16);
  // V^T fragment for (mb, t, half): row 16 t + 8 half + 4 g + (L >> 2), logical chunk 4 mb + 2 (G & 1) + ((L & 3) >> 1)
  const int L = lane & 15, G = lane >> 4;
  const int v_row = 4 * g + (L >> 2);
  int vaddr[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
    vaddr[mb] = v_row * ROWB + (L & 1) * 8 + (((4 * mb + 2 * (G & 1) + ((L & 3) >> 1)) ^ swzV<DP>(v_row)) * 16);
  // The same offsets as LDS pointers held in registers (the compiler otherwise re-adds the LDS base, a link-time
  // constant it cannot fold, to every fragment address of every tile: 8 + 4 vector adds per tile); buffer and
  // row-block displacements are immediates of the read instructions.  The bias variants have no registers to spare
  // for that and keep the adds; so does head_dim 256 (measured: 2 % slower with the pointers).
  LDS_AS const unsigned char* kptr[KS];
  LDS_AS const unsigned char* vptr[MB];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    kptr[ks] = (LDS_AS const unsigned char*)smem + kaddr[ks];
    if constexpr (BIAS == 0 && DP <= 128) asm volatile("" : "+v"(kptr[ks]));
  }
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    vptr[mb] = (LDS_AS const unsigned char*)smem + 2 * TILE + vaddr[mb];
    if constexpr (BIAS == 0 && DP <= 128) asm volatile("" : "+v"(vptr[mb]));
  }
  // without a bias the scores stay raw and scale * log2(e) is folded into the exponent's FMA; with one they become
  // scale * s + bias when the bias is added, and the factor from there on is log2(e)
  const float c = BIAS ? kLog2e : a.scale_log2;
  const float lazy = kLazyLog2 / c;  // threshold in score units

  for (int own = 0; own < n_own; ++own) {
  const int m0 = (own == 0 ? blk_first : blk_second) * BM;
  int n_end = Lk;
  if (a.is_causal) n_end = min(Lk, m0 + BM + off);
  if (n_end < 0) n_end = 0;
  const int ntiles_all = (n_end + BN - 1) / BN;
  int jt0 = 0, ntiles = ntiles_all;  // this workgroup's tiles: [jt0, ntiles)
  if (a.n_splits > 1) {
    const int per_split = (ntiles_all + a.n_splits - 1) / a.n_splits;
    jt0 = split * per_split;
    ntiles = min(ntiles_all, jt0 + per_split);
  }
  const int row = m0 + 32 * wave + c32;  // this lane's query row (lanes l and l^32 share it)
  if (own) __syncthreads();  // the previous block's last LDS reads are done
  if (ntiles > jt0) issue_tile(jt0, 0);
  if constexpr (PAGED) {
    if (ntiles > jt0) {
      lookup_seek(jt0 + 1);
      page_next = lookup_next();
      page_after = lookup_next();
    }
  }

  // ---- Q fragments (B operand): lane (c32, g) holds Q[row][16 ks + 8 g .. +8] -----------------------------
  // The block's 128 rows come in through LDS like two K tiles (rows 0-63 into K buffer 1, rows 64-127 into V buffer
  // 1, same swizzle, whole rows per DMA instruction; rows beyond the sequence repeat its last row) and each lane
  // picks its fragments up from there: loading them straight from global memory takes 16 bytes from each of 32 rows
  // per instruction, measured at 3.7 us per block.
  s16x8 qf[KS];
  {
    const unsigned char* qt = qp + (int64_t)m0 * a.q_ss;
    const int rmaxq = Lq - 1 - m0;  // >= 0: the block exists
    const unsigned q_ss = (unsigned)a.q_ss;
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const unsigned r = (unsigned)min(64 * half + dma_r + i * 4 * RPI, rmaxq);
        dma16s(qt, r * q_ss + ((DP == 256 && (i & 1)) ? lck_odd : lck) * 16, lds0 + (half ? 3 * TILE : TILE) + i * 4096);
      }
    WAIT_VMCNT(0);
    __syncthreads();
    const unsigned char* qs = smem + ((wave >> 1) ? 3 * TILE : TILE) + (wave & 1) * 32 * ROWB;
    const unsigned flip = a.neg_scale ? 0x80008000u : 0u;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 x = *(const u32x4*)(qs + kaddr[ks]);
      if ((2 * ks + g) * 8 >= D) x = u32x4{0, 0, 0, 0};  // pad chunks hold a copy of chunk 0
      x ^= flip;
      qf[ks] = __builtin_bit_cast(s16x8, x);
    }
    // the fragments are in registers before any wavefront passes the first tile's barrier and sends the second
    // tile into these two buffers
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }

  f32x16 o[MB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[i][v] = 0.f;
  float m_run = -INFINITY, l_run = 0.f, mc_run = 0.f;

  const int causal_row_lim = a.is_causal ? row + off : 0x7fffffff;
  const int wave_row_lo = m0 + 32 * wave, wave_row_hi = wave_row_lo + 31;
  // dropout: key ^ row term of this lane's row pair, and which half of a patch word belongs to this row
  const uint32_t drop_row = DROP ? (drop_key ^ drop_row_term((uint32_t)row >> 1)) : 0u;
  const int drop_sh = 16 * (row & 1);
  // v_perm_b32 selector: bytes 2 (row & 1) and 2 (row & 1) + 1 of a word into the low bytes of the two halves
  const uint32_t drop_sel = 0x0c000c00u | (uint32_t)(2 * (row & 1)) | ((uint32_t)(2 * (row & 1) + 1) << 16);
  const uint32_t drop_thr2 = a.drop_thr | (a.drop_thr << 16);
  const unsigned char* brow = nullptr;  // this lane's bias row, at its first key group (4 g)
  unsigned char* drow = nullptr;  // this lane's row of the debug mask
  if constexpr (DROP && DMASK)
    if (a.dmask) drow = a.dmask + (((int64_t)b * a.heads_q + h) * a.seqlen_q + min(row, min(Lq, a.seqlen_q) - 1)) * (int64_t)a.seqlen_k * 2;
  if constexpr (BIAS == 1)
    brow = a.bias + (int64_t)b * a.bias_sb + (int64_t)h * a.bias_sh + (int64_t)min(row, Lq - 1) * a.bias_sq + 8 * g;
  // BIAS == 2: this wavefront's 32 rows x 64 keys of the bias tile (4 KiB) go through a private LDS area by DMA, one
  // tile ahead.  DMA instruction i brings rows 8 i .. 8 i + 7; lane l fetches 16 bytes (8 keys): row 8 i + l / 8, key
  // chunk (l % 8) ^ (l / 8), so that row r keeps chunk ch at r * 128 + ((ch ^ (r & 7)) * 16).
  const unsigned char* bbase = nullptr;  // wavefront-uniform: this block's first bias row
  unsigned boff[BIAS == 2 ? 4 : 1];      // per-lane byte offsets of the four DMA instructions
  const int bchunk = (lane & 7) ^ (lane >> 3);
  const unsigned blds = lds0 - wave * 1024 + 4 * TILE + wave * 4096;  // LDS byte address of this wavefront's area
  int baddr = 0;  // per-lane LDS read offset of key chunk 0; chunk ch is at baddr ^ (ch * 16)
  if constexpr (BIAS == 2) {
    bbase = a.bias + (int64_t)b * a.bias_sb + (int64_t)h * a.bias_sh + (int64_t)m0 * a.bias_sq;
    const int rmax = Lq - 1 - m0;  // >= 0
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
    if (ntiles > jt0) issue_bias(jt0);

  auto tile = [&](int j, auto bufc) {
    constexpr int BUF = decltype(bufc)::value;
    WAIT_VMCNT(0);       // my DMA for tile j has landed
    __syncthreads();     // everyone's has; everyone is done reading the other buffer
    // next tile: fully inside K -> its DMA instructions are interleaved with this tile's MFMAs; partial -> issued here
    const bool more = j + 1 < ntiles;
    const bool spread = more && (j + 2) * BN <= Lk && !(a.is_causal && j * BN > wave_row_hi + off);
    if (more && !spread) issue_tile(j + 1, BUF ^ 1);
    const PageRef pages = page_next;  // (PAGED) of tile j + 1
    if constexpr (PAGED) {
      page_next = page_after;
      page_after = lookup_next();  // tile j + 3
    }

    // wavefront-uniform skip: every score of this tile is masked for all 32 rows of this wavefront
    if (a.is_causal && j * BN > wave_row_hi + off) return;


    // bias of a full tile: 8 loads of 4 keys each, issued now and consumed after the S MFMAs
    const bool full_tile = j * BN + BN <= Lk;
    u32x2 braw[BIAS ? 8 : 1];
    if constexpr (BIAS == 1) {
      if (full_tile) {
        const unsigned char* bt = brow + (int64_t)j * (BN * 2);
#pragma unroll
        for (int i = 0; i < 8; ++i) braw[i] = *(const u32x2*)(bt + (32 * (i >> 2) + 8 * (i & 3)) * 2);
      }
    }

    // ---- S^T = K Q^T : two 32(kv) x 32(q) blocks; K fragments are fetched two k-steps ahead of their MFMAs ----
    f32x16 s0, s1;
#pragma unroll
    for (int v = 0; v < 16; ++v) { s0[v] = 0.f; s1[v] = 0.f; }
    {
      s16x8 ka[2][2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        ka[ks][0] = *(LDS_AS const s16x8*)(kptr[ks] + BUF * TILE);
        ka[ks][1] = *(LDS_AS const s16x8*)(kptr[ks] + BUF * TILE + 32 * ROWB);
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        s0 = Mma<T>::m32(ka[ks & 1][0], qf[ks], s0);
        s1 = Mma<T>::m32(ka[ks & 1][1], qf[ks], s1);
        // next tile's K and V: 2 NI DMA instructions spread over the KS k-steps (K block i, then V block i)
        if (spread) {
#pragma unroll
          for (int x = (ks * 2 * NI) / KS; x < ((ks + 1) * 2 * NI) / KS; ++x) issue_one(j + 1, BUF ^ 1, x & 1, x >> 1, pages);
        }
        if (ks + 2 < KS) {
          ka[ks & 1][0] = *(LDS_AS const s16x8*)(kptr[ks + 2] + BUF * TILE);
          ka[ks & 1][1] = *(LDS_AS const s16x8*)(kptr[ks + 2] + BUF * TILE + 32 * ROWB);
        }
      }
    }

    // ---- bias: register v of block blk <-> key j BN + 32 blk + 8 (v >> 2) + 4 g + (v & 3); scores become
    //      scale * s + bias (natural units) ----
    if constexpr (BIAS) {
      const float cs = a.scale_abs;
      typedef T T4 __attribute__((ext_vector_type(4)));
      if (BIAS == 2 || full_tile) {
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            if constexpr (BIAS == 2) braw[4 * blk + q4] = *(const u32x2*)(smem + (baddr ^ ((4 * blk + q4) * 16)));
            const T4 bv = __builtin_bit_cast(T4, braw[4 * blk + q4]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if (blk) s1[4 * q4 + e] = s1[4 * q4 + e] * cs + (float)bv[e];
              else s0[4 * q4 + e] = s0[4 * q4 + e] * cs + (float)bv[e];
            }
          }
      } else {  // last, partial tile: element-wise, columns clamped to the last valid one (masked below anyway)
        const T* be = (const T*)(brow + (int64_t)j * (BN * 2));
        const int cmax = last_k - j * BN - 4 * g;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int e = 8 * (v >> 2) + (v & 3);
          s0[v] = s0[v] * cs + (float)be[min(e, cmax)];
          s1[v] = s1[v] * cs + (float)be[min(32 + e, cmax)];
        }
      }
    }

    // ---- mask (tail of K, causal diagonal) ----
    const bool need_mask = (j * BN + BN > Lk) || (a.is_causal && j * BN + BN - 1 > wave_row_lo + off);
    if (need_mask) {
      const int lim = min(last_k, causal_row_lim) - j * BN - 4 * g;  // element index e is visible iff e <= lim
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int e = 8 * (v >> 2) + (v & 3);
        if (e > lim) s0[v] = -INFINITY;
        if (32 + e > lim) s1[v] = -INFINITY;
      }
    }

    // ---- online softmax (one lane = one query row x 32 of the 64 columns) ----
    // The maximum is exact whatever the order: two interleaved chains per product (half the latency of one chain, and
    // fewer readers right behind their `asm` producer, each of which costs a compiler-inserted wait state).  The MFMA
    // results must not be read before the matrix pipe has written them, and the compiler only inserts that wait in
    // front of instructions it knows: the first read of each product's accumulators is therefore a canonicalize
    // (a `v_max_f32 x, x` the compiler emits itself), and every `asm` maximum of that product depends on it.
    const float g0 = __builtin_canonicalizef(s0[15]);
    float c0 = max3d(s0[0], s0[1], s0[2], g0), c1 = max3d(s0[8], s0[9], s0[10], g0);
#pragma unroll
    for (int v = 3; v < 7; v += 2) {
      c0 = max3(c0, s0[v], s0[v + 1]);
      c1 = max3(c1, s0[v + 8], s0[v + 9]);
    }
    c0 = max3(c0, s0[7], g0);
    const float g1 = __builtin_canonicalizef(s1[15]);
    float c2 = max3d(s1[0], s1[1], s1[2], g1), c3 = max3d(s1[8], s1[9], s1[10], g1);
#pragma unroll
    for (int v = 3; v < 7; v += 2) {
      c2 = max3(c2, s1[v], s1[v + 1]);
      c3 = max3(c3, s1[v + 8], s1[v + 9]);
    }
    c2 = max3(c2, s1[7], g1);
    float mx = max3(c0, c1, c2);
    mx = max2(mx, c3);
    mx = pair_max32(mx);
    if constexpr (BIAS == 2) {
      // the next tile's bias may overwrite this one now: the maximum depends on every value that was read
      asm volatile("" : : "v"(mx) : "memory");
      if (more) issue_bias(j + 1);
    }
    const bool grow = mx > m_run + lazy;  // first visible tile: m_run = -inf
    if (__builtin_amdgcn_ballot_w64(grow) != 0) {
      const float m_new = grow ? mx : m_run;
      const float alpha = grow ? fast_exp2((m_run - m_new) * c) : 1.0f;  // exp2(-inf) = 0 on the first tile
      m_run = m_new;
      mc_run = (m_run == -INFINITY) ? 0.f : m_run * c;
      l_run *= alpha;
#pragma unroll
      for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[i][v] *= alpha;
    }
    const float mc = mc_run;  // m_run c, kept alongside m_run (0 while no key has been seen)
    // dropout: counter of a patch = key ^ row term ^ column term; the column pair of this lane's groups is
    // 32 j + 2 g + a compile-time constant with disjoint bits
    const uint32_t drop_tile = DROP ? (drop_row ^ drop_col_term((uint32_t)(j * (BN / 2) + 2 * g))) : 0u;

    // ---- per 16-key chunk t: P = exp2(S c - m c), row sums, P^T as B operand, O^T += V^T P^T.  The V^T fragments
    //      of chunk t + 1 are fetched while chunk t's MFMAs run. ----
    auto vfrag = [&](int mb, int t) {
      const s16x4 lo = lds_read_tr_lds(vptr[mb] + BUF * TILE + (16 * t) * ROWB);
      const s16x4 hi = lds_read_tr_lds(vptr[mb] + BUF * TILE + (16 * t + 8) * ROWB);
      return s16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    s16x8 va[2][MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) va[0][mb] = vfrag(mb, 0);
    float rs = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      if (t + 1 < 4) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) va[(t + 1) & 1][mb] = vfrag(mb, t + 1);
      }
      u32x4 w;
#pragma unroll
      for (int e2 = 0; e2 < 4; ++e2) {
        const int v = 8 * (t & 1) + 2 * e2;
        const float x0 = (t < 2) ? s0[v] : s1[v], x1 = (t < 2) ? s0[v + 1] : s1[v + 1];
        float p0 = fast_exp2(x0 * c - mc), p1 = fast_exp2(x1 * c - mc);
        // row sums are those of the undropped probabilities, so with dropout they are taken before the mask
        constexpr bool sum_packed = Mma<T>::kSumPacked && !DROP;
        if constexpr (!sum_packed) rs += p0 + p1;
        if constexpr (DROP) {
          // keys j BN + 32 (t >> 1) + 8 (v >> 2) + 4 g + (v & 3), + 1: one column pair, one patch word
          const uint32_t cp_const = 16 * (t >> 1) + 4 * (v >> 2) + ((v & 3) >> 1);
          const uint32_t word_full = drop_word(drop_tile ^ cp_const, drop_key2);
          if constexpr (!DMASK) {
            // The pair's two bytes go to the low bytes of the two 16-bit halves (one v_perm_b32), threshold minus
            // byte is negative exactly where the element is dropped, and its sign, spread over the half by an
            // arithmetic shift, clears that half of the packed pair: 4 instructions for what compare-and-select on
            // the two floats does in 6.
            typedef short i16x2 __attribute__((ext_vector_type(2)));
            const uint32_t bytes = __builtin_amdgcn_perm(word_full, word_full, drop_sel);
            const i16x2 diff = __builtin_bit_cast(i16x2, drop_thr2) - __builtin_bit_cast(i16x2, bytes);
            const uint32_t gone = __builtin_bit_cast(uint32_t, diff >> 15);  // 0xffff per dropped half
            w[e2] = Mma<T>::pack2(p0, p1) & ~gone;
            continue;
          }
          const uint32_t word = word_full >> drop_sh;
          const bool k0 = (word & 0xffu) <= a.drop_thr, k1 = ((word >> 8) & 0xffu) <= a.drop_thr;
          if (DMASK && a.dmask) {
            const int col = j * BN + 32 * (t >> 1) + 8 * (v >> 2) + 4 * g + (v & 3);
            // (packed: a sequence longer than the seqlen_q x seqlen_k the caller stated gets its first rows and keys
            // only; nothing is stored outside the [seqlen_q, seqlen_k] plane of this (sequence, head))
            const bool row_in = row < Lq && row < a.seqlen_q;
            const int col_lim = min(min(last_k, causal_row_lim), a.seqlen_k - 1);
            if (row_in && col + 1 <= col_lim) {
              *(unsigned*)(drow + (int64_t)col * 2) = Mma<T>::pack2(k0 ? 1.f : -1.f, k1 ? 1.f : -1.f);
            } else if (row_in && col <= col_lim) {
              *(T*)(drow + (int64_t)col * 2) = (T)(k0 ? 1.f : -1.f);
            }
          }
          p0 = k0 ? p0 : 0.f;
          p1 = k1 ? p1 : 0.f;
        }
        w[e2] = Mma<T>::pack2(p0, p1);
        if constexpr (sum_packed) rs = Mma<T>::add_pair(w[e2], rs);
      }
      const s16x8 pb = __builtin_bit_cast(s16x8, w);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) o[mb] = Mma<T>::m32(va[t & 1][mb], pb, o[mb]);
    }
    l_run += rs;
  };

  if (wave_row_lo >= Lq) {
    // A wavefront without a query row (a block shorter than 128 rows: few-query calls against a long K/V) only
    // moves its share of the tiles and keeps the barriers; one barrier per tile, as in tile().
    for (int j = jt0; j < ntiles; ++j) {
      WAIT_VMCNT(0);
      __syncthreads();
      if (j + 1 < ntiles) issue_tile(j + 1, (j + 1 - jt0) & 1);
    }
  } else {
    int j = jt0;
    for (; j + 1 < ntiles; j += 2) {
      tile(j, IC<0>{});
      tile(j + 1, IC<1>{});
    }
    if (j < ntiles) tile(j, IC<0>{});
  }

  // ---- epilogue ----
  l_run = pair_sum32(l_run);
  if (a.n_splits > 1) {  // sliced: unnormalised partials of this slice, one slot per (sequence, head, row, slice)
    // (packed: the workspace holds seqlen_q rows per sequence; a sequence that is longer than the caller said gets
    // its first seqlen_q rows only, instead of partials that land in another head's slots)
    if (row < Lq && row < a.seqlen_q) {
      const int64_t slot = (((int64_t)b * a.heads_q + h) * a.seqlen_q + row) * a.n_splits + split;
      float* dst = a.ws_o + slot * D;
      int g_e = g;  // (kept out of loop-invariant hoisting, as below)
      asm volatile("" : "+v"(g_e));
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) {
          const int d = 32 * mb + 8 * v4 + 4 * g_e;
          if (d < D) *(f32x4*)(dst + d) = f32x4{o[mb][4 * v4 + 0], o[mb][4 * v4 + 1], o[mb][4 * v4 + 2], o[mb][4 * v4 + 3]};
        }
      if (g == 0) {
        a.ws_ml[slot * 2 + 0] = (m_run == -INFINITY) ? -INFINITY : m_run * c;
        a.ws_ml[slot * 2 + 1] = l_run;
      }
    }
    continue;
  }
  const float inv = (l_run > 0.f) ? (DROP ? a.drop_rp : 1.f) / l_run : 0.f;
  // O goes out through LDS: in the accumulator layout a store instruction would write 16 bytes into each of 32 rows
  // (every cache line of the block in 8 pieces, measured at 3.8 us per block); staged, it writes whole rows.  Each
  // wavefront stages its own 32 rows (row stride padded by 16 bytes: the 8-byte writes of rows r and r + 16 share a
  // bank, the 16-byte reads are conflict-free).
  __syncthreads();  // every wavefront is done with the K/V buffers of the last tile
  {
    constexpr int OSTR = ROWB + 16;
    unsigned char* stage = smem + wave * (32 * OSTR);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int v4 = 0; v4 < 4; ++v4) {
        u32x2 w;
        w[0] = Mma<T>::pack2(o[mb][4 * v4 + 0] * inv, o[mb][4 * v4 + 1] * inv);
        w[1] = Mma<T>::pack2(o[mb][4 * v4 + 2] * inv, o[mb][4 * v4 + 3] * inv);
        *(u32x2*)(stage + c32 * OSTR + (32 * mb + 8 * v4 + 4 * g) * 2) = w;
      }
    constexpr int RPS = 64 / CPR;  // rows per store instruction
    unsigned char* oblk = a.out + ob + (int64_t)(q0 + m0 + 32 * wave) * a.o_ss + (int64_t)h * a.o_sh;
    const int sr = lane / CPR, sch = lane % CPR;
    const int rows_left = Lq - (m0 + 32 * wave);  // rows of this wavefront that exist
#pragma unroll
    for (int i = 0; i < 32 / RPS; ++i) {
      const int r = i * RPS + sr;
      const u32x4 x = *(const u32x4*)(stage + r * OSTR + sch * 16);
      if (r < rows_left && sch * 8 < D) *(u32x4*)(oblk + (int64_t)r * a.o_ss + sch * 16) = x;
    }
  }
  if (row < Lq) {
    if (g == 0) {
      const float lse = (l_run > 0.f) ? (m_run * c + __builtin_log2f(l_run)) * kLn2 : INFINITY;
      a.lse[lb + (int64_t)h * a.lse_sh + (int64_t)(q0 + row) * a.lse_ss] = lse;
    }
  }
  }  // own
}

// ---------------------------------------------------------------------------------------------------------
// Split-KV kernel (seqlen_q == 1, group <= 16)
// ---------------------------------------------------------------------------------------------------------
template <int DP>
__device__ __forceinline__ int swzKd(int row) {  // 16 lanes = 16 rows, same logical chunk, ds_read_b128
  if constexpr (DP == 64) return (row >> 1) & 7;
  return row & 15;
}
template <int DP>
__device__ __forceinline__ int swzVd(int row) {  // 8 rows x 32 bytes per half-wave, ds_read_b64_tr_b16
  if constexpr (DP == 64) return ((row >> 1) & 3) << 1;
  return (row & 7) << 1;
}

template <int DP>
struct SplitCfg {
  static constexpr int NW = (DP == 256) ? 2 : 4;        // wavefronts per workgroup
  static constexpr int STAGE = 2 * 32 * DP * 2;         // K block + V block, 32 rows each
  static constexpr int RING = 2 * STAGE;                // per wavefront
  static constexpr int LDS = NW * RING;
};

template <typename T, int DP, bool DROP = false>
__global__ void __launch_bounds__(SplitCfg<DP>::NW * 64, 1) fa_splitkv_kernel(const KArgs a) {
  constexpr int NW = SplitCfg<DP>::NW;
  constexpr int CPR = DP / 8;
  constexpr int ROWB = DP * 2;
  constexpr int BLK = 32 * ROWB;        // bytes of a 32-row K (or V) block
  constexpr int NI = BLK / 1024;        // DMA instructions per block
  constexpr int RPI = 64 / CPR;         // rows per DMA instruction
  constexpr int KS = DP / 32;           // k-steps of the 16x16x32 MFMA over head dim
  constexpr int MB = DP / 16;           // 16-row blocks of O^T
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int L = lane & 15, G = lane >> 4;

  const int split = blockIdx.x % a.n_splits;
  const int bhk = blockIdx.x / a.n_splits;
  const int hk = bhk % a.heads_k, b = bhk / a.heads_k;

  int q0 = 0, k0 = 0, Lk = a.seqlen_k;  // dense: the query of sequence b is row 0 of batch b
  int64_t qb = (int64_t)b * a.q_sb, kb = (int64_t)b * a.k_sb, vb = (int64_t)b * a.v_sb, ob = (int64_t)b * a.o_sb;
  int64_t lb = (int64_t)b * a.lse_sb;
  int Lq = a.seqlen_q;  // dense: up to 16 / group query rows (a few speculative tokens); packed: one
  if (a.cu_q) {
    q0 = a.cu_q[b];
    Lq = a.cu_q[b + 1] - q0;
    k0 = a.cu_k[b];
    Lk = a.cu_k[b + 1] - k0;
    qb = kb = vb = ob = 0;
    lb = (int64_t)q0 * a.lse_ss;
  }
  if (a.seqused_k) Lk = min(Lk, max(a.seqused_k[b], 0));
  const int D = a.head_dim;
  const int group = a.group;
  const int h0 = hk * group;
  // q slot L of the MFMA's N dimension <-> (query row L / group, head h0 + L % group); slots >= nslots are zero
  // (packed: a sequence longer than the seqlen_q the caller gave is cut to its first seqlen_q rows — the 16 MFMA
  // columns and the workspace are sized by it; the causal alignment below keeps the true length)
  const int nslots = group * max(min(Lq, a.seqlen_q), 0);
  const int slot_r = L / group, slot_g = L % group;
  // keys this lane's slot may see: bottom-right causal lets row r see keys <= Lk - Lq + r
  const int slot_lim = a.is_causal ? min(Lk - 1, Lk - Lq + slot_r) : Lk - 1;
  const int mask_from = a.is_causal ? Lk - (Lq - 1) : Lk;  // first key that some slot does not see
  // dropout: the tile kernel's mask (same patch words): this lane's slot is one (head, row), its registers are keys
  uint32_t drop_row = 0, drop_key2 = 0;
  const int drop_sh = 16 * (slot_r & 1);
  if constexpr (DROP) {
    const uint64_t seed = a.seed_ptr ? (uint64_t)*a.seed_ptr : a.seed;
    const uint64_t offset = a.offset_ptr ? (uint64_t)*a.offset_ptr + a.offset : a.offset;
    const DropKeys dk = drop_head_keys(seed, offset, (uint32_t)(b * a.heads_q + h0 + slot_g));
    drop_row = dk.k1 ^ drop_row_term((uint32_t)slot_r >> 1);
    drop_key2 = dk.k2;
    if (blockIdx.x == 0 && tid == 0) {
      if (a.rng_seed_out) *a.rng_seed_out = (int64_t)seed;
      if (a.rng_offset_out) *a.rng_offset_out = (int64_t)offset;
    }
  }

  // slice of 32-row blocks owned by this workgroup, then by this wavefront (interleaved)
  const int nblk = (Lk + 31) >> 5;
  const int per = (nblk + a.n_splits - 1) / a.n_splits;
  const int blk_begin = split * per;
  const int blk_end = min(nblk, blk_begin + per);
  const int last_k = Lk - 1;

  const unsigned char* kp = a.k + kb + (int64_t)k0 * a.k_ss + (int64_t)hk * a.k_sh;
  const unsigned char* vp = a.v + vb + (int64_t)k0 * a.v_ss + (int64_t)hk * a.v_sh;
  const unsigned k_ss = (unsigned)a.k_ss, v_ss = (unsigned)a.v_ss;

  unsigned char* ring = smem + wave * SplitCfg<DP>::RING;
  const int dma_r = lane / CPR, dma_pc = lane % CPR;

  // Paged cache: a 32-row block lies inside one page (page_size is a multiple of 32), so the page is one scalar
  // table entry per block; `page` is that entry (fetched an iteration ahead of its use) and the rows count from the
  // page's first row.  Without a table `page` is 0 and the rows count from the sequence's first key.
  const int32_t* tbl = a.block_table ? a.block_table + (int64_t)b * a.bt_stride : nullptr;
  const int psz = a.page_size;
  auto page_of = [&](int blk_) -> int { return tbl ? tbl[min(blk_ * 32, last_k) / psz] : 0; };
  auto issue_block = [&](int blk, int stage, int page) {
    unsigned char* kdst = ring + stage * SplitCfg<DP>::STAGE;
    unsigned char* vdst = kdst + BLK;
    const unsigned char* kpg = kp;
    const unsigned char* vpg = vp;
    int row0 = 0;  // first key row of what kpg / vpg point at
    if (tbl) {
      kpg = a.k + (int64_t)page * a.k_sb + (int64_t)hk * a.k_sh;
      vpg = a.v + (int64_t)page * a.v_sb + (int64_t)hk * a.v_sh;
      row0 = min(blk * 32, last_k) / psz * psz;
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int r = dma_r + i * RPI;
      int lc = dma_pc ^ swzKd<DP>(r);
      if (lc * 8 >= D) lc = 0;
      const int gr = min(blk * 32 + r, last_k) - row0;
      dma16(kpg + (uint64_t)(unsigned)gr * k_ss + lc * 16, kdst + i * 1024);
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int r = dma_r + i * RPI;
      int lc = dma_pc ^ swzVd<DP>(r);
      if (lc * 8 >= D) lc = 0;
      const int gr = min(blk * 32 + r, last_k) - row0;
      dma16(vpg + (uint64_t)(unsigned)gr * v_ss + lc * 16, vdst + i * 1024);
    }
  };

  int blk = blk_begin + wave;
  const bool any = blk < blk_end && Lq > 0;
  if (any) issue_block(blk, 0, page_of(blk));
  int page_next = (any && blk + NW < blk_end) ? page_of(blk + NW) : 0;  // the table entry of the next block to fetch

  // Q^T as B operand of 16x16x32: lane (q slot = L, G) holds Q[row][head][32 ks + 8 G .. +8] of its slot
  s16x8 qf[KS];
  {
    const unsigned flip = a.neg_scale ? 0x80008000u : 0u;
    const unsigned char* qrow = a.q + qb + (int64_t)(q0 + slot_r) * a.q_ss + (int64_t)(h0 + slot_g) * a.q_sh;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int ch = 4 * ks + G;
      u32x4 x = {0, 0, 0, 0};
      if (L < nslots && ch * 8 < D) {
        x = *(const u32x4*)(qrow + ch * 16);
        x ^= flip;
      }
      qf[ks] = __builtin_bit_cast(s16x8, x);
    }
  }

  f32x4 o[MB];
#pragma unroll
  for (int i = 0; i < MB; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;  // per q slot (replicated over G); l_run is this lane's partial sum
  const float c = a.scale_log2;

  const int ksw = swzKd<DP>(L);                 // rows L and 16 + L
  const int vrow = 4 * G + (L >> 2);            // + 16 for the second half of the contraction
  const int vsw = swzVd<DP>(vrow);              // same for vrow + 16
  const int v_lane_off = vrow * ROWB + (L & 1) * 8;
  const int v_lc0 = (L & 3) >> 1;

  int stage = 0;
  for (; blk < blk_end && Lq > 0; blk += NW) {
    const int nxt = blk + NW;
    if (nxt < blk_end) {
      issue_block(nxt, stage ^ 1, page_next);
      page_next = (nxt + NW < blk_end) ? page_of(nxt + NW) : 0;
      if constexpr (NI == 4) WAIT_VMCNT(8);
      else if constexpr (NI == 8) WAIT_VMCNT(16);
      else WAIT_VMCNT(32);
    } else {
      WAIT_VMCNT(0);
    }
    const unsigned char* kt = ring + stage * SplitCfg<DP>::STAGE;
    const unsigned char* vt = kt + BLK;

    // S^T (kv x q slot): two 16-row tiles
    f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int pc = (4 * ks + G) ^ ksw;
      const s16x8 a0 = *(const s16x8*)(kt + L * ROWB + pc * 16);
      const s16x8 a1 = *(const s16x8*)(kt + (16 + L) * ROWB + pc * 16);
      sa = Mma<T>::m16(a0, qf[ks], sa);
      sb = Mma<T>::m16(a1, qf[ks], sb);
    }
    if (blk * 32 + 32 > mask_from) {
      const int lim = slot_lim - blk * 32 - 4 * G;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        if (v > lim) sa[v] = -INFINITY;
        if (16 + v > lim) sb[v] = -INFINITY;
      }
    }
    float mx = fmaxf(fmaxf(sa[0], sa[1]), fmaxf(sa[2], sa[3]));
    mx = fmaxf(mx, fmaxf(fmaxf(sb[0], sb[1]), fmaxf(sb[2], sb[3])));
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = pair_max32(mx);
    // a slot may have seen no key yet (causal rows against the last blocks of a slice): keep m = -inf, p = 0 then
    const float m_new = fmaxf(m_run, mx);
    const float alpha = (m_new == -INFINITY) ? 1.f : fast_exp2((m_run - m_new) * c);
    const float mc = (m_new == -INFINITY) ? 0.f : m_new * c;
    m_run = m_new;
    float rs = 0.f;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      sa[v] = fast_exp2(sa[v] * c - mc);
      sb[v] = fast_exp2(sb[v] * c - mc);
      rs += sa[v] + sb[v];
    }
    l_run = l_run * alpha + rs;
#pragma unroll
    for (int i = 0; i < MB; ++i) o[i] *= alpha;
    if constexpr (DROP) {
      // row sums are those of the undropped probabilities.  Registers (2 pr, 2 pr + 1) of sa / sb hold keys
      // 32 blk + 16 half + 4 G + 2 pr, + 1: column pair 16 blk + 8 half + 2 G + pr
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int pr = 0; pr < 2; ++pr) {
          const uint32_t cp = (uint32_t)(16 * blk + 8 * half + 2 * G + pr);
          const uint32_t word = drop_word(drop_row ^ drop_col_term(cp), drop_key2) >> drop_sh;
          const bool k0 = (word & 0xffu) <= a.drop_thr, k1 = ((word >> 8) & 0xffu) <= a.drop_thr;
          if (half) {
            sb[2 * pr] = k0 ? sb[2 * pr] : 0.f;
            sb[2 * pr + 1] = k1 ? sb[2 * pr + 1] : 0.f;
          } else {
            sa[2 * pr] = k0 ? sa[2 * pr] : 0.f;
            sa[2 * pr + 1] = k1 ? sa[2 * pr + 1] : 0.f;
          }
        }
    }

    u32x4 w;
    w[0] = Mma<T>::pack2(sa[0], sa[1]);
    w[1] = Mma<T>::pack2(sa[2], sa[3]);
    w[2] = Mma<T>::pack2(sb[0], sb[1]);
    w[3] = Mma<T>::pack2(sb[2], sb[3]);
    const s16x8 pb = __builtin_bit_cast(s16x8, w);

#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int pc = (2 * mb + v_lc0) ^ vsw;
      const unsigned char* vbase = vt + v_lane_off + pc * 16;
      const s16x4 lo = lds_read_tr(vbase);
      const s16x4 hi = lds_read_tr(vbase + 16 * ROWB);
      const s16x8 av = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      o[mb] = Mma<T>::m16(av, pb, o[mb]);
    }
    stage ^= 1;
  }

  // ---- merge the NW wavefronts' partials through LDS ----
  l_run += __shfl_xor(l_run, 16);
  l_run = pair_sum32(l_run);
  __syncthreads();  // all rings are idle (every wavefront waited for its last DMA before its last block)
  float* so = (float*)smem;                       // [NW][16][DP]
  float* sml = (float*)(smem + NW * 16 * DP * 4); // [NW][16][2]
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int v = 0; v < 4; ++v) so[(wave * 16 + L) * DP + 16 * mb + 4 * G + v] = o[mb][v];
  if (G == 0) {
    sml[(wave * 16 + L) * 2 + 0] = (m_run == -INFINITY) ? -INFINITY : m_run * c;
    sml[(wave * 16 + L) * 2 + 1] = l_run;
  }
  __syncthreads();
  if (Lq <= 0) return;
  // thread -> (q slot, 16 d-values)
  constexpr int TPQ = DP / 16;  // threads per q slot
  for (int item = tid; item < nslots * TPQ; item += NW * 64) {
    const int qs = item / TPQ, d0 = (item % TPQ) * 16;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, sml[(w * 16 + qs) * 2]);
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    float lsum = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float mw = sml[(w * 16 + qs) * 2];
      const float sc = (mw == -INFINITY) ? 0.f : fast_exp2(mw - M);
      lsum += sml[(w * 16 + qs) * 2 + 1] * sc;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] += so[(w * 16 + qs) * DP + d0 + i] * sc;
    }
    const int qr = qs / group;  // query row of this slot (0 in packed mode)
    const int h = h0 + qs % group;
    if (a.n_splits == 1) {
      const float inv = (lsum > 0.f) ? (DROP ? a.drop_rp : 1.f) / lsum : 0.f;
      if (d0 < D) {
        unsigned char* orow = a.out + ob + (int64_t)(q0 + qr) * a.o_ss + (int64_t)h * a.o_sh + d0 * 2;
        u32x4 w0, w1;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          w0[i] = Mma<T>::pack2(acc[2 * i] * inv, acc[2 * i + 1] * inv);
          w1[i] = Mma<T>::pack2(acc[8 + 2 * i] * inv, acc[8 + 2 * i + 1] * inv);
        }
        *(u32x4*)orow = w0;
        if (d0 + 8 < D) *(u32x4*)(orow + 16) = w1;
      }
      if (d0 == 0)
        a.lse[lb + (int64_t)h * a.lse_sh + (int64_t)qr * a.lse_ss] = (lsum > 0.f) ? (M + __builtin_log2f(lsum)) * kLn2 : INFINITY;
    } else {
      // one slot per (sequence, head, query row, slice): what fa_merge_rows_kernel reads (packed: seqlen_q is the
      // longest sequence, shorter ones leave their last slots unused)
      const int64_t slot = (((int64_t)b * a.heads_q + h) * a.seqlen_q + qr) * a.n_splits + split;
      if (d0 < D) {
        float* dst = a.ws_o + slot * D + d0;
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (d0 + i < D) dst[i] = acc[i];
      }
      if (d0 == 0) {
        a.ws_ml[slot * 2 + 0] = M;
        a.ws_ml[slot * 2 + 1] = lsum;
      }
    }
  }
}

// Merge the per-slice partials of either kernel: one wavefront per (sequence, query head, query row), four rows per
// workgroup; lane -> head_dim elements lane, lane+64, ...  Packed mode: seqlen_q is the longest sequence; rows beyond
// a sequence's own length have no partials and are skipped.
template <typename T>
__global__ void __launch_bounds__(256) fa_merge_rows_kernel(const KArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // (b * heads_q + h) * seqlen_q + row
  const int64_t rows = (int64_t)a.batch * a.heads_q * a.seqlen_q;
  if (r >= rows) return;
  const int row = (int)(r % a.seqlen_q);
  const int bh = (int)(r / a.seqlen_q);
  const int h = bh % a.heads_q, b = bh / a.heads_q;
  const int D = a.head_dim, ns = a.n_splits;
  int64_t orow_off = (int64_t)b * a.o_sb + (int64_t)row * a.o_ss;
  int64_t lse_off = (int64_t)b * a.lse_sb + (int64_t)row * a.lse_ss;
  if (a.cu_q) {
    const int q0 = a.cu_q[b];
    if (row >= a.cu_q[b + 1] - q0) return;
    orow_off = (int64_t)(q0 + row) * a.o_ss;
    lse_off = (int64_t)(q0 + row) * a.lse_ss;
  }
  const float* ml = a.ws_ml + r * ns * 2;
  const float* po = a.ws_o + r * ns * D;
  // lane s holds slice s's (m, l) (at most 64 slices); the maximum, the scale factors and the sum of l are formed
  // across the wavefront, then the slices' rows are accumulated with independent loads
  float ms = -INFINITY, ls = 0.f;
  if (lane < ns) {
    const f32x2 v = *(const f32x2*)(ml + 2 * lane);
    ms = v[0];
    ls = v[1];
  }
  float M = ms;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) M = fmaxf(M, __shfl_xor(M, o));
  const float scl = (ms == -INFINITY) ? 0.f : fast_exp2(ms - M);  // 0: a slice without a visible key for this row
  float lsum = ls * scl;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) lsum += __shfl_xor(lsum, o);
  float acc[4] = {0.f, 0.f, 0.f, 0.f};  // head_dim <= 256
#pragma unroll 4
  for (int s = 0; s < ns; ++s) {
    const float sc = __shfl(scl, s);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      // a slice that saw no key leaves zeros (the tile kernel) or finite partial sums; its factor is 0 either way
      if (d < D) acc[i] += po[(int64_t)s * D + d] * sc;
    }
  }
  const float inv = (lsum > 0.f) ? a.drop_rp / lsum : 0.f;  // 1 / keep: the split-KV kernel's partials under dropout
  T* orow = (T*)(a.out + orow_off + (int64_t)h * a.o_sh);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    if (d < D) orow[d] = (T)(acc[i] * inv);
  }
  if (lane == 0)
    a.lse[lse_off + (int64_t)h * a.lse_sh] = (lsum > 0.f) ? (M + __builtin_log2f(lsum)) * kLn2 : INFINITY;
}

// ---------------------------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------------------------
using namespace fa::host;

KArgs make_args(const fa_fwd_params* p, int kern, int ns, void* ws) {
  KArgs a;
  a.q = (const unsigned char*)p->q;
  a.k = (const unsigned char*)p->k;
  a.v = (const unsigned char*)p->v;
  a.out = (unsigned char*)p->out;
  a.lse = p->lse;
  a.cu_q = p->cu_seqlens_q;
  a.cu_k = p->cu_seqlens_k;
  a.q_sb = p->q_stride_b * 2; a.q_ss = p->q_stride_s * 2; a.q_sh = p->q_stride_h * 2;
  a.k_sb = p->k_stride_b * 2; a.k_ss = p->k_stride_s * 2; a.k_sh = p->k_stride_h * 2;
  a.v_sb = p->v_stride_b * 2; a.v_ss = p->v_stride_s * 2; a.v_sh = p->v_stride_h * 2;
  a.o_sb = p->o_stride_b * 2; a.o_ss = p->o_stride_s * 2; a.o_sh = p->o_stride_h * 2;
  a.lse_sb = p->lse_stride_b; a.lse_sh = p->lse_stride_h; a.lse_ss = p->lse_stride_s;
  a.batch = p->batch; a.heads_q = p->heads_q; a.heads_k = p->heads_k; a.group = p->heads_q / p->heads_k;
  a.seqlen_q = p->seqlen_q; a.seqlen_k = p->seqlen_k; a.head_dim = p->head_dim;
  a.n_mblk = (p->seqlen_q + 127) / 128;
  a.pair = 0;
  a.n_splits = ns;
  a.is_causal = p->is_causal ? 1 : 0;
  a.causal_tl = p->is_causal == FA_MASK_CAUSAL_TOP_LEFT ? 1 : 0;
  a.seqused_k = p->seqused_k;
  a.block_table = p->block_table; a.bt_stride = p->block_table_stride; a.page_size = p->page_size;
  a.bias = (const unsigned char*)p->bias;
  a.bias_sb = p->bias_stride_b * 2; a.bias_sh = p->bias_stride_h * 2; a.bias_sq = p->bias_stride_q * 2;
  a.neg_scale = p->scale < 0.f ? 1 : 0;
  a.scale_log2 = (p->scale < 0.f ? -p->scale : p->scale) * kLog2e;
  // scale == 0: masked scores are -inf and -inf * 0 is NaN; a tiny positive factor keeps -inf masked and maps every
  // finite score to (numerically) zero, which is the scale == 0 answer.
  if (!(a.scale_log2 > 0.f)) a.scale_log2 = 1e-30f;
  a.scale_abs = a.scale_log2 * kLn2;
  const float p_keep = 1.f - p->dropout_p;
  a.drop_thr = (uint32_t)floorf(p_keep * 255.f);
  a.drop_rp = 256.f / (float)(a.drop_thr + 1u);  // the reciprocal of the keep probability the mask realises
  a.seed = p->philox_seed; a.offset = p->philox_offset;
  a.seed_ptr = p->philox_seed_ptr; a.offset_ptr = p->philox_offset_ptr;
  a.rng_seed_out = p->rng_seed_out; a.rng_offset_out = p->rng_offset_out;
  a.dmask = (unsigned char*)p->dropout_mask;
  a.ws_o = nullptr;
  a.ws_ml = nullptr;
  if (ws && ns > 1) {
    const size_t slots = partial_slots(p, kern, ns);
    a.ws_o = (float*)ws;
    a.ws_ml = (float*)((unsigned char*)ws + slots * (size_t)p->head_dim * 4);
  }
  return a;
}

template <typename T, int DP, int MINB, int BIAS, bool DROP = false, bool DMASK = false, bool PAGED = false>
int launch_tile(KArgs a, hipStream_t st) {
  constexpr int lds = 4 * 64 * DP * 2 + (BIAS == 2 ? 4 * 4096 : 0);
  constexpr auto kfn = fa_tile_kernel<T, DP, MINB, BIAS, DROP, DMASK, PAGED>;
  if (!ensure_dynamic_lds<kfn>(lds)) return FA_ERR_LAUNCH;
  const int nblk = (a.seqlen_q + 127) / 128;
  a.pair = (DP != 256 && a.n_splits == 1 && a.is_causal && nblk >= 2 &&
            (int64_t)a.batch * a.heads_q * ((nblk + 1) / 2) >= 1024) ? 1 : 0;
  // packed: the kernel finds the pairs itself with one lane per sequence, in a loop over the block index
  if (a.cu_q && (a.batch > 64 || nblk > 1024)) a.pair = 0;
  a.n_mblk = (a.pair && !a.cu_q) ? (nblk + 1) / 2 : nblk;
  a.hgroup = 1;
  if (BIAS && !a.cu_q && a.bias_sh == 0)
    for (int gsz = FA_HGROUP; gsz > 1; gsz >>= 1)
      if (a.heads_q % gsz == 0) {
        a.hgroup = gsz;
        break;
      }
  // (packed and paired: at most (n + 1) / 2 pairs per sequence; what the shorter sequences leave over exits)
  const int64_t grid = (int64_t)a.batch * a.heads_q * ((a.pair && a.cu_q) ? (nblk + 1) / 2 : a.n_mblk) * a.n_splits;
  if (grid <= 0) return FA_OK;
  if (grid > 0x7fffffffLL) return FA_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kfn, dim3((unsigned)grid), dim3(256), lds, st, a);
  if (hipGetLastError() != hipSuccess) return FA_ERR_LAUNCH;
  if (a.n_splits > 1) {
    const int64_t rows = (int64_t)a.batch * a.heads_q * a.seqlen_q;
    hipLaunchKernelGGL(fa_merge_rows_kernel<T>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, a);
    if (hipGetLastError() != hipSuccess) return FA_ERR_LAUNCH;
  }
  return FA_OK;
}

template <typename T, int DP, bool DROP>
int launch_splitkv(const KArgs& a, hipStream_t st) {
  constexpr int lds = SplitCfg<DP>::LDS;
  constexpr auto kfn = fa_splitkv_kernel<T, DP, DROP>;
  if (!ensure_dynamic_lds<kfn>(lds)) return FA_ERR_LAUNCH;
  const int64_t grid = (int64_t)a.batch * a.heads_k * a.n_splits;
  if (grid > 0x7fffffffLL) return FA_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kfn, dim3((unsigned)grid), dim3(SplitCfg<DP>::NW * 64), lds, st, a);
  if (hipGetLastError() != hipSuccess) return FA_ERR_LAUNCH;
  if (a.n_splits > 1) {
    const int64_t rows = (int64_t)a.batch * a.heads_q * a.seqlen_q;
    hipLaunchKernelGGL(fa_merge_rows_kernel<T>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, a);
    if (hipGetLastError() != hipSuccess) return FA_ERR_LAUNCH;
  }
  return FA_OK;
}

template <typename T>
int dispatch(const KArgs& a, int kern, hipStream_t st) {
  const int dp = padded_dim(a.head_dim);
  if (kern == FA_KERNEL_SPLITKV) {
    if (a.drop_thr < 255u) {  // dropout_p > 0
      if (dp == 64) return launch_splitkv<T, 64, true>(a, st);
      if (dp == 128) return launch_splitkv<T, 128, true>(a, st);
      return launch_splitkv<T, 256, true>(a, st);
    }
    if (dp == 64) return launch_splitkv<T, 64, false>(a, st);
    if (dp == 128) return launch_splitkv<T, 128, false>(a, st);
    return launch_splitkv<T, 256, false>(a, st);
  }
  if (a.drop_thr < 255u && a.dmask) {  // dropout_p > 0 and the keep-mask is wanted (tests)
    if (a.bias) {
      if (dp == 64) return launch_tile<T, 64, 2, true, true, true>(a, st);
      if (dp == 128) return launch_tile<T, 128, 2, true, true, true>(a, st);
      return launch_tile<T, 256, 1, true, true, true>(a, st);
    }
    if (dp == 64) return launch_tile<T, 64, 2, false, true, true>(a, st);
    if (dp == 128) return launch_tile<T, 128, 2, false, true, true>(a, st);
    return launch_tile<T, 256, 1, false, true, true>(a, st);
  }
  if (a.drop_thr < 255u) {  // dropout_p > 0
    if (a.bias) {
      if (dp == 64) return launch_tile<T, 64, 2, true, true>(a, st);
      if (dp == 128) return launch_tile<T, 128, 2, true, true>(a, st);
      return launch_tile<T, 256, 1, true, true>(a, st);
    }
    if (dp == 64) return launch_tile<T, 64, 2, false, true>(a, st);
    if (dp == 128) return launch_tile<T, 128, 2, false, true>(a, st);
    return launch_tile<T, 256, 1, false, true>(a, st);
  }
  if (a.bias) {
    // 16-byte pieces of bias rows can be fetched by DMA one tile ahead when every row starts 16-byte aligned and no
    // piece straddles the end of a row; otherwise the kernel reads 8-byte pieces directly
    const bool staged = !a.cu_q && !a.seqused_k && a.seqlen_k % 8 == 0 && (uintptr_t)a.bias % 16 == 0 &&
                        a.bias_sb % 16 == 0 && a.bias_sh % 16 == 0 && a.bias_sq % 16 == 0 &&
                        a.bias_sq <= kMaxRowStrideBytes;
    if (staged && dp == 64) return launch_tile<T, 64, 2, 2>(a, st);
    if (staged && dp == 128) return launch_tile<T, 128, 2, 2>(a, st);
    if (dp == 64) return launch_tile<T, 64, 2, 1>(a, st);
    if (dp == 128) return launch_tile<T, 128, 2, 1>(a, st);
    return launch_tile<T, 256, 1, 1>(a, st);
  }
  if (a.block_table) {  // a prefill chunk against a paged KV cache
    if (dp == 64) return launch_tile<T, 64, 2, 0, false, false, true>(a, st);
    if (dp == 128) return launch_tile<T, 128, 2, 0, false, false, true>(a, st);
    return launch_tile<T, 256, 1, 0, false, false, true>(a, st);
  }
  if (dp == 64) return launch_tile<T, 64, 2, false>(a, st);
  if (dp == 128) return launch_tile<T, 128, 2, false>(a, st);
  return launch_tile<T, 256, 1, false>(a, st);
}

}  // namespace

extern "C" {

int fa_fwd_version(void) { return FA_FWD_ABI_VERSION; }

const char* fa_fwd_error_string(int rc) {
  switch (rc) {
    case FA_OK: return "ok";
    case FA_ERR_BAD_ARG: return "bad argument (null pointer, non-positive size, misaligned pointer or stride, short workspace)";
    case FA_ERR_UNSUPPORTED: return "unsupported shape or dtype";
    case FA_ERR_LAUNCH: return "HIP launch failure";
    case FA_ERR_WORKSPACE: return "the plan needs more scratch than fa_fwd_launch_static holds (FA_STATIC_WORKSPACE_BYTES); use fa_fwd_launch with a workspace";
    default: return "unknown error";
  }
}

int fa_fwd_validate(const fa_fwd_params* p) { return validate(p); }

int fa_fwd_plan(const fa_fwd_params* p, int32_t* kernel, int32_t* num_splits) {
  const int rc = validate(p);
  if (rc != FA_OK) return rc;
  int k, s;
  plan(p, &k, &s);
  if (kernel) *kernel = k;
  if (num_splits) *num_splits = s;
  return FA_OK;
}

size_t fa_fwd_workspace_bytes(const fa_fwd_params* p) {
  if (validate(p) != FA_OK) return 0;
  int k, s;
  plan(p, &k, &s);
  return workspace_bytes(p, k, s);
}

}  // extern "C"

// Scratch of fa_fwd_launch_static: the per-slice partials of the split-KV and sliced tile kernels, in device memory
// that belongs to the code object (present on every device the library is loaded on, for the life of the process).
// The name below is a host-side handle only; the device address is looked up once per device.
static __device__ __align__(256) unsigned char scratch[FA_STATIC_WORKSPACE_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device; nullptr when the runtime cannot give one.
void* static_scratch() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr) return ptr;
  if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
    (void)hipGetLastError();
    return nullptr;
  }
  g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // every thread gets the same answer, so a race is harmless
  return ptr;
}
}  // namespace

extern "C" {

int fa_fwd_launch_static(const fa_fwd_params* p, void* stream) {
  const int rc = validate(p);
  if (rc != FA_OK) return rc;
  int kern, ns;
  plan(p, &kern, &ns);
  const size_t need = workspace_bytes(p, kern, ns);
  if (need > (size_t)FA_STATIC_WORKSPACE_BYTES) return FA_ERR_WORKSPACE;
  void* ws = nullptr;
  if (need > 0) {
    ws = static_scratch();
    if (!ws) return FA_ERR_LAUNCH;
  }
  return fa_fwd_launch(p, ws, need > 0 ? (size_t)FA_STATIC_WORKSPACE_BYTES : 0, stream);
}

int fa_fwd_launch(const fa_fwd_params* p, void* workspace, size_t workspace_bytes_given, void* stream) {
  const int rc = validate(p);
  if (rc != FA_OK) return rc;
  int kern, ns;
  plan(p, &kern, &ns);
  const size_t need = workspace_bytes(p, kern, ns);
  if (need > 0 && (!workspace || workspace_bytes_given < need || ((uintptr_t)workspace & 15))) return FA_ERR_BAD_ARG;
  if (p->seqlen_q == 0) return FA_OK;  // nothing to write
  const KArgs a = make_args(p, kern, ns, workspace);
  hipStream_t st = (hipStream_t)stream;
  return p->dtype == FA_DTYPE_BF16 ? dispatch<__bf16>(a, kern, st) : dispatch<_Float16>(a, kern, st);
}

}  // extern "C"
