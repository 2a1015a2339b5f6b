// Flash-attention forward for MI355X (gfx950): the 256-row tile kernel.
//
// Same arithmetic and the same lane layout as fa_tile_kernel (fa_fwd_kernels.hip) — S^T = K Q^T with
// v_mfma_f32_32x32x16, one lane owns one query row's scores, P^T is already the B operand of O^T += V^T P^T — but one
// wavefront owns 64 query rows (two 32-row halves, A and B), a workgroup of 4 wavefronts 256 rows, and a CU runs one
// workgroup with one wavefront per SIMD and the whole 512-entry register file:
//   * every K / V fragment read from LDS and every byte moved from L2 into LDS by DMA feeds twice the MFMA work;
//   * matrix and vector work overlap inside the wavefront instead of between two wavefronts of a SIMD: the loop is
//     software-pipelined over 32-key blocks — while the MFMAs of S(u) = K(u) Q^T and of O += V(u-1) P(u-1) issue, the
//     vector ALU forms P(u-1) from S(u-1) between them, a few operations after each MFMA (a 32x32x16 MFMA keeps the
//     matrix pipe busy for 32 cycles but blocks vector issue for about 16 of them);
//   * the O accumulators (128 registers at head_dim 128) and the Q fragments (64) live in accumulation registers,
//     which only MFMAs touch in the loop; the S accumulators live in ordinary vector registers, where the softmax
//     reads them.  The compiler places all MFMA results of a kernel in one of the two files, so every MFMA here is
//     inline assembly with the register file of each operand spelled out.  The compiler then cannot see the MFMA
//     hazards either; the code keeps them by construction (see mfma_drain).
// Replaces, like fa_tile_kernel, the vendor call cnnlFlashAttentionForward_v2
// (torch_mlu/csrc/aten/operators/cnnl/internal/FlashAttention_internal.cpp:231-258).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "fa_device.h"
#include "fa_fwd.h"
#include "fa_fwd_common.h"

namespace fa {
namespace {

// ---- accumulation registers, assigned by hand -------------------------------------------------------------
// The compiler keeps all MFMA results of a kernel in one register file, so the MFMAs here are inline assembly that
// names its accumulation registers itself (NH = 32-row halves per wavefront, X = half, mb = 32-row block of O^T):
//   a[AccMap<NH>::kO + 16 (X MB + mb) .. +15]  O^T accumulator
//   a[AccMap<NH>::kQ + 4 (X KS + ks) .. +3]    Q fragment (B operand) of k-step ks
// The compiler may park a few long-lived values of its own in accumulation registers; it takes them from a0 upwards.
// The registers below kO are left to it, the first statement of the kernel names the hand-assigned ones as clobbered
// so that they are allocated, and the build checks the generated code: an accumulation register at or above kO
// outside the assembly statements below fails it (torch_mlu_amd/_build.py).
template <int NH>
struct AccMap;
template <>
struct AccMap<2> {  // one wavefront per SIMD, 512 registers: a64 .. a191 O, a192 .. a255 Q
  static constexpr int kO = 64, kQ = 192, kEnd = 256;
};
template <>
struct AccMap<1> {  // two wavefronts per SIMD, 128 + 128 registers: a32 .. a95 O, a96 .. a127 Q
  static constexpr int kO = 32, kQ = 96, kEnd = 128;
};
#define FA_ACC_CLOBBERS_NH2 \
  "a64", "a65", "a66", "a67", "a68", "a69", "a70", "a71", "a72", "a73", "a74", "a75", "a76", "a77", "a78", "a79", \
  "a80", "a81", "a82", "a83", "a84", "a85", "a86", "a87", "a88", "a89", "a90", "a91", "a92", "a93", "a94", "a95", \
  "a96", "a97", "a98", "a99", "a100", "a101", "a102", "a103", "a104", "a105", "a106", "a107", "a108", "a109", \
  "a110", "a111", "a112", "a113", "a114", "a115", "a116", "a117", "a118", "a119", "a120", "a121", "a122", "a123", \
  "a124", "a125", "a126", "a127", "a128", "a129", "a130", "a131", "a132", "a133", "a134", "a135", "a136", "a137", \
  "a138", "a139", "a140", "a141", "a142", "a143", "a144", "a145", "a146", "a147", "a148", "a149", "a150", "a151", \
  "a152", "a153", "a154", "a155", "a156", "a157", "a158", "a159", "a160", "a161", "a162", "a163", "a164", "a165", \
  "a166", "a167", "a168", "a169", "a170", "a171", "a172", "a173", "a174", "a175", "a176", "a177", "a178", "a179", \
  "a180", "a181", "a182", "a183", "a184", "a185", "a186", "a187", "a188", "a189", "a190", "a191", "a192", "a193", \
  "a194", "a195", "a196", "a197", "a198", "a199", "a200", "a201", "a202", "a203", "a204", "a205", "a206", "a207", \
  "a208", "a209", "a210", "a211", "a212", "a213", "a214", "a215", "a216", "a217", "a218", "a219", "a220", "a221", \
  "a222", "a223", "a224", "a225", "a226", "a227", "a228", "a229", "a230", "a231", "a232", "a233", "a234", "a235", \
  "a236", "a237", "a238", "a239", "a240", "a241", "a242", "a243", "a244", "a245", "a246", "a247", "a248", "a249", \
  "a250", "a251", "a252", "a253", "a254", "a255"
#define FA_ACC_CLOBBERS_NH1 \
  "a32", "a33", "a34", "a35", "a36", "a37", "a38", "a39", "a40", "a41", "a42", "a43", "a44", "a45", "a46", "a47", \
  "a48", "a49", "a50", "a51", "a52", "a53", "a54", "a55", "a56", "a57", "a58", "a59", "a60", "a61", "a62", "a63", \
  "a64", "a65", "a66", "a67", "a68", "a69", "a70", "a71", "a72", "a73", "a74", "a75", "a76", "a77", "a78", "a79", \
  "a80", "a81", "a82", "a83", "a84", "a85", "a86", "a87", "a88", "a89", "a90", "a91", "a92", "a93", "a94", "a95", \
  "a96", "a97", "a98", "a99", "a100", "a101", "a102", "a103", "a104", "a105", "a106", "a107", "a108", "a109", \
  "a110", "a111", "a112", "a113", "a114", "a115", "a116", "a117", "a118", "a119", "a120", "a121", "a122", "a123", \
  "a124", "a125", "a126", "a127"

// S^T (+)= K Q^T: accumulator in vector registers, Q fragment in accumulation registers a[QA .. QA + 3].
template <typename T, int QA>
__device__ __forceinline__ void s_mma_first(f32x16& acc, const s16x8& k) {
  if constexpr (std::is_same_v<T, __bf16>)
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, a[%2:%3], 0" : "=&v"(acc) : "v"(k), "n"(QA), "n"(QA + 3));
  else
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, a[%2:%3], 0" : "=&v"(acc) : "v"(k), "n"(QA), "n"(QA + 3));
}
template <typename T, int QA>
__device__ __forceinline__ void s_mma(f32x16& acc, const s16x8& k) {
  if constexpr (std::is_same_v<T, __bf16>)
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, a[%2:%3], %0" : "+v"(acc) : "v"(k), "n"(QA), "n"(QA + 3));
  else
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, a[%2:%3], %0" : "+v"(acc) : "v"(k), "n"(QA), "n"(QA + 3));
}
// O^T += V^T P^T: accumulator a[OA .. OA + 15].
template <typename T, int OA>
__device__ __forceinline__ void pv_mma(const s16x8& v, const s16x8& p) {
  if constexpr (std::is_same_v<T, __bf16>)
    asm volatile("v_mfma_f32_32x32x16_bf16 a[%2:%3], %0, %1, a[%2:%3]" : : "v"(v), "v"(p), "n"(OA), "n"(OA + 15));
  else
    asm volatile("v_mfma_f32_32x32x16_f16 a[%2:%3], %0, %1, a[%2:%3]" : : "v"(v), "v"(p), "n"(OA), "n"(OA + 15));
}
// Keeps the computation of the given values where it is written: the compiler would otherwise sink vector work that
// only a later MFMA phase consumes out of the phase it is meant to overlap with (the MFMAs, being volatile assembly,
// keep their order relative to this).
template <typename... Ts>
__device__ __forceinline__ void pin(Ts&... xs) {
  (..., [](auto& x) { asm volatile("" : "+v"(x)); }(xs));
}
template <int I>
__device__ __forceinline__ float acc_read() {
  float x;
  asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(I));
  return x;
}
template <int I>
__device__ __forceinline__ void acc_write(float x) {
  asm volatile("v_accvgpr_write_b32 a[%1], %0" : : "v"(x), "n"(I));
}
// The hardware does not interlock a vector-ALU access to a register that an MFMA in flight is still going to write,
// and the compiler cannot see the MFMAs above.  Inside the pipelined loop a block's S is first read a whole MFMA phase
// after its last MFMA; everywhere else (the first block, the mask of a partial block, the rare rescale, the
// epilogue) this waits out the longest MFMA (8 passes of 4 cycles + issue) first.
__device__ __forceinline__ void mfma_drain_asm() { asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 7" ::: "memory"); }

// NH = 2: 4 wavefronts of 64 rows, one per SIMD.  NH = 1: 8 wavefronts of 32 rows, two per SIMD (same pipeline per
// wavefront; a second wavefront fills the issue slots that a lone one leaves between its own instructions).
template <typename T, int DP, int NH>
__global__ void __launch_bounds__(NH == 2 ? 256 : 512) __attribute__((amdgpu_waves_per_eu(3 - NH, 3 - NH)))
fa_tile256_kernel(const KArgs a) {
  constexpr int NW = NH == 2 ? 4 : 8;  // wavefronts per workgroup
  constexpr int kOBase = AccMap<NH>::kO, kQBase = AccMap<NH>::kQ;
  constexpr int CPR = DP / 8;          // 16-byte chunks per row
  constexpr int ROWB = DP * 2;         // bytes per LDS row
  constexpr int BM = 256, BN = 64;
  constexpr int TILE = BN * ROWB;      // bytes per K (or V) tile
  constexpr int NI = TILE / 1024 / NW;  // DMA instructions per wavefront per tile
  constexpr int RPI = 64 / CPR;        // rows covered by one DMA instruction
  constexpr int KS = DP / 16;          // MFMA k-steps over the head dim
  constexpr int MB = DP / 32;          // 32-row blocks of O^T
  constexpr int NS = NH * KS;          // MFMAs of a block's S phase (halves x KS)
  constexpr int NP = 2 * NH * MB;      // MFMAs of a block's PV phase (2 chunks x halves x MB)
  constexpr int VOFF = 2 * TILE;       // LDS: K0 K1 V0 V1 V2
  constexpr int KPRE = NH == 2 ? (KS < 4 ? KS : 4) : 2;  // K fragments in flight (an LDS read outlasts two MFMAs)
  static_assert(NI >= 1 && kOBase + NH * MB * 16 <= kQBase && kQBase + NH * KS * 4 <= AccMap<NH>::kEnd, "register map");
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  constexpr bool ACC = true;  // (false: O and Q as ordinary variables and builtin MFMAs, for experiments)
  // a lone wavefront per SIMD has nobody to hide an LDS read behind: it requests the first fragments of a phase during
  // the phase before.  With two wavefronts per SIMD the registers for that are not there, and the other wavefront is.
  constexpr bool XPRE = NH == 2;
  if constexpr (NH == 2) asm volatile("; accumulation registers a64 .. a255 are assigned by hand" ::: FA_ACC_CLOBBERS_NH2);
  else asm volatile("; accumulation registers a32 .. a127 are assigned by hand" ::: FA_ACC_CLOBBERS_NH1);
  auto mfma_drain = [&]() __attribute__((always_inline)) {
    if constexpr (ACC) mfma_drain_asm();
  };
  f32x16 o[NH][MB];  // NH == 1 only
  s16x8 qf[NH][KS];  // NH == 1 only

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, c32 = lane & 31;

  // ---- which (sequence, head, query block), as in fa_tile_kernel: dense -> XCD-contiguous ranges of logical ids,
  //      packed -> block-major (the heaviest block index of every sequence first) ----
  int lid = blockIdx.x;
  int pslot, bh;
  if (a.cu_q) {
    const int nbh = a.batch * a.heads_q;
    pslot = lid / nbh;
    bh = lid % nbh;
  } else {
    const int total = gridDim.x, per = total >> 3;
    if (lid < (per << 3)) lid = (lid & 7) * per + (lid >> 3);
    pslot = lid % a.n_mblk;
    bh = lid / a.n_mblk;
  }
  const int h = bh % a.heads_q, b = bh / a.heads_q;
  const int hk = h / a.group;

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
  const int nblk = (Lq + BM - 1) / BM;
  const int blk_first = (a.cu_q ? a.n_mblk : nblk) - 1 - pslot;
  if (a.pair ? (2 * pslot >= nblk) : (blk_first < 0 || blk_first >= nblk)) return;
  const int n_own = (a.pair && blk_first != pslot) ? 2 : 1;
  const int off = a.causal_tl ? 0 : Lk - Lq;  // causal: col visible iff col <= row + off

  const unsigned char* qp = a.q + qb + (int64_t)q0 * a.q_ss + (int64_t)h * a.q_sh;
  const unsigned char* kp = a.k + kb + (int64_t)k0 * a.k_ss + (int64_t)hk * a.k_sh;
  const unsigned char* vp = a.v + vb + (int64_t)k0 * a.v_ss + (int64_t)hk * a.v_sh;
  const int D = a.head_dim;

  // ---- DMA bookkeeping (as in fa_tile_kernel: scalar base + fixed per-lane offset, swizzles on the global side) ----
  const int dma_r = wave * RPI + lane / CPR;
  const int dma_pc = lane % CPR;
  int lck = dma_pc ^ swzK<DP>(dma_r);
  int lcv = dma_pc ^ swzV<DP>(dma_r);
  if (lck * 8 >= D) lck = 0;
  if (lcv * 8 >= D) lcv = 0;
  const unsigned k_ss = (unsigned)a.k_ss, v_ss = (unsigned)a.v_ss;
  const unsigned koff = (unsigned)dma_r * k_ss + lck * 16;
  const unsigned voff = (unsigned)dma_r * v_ss + lcv * 16;
  const int last_k = Lk - 1;
  const unsigned lds0 = (unsigned)(uintptr_t)(LDS_AS unsigned char*)smem + wave * 1024;

  // K and V of tile j into K buffer j % 2 and V buffer j % 3: full tiles with scalar address arithmetic only, the last,
  // partial tile with rows clamped per lane
  auto issue_tile = [&](int j) __attribute__((always_inline)) {
    const unsigned kdst = lds0 + (j & 1) * TILE, vdst = lds0 + VOFF + (j % 3) * TILE;
    const unsigned char* kt = kp + (uint64_t)(unsigned)(j * BN) * k_ss;
    const unsigned char* vt = vp + (uint64_t)(unsigned)(j * BN) * v_ss;
    if ((j + 1) * BN <= Lk) {
#pragma unroll
      for (int i = 0; i < NI; ++i) dma16s(kt + (uint64_t)(unsigned)(i * NW * RPI) * k_ss, koff, kdst + i * (NW * 1024));
#pragma unroll
      for (int i = 0; i < NI; ++i) dma16s(vt + (uint64_t)(unsigned)(i * NW * RPI) * v_ss, voff, vdst + i * (NW * 1024));
    } else {
      const int rmax = last_k - j * BN;  // >= 0: the tile exists
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const unsigned r = (unsigned)min(dma_r + i * NW * RPI, rmax);
        dma16s(kt, r * k_ss + lck * 16, kdst + i * (NW * 1024));
      }
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const unsigned r = (unsigned)min(dma_r + i * NW * RPI, rmax);
        dma16s(vt, r * v_ss + lcv * 16, vdst + i * (NW * 1024));
      }
    }
  };

  // DMA instruction x (0 .. 2 NI - 1) of a full tile j: K block x for x < NI, V block x - NI otherwise
  auto issue_one = [&](int j, int x) __attribute__((always_inline)) {
    if (x < NI) {
      const unsigned char* base = kp + (uint64_t)(unsigned)(j * BN + x * NW * RPI) * k_ss;
      dma16s(base, koff, lds0 + (j & 1) * TILE + x * (NW * 1024));
    } else {
      const int i = x - NI;
      const unsigned char* base = vp + (uint64_t)(unsigned)(j * BN + i * NW * RPI) * v_ss;
      dma16s(base, voff, lds0 + VOFF + (j % 3) * TILE + i * (NW * 1024));
    }
  };

  // ---- per-lane LDS read offsets (bytes from the start of K buffer 0 / of V buffer 0) ----
  const int L = lane & 15, G = lane >> 4;
  const int v_row = 4 * g + (L >> 2);
  auto kaddr0 = [&](int ks) __attribute__((always_inline)) { return c32 * ROWB + (((2 * ks + g) ^ swzK<DP>(c32)) * 16); };
  auto vaddr0 = [&](int mb) __attribute__((always_inline)) {
    return VOFF + v_row * ROWB + (L & 1) * 8 + (((4 * mb + 2 * (G & 1) + ((L & 3) >> 1)) ^ swzV<DP>(v_row)) * 16);
  };
  const float c = a.scale_log2;
  const float lazy = kLazyLog2 / c;  // threshold in score units

  for (int own = 0; own < n_own; ++own) {
  const int m0 = (own == 0 ? blk_first : pslot) * BM;
  int n_end = Lk;
  if (a.is_causal) n_end = min(Lk, m0 + BM + off);
  if (n_end < 0) n_end = 0;
  const int ntiles = (n_end + BN - 1) / BN;  // tiles the workgroup moves
  const int wave_row_lo = m0 + 32 * NH * wave, wave_row_hi = wave_row_lo + 32 * NH - 1;
  // 32-key blocks this wavefront computes: [0, nu_w); blocks past the causal diagonal of its last row are left out
  int nu_w = (n_end + 31) / 32;
  if (a.is_causal) nu_w = min(nu_w, max(0, (wave_row_hi + off) / 32 + 1));
  if ((a.is_causal && wave_row_hi + off < 0) || wave_row_lo >= Lq) nu_w = 0;
  int rowX[NH];
#pragma unroll
  for (int X = 0; X < NH; ++X) rowX[X] = wave_row_lo + 32 * X + c32;
  if (own) __syncthreads();  // the previous block's last LDS reads are done
  if (ntiles > 0) issue_tile(0);

  // ---- Q fragments (B operand) of the two halves: lane (c32, g) holds Q[row][16 ks + 8 g .. +8]; O = 0.
  //      Addresses are a scalar base (the block's first row) plus one 32-bit offset per lane and half, so that the
  //      loads of all k-steps differ by an immediate only (the launcher keeps 256 rows x stride within 32 bits) ----
  {
    const unsigned flip = a.neg_scale ? 0x80008000u : 0u;
    const unsigned char* qblk = qp + (int64_t)m0 * a.q_ss;
    static_for<0, NH>([&](auto xc) {
      constexpr int X = decltype(xc)::value;
      const unsigned qoff = (unsigned)(min(rowX[X], Lq - 1) - m0) * (unsigned)a.q_ss + 16 * g;
      static_for<0, KS>([&](auto ksc) {
        constexpr int ks = decltype(ksc)::value;
        u32x4 x;
        if (D == DP) {
          x = *(const u32x4*)(qblk + qoff + 32 * ks);
        } else {  // head_dim below the padded one: chunks beyond it are zeros (and are not read)
          const bool in = (2 * ks + g) * 8 < D;
          x = *(const u32x4*)(qblk + (in ? qoff + 32 * ks : qoff - 16 * g));
          if (!in) x = u32x4{0, 0, 0, 0};
        }
        x ^= flip;
        static_for<0, 4>([&](auto ec) {
          constexpr int e = decltype(ec)::value;
          const unsigned word = x[e];  // (a bit cast applied to the vector element itself reads element 0)
          if constexpr (ACC) acc_write<kQBase + 4 * (X * KS + ks) + e>(__builtin_bit_cast(float, word));
        });
        if constexpr (!ACC) qf[X][ks] = __builtin_bit_cast(s16x8, x);
        if constexpr (ks % 4 == 3) __builtin_amdgcn_sched_barrier(0);  // at most four loads of a half in flight
      });
    });
    if constexpr (ACC) {
      static_for<0, NH * MB * 16>([&](auto ic) { acc_write<kOBase + decltype(ic)::value>(0.f); });
    } else {
#pragma unroll
      for (int X = 0; X < NH; ++X)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int v = 0; v < 16; ++v) o[X][mb][v] = 0.f;
    }
  }
  float m_run[NH], l_run[NH], mc[NH];
  int causal_row_lim[NH];
#pragma unroll
  for (int X = 0; X < NH; ++X) {
    m_run[X] = -INFINITY;
    l_run[X] = mc[X] = 0.f;
    causal_row_lim[X] = a.is_causal ? rowX[X] + off : 0x7fffffff;
  }

  // S accumulators of two consecutive 32-key blocks: S[block parity][half]
  f32x16 S[2][NH];
  // LDS read addresses of the tiles in use: K of tile j; V of tile j and of tile j - 1
  int kcur[KS], vcur[MB], vprev[MB];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) kcur[ks] = kaddr0(ks);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) vcur[mb] = vprev[mb] = vaddr0(mb);

  // State of the unit in flight, shared by its two phases.  Unit u = 2 j + BK: phase 1 computes S(u) from K rows
  // 32 BK .. of tile j, phase 2 finishes block u - 1 (P from S[BK ^ 1], V rows of tile j - 1 for BK == 0, of tile j
  // otherwise); the vector ALU forms P(u - 1) between the MFMAs of both phases.
  u32x4 w[2][NH];    // P^T operands of block u - 1: [16-key chunk][half]
  float tq[2][4];    // two quads of probabilities in the making
  float rs[NH];      // row sums of block u - 1
  float mx[NH];      // row maxima of S(u)
  s16x8 ka_pre[KPRE];  // K fragments of the next phase 1 (its first k-steps), fetched during phase 2
  s16x8 va_pre[MB];  // V^T fragments of the next phase 2 (first chunk), fetched during phase 1

  constexpr int NVS = 16 * NH;             // vector slots of a block (4 per quad)
  constexpr int NV1 = NH == 2 ? 18 : 11;   // ... of them in phase 1: the first chunk's operands must be complete there
  constexpr int NMS = 3 * NH;              // row-maximum pieces
  // ---- vector stream of block u - 1: quads of 4 probabilities, chunk-major (16-key chunk cl, half X, which 4 of
  //      the lane's 8 values), each in 4 phases so that dependent operations sit one MFMA apart:
  //      0: x c - m c   1, 2: exp2   3: row sum + pack to the MFMA operand type ----
  auto vslot = [&](auto bkc, auto nc) __attribute__((always_inline)) {
    constexpr int BK = decltype(bkc)::value;
    constexpr int n = decltype(nc)::value;
    // slot order: F(0) E1(0) E2(0) F(1) P(0) E1(1) E2(1) F(2) P(1) ... E1(n) E2(n) P(n): the operations that depend
    // on each other (F -> E1, E2 -> P) always have another quad's work between them
    // (with a single quad buffer, NH == 1: F(q) E1(q) E2(q) P(q) in turn)
    constexpr int kind = !XPRE ? n % 4
                               : (n < 3 ? n : (n == NVS - 1 ? 3 : ((n - 3) % 4 == 0 ? 0 : ((n - 3) % 4 == 1 ? 3 : (n - 3) % 4 - 1))));
    constexpr int Q = !XPRE ? n / 4
                            : (n < 3 ? 0 : (n == NVS - 1 ? NVS / 4 - 1 : ((n - 3) % 4 == 1 ? (n - 3) / 4 : (n - 3) / 4 + 1)));
    constexpr int cl = Q / (2 * NH), X = (Q / 2) % NH, hf = Q % 2;
    constexpr int v0 = 8 * cl + 4 * hf;
    float(&t)[4] = tq[XPRE ? (Q & 1) : 0];
    f32x16(&Sp)[NH] = S[BK ^ 1];
    if constexpr (kind == 0) {
#pragma unroll
      for (int e = 0; e < 4; ++e) t[e] = Sp[X][v0 + e] * c - mc[X];
      pin(t[0], t[1], t[2], t[3]);
    } else if constexpr (kind == 1) {
      t[0] = fast_exp2(t[0]);
      t[1] = fast_exp2(t[1]);
      pin(t[0], t[1]);
    } else if constexpr (kind == 2) {
      t[2] = fast_exp2(t[2]);
      t[3] = fast_exp2(t[3]);
      pin(t[2], t[3]);
    } else {
      unsigned w0 = Mma<T>::pack2(t[0], t[1]), w1 = Mma<T>::pack2(t[2], t[3]);
      if constexpr (Mma<T>::kSumPacked) {
        rs[X] = Mma<T>::add_pair(w0, rs[X]);
        rs[X] = Mma<T>::add_pair(w1, rs[X]);
      } else {
        rs[X] += (t[0] + t[1]) + (t[2] + t[3]);
      }
      pin(w0, w1, rs[X]);
      w[cl][X][2 * hf] = w0;
      w[cl][X][2 * hf + 1] = w1;
    }
  };
  // ---- row maxima of S(u), in pieces of a few operations ----
  auto mslot = [&](auto bkc, auto nc) __attribute__((always_inline)) {
    constexpr int BK = decltype(bkc)::value;
    constexpr int n = decltype(nc)::value;
    constexpr int X = n % NH, part = n / NH;
    const f32x16& s = S[BK][X];
    if constexpr (part == 0) {
      mx[X] = max3(s[0], s[1], s[2]);
      mx[X] = max3(mx[X], s[3], s[4]);
      mx[X] = max3(mx[X], s[5], s[6]);
      pin(mx[X]);
    } else if constexpr (part == 1) {
      mx[X] = max3(mx[X], s[7], s[8]);
      mx[X] = max3(mx[X], s[9], s[10]);
      mx[X] = max3(mx[X], s[11], s[12]);
      pin(mx[X]);
    } else {
      mx[X] = max3(mx[X], s[13], s[14]);
      mx[X] = fmaxf(mx[X], s[15]);
      mx[X] = pair_max32(mx[X]);
      pin(mx[X]);
    }
  };

  // V^T fragment of 16-key chunk t (0 .. 3 inside its tile) for 32-row block mb of O^T
  auto vfrag = [&](const int(&vad)[MB], int mb, int t) __attribute__((always_inline)) {
    const s16x4 lo = lds_read_tr(smem + vad[mb] + (16 * t) * ROWB);
    const s16x4 hi = lds_read_tr(smem + vad[mb] + (16 * t + 8) * ROWB);
    return s16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };

  // ---- phase 1 of unit u: S(u)^T = K Q^T for both halves (K fragments two k-steps ahead; the first two came with
  //      the previous phase 2); the first V^T fragments of phase 2 are requested here ----
  auto phase1 = [&](int u, auto bkc, auto dosc, auto dopvc) __attribute__((always_inline)) {
    constexpr int BK = decltype(bkc)::value;
    constexpr bool DO_S = decltype(dosc)::value, DO_PV = decltype(dopvc)::value;
    constexpr int NV = DO_PV ? NV1 : 0;
    f32x16(&Sc)[NH] = S[BK];
#pragma unroll
    for (int X = 0; X < NH; ++X) rs[X] = 0.f;
    if constexpr (DO_PV && XPRE) {
      constexpr int TB = 2 * (BK ^ 1);  // first 16-key chunk of block u - 1 inside its tile
      const int(&vad)[MB] = BK == 0 ? vprev : vcur;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) va_pre[mb] = vfrag(vad, mb, TB);
    }
    if constexpr (DO_S) {
      s16x8 ka[KPRE];
#pragma unroll
      for (int i = 0; i < KPRE; ++i) {
        if constexpr (XPRE) ka[i] = ka_pre[i];
        else ka[i] = *(const s16x8*)(smem + kcur[i] + 32 * BK * ROWB);
      }
      static_for<0, KS>([&](auto ksc) {
        constexpr int ks = decltype(ksc)::value;
        static_for<0, NH>([&](auto xc) {
          constexpr int X = decltype(xc)::value;
          constexpr int mi = NH * ks + X;  // MFMA index in this phase
          if constexpr (ACC) {
            if constexpr (ks == 0) s_mma_first<T, kQBase + 4 * (X * KS)>(Sc[X], ka[0]);
            else s_mma<T, kQBase + 4 * (X * KS + ks)>(Sc[X], ka[ks % KPRE]);
          } else {
            if constexpr (ks == 0) {
              f32x16 z;
#pragma unroll
              for (int v = 0; v < 16; ++v) z[v] = 0.f;
              Sc[X] = Mma<T>::m32(ka[0], qf[X][0], z);
            } else {
              Sc[X] = Mma<T>::m32(ka[ks % KPRE], qf[X][ks], Sc[X]);
            }
          }
          static_for<(mi * NV) / NS, ((mi + 1) * NV) / NS>([&](auto nc) { vslot(bkc, nc); });
          if constexpr (X == NH - 1 && ks + KPRE < KS)
            ka[ks % KPRE] = *(const s16x8*)(smem + kcur[ks + KPRE] + 32 * BK * ROWB);
          __builtin_amdgcn_sched_barrier(0);
        });
      });
      if constexpr (!DO_PV) mfma_drain();
      // mask S(u) (tail of K, causal diagonal): rare, wave-uniform
      const int kb0 = u * 32;  // first key of the block
      const bool need_mask = (kb0 + 32 > Lk) || (a.is_causal && kb0 + 31 > wave_row_lo + off);
      if (need_mask) {
        mfma_drain();
#pragma unroll
        for (int X = 0; X < NH; ++X) {
          const int lim = min(last_k, causal_row_lim[X]) - kb0 - 4 * g;  // element index e is visible iff e <= lim
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int e = 8 * (v >> 2) + (v & 3);
            if (e > lim) Sc[X][v] = -INFINITY;
          }
        }
      }
    } else {
      static_for<0, NV>([&](auto nc) { vslot(bkc, nc); });
    }
  };

  // ---- phase 2 of unit u: O^T += V^T P^T of block u - 1 for both halves, 16-key chunk by chunk; the rest of the
  //      vector stream and the row maxima of S(u) run between the MFMAs; then the lazy rescale.  PRE_K: 0 = no K
  //      prefetch, 1 = the first K fragments of the next unit, same tile (BK == 0), 2 = of the next tile (BK == 1).
  //      SPREAD: the DMA of tile jn is issued between the MFMAs ----
  auto phase2 = [&](int u, auto bkc, auto dosc, auto dopvc, auto prekc, auto spreadc, int jn) __attribute__((always_inline)) {
    constexpr int BK = decltype(bkc)::value;
    constexpr bool DO_S = decltype(dosc)::value, DO_PV = decltype(dopvc)::value, SPREAD = decltype(spreadc)::value;
    constexpr int PRE_K = decltype(prekc)::value;
    constexpr int NM = DO_S ? NMS : 0;
    auto prefetch_k = [&]() __attribute__((always_inline)) {
      if constexpr (!XPRE) {
      } else if constexpr (PRE_K == 1) {
#pragma unroll
        for (int i = 0; i < KPRE; ++i) ka_pre[i] = *(const s16x8*)(smem + kcur[i] + 32 * ROWB);
      } else if constexpr (PRE_K == 2) {
#pragma unroll
        for (int i = 0; i < KPRE; ++i) ka_pre[i] = *(const s16x8*)(smem + (kcur[i] ^ TILE));
      }
    };
    if constexpr (DO_PV) {
      constexpr int TB = 2 * (BK ^ 1);
      const int(&vad)[MB] = BK == 0 ? vprev : vcur;
      // the first chunk's V^T fragments came with phase 1; each is replaced by the second chunk's as soon as the
      // last half has used it
      s16x8 va[MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        if constexpr (XPRE) va[mb] = va_pre[mb];
        else va[mb] = vfrag(vad, mb, TB);
      }
      // vector slots: over the MFMAs before the last half's second chunk, whose P^T operand is the last to complete;
      // row-maximum pieces: over the second half
      constexpr int NV2 = NVS - NV1, NPV = NP - MB, NPM = NP / 2;
      static_for<0, 2>([&](auto tc) {
        constexpr int t = decltype(tc)::value;
        if constexpr (t == 1) prefetch_k();
        static_for<0, NH * MB>([&](auto ic) {
          constexpr int i = decltype(ic)::value;
          constexpr int X = i / MB, mb = i % MB;
          constexpr int mi = t * NH * MB + i;
          if constexpr (ACC) pv_mma<T, kOBase + 16 * (X * MB + mb)>(va[mb], __builtin_bit_cast(s16x8, w[t][X]));
          else o[X][mb] = Mma<T>::m32(va[mb], __builtin_bit_cast(s16x8, w[t][X]), o[X][mb]);
          if constexpr (t == 0 && X == NH - 1) va[mb] = vfrag(vad, mb, TB + 1);
          if constexpr (mi < NPV)
            static_for<(mi * NV2) / NPV, ((mi + 1) * NV2) / NPV>([&](auto nc) { vslot(bkc, IC<NV1 + decltype(nc)::value>{}); });
          if constexpr (mi >= NP - NPM)
            static_for<((mi - (NP - NPM)) * NM) / NPM, ((mi - (NP - NPM) + 1) * NM) / NPM>([&](auto nc) { mslot(bkc, nc); });
          if constexpr (SPREAD) {
#pragma unroll
            for (int x = (mi * 2 * NI) / NP; x < ((mi + 1) * 2 * NI) / NP; ++x) issue_one(jn, x);
          }
          __builtin_amdgcn_sched_barrier(0);
        });
      });
#pragma unroll
      for (int X = 0; X < NH; ++X) l_run[X] += rs[X];
    } else {
      prefetch_k();
      if constexpr (DO_S) static_for<0, NM>([&](auto nc) { mslot(bkc, nc); });
    }

    // lazy rescale: only when some row's maximum outgrew the one in use by more than 2^kLazyLog2
    if constexpr (DO_S) {
      bool grow[NH], any_grow = false, any_live = false;
#pragma unroll
      for (int X = 0; X < NH; ++X) {
        grow[X] = mx[X] > m_run[X] + lazy;
        any_grow = any_grow || grow[X];
        any_live = any_live || m_run[X] != -INFINITY;
      }
      if (__builtin_amdgcn_ballot_w64(any_grow) != 0) {
        mfma_drain();
        // nothing has been accumulated yet while every row's maximum is still -inf
        const bool o_live = __builtin_amdgcn_ballot_w64(any_live) != 0;
        static_for<0, NH>([&](auto xc) {
          constexpr int X = decltype(xc)::value;
          const float m_new = grow[X] ? mx[X] : m_run[X];
          const float alpha = grow[X] ? fast_exp2((m_run[X] - m_new) * c) : 1.0f;  // exp2(-inf) = 0 on the first block
          m_run[X] = m_new;
          l_run[X] *= alpha;
          mc[X] = (m_run[X] == -INFINITY) ? 0.f : m_run[X] * c;
          if (o_live) {
            if constexpr (ACC) {
              static_for<0, MB * 16>([&](auto ic) {
                constexpr int r = kOBase + 16 * MB * X + decltype(ic)::value;
                acc_write<r>(acc_read<r>() * alpha);
              });
            } else {
#pragma unroll
              for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int v = 0; v < 16; ++v) o[X][mb][v] *= alpha;
            }
          }
        });
      }
    }
  };

  // which of the variants of a phase runs is wave-uniform
  auto with_flags = [&](bool do_s, bool do_pv, auto&& f) __attribute__((always_inline)) {
    if (do_s && do_pv) f(IC<1>{}, IC<1>{});
    else if (do_s) f(IC<1>{}, IC<0>{});
    else if (do_pv) f(IC<0>{}, IC<1>{});
  };

  // ---- the pipeline ----------------------------------------------------------------------------------------
  // Tile j + 1 is known to have landed at the synchronisation point of tile j, which sits between the two phases of
  // unit 2 j + 1: by then this wavefront has read all of K(j) and of V(j - 1), so tile j + 2 may be requested right
  // after it (K into the buffer of K(j), V into the buffer of V(j - 1): 2 K and 3 V buffers), and phase 2 of unit
  // 2 j + 1 can already fetch the first K fragments of tile j + 1.
  if (ntiles > 0) {
    WAIT_VMCNT(0);    // tile 0 (and the Q fragments)
    __syncthreads();
    if (ntiles > 1) issue_tile(1);
    if constexpr (XPRE) {
#pragma unroll
      for (int i = 0; i < KPRE; ++i) ka_pre[i] = *(const s16x8*)(smem + kcur[i]);
    }
  }
  for (int j = 0; j < ntiles; ++j) {
    if (j > 0) {  // K buffer j % 2 (the other one), V buffer j % 3 (the next one, cyclically)
      const int dv = (j % 3 == 0) ? -2 * TILE : TILE;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) kcur[ks] ^= TILE;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        vprev[mb] = vcur[mb];
        vcur[mb] += dv;
      }
    }
    {
      const int u = 2 * j;
      const bool do_s = u < nu_w, do_pv = u >= 1 && u - 1 < nu_w;
      with_flags(do_s, do_pv, [&](auto dosc, auto dopvc) __attribute__((always_inline)) {
        phase1(u, IC<0>{}, dosc, dopvc);
        phase2(u, IC<0>{}, dosc, dopvc, IC<1>{}, IC<0>{}, 0);
      });
    }
    {
      const int u = 2 * j + 1;
      const bool do_s = u < nu_w, do_pv = u - 1 < nu_w;
      with_flags(do_s, do_pv, [&](auto dosc, auto dopvc) __attribute__((always_inline)) { phase1(u, IC<1>{}, dosc, dopvc); });
      // synchronisation point of tile j
      const bool more = j + 1 < ntiles, fetch = j + 2 < ntiles;
      if (more) {
        WAIT_VMCNT(0);    // my DMA for tile j + 1 has landed
        __syncthreads();  // everyone's has; everyone is done with K(j) and V(j - 1)
      }
      // full tiles are requested between the MFMAs of phase 2, the last, partial one (rows clamped per lane) and
      // those of wavefronts without a full phase 2 right here
      const bool spread = fetch && do_s && do_pv && (j + 3) * BN <= Lk;
      if (fetch && !spread) issue_tile(j + 2);
      if (more) {
        if (spread)
          phase2(u, IC<1>{}, IC<1>{}, IC<1>{}, IC<2>{}, IC<1>{}, j + 2);
        else
          with_flags(do_s, do_pv, [&](auto dosc, auto dopvc) __attribute__((always_inline)) {
            phase2(u, IC<1>{}, dosc, dopvc, IC<2>{}, IC<0>{}, 0);
          });
      } else {
        with_flags(do_s, do_pv, [&](auto dosc, auto dopvc) __attribute__((always_inline)) {
          phase2(u, IC<1>{}, dosc, dopvc, IC<0>{}, IC<0>{}, 0);
        });
      }
    }
  }
  // drain: the last block's P V (its V tile is still in LDS)
  if (ntiles > 0) {
    const int u = 2 * ntiles;
    if (u - 1 < nu_w) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) vprev[mb] = vcur[mb];
      phase1(u, IC<0>{}, IC<0>{}, IC<1>{});
      phase2(u, IC<0>{}, IC<0>{}, IC<1>{}, IC<0>{}, IC<0>{}, 0);
    }
  }

  // ---- epilogue ----
  mfma_drain();
  static_for<0, NH>([&](auto xc) {
    constexpr int X = decltype(xc)::value;
    const int row = rowX[X];
    const float l = pair_sum32(l_run[X]);
    const float inv = (l > 0.f) ? 1.f / l : 0.f;
    if (row < Lq) {
      // scalar base (the block's first row) + one 32-bit offset per lane + an immediate per store
      unsigned char* oblk = a.out + ob + (int64_t)(q0 + m0) * a.o_ss + (int64_t)h * a.o_sh;
      const unsigned ooff = (unsigned)(row - m0) * (unsigned)a.o_ss + 8 * g;
      static_for<0, MB * 4>([&](auto ic) {
        constexpr int mb = decltype(ic)::value / 4, v4 = decltype(ic)::value % 4;
        constexpr int r = kOBase + 16 * (X * MB + mb) + 4 * v4;
        const int d = 32 * mb + 8 * v4 + 4 * g;
        if (D == DP || d < D) {
          u32x2 ww;
          if constexpr (ACC) {
            ww[0] = Mma<T>::pack2(acc_read<r>() * inv, acc_read<r + 1>() * inv);
            ww[1] = Mma<T>::pack2(acc_read<r + 2>() * inv, acc_read<r + 3>() * inv);
          } else {
            ww[0] = Mma<T>::pack2(o[X][mb][4 * v4 + 0] * inv, o[X][mb][4 * v4 + 1] * inv);
            ww[1] = Mma<T>::pack2(o[X][mb][4 * v4 + 2] * inv, o[X][mb][4 * v4 + 3] * inv);
          }
          *(u32x2*)(oblk + ooff + (64 * mb + 16 * v4)) = ww;
        }
      });
      if (g == 0) {
        const float lse = (l > 0.f) ? (m_run[X] * c + __builtin_log2f(l)) * kLn2 : INFINITY;
        a.lse[lb + (int64_t)h * a.lse_sh + (int64_t)(q0 + row) * a.lse_ss] = lse;
      }
    }
  });
  }  // own
}

template <typename T, int DP, int NH>
int launch(KArgs a, hipStream_t st) {
  constexpr int lds = 5 * 64 * DP * 2;
  constexpr auto kfn = fa_tile256_kernel<T, DP, NH>;
  if (!ensure_dynamic_lds<kfn>(lds)) return FA_ERR_LAUNCH;
  const int nblk = (a.seqlen_q + 255) / 256;
  a.pair = (!a.cu_q && a.is_causal && nblk >= 2) ? 1 : 0;
  a.n_mblk = a.pair ? (nblk + 1) / 2 : nblk;
  a.hgroup = 1;
  const int64_t grid = (int64_t)a.batch * a.heads_q * a.n_mblk;
  if (grid <= 0) return FA_OK;
  if (grid > 0x7fffffffLL) return FA_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kfn, dim3((unsigned)grid), dim3(NH == 2 ? 256 : 512), lds, st, a);
  return hipGetLastError() == hipSuccess ? FA_OK : FA_ERR_LAUNCH;
}

}  // namespace

bool tile256_eligible(const KArgs& a) {
  // the kernel addresses the 256 rows of a query block with 32-bit offsets from the block's first row
  const int64_t lim = 0xffffffffLL / 256;
  return a.head_dim <= 128 && !a.bias && !(a.drop_thr < 255u) && a.n_splits == 1 && a.q_ss <= lim && a.o_ss <= lim;
}

int launch_tile256(const KArgs& a, int dtype, int halves, hipStream_t st) {
  const bool d64 = a.head_dim <= 64;
  if (halves == 2) {
    if (dtype == FA_DTYPE_BF16) return d64 ? launch<__bf16, 64, 2>(a, st) : launch<__bf16, 128, 2>(a, st);
    return d64 ? launch<_Float16, 64, 2>(a, st) : launch<_Float16, 128, 2>(a, st);
  }
  if (dtype == FA_DTYPE_BF16) return d64 ? launch<__bf16, 64, 1>(a, st) : launch<__bf16, 128, 1>(a, st);
  return d64 ? launch<_Float16, 64, 1>(a, st) : launch<_Float16, 128, 1>(a, st);
}

}  // namespace fa
