// Device-side helpers shared by the forward and backward kernels (gfx950 only).
#ifndef FA_DEVICE_H_
#define FA_DEVICE_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace fa {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

#define LDS_AS __attribute__((address_space(3)))
#define GLB_AS __attribute__((address_space(1)))

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

template <typename T>
struct Mma;
template <>
struct Mma<__bf16> {
  static __device__ __forceinline__ f32x16 m32(s16x8 a, s16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 m16(s16x8 a, s16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ unsigned pack2(float a, float b) {
    f32x2 f = {a, b};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f, bf16x2));
  }
  static __device__ __forceinline__ float to_float(unsigned short bits) { return __builtin_bit_cast(float, (unsigned)bits << 16); }
  // A pair of probabilities is summed in fp32 before it is rounded: bf16 keeps 8 bits, and a row sum of rounded
  // values could be off by 2^-9 relative when one key dominates, which the logsumexp would show.
  static constexpr bool kSumPacked = false;
  static __device__ __forceinline__ float add_pair(unsigned, float acc) { return acc; }
  static constexpr unsigned short kOne = 0x3f80;     // 1.0
  static constexpr unsigned short kNegMax = 0xff7f;  // the most negative finite value; -inf is the next bit pattern
};
template <>
struct Mma<_Float16> {
  static __device__ __forceinline__ f32x16 m32(s16x8 a, s16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 m16(s16x8 a, s16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ unsigned pack2(float a, float b) {
    f32x2 f = {a, b};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f, f16x2));
  }
  static __device__ __forceinline__ float to_float(unsigned short bits) { return (float)__builtin_bit_cast(_Float16, bits); }
  // fp16 keeps 11 bits: the row sum is taken over the packed, rounded pair with one v_dot2c_f32_f16 (pair . (1, 1)
  // + acc, fp32 accumulation) instead of two fp32 adds; the sum is then also exactly that of the values the PV
  // product uses.  Worst-case relative error of a row sum 2^-12.
  static constexpr bool kSumPacked = true;
  static __device__ __forceinline__ float add_pair(unsigned w, float acc) {
    const f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, w), ones, acc, false);
  }
  static constexpr unsigned short kOne = 0x3c00;
  static constexpr unsigned short kNegMax = 0xfbff;
};

// 16-byte global -> LDS DMA.  Lane i of the wavefront writes LDS bytes [lds_wave_base + 16 i, +16); the global
// address is per lane.  lds_wave_base must be wavefront-uniform.  Written as inline assembly on purpose: the
// compiler then does not know these loads write LDS, so it does not put a conservative "wait for every
// outstanding load" in front of the LDS reads of the tile being computed.  Completion is tracked by hand
// with WAIT_VMCNT (the loads retire in order).
__device__ __forceinline__ void dma16(const unsigned char* gptr, unsigned char* lds_wave_base) {
  const unsigned lds = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)(LDS_AS unsigned char*)lds_wave_base);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds), "v"(gptr) : "memory", "m0");
}

// Same, with the global address split into a wavefront-uniform 64-bit base (scalar registers) and a per-lane
// 32-bit byte offset, and the LDS destination given as a wavefront-uniform LDS byte address.
__device__ __forceinline__ void dma16s(const unsigned char* sbase, unsigned voff, unsigned lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_wave_base), "v"(voff), "s"(sbase)
               : "m0");
}

// Same, with a per-lane 64-bit global address and the LDS destination given as a wavefront-uniform LDS byte address.
__device__ __forceinline__ void dma16v(const unsigned char* gptr, unsigned lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_wave_base), "v"(gptr) : "m0");
}

// Transposed LDS read: within each group of 16 lanes, lane j receives element (j % 4) of the four 8-byte pieces
// addressed by lanes 4 i + j / 4 (i = 0..3) of the same group.
__device__ __forceinline__ s16x4 lds_read_tr(const unsigned char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 LDS_AS*)p);
}

// the same through a pointer that is already an LDS address
__device__ __forceinline__ s16x4 lds_read_tr_lds(LDS_AS const unsigned char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 LDS_AS*)p);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// max of two as one instruction (fmaxf first canonicalises both operands: three instructions)
__device__ __forceinline__ float max2(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
// max over the lane pair (l, l ^ 32)
__device__ __forceinline__ float pair_max32(float x) {
  unsigned u = __builtin_bit_cast(unsigned, x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return max2(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
}
__device__ __forceinline__ float pair_sum32(float x) {
  unsigned u = __builtin_bit_cast(unsigned, x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
}

#define WAIT_VMCNT(n) asm volatile("s_waitcnt vmcnt(" #n ")" ::: "memory")

template <int N>
struct IC {
  static constexpr int value = N;
};

// f(IC<B>{}), f(IC<B + 1>{}), ..., f(IC<E - 1>{}): a loop whose index is a compile-time constant in the body
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(IC<B>{});
    static_for<B + 1, E>(f);
  }
}

__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
// the same, ordered behind the instruction that produced `after` (an input the instruction does not use)
__device__ __forceinline__ float max3d(float a, float b, float c, float after) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c), "v"(after));
  return r;
}

// ---- dropout ---------------------------------------------------------------------------------------------
// One 32-bit word per 2 x 2 patch of the attention matrix of one (sequence, query head); element (row, col) keeps its
// probability iff byte 2 (row & 1) + (col & 1) of the patch's word is <= the threshold.  The word is a murmur3
// finaliser over a counter that is unique per patch while both pair indices are below 65536 (beyond that the high
// parts are folded in), so forward and backward — whose lanes own different elements — regenerate the same mask from
// (seed, offset, sequence, head, row, col) alone.  A (sequence, head) has two 32-bit keys: the first is XORed into the
// counter, the second is added between the finaliser's two multiplications, so the masks of two heads are not
// translates of one another (with the first key alone, head h' would see head h's table with its row and column pair
// indices XORed by a constant).
__device__ __forceinline__ uint32_t drop_mix(uint32_t h) {
  h ^= h >> 16;
  h *= 0x85ebca6bu;
  h ^= h >> 13;
  h *= 0xc2b2ae35u;
  h ^= h >> 16;
  return h;
}
__device__ __forceinline__ uint32_t drop_word(uint32_t counter, uint32_t key2) {
  uint32_t h = counter;
  h ^= h >> 16;
  h *= 0x85ebca6bu;
  h = (h ^ (h >> 13)) + key2;
  h *= 0xc2b2ae35u;
  h ^= h >> 16;
  return h;
}
// keys of one (sequence b, query head h) of one call: bh = b * heads_q + h
struct DropKeys {
  uint32_t k1, k2;
};
__device__ __forceinline__ DropKeys drop_head_keys(uint64_t seed, uint64_t offset, uint32_t bh) {
  uint32_t k = drop_mix((uint32_t)seed ^ 0x2545f491u) + (uint32_t)(seed >> 32);
  k = drop_mix(k) ^ (uint32_t)offset;
  k = drop_mix(k) + (uint32_t)(offset >> 32);
  uint32_t m = drop_mix((uint32_t)(seed >> 32) ^ 0x3c6ef372u) + (uint32_t)seed;
  m = drop_mix(m) ^ (uint32_t)(offset >> 32);
  m = drop_mix(m) + (uint32_t)offset;
  return DropKeys{drop_mix(k ^ (bh * 0x9e3779b1u + 0x7f4a7c15u)), drop_mix(m ^ (bh * 0x85ebca77u + 0x165667b1u))};
}
// the part of a patch's counter that depends on its row pair / on its column pair; the counter is their XOR with the key
__device__ __forceinline__ uint32_t drop_row_term(uint32_t rowpair) { return (rowpair << 16) ^ ((rowpair >> 16) * 0x9e3779b1u); }
__device__ __forceinline__ uint32_t drop_col_term(uint32_t colpair) { return (colpair & 0xffffu) ^ ((colpair >> 16) * 0x7f4a7c15u); }

// ---- host: opt a kernel into more than 64 KiB of dynamic LDS, once per kernel and device ---------------------
template <auto KFN>
inline bool ensure_dynamic_lds(int bytes) {
  static std::atomic<uint64_t> done{0};  // bit d: set for device d
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  const uint64_t bit = dev < 64 ? (uint64_t)1 << dev : 0;
  if (bit && (done.load(std::memory_order_acquire) & bit)) return true;
  if (hipFuncSetAttribute((const void*)KFN, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  done.fetch_or(bit, std::memory_order_release);
  return true;
}

}  // namespace fa

#endif  // FA_DEVICE_H_
