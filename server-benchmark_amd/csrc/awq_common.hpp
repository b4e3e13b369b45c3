// Shared device helpers for the AWQ W4A16 kernels (gfx950 / CDNA4, wave64).
//
// AWQ packing: nibble i (bits 4i..4i+3) of the int32 at word-column c holds logical column
// 8c + P[i], P = {0,2,4,6,1,3,5,7}.  Consequences used throughout:
//   * (q >> 4j) & 0x000F000F  -> logical columns (2j, 2j+1) in the (low, high) half-words;
//   * byte b of a word holds columns P[2b] (low nibble) and P[2b+1] (high nibble).
// fp16 "magic" conversion: (nibble | 0x6400) is the fp16 number 1024 + nibble, and a nibble
// left in bits 4..7 under 0x5400 is 64 + nibble (ulp 1/16); subtracting 1024 + z resp.
// 64 + z gives the exact integer w - z with no int->float conversion.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace awqmi {

typedef _Float16 half_t;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef uint32_t u2v __attribute__((ext_vector_type(2)));
typedef uint32_t u4v __attribute__((ext_vector_type(4)));

constexpr uint32_t MAGIC_LO = 0x64006400u;   // 1024.0 in both halves
constexpr uint32_t MAGIC_HI = 0x54005400u;   // 64.0 in both halves
constexpr uint32_t MASK_LO = 0x000F000Fu;
constexpr uint32_t MASK_HI = 0x00F000F0u;

__device__ __forceinline__ h2 as_h2(uint32_t v) { return __builtin_bit_cast(h2, v); }
__device__ __forceinline__ uint32_t as_u32(h2 v) { return __builtin_bit_cast(uint32_t, v); }
__device__ __forceinline__ h8 as_h8(u4v v) { return __builtin_bit_cast(h8, v); }
__device__ __forceinline__ u4v as_u4(h8 v) { return __builtin_bit_cast(u4v, v); }

// Nibble masks held in VGPRs on purpose: with the mask in a register and the magic constant
// in an SGPR, (t & mask) | magic is a single v_and_or_b32 (a VOP3 op may read one scalar
// constant only); as literals the compiler has to emit v_and + v_or.
struct NibbleMasks {
  uint32_t lo, hi;
  __device__ __forceinline__ void init() {
    asm volatile("v_mov_b32 %0, 0x000f000f" : "=v"(lo));
    asm volatile("v_mov_b32 %0, 0x00f000f0" : "=v"(hi));
  }
};

// packed fp16 subtract / multiply on raw 32-bit lanes (v_pk_add_f16 / v_pk_mul_f16)
__device__ __forceinline__ uint32_t pk_sub(uint32_t a, uint32_t b) { return as_u32(as_h2(a) - as_h2(b)); }
__device__ __forceinline__ uint32_t pk_mul(uint32_t a, uint32_t b) { return as_u32(as_h2(a) * as_h2(b)); }

// logical column (0..7) held by nibble `nib` of a packed word
__host__ __device__ constexpr int awq_col_of_nibble(int nib) {
  return nib < 4 ? 2 * nib : 2 * (nib - 4) + 1;
}
// nibble holding logical column j
__host__ __device__ constexpr int awq_nibble_of_col(int j) { return (j & 1) ? 4 + (j >> 1) : (j >> 1); }

// byte b of `lo` into half-word 0 and byte b of `hi` into half-word 1, upper bytes zero
template <int B>
__device__ __forceinline__ uint32_t byte_pair(uint32_t hi, uint32_t lo) {
  constexpr uint32_t sel = 0x0c000c00u | (uint32_t)B | ((uint32_t)(4 + B) << 16);
  return __builtin_amdgcn_perm(hi, lo, sel);
}

// Fill kernel: n 16-byte words of zeros (one thread per word).  Used instead of memset nodes
// for the arrival counters, so that a captured call replays the same way as an eager one.
__global__ __launch_bounds__(256) void awq_zero_words_kernel(u4v* __restrict__ p, unsigned n) {
  const unsigned i = blockIdx.x * 256u + threadIdx.x;
  if (i < n) p[i] = u4v{0u, 0u, 0u, 0u};
}

}  // namespace awqmi
