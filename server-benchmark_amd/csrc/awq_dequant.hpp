// awq_dequantize: fp16 [K, N] = fp16((w - z) * s), bit-exact, write-bound (2 B out per
// 0.53 B in).  One lane owns one packed word column: a 4-byte load becomes one 16-byte
// store, a wave covers 256 B of input and 1 KiB of output per row, and the lane's zero
// word and eight scales stay in registers for ROWS rows of the same group.
//
// Exactness: (nibble | 0x6400) is fp16 1024 + nibble, so the packed subtract gives the
// integer w - z exactly; the single packed fp16 multiply by s rounds the exact product
// once, which is what fp16_rn(float(w - z) * float(s)) does.
//
// Also here: a slow any-shape GEMM used only for shapes outside the tiled kernels.
#pragma once
#include "awq_common.hpp"

namespace awqmi {

__device__ __forceinline__ u4v dequant_word(uint32_t q, const uint32_t (&zz)[4], u4v s) {
  u4v o;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t v = ((q >> (4 * j)) & MASK_LO) | MAGIC_LO;
    const h2 d = (as_h2(v) - as_h2(zz[j])) * as_h2(s[j]);
    o[j] = as_u32(d);
  }
  return o;
}

template <int ROWS>
__global__ __launch_bounds__(256) void awq_dequant_kernel(const uint32_t* __restrict__ qw,
                                                          const half_t* __restrict__ sc,
                                                          const uint32_t* __restrict__ qz,
                                                          half_t* __restrict__ out, int k_base,
                                                          int NW, int G, int ldw) {
  const int wc = blockIdx.x * 256 + threadIdx.x;
  if (wc >= NW) return;
  const size_t N = (size_t)NW * 8;
  const int k0 = k_base + blockIdx.y * ROWS;   // launches cover at most 65535 row slabs each
  const int g = k0 / G;
  const uint32_t z = qz[(size_t)g * NW + wc];
  const u4v s = *reinterpret_cast<const u4v*>(sc + (size_t)g * N + 8 * (size_t)wc);
  uint32_t zz[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) zz[j] = ((z >> (4 * j)) & MASK_LO) | MAGIC_LO;
  uint32_t q[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) q[r] = __builtin_nontemporal_load(qw + (size_t)(k0 + r) * ldw + wc);
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const u4v o = dequant_word(q[r], zz, s);
    __builtin_nontemporal_store(o, reinterpret_cast<u4v*>(out + (size_t)(k0 + r) * N + 8 * (size_t)wc));
  }
}

// Any-shape fallback: one lane per (row m, word column), K walked serially, weights
// dequantised exactly as above, fp32 accumulation.
__global__ __launch_bounds__(256) void awq_gemm_generic_kernel(const half_t* __restrict__ x,
                                                               const uint32_t* __restrict__ qw,
                                                               const half_t* __restrict__ sc,
                                                               const uint32_t* __restrict__ qz,
                                                               half_t* __restrict__ y, int M, int K,
                                                               int NW, int G, int ldw) {
  const int wc = blockIdx.x * 256 + threadIdx.x;
  const int m = blockIdx.y;
  if (wc >= NW || m >= M) return;
  const size_t N = (size_t)NW * 8;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  uint32_t zz[4];
  u4v s = {0, 0, 0, 0};
  for (int k = 0; k < K; ++k) {
    if (k % G == 0) {
      const int g = k / G;
      const uint32_t z = qz[(size_t)g * NW + wc];
      s = *reinterpret_cast<const u4v*>(sc + (size_t)g * N + 8 * (size_t)wc);
#pragma unroll
      for (int j = 0; j < 4; ++j) zz[j] = ((z >> (4 * j)) & MASK_LO) | MAGIC_LO;
    }
    const u4v w = dequant_word(qw[(size_t)k * ldw + wc], zz, s);
    const float xv = (float)x[(size_t)m * K + k];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const h2 p = as_h2(w[j]);
      acc[2 * j] += xv * (float)p.x;
      acc[2 * j + 1] += xv * (float)p.y;
    }
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) y[(size_t)m * N + 8 * (size_t)wc + j] = (half_t)acc[j];
}

}  // namespace awqmi
