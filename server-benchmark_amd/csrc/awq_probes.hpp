// Measurement probes behind the development entry points: the ceilings the kernels are priced
// against, measured on the machine instead of quoted.
//   * awq_stream_probe_kernel: the skinny kernel's weight access pattern with the arithmetic
//     removed (what HBM delivers for that pattern), or a plain linear read;
//   * awq_mfma_probe_kernel: a bare loop of fp16 MFMAs on random operands held in registers (what
//     the matrix pipe sustains under the chip's power limit, per instruction shape).
#pragma once
#include "awq_common.hpp"

namespace awqmi {

// PATTERN 0: the skinny kernel's pattern on a [K, ldw] word matrix.  Workgroup (cb, part): column
// block cb (256 columns = one 128-byte line per row), K range `part` of `parts`; its four waves
// take quarters of that range in 128-row chunks; a lane loads the 8 bytes (two packed words) of
// row 8 h + i, i = 0 .. 7, that the kernel's lane would, four 32-row steps in flight.
// PATTERN 1: every wave reads one contiguous slab, 1 KiB per instruction, 16 KiB in flight.
// Loaded words are folded into one value per lane and stored, so nothing is optimised away.
template <int PATTERN>
__global__ __launch_bounds__(256, 1) void awq_stream_probe_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ out,
                                                                  int K, int ldw, int parts, size_t total_bytes) {  // ldw: row pitch in words
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  u2v fold = {0u, 0u};
  if constexpr (PATTERN == 0 || PATTERN == 2) {
    const int cb = blockIdx.x, part = blockIdx.y;
    const int j = lane & 15, h = lane >> 4;
    const int nchunks = K >> 7;
    const unsigned pw = (unsigned)part * 4u + (unsigned)wave, np = (unsigned)parts * 4u;
    const int c0 = (int)(pw * (unsigned)nchunks / np), c1 = (int)((pw + 1) * (unsigned)nchunks / np);
    // PATTERN 2: the same reads on a column-block-major copy of the matrix (the K x 128 bytes of a
    // column block contiguous, rows 128 bytes apart)
    const char* base = PATTERN == 2 ? reinterpret_cast<const char*>(src) + ((size_t)cb * K * 32 + (size_t)(8 * h) * 32 + 2 * j) * 4
                                    : reinterpret_cast<const char*>(src) + ((size_t)(8 * h) * ldw + cb * 32 + 2 * j) * 4;
    if (PATTERN == 2) ldw = 32;
    u2v q[4][8];
    auto issue = [&](int d, int step) {
      const char* rb = base + (size_t)step * 32 * ldw * 4;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        q[d][i] = __builtin_nontemporal_load(reinterpret_cast<const u2v*>(rb + (size_t)i * ldw * 4));
    };
    const int s0 = 4 * c0, s1 = 4 * c1;
    if (s1 > s0) {
#pragma unroll
      for (int d = 0; d < 4; ++d) issue(d, s0 + d);      // ranges are whole chunks: at least four steps
      for (int s = s0; s < s1; s += 4) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
#pragma unroll
          for (int i = 0; i < 8; ++i) fold ^= q[d][i];
          __builtin_amdgcn_sched_barrier(0);
          issue(d, min(s + 4 + d, s1 - 1));              // past the end: the last step again
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  } else {
    const size_t nwaves = (size_t)gridDim.x * 4;
    const size_t wid = (size_t)blockIdx.x * 4 + wave;
    const size_t kib = total_bytes >> 10;
    const size_t k0 = wid * kib / nwaves, k1 = (wid + 1) * kib / nwaves;
    const char* base = reinterpret_cast<const char*>(src) + (size_t)lane * 16;
    u4v q[16];
    if (k1 > k0) {
#pragma unroll
      for (int d = 0; d < 16; ++d) q[d] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(base + ((k0 + d < k1 ? k0 + d : k1 - 1) << 10)));
      for (size_t k = k0; k < k1; k += 16) {
#pragma unroll
        for (int d = 0; d < 16; ++d) {
          fold[0] ^= q[d][0] ^ q[d][2];
          fold[1] ^= q[d][1] ^ q[d][3];
          __builtin_amdgcn_sched_barrier(0);
          const size_t kn = k + 16 + d;
          q[d] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(base + ((kn < k1 ? kn : k1 - 1) << 10)));
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  }
  out[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 256 + tid] = fold[0] ^ fold[1];
}

// SHAPE 0: v_mfma_f32_32x32x16_f16, 4 x 4 accumulator tiles per wave; SHAPE 1: v_mfma_f32_16x16x32_f16,
// 8 x 8 tiles: the two ways to hold a 128 x 128 wave tile.  Two fragment sets of random fp16 values
// (read once from src: 64 KiB per workgroup) alternate, so consecutive k-steps see different
// operands as they do in a GEMM; the MFMAs of a k-step run over 2 x 2 blocks of accumulator tiles so
// that one operand changes from one instruction to the next (the order that sustains the most under
// the power limit: 3 % over row-major, 6 % over an order that changes both operands every time).
// One iteration = 2 k-steps = 2 x 128 x 128 x 32 x 2 = 2097152 flop per wave.
template <int SHAPE>
__global__ __launch_bounds__(256, 1) void awq_mfma_probe_kernel(const uint32_t* __restrict__ src, float* __restrict__ out,
                                                                int iters) {
  const int tid = threadIdx.x, lane = tid & 63;
  const u4v* base = reinterpret_cast<const u4v*>(src) + ((size_t)blockIdx.x * 4 + (tid >> 6)) * 1024;
  float total = 0.f;
  if constexpr (SHAPE == 0) {
    f16v acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    h8 a[2][4], b[2][4];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a[s][i] = as_h8(base[(s * 8 + i) * 64 + lane]);
        b[s][i] = as_h8(base[(s * 8 + 4 + i) * 64 + lane]);
      }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
          for (int blk = 0; blk < 4; ++blk) {   // 2 x 2 blocks of tiles, one operand changing per MFMA
            const int i = 2 * (blk >> 1), j = (blk & 2) ? 2 - 2 * (blk & 1) : 2 * (blk & 1);
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[s ^ ks][i], b[s][j], acc[i][j], 0, 0, 0);
            acc[i + 1][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[s ^ ks][i + 1], b[s][j], acc[i + 1][j], 0, 0, 0);
            acc[i + 1][j + 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[s ^ ks][i + 1], b[s][j + 1], acc[i + 1][j + 1], 0, 0, 0);
            acc[i][j + 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[s ^ ks][i], b[s][j + 1], acc[i][j + 1], 0, 0, 0);
          }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) total += acc[i][j][r];
  } else {
    f4 acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};
    h8 a[2][8], b[2][8];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        a[s][i] = as_h8(base[((s * 16 + i) * 64 + lane) & 1023]);
        b[s][i] = as_h8(base[((s * 16 + 8 + i) * 64 + lane) & 1023]);
      }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int blk = 0; blk < 16; ++blk) {    // the dense GEMM kernel's order: 2 x 2 blocks of tiles, block rows forth and back
          const int i = 2 * (blk >> 2), j = (blk & 4) ? 6 - 2 * (blk & 3) : 2 * (blk & 3);
          asm("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(a[s][i]), "v"(b[s][j]));
          asm("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i + 1][j]) : "v"(a[s][i + 1]), "v"(b[s][j]));
          asm("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i + 1][j + 1]) : "v"(a[s][i + 1]), "v"(b[s][j + 1]));
          asm("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j + 1]) : "v"(a[s][i]), "v"(b[s][j + 1]));
        }
    }
    asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) total += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
  }
  out[(size_t)blockIdx.x * 256 + tid] = total;
}

}  // namespace awqmi
