// Skinny AWQ GEMM (16 rows per row block, one or two row blocks per pass): Y[M,N] = X[M,K] @
// dequant(W), HBM-bound.
//
// One wave owns a block of 128*WPL output columns and a contiguous range of 128-row chunks
// of K.  Per 32-row step each lane loads 8 rows x WPL packed words (16 lanes side by side
// cover 64*WPL contiguous bytes of a row, the four 16-lane groups take four 8-row slabs) and
// turns the 8x8 nibble block of every word into B operands of v_mfma_f32_16x16x32_f16 without
// converting anything: a nibble left in place in a 16-bit lane IS the fp16 subnormal w * 2^-24
// (w * 2^-20 for the high nibble of a byte), which the matrix core takes exactly.  Per four
// weights that is one v_perm_b32 (byte gather in AWQ nibble order) and one v_and_b32: the low
// nibble is not masked, the whole byte goes in as (16 w' + w) * 2^-24 and the high-nibble tile's
// sum is taken off again in fp32 when the group ends.  The operands run against the 16xK
// activation slab (A operand, straight from global memory).  The zero point costs one 16-deep
// MFMA per group (A = the lane's sum of activations in four fp16 pieces, B = -z * 2^-e); the
// group scale is applied to the per-group accumulator in fp32 and 2^e once at the end, so no
// per-weight subtract or multiply is spent.  Four waves of a workgroup split the workgroup's K
// range and meet in LDS; workgroups of a split-K launch meet through fp32 partials in the
// workspace, summed in fixed order by whichever workgroup arrives last (arrival counter per
// column block, left at zero).
#pragma once
#include "awq_common.hpp"
#include "awq_moe.hpp"

#ifndef AWQMI_GEMV_WAVES_PER_SIMD
#define AWQMI_GEMV_WAVES_PER_SIMD 1
#endif

namespace awqmi {

struct GemvParams {
  const half_t* x;
  const uint32_t* qw;
  const half_t* sc;
  const uint32_t* qz;
  half_t* y;
  float* part;  // [split][nblk*ncb][16][128*WPL] fp32 partial tiles (tile-major columns)
  int* cnt;     // [nblk*ncb] arrival counters
  int M, K, N, NW, G;
  int ldw;      // words between consecutive rows of qweight (NW, or more when the rows are padded)
  int split_k;
  int ncb;      // column blocks
  // expert-grouped launch
  const int* sorted_ids;
  const int* expert_ids;
  const int* n_post_pad;
  const float* topk_w;
  int n_slots;
  int a_row_div;
  int tile_m;   // rows per sorted-token block: 16 * MB
  int ldy;      // elements between output rows (N, or N / 2 when the activation is fused)
  int nblk;     // sorted-token blocks covered by the launch (a multiple of grp)
  int nblk_cap; // blocks that sorted_ids / expert_ids hold (the align capacity; <= nblk)
  int grp;      // sorted-token blocks per XCD run
  int act_split; // split-K launch over [gate | up] columns: the last arriver of a gate block and
                 // its up block writes silu(gate) * up (one 16-row block, four waves per column block)
  long long w_stride, s_stride, z_stride;  // elements per expert
  // Routing folded into the launch (ROUTE instantiations: at most eight tokens, 64 slots): every
  // workgroup works the routing and the block list out by itself from the router logits, and
  // the first workgroup also leaves them in memory for the launches that follow.
  const float* r_logits;   // [r_T][r_E]
  const float* r_bias;     // score-correction bias or null (sigmoid scoring)
  int r_T, r_E, r_topk, r_renorm;
  float r_scale;
  int* r_ids;              // out [n_slots]
  float* r_wts;            // out [n_slots]
  int* r_sorted;           // out: 16 entries per block that runs
  int* r_experts;          // out: one per block that runs
  int* r_npp;              // out: 16 x blocks that run
  // Dense launches only, null outside the timeline probe: eight time stamps per workgroup
  // (constant-rate 100 MHz counter) at the phase boundaries of the kernel.
  unsigned long long* trace;
};

typedef float f2 __attribute__((ext_vector_type(2)));

// Expert-grouped launches use a 1-D grid and place work by XCD (workgroup i runs on XCD
// i % 8, each XCD has its own L2): grp consecutive sorted-token blocks -- mostly blocks of
// one or two experts -- times one (column block, K part) form a run of consecutive slots on
// ONE XCD, so the blocks that share an expert read its weights through the same L2 at about
// the same time instead of fetching them once per XCD.  grp = 1 is the plain order (column
// block fastest), used when few experts get more than one block.
constexpr int MOE_BLOCK_GROUP_MAX = 32;

// 8-byte device-coherent store / load (relaxed, agent scope)
__device__ __forceinline__ void st_coherent(float* p, f2 v) {
  __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), __builtin_bit_cast(unsigned long long, v),
                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ f2 ld_coherent(const float* p) {
  return __builtin_bit_cast(f2, __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p),
                                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}

template <int WPL>
struct WordVec;
template <>
struct WordVec<1> {
  typedef uint32_t type;
  static __device__ __forceinline__ uint32_t get(uint32_t v, int) { return v; }
};
template <>
struct WordVec<2> {
  typedef u2v type;
  static __device__ __forceinline__ uint32_t get(u2v v, int w) { return w ? v.y : v.x; }
};

// Per-wave main loop.  Ring of RING 32-row steps in flight (RING x 8 rows x WPL words + the
// matching 16-byte activation slices per lane); ring slot = step index mod RING with RING
// dividing 4, so a "chunk" is four steps aligned to 128 rows and group boundaries fall on fixed
// slots.  RING = 4 is the streaming configuration (one wave per SIMD, 16 KB in flight per wave);
// RING = 2 fits two waves per SIMD, for launches made of many short workgroups whose start-up
// and epilogue then overlap another workgroup's loads.
//
// Arithmetic.  A nibble left in place under the mask 0x000F000F (0x00F000F0) *is* the fp16
// subnormal w * 2^-24 (w * 2^-20), and the matrix core takes subnormal fp16 inputs exactly.
// The high nibble w' of a byte is fed under its mask; the low nibble w is not masked at all:
// the whole byte is the subnormal (16 w' + w) * 2^-24, its tile sums 16 x w' + x w, and the high
// nibble's tile (the same 16 x w' * 2^-24, written as x w' * 2^-20) is subtracted when the group
// ends - exact for one-hot rows, 16 units of fp32 rounding instead of one otherwise.  So the B
// operand costs one v_perm_b32 + one v_and_b32 per four weights and no conversion.
// Per quantisation group and 16-column tile the wave keeps accg = 2^-e * sum_k x_k (w_k - z):
// the sum over w comes from the unpacked nibbles, the zero point from one more MFMA whose A
// operand holds this lane's sum of x over the group (split into four fp16 pieces) and whose
// B operand holds -z * 2^-e.  At the end of the group acc += s * accg (fp32, one v_fma_mix per
// element); the factor 2^e is applied once when the wave leaves the loop.
//
// MB row blocks of 16 share every B operand (MB = 2 serves up to 32 rows per pass with the
// unpack work of one).  GMODE: 0 -> G = 32, 1 -> G = 64, 2 -> G = 128, 3 -> G = 128 * i.
//
// LDSQ: the weight ring lives in LDS instead of registers.  With WPL = 2 a 32-row step of a wave
// is 4 KiB (32 rows x 128 bytes); four `buffer_load_dwordx4 ... lds` instructions fetch it
// (lane l of instruction i brings 16 bytes of row 8 i + l / 8), and the step is read back as
// eight 8-byte LDS loads per lane right before its compute.  With WPL = 1 a step is 2 KiB (32 rows
// x 64 bytes), fetched by two instructions (lane l of instruction i brings 16 bytes of row
// 4 i + l / 16 + 8 ((l / 4) % 4), so that row 8 h + r lands in 64-byte piece 4 r + h of the slot and
// the four 16-lane groups of a read hit four different quarters of the banks) and read back as
// eight 4-byte LDS loads per lane.  Ring slot d of all waves is one LDS object of its own, so that
// the compiler's wait before reading a slot counts only the loads issued after that slot's.  This
// buys a ring of four steps at two waves per SIMD.
//
// TAIL (G = 128, register ring of four): after its whole chunks the wave takes one more 32-row
// step of a chunk that the launch's waves share step by step.  When the chunk count leaves
// L chunks over after every wave got the same number (and 4 L <= waves), the busiest wave then
// runs 4 n + 1 steps instead of 4 (n + 1).  The tail step goes into ring slot 0 as soon as the
// last chunk has used it; it is a group of its own (32 rows of x against that chunk's zero
// point and scale).  A wave without a tail step fetches a valid step and multiplies it by zeros.
template <int WPL, int GMODE, int MB, int RING = 4, bool LDSQ = false, bool TAIL = false>
struct GemvWave {
  static_assert(!TAIL || (GMODE == 2 && RING == 4 && !LDSQ), "tail steps: G = 128, register ring of four");
  static constexpr int NT = 8 * WPL;                                   // 16-column tiles per wave
  static constexpr int KSPG = GMODE == 0 ? 1 : (GMODE == 1 ? 2 : 4);  // group boundaries per chunk
  typedef typename WordVec<WPL>::type qvec;

  const uint32_t* qw_u;      // wave-uniform base of the expert's qweight
  const half_t* x_lane[MB];  // this lane's activation row per row block, 8h applied
  uint32_t q_off;            // this lane's byte offset inside a 32-row step: (8h * LDW + wc) * 4
  const half_t* sc;          // lane's scale pointer (8 * wc applied)
  const uint32_t* qz;        // lane's zero-word pointer (wc applied)
  int NW, LDW, N, kspg, ngroups;  // LDW: words between qweight rows; kspg: 32-row steps per quantisation group

  qvec q[LDSQ ? 2 : RING][8];   // LDSQ: the step being computed and the next one, read from the LDS ring
  u4v a[RING][MB];
  // LDSQ only
  unsigned char* slot[RING];      // this wave's 2 KiB x WPL in each ring slot object
  __amdgpu_buffer_rsrc_t rq;      // the (expert's) qweight as a buffer: loads past its end return 0
  // Row r of a step sits in 128-byte line r ^ ((r >> 3) & 1) of the slot: the two 8-row
  // blocks that one half-wave reads together then fall into different halves of the 64 banks.
  uint32_t dma_v[2];              // lane's byte offset inside an 8-row slab, for even / odd slabs
  uint32_t rd_off[2];             // lane's byte offset inside a slot for even / odd rows of its 8
  f4 acc[MB][NT];    // sum over finished groups of s * accg (still carrying 2^-e)
  f4 accg[MB][NT];   // current group
  qvec znext, zcur;
  u4v snext[WPL], scur[WPL];
  float xsum[MB];    // this lane's sum of x over the current group
  NibbleMasks nm;

  __device__ __forceinline__ void issue(int d, int ks) {
    if constexpr (LDSQ) {
#if defined(__HIP_DEVICE_COMPILE__)
      typedef __attribute__((address_space(3))) void lds_void;
      const uint32_t so = (uint32_t)ks * 32u * (uint32_t)LDW * 4u;
      if constexpr (WPL == 2) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rq, (lds_void*)(slot[d] + i * 1024), 16, dma_v[i & 1],
                                                   so + (uint32_t)i * 8u * (uint32_t)LDW * 4u, 0, 0);
      } else {
#pragma unroll
        for (int i = 0; i < 2; ++i)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rq, (lds_void*)(slot[d] + i * 1024), 16, dma_v[0],
                                                   so + (uint32_t)i * 4u * (uint32_t)LDW * 4u, 0, 0);
      }
#endif
    } else {
      const char* rowbase = reinterpret_cast<const char*>(qw_u) + (size_t)ks * 32 * LDW * 4;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        q[d][i] = __builtin_nontemporal_load(
            reinterpret_cast<const qvec*>(rowbase + (size_t)i * LDW * 4 + q_off));
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      a[d][mb] = *reinterpret_cast<const u4v*>(x_lane[mb] + (size_t)ks * 32);
  }

  // LDSQ: ring slot d -> register set d % 2
  __device__ __forceinline__ void fetch(int d) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if constexpr (WPL == 2) q[d & 1][i] = *reinterpret_cast<const qvec*>(slot[d] + rd_off[i & 1] + (i & 6) * 128);
      else q[d & 1][i] = *reinterpret_cast<const qvec*>(slot[d] + rd_off[0] + i * 256);
    }
  }

  __device__ __forceinline__ int clamp_group(int step) const {
    // steps per group are a compile-time power of two except for G = 128 * i
    const int g = GMODE == 3 ? step / kspg : step >> GMODE;
    return g < ngroups ? g : ngroups - 1;
  }

  __device__ __forceinline__ void load_group(int g) {
    znext = *reinterpret_cast<const qvec*>(qz + (size_t)g * NW);
#pragma unroll
    for (int w = 0; w < WPL; ++w) snext[w] = *reinterpret_cast<const u4v*>(sc + (size_t)g * N + 8 * w);
  }

  // take over the prefetched group parameters
  __device__ __forceinline__ void adopt_group() {
#pragma unroll
    for (int w = 0; w < WPL; ++w) scur[w] = snext[w];
    zcur = znext;
  }

  template <int B>
  __device__ __forceinline__ void tile_pair(int d, int w, bool first) {
    u4v lo, hi;
#pragma unroll
    for (int rp = 0; rp < 4; ++rp) {
      const uint32_t t = byte_pair<B>(WordVec<WPL>::get(q[LDSQ ? (d & 1) : d][2 * rp + 1], w),
                                      WordVec<WPL>::get(q[LDSQ ? (d & 1) : d][2 * rp], w));
      lo[rp] = t;           // whole byte: (16 w' + w) * 2^-24 of the high- (w') and low-nibble column
      hi[rp] = t & nm.hi;   // (w'_k, w'_k+1) * 2^-20
    }
    const int t0 = w * 8 + 2 * B;
    const f4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const h8 av = as_h8(a[d][mb]);
      accg[mb][t0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, as_h8(lo), first ? zero : accg[mb][t0], 0, 0, 0);
      accg[mb][t0 + 1] =
          __builtin_amdgcn_mfma_f32_16x16x32_f16(av, as_h8(hi), first ? zero : accg[mb][t0 + 1], 0, 0, 0);
    }
  }

  __device__ __forceinline__ void compute(int d, bool first) {
    // this lane's share of sum_k x_k
    const h2 ones = {(half_t)1.f, (half_t)1.f};
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      float xs = first ? 0.f : xsum[mb];
#pragma unroll
      for (int i = 0; i < 4; ++i) xs = __builtin_amdgcn_fdot2(as_h2(a[d][mb][i]), ones, xs, false);
      xsum[mb] = xs;
    }
#pragma unroll
    for (int w = 0; w < WPL; ++w) {
      tile_pair<0>(d, w, first);
      tile_pair<1>(d, w, first);
      tile_pair<2>(d, w, first);
      tile_pair<3>(d, w, first);
    }
  }

  static __device__ __forceinline__ uint32_t zbyte(uint32_t zw, int b) {
    return b == 0 ? byte_pair<0>(zw, zw) : b == 1 ? byte_pair<1>(zw, zw)
         : b == 2 ? byte_pair<2>(zw, zw) : byte_pair<3>(zw, zw);
  }

  // Zero-point MFMA: accg -= 2^-e * z * (this lane's sum of x since the last call).  The sum goes
  // in as four fp16 pieces, each clamped to the fp16 range before it is taken off the rest: a
  // sum below 65504 in magnitude splits as before (first piece = the rounded sum, the others its
  // residuals, 33+ significant bits), and larger sums (large-mean or outlier activations) stay
  // exact up to 4 x 65504 instead of turning into inf.  A lane adds at most 32 activations
  // between two calls (G = 128 * i calls this once per 128-row chunk for that reason).
  __device__ __forceinline__ void flush_zero() {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      constexpr float HMAX = 65504.f;
      float r = xsum[mb];
      const half_t x0 = (half_t)__builtin_fmaxf(-HMAX, __builtin_fminf(HMAX, r));
      r -= (float)x0;
      const half_t x1 = (half_t)__builtin_fmaxf(-HMAX, __builtin_fminf(HMAX, r));
      r -= (float)x1;
      const half_t x2 = (half_t)__builtin_fmaxf(-HMAX, __builtin_fminf(HMAX, r));
      r -= (float)x2;
      const half_t x3 = (half_t)__builtin_fmaxf(-HMAX, __builtin_fminf(HMAX, r));
      const h2 xp01 = {x0, x1}, xp23 = {x2, x3};
      // (the 16-deep MFMA: its four k-slots per lane hold the four pieces, so neither operand
      // needs zero padding registers)
      const h4 az = __builtin_bit_cast(h4, u2v{as_u32(xp01), as_u32(xp23)});
#pragma unroll
      for (int w = 0; w < WPL; ++w) {
        const uint32_t zw = WordVec<WPL>::get(zcur, w);
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          // B operand word of the zero-point MFMA: -z * 2^-e in all four k-slots
          const uint32_t t = zbyte(zw, b);
          const uint32_t zlo = t | 0x80008000u, zhi = (t & nm.hi) | 0x80008000u;
          const int t0 = w * 8 + 2 * b;
          accg[mb][t0] = __builtin_amdgcn_mfma_f32_16x16x16f16(
              az, __builtin_bit_cast(h4, u2v{zlo, zlo}), accg[mb][t0], 0, 0, 0);
          accg[mb][t0 + 1] = __builtin_amdgcn_mfma_f32_16x16x16f16(
              az, __builtin_bit_cast(h4, u2v{zhi, zhi}), accg[mb][t0 + 1], 0, 0, 0);
        }
      }
      if (GMODE == 3) xsum[mb] = 0.f;
    }
  }

  // end of a group: acc += s * accg
  __device__ __forceinline__ void flush_scale() {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
      for (int w = 0; w < WPL; ++w) {
        const h8 sv = as_h8(scur[w]);
#pragma unroll
        for (int nib = 0; nib < 8; ++nib) {
          const float s = (float)sv[awq_col_of_nibble(nib)];
          const int t = w * 8 + nib;
          // an even tile was fed whole bytes: its sum still holds the odd tile's column 16-fold
          // (both in units of 2^-24, zero points included), which the odd tile's sum takes out
          if (nib & 1) acc[mb][t] += s * accg[mb][t];
          else acc[mb][t] += s * (accg[mb][t] - accg[mb][t + 1]);
        }
      }
    }
  }

  __device__ __forceinline__ void flush() {
    flush_zero();
    flush_scale();
  }

  // one aligned 128-row chunk (four ring slots); REFILL: chunk c + 1 belongs to this wave too.
  // No load sits behind a branch: a branch around a load makes the compiler wait for every
  // outstanding load at the join, which would empty the ring.
  template <bool REFILL>
  __device__ __forceinline__ void chunk(int c, int c_begin, int c_end, int tail_step = 0) {
    bool wide_first = false;
    if (GMODE == 3) {
      const int cpg = kspg >> 2;
      wide_first = (c == c_begin) || (c % cpg == 0);
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      if (d % KSPG == 0) {
        adopt_group();
        if (REFILL || d + KSPG < 4) load_group(clamp_group(4 * c + d + KSPG));
        else if (TAIL && d == 0) load_group(clamp_group(tail_step));
      }
      // LDSQ: the next step's weights leave the ring while this step computes
      if (LDSQ && (REFILL || d < 3)) fetch((d + 1) % RING);
      if (GMODE == 3) {
        if (d == 0 && wide_first) {
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
            for (int t = 0; t < NT; ++t) accg[mb][t] = f4{0.f, 0.f, 0.f, 0.f};
            xsum[mb] = 0.f;
          }
        }
        compute(d % RING, false);
      } else {
        compute(d % RING, d % KSPG == 0);
      }
      // pin the refill right behind its slot's compute: sunk to the end of the chunk the
      // four-deep ring degenerates into load-all / wait-all / compute-all
      __builtin_amdgcn_sched_barrier(0);
      if (REFILL || d + RING < 4) issue(d % RING, 4 * c + d + RING);
      else if (TAIL && d == 0) issue(0, tail_step);
      __builtin_amdgcn_sched_barrier(0);
      if (GMODE != 3 && (d + 1) % KSPG == 0) flush();
    }
    if (GMODE == 3) {
      const int cpg = kspg >> 2;
      flush_zero();
      if (c + 1 == c_end || (c + 1) % cpg == 0) flush_scale();
    }
  }

  // tail_step (TAIL only): the extra 32-row step, or -1 when this wave has none
  __device__ __forceinline__ void run(int c_begin, int c_end, int tail_step = -1) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[mb][t] = f4{0.f, 0.f, 0.f, 0.f};
      xsum[mb] = 0.f;
    }
    if (c_begin >= c_end) return;
    nm.init();
    load_group(clamp_group(4 * c_begin));
#pragma unroll
    for (int d = 0; d < RING; ++d) issue(d, 4 * c_begin + d);
    if (LDSQ) fetch(0);
    int c = c_begin;
    for (; c + 1 < c_end; ++c) chunk<true>(c, c_begin, c_end);
    if constexpr (TAIL) {
      const bool has_tail = tail_step >= 0;
      chunk<false>(c, c_begin, c_end, has_tail ? tail_step : 4 * c);
      adopt_group();
      if (!has_tail) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) a[0][mb] = u4v{0u, 0u, 0u, 0u};
      }
      compute(0, true);
      flush();
    } else {
      chunk<false>(c, c_begin, c_end);
    }
    // undo the 2^-24 / 2^-20 carried by the low- / high-nibble tiles
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[mb][t] *= (t & 1) ? 1048576.f : 16777216.f;
  }
};

// KW = waves of a workgroup that share one column block and split its K range (4, or 2: the
// workgroup then covers two neighbouring column blocks with two waves each, which keeps the
// waves' ranges long and even when K is only a few chunks; launches with KW = 2 do not split K
// across workgroups).
// ACT (with KW = 2): the weight columns are [gate | up]; the workgroup takes a gate column
// block and the up column block N / 2 columns further, and writes silu(gate) * up (both rounded
// to fp16 first, as the unfused path stores them) to a [.., N / 2] output.
// LDSQ: weight ring of RING = 4 steps in LDS (see GemvWave), two workgroups per CU.
// TAIL (dense launches, see GemvWave): every wave gets the same number of whole chunks and the
// chunks left over are taken one 32-row step per wave.
// RPER > 0 (MoE launches of a few tokens, at most 64 slots, 16-row blocks): the launch does its
// own routing.  The four waves of EVERY workgroup run the top-k of the tokens in turn (RPER experts
// per lane, RSIG = sigmoid scoring) into LDS; every wave then sorts the slots by expert in
// registers (lane = slot: equal-expert mask from one ballot per id bit, block index = number of
// distinct smaller experts) and so knows its block's expert and rows without a trip to memory.
// A token picks distinct experts, so an expert holds at most T <= 8 slots and every block is one
// expert's single block.  Workgroup 0 writes ids, weights, block list and padded count out for
// the launches that follow (same layout as the align kernel's, entries past the last block that
// runs left unwritten: nothing reads them).
template <int WPL, int GMODE, int MB, bool MOE, int RING, int KW, bool ACT, bool LDSQ, bool TAIL, int RPER = 0,
          bool RSIG = false>
__device__ __forceinline__ void awq_gemv_body(const GemvParams& p) {
  static_assert(RPER == 0 || (MOE && MB == 1 && !TAIL), "folded routing: expert-grouped launches of 16-row blocks");
  static_assert(!ACT || (KW == 2 && MB == 1), "fused activation pairs two column blocks");
  static_assert(!LDSQ || RING == 4, "the LDS ring holds four steps");
  static_assert(!LDSQ || WPL == 2 || (MB == 2 && KW == 2), "one word per lane in LDS: the 32-row form");
  static_assert(!TAIL || (!MOE && KW == 4 && !ACT), "tail steps are for dense launches");
  constexpr int CW = 4 / KW;       // column blocks per workgroup
  constexpr int NT = 8 * WPL;
  constexpr int CB = 128 * WPL;
  // LDS row stride of the cross-wave sum in floats: padded so that 4h rows land 16 banks apart,
  // unpadded where the two buffers take the place of ring slots 0 and 1 (16 KiB each)
  constexpr int RS = LDSQ ? NT * 16 : NT * 16 + 4;
  constexpr int TM = 16 * MB;      // rows per pass
  constexpr int SLOT = LDSQ ? 8192 * WPL : 16;   // bytes of one ring slot object: four waves x 2 KiB x WPL
  __shared__ __align__(16) unsigned char lq0[SLOT], lq1[SLOT], lq2[SLOT], lq3[SLOT];
  __shared__ __align__(16) float red_own[LDSQ ? 1 : 2][LDSQ ? 1 : 16][RS];
  auto red = [&](int b) -> float (*)[RS] {
    if constexpr (LDSQ) return reinterpret_cast<float (*)[RS]>(b ? lq1 : lq0);
    else return red_own[b];
  };
  __shared__ int s_last;
  __shared__ int s_sid[32];     // MoE: slot id of every row of this block (pads: n_slots)
  __shared__ float s_tw[32];    // MoE: routing weight of the row (1 when not applied)
  __shared__ int s_rows;

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, j = lane & 15, h = lane >> 4;
  int cb = blockIdx.x, sp = blockIdx.y;
  // phase stamps of the timeline probe: 0 start, 1 main loop left, 2 cross-wave sum done,
  // 3 partial stores acknowledged, 4 arrival counted, 5 (last arriver) partials summed, 6 output stored
  auto stamp = [&](int k) {
    if constexpr (!MOE) {
      if (p.trace && tid == 0)
        p.trace[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 8 + k] = __builtin_amdgcn_s_memrealtime();
    }
  };
  stamp(0);
  int blk = 0;
  float row_tw = 1.f;   // MoE: routing weight of row tid (threads below TM), parked in s_tw after the loop
  const uint32_t* qw = p.qw;
  const half_t* sc = p.sc;
  const uint32_t* qz = p.qz;
  if (MOE) {
    const int B = p.grp;
    const int lin = blockIdx.x, xcd = lin & 7, slot = lin >> 3;
    const int g = (slot / B) * 8 + xcd;            // run index: (block group, column block, part)
    const int ncbs = (ACT ? p.ncb / 2 : (p.ncb + CW - 1) / CW) * p.split_k;
    const int bg = g / ncbs, cbs = g % ncbs;
    blk = bg * B + slot % B;
    cb = cbs / p.split_k;          // column group of the workgroup (a column block when CW = 1)
    sp = cbs % p.split_k;
    int e, sid = p.n_slots;
    if constexpr (RPER > 0) {
      __shared__ int r_ids_s[64];
      __shared__ float r_wts_s[64];
      __shared__ int r_stage[64 * 16];
      __shared__ int r_exp_s[64];
      const int n = p.n_slots;
      for (int t = wave; t < p.r_T; t += 4)
        moe_topk_token<RPER, RSIG>(p.r_logits, p.r_bias, t, p.r_E, p.r_topk, p.r_renorm, p.r_scale, r_ids_s,
                                   r_wts_s);
      __syncthreads();
      const bool valid = lane < n;
      const int e_i = valid ? r_ids_s[lane] : 0x7fffffff;
      unsigned long long same = __ballot(valid);
      const int nbits = 32 - __builtin_clz(max(p.r_E - 1, 1));
      for (int b = 0; b < nbits; ++b) {
        const bool bit = (e_i >> b) & 1;
        const unsigned long long bal = __ballot(bit);
        same &= bit ? bal : ~bal;
      }
      const int r_i = __popcll(same & ((1ull << lane) - 1ull));     // row inside the expert's block
      const unsigned long long firsts = __ballot(valid && r_i == 0);
      int b_i = 0;                                                  // block = distinct smaller experts
      for (int jj = 0; jj < n; ++jj) {
        const int ej = __builtin_amdgcn_readlane(e_i, jj);
        if (((firsts >> jj) & 1ull) && ej < e_i) ++b_i;
      }
      const int nb = __popcll(firsts);
      if (blockIdx.x == 0) {
        // the lists for the launches that follow, staged in LDS so that pads and slots do not race
        for (int i = tid; i < nb * 16; i += 256) r_stage[i] = n;
        __syncthreads();
        if (wave == 0 && valid) {
          r_stage[b_i * 16 + r_i] = lane;
          if (r_i == 0) r_exp_s[b_i] = e_i;
        }
        __syncthreads();
        for (int i = tid; i < nb * 16; i += 256) p.r_sorted[i] = r_stage[i];
        if (tid < nb) p.r_experts[tid] = r_exp_s[tid];
        if (tid < n) {
          p.r_ids[tid] = r_ids_s[tid];
          p.r_wts[tid] = r_wts_s[tid];
        }
        if (tid == 0) p.r_npp[0] = nb * 16;
      }
      if (blk >= nb) return;
      const unsigned long long mine = __ballot(valid && b_i == blk);
      e = __builtin_amdgcn_readlane(e_i, __builtin_ctzll(mine));
      // thread r takes the slot of row r: the r-th set lane of `mine` (at most eight rows)
      unsigned long long m = mine;
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if (m) {
          if (tid == k) sid = __builtin_ctzll(m);
          m &= m - 1ull;
        }
      }
    } else {
    // The block's padded count, expert and slot ids are read side by side (one trip to memory
    // instead of three in a row; blocks past the lists' end read the last block's entries and
    // leave right after), the routing weights behind them while the main loop runs.
    const int blk_c = min(blk, p.nblk_cap - 1);
    const int npp = *p.n_post_pad;
    e = p.expert_ids[blk_c];
    if (tid < TM) sid = p.sorted_ids[blk_c * TM + tid];
    if (blk >= p.nblk_cap || blk * TM >= npp) return;
    }
    qw += (size_t)e * p.w_stride;
    sc += (size_t)e * p.s_stride;
    qz += (size_t)e * p.z_stride;
    // one global read per row of the block; everything later takes ids / weights from LDS
    if (tid < 64) {
      const bool ok = sid < p.n_slots;
      if (tid < TM) {
        s_sid[tid] = sid;
        if (ok && p.topk_w) row_tw = p.topk_w[sid];
      }
      const unsigned long long m = __ballot(ok);
      if (tid == 0) s_rows = __popcll(m);   // valid slots sit at the front of a block
    }
    __syncthreads();
  }

  // Lanes past the last word column / past the last row read valid memory of column block 0
  // / row 0 instead; their B column (resp. A row) only feeds outputs that are never stored.
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int cbw = ACT ? cb + (wave_u / KW) * (p.ncb / 2) : cb * CW + wave_u / KW;   // this wave's column block
  int wc = cbw * (16 * WPL) + WPL * j;
  if (wc >= p.NW) wc = 0;

  GemvWave<WPL, GMODE, MB, RING, LDSQ, TAIL> w;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int r = mb * 16 + j;
    size_t arow;
    if (!MOE) {
      arow = r < p.M ? (size_t)r : 0;
    } else {
      const int sid = s_sid[r];
      arow = sid < p.n_slots ? (size_t)(sid / p.a_row_div) : 0;
    }
    w.x_lane[mb] = p.x + arow * p.K + 8 * h;
  }
  w.qw_u = qw;
  if constexpr (LDSQ) {
    unsigned char* const slots[4] = {lq0, lq1, lq2, lq3};
#pragma unroll
    for (int d = 0; d < RING; ++d) w.slot[d] = slots[d] + wave_u * (2048 * WPL);
    w.rq = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(qw), 0, (int)((size_t)p.K * p.ldw * 4), 0x00020000);
    if constexpr (WPL == 2) {
      const int wc4 = cbw * (16 * WPL) + 4 * (lane & 7);       // first of the four words this lane fetches
      // line 8 i + l / 8 of the slot (instruction i, lane l) holds row 8 i + ((l / 8) ^ (i & 1))
      w.dma_v[0] = (uint32_t)(((size_t)(lane >> 3) * p.ldw + (wc4 < p.NW ? wc4 : 0)) * 4);
      w.dma_v[1] = (uint32_t)(((size_t)((lane >> 3) ^ 1) * p.ldw + (wc4 < p.NW ? wc4 : 0)) * 4);
      // row 8 h + i is read from line 8 h + (i ^ (h & 1))
      w.rd_off[0] = (uint32_t)((8 * h + (h & 1)) * 128 + 8 * j);
      w.rd_off[1] = (uint32_t)((8 * h + (1 ^ (h & 1))) * 128 + 8 * j);
    } else {
      const int wc4 = cbw * 16 + 4 * (lane & 3);
      // 64-byte piece 16 i + l / 4 of the slot (instruction i, lane l) holds row 4 i + l / 16 + 8 ((l / 4) % 4)
      w.dma_v[0] = (uint32_t)(((size_t)((lane >> 4) + 8 * ((lane >> 2) & 3)) * p.ldw + (wc4 < p.NW ? wc4 : 0)) * 4);
      w.dma_v[1] = 0;
      // row 8 h + i is read from piece 4 i + h
      w.rd_off[0] = (uint32_t)(h * 64 + 4 * j);
      w.rd_off[1] = 0;
    }
  }
  w.q_off = (uint32_t)(((size_t)8 * h * p.ldw + wc) * 4);
  w.sc = sc + 8 * (size_t)wc;
  w.qz = qz + wc;
  w.NW = p.NW;
  w.LDW = p.ldw;
  w.N = p.N;
  w.kspg = p.G / 32;
  w.ngroups = GMODE == 3 ? p.K / p.G : p.K >> (5 + GMODE);

  // this wave's share of K, in 128-row chunks; the wave index is made scalar so that the
  // row base addresses stay in SGPRs
  // (32-bit: at most 64 parts, K below 2^31)
  const unsigned parts = (unsigned)KW * (unsigned)p.split_k;
  const unsigned pw = (unsigned)sp * KW + (unsigned)wave_u % KW;
  const int nchunks = p.K >> 7;
  if constexpr (TAIL) {
    // the host launches this form only with at least one whole chunk per wave and at most one
    // left-over step per wave
    const int base = nchunks / (int)parts;
    const int left_steps = 4 * (nchunks - base * (int)parts);
    w.run((int)pw * base, (int)pw * base + base, (int)pw < left_steps ? 4 * base * (int)parts + (int)pw : -1);
  } else {
    const int c_begin = (int)(pw * (unsigned)nchunks / parts);
    const int c_end = (int)((pw + 1) * (unsigned)nchunks / parts);
    w.run(c_begin, c_end);
  }
  stamp(1);
  if (LDSQ) __syncthreads();   // the cross-wave sum below reuses ring slots 0 and 1
  if (MOE && tid < TM) s_tw[tid] = row_tw;   // read behind the barriers of the cross-wave sum

  const int rows_total = MOE ? s_rows : p.M;
  const size_t tile = (size_t)blk * p.ncb + cb;
  const size_t ntiles = (size_t)(MOE ? p.nblk : 1) * p.ncb;
  constexpr int TILE_F = 16 * NT * 16;   // floats per partial tile (one row block)
  const bool split = p.split_k > 1;

  // tile-major LDS (red[0], optionally + red[1]) -> row-major fp16 output of row block mb;
  // one thread gathers the eight columns of a packed word and stores them as 16 bytes
  auto emit = [&](int mb, int rows, bool two, int buf = 0, int cbo = -1) {
    constexpr int WPB = 16 * WPL;   // packed words per row of the block
    if (cbo < 0) cbo = cb;
    for (int it = tid; it < rows * WPB; it += 256) {
      const int m = it / WPB, wl = it % WPB;
      const int jj = wl / WPL, ww = wl % WPL;
      const int col = cbo * CB + wl * 8;
      if (col >= p.N) continue;
      float v[8];
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const int t = ww * 8 + awq_nibble_of_col(c);
        v[c] = red(buf)[m][t * 16 + jj];
        if (two) v[c] += red(1)[m][t * 16 + jj];
      }
      size_t orow = (size_t)(mb * 16 + m);
      if (MOE) {
        const int sid = s_sid[mb * 16 + m];
        if (sid >= p.n_slots) continue;
        const float tw = s_tw[mb * 16 + m];
#pragma unroll
        for (int c = 0; c < 8; ++c) v[c] *= tw;
        orow = (size_t)sid;
      }
      h8 o;
#pragma unroll
      for (int c = 0; c < 8; ++c) o[c] = (half_t)v[c];
      *reinterpret_cast<h8*>(p.y + orow * p.ldy + col) = o;
    }
  };
  // gate tile in red[0], up tile in red[1] -> silu(gate) * up, 16 bytes per thread
  auto emit_act = [&](int rows, int cbo) {
    constexpr int WPB = 16 * WPL;
    for (int it = tid; it < rows * WPB; it += 256) {
      const int m = it / WPB, wl = it % WPB;
      const int jj = wl / WPL, ww = wl % WPL;
      const int col = cbo * CB + wl * 8;
      const int sid = s_sid[m];
      if (sid >= p.n_slots) continue;
      h8 o;
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const int t = ww * 8 + awq_nibble_of_col(c);
        const float gv = (float)(half_t)red(0)[m][t * 16 + jj];
        const float uv = (float)(half_t)red(1)[m][t * 16 + jj];
        o[c] = (half_t)(gv / (1.f + __expf(-gv)) * uv);
      }
      *reinterpret_cast<h8*>(p.y + (size_t)sid * p.ldy + col) = o;
    }
  };

#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int rows = min(16, max(0, rows_total - 16 * mb));
    if (KW == 2) {
      // two column blocks, two waves each: the odd wave of a pair writes, the even one adds,
      // and each buffer is written out on its own
      if (wave & 1) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (4 * h + r < rows) {
#pragma unroll
            for (int t = 0; t < NT; ++t) red(wave >> 1)[4 * h + r][t * 16 + j] = w.acc[mb][t][r];
          }
      }
      __syncthreads();
      if (!(wave & 1)) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (4 * h + r < rows) {
#pragma unroll
            for (int t = 0; t < NT; ++t) red(wave >> 1)[4 * h + r][t * 16 + j] += w.acc[mb][t][r];
          }
      }
      __syncthreads();
      if (ACT) {
        emit_act(rows, cb);
      } else {
        emit(mb, rows, false, 0, cb * 2);
        if (cb * 2 + 1 < p.ncb) emit(mb, rows, false, 1, cb * 2 + 1);
      }
      __syncthreads();
      continue;
    }
    // ---- cross-wave sum in LDS: red(b)[row][tile*16 + j] ----
    // (rows past the block's last one are never read back)
    if (wave >= 2) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (4 * h + r < rows) {
#pragma unroll
          for (int t = 0; t < NT; ++t) red(wave - 2)[4 * h + r][t * 16 + j] = w.acc[mb][t][r];
        }
    }
    __syncthreads();
    if (wave < 2) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (4 * h + r < rows) {
#pragma unroll
          for (int t = 0; t < NT; ++t) red(wave)[4 * h + r][t * 16 + j] += w.acc[mb][t][r];
        }
    }
    __syncthreads();
    if (mb == 0) stamp(2);
    if (split) {
      // fp32 partial tile of this workgroup.  Partials and the arrival counter go through
      // device-coherent accesses (they bypass the per-XCD L2 for other XCDs' data) instead of
      // release / acquire fences: a fence here writes back and invalidates the whole L2 once
      // per workgroup, which costs far more than the few KB of partials.
      float* mine = p.part + (((size_t)sp * ntiles + tile) * MB + mb) * TILE_F;
      const int nelem = rows * (NT * 16);
      // neighbouring lanes write neighbouring 8-byte pairs: whole 32-byte sectors per store
      for (int i = tid * 2; i < nelem; i += 512) {
        const int m = i / (NT * 16), c = i % (NT * 16);
        const f2 v = *reinterpret_cast<const f2*>(&red(0)[m][c]) + *reinterpret_cast<const f2*>(&red(1)[m][c]);
        st_coherent(mine + i, v);
      }
    } else {
      emit(mb, rows, true);
    }
    __syncthreads();
  }
  if (!split) {
    stamp(6);
    return;
  }

  // Ordering: every store of this workgroup has completed (vmcnt 0, then the barrier)
  // before its arrival is counted; whoever arrives last sums all partials in fixed order.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  stamp(3);
  // fused activation: a gate block and its up block (half the column blocks further on) share
  // one counter, and the last of their 2 x split workgroups finishes both tiles
  const bool acts = MOE && MB == 1 && KW == 4 && !ACT && p.act_split;
  const int hcb = p.ncb / 2;
  const int cbg = acts ? cb % hcb : cb;
  const size_t ctile = acts ? (size_t)blk * hcb + cbg : tile;
  const int arrivals = acts ? 2 * p.split_k : p.split_k;
  if (tid == 0) s_last = (atomicAdd(p.cnt + ctile, 1) == arrivals - 1);
  __syncthreads();
  stamp(4);
  if (!s_last) return;
  const size_t sstride = ntiles * MB * TILE_F;
  // U pairs per thread x 8 parts per batch: 8 * U independent 8-byte loads in flight; parts
  // are added in index order whatever the arrival order was.  Out-of-range slots read a valid
  // address and are dropped by a select, so no load sits behind a branch.
  auto finish = [&](auto u_tag, const float* base, int nelem, int buf = 0) {
    constexpr int U = decltype(u_tag)::value;
    constexpr int SU = 8;
    f2 v[U];
    int idx[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      v[u] = f2{0.f, 0.f};
      idx[u] = tid * 2 + 512 * u;
    }
    for (int s0 = 0; s0 < p.split_k; s0 += SU) {
      f2 t[SU][U];
#pragma unroll
      for (int su = 0; su < SU; ++su) {
        const int sidx = min(s0 + su, p.split_k - 1);
#pragma unroll
        for (int u = 0; u < U; ++u)
          t[su][u] = ld_coherent(base + (size_t)sidx * sstride + min(idx[u], nelem - 2));
      }
#pragma unroll
      for (int su = 0; su < SU; ++su) {
        const bool ok = s0 + su < p.split_k;
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] += ok ? t[su][u] : f2{0.f, 0.f};
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (idx[u] < nelem) *reinterpret_cast<f2*>(&red(buf)[idx[u] / (NT * 16)][idx[u] % (NT * 16)]) = v[u];
  };
  if (acts) {
    const int rows = min(16, rows_total);
    const int nelem = rows * (NT * 16);
    if (nelem > 0) {
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const float* base = p.part + ((size_t)blk * p.ncb + cbg + half * hcb) * TILE_F;
        if (nelem <= 512) finish(std::integral_constant<int, 1>{}, base, nelem, half);
        else if (nelem <= 1024) finish(std::integral_constant<int, 2>{}, base, nelem, half);
        else if (nelem <= 2048) finish(std::integral_constant<int, 4>{}, base, nelem, half);
        else finish(std::integral_constant<int, 8>{}, base, nelem, half);
      }
    }
    __syncthreads();
    emit_act(rows, cbg);
    if (tid == 0) __hip_atomic_store(p.cnt + ctile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return;
  }
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int rows = min(16, max(0, rows_total - 16 * mb));
    const int nelem = rows * (NT * 16);
    const float* base = p.part + (tile * MB + mb) * TILE_F;
    if (nelem > 0) {
      if (nelem <= 512) finish(std::integral_constant<int, 1>{}, base, nelem);
      else if (nelem <= 1024) finish(std::integral_constant<int, 2>{}, base, nelem);
      else if (nelem <= 2048) finish(std::integral_constant<int, 4>{}, base, nelem);
      else finish(std::integral_constant<int, 8>{}, base, nelem);
    }
    __syncthreads();
    if (mb == 0) stamp(5);
    emit(mb, rows, false);
    __syncthreads();
  }
  stamp(6);
  if (tid == 0) __hip_atomic_store(p.cnt + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int WPL, int GMODE, int MB, bool MOE, int RING = 4, int KW = 4, bool ACT = false, bool LDSQ = false>
__global__ __launch_bounds__(256, ((RING == 4 && !LDSQ) || (MB == 2 && WPL == 2)) ? 1 : 2) void awq_gemv_kernel(const GemvParams p) {
  awq_gemv_body<WPL, GMODE, MB, MOE, RING, KW, ACT, LDSQ, false>(p);
}

// the expert-grouped launch of 16-row blocks (two words per lane, register ring of two) with the
// routing folded in: RPER experts per lane, RSIG = sigmoid scoring
template <int GMODE, int RPER, bool RSIG>
__global__ __launch_bounds__(256, 2) void awq_gemv_route_kernel(const GemvParams p) {
  awq_gemv_body<2, GMODE, 1, true, 2, 4, false, false, false, RPER, RSIG>(p);
}

// the dense G = 128 launch in its TAIL form (left-over chunks step by step)
template <int WPL, int MB>
__global__ __launch_bounds__(256, 1) void awq_gemv_tail_kernel(const GemvParams p) {
  awq_gemv_body<WPL, 2, MB, false, 4, 4, false, false, true>(p);
}

}  // namespace awqmi
