// Routing-side kernels of the expert-grouped AWQ path: softmax + top-k, the stable
// sort/pad of routed slots by expert, the SiLU(gate) * up activation between the two expert
// GEMMs, and the final sum over a token's slots.  All are latency-sized integer / elementwise
// work; the expert GEMMs themselves are the MOE instantiation of the skinny kernel.
#pragma once
#include <type_traits>
#include "awq_common.hpp"

namespace awqmi {

// Wave-wide max / sum by DPP row shifts and row broadcasts (full-rate VALU, no LDS crossbar
// trips); the result is taken from lane 63 and returned wave-uniform.
template <bool IS_MAX>
__device__ __forceinline__ float wave_reduce_f32(float v) {
  const int ident = IS_MAX ? (int)0xff800000u : 0;   // -inf / 0.0f
  auto step = [&](auto CTRL, auto ROWS) {
    const int o = __builtin_amdgcn_update_dpp(ident, __builtin_bit_cast(int, v), decltype(CTRL)::value,
                                              decltype(ROWS)::value, 0xf, false);
    const float f = __builtin_bit_cast(float, o);
    v = IS_MAX ? fmaxf(v, f) : v + f;
  };
  using std::integral_constant;
  step(integral_constant<int, 0x111>{}, integral_constant<int, 0xf>{});   // row_shr:1
  step(integral_constant<int, 0x112>{}, integral_constant<int, 0xf>{});   // row_shr:2
  step(integral_constant<int, 0x114>{}, integral_constant<int, 0xf>{});   // row_shr:4
  step(integral_constant<int, 0x118>{}, integral_constant<int, 0xf>{});   // row_shr:8: lane 15 of a row = row total
  step(integral_constant<int, 0x142>{}, integral_constant<int, 0xa>{});   // row_bcast:15 into rows 1, 3
  step(integral_constant<int, 0x143>{}, integral_constant<int, 0xc>{});   // row_bcast:31 into rows 2, 3
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// One wave per token.  PER = experts per lane (E <= 64 * PER).
// SIGMOID = false: softmax scores; selection runs on the raw logits (softmax is monotonic).
// SIGMOID = true: score = sigmoid(logit); selection runs on score + bias[e] (bias may be
// null), the weight is the score itself.  Ties go to the lowest expert id.  Weights are
// optionally renormalised over the selected experts and multiplied by `scale`.
// Each pick is one wave-wide max of the remaining keys, then a ballot of the lanes that hold
// it (lowest expert id first); the winner's id and key are wave-uniform from there on.
template <int PER, bool SIGMOID>
__device__ __forceinline__ void moe_topk_token(const float* __restrict__ logits,
                                               const float* __restrict__ bias, int t, int E, int topk,
                                               int renorm, float scale, int* __restrict__ ids,
                                               float* __restrict__ wts) {
  const int lane = threadIdx.x & 63;
  float v[PER];      // selection key
  float sc[PER];     // score (SIGMOID only)
  bool open[PER];    // expert exists and is not picked yet
  float lmax = -INFINITY;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = lane + 64 * i;
    open[i] = e < E;
    const float x = e < E ? logits[(size_t)t * E + e] : -INFINITY;
    if (SIGMOID) {
      sc[i] = 1.f / (1.f + __expf(-x));
      v[i] = e < E ? sc[i] + (bias ? bias[e] : 0.f) : -INFINITY;
    } else {
      sc[i] = 0.f;
      v[i] = x;
      lmax = fmaxf(lmax, x);
    }
  }
  float mx = 0.f, sum = 1.f;
  if (!SIGMOID) {
    mx = wave_reduce_f32<true>(lmax);
    float ls = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (lane + 64 * i < E) ls += __expf(v[i] - mx);
    sum = wave_reduce_f32<false>(ls);
  }

  float sel_sum = 0.f;
  float my_w = 0.f;   // lane j keeps the weight of pick j (topk <= 64)
  int my_id = 0;
  for (int it = 0; it < topk; ++it) {
    float loc = -INFINITY;
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (open[i]) loc = fmaxf(loc, v[i]);
    const float best = wave_reduce_f32<true>(loc);
    int bidx = E;                                    // stays E only if every key left is NaN
#pragma unroll
    for (int i = PER - 1; i >= 0; --i) {             // descending, so the lowest id wins
      const unsigned long long b = __ballot(open[i] && v[i] == best);
      if (b) bidx = 64 * i + __builtin_ctzll(b);
    }
    if (bidx == E) {
      // only NaN keys are left (fmaxf skipped them, nothing equals `best`): take the lowest
      // expert that is still open, so that every id stays inside [0, E) and every slot gets its
      // rows written; the weight computed below is NaN and carries the bad logit forward
#pragma unroll
      for (int i = PER - 1; i >= 0; --i) {
        const unsigned long long b = __ballot(open[i]);
        if (b) bidx = 64 * i + __builtin_ctzll(b);
      }
    }
    float bsc = 0.f;
    if (SIGMOID) {
#pragma unroll
      for (int i = 0; i < PER; ++i)
        if ((bidx >> 6) == i)
          bsc = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sc[i]), bidx & 63));
    }
    float bkey = best;                               // the winner's own key (NaN when only NaN keys are left)
    if (!SIGMOID) {
#pragma unroll
      for (int i = 0; i < PER; ++i)
        if ((bidx >> 6) == i)
          bkey = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v[i]), bidx & 63));
    }
    const float pw = SIGMOID ? bsc : __expf(bkey - mx) / sum;
    sel_sum += pw;
    if (lane == it) { my_w = pw; my_id = bidx; }
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (lane + 64 * i == bidx) open[i] = false;
  }
  if (lane < topk) {
    ids[(size_t)t * topk + lane] = my_id;
    wts[(size_t)t * topk + lane] = (renorm ? my_w / sel_sum : my_w) * scale;
  }
}

template <int PER, bool SIGMOID>
__global__ __launch_bounds__(256) void moe_topk_kernel(const float* __restrict__ logits,
                                                       const float* __restrict__ bias, int T, int E,
                                                       int topk, int renorm, float scale,
                                                       int* __restrict__ ids, float* __restrict__ wts) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  moe_topk_token<PER, SIGMOID>(logits, bias, t, E, topk, renorm, scale, ids, wts);
}

// Single workgroup of 16 waves.  Dynamic LDS: cnt[16][E] + padded[E] + start[E].
// Wave w owns the contiguous slice [w*seg, (w+1)*seg) of the flat slot list, so placing
// slices in wave order and slots in index order inside a slice gives a stable sort.  Inside a
// batch of 64 slots a lane's rank among equal expert ids is the number of lower lanes with
// the same id (a lane mask built from one ballot per id bit, no LDS round trips); the running
// position per (wave, expert) lives in LDS and is bumped by one LDS atomic per slot after all
// lanes of the batch have read it.
constexpr int MOE_ALIGN_WAVES = 16;
// MODE 0: the whole job in one workgroup.  For long slot lists the job is split over the
// workgroups of three launches (one workgroup scatters about one slot per clock, whatever it
// does): MODE 1 = count the experts of this workgroup's part [s0, s1) into block_cnt[block][E];
// (moe_align_scan_kernel turns the counts into each part's first position per expert and writes
// the padding;) MODE 2 = place this part's slots from block_start[block][E].
template <int MODE>
__device__ __forceinline__ void moe_align_block(const int* __restrict__ ids, int n, int E, int tile_m,
                                                int cap, int* __restrict__ sorted,
                                                int* __restrict__ expert_ids, int* __restrict__ npp,
                                                int* sm, int s0 = 0, int s1 = 0,
                                                int* __restrict__ block_tab = nullptr) {
  constexpr int NWV = MOE_ALIGN_WAVES;
  int* cnt = sm;               // [NWV][E], later the running write position
  int* padded = sm + NWV * E;  // [E]
  int* start = padded + E;     // [E]
  __shared__ int s_total;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  if (MODE == 0) { s0 = 0; s1 = n; }

  for (int i = tid; i < NWV * E; i += 1024) cnt[i] = 0;
  __syncthreads();

  const int seg = ((s1 - s0 + NWV * 64 - 1) / (NWV * 64)) * 64;
  const int sb = s0 + wave * seg, se = min(s1, sb + seg);
  // ids are read eight batches of 64 at a time (eight loads in flight instead of one
  // dependent load per batch); the first eight batches stay in registers for the second pass
  constexpr int NB = 8;
  int first[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    const int i = sb + 64 * b + lane;
    first[b] = i < se ? ids[i] : -1;
  }
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    const int e = first[b];
    if (e >= 0 && e < E) atomicAdd(&cnt[wave * E + e], 1);
  }
  for (int c0 = sb + 64 * NB; c0 < se; c0 += 64 * NB) {
    int more[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int i = c0 + 64 * b + lane;
      more[b] = i < se ? ids[i] : -1;
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int e = more[b];
      if (e >= 0 && e < E) atomicAdd(&cnt[wave * E + e], 1);
    }
  }
  __syncthreads();

  if (MODE == 1) {
    for (int e = tid; e < E; e += 1024) {
      int tot = 0;
      for (int w = 0; w < NWV; ++w) tot += cnt[w * E + e];
      block_tab[(size_t)blockIdx.x * E + e] = tot;
    }
    return;
  }
  if (MODE == 2) {
    for (int e = tid; e < E; e += 1024) {
      int pos = block_tab[(size_t)blockIdx.x * E + e];
      for (int w = 0; w < NWV; ++w) { const int c = cnt[w * E + e]; cnt[w * E + e] = pos; pos += c; }
    }
    __syncthreads();
  }
  if constexpr (MODE == 0) {
  for (int e = tid; e < E; e += 1024) {
    int tot = 0;
    for (int w = 0; w < NWV; ++w) tot += cnt[w * E + e];
    padded[e] = (tot + tile_m - 1) / tile_m * tile_m;
  }
  __syncthreads();
  if (wave == 0) {   // exclusive prefix sum of padded[] by one wave: lane owns a contiguous run
    const int per = (E + 63) / 64;
    int local = 0;
    for (int k = 0; k < per; ++k) {
      const int e = lane * per + k;
      if (e < E) local += padded[e];
    }
    int incl = local;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int v = __shfl_up(incl, o);
      if (lane >= o) incl += v;
    }
    int pos = incl - local;
    for (int k = 0; k < per; ++k) {
      const int e = lane * per + k;
      if (e < E) { start[e] = pos; pos += padded[e]; }
    }
    if (lane == 63) { s_total = incl; npp[0] = incl; }
  }
  __syncthreads();
  const int total = s_total;
  for (int e = tid; e < E; e += 1024) {
    int pos = start[e];
    const int e0 = pos;
    for (int w = 0; w < NWV; ++w) { const int c = cnt[w * E + e]; cnt[w * E + e] = pos; pos += c; }
    for (int i = pos; i < e0 + padded[e]; ++i) sorted[i] = n;            // pad entries
    for (int b = 0; b < padded[e] / tile_m; ++b) expert_ids[e0 / tile_m + b] = e;
  }
  for (int i = total + tid; i < cap; i += 1024) sorted[i] = n;           // unused tail
  for (int i = total / tile_m + tid; i < cap / tile_m; i += 1024) expert_ids[i] = -1;
  __syncthreads();
  }   // MODE == 0

  const int nbits = 32 - __builtin_clz(max(E - 1, 1));
  auto place = [&](int i, int e) {
    const bool valid = e >= 0 && e < E;
    // lanes of the batch that hold the same expert id: one ballot per id bit
    unsigned long long same = __ballot(valid);
    for (int b = 0; b < nbits; ++b) {
      const bool bit = (e >> b) & 1;
      const unsigned long long bal = __ballot(bit);
      same &= bit ? bal : ~bal;
    }
    const int rank = __popcll(same & ((1ull << lane) - 1ull));   // equal ids in lower lanes
    int base = 0;
    if (valid) base = cnt[wave * E + e];
    __builtin_amdgcn_wave_barrier();
    if (valid) {
      sorted[base + rank] = i;
      atomicAdd(&cnt[wave * E + e], 1);
    }
  };
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    if (sb + 64 * b < se) place(sb + 64 * b + lane, first[b]);     // wave-uniform condition
  }
  for (int c0 = sb + 64 * NB; c0 < se; c0 += 64 * NB) {
    int more[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int i = c0 + 64 * b + lane;
      more[b] = i < se ? ids[i] : -1;
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if (c0 + 64 * b < se) place(c0 + 64 * b + lane, more[b]);
    }
  }
}

__global__ __launch_bounds__(1024) void moe_align_kernel(const int* __restrict__ ids, int n, int E,
                                                         int tile_m, int cap,
                                                         int* __restrict__ sorted,
                                                         int* __restrict__ expert_ids,
                                                         int* __restrict__ npp) {
  extern __shared__ int sm[];
  moe_align_block<0>(ids, n, E, tile_m, cap, sorted, expert_ids, npp, sm);
}

// Long slot lists: part b of gridDim.x parts covers slots [b * part, (b + 1) * part).
__global__ __launch_bounds__(1024) void moe_align_count_kernel(const int* __restrict__ ids, int n, int E,
                                                               int part, int* __restrict__ block_cnt) {
  extern __shared__ int sm[];
  const int s0 = min(n, (int)blockIdx.x * part), s1 = min(n, s0 + part);
  moe_align_block<1>(ids, n, E, 1, 0, nullptr, nullptr, nullptr, sm, s0, s1, block_cnt);
}

// One workgroup: per expert the padded length and first position, then every part's first
// position per expert (in place: counts in, positions out), the padding entries, the block
// owners and the unused tails.
__global__ __launch_bounds__(1024) void moe_align_scan_kernel(int n, int E, int tile_m, int cap, int parts,
                                                              int* __restrict__ block_tab,
                                                              int* __restrict__ sorted,
                                                              int* __restrict__ expert_ids,
                                                              int* __restrict__ npp) {
  extern __shared__ int sm[];
  int* padded = sm;        // [E]
  int* start = sm + E;     // [E]
  __shared__ int s_total;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // thread e keeps its expert's counts of all parts in registers (one memory round trip;
  // E <= 1024 = the workgroup size, parts <= 64)
  constexpr int PMAX = 64;
  int c[PMAX];
  const int my_e = tid < E ? tid : 0;
#pragma unroll
  for (int b = 0; b < PMAX; ++b) c[b] = block_tab[(size_t)min(b, parts - 1) * E + my_e];
  if (tid < E) {
    int tot = 0;
#pragma unroll
    for (int b = 0; b < PMAX; ++b) tot += b < parts ? c[b] : 0;
    padded[tid] = (tot + tile_m - 1) / tile_m * tile_m;
  }
  __syncthreads();
  if (wave == 0) {
    const int per = (E + 63) / 64;
    int local = 0;
    for (int k = 0; k < per; ++k) {
      const int e = lane * per + k;
      if (e < E) local += padded[e];
    }
    int incl = local;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int v = __shfl_up(incl, o);
      if (lane >= o) incl += v;
    }
    int pos = incl - local;
    for (int k = 0; k < per; ++k) {
      const int e = lane * per + k;
      if (e < E) { start[e] = pos; pos += padded[e]; }
    }
    if (lane == 63) { s_total = incl; npp[0] = incl; }
  }
  __syncthreads();
  const int total = s_total;
  if (tid < E) {
    const int e = tid;
    int pos = start[e];
    const int e0 = pos;
#pragma unroll
    for (int b = 0; b < PMAX; ++b) {
      if (b < parts) {
        block_tab[(size_t)b * E + e] = pos;
        pos += c[b];
      }
    }
    padded[e] = pos;          // from here on: first padding position of the expert's run
    (void)e0;
  }
  __syncthreads();
  // padding entries and block owners, one wave per expert at a time (coalesced stores)
  for (int e = wave; e < E; e += 16) {
    const int e0 = start[e];
    const int e1 = e + 1 < E ? start[e + 1] : total;
    for (int i = padded[e] + lane; i < e1; i += 64) sorted[i] = n;
    for (int b = e0 / tile_m + lane; b < e1 / tile_m; b += 64) expert_ids[b] = e;
  }
  for (int i = total + tid; i < cap; i += 1024) sorted[i] = n;
  for (int i = total / tile_m + tid; i < cap / tile_m; i += 1024) expert_ids[i] = -1;
}

__global__ __launch_bounds__(1024) void moe_align_place_kernel(const int* __restrict__ ids, int n, int E,
                                                               int part, int* __restrict__ block_start,
                                                               int* __restrict__ sorted) {
  extern __shared__ int sm[];
  const int s0 = min(n, (int)blockIdx.x * part), s1 = min(n, s0 + part);
  moe_align_block<2>(ids, n, E, 1, 0, sorted, nullptr, nullptr, sm, s0, s1, block_start);
}

// Routing and align in one launch for batches of at most 16 tokens (one wave per token, the
// same single workgroup then sorts the T * topk slots): a decode step of a few sequences
// spends more on the second launch than on either kernel's work.
template <int PER, bool SIGMOID>
__global__ __launch_bounds__(1024) void moe_route_align_kernel(const float* __restrict__ logits,
                                                               const float* __restrict__ bias, int T,
                                                               int E, int topk, int renorm, float scale,
                                                               int* ids, float* __restrict__ wts, int tile_m,
                                                               int cap, int* __restrict__ sorted,
                                                               int* __restrict__ expert_ids,
                                                               int* __restrict__ npp) {
  extern __shared__ int sm[];
  const int wave = threadIdx.x >> 6;
  if (wave < T) moe_topk_token<PER, SIGMOID>(logits, bias, wave, E, topk, renorm, scale, ids, wts);
  __syncthreads();   // the ids written above are read back by the same workgroup
  moe_align_block<0>(ids, T * topk, E, tile_m, cap, sorted, expert_ids, npp, sm);
}

__global__ __launch_bounds__(256) void silu_and_mul_kernel(const half_t* __restrict__ in,
                                                           half_t* __restrict__ out, int rows,
                                                           int inter) {
  // 8 halves per thread; inter % 8 == 0
  const int per_row = inter / 8;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (size_t)rows * per_row) return;
  const size_t r = idx / per_row, c = (idx % per_row) * 8;
  const h8 g = *reinterpret_cast<const h8*>(in + r * 2 * inter + c);
  const h8 u = *reinterpret_cast<const h8*>(in + r * 2 * inter + inter + c);
  h8 o;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float gv = (float)g[i];
    o[i] = (half_t)(gv / (1.f + __expf(-gv)) * (float)u[i]);
  }
  *reinterpret_cast<h8*>(out + r * inter + c) = o;
}

__global__ __launch_bounds__(256) void moe_sum_kernel(const half_t* __restrict__ in,
                                                      half_t* __restrict__ out, int T, int topk,
                                                      int H) {
  const int per_row = H / 8;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (size_t)T * per_row) return;
  const size_t t = idx / per_row, c = (idx % per_row) * 8;
  float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // eight slot rows in flight at a time (a loop of single loads pays one memory round trip
  // per slot); the sum runs in slot order either way
  for (int j0 = 0; j0 < topk; j0 += 8) {
    h8 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int j = min(j0 + u, topk - 1);
      v[u] = *reinterpret_cast<const h8*>(in + (t * topk + j) * H + c);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (j0 + u < topk) {
#pragma unroll
        for (int i = 0; i < 8; ++i) s[i] += (float)v[u][i];
      }
    }
  }
  h8 o;
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = (half_t)s[i];
  *reinterpret_cast<h8*>(out + t * H + c) = o;
}

}  // namespace awqmi
