// Prefill AWQ GEMM for many rows (M in the thousands): dequantise once, then a dense fp16 GEMM.
//
// At M = 8192 the fused kernel (awq_gemm_mfma.hpp) unpacks every weight 32 times, once per
// 256-row tile.  Here the weights are dequantised once per call into an fp16 panel in the
// caller's workspace (awq_dequant_panel_kernel, bit-exact (w - z) * s, the same arithmetic as
// awq_dequantize) and awq_gemm_dense_kernel multiplies X by that panel with no unpack
// arithmetic, no LDS writes from registers and no operand trip through registers at all:
// both operands go from global memory straight into LDS (`buffer_load_dwordx4 ... lds`).
//
// Panel layout.  The panel is not [K, N]: it is the sequence of LDS images the GEMM wants.
// Block (column tile c, k-stage t) of 16 KiB, at byte ((c * K / 32 + t) * 16384), holds the 256
// columns of tile c for k = 32 t .. 32 t + 31 as [column][4 slots of 8 halves], slot l of
// column j stored at physical slot l ^ ((j >> 2) & 3).  A k-stage of a column tile is one
// contiguous 16 KiB run, so its fetch is 16 fully coalesced 1 KiB wave loads, and all k-stages
// of a column tile are consecutive in memory.  Columns past N hold zeros.
//
// LDS.  A ring of NST stages of 32 KiB (X tile 256 x 32, W tile 256 x 32, both [row][64 B] with
// the slot swizzle above: 16 consecutive lanes of a fragment read -- rows i .. i + 15, one
// logical slot -- touch 16 different 16-byte bank groups).  Stage t + NST is requested as soon
// as every wave has left stage t, NST - 1 stage times before it is needed.  Every ring slot is an
// LDS object of its own, so that the compiler's wait before reading a slot counts only the
// loads issued after that slot's.
//
// Workgroup tile 256 x 256, four waves 2 x 2, each 128 x 128 = 4 x 4 v_mfma_f32_32x32x16_f16
// accumulators (the arrangement with the fewest LDS bytes per flop that fits the register
// file).  Per stage a wave issues 32 MFMAs, 16 fragment reads, 8 direct-to-LDS loads and one
// barrier.  The k-steps are accumulated in the same order as in the fused kernel, so for the
// same K split both kernels return the same bits.
#pragma once
#include <type_traits>

#include "awq_common.hpp"
#include "awq_gemm_mfma.hpp"

namespace awqmi {

constexpr int DG_BK = 32;                           // k per stage
constexpr int DG_ROW_BYTES = DG_BK * 2;             // 64 B per row and stage
constexpr int DG_OP_BYTES = 256 * DG_ROW_BYTES;     // 16 KiB per operand and stage
constexpr int DG_STAGE_BYTES = 2 * DG_OP_BYTES;     // X tile, then W tile

__host__ __device__ constexpr int dg_swz(int row) { return (row >> 2) & 3; }

// bytes of the panel of a [K, N] weight matrix (K % 64 == 0)
__host__ __device__ constexpr size_t dg_panel_bytes(int K, int N) {
  return (size_t)((N + 255) / 256) * (size_t)(K / DG_BK) * DG_OP_BYTES;
}

// ---------------------------------------------------------------------------------------------
// Dequantise into the panel.  One workgroup per (column tile, 64 rows of K): thread (kk, wcl)
// takes rows 8 kk .. 8 kk + 7 of packed word column wcl of the tile, i.e. for each of its eight
// logical columns one run of eight consecutive k = one 16-byte slot of the panel.  The 32 KiB
// (two k-stages) are collected in LDS and leave as 16-byte stores in address order.
// G % 8 == 0 (a thread's eight rows share a group).
__global__ __launch_bounds__(256) void awq_dequant_panel_kernel(const uint32_t* __restrict__ qw,
                                                                const half_t* __restrict__ sc,
                                                                const uint32_t* __restrict__ qz,
                                                                unsigned char* __restrict__ panel, int K, int N,
                                                                int NW, int G, int ldw) {
  // staging layout: 16-byte unit (kk, column j) at kk * 4096 + (j >> 3) * 128 + (((j & 7) ^ ((j >> 4) & 7)) << 4):
  // the 32 lanes that store one column each (j = 8 wcl + c) spread over all bank groups
  __shared__ __align__(16) unsigned char tile[2 * DG_OP_BYTES];
  const int tid = threadIdx.x;
  const int nt_i = blockIdx.x, k64 = blockIdx.y;
  const int kk = tid >> 5, wcl = tid & 31;
  const int wcg = nt_i * 32 + wcl;
  const int k0 = k64 * 64 + 8 * kk;
  uint32_t w[8], z = 0;
  u4v s = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int i = 0; i < 8; ++i) w[i] = 0;
  if (wcg < NW) {
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = __builtin_nontemporal_load(qw + (size_t)(k0 + i) * ldw + wcg);
    const int g = k0 / G;
    z = qz[(size_t)g * NW + wcg];
    s = *reinterpret_cast<const u4v*>(sc + (size_t)g * N + 8 * (size_t)wcg);
  }
  NibbleMasks nm;
  nm.init();
  unsigned char* const mine = tile + kk * 4096 + wcl * 128;
  const int sx = (wcl >> 1) & 7;
  auto byte_runs = [&](auto BTAG) {
    constexpr int B = decltype(BTAG)::value;
    constexpr int cl = awq_col_of_nibble(2 * B), ch = awq_col_of_nibble(2 * B + 1);
    const uint32_t tz = byte_pair<B>(z, z);
    const uint32_t zl = (tz & nm.lo) | MAGIC_LO, zh = (tz & nm.hi) | MAGIC_HI;
    const uint32_t sw_l = s[cl >> 1], sw_h = s[ch >> 1];
    const uint32_t sl = (cl & 1) ? __builtin_amdgcn_perm(sw_l, sw_l, 0x03020302u)
                                 : __builtin_amdgcn_perm(sw_l, sw_l, 0x01000100u);
    const uint32_t sh = (ch & 1) ? __builtin_amdgcn_perm(sw_h, sw_h, 0x03020302u)
                                 : __builtin_amdgcn_perm(sw_h, sw_h, 0x01000100u);
    u4v lo, hi;
#pragma unroll
    for (int rp = 0; rp < 4; ++rp) {
      const uint32_t t = byte_pair<B>(w[2 * rp + 1], w[2 * rp]);
      lo[rp] = pk_mul(pk_sub((t & nm.lo) | MAGIC_LO, zl), sl);
      hi[rp] = pk_mul(pk_sub((t & nm.hi) | MAGIC_HI, zh), sh);
    }
    *reinterpret_cast<u4v*>(mine + ((cl ^ sx) << 4)) = lo;
    *reinterpret_cast<u4v*>(mine + ((ch ^ sx) << 4)) = hi;
  };
  byte_runs(std::integral_constant<int, 0>{});
  byte_runs(std::integral_constant<int, 1>{});
  byte_runs(std::integral_constant<int, 2>{});
  byte_runs(std::integral_constant<int, 3>{});
  __syncthreads();
  unsigned char* dst = panel + ((size_t)nt_i * (size_t)(K / DG_BK) + 2 * (size_t)k64) * DG_OP_BYTES;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int q = i * 256 + tid;                 // 16-byte unit of the two stage blocks, in address order
    const int stage = q >> 10, row = (q >> 2) & 255, ps = q & 3;
    const int skk = stage * 4 + (ps ^ dg_swz(row));
    const int swc = row >> 3;
    const u4v v = *reinterpret_cast<const u4v*>(tile + skk * 4096 + swc * 128 + (((row & 7) ^ ((swc >> 1) & 7)) << 4));
    __builtin_nontemporal_store(v, reinterpret_cast<u4v*>(dst + (size_t)q * 16));
  }
}

// ---------------------------------------------------------------------------------------------
struct DenseGemmParams {
  const half_t* x;               // [M, K]
  const unsigned char* panel;    // dg_panel_bytes(K, N)
  half_t* y;                     // [M, N]
  int M, K, N;
  int mt, nt;                    // 256-row and 256-column tile counts
  int per_xcd;                   // ceil(dp_tiles / 8)
  // as in MfmaGemmParams: tiles [0, dp_tiles) one workgroup each; the sk_tiles tiles of a sparse
  // last round are split in K over sk_split workgroups and summed by the reduce kernel
  int dp_tiles, sk_tiles, sk_split;
  float* sk_part;
};

// Wait until at most VM of this thread's loads are outstanding and its LDS reads have returned,
// then the workgroup barrier.  Written as one asm statement with a memory clobber: no LDS access
// moves across it, and the compiler's own fences, which would wait for every direct-to-LDS load
// in flight (vmcnt(0)), stay out.
template <int VM>
__device__ __forceinline__ void dg_wait_and_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(VM) : "memory");
}

template <int NST>
__global__ __launch_bounds__(256, 1) void awq_gemm_dense_kernel(const DenseGemmParams p) {
  static_assert(NST >= 3 && NST <= 5, "ring of three to five 32 KiB stages");
  typedef __attribute__((address_space(3))) void lds_void;
  __shared__ __align__(1024) unsigned char st0[DG_STAGE_BYTES];
  __shared__ __align__(1024) unsigned char st1[DG_STAGE_BYTES];
  __shared__ __align__(1024) unsigned char st2[DG_STAGE_BYTES];
  __shared__ __align__(1024) unsigned char st3[NST > 3 ? DG_STAGE_BYTES : 16];
  __shared__ __align__(1024) unsigned char st4[NST > 4 ? DG_STAGE_BYTES : 16];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int id = blockIdx.x;
  const int KT64 = p.K / 64;
  int nid = 0, kb = 0, ke = 2 * KT64, part = -1;
  if (id < 8 * p.per_xcd) {
    nid = (id & 7) * p.per_xcd + (id >> 3);
    if (nid >= p.dp_tiles) return;
  } else {
    const int j = id - 8 * p.per_xcd;
    nid = p.dp_tiles + j / p.sk_split;
    part = j % p.sk_split;
    kb = 2 * (int)((long long)KT64 * part / p.sk_split);
    ke = 2 * (int)((long long)KT64 * (part + 1) / p.sk_split);
  }
  const int gsize = PF_GROUP_M * p.nt;
  const int first_m = (nid / gsize) * PF_GROUP_M;
  const int gm = min(p.mt - first_m, PF_GROUP_M);
  const int mt_i = first_m + (nid % gsize) % gm;
  const int nt_i = (nid % gsize) / gm;
  const int m0 = mt_i * 256, n0 = nt_i * 256;
  const int wm = (wave >> 1) * 128, wn = (wave & 1) * 128;

  const __amdgpu_buffer_rsrc_t rx = pf_rsrc(p.x, (size_t)p.M * p.K * 2);
  const size_t col_tile_bytes = (size_t)(p.K / DG_BK) * DG_OP_BYTES;
  const __amdgpu_buffer_rsrc_t rw = pf_rsrc(p.panel + (size_t)nt_i * col_tile_bytes, col_tile_bytes);

  // ---- global -> LDS roles ---------------------------------------------------------------
  // X: instruction i of wave w fills rows 16 (4 i + w) .. + 15 of the stage (1 KiB); lane l
  // lands in row + l / 4, physical slot l % 4, so it fetches logical slot (l % 4) ^ swz(row),
  // and swz(row) = (l >> 4) & 3 for every i.  Rows past M re-read row M - 1 (never stored).
  uint32_t x_voff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 16 * (4 * i + wave) + (lane >> 2);
    const int gr = min(m0 + r, p.M - 1);
    x_voff[i] = (uint32_t)(((size_t)gr * p.K + 8 * ((lane & 3) ^ ((lane >> 4) & 3))) * 2);
  }
  // W: the stage block is the LDS image; instruction i of wave w copies its KiB 4 i + w
  const uint32_t w_voff = (uint32_t)lane * 16u;

  // ---- LDS -> fragment roles -------------------------------------------------------------
  // lane (fi = lane % 32, fh = lane / 32) reads row base + fi, logical slot 2 ks + fh
  const int fi = lane & 31, fh = lane >> 5;
  uint32_t fa_off[2], fb_off[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    const uint32_t o = (uint32_t)(fi * DG_ROW_BYTES + (((2 * ks + fh) ^ dg_swz(fi)) << 4));
    fa_off[ks] = o + (uint32_t)(wm * DG_ROW_BYTES);
    fb_off[ks] = o + (uint32_t)(DG_OP_BYTES + wn * DG_ROW_BYTES);
  }

  f16v acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  auto slot_ptr = [&](auto STAG) -> unsigned char* {
    constexpr int S = decltype(STAG)::value;
    if constexpr (S == 0) return st0;
    else if constexpr (S == 1) return st1;
    else if constexpr (S == 2) return st2;
    else if constexpr (S == 3) return st3;
    else return st4;
  };
  // request k-stage kt into ring slot S (stages past the end fetch the last one again: the
  // number of loads in flight behind any stage stays the same to the end of the loop)
  auto issue = [&](auto STAG, int kt) {
    unsigned char* const st = slot_ptr(STAG);
    const int ktc = min(kt, ke - 1);
    const uint32_t sx = (uint32_t)ktc * DG_ROW_BYTES;
    const uint32_t sw = (uint32_t)ktc * DG_OP_BYTES + (uint32_t)wave * 1024u;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_void*)(st + (4 * i + wave) * 1024), 16, x_voff[i], sx, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_void*)(st + DG_OP_BYTES + (4 * i + wave) * 1024), 16, w_voff,
                                               sw + (uint32_t)i * 4096u, 0, 0);
  };

  h8 af[2][4], bf[2][4];
  auto frags = [&](auto STAG, auto KS, auto FS) {
    constexpr int ks = decltype(KS)::value, fs = decltype(FS)::value;
    const unsigned char* const st = slot_ptr(STAG);
#pragma unroll
    for (int i = 0; i < 4; ++i) af[fs][i] = *reinterpret_cast<const h8*>(st + 32 * i * DG_ROW_BYTES + fa_off[ks]);
#pragma unroll
    for (int j = 0; j < 4; ++j) bf[fs][j] = *reinterpret_cast<const h8*>(st + 32 * j * DG_ROW_BYTES + fb_off[ks]);
  };
  auto mfma_step = [&](auto FS) {
    constexpr int fs = decltype(FS)::value;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[fs][i], bf[fs][j], acc[i][j], 0, 0, 0);
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;

  // One k-stage kt in ring slot S.  On entry fragment set 0 holds its first k-step.
  auto body = [&](auto STAG, int kt) {
    constexpr int S = decltype(STAG)::value;
    using SN = std::integral_constant<int, (S + 1) % NST>;
    // first k-step from registers while the second one's fragments are read
    frags(STAG, I1{}, I1{});
    mfma_step(I0{});
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    // stage kt + 1 has landed (own loads; the barrier extends that to every thread's) and this
    // wave's reads of stage kt have returned
    dg_wait_and_barrier<(NST - 2) * 8>();
    __builtin_amdgcn_sched_barrier(0);
    // slot S is free: request stage kt + NST into it; second k-step from registers while the
    // first fragments of stage kt + 1 are read
    issue(STAG, kt + NST);
    frags(SN{}, I0{}, I0{});
    mfma_step(I1{});
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // prologue: fill the ring
  issue(std::integral_constant<int, 0>{}, kb);
  issue(std::integral_constant<int, 1>{}, kb + 1);
  issue(std::integral_constant<int, 2>{}, kb + 2);
  if constexpr (NST > 3) issue(std::integral_constant<int, 3>{}, kb + 3);
  if constexpr (NST > 4) issue(std::integral_constant<int, 4>{}, kb + 4);
  dg_wait_and_barrier<(NST - 1) * 8>();
  frags(I0{}, I0{}, I0{});
  __builtin_amdgcn_sched_barrier(0);
  int kt = kb;
  for (int full = (ke - kb) / NST; full > 0; --full, kt += NST) {
    body(std::integral_constant<int, 0>{}, kt);
    body(std::integral_constant<int, 1>{}, kt + 1);
    body(std::integral_constant<int, 2>{}, kt + 2);
    if constexpr (NST > 3) body(std::integral_constant<int, 3>{}, kt + 3);
    if constexpr (NST > 4) body(std::integral_constant<int, 4>{}, kt + 4);
  }
  // the stages left over when the count is not a multiple of the ring length
  if (kt < ke) {
    body(std::integral_constant<int, 0>{}, kt);
    if (kt + 1 < ke) {
      body(std::integral_constant<int, 1>{}, kt + 1);
      if (kt + 2 < ke) {
        body(std::integral_constant<int, 2>{}, kt + 2);
        if constexpr (NST > 4) {
          if (kt + 3 < ke) body(std::integral_constant<int, 3>{}, kt + 3);
        }
      }
    }
  }
  // no load may still be writing this workgroup's LDS when it is handed to the next one
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // ---- split-K tiles: fp32 partial to the workspace (layout of awq_gemm_mfma_reduce_kernel<4, 4>)
  if (part >= 0) {
    const int tl = nid - p.dp_tiles;
    float* mine = p.sk_part + ((size_t)tl * p.sk_split + part) * PF_SK_SLOT_FLOATS;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; r += 4) {
          const int q = ((i * 4 + j) * 16 + r) >> 2;
          const f4 v = {acc[i][j][r], acc[i][j][r + 1], acc[i][j][r + 2], acc[i][j][r + 3]};
          *reinterpret_cast<f4*>(mine + ((size_t)q * 256 + tid) * 4) = v;
        }
    return;
  }

  // D[i][j] of a 32x32 tile: j = lane % 32, i = 8 * (r / 4) + 4 * (lane / 32) + r % 4
  const int col_l = lane & 31, row_l = 4 * (lane >> 5);
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + wn + 32 * j + col_l;
      if (col >= p.N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm + 32 * i + 8 * (r >> 2) + row_l + (r & 3);
        if (row < p.M) p.y[(size_t)row * p.N + col] = (half_t)acc[i][j][r];
      }
    }
}

}  // namespace awqmi
