// Prefill AWQ GEMM (M > 16): Y[M,N] = X[M,K] @ dequant(W) on fp16 MFMA, fp32 accumulate.
//
// Workgroup tile 256 x 256 x 64, four waves in a 2 x 2 arrangement, each wave a 128 x 128
// block of 4 x 4 v_mfma_f32_32x32x16_f16 accumulators (256 accumulator registers).  Both
// operands sit in LDS k-contiguous ([row][k], row stride 72 halves = 144 B so that eight
// neighbouring 16-byte reads fall in eight different 16-byte bank groups):
//   * X tile: 16-byte global loads -> registers -> 16-byte LDS stores;
//   * W tile: each thread takes 8 rows x 1 packed word (32 threads side by side read 128
//     contiguous bytes of a row), dequantises its 8 x 8 block to exact fp16 (w - z) * s with
//     the byte-pair trick (one perm + two and-or per four weights, then packed subtract and
//     packed multiply), and stores one 16-byte k-run per output column.
// LDS is double buffered: the global loads of k-tile t+1 are issued before the MFMA loop of
// tile t, the dequant and LDS stores of t+1 follow it, one barrier per k-tile.
// Workgroup ids are spread over the eight XCDs in contiguous ranges and walked in
// 8-row-tile groups so that the 32 workgroups resident on one XCD share X and W tiles
// through that XCD's L2.
#pragma once
#include "awq_common.hpp"

namespace awqmi {

struct MfmaGemmParams {
  const half_t* x;
  const uint32_t* qw;
  const half_t* sc;
  const uint32_t* qz;
  half_t* y;
  int M, K, N, NW, G;
  int mt, nt;     // tile counts
  int total;      // mt * nt
  int per_xcd;    // ceil(total / 8)
};

constexpr int PF_BM = 256, PF_BN = 256, PF_BK = 64;
constexpr int PF_ROW_BYTES = PF_BK * 2;                       // 128 B = eight 16-byte slots
constexpr int PF_TILE_BYTES = PF_BM * PF_ROW_BYTES;           // 32 KiB per operand per buffer
constexpr int PF_LDS_BYTES = 4 * PF_TILE_BYTES;               // A0 A1 B0 B1

// LDS layout of both operands: [row][64 halves], no padding, the 16-byte slot index XORed
// with (row ^ (row >> 3)) & 7.  Eight neighbouring rows then put the same logical slot into
// eight different bank groups (conflict-free fragment reads, lanes = rows), and the eight
// word columns a wave's neighbouring lanes dequantise (rows 8 apart) do too (conflict-free
// stores of the dequantised W tile).
__device__ __forceinline__ int pf_swz(int row) { return (row ^ (row >> 3)) & 7; }

__global__ __launch_bounds__(256, 1) void awq_gemm_mfma_kernel(const MfmaGemmParams p) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  unsigned char* const As = smem_raw;                        // [2][256][128 B]
  unsigned char* const Bs = smem_raw + 2 * PF_TILE_BYTES;    // [2][256][128 B]

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int id = blockIdx.x;
  const int nid = (id & 7) * p.per_xcd + (id >> 3);
  if (nid >= p.total) return;
  const int gsize = 8 * p.nt;
  const int first_m = (nid / gsize) * 8;
  const int gm = min(p.mt - first_m, 8);
  const int mt_i = first_m + (nid % gsize) % gm;
  const int nt_i = (nid % gsize) / gm;
  const int m0 = mt_i * PF_BM, n0 = nt_i * PF_BN;
  const int wm = (wave >> 1) * 128, wn = (wave & 1) * 128;

  // ---- global -> LDS roles -------------------------------------------------------------
  // X tile: thread (a_row + 32 i, a_seg) moves 16 bytes; rows past M re-read row M - 1 (their
  // outputs are never stored), so no load sits behind a branch.  Addresses are a uniform
  // base (advanced per k-tile on the scalar unit) plus a 32-bit lane offset.
  const int a_row = tid >> 3, a_seg = tid & 7;
  uint32_t a_off[8];
  int a_dst[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = a_row + 32 * i;
    const int gr = min(m0 + r, p.M - 1);
    a_off[i] = (uint32_t)(((size_t)gr * p.K + 8 * a_seg) * 2);
    a_dst[i] = r * PF_ROW_BYTES + ((a_seg ^ pf_swz(r)) << 4);
  }
  // W tile: thread (kk, wcl) takes rows 8kk..8kk+7 of word column wcl
  const int kk = tid >> 5, wcl = tid & 31;
  int wcg = n0 / 8 + wcl;
  if (wcg >= p.NW) wcg = 0;                      // columns never stored; keep loads in bounds
  const uint32_t w_off = (uint32_t)(((size_t)8 * kk * p.NW + wcg) * 4);
  const uint32_t w_row = (uint32_t)p.NW * 4;     // bytes between rows
  const int b_t = kk ^ (wcl & 7);                // slot of column c: (b_t ^ c)
  const int b_base = wcl * 8 * PF_ROW_BYTES;

  // ---- LDS -> fragment roles -----------------------------------------------------------
  // lane (i = lane % 32, hh = lane / 32) reads row base + i, logical slot 2 ks + hh; with
  // u = hh ^ swz(i) the physical slot is u ^ (2 ks) ^ (4 (tile & 1)): four lane offsets
  const int fi = lane & 31, fh = lane >> 5;
  const int fu = fh ^ pf_swz(fi);
  int f_off[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) f_off[c] = fi * PF_ROW_BYTES + ((fu ^ (2 * c)) << 4);

  f16v acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  NibbleMasks nm;
  nm.init();
  u4v areg[8];          // X tile in flight
  uint32_t wreg[2][8];  // two W tiles in flight (parity of the k-tile)
  uint32_t zreg[2];
  u4v sreg[2];
  const int KT = p.K / PF_BK;

  auto gload_a = [&](int kt) {
    const char* base = reinterpret_cast<const char*>(p.x) + (size_t)kt * PF_BK * 2;
#pragma unroll
    for (int i = 0; i < 8; ++i) areg[i] = *reinterpret_cast<const u4v*>(base + a_off[i]);
  };
  auto gload_w = [&](int kt, int set) {
    const char* base = reinterpret_cast<const char*>(p.qw) + (size_t)kt * PF_BK * p.NW * 4;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      wreg[set][i] = *reinterpret_cast<const uint32_t*>(base + (size_t)i * w_row + w_off);
    const int g = (kt * PF_BK + 8 * kk) / p.G;
    zreg[set] = p.qz[(size_t)g * p.NW + wcg];
    sreg[set] = *reinterpret_cast<const u4v*>(p.sc + (size_t)g * p.N + 8 * (size_t)wcg);
  };
  auto store_a = [&](int buf) {
    unsigned char* as = As + buf * PF_TILE_BYTES;
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u4v*>(as + a_dst[i]) = areg[i];
  };
  // dequantise byte B (two columns x eight rows) of W register set `set` into buffer `buf`
  auto dq_byte = [&](int buf, int set, auto BTAG) {
    constexpr int B = decltype(BTAG)::value;
    unsigned char* bs = Bs + buf * PF_TILE_BYTES;
    const uint32_t tz = byte_pair<B>(zreg[set], zreg[set]);
    const uint32_t zl = (tz & nm.lo) | MAGIC_LO, zh = (tz & nm.hi) | MAGIC_HI;
    constexpr int cl = awq_col_of_nibble(2 * B), ch = awq_col_of_nibble(2 * B + 1);
    const uint32_t sw_l = sreg[set][cl >> 1], sw_h = sreg[set][ch >> 1];
    const uint32_t sl = (cl & 1) ? __builtin_amdgcn_perm(sw_l, sw_l, 0x03020302u)
                                 : __builtin_amdgcn_perm(sw_l, sw_l, 0x01000100u);
    const uint32_t sh = (ch & 1) ? __builtin_amdgcn_perm(sw_h, sw_h, 0x03020302u)
                                 : __builtin_amdgcn_perm(sw_h, sw_h, 0x01000100u);
    u4v lo, hi;
#pragma unroll
    for (int rp = 0; rp < 4; ++rp) {
      const uint32_t t = byte_pair<B>(wreg[set][2 * rp + 1], wreg[set][2 * rp]);
      lo[rp] = pk_mul(pk_sub((t & nm.lo) | MAGIC_LO, zl), sl);
      hi[rp] = pk_mul(pk_sub((t & nm.hi) | MAGIC_HI, zh), sh);
    }
    *reinterpret_cast<u4v*>(bs + b_base + cl * PF_ROW_BYTES + ((b_t ^ cl) << 4)) = lo;
    *reinterpret_cast<u4v*>(bs + b_base + ch * PF_ROW_BYTES + ((b_t ^ ch) << 4)) = hi;
  };

  h8 af[2][4], bf[2][4];   // fragments of two 16-wide k-steps
  auto load_frags = [&](int buf, int ks, int fs) {
    const unsigned char* as = As + buf * PF_TILE_BYTES + wm * PF_ROW_BYTES;
    const unsigned char* bs = Bs + buf * PF_TILE_BYTES + wn * PF_ROW_BYTES;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      af[fs][i] = *reinterpret_cast<const h8*>(as + 32 * i * PF_ROW_BYTES + f_off[ks ^ (2 * (i & 1))]);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      bf[fs][j] = *reinterpret_cast<const h8*>(bs + 32 * j * PF_ROW_BYTES + f_off[ks ^ (2 * (j & 1))]);
  };
  auto mfma_step = [&](int fs) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[fs][i], bf[fs][j], acc[i][j], 0, 0, 0);
  };

  // Interleave recipe for one phase (16 MFMAs of one 16-wide k-step, the eight fragment
  // reads of the next one, the dequantisation of one byte of the next W tile): an MFMA
  // occupies the matrix pipe for eight passes, during which the wave can issue about seven
  // other instructions, so spread the VALU / LDS work evenly between the MFMAs.
  auto phase_schedule = [&](bool with_reads) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);               // MFMA
      if (with_reads) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
      __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);               // VALU
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);               // MFMA
      __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);               // VALU
    }
    __builtin_amdgcn_sched_group_barrier(0x200, 2, 0);                 // DS write
  };

  // One k-tile, PAR = kt & 1.  On entry: LDS buffer PAR holds tile kt, areg and W set PAR^1
  // hold tile kt + 1, W set PAR is free.  The body stores X(kt+1), refills areg and W set
  // PAR with tile kt + 2, then runs the four 16-wide k-steps of tile kt: each step's MFMAs
  // overlap the fragment reads of the next step and one byte of the dequantisation of
  // W(kt+1).  Tiles past the end re-read the last tile and are never used.
  auto body = [&](int kt, auto PTAG) {
    constexpr int PAR = decltype(PTAG)::value;
    const int kt2 = min(kt + 2, KT - 1);
    store_a(PAR ^ 1);
    __builtin_amdgcn_sched_barrier(0);
    gload_a(kt2);
    gload_w(kt2, PAR);
    load_frags(PAR, 0, 0);
    __builtin_amdgcn_sched_barrier(0);

    mfma_step(0);
    load_frags(PAR, 1, 1);
    dq_byte(PAR ^ 1, PAR ^ 1, std::integral_constant<int, 0>{});
    phase_schedule(true);
    __builtin_amdgcn_sched_barrier(0);

    mfma_step(1);
    load_frags(PAR, 2, 0);
    dq_byte(PAR ^ 1, PAR ^ 1, std::integral_constant<int, 1>{});
    phase_schedule(true);
    __builtin_amdgcn_sched_barrier(0);

    mfma_step(0);
    load_frags(PAR, 3, 1);
    dq_byte(PAR ^ 1, PAR ^ 1, std::integral_constant<int, 2>{});
    phase_schedule(true);
    __builtin_amdgcn_sched_barrier(0);

    mfma_step(1);
    dq_byte(PAR ^ 1, PAR ^ 1, std::integral_constant<int, 3>{});
    phase_schedule(false);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
  };

  // prologue: tile 0 into LDS buffer 0, tile 1 into registers
  gload_a(0);
  gload_w(0, 0);
  store_a(0);
  dq_byte(0, 0, std::integral_constant<int, 0>{});
  dq_byte(0, 0, std::integral_constant<int, 1>{});
  dq_byte(0, 0, std::integral_constant<int, 2>{});
  dq_byte(0, 0, std::integral_constant<int, 3>{});
  gload_a(min(1, KT - 1));
  gload_w(min(1, KT - 1), 1);
  __syncthreads();
  int kt = 0;
  for (; kt + 1 < KT; kt += 2) {
    body(kt, std::integral_constant<int, 0>{});
    body(kt + 1, std::integral_constant<int, 1>{});
  }
  if (kt < KT) body(kt, std::integral_constant<int, 0>{});

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
