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
  // outputs are never stored), so no load sits behind a branch.
  const int a_row = tid >> 3, a_seg = tid & 7;
  const half_t* a_src[8];
  int a_dst[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = a_row + 32 * i;
    const int gr = min(m0 + r, p.M - 1);
    a_src[i] = p.x + (size_t)gr * p.K + 8 * a_seg;
    a_dst[i] = r * PF_ROW_BYTES + ((a_seg ^ pf_swz(r)) << 4);
  }
  // W tile: thread (kk, wcl) takes rows 8kk..8kk+7 of word column wcl
  const int kk = tid >> 5, wcl = tid & 31;
  int wcg = n0 / 8 + wcl;
  if (wcg >= p.NW) wcg = 0;                      // columns never stored; keep loads in bounds
  const uint32_t* w_src = p.qw + (size_t)8 * kk * p.NW + wcg;
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
  u4v areg[8];
  uint32_t wreg[8];
  uint32_t zreg;
  u4v sreg;

  auto gload = [&](int kt) {
    const int k0 = kt * PF_BK;
#pragma unroll
    for (int i = 0; i < 8; ++i) areg[i] = *reinterpret_cast<const u4v*>(a_src[i] + k0);
    const uint32_t* ws = w_src + (size_t)k0 * p.NW;
#pragma unroll
    for (int i = 0; i < 8; ++i) wreg[i] = ws[(size_t)i * p.NW];
    const int g = (k0 + 8 * kk) / p.G;
    zreg = p.qz[(size_t)g * p.NW + wcg];
    sreg = *reinterpret_cast<const u4v*>(p.sc + (size_t)g * p.N + 8 * (size_t)wcg);
  };

  auto dq_byte = [&](unsigned char* bs, auto BTAG) {
    constexpr int B = decltype(BTAG)::value;
    const uint32_t tz = byte_pair<B>(zreg, zreg);
    const uint32_t zl = (tz & nm.lo) | MAGIC_LO, zh = (tz & nm.hi) | MAGIC_HI;
    constexpr int cl = awq_col_of_nibble(2 * B), ch = awq_col_of_nibble(2 * B + 1);
    // scale of the column in both half-words
    const uint32_t sw_l = sreg[cl >> 1], sw_h = sreg[ch >> 1];
    const uint32_t sl = (cl & 1) ? __builtin_amdgcn_perm(sw_l, sw_l, 0x03020302u)
                                 : __builtin_amdgcn_perm(sw_l, sw_l, 0x01000100u);
    const uint32_t sh = (ch & 1) ? __builtin_amdgcn_perm(sw_h, sw_h, 0x03020302u)
                                 : __builtin_amdgcn_perm(sw_h, sw_h, 0x01000100u);
    u4v lo, hi;
#pragma unroll
    for (int rp = 0; rp < 4; ++rp) {
      const uint32_t t = byte_pair<B>(wreg[2 * rp + 1], wreg[2 * rp]);
      lo[rp] = pk_mul(pk_sub((t & nm.lo) | MAGIC_LO, zl), sl);
      hi[rp] = pk_mul(pk_sub((t & nm.hi) | MAGIC_HI, zh), sh);
    }
    *reinterpret_cast<u4v*>(bs + b_base + cl * PF_ROW_BYTES + ((b_t ^ cl) << 4)) = lo;
    *reinterpret_cast<u4v*>(bs + b_base + ch * PF_ROW_BYTES + ((b_t ^ ch) << 4)) = hi;
  };

  auto sstore = [&](int buf) {
    unsigned char* as = As + buf * PF_TILE_BYTES;
    unsigned char* bs = Bs + buf * PF_TILE_BYTES;
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u4v*>(as + a_dst[i]) = areg[i];
    dq_byte(bs, std::integral_constant<int, 0>{});
    dq_byte(bs, std::integral_constant<int, 1>{});
    dq_byte(bs, std::integral_constant<int, 2>{});
    dq_byte(bs, std::integral_constant<int, 3>{});
  };

  auto compute = [&](int buf) {
    const unsigned char* as = As + buf * PF_TILE_BYTES + wm * PF_ROW_BYTES;
    const unsigned char* bs = Bs + buf * PF_TILE_BYTES + wn * PF_ROW_BYTES;
#pragma unroll
    for (int ks = 0; ks < PF_BK / 16; ++ks) {
      h8 af[4], bf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        af[i] = *reinterpret_cast<const h8*>(as + 32 * i * PF_ROW_BYTES + f_off[ks ^ (2 * (i & 1))]);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        bf[j] = *reinterpret_cast<const h8*>(bs + 32 * j * PF_ROW_BYTES + f_off[ks ^ (2 * (j & 1))]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
  };

  const int KT = p.K / PF_BK;
  gload(0);
  sstore(0);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    const bool more = kt + 1 < KT;
    if (more) gload(kt + 1);
    compute(buf);
    if (more) sstore(buf ^ 1);
    __syncthreads();
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
