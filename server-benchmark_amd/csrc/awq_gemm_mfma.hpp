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

constexpr int PF_BM = 256, PF_BN = 256, PF_BK = 64, PF_LD = 72;
constexpr int PF_LDS_BYTES = 2 * (PF_BM + PF_BN) * PF_LD * 2;

__global__ __launch_bounds__(256, 1) void awq_gemm_mfma_kernel(const MfmaGemmParams p) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  half_t* As = reinterpret_cast<half_t*>(smem_raw);   // [2][256][72]
  half_t* Bs = As + 2 * PF_BM * PF_LD;                // [2][256][72]

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

  // global->LDS roles
  const int a_row = tid >> 3, a_seg = tid & 7;   // + 32 * i rows
  const int kk = tid >> 5, wcl = tid & 31;       // 8-row slab, word column in tile
  int wcg = n0 / 8 + wcl;
  if (wcg >= p.NW) wcg = 0;                      // columns never stored; keep loads in bounds

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
    for (int i = 0; i < 8; ++i) {
      const int gr = m0 + a_row + 32 * i;
      areg[i] = gr < p.M ? *reinterpret_cast<const u4v*>(p.x + (size_t)gr * p.K + k0 + 8 * a_seg)
                         : u4v{0, 0, 0, 0};
    }
    const int kr = k0 + 8 * kk;
#pragma unroll
    for (int i = 0; i < 8; ++i) wreg[i] = p.qw[(size_t)(kr + i) * p.NW + wcg];
    const int g = kr / p.G;
    zreg = p.qz[(size_t)g * p.NW + wcg];
    sreg = *reinterpret_cast<const u4v*>(p.sc + (size_t)g * p.N + 8 * (size_t)wcg);
  };

  auto dq_byte = [&](half_t* bs, auto BTAG) {
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
    *reinterpret_cast<u4v*>(bs + (8 * wcl + cl) * PF_LD + 8 * kk) = lo;
    *reinterpret_cast<u4v*>(bs + (8 * wcl + ch) * PF_LD + 8 * kk) = hi;
  };

  auto sstore = [&](int buf) {
    half_t* as = As + buf * PF_BM * PF_LD;
    half_t* bs = Bs + buf * PF_BN * PF_LD;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      *reinterpret_cast<u4v*>(as + (a_row + 32 * i) * PF_LD + 8 * a_seg) = areg[i];
    dq_byte(bs, std::integral_constant<int, 0>{});
    dq_byte(bs, std::integral_constant<int, 1>{});
    dq_byte(bs, std::integral_constant<int, 2>{});
    dq_byte(bs, std::integral_constant<int, 3>{});
  };

  auto compute = [&](int buf) {
    const half_t* as = As + buf * PF_BM * PF_LD + (wm + (lane & 31)) * PF_LD + 8 * (lane >> 5);
    const half_t* bs = Bs + buf * PF_BN * PF_LD + (wn + (lane & 31)) * PF_LD + 8 * (lane >> 5);
#pragma unroll
    for (int ks = 0; ks < PF_BK / 16; ++ks) {
      h8 af[4], bf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const h8*>(as + 32 * i * PF_LD + 16 * ks);
#pragma unroll
      for (int j = 0; j < 4; ++j) bf[j] = *reinterpret_cast<const h8*>(bs + 32 * j * PF_LD + 16 * ks);
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
