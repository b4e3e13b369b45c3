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
// Block (column tile c, k-stage t) of 32 KiB, at byte ((c * K / 64 + t) * 32768), holds the 256
// columns of tile c for k = 64 t .. 64 t + 63 as [column][8 slots of 8 halves], slot l of
// column j stored at physical slot l ^ ((j >> 1) & 7).  A k-stage of a column tile is one
// contiguous 32 KiB run, so its fetch is 32 fully coalesced 1 KiB wave loads, and all k-stages
// of a column tile are consecutive in memory.  Columns past N hold zeros.
//
// LDS.  Five tile buffers of 32 KiB -- all 160 KiB of a CU -- each [row][128 B] with the slot
// swizzle above (the 16 consecutive lanes of a fragment read -- rows i .. i + 15, one logical
// slot -- touch 16 different 16-byte bank groups; an X row of a stage is one whole 128-byte
// line).  A stage (64 k) is an X tile and a W tile; four buffers hold the stage being multiplied
// and the next one, and the fifth lets the X tile of the stage after that be requested half a
// stage early, so that the direct-to-LDS loads are spread evenly over the loop (X tiles while
// the first k-step of a stage is multiplied, W tiles during the second) instead of running at
// the load path's full rate for half of the time.  Each buffer is an LDS object of its own, so
// that the compiler's wait before reading one counts only the loads issued after it.
//
// Workgroup tile 256 x 256, four waves 2 x 2, each 128 x 128 = 8 x 8 v_mfma_f32_16x16x32_f16
// accumulators.  The 16 x 16 x 32 shape is the one that gives the most flops under the chip's
// power limit: a bare loop of it holds 2.0 GHz with random operands where the 32 x 32 x 16 shape
// holds 1.7 GHz (about 1.95 against 1.7 PFLOP/s sustained).  The weights are the A operand and the
// activations the B operand, so that a lane's four accumulator values of a tile are four
// consecutive output columns of one row (8 bytes; they are gathered into whole 256-byte row
// pieces through LDS before they are stored).  Per stage a wave issues 128 MFMAs,
// 32 fragment reads, 16 direct-to-LDS loads and one barrier.
#pragma once
#include <type_traits>

#include "awq_common.hpp"
#include "awq_gemm_mfma.hpp"

namespace awqmi {

constexpr int DG_BK = 64;                           // k per stage
constexpr int DG_ROW_BYTES = DG_BK * 2;             // 128 B per row and stage
constexpr int DG_OP_BYTES = 256 * DG_ROW_BYTES;     // 32 KiB per operand and stage
constexpr int DG_STAGE_BYTES = 2 * DG_OP_BYTES;     // X tile, then W tile

__host__ __device__ constexpr int dg_swz(int row) { return (row >> 1) & 7; }

// bytes of the panel of a [K, N] weight matrix (K % 64 == 0)
__host__ __device__ constexpr size_t dg_panel_bytes(int K, int N) {
  return (size_t)((N + 255) / 256) * (size_t)(K / DG_BK) * DG_OP_BYTES;
}

// ---------------------------------------------------------------------------------------------
// Dequantise into the panel.  One workgroup per (column tile, k-stage): thread (kk, wcl) takes
// rows 8 kk .. 8 kk + 7 of packed word column wcl of the tile, i.e. for each of its eight logical
// columns one run of eight consecutive k = one 16-byte slot of the panel.  The 32 KiB are
// collected in LDS and leave as 16-byte stores in address order.  G % 8 == 0 (a thread's eight
// rows share a group).
__global__ __launch_bounds__(256) void awq_dequant_panel_kernel(const uint32_t* __restrict__ qw,
                                                                const half_t* __restrict__ sc,
                                                                const uint32_t* __restrict__ qz,
                                                                unsigned char* __restrict__ panel, int K, int N,
                                                                int NW, int G, int ldw) {
  // staging layout: 16-byte unit (kk, column j) at kk * 4096 + (j >> 3) * 128 + (((j & 7) ^ ((j >> 4) & 7)) << 4):
  // the 32 lanes that store one column each (j = 8 wcl + c) spread over all bank groups
  __shared__ __align__(16) unsigned char tile[DG_OP_BYTES];
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
  unsigned char* dst = panel + ((size_t)nt_i * (size_t)(K / DG_BK) + (size_t)k64) * DG_OP_BYTES;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int q = i * 256 + tid;                 // 16-byte unit of the stage block, in address order
    const int row = q >> 3, ps = q & 7;
    const int skk = ps ^ dg_swz(row);
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
// in flight whatever VM says, stay out.
template <int VM>
__device__ __forceinline__ void dg_wait_and_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(VM) : "memory");
}

// acc += A(16 x 32) * B(32 x 16) with the accumulator tile in place in the accumulation
// registers.  As an asm statement the result is tied to its input, which keeps each of the 64
// tiles in one register tuple for the whole loop (as a builtin the allocator gives some results
// other registers and then permutes the tiles at the loop's back edge: 2.4 moves per MFMA).
// A tile is touched once per 64 MFMAs, so no dependent-issue wait states are needed.
__device__ __forceinline__ void dg_mfma(f4& c, const h8& a, const h8& b) {
  asm("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

__global__ __launch_bounds__(256, 1) void awq_gemm_dense_kernel(const DenseGemmParams p) {
  typedef __attribute__((address_space(3))) void lds_void;
  // five tile buffers of 32 KiB, the whole LDS of a CU: stage t keeps its X tile in buffer
  // 2 t mod 5 and its W tile in buffer (2 t + 1) mod 5
  __shared__ __align__(1024) unsigned char tb0[DG_OP_BYTES];
  __shared__ __align__(1024) unsigned char tb1[DG_OP_BYTES];
  __shared__ __align__(1024) unsigned char tb2[DG_OP_BYTES];
  __shared__ __align__(1024) unsigned char tb3[DG_OP_BYTES];
  __shared__ __align__(1024) unsigned char tb4[DG_OP_BYTES];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int id = blockIdx.x;
  const int KT = p.K / DG_BK;
  int nid = 0, kb = 0, ke = KT, part = -1;
  if (id < 8 * p.per_xcd) {
    nid = (id & 7) * p.per_xcd + (id >> 3);
    if (nid >= p.dp_tiles) return;
  } else {
    const int j = id - 8 * p.per_xcd;
    nid = p.dp_tiles + j / p.sk_split;
    part = j % p.sk_split;
    kb = (int)((long long)KT * part / p.sk_split);
    ke = (int)((long long)KT * (part + 1) / p.sk_split);
  }
  const int gsize = PF_GROUP_M * p.nt;
  const int first_m = (nid / gsize) * PF_GROUP_M;
  const int gm = min(p.mt - first_m, PF_GROUP_M);
  const int mt_i = first_m + (nid % gsize) % gm;
  const int nt_i = (nid % gsize) / gm;
  const int m0 = mt_i * 256, n0 = nt_i * 256;
  const int wm = (wave >> 1) * 128, wn = (wave & 1) * 128;

  const __amdgpu_buffer_rsrc_t rx = pf_rsrc(p.x, (size_t)p.M * p.K * 2);
  const size_t col_tile_bytes = (size_t)KT * DG_OP_BYTES;
  const __amdgpu_buffer_rsrc_t rw = pf_rsrc(p.panel + (size_t)nt_i * col_tile_bytes, col_tile_bytes);

  // ---- global -> LDS roles ---------------------------------------------------------------
  // X: instruction i of wave w fills rows 8 (4 i + w) .. + 7 of the tile (1 KiB); lane l lands in
  // row + l / 8, physical slot l % 8, so it fetches logical slot (l % 8) ^ swz(row), and
  // swz(row) = (l >> 4) + 4 (w & 1) for every i.  Rows past M re-read row M - 1 (never stored).
  uint32_t x_voff[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = 8 * (4 * i + wave) + (lane >> 3);
    const int gr = min(m0 + r, p.M - 1);
    x_voff[i] = (uint32_t)(((size_t)gr * p.K + 8 * ((lane & 7) ^ dg_swz(r))) * 2);
  }
  // W: the stage block is the LDS image; instruction i of wave w copies its KiB 4 i + w
  const uint32_t w_voff = (uint32_t)lane * 16u;

  // ---- LDS -> fragment roles -------------------------------------------------------------
  // lane (fi = lane % 16, fq = lane / 16) reads row base + fi, logical slot 4 ks + fq
  const int fi = lane & 15, fq = lane >> 4;
  uint32_t fx_off[2], fw_off[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    const uint32_t o = (uint32_t)(fi * DG_ROW_BYTES + (((4 * ks + fq) ^ dg_swz(fi)) << 4));
    fx_off[ks] = o + (uint32_t)(wm * DG_ROW_BYTES);
    fw_off[ks] = o + (uint32_t)(wn * DG_ROW_BYTES);
  }

  // acc[in][im]: columns n0 + wn + 16 in + 4 (lane / 16) + 0..3 of row m0 + wm + 16 im + lane % 16
  f4 acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};

  auto buf = [&](auto BTAG) -> unsigned char* {
    constexpr int B = decltype(BTAG)::value;
    if constexpr (B == 0) return tb0;
    else if constexpr (B == 1) return tb1;
    else if constexpr (B == 2) return tb2;
    else if constexpr (B == 3) return tb3;
    else return tb4;
  };
  auto load_x = [&](unsigned char* dst, int kt, int i) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_void*)(dst + (4 * i + wave) * 1024), 16, x_voff[i],
                                             (uint32_t)min(kt, ke - 1) * DG_ROW_BYTES, 0, 0);
  };
  auto load_w = [&](unsigned char* dst, int kt, int i) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_void*)(dst + (4 * i + wave) * 1024), 16, w_voff,
                                             (uint32_t)min(kt, ke - 1) * DG_OP_BYTES + (uint32_t)(4 * i + wave) * 1024u, 0, 0);
  };
  h8 xf[2][8], wf[2][8];

  // One k-step of 64 MFMAs out of fragment set FS, in 32 pairs.  Between the pairs go the 16 fragment reads of the next k-step (k-step
  // KSN of tiles xr / wr, into the other fragment set) and eight direct-to-LDS loads: of the X
  // tile (WLOAD = 0) or the W tile (WLOAD = 1) of k-stage kt_load into buffer dst.  The order is
  // pinned as written: the MFMAs are asm statements, which the scheduler's instruction groups
  // cannot name.
  auto kstep = [&](auto FS, const unsigned char* xr, const unsigned char* wr, auto KSN, auto WLOAD, unsigned char* dst,
                   int kt_load) {
    constexpr int fs = decltype(FS)::value, ksn = decltype(KSN)::value;
#pragma unroll
    for (int h = 0; h < 32; ++h) {
      // 2 x 2 blocks of accumulator tiles, walked so that one operand changes from one MFMA to the
      // next (block rows run forth and back): under the power limit this order sustains 3 % more
      // than "one weight fragment against all eight activation fragments" in a bare MFMA loop
      const int b = h >> 1, i = 2 * (b >> 2), j = (b & 4) ? 6 - 2 * (b & 3) : 2 * (b & 3);
      if (!(h & 1)) {
        dg_mfma(acc[i][j], wf[fs][i], xf[fs][j]);
        dg_mfma(acc[i + 1][j], wf[fs][i + 1], xf[fs][j]);
      } else {
        dg_mfma(acc[i + 1][j + 1], wf[fs][i + 1], xf[fs][j + 1]);
        dg_mfma(acc[i][j + 1], wf[fs][i], xf[fs][j + 1]);
      }
      __builtin_amdgcn_sched_barrier(0);
      // at most one memory instruction per pair of MFMAs (the next k-step starts with wf[0..1],
      // xf[0..1], which are read first)
      const int f = h >> 2;
      if ((h & 3) == 0) wf[fs ^ 1][f] = *reinterpret_cast<const h8*>(wr + 16 * f * DG_ROW_BYTES + fw_off[ksn]);
      else if ((h & 3) == 2) xf[fs ^ 1][f] = *reinterpret_cast<const h8*>(xr + 16 * f * DG_ROW_BYTES + fx_off[ksn]);
      else if ((h & 3) == 1) {
        if constexpr (decltype(WLOAD)::value) load_w(dst, kt_load, f);
        else load_x(dst, kt_load, f);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;

  // One k-stage kt, R = (kt - kb) mod 5.  On entry fragment set 0 holds its first k-step, its
  // tiles and stage kt + 1's W tile are in LDS or on their way, and one buffer is free.
  auto body = [&](auto RTAG, int kt) {
    constexpr int R = decltype(RTAG)::value;
    unsigned char* const xb = buf(std::integral_constant<int, (2 * R) % 5>{});
    unsigned char* const wb = buf(std::integral_constant<int, (2 * R + 1) % 5>{});
    unsigned char* const xn = buf(std::integral_constant<int, (2 * R + 2) % 5>{});
    unsigned char* const wn_ = buf(std::integral_constant<int, (2 * R + 3) % 5>{});
    unsigned char* const spare = buf(std::integral_constant<int, (2 * R + 4) % 5>{});
    // first k-step from registers while the second one's fragments are read and the X tile of
    // stage kt + 2 is requested into the free buffer
    kstep(I0{}, xb, wb, I1{}, I0{}, spare, kt + 2);
    // stage kt + 1 has landed -- everything but the eight loads just issued (own loads; the
    // barrier extends that to every thread's) -- and this wave's reads of stage kt have returned
    dg_wait_and_barrier<8>();
    __builtin_amdgcn_sched_barrier(0);
    // stage kt's buffers are free: its X buffer takes the W tile of stage kt + 2; second k-step
    // from registers while the first fragments of stage kt + 1 are read
    kstep(I1{}, xn, wn_, I0{}, I1{}, xb, kt + 2);
  };

  // prologue: stages kb and kb + 1 requested, the first one waited for
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    load_x(tb0, kb, i);
    load_w(tb1, kb, i);
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    load_x(tb2, kb + 1, i);
    load_w(tb3, kb + 1, i);
  }
  dg_wait_and_barrier<16>();
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    wf[0][i] = *reinterpret_cast<const h8*>(tb1 + 16 * i * DG_ROW_BYTES + fw_off[0]);
    xf[0][i] = *reinterpret_cast<const h8*>(tb0 + 16 * i * DG_ROW_BYTES + fx_off[0]);
  }
  __builtin_amdgcn_sched_barrier(0);
  int kt = kb;
  for (int full = (ke - kb) / 5; full > 0; --full, kt += 5) {
    body(std::integral_constant<int, 0>{}, kt);
    body(std::integral_constant<int, 1>{}, kt + 1);
    body(std::integral_constant<int, 2>{}, kt + 2);
    body(std::integral_constant<int, 3>{}, kt + 3);
    body(std::integral_constant<int, 4>{}, kt + 4);
  }
  // the stages left over when the count is not a multiple of five
  if (kt < ke) {
    body(std::integral_constant<int, 0>{}, kt);
    if (kt + 1 < ke) {
      body(std::integral_constant<int, 1>{}, kt + 1);
      if (kt + 2 < ke) {
        body(std::integral_constant<int, 2>{}, kt + 2);
        if (kt + 3 < ke) body(std::integral_constant<int, 3>{}, kt + 3);
      }
    }
  }
  // no load may still be writing this workgroup's LDS when it is handed to the next one; the
  // last MFMAs have left the pipe before their results are read (they are asm statements, for
  // which the compiler inserts no wait states)
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");

  // ---- split-K tiles: fp32 partial to the workspace, [accumulator tile][thread] groups of four
  if (part >= 0) {
    const int tl = nid - p.dp_tiles;
    float* mine = p.sk_part + ((size_t)tl * p.sk_split + part) * PF_SK_SLOT_FLOATS;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) *reinterpret_cast<f4*>(mine + ((size_t)(i * 8 + j) * 256 + tid) * 4) = acc[i][j];
    return;   // summed and written out by awq_gemm_dense_reduce_kernel, launched behind this kernel
  }

  // Output.  A lane's four values of an accumulator tile are 8 bytes of one row; stored like that,
  // a store instruction carries sixteen 32-byte pieces, and when all workgroups finish their tiles
  // together the write path takes 8 - 9 us per tile for them.  So the wave's 128 x 128 results go
  // through its own 32 KiB of LDS first (every wave has read its last fragments by then: the
  // barrier) -- row = 256 bytes, 16-byte chunk c of row r kept at chunk c ^ (r % 16), which makes
  // the 8-byte writes of a half-wave and the 16-byte reads conflict-free -- and leave sixteen rows
  // at a time as 16 bytes per lane, 256 contiguous bytes per row (1 % faster at K = 8192, 4 % at
  // K = 2048, same bits).
  dg_wait_and_barrier<0>();
  unsigned char* const st = wave == 0 ? tb0 : (wave == 1 ? tb1 : (wave == 2 ? tb2 : tb3));
  const int r_l = lane & 15, g = lane >> 4;
  unsigned char* const wbase = st + r_l * 256 + 8 * (g & 1);
  const unsigned char* const rbase = st + g * 256;
  const int c16 = lane & 15;
  const int col = n0 + wn + 8 * c16;      // N % 8 == 0: the eight columns are all inside or all outside
#pragma unroll
  for (int j = 0; j < 8; ++j) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const h4 v = {(half_t)acc[i][j][0], (half_t)acc[i][j][1], (half_t)acc[i][j][2], (half_t)acc[i][j][3]};
      const int c = 2 * i + (g >> 1);
      *reinterpret_cast<h4*>(wbase + 16 * j * 256 + ((c ^ r_l) << 4)) = v;
    }
    // rows 16 j .. 16 j + 15 of the wave's block are complete (this wave alone wrote them)
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int row = 16 * j + 4 * it + g;
      const u4v v = *reinterpret_cast<const u4v*>(rbase + (16 * j + 4 * it) * 256 + ((c16 ^ (row & 15)) << 4));
      const int grow = m0 + wm + row;
      if (grow < p.M && col < p.N) *reinterpret_cast<u4v*>(p.y + (size_t)grow * p.N + col) = v;
    }
  }
}

// Sum of the split-K partial tiles of awq_gemm_dense_kernel, parts added in index order.  One
// workgroup takes eight accumulator tiles (one i, all j) of one output tile.
__global__ __launch_bounds__(256) void awq_gemm_dense_reduce_kernel(const DenseGemmParams p) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int tl = blockIdx.x >> 3, i = blockIdx.x & 7;
  const int nid = p.dp_tiles + tl;
  const int gsize = PF_GROUP_M * p.nt;
  const int first_m = (nid / gsize) * PF_GROUP_M;
  const int gm = min(p.mt - first_m, PF_GROUP_M);
  const int mt_i = first_m + (nid % gsize) % gm;
  const int nt_i = (nid % gsize) / gm;
  const int m0 = mt_i * 256, n0 = nt_i * 256;
  const int wm = (wave >> 1) * 128, wn = (wave & 1) * 128;
  const float* tile_base = p.sk_part + (size_t)tl * p.sk_split * PF_SK_SLOT_FLOATS;
  f4 v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = f4{0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < p.sk_split; ++s) {
    f4 t[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      t[j] = *reinterpret_cast<const f4*>(tile_base + (size_t)s * PF_SK_SLOT_FLOATS + ((size_t)(i * 8 + j) * 256 + tid) * 4);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] += t[j];
  }
  const int col = n0 + wn + 16 * i + 4 * (lane >> 4);
  if (col >= p.N) return;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int row = m0 + wm + 16 * j + (lane & 15);
    if (row >= p.M) continue;
    const h4 o = {(half_t)v[j][0], (half_t)v[j][1], (half_t)v[j][2], (half_t)v[j][3]};
    *reinterpret_cast<h4*>(p.y + (size_t)row * p.N + col) = o;
  }
}

}  // namespace awqmi
