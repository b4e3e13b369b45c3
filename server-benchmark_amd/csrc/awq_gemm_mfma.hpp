// Prefill AWQ GEMM (M > 16): Y[M,N] = X[M,K] @ dequant(W) on fp16 MFMA, fp32 accumulate.
//
// Workgroup tile 256 x 256 x 64, four waves in a 2 x 2 arrangement, each wave a 128 x 128
// block of 4 x 4 v_mfma_f32_32x32x16_f16 accumulators (256 accumulator registers, one wave
// per SIMD).  Both operands sit in LDS k-contiguous ([row][64 halves], swizzled, see below):
//   * X tile: 16-byte buffer loads -> registers -> 16-byte LDS stores;
//   * W tile: each thread takes 8 rows x 1 packed word (32 threads side by side read 128
//     contiguous bytes of a row), dequantises its 8 x 8 block to exact fp16 (w - z) * s with
//     the byte-pair trick (one perm + two and-or per four weights, then packed subtract and
//     packed multiply), and stores one 16-byte k-run per output column.
//
// Pipeline per k-tile (64 MFMAs per wave = four phases of 16): while tile t is multiplied
// out of LDS buffer t & 1, tile t + 1 goes from registers into the other buffer (X stores in
// phase 1, W dequantisation spread over phases 1-3, each interleaved between the MFMAs) and
// tile t + 2 is fetched from global memory into the freed registers.  The workgroup barrier
// sits between phase 3 and phase 4: phase 4 multiplies fragments that are already in
// registers, so behind the barrier it overlaps the first fragment reads of tile t + 1.
// Global addresses are buffer loads with a loop-invariant lane offset and a scalar offset
// that advances per tile, so the loop carries no vector address arithmetic.
//
// Workgroup ids are spread over the eight XCDs in contiguous ranges and walked in
// 8-row-tile groups so that the 32 workgroups resident on one XCD share X and W tiles
// through that XCD's L2.
//
// The weights are the MFMA's A operand and the activations its B operand: a lane's results of a
// tile are then 8-byte runs of an output row, which are gathered through LDS into 16 bytes per
// lane and stored as whole row pieces.
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
  int ldw;        // words between consecutive rows of qweight (NW, or more when the rows are padded)
  int gshift;     // log2(G) when G is a power of two (kernel instantiation POW2G)
  int mt, nt;     // tile counts
  int total;      // mt * nt
  int per_xcd;    // ceil(dp_tiles / 8)
  // Work split.  Tiles [0, dp_tiles) run one workgroup per tile over all of K (launch ids
  // [0, 8 * per_xcd)).  The remaining sk_tiles tiles (a last round that would leave most CUs
  // idle) are split in K over sk_split workgroups each (launch ids from 8 * per_xcd on,
  // tile-major) and leave fp32 partial tiles in the workspace; a second, short kernel on the
  // same stream sums them in part order and writes fp16 (a single finishing workgroup per
  // tile would have to pull sk_split x 256 KiB by itself, which took longer than the GEMM).
  int dp_tiles, sk_tiles, sk_split;
  float* sk_part;   // [sk_tiles][sk_split][256 * 256] fp32
  // Expert-grouped launch (kernel instantiation GROUPED): workgroup (blk, column tile); blk is
  // a block of BM sorted slots of one expert (moe_align with tile_m = BM).
  const int* sorted_ids;
  const int* expert_ids;
  const int* n_post_pad;
  const float* topk_w;      // optional per-slot output weight
  int n_slots;
  int a_row_div;            // X row of a slot = slot / a_row_div
  long long w_stride, s_stride, z_stride;   // elements per expert
};

// Tile order: groups of PF_GROUP_M row tiles walk the column tiles together, so that the 32
// tiles an XCD runs at a time share a few X and W slabs through its L2 (2, 4, 8 and 16 measured
// the same within noise: the re-reads that remain are served by the memory-side cache).
constexpr int PF_GROUP_M = 8;
constexpr int PF_SK_SLOT_FLOATS = 256 * 256;

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

__device__ __forceinline__ __amdgpu_buffer_rsrc_t pf_rsrc(const void* base, size_t bytes) {
  const uint32_t n = bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : (uint32_t)bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)n, 0x00020000);
}

// POW2G: G is a power of two (group index by shift, any G >= 8); otherwise G % 64 == 0 and
// a k-tile lies inside one group (group index on the scalar unit).
//
// MI = 32-row MFMA tiles per wave along M: 4 gives the 256-row workgroup tile; 3, 2 and 1
// give 192-, 128- and 64-row tiles (each wave 32 MI x 128) for launches of at most that many
// rows, which would leave part of a 256-row tile multiplying padding.
//
// NWV = waves per workgroup.  4: one wave per SIMD, each 32 MI x 128 (the prefill
// configuration: 256 accumulator registers per wave leave no room for a second wave).
// 8: two waves per SIMD, each 32 MI x 64, for MI <= 2: with half the accumulators two waves
// fit, and the waits of one (fragment reads, the barrier, operand loads) are covered by the
// MFMAs of the other -- the small tiles spend most of a k-tile in such waits otherwise.
// GROUPED: the expert-grouped form for MoE batches with many rows per expert: X rows are
// gathered through the sorted slot list, the weight triple is the block's expert's, output
// rows go to their slot rows (times the routing weight when given).
template <bool POW2G, int MI = 4, int NWV = 4, bool GROUPED = false>
__global__ __launch_bounds__(64 * NWV, NWV / 4) void awq_gemm_mfma_kernel(const MfmaGemmParams p) {
  constexpr int BM = 64 * MI;            // workgroup tile rows
  constexpr int NTH = 64 * NWV;          // threads
  constexpr int NJ = 16 / NWV;           // 32-column MFMA tiles per wave (4 or 2)
  constexpr int ARP = NTH / 8;           // X rows moved per pass of the workgroup
  constexpr int AL = BM / ARP;           // 16-byte X loads per thread and k-tile
  constexpr int RW = 2048 / NTH;         // rows of one word column a thread dequantises (8 or 4)
  extern __shared__ __align__(16) unsigned char smem_raw[];
  unsigned char* const As = smem_raw;                        // [2][256][128 B]
  unsigned char* const Bs = smem_raw + 2 * PF_TILE_BYTES;    // [2][256][128 B]

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int id = blockIdx.x;
  const int KT = p.K / PF_BK;
  int nid = 0, kb = 0, ke = KT, part = -1;
  __shared__ int s_sid[GROUPED ? 64 * MI : 1];
  __shared__ float s_tw[GROUPED ? 64 * MI : 1];
  const uint32_t* qw_base = p.qw;
  const uint32_t* qz_base = p.qz;
  const half_t* sc_base = p.sc;
  int g_m0 = 0, g_n0 = 0;
  if (GROUPED) {
    const int blk = id / p.nt;
    if (blk * BM >= *p.n_post_pad) return;
    const int e = p.expert_ids[blk];
    qw_base += (size_t)e * p.w_stride;
    qz_base += (size_t)e * p.z_stride;
    sc_base += (size_t)e * p.s_stride;
    g_m0 = blk * BM;
    g_n0 = (id % p.nt) * PF_BN;
    for (int r = tid; r < BM; r += NTH) {
      const int sid = p.sorted_ids[g_m0 + r];
      s_sid[r] = sid;
      s_tw[r] = (sid < p.n_slots && p.topk_w) ? p.topk_w[sid] : 1.f;
    }
    __syncthreads();
  } else if (id < 8 * p.per_xcd) {
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
  const int m0 = GROUPED ? g_m0 : mt_i * BM, n0 = GROUPED ? g_n0 : nt_i * PF_BN;
  const int wm = (wave / (NWV / 2)) * (32 * MI), wn = (wave % (NWV / 2)) * (32 * NJ);

  const __amdgpu_buffer_rsrc_t rx = pf_rsrc(p.x, (size_t)p.M * p.K * 2);
  const __amdgpu_buffer_rsrc_t rw = pf_rsrc(qw_base, (size_t)p.K * p.ldw * 4);
  const __amdgpu_buffer_rsrc_t rz = pf_rsrc(qz_base, (size_t)(p.K / p.G) * p.NW * 4);
  const __amdgpu_buffer_rsrc_t rs = pf_rsrc(sc_base, (size_t)(p.K / p.G) * p.N * 2);

  // ---- global -> LDS roles -------------------------------------------------------------
  // X tile: thread (a_row + 32 i, a_seg) moves 16 bytes; rows past M re-read row M - 1 (their
  // outputs are never stored), so no load sits behind a branch.
  const int a_row = tid >> 3, a_seg = tid & 7;
  uint32_t a_off[AL];
  int a_dst[AL];
#pragma unroll
  for (int i = 0; i < AL; ++i) {
    const int r = a_row + ARP * i;
    int gr;
    if (GROUPED) {
      const int sid = s_sid[r];
      gr = sid < p.n_slots ? sid / p.a_row_div : 0;     // pad rows read row 0, never stored
    } else {
      gr = min(m0 + r, p.M - 1);
    }
    a_off[i] = (uint32_t)(((size_t)gr * p.K + 8 * a_seg) * 2);
    a_dst[i] = r * PF_ROW_BYTES + ((a_seg ^ pf_swz(r)) << 4);
  }
  // W tile: thread (kk, wcl) takes rows RW kk .. RW kk + RW - 1 of word column wcl
  const int kk = tid >> 5, wcl = tid & 31;
  int wcg = n0 / 8 + wcl;
  if (wcg >= p.NW) wcg = 0;                      // columns never stored; keep loads in bounds
  const uint32_t w_off = (uint32_t)(((size_t)RW * kk * p.ldw + wcg) * 4);
  const uint32_t row_w = (uint32_t)p.ldw * 4;    // bytes between qweight rows
  const uint32_t row_b = (uint32_t)p.NW * 4;     // bytes between qzeros rows
  const int b_t = (RW == 8 ? kk : (kk >> 1)) ^ (wcl & 7);   // physical 16-byte slot of column c: b_t ^ c
  const int b_half = RW == 8 ? 0 : (kk & 1) * 8;            // 8-byte half of the slot (RW = 4)
  const int b_base = wcl * 8 * PF_ROW_BYTES;

  // ---- LDS -> fragment roles -----------------------------------------------------------
  // lane (i = lane % 32, hh = lane / 32) reads row base + i, logical slot 2 ks + hh; with
  // u = hh ^ swz(i) the physical slot is u ^ (2 ks) ^ (4 (tile & 1)): four lane offsets
  const int fi = lane & 31, fh = lane >> 5;
  const int fu = fh ^ pf_swz(fi);
  int f_off[4], fa_off[4];
  // a wave whose first X row is an odd multiple of 32 (192-row tile, second wave row) sees
  // the swizzle of its rows flipped in bit 2
  const int fua = fu ^ (((wm >> 5) & 1) << 2);
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    f_off[c] = fi * PF_ROW_BYTES + ((fu ^ (2 * c)) << 4);
    fa_off[c] = fi * PF_ROW_BYTES + ((fua ^ (2 * c)) << 4);
  }

  f16v acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  NibbleMasks nm;
  nm.init();
  u4v areg[AL];         // X tile in flight
  uint32_t wreg[2][RW]; // two W tiles in flight (parity of the k-tile)
  uint32_t zreg[2];
  u4v sreg[2];
  auto gload_a = [&](int kt) {
    const int so = kt * (PF_BK * 2);
#pragma unroll
    for (int i = 0; i < AL; ++i) areg[i] = __builtin_amdgcn_raw_buffer_load_b128(rx, a_off[i], so, 0);
  };
  auto gload_w = [&](int kt, int set) {
    const uint32_t so = (uint32_t)kt * PF_BK * row_w;
#pragma unroll
    for (int i = 0; i < RW; ++i)
      wreg[set][i] = __builtin_amdgcn_raw_buffer_load_b32(rw, w_off, so + i * row_w, 0);
    if (POW2G) {
      const uint32_t g = (uint32_t)(kt * PF_BK + RW * kk) >> p.gshift;
      zreg[set] = __builtin_amdgcn_raw_buffer_load_b32(rz, g * row_b + wcg * 4, 0, 0);
      sreg[set] = __builtin_amdgcn_raw_buffer_load_b128(rs, (g * (uint32_t)p.N + 8 * wcg) * 2, 0, 0);
    } else {
      const uint32_t g = (uint32_t)(kt * PF_BK) / (uint32_t)p.G;
      zreg[set] = __builtin_amdgcn_raw_buffer_load_b32(rz, wcg * 4, g * row_b, 0);
      sreg[set] = __builtin_amdgcn_raw_buffer_load_b128(rs, wcg * 16, g * (uint32_t)p.N * 2, 0);
    }
  };
  auto store_a = [&](int buf) {
    unsigned char* as = As + buf * PF_TILE_BYTES;
#pragma unroll
    for (int i = 0; i < AL; ++i) *reinterpret_cast<u4v*>(as + a_dst[i]) = areg[i];
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
    uint32_t lo[RW / 2], hi[RW / 2];
#pragma unroll
    for (int rp = 0; rp < RW / 2; ++rp) {
      const uint32_t t = byte_pair<B>(wreg[set][2 * rp + 1], wreg[set][2 * rp]);
      lo[rp] = pk_mul(pk_sub((t & nm.lo) | MAGIC_LO, zl), sl);
      hi[rp] = pk_mul(pk_sub((t & nm.hi) | MAGIC_HI, zh), sh);
    }
    unsigned char* dl = bs + b_base + cl * PF_ROW_BYTES + ((b_t ^ cl) << 4) + b_half;
    unsigned char* dh = bs + b_base + ch * PF_ROW_BYTES + ((b_t ^ ch) << 4) + b_half;
    if constexpr (RW == 8) {
      *reinterpret_cast<u4v*>(dl) = u4v{lo[0], lo[1], lo[2], lo[3]};
      *reinterpret_cast<u4v*>(dh) = u4v{hi[0], hi[1], hi[2], hi[3]};
    } else {
      *reinterpret_cast<u2v*>(dl) = u2v{lo[0], lo[1]};
      *reinterpret_cast<u2v*>(dh) = u2v{hi[0], hi[1]};
    }
  };

  h8 af[2][MI], bf[2][NJ];  // fragments of two 16-wide k-steps
  auto load_frags = [&](int buf, int ks, int fs) {
    const unsigned char* as = As + buf * PF_TILE_BYTES + wm * PF_ROW_BYTES;
    const unsigned char* bs = Bs + buf * PF_TILE_BYTES + wn * PF_ROW_BYTES;
#pragma unroll
    for (int i = 0; i < MI; ++i)
      af[fs][i] = *reinterpret_cast<const h8*>(as + 32 * i * PF_ROW_BYTES + fa_off[ks ^ (2 * (i & 1))]);
#pragma unroll
    for (int j = 0; j < NJ; ++j)
      bf[fs][j] = *reinterpret_cast<const h8*>(bs + 32 * j * PF_ROW_BYTES + f_off[ks ^ (2 * (j & 1))]);
  };
  // 2 x 2 blocks of accumulator tiles, block rows walked forth and back, so that one operand
  // changes from one MFMA to the next: the order that sustains the most under the power limit
  auto mfma_step = [&](int fs) {
    // the weights are the A operand and the activations the B operand, so that a lane's values of
    // a tile are runs of four consecutive output columns of one row
    auto one = [&](int i, int j) {
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[fs][j], af[fs][i], acc[i][j], 0, 0, 0);
    };
#pragma unroll
    for (int bi = 0; bi < (MI + 1) / 2; ++bi) {
      const int i = 2 * bi;
#pragma unroll
      for (int bb = 0; bb < (NJ + 1) / 2; ++bb) {
        const int j = (bi & 1) ? 2 * ((NJ + 1) / 2 - 1 - bb) : 2 * bb;
        one(i, j);
        if (i + 1 < MI) one(i + 1, j);
        if (j + 1 < NJ) {
          if (i + 1 < MI) one(i + 1, j + 1);
          one(i, j + 1);
        }
      }
    }
  };

  // Interleave recipe for one phase of 16 MFMAs: an MFMA occupies the matrix pipe for eight
  // passes, during which the wave can issue about seven other instructions, so the other
  // work of the phase is dealt out evenly between the MFMAs: per MFMA pair `valu` VALU ops,
  // `dsr` LDS reads, `dsw` LDS writes and `vm` buffer loads.
  constexpr int NPAIR = MI * NJ / 2 > 0 ? MI * NJ / 2 : 1;   // MFMA pairs per phase
  auto phase_schedule = [&](auto VALU, auto DSR, auto DSW, auto VM) {
    constexpr int valu = decltype(VALU)::value, dsr = decltype(DSR)::value;
    constexpr int dsw = decltype(DSW)::value, vm = decltype(VM)::value;
#pragma unroll
    for (int i = 0; i < NPAIR; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (dsr) __builtin_amdgcn_sched_group_barrier(0x100, dsr, 0);
      if (vm) __builtin_amdgcn_sched_group_barrier(0x020, vm, 0);
      if (valu) __builtin_amdgcn_sched_group_barrier(0x002, (valu + 1) / 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (dsw) __builtin_amdgcn_sched_group_barrier(0x200, dsw, 0);
      if (valu / 2) __builtin_amdgcn_sched_group_barrier(0x002, valu / 2, 0);
    }
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  // per-MFMA-pair shares of the phase's other work (smaller tiles have fewer MFMAs per phase
  // for the same W work; with eight waves a thread has half the W and X work)
  constexpr auto cdiv = [](int a, int b) { return (a + b - 1) / b; };
  using VA = std::integral_constant<int, cdiv(6 * RW, NPAIR)>;        // dequant VALU of one byte, phases 1 and 2
  using VB = std::integral_constant<int, cdiv(12 * RW, NPAIR)>;       // two bytes, phase 3
  using DR = std::integral_constant<int, cdiv(MI + NJ, NPAIR)>;       // fragment reads
  using DW1 = std::integral_constant<int, (MI == 4 && NWV == 4) ? 1 : cdiv(AL + 2, NPAIR)>;  // X tile + byte 0
  using DW2 = std::integral_constant<int, cdiv(2, NPAIR)>;
  using DW3 = std::integral_constant<int, cdiv(4, NPAIR)>;
  using VM1 = std::integral_constant<int, cdiv(RW + 2, NPAIR)>;       // W / zero / scale loads, phase 1
  using VM2 = std::integral_constant<int, cdiv(AL, NPAIR)>;           // X loads, phase 2

  // One k-tile, PAR = kt & 1.  On entry: LDS buffer PAR holds tile kt and fragment set 0 its
  // first k-step; areg and W set PAR^1 hold tile kt + 1; W set PAR is free.  Tiles past the
  // end re-read the last tile and are never used.
  auto body = [&](int kt, auto PTAG) {
    constexpr int PAR = decltype(PTAG)::value;
    const int kt2 = min(kt + 2, ke - 1);

    // phase 1: X(kt+1) -> LDS, W(kt+2) -> registers, byte 0 of W(kt+1)
    mfma_step(0);
    load_frags(PAR, 1, 1);
    store_a(PAR ^ 1);
    gload_w(kt2, PAR);
    dq_byte(PAR ^ 1, PAR ^ 1, I0{});
    phase_schedule(VA{}, DR{}, DW1{}, VM1{});
    __builtin_amdgcn_sched_barrier(0);

    // phase 2: X(kt+2) -> registers, byte 1 of W(kt+1)
    mfma_step(1);
    load_frags(PAR, 2, 0);
    gload_a(kt2);
    dq_byte(PAR ^ 1, PAR ^ 1, I1{});
    phase_schedule(VA{}, DR{}, DW2{}, VM2{});
    __builtin_amdgcn_sched_barrier(0);

    // phase 3: bytes 2 and 3 of W(kt+1)
    mfma_step(0);
    load_frags(PAR, 3, 1);
    dq_byte(PAR ^ 1, PAR ^ 1, I2{});
    dq_byte(PAR ^ 1, PAR ^ 1, I3{});
    phase_schedule(VB{}, DR{}, DW3{}, I0{});
    __builtin_amdgcn_sched_barrier(0);

    // every LDS write of tile kt + 1 is out and every read of tile kt has returned
    __syncthreads();

    // phase 4: last k-step from registers, first fragments of tile kt + 1
    mfma_step(1);
    load_frags(PAR ^ 1, 0, 0);
    phase_schedule(I0{}, DR{}, I0{}, I0{});
    __builtin_amdgcn_sched_barrier(0);
  };

  // prologue: tile 0 into LDS buffer 0, tile 1 into registers
  gload_a(kb);
  gload_w(kb, 0);
  store_a(0);
  dq_byte(0, 0, I0{});
  dq_byte(0, 0, I1{});
  dq_byte(0, 0, I2{});
  dq_byte(0, 0, I3{});
  gload_a(min(kb + 1, ke - 1));
  gload_w(min(kb + 1, ke - 1), 1);
  __syncthreads();
  load_frags(0, 0, 0);
  __builtin_amdgcn_sched_barrier(0);
  int kt = kb;
  for (; kt + 1 < ke; kt += 2) {
    body(kt, I0{});
    body(kt + 1, I1{});
  }
  if (kt < ke) body(kt, I0{});

  // ---- split-K tiles: fp32 partial to the workspace ------------------------------------
  if (part >= 0) {
    const int tl = nid - p.dp_tiles;
    float* tile_base = p.sk_part + (size_t)tl * p.sk_split * PF_SK_SLOT_FLOATS;
    float* mine = tile_base + (size_t)part * PF_SK_SLOT_FLOATS;
    // layout [group of four accumulator registers][thread]: coalesced 16-byte accesses
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int r = 0; r < 16; r += 4) {
          const int q = ((i * NJ + j) * 16 + r) >> 2;
          const f4 v = {acc[i][j][r], acc[i][j][r + 1], acc[i][j][r + 2], acc[i][j][r + 3]};
          *reinterpret_cast<f4*>(mine + ((size_t)q * NTH + tid) * 4) = v;
        }
    // summed and written out by awq_gemm_mfma_reduce_kernel, launched behind this kernel
    return;
  }

  // Output.  acc[i][j][r] is row wm + 32 i + lane % 32, column wn + 32 j + 8 (r / 4) + 4 (lane / 32)
  // + r % 4 of the workgroup tile: a lane holds 8-byte runs of a row.  They go through the wave's own
  // piece of LDS (every wave has read its last fragments: the barrier) and leave as 16 bytes per
  // lane, 64 NJ contiguous bytes per row -- stored directly, every instruction would carry 32
  // separate 8-byte pieces.  LDS row = 64 NJ bytes, 16-byte chunk c of row r kept at chunk
  // c ^ (r % 16) (NJ = 4) or c ^ ((r / 2) % 8) (NJ = 2): reads are conflict-free, the writes of rows
  // r and r + 16 share banks (two passes).
  __syncthreads();
  constexpr int RB = 64 * NJ;                         // bytes per staged row
  constexpr int CPR = RB / 16;                        // 16-byte chunks per row (16 or 8)
  constexpr int RPI = 64 / CPR;                       // rows per read instruction (4 or 8)
  unsigned char* const st = smem_raw + wave * (32 * MI * RB);
  const int wr = lane & 31, wh = lane >> 5;
  const int wswz = NJ == 4 ? (wr & 15) : ((wr >> 1) & 7);
  const int rc = lane % CPR, rr0 = lane / CPR;
  const int col = n0 + wn + 8 * rc;                   // N % 8 == 0: a chunk is all inside or all outside
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    float tw = 1.f;
    if (GROUPED) tw = s_tw[wm + 32 * i + wr];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const h4 v = {(half_t)(acc[i][j][4 * rg] * tw), (half_t)(acc[i][j][4 * rg + 1] * tw),
                      (half_t)(acc[i][j][4 * rg + 2] * tw), (half_t)(acc[i][j][4 * rg + 3] * tw)};
        const int c = 4 * j + rg;
        *reinterpret_cast<h4*>(st + (32 * i + wr) * RB + ((c ^ wswz) << 4) + 8 * wh) = v;
      }
    // rows 32 i .. 32 i + 31 of the wave's block are complete (this wave alone wrote them)
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) {
      const int lr = 32 * i + RPI * it + rr0;
      const int rswz = NJ == 4 ? (lr & 15) : ((lr >> 1) & 7);
      const u4v v = *reinterpret_cast<const u4v*>(st + lr * RB + ((rc ^ rswz) << 4));
      if (col >= p.N) continue;
      if (GROUPED) {
        const int sid = s_sid[wm + lr];
        if (sid < p.n_slots) *reinterpret_cast<u4v*>(p.y + (size_t)sid * p.N + col) = v;
      } else {
        const int row = m0 + wm + lr;
        if (row < p.M) *reinterpret_cast<u4v*>(p.y + (size_t)row * p.N + col) = v;
      }
    }
  }
}

// Sum of the split-K partial tiles.  Partial layout per (tile, part): [q][thread] groups of
// four floats, q = (i * NJ + j) * 4 + r / 4 over the MI x NJ accumulator tiles of the producing
// thread (same thread count and wave arrangement as the producer).  One workgroup takes four
// q of one tile; parts are added in index order.
template <int MI, int NWV = 4>
__global__ __launch_bounds__(64 * NWV) void awq_gemm_mfma_reduce_kernel(const MfmaGemmParams p) {
  constexpr int QPW = 4;
  constexpr int NJ = 16 / NWV, NTH = 64 * NWV;
  constexpr int QT = 4 * MI * NJ;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int tl = blockIdx.x / (QT / QPW);
  const int q0 = (blockIdx.x % (QT / QPW)) * QPW;
  const int nid = p.dp_tiles + tl;
  const int gsize = PF_GROUP_M * p.nt;
  const int first_m = (nid / gsize) * PF_GROUP_M;
  const int gm = min(p.mt - first_m, PF_GROUP_M);
  const int mt_i = first_m + (nid % gsize) % gm;
  const int nt_i = (nid % gsize) / gm;
  const int m0 = mt_i * (64 * MI), n0 = nt_i * PF_BN;
  const int wm = (wave / (NWV / 2)) * (32 * MI), wn = (wave % (NWV / 2)) * (32 * NJ);
  const int row_l = lane & 31;
  const float* tile_base = p.sk_part + (size_t)tl * p.sk_split * PF_SK_SLOT_FLOATS;
  f4 v[QPW];
#pragma unroll
  for (int u = 0; u < QPW; ++u) v[u] = f4{0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < p.sk_split; ++s) {
    f4 t[QPW];
#pragma unroll
    for (int u = 0; u < QPW; ++u)
      t[u] = *reinterpret_cast<const f4*>(tile_base + (size_t)s * PF_SK_SLOT_FLOATS +
                                          ((size_t)(q0 + u) * NTH + tid) * 4);
#pragma unroll
    for (int u = 0; u < QPW; ++u) v[u] += t[u];
  }
  // The four groups of a thread are columns 8 rg + 4 (lane / 32) + 0..3, rg = 0..3, of one row of one
  // 32 x 32 accumulator tile (see the producer's output comment; q0 is a multiple of four): lane l
  // and lane l ^ 32 hold the two interleaved halves of 32 consecutive columns.  They trade two groups
  // each, so that the lower lane stores columns 0..15 and the upper one columns 16..31 as 32 bytes.
  static_assert(QPW == 4, "one accumulator tile row per thread");
  const int ij = q0 >> 2;
  const bool upper = lane >= 32;
  u2v hv[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const h4 o = {(half_t)v[u][0], (half_t)v[u][1], (half_t)v[u][2], (half_t)v[u][3]};
    hv[u] = __builtin_bit_cast(u2v, o);
  }
  u2v got[2];
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const u2v give = upper ? hv[k] : hv[2 + k];
    got[k][0] = (uint32_t)__shfl_xor((int)give[0], 32, 64);
    got[k][1] = (uint32_t)__shfl_xor((int)give[1], 32, 64);
  }
  // lower lane: own 0, partner's 0, own 1, partner's 1; upper lane: partner's 2, own 2, partner's 3, own 3
  const u4v lo = upper ? u4v{got[0][0], got[0][1], hv[2][0], hv[2][1]} : u4v{hv[0][0], hv[0][1], got[0][0], got[0][1]};
  const u4v hi = upper ? u4v{got[1][0], got[1][1], hv[3][0], hv[3][1]} : u4v{hv[1][0], hv[1][1], got[1][0], got[1][1]};
  const int col = n0 + wn + 32 * (ij % NJ) + (upper ? 16 : 0);
  const int row = m0 + wm + 32 * (ij / NJ) + row_l;
  if (row < p.M) {        // N % 8 == 0: eight columns are all inside or all outside
    if (col < p.N) *reinterpret_cast<u4v*>(p.y + (size_t)row * p.N + col) = lo;
    if (col + 8 < p.N) *reinterpret_cast<u4v*>(p.y + (size_t)row * p.N + col + 8) = hi;
  }
}

}  // namespace awqmi
