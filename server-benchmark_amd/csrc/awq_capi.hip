// C ABI of libawq_mi355x.so: host-side validation and launch of the gfx950 kernels.
// Every entry point checks its arguments before touching the device, launches on the
// caller's stream and returns; nothing here allocates, synchronises or keeps state apart
// from the thread-local last HIP error and the one-time kernel attribute set-up.  Launch
// shapes assume the MI355X's 256 CUs in 8 XCDs.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <type_traits>

#include "../../include/awq_mi355x.h"
#include "../../include/awq_mi355x_dev.h"
#include "awq_dequant.hpp"
#include "awq_gemm_dense.hpp"
#include "awq_gemm_mfma.hpp"
#include "awq_gemv.hpp"
#include "awq_moe.hpp"
#include "awq_probes.hpp"

using namespace awqmi;

// Scratch of the allocation-free entry point (awqmi_gemm_f16_noalloc): split-K arrival counters
// (the first AWQMI_WS_COUNTER_BYTES) and fp32 partial tiles.  Every GPU the library runs on
// holds its own copy of this array at its own address until the process ends.  The name below
// is a host-side stand-in, not a device address: host code only ever uses the pointer that
// hipGetSymbolAddress returned for the current device (static_scratch_ptr).
static __device__ __align__(256) unsigned char scratch[AWQMI_STATIC_SCRATCH_BYTES];

namespace {

thread_local int t_last_hip_error = 0;
// which kernel family the last awqmi_gemm_* call on this thread launched (awqmi_dev_last_gemm_form)
thread_local int t_last_gemm_form = 0;
// time-stamp buffer of the call in progress (awqmi_dev_gemm_timeline_f16 only; null otherwise)
thread_local unsigned long long* t_trace = nullptr;

// Launch-rule variant of the call in progress on this thread: -1 (every default) for the whole
// public C ABI; the awqmi_dev_* entry points set it for the duration of their own call only, so
// no call can change what another call, on this thread or any other, launches.
thread_local int t_variant = -1;
struct VariantScope {
  int prev;
  explicit VariantScope(int v) : prev(t_variant) { t_variant = v; }
  ~VariantScope() { t_variant = prev; }
};

// Bits of the `variant` argument of the awqmi_dev_* entry points: each turns one launch choice
// off, or forces one, so that two forms can be compared and timed in one process.
enum : int {
  VAR_WPL1 = 1,               // one packed word per lane for every shape
  VAR_MOE_RING4 = 2,          // MoE launches with the dense kernel's register ring of four steps
  VAR_XCD_RUN_SHIFT = 2,      // bits 2..4 = v: force runs of 1 << (v - 1) blocks per XCD
  VAR_NO_PAIR_COLS = 64,      // never two column blocks per workgroup
  VAR_MFMA_FOUR_WAVES = 512,  // 64- / 128-row MFMA tiles with four waves instead of eight
  VAR_NO_FUSED_ACT = 1024,    // the one-call MoE block always runs the separate activation kernel
  VAR_MOE_TILE16 = 2048,      // the one-call MoE block always uses 16-row blocks
  VAR_NO_LDS_RING = 4096,     // every launch keeps the weight ring in registers
  VAR_ALIGN_ONE_WG = 16384,   // align always in one workgroup
  VAR_MOE_TILE_SHIFT = 16,    // bits 16..17 = v: the one-call MoE block uses 64 / 128 / 256-row blocks (v = 1 / 2 / 3)
  VAR_MID_M_SKINNY = 1 << 18, // awq_gemm with 17..64 rows: skinny passes wherever they can run
  VAR_MID_M_MFMA = 1 << 19,   // awq_gemm with 17..64 rows: the MFMA kernel wherever it can run
  VAR_MFMA_ROWS_SHIFT = 20,   // bits 20..22 = v: MFMA tiles of 64 v rows (v = 1..4) whatever M is
  VAR_NO_TAIL_STEP = 1 << 23, // dense skinny launches never share left-over chunks step by step
  VAR_NO_FOLDED_ROUTE = 1 << 24, // the one-call MoE block always routes in a launch of its own
  VAR_NO_DENSE = 1 << 25,        // awq_gemm never takes the dequantise-once form
  VAR_DENSE = 1 << 26,           // awq_gemm takes the dequantise-once form from 257 rows on (workspace permitting)
  VAR_MOE_T32_WIDE = 1 << 27,    // 32-row MoE blocks in the two-words-per-lane form (one workgroup per CU)
};
inline bool variant_on(int bit) {
  return t_variant >= 0 && (t_variant & bit);
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Device address of `scratch` on the current GPU, looked up once per device.
constexpr int MAX_DEVICES = 64;
std::atomic<void*> g_scratch_ptr[MAX_DEVICES];
int static_scratch_ptr(void** out, bool* first_use) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { t_last_hip_error = (int)e; return AWQMI_LAUNCH_FAILED; }
  if (dev < 0 || dev >= MAX_DEVICES) return AWQMI_BAD_ARGUMENT;
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  *first_use = ptr == nullptr;
  if (!ptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) { t_last_hip_error = (int)e; return AWQMI_LAUNCH_FAILED; }
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return AWQMI_OK;
}

inline int launch_status() {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    t_last_hip_error = (int)e;
    return AWQMI_LAUNCH_FAILED;
  }
  return AWQMI_OK;
}

inline int norm_group(int K, int group) { return group <= 0 ? K : group; }

int check_awq_shape(int K, int N, int G) {
  if (K <= 0 || N <= 0 || G <= 0) return AWQMI_BAD_SHAPE;
  if (N % 8 != 0 || K % G != 0) return AWQMI_BAD_SHAPE;
  return AWQMI_OK;
}

// tiled skinny kernel covers: K a multiple of 128 and G in {32, 64, 128 * i}
inline bool gemv_tiled_ok(int K, int G) { return K % 128 == 0 && (G == 32 || G == 64 || G % 128 == 0); }

inline int gemv_wpl(int N) {
  return (variant_on(VAR_WPL1) || (N / 8) % 2 != 0) ? 1 : 2;
}

// Split-K choice.  The skinny kernel runs one workgroup (one wave per SIMD, 16 KiB of loads
// in flight per wave) per CU and that saturates HBM; a second round of workgroups costs a
// drain and refill of the memory pipeline.  So: split K just far enough that the launch is
// one round of at most 256 workgroups, preferring a split whose 4 x split wave ranges
// divide the 128-row chunks evenly, never below one chunk per wave.
// Left-over chunks shared one 32-row step per wave (the kernel's TAIL form): every wave gets
// nchunks / parts whole chunks, and the L chunks left are 4 L steps for the first 4 L waves.
// Used for the split already chosen (down_proj of the 72B shapes, 231 chunks over 32 waves:
// 29 steps on the busiest wave instead of 32, 1.2 - 1.9 us of 30 - 36); letting the split
// choice count on it picked five parts for a 8192 x 10240 layer, which measured 4 % slower
// than six without tail steps.
inline bool gemv_tail_ok(int nchunks, int split) {
  const int parts = 4 * split, base = nchunks / parts, left = nchunks - base * parts;
  return base >= 1 && left > 0 && 4 * left <= parts;
}

// dense launches of up to 16 rows with two words per lane and G = 128 can take the TAIL form
inline bool gemv_tail_shape(int M, int N, int G) {
  return M <= 16 && G == 128 && gemv_wpl(N) == 2 && !variant_on(VAR_NO_TAIL_STEP);
}

// dense: a dense launch (blocks_z = 1), which takes the TAIL form where its shape and the split
// allow; the busiest wave is then counted in 32-row steps (on 21 layer shapes of eight model
// sizes at 1 and 16 rows, every split forced in turn: the pick is the best split or within 2 % of
// it on all 42 points; counting whole chunks was 6 - 8 % behind on the 5120-wide layers).
int pick_split_k(int rows, int K, int N, int G, long long blocks_z, bool dense = false) {
  const bool tail_form = dense && blocks_z == 1 && gemv_tail_shape(rows, N, G);
  const int nchunks = K / 128;
  const long long ncb = (N + 255) / 256;
  const long long wg = ncb * blocks_z;            // workgroups at split 1
  long long smax = 256 / wg;                      // largest split that stays within one round
  if (smax > nchunks / 4) smax = nchunks / 4;
  if (smax > AWQMI_MAX_SPLIT_K) smax = AWQMI_MAX_SPLIT_K;
  if (smax < 1) smax = 1;
  // among splits >= smax / 2 take the one with the best balance (work of the busiest wave)
  long long best = smax;
  double best_cost = 1e300;
  for (long long s = smax; s >= 1 && 2 * s >= smax; --s) {
    const long long parts = 4 * s;
    const double fill = (double)(wg * s) / 256.0;            // fraction of the round used
    double cost;
    if (tail_form) {
      const long long steps = gemv_tail_ok(nchunks, (int)s) ? 4 * (nchunks / parts) + 1
                                                            : 4 * ((nchunks + parts - 1) / parts);
      // the finishing workgroup reads the parts eight at a time: every further batch is one more
      // dependent trip to memory, over partial tiles that grow with the split
      const double batches = (double)((s + 7) / 8 - 1);
      cost = (double)steps * (double)parts / (4.0 * nchunks) / (0.4 + 0.6 * fill) * (1.0 + 0.15 * batches * batches);
      if (cost <= best_cost + 1e-9) { best_cost = cost; best = s; }     // ties go to the smaller split
      continue;
    }
    const long long busiest = (nchunks + parts - 1) / parts;
    cost = (double)busiest * (double)parts / (double)nchunks / (0.5 + 0.5 * fill);
    if (cost < best_cost - 1e-9) { best_cost = cost; best = s; }
  }
  return (int)best;
}

inline size_t gemv_partial_bytes(int N, int split, long long blocks_z, int tile_m = 16) {
  if (split <= 1) return 0;
  const size_t npad = ((size_t)N + 255) / 256 * 256;
  return (size_t)split * (size_t)blocks_z * tile_m * npad * sizeof(float);
}

template <int WPL, int MB, bool MOE, int RING = 4, int KW = 4, bool ACT = false, bool LDSQ = false>
void launch_gemv(const GemvParams& p, dim3 grid, hipStream_t st) {
  if (p.G == 32) hipLaunchKernelGGL((awq_gemv_kernel<WPL, 0, MB, MOE, RING, KW, ACT, LDSQ>), grid, dim3(256), 0, st, p);
  else if (p.G == 64) hipLaunchKernelGGL((awq_gemv_kernel<WPL, 1, MB, MOE, RING, KW, ACT, LDSQ>), grid, dim3(256), 0, st, p);
  else if (p.G == 128) hipLaunchKernelGGL((awq_gemv_kernel<WPL, 2, MB, MOE, RING, KW, ACT, LDSQ>), grid, dim3(256), 0, st, p);
  else hipLaunchKernelGGL((awq_gemv_kernel<WPL, 3, MB, MOE, RING, KW, ACT, LDSQ>), grid, dim3(256), 0, st, p);
}

// rows the skinny kernel takes in one awq_gemm call (passes of up to 32 rows)
constexpr int SKINNY_MAX_M = 64;

// Up to 32 rows one skinny pass (two row blocks share every unpacked operand); from 33 rows on
// the 64-row MFMA tile beats two skinny passes on every layer shape measured (nine shapes from
// 2048 x 5120 to 8192 x 59136, weights read from HBM: equal at worst, up to 2 x on small layers).
inline bool skinny_rows(int M, int /*N*/) { return M <= 32; }

// Work split of the MFMA kernel: whole rounds of 256 tiles run one workgroup per tile; a
// last round of fewer than 129 tiles (and any launch that small) is split in K over
// floor(256 / tiles) workgroups per tile (at most 8, at least 4 k-tiles each).
// The MFMA kernel addresses X through 32-bit buffer offsets: calls with more than 4 GiB of
// activations run as consecutive row slabs (multiples of 256 rows).
inline int mfma_slab_rows(int M, int K) {
  const long long fit = ((1LL << 32) - 1) / ((long long)K * 2);
  const long long rows = fit / 256 * 256;
  return rows <= 0 ? 0 : (int)(rows < M ? rows : M);
}

struct MfmaPlan { int dp_tiles, sk_tiles, sk_split; size_t part_bytes; };
MfmaPlan plan_mfma(int M, int K, int N, int bm) {
  const int mt = (M + bm - 1) / bm, nt = (N + PF_BN - 1) / PF_BN;
  const int tiles = mt * nt, KT = K / PF_BK;
  MfmaPlan pl{tiles, 0, 1, 0};
  const int rem = tiles % 256;
  if (rem == 0) return pl;
  int c = 256 / rem;
  if (c > 8) c = 8;
  while (c > 1 && KT / c < 4) --c;
  if (c < 2) return pl;
  pl.dp_tiles = tiles - rem;
  pl.sk_tiles = rem;
  pl.sk_split = c;
  pl.part_bytes = (size_t)rem * c * PF_SK_SLOT_FLOATS * sizeof(float);
  return pl;
}

// Dequantise-once form (awq_gemm_dense.hpp): the weights go through awq_dequant_panel_kernel into
// an fp16 panel in the workspace, then awq_gemm_dense_kernel.  Under sustained load on the 72B
// layer shapes (fused kernel against panel pass + dense kernel, timed in turn): 512 rows 0.70,
// 1024 rows 0.79 - 0.90, 2048 rows 1.01 - 1.03, 3072 rows 1.01 - 1.07, 4096 rows 1.08, 8192 rows
// 1.11 - 1.16 of the fused kernel's rate; so it is taken from 2048 rows on.  Between 2048 and
// 4095 rows only when the 256 x 256 tiles make at least three quarters of a round of workgroups:
// with fewer the fused kernel's smaller row tiles fill the chip better (layers of 7B ... 32B-class
// models at 2048 rows: 0.90 - 0.99 with 64 - 160 tiles, 1.02 - 1.08 from 224 tiles on; at 4096 rows
// 0.98 - 1.16, at 8192 rows 1.14 - 1.21 whatever the tile count).  K % 64 == 0 and G % 8 == 0 (both
// implied by the MFMA path's conditions).
constexpr int DENSE_MIN_ROWS = 2048;
inline bool dense_default(int M, int N) {
  if (M < DENSE_MIN_ROWS) return false;
  return M >= 2 * DENSE_MIN_ROWS || (long long)((M + 255) / 256) * ((N + 255) / 256) >= 192;
}
inline bool dense_rows(int M, int N) {
  if (variant_on(VAR_NO_DENSE)) return false;
  if (variant_on(VAR_DENSE)) return M > 256;
  return dense_default(M, N);
}
// workspace of the dequantise-once form: counters, K-split partial tiles, then the panel
inline size_t dense_panel_offset(size_t part_bytes) {
  return (AWQMI_WS_COUNTER_BYTES + part_bytes + 1023) / 1024 * 1024;
}

// Rows of the MFMA tile (64, 128, 192 or 256) for one launch.  Smaller tiles pad less and give
// more workgroups; larger ones unpack each weight for more rows.  Cost of a choice, in units of
// one k-tile of one row: rounds of 256 workgroups (a partial last round without a K split counts
// as at least 0.8) x (k-tiles + 12) x (rows + 64), plus the K-split round if there is one.
// Fitted on 96 points (six layer shapes, M = 65 ... 2048, every tile size forced in turn, two
// runs): the choice is within 4 % of the best size on every point (0.04 % behind on average),
// where "256 rows from 193 rows on" was 9 % behind on average.
int mfma_pick_rows(int M, int K, int N) {
  if (M <= 64) return 64;
  const int KT = K / PF_BK;
  double best = 1e300;
  int rows = 256;
  for (int bm = 64; bm <= 256; bm += 64) {
    const MfmaPlan pl = plan_mfma(M, K, N, bm);
    const double tk = bm + 64.0;
    const int whole = pl.dp_tiles / 256;
    const double part = (pl.dp_tiles % 256) / 256.0;
    double t = (whole + (part > 0 ? std::max(part, 0.8) : 0.0)) * (KT + 12) * tk;
    if (pl.sk_tiles > 0) t += ((double)KT / pl.sk_split + 12) * tk;
    if (t < best) { best = t; rows = bm; }
  }
  return rows;
}

}  // namespace

// Kernels that use more dynamic LDS than the default limit need a function attribute; it is
// set once per device for all of them (by awqmi_init, or by the first call on that device that
// needs one).
static int ensure_kernel_attributes() {
  static std::atomic<bool> done[MAX_DEVICES];
  int dev = -1;
  const hipError_t ge = hipGetDevice(&dev);
  if (ge != hipSuccess) { t_last_hip_error = (int)ge; return AWQMI_LAUNCH_FAILED; }
  if (dev < 0 || dev >= MAX_DEVICES) return AWQMI_BAD_ARGUMENT;
  if (done[dev].load(std::memory_order_acquire)) return AWQMI_OK;
  const void* mfma[] = {
      reinterpret_cast<const void*>(awq_gemm_mfma_kernel<true, 1, 8>), reinterpret_cast<const void*>(awq_gemm_mfma_kernel<false, 1, 8>),
      reinterpret_cast<const void*>(awq_gemm_mfma_kernel<true, 2, 8>), reinterpret_cast<const void*>(awq_gemm_mfma_kernel<false, 2, 8>),
      reinterpret_cast<const void*>(awq_gemm_mfma_kernel<true, 1>), reinterpret_cast<const void*>(awq_gemm_mfma_kernel<false, 1>),
      reinterpret_cast<const void*>(awq_gemm_mfma_kernel<true, 2>), reinterpret_cast<const void*>(awq_gemm_mfma_kernel<false, 2>),
      reinterpret_cast<const void*>(awq_gemm_mfma_kernel<true, 3>), reinterpret_cast<const void*>(awq_gemm_mfma_kernel<false, 3>),
      reinterpret_cast<const void*>(awq_gemm_mfma_kernel<true, 4>), reinterpret_cast<const void*>(awq_gemm_mfma_kernel<false, 4>),
      reinterpret_cast<const void*>(awq_gemm_mfma_kernel<true, 1, 8, true>), reinterpret_cast<const void*>(awq_gemm_mfma_kernel<false, 1, 8, true>),
      reinterpret_cast<const void*>(awq_gemm_mfma_kernel<true, 2, 8, true>), reinterpret_cast<const void*>(awq_gemm_mfma_kernel<false, 2, 8, true>),
      reinterpret_cast<const void*>(awq_gemm_mfma_kernel<true, 4, 4, true>), reinterpret_cast<const void*>(awq_gemm_mfma_kernel<false, 4, 4, true>)};
  for (const void* fn : mfma) {
    const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, PF_LDS_BYTES);
    if (e != hipSuccess) { t_last_hip_error = (int)e; return AWQMI_LAUNCH_FAILED; }
  }
  const void* align[] = {
      reinterpret_cast<const void*>(moe_align_kernel),
      reinterpret_cast<const void*>(moe_align_count_kernel), reinterpret_cast<const void*>(moe_align_place_kernel),
      reinterpret_cast<const void*>(moe_route_align_kernel<1, false>), reinterpret_cast<const void*>(moe_route_align_kernel<2, false>),
      reinterpret_cast<const void*>(moe_route_align_kernel<4, false>), reinterpret_cast<const void*>(moe_route_align_kernel<8, false>),
      reinterpret_cast<const void*>(moe_route_align_kernel<16, false>),
      reinterpret_cast<const void*>(moe_route_align_kernel<1, true>), reinterpret_cast<const void*>(moe_route_align_kernel<2, true>),
      reinterpret_cast<const void*>(moe_route_align_kernel<4, true>), reinterpret_cast<const void*>(moe_route_align_kernel<8, true>),
      reinterpret_cast<const void*>(moe_route_align_kernel<16, true>)};
  for (const void* fn : align) {
    const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                             (MOE_ALIGN_WAVES + 2) * AWQMI_MAX_EXPERTS * (int)sizeof(int));
    if (e != hipSuccess) { t_last_hip_error = (int)e; return AWQMI_LAUNCH_FAILED; }
  }
  done[dev].store(true, std::memory_order_release);
  return AWQMI_OK;
}

// routing and align in one launch (at most 16 tokens); same results as the two calls
template <int P>
static int moe_route_align_launch(const float* logits, const float* bias, int T, int E, int topk, int scoring,
                                  int renormalize, float scale, int32_t* ids, float* wts, int tile_m, int cap,
                                  int32_t* sorted, int32_t* experts, int32_t* npp, hipStream_t st) {
  if (const int rc = ensure_kernel_attributes()) return rc;
  const size_t lds = (size_t)(MOE_ALIGN_WAVES + 2) * E * sizeof(int);
  if (scoring == 1)
    hipLaunchKernelGGL((moe_route_align_kernel<P, true>), dim3(1), dim3(1024), lds, st, logits, bias, T, E, topk,
                       renormalize, scale, ids, wts, tile_m, cap, sorted, experts, npp);
  else
    hipLaunchKernelGGL((moe_route_align_kernel<P, false>), dim3(1), dim3(1024), lds, st, logits, (const float*)nullptr,
                       T, E, topk, renormalize, scale, ids, wts, tile_m, cap, sorted, experts, npp);
  return launch_status();
}

static int moe_route_align_small(const float* logits, const float* bias, int T, int E, int topk, int scoring,
                                 int renormalize, float scale, int32_t* ids, float* wts, int tile_m,
                                 int32_t* sorted, int32_t* experts, int32_t* npp, void* stream) {
  const int cap = (int)awqmi_moe_align_capacity(T * topk, E, tile_m);
  hipStream_t st = (hipStream_t)stream;
#define AWQMI_RA(P) \
  return moe_route_align_launch<P>(logits, bias, T, E, topk, scoring, renormalize, scale, ids, wts, tile_m, cap, \
                                   sorted, experts, npp, st)
  if (E <= 64) AWQMI_RA(1);
  if (E <= 128) AWQMI_RA(2);
  if (E <= 256) AWQMI_RA(4);
  if (E <= 512) AWQMI_RA(8);
  AWQMI_RA(16);
#undef AWQMI_RA
}

// Routing of one MoE block: inputs and the five lists it produces.
struct MoeRoute {
  const float* logits;
  const float* bias;
  int T, E, topk, scoring, renorm;
  float scale;
  int32_t* ids;
  float* wts;
  int32_t* sorted;
  int32_t* experts;
  int32_t* npp;
};

// Routing + align of a short slot list as launches of their own (one launch for up to 16
// tokens, else top-k and align apart).
static int moe_route_launches(const MoeRoute& r, int tile, void* stream) {
  if (r.T <= MOE_ALIGN_WAVES)
    return moe_route_align_small(r.logits, r.bias, r.T, r.E, r.topk, r.scoring, r.renorm, r.scale, r.ids, r.wts, tile,
                                 r.sorted, r.experts, r.npp, stream);
  if (const int st = awqmi_moe_topk_f32(r.logits, r.bias, r.T, r.E, r.topk, r.scoring, r.renorm, r.scale, r.ids, r.wts,
                                        stream))
    return st;
  return awqmi_moe_align(r.ids, r.T * r.topk, r.E, tile, r.sorted, r.experts, r.npp, stream);
}

// Folded routing: at most four tokens (one per wave of a workgroup; the kernel would take up to
// eight in turn, but from five tokens on every workgroup spends on the second round what the
// saved launch gains: 128 experts, top-8, weights from HBM: 3.5 us of 29 - 38 faster at 1 - 4
// tokens, 0.9 us at 5, nothing at 6 - 8), 64 slots (one lane each), 256 experts (four per lane).
static bool moe_route_foldable(int T, int E, int topk, int tile) {
  return T <= 4 && T * topk <= 64 && E <= 256 && tile == 16 && !variant_on(VAR_NO_FOLDED_ROUTE);
}

extern "C" {

int awqmi_init(void) {
  if (const int rc = ensure_kernel_attributes()) return rc;
  // the current device's static scratch array: look its address up and put its arrival counters
  // at zero (they are zero when the code object is loaded and every completed call leaves them
  // so; calling this again is the way back after a call that was cut short)
  void* ptr = nullptr;
  bool first = false;
  if (const int rc = static_scratch_ptr(&ptr, &first)) return rc;
  hipLaunchKernelGGL(awq_zero_words_kernel, dim3(AWQMI_WS_COUNTER_BYTES / 16 / 256), dim3(256), 0, (hipStream_t) nullptr,
                     reinterpret_cast<u4v*>(ptr), AWQMI_WS_COUNTER_BYTES / 16);
  if (const int rc = launch_status()) return rc;
  const hipError_t e = hipStreamSynchronize(nullptr);
  if (e != hipSuccess) { t_last_hip_error = (int)e; return AWQMI_LAUNCH_FAILED; }
  return AWQMI_OK;
}

int awqmi_version(void) { return AWQMI_VERSION; }

const char* awqmi_status_string(int s) {
  switch (s) {
    case AWQMI_OK: return "ok";
    case AWQMI_BAD_SHAPE: return "bad shape (need N % 8 == 0, K % group == 0, positive sizes)";
    case AWQMI_BAD_ALIGN: return "pointer not 16-byte aligned";
    case AWQMI_WORKSPACE_TOO_SMALL: return "workspace too small";
    case AWQMI_UNSUPPORTED_GROUP: return "unsupported group size";
    case AWQMI_LAUNCH_FAILED: return "kernel launch failed";
    case AWQMI_NULL_POINTER: return "null pointer";
    case AWQMI_BAD_ARGUMENT: return "bad argument";
    case AWQMI_SCRATCH_LIMIT:
      return "call needs more scratch than the static array holds (AWQMI_STATIC_SCRATCH_BYTES); "
             "use awqmi_gemm_f16 with a caller-owned workspace";
    default: return "unknown status";
  }
}

int awqmi_last_hip_error(void) { return t_last_hip_error; }

int awqmi_dequantize_f16(const int32_t* qweight, const void* scales, const int32_t* qzeros,
                         void* out, int K, int N, int group, void* stream) {
  return awqmi_dequantize_ld_f16(qweight, N / 8, scales, qzeros, out, K, N, group, stream);
}

int awqmi_dequantize_ld_f16(const int32_t* qweight, int ldw, const void* scales, const int32_t* qzeros,
                            void* out, int K, int N, int group, void* stream) {
  if (!qweight || !scales || !qzeros || !out) return AWQMI_NULL_POINTER;
  const int G = norm_group(K, group);
  if (const int rc = check_awq_shape(K, N, G)) return rc;
  if (ldw < N / 8 || (ldw != N / 8 && ldw % 4 != 0)) return AWQMI_BAD_ARGUMENT;
  if (!aligned16(scales) || !aligned16(out) || !aligned16(qweight) || !aligned16(qzeros))
    return AWQMI_BAD_ALIGN;
  const int NW = N / 8;
  hipStream_t st = (hipStream_t)stream;
  const uint32_t* qw = reinterpret_cast<const uint32_t*>(qweight);
  const uint32_t* qz = reinterpret_cast<const uint32_t*>(qzeros);
  const half_t* sc = reinterpret_cast<const half_t*>(scales);
  half_t* o = reinterpret_cast<half_t*>(out);
  const unsigned gx = (NW + 255) / 256;
#define AWQMI_DQ(R)                                                                              \
  for (int k0 = 0; k0 < K; k0 += 65535 * R) {                                                    \
    const int slabs = (K - k0) / R < 65535 ? (K - k0) / R : 65535;                               \
    hipLaunchKernelGGL((awq_dequant_kernel<R>), dim3(gx, slabs), dim3(256), 0, st, qw, sc, qz, o, k0, \
                       NW, G, ldw);                                                              \
  }
  if (G % 16 == 0) AWQMI_DQ(16)
  else if (G % 8 == 0) AWQMI_DQ(8)
  else if (G % 4 == 0) AWQMI_DQ(4)
  else if (G % 2 == 0) AWQMI_DQ(2)
  else AWQMI_DQ(1)
#undef AWQMI_DQ
  return launch_status();
}

int awqmi_gemm_auto_split_k(int M, int K, int N, int group) {
  const int G = norm_group(K, group);
  if (check_awq_shape(K, N, G) != AWQMI_OK || M <= 0) return 1;
  if (!skinny_rows(M, N) || !gemv_tiled_ok(K, G)) return 1;
  return pick_split_k(M, K, N, G, 1, true);
}

size_t awqmi_gemm_workspace_bytes(int M, int K, int N, int split_k) {
  if (M <= 0 || K <= 0 || N <= 0) return 0;
  // the group size decides between the kernels for some shapes, so cover both
  size_t mfma = 0, skinny = 0;
  if (M > 16 && K % PF_BK == 0) {
    const int slab = mfma_slab_rows(M, K);
    if (slab > 0) {
      // the tile rows the call will pick (a forced size that needs more falls back to no K split)
      mfma = plan_mfma(slab, K, N, mfma_pick_rows(slab, K, N)).part_bytes;
      if (M % slab) mfma = std::max(mfma, plan_mfma(M % slab, K, N, mfma_pick_rows(M % slab, K, N)).part_bytes);
      // the dequantise-once form of many-row calls: 256-row tiles, and the fp16 panel behind the
      // partial tiles (a call with a smaller workspace runs the fused kernel instead)
      if (dense_default(M, N)) {
        size_t part = plan_mfma(slab, K, N, 256).part_bytes;
        if (M % slab) part = std::max(part, plan_mfma(M % slab, K, N, 256).part_bytes);
        const size_t dense = dense_panel_offset(part) + dg_panel_bytes(K, N) - AWQMI_WS_COUNTER_BYTES;
        mfma = std::max(mfma, dense);
      }
    }
  }
  if (M <= SKINNY_MAX_M) {
    int s = split_k;
    // the pick depends on the group size (TAIL form only at G = 128): cover both
    if (s <= 0) s = (K % 128 == 0) ? std::max(pick_split_k(M, K, N, 128, 1, true), pick_split_k(M, K, N, 64, 1, true)) : 1;
    skinny = gemv_partial_bytes(N, s, 1, 32);
  }
  return AWQMI_WS_COUNTER_BYTES + (mfma > skinny ? mfma : skinny);
}

int awqmi_gemm_f16(const void* x, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                   void* y, void* workspace, size_t workspace_bytes, int M, int K, int N, int group,
                   int split_k, void* stream) {
  return awqmi_gemm_ld_f16(x, qweight, N / 8, scales, qzeros, y, workspace, workspace_bytes, M, K, N, group, split_k,
                           stream);
}

int awqmi_gemm_ld_f16(const void* x, const int32_t* qweight, int ldw, const void* scales, const int32_t* qzeros,
                      void* y, void* workspace, size_t workspace_bytes, int M, int K, int N, int group,
                      int split_k, void* stream) {
  if (!x || !qweight || !scales || !qzeros || !y) return AWQMI_NULL_POINTER;
  const int G = norm_group(K, group);
  if (const int rc = check_awq_shape(K, N, G)) return rc;
  if (M <= 0) return AWQMI_BAD_SHAPE;
  if (split_k < 0 || split_k > AWQMI_MAX_SPLIT_K) return AWQMI_BAD_ARGUMENT;
  if (ldw < N / 8 || (ldw != N / 8 && ldw % 4 != 0)) return AWQMI_BAD_ARGUMENT;
  if (!aligned16(x) || !aligned16(scales) || !aligned16(qweight) || !aligned16(qzeros) ||
      !aligned16(y))
    return AWQMI_BAD_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const int NW = N / 8;
  const uint32_t* qw = reinterpret_cast<const uint32_t*>(qweight);
  const uint32_t* qz = reinterpret_cast<const uint32_t*>(qzeros);
  const half_t* sc = reinterpret_cast<const half_t*>(scales);
  const half_t* xx = reinterpret_cast<const half_t*>(x);
  half_t* yy = reinterpret_cast<half_t*>(y);

  const int wpl = gemv_wpl(N);
  const bool mfma_ok = K % PF_BK == 0 && (((G & (G - 1)) == 0 && G >= 8) || G % 64 == 0) &&
                       mfma_slab_rows(M, K) > 0 && (size_t)K * ldw * 4 < (1ull << 32) &&
                       (size_t)(K / G) * N * 2 < (1ull << 32);
  bool mid_skinny = skinny_rows(M, N);
  if (variant_on(VAR_MID_M_SKINNY)) mid_skinny = true;
  if (variant_on(VAR_MID_M_MFMA)) mid_skinny = false;
  if (gemv_tiled_ok(K, G) &&
      (M <= 16 || (M <= SKINNY_MAX_M && wpl == 2 && (mid_skinny || !mfma_ok)))) {
    int split = split_k > 0 ? split_k : pick_split_k(M, K, N, G, 1, true);
    const int nchunks = K / 128;
    if (split > nchunks) split = nchunks;
    const int ncb = (NW + 16 * wpl - 1) / (16 * wpl);
    if (split > 1) {
      if (!workspace) return AWQMI_NULL_POINTER;
      if (!aligned16(workspace)) return AWQMI_BAD_ALIGN;
      if ((size_t)ncb * sizeof(int) > AWQMI_WS_COUNTER_BYTES) return AWQMI_BAD_SHAPE;
      if (workspace_bytes < AWQMI_WS_COUNTER_BYTES + gemv_partial_bytes(N, split, 1, M > 16 ? 32 : 16))
        return AWQMI_WORKSPACE_TOO_SMALL;
    }
    t_last_gemm_form = AWQMI_FORM_SKINNY;
    GemvParams p{};
    p.qw = qw; p.sc = sc; p.qz = qz;
    p.cnt = reinterpret_cast<int*>(workspace);
    p.part = workspace ? reinterpret_cast<float*>(static_cast<char*>(workspace) + AWQMI_WS_COUNTER_BYTES)
                       : nullptr;
    p.K = K; p.N = N; p.NW = NW; p.ldw = ldw; p.G = G; p.ldy = N;
    p.split_k = split; p.ncb = ncb;
    p.trace = t_trace;
    const dim3 grid(ncb, split, 1);
    // passes of up to 32 rows; each pass streams the weights once
    for (int r0 = 0; r0 < M; r0 += 32) {
      p.x = xx + (size_t)r0 * K;
      p.y = yy + (size_t)r0 * N;
      p.M = M - r0 < 32 ? M - r0 : 32;
      // 17 .. 32 rows with long wave ranges (six chunks or more): the weight ring in LDS leaves the
      // register file to the two accumulator sets (gate_up / down_proj of the 72B shapes 3 - 11 %
      // faster, bit-identical; short ranges measured equal or 1 - 2 % slower)
      const bool lds32 = nchunks >= 24 * split && (size_t)K * ldw * 4 < (1ull << 31) && !variant_on(VAR_NO_LDS_RING);
      if (p.M > 16 && lds32) launch_gemv<2, 2, false, 4, 4, false, true>(p, grid, st);
      else if (p.M > 16) launch_gemv<2, 2, false>(p, grid, st);
      else if (gemv_tail_shape(p.M, N, G) && gemv_tail_ok(nchunks, split))
        hipLaunchKernelGGL((awq_gemv_tail_kernel<2, 1>), grid, dim3(256), 0, st, p);
      else if (wpl == 2) launch_gemv<2, 1, false>(p, grid, st);
      else launch_gemv<1, 1, false>(p, grid, st);
    }
    return launch_status();
  }

  // MFMA kernel: K % 64 == 0, G a power of two >= 8 or a multiple of 64; buffer offsets are
  // 32-bit, so every operand must stay below 4 GiB
  const bool pow2g = (G & (G - 1)) == 0 && G >= 8;
  if (mfma_ok) {
    if (const int rc = ensure_kernel_attributes()) return rc;
    const int slab = mfma_slab_rows(M, K);
    // many rows: dequantise once into the workspace, then the dense kernel (same bits as the fused
    // kernel with 256-row tiles); needs the workspace to hold the panel
    if (dense_rows(M, N) && workspace && aligned16(workspace)) {
      size_t part = plan_mfma(slab < M ? slab : M, K, N, 256).part_bytes;
      if (M % slab) part = std::max(part, plan_mfma(M % slab, K, N, 256).part_bytes);
      const size_t panel_off = dense_panel_offset(part);
      if (workspace_bytes >= panel_off + dg_panel_bytes(K, N)) {
        t_last_gemm_form = AWQMI_FORM_DENSE;
        unsigned char* const panel = static_cast<unsigned char*>(workspace) + panel_off;
        const int nt = (N + 255) / 256;
        hipLaunchKernelGGL(awq_dequant_panel_kernel, dim3(nt, K / 64), dim3(256), 0, st, qw, sc, qz, panel, K, N, NW, G,
                           ldw);
        for (int r0 = 0; r0 < M; r0 += slab) {
          const int Ms = M - r0 < slab ? M - r0 : slab;
          const MfmaPlan pl = plan_mfma(Ms, K, N, 256);
          DenseGemmParams d{};
          d.x = xx + (size_t)r0 * K; d.panel = panel; d.y = yy + (size_t)r0 * N;
          d.M = Ms; d.K = K; d.N = N;
          d.mt = (Ms + 255) / 256; d.nt = nt;
          d.dp_tiles = pl.dp_tiles; d.sk_tiles = pl.sk_tiles; d.sk_split = pl.sk_split;
          d.per_xcd = (pl.dp_tiles + 7) / 8;
          d.sk_part = reinterpret_cast<float*>(static_cast<char*>(workspace) + AWQMI_WS_COUNTER_BYTES);
          hipLaunchKernelGGL(awq_gemm_dense_kernel, dim3(d.per_xcd * 8 + d.sk_tiles * d.sk_split), dim3(256), 0, st, d);
          if (d.sk_tiles > 0)
            hipLaunchKernelGGL(awq_gemm_dense_reduce_kernel, dim3(d.sk_tiles * 8), dim3(256), 0, st, d);
        }
        return launch_status();
      }
    }
    t_last_gemm_form = AWQMI_FORM_FUSED;
    for (int r0 = 0; r0 < M; r0 += slab) {
      const int Ms = M - r0 < slab ? M - r0 : slab;
      MfmaGemmParams p{};
      p.x = xx + (size_t)r0 * K; p.qw = qw; p.sc = sc; p.qz = qz; p.y = yy + (size_t)r0 * N;
      p.M = Ms; p.K = K; p.N = N; p.NW = NW; p.ldw = ldw; p.G = G;
      p.gshift = 0;
      if (pow2g) while ((1 << p.gshift) < G) ++p.gshift;
      int mi = mfma_pick_rows(Ms, K, N) / 64;
      const int vrows = t_variant;
      if (vrows >= 0 && ((vrows >> VAR_MFMA_ROWS_SHIFT) & 7) >= 1 && ((vrows >> VAR_MFMA_ROWS_SHIFT) & 7) <= 4)
        mi = (vrows >> VAR_MFMA_ROWS_SHIFT) & 7;
      const int bm = 64 * mi;
      p.mt = (Ms + bm - 1) / bm; p.nt = (N + PF_BN - 1) / PF_BN;
      p.total = p.mt * p.nt;
      MfmaPlan pl = plan_mfma(Ms, K, N, bm);
      // the K split needs the caller's workspace (counters + partial tiles); without it every
      // tile runs on one workgroup
      if (pl.sk_tiles > 0 && (!workspace || !aligned16(workspace) ||
                              workspace_bytes < AWQMI_WS_COUNTER_BYTES + pl.part_bytes))
        pl = MfmaPlan{p.total, 0, 1, 0};
      p.dp_tiles = pl.dp_tiles; p.sk_tiles = pl.sk_tiles; p.sk_split = pl.sk_split;
      p.per_xcd = (pl.dp_tiles + 7) / 8;
      p.sk_part = workspace ? reinterpret_cast<float*>(static_cast<char*>(workspace) + AWQMI_WS_COUNTER_BYTES)
                            : nullptr;
      const dim3 grid(p.per_xcd * 8 + p.sk_tiles * p.sk_split);
#define AWQMI_MFMA(MIV, NWVV)                                                                      \
  do {                                                                                           \
    if (pow2g)                                                                                   \
      hipLaunchKernelGGL((awq_gemm_mfma_kernel<true, MIV, NWVV>), grid, dim3(64 * NWVV), PF_LDS_BYTES, st, p);  \
    else                                                                                         \
      hipLaunchKernelGGL((awq_gemm_mfma_kernel<false, MIV, NWVV>), grid, dim3(64 * NWVV), PF_LDS_BYTES, st, p); \
    if (p.sk_tiles > 0)                                                                          \
      hipLaunchKernelGGL((awq_gemm_mfma_reduce_kernel<MIV, NWVV>), dim3(p.sk_tiles * MIV * (16 / NWVV)),       \
                         dim3(64 * NWVV), 0, st, p);                                              \
  } while (0)
      const bool eight = !variant_on(VAR_MFMA_FOUR_WAVES);
      if (mi == 1 && eight) AWQMI_MFMA(1, 8);
      else if (mi == 2 && eight) AWQMI_MFMA(2, 8);
      else if (mi == 1) AWQMI_MFMA(1, 4);
      else if (mi == 2) AWQMI_MFMA(2, 4);
      else if (mi == 3) AWQMI_MFMA(3, 4);
      else AWQMI_MFMA(4, 4);
#undef AWQMI_MFMA
    }
    return launch_status();
  }

  // any other shape: one thread per packed word and row; the row index is the grid's second
  // dimension (at most 65535), so more rows run as consecutive slabs
  t_last_gemm_form = AWQMI_FORM_GENERIC;
  for (int r0 = 0; r0 < M; r0 += 32768) {
    const int Ms = M - r0 < 32768 ? M - r0 : 32768;
    hipLaunchKernelGGL(awq_gemm_generic_kernel, dim3((NW + 255) / 256, Ms), dim3(256), 0, st,
                       xx + (size_t)r0 * K, qw, sc, qz, yy + (size_t)r0 * N, Ms, K, NW, G, ldw);
  }
  return launch_status();
}

int awqmi_gemm_f16_noalloc(const void* x, const int32_t* qweight, int ldw, const void* scales, const int32_t* qzeros,
                           void* y, int M, int K, int N, int group, int split_k, void* stream) {
  void* ptr = nullptr;
  bool first = false;
  if (const int rc = static_scratch_ptr(&ptr, &first)) return rc;
  // exactly awqmi_gemm_ld_f16 with this GPU's static array as the workspace (it validates before
  // it launches, so a skinny call whose split-K partial tiles do not fit launches nothing)
  const int rc = awqmi_gemm_ld_f16(x, qweight, ldw == 0 ? N / 8 : ldw, scales, qzeros, y, ptr, AWQMI_STATIC_SCRATCH_BYTES,
                                   M, K, N, group, split_k, stream);
  return rc == AWQMI_WORKSPACE_TOO_SMALL ? AWQMI_SCRATCH_LIMIT : rc;
}

int awqmi_moe_topk_f32(const float* logits, const float* score_bias, int T, int E, int topk, int scoring,
                       int renormalize, float scale, int32_t* topk_ids, float* topk_weights, void* stream) {
  if (!logits || !topk_ids || !topk_weights) return AWQMI_NULL_POINTER;
  if (T <= 0 || E <= 0) return AWQMI_BAD_SHAPE;
  if (E > AWQMI_MAX_EXPERTS || topk <= 0 || topk > E || topk > 64 || (scoring != 0 && scoring != 1))
    return AWQMI_BAD_ARGUMENT;
  if (scoring == 0 && score_bias) return AWQMI_BAD_ARGUMENT;   // the bias belongs to sigmoid scoring
  const dim3 grid((T + 3) / 4);
  hipStream_t st = (hipStream_t)stream;
#define AWQMI_TOPK(P)                                                                              \
  do {                                                                                             \
    if (scoring == 1)                                                                              \
      hipLaunchKernelGGL((moe_topk_kernel<P, true>), grid, dim3(256), 0, st, logits, score_bias, T, E, topk, \
                         renormalize, scale, topk_ids, topk_weights);                              \
    else                                                                                           \
      hipLaunchKernelGGL((moe_topk_kernel<P, false>), grid, dim3(256), 0, st, logits, score_bias, T, E, topk, \
                         renormalize, scale, topk_ids, topk_weights);                              \
  } while (0)
  if (E <= 64) AWQMI_TOPK(1);
  else if (E <= 128) AWQMI_TOPK(2);
  else if (E <= 256) AWQMI_TOPK(4);
  else if (E <= 512) AWQMI_TOPK(8);
  else AWQMI_TOPK(16);
#undef AWQMI_TOPK
  return launch_status();
}

int awqmi_moe_topk_softmax_f32(const float* logits, int T, int E, int topk, int renormalize,
                               int32_t* topk_ids, float* topk_weights, void* stream) {
  return awqmi_moe_topk_f32(logits, nullptr, T, E, topk, 0, renormalize, 1.f, topk_ids, topk_weights, stream);
}

size_t awqmi_moe_align_capacity(int n_slots, int E, int tile_m) {
  if (n_slots < 0 || E <= 0 || tile_m <= 0) return 0;
  const size_t worst = (size_t)n_slots + (size_t)E * (tile_m - 1);
  return (worst + tile_m - 1) / tile_m * tile_m;
}

int awqmi_moe_align(const int32_t* topk_ids, int n_slots, int E, int tile_m, int32_t* sorted_token_ids,
                    int32_t* expert_ids, int32_t* num_tokens_post_padded, void* stream) {
  if (!topk_ids || !sorted_token_ids || !expert_ids || !num_tokens_post_padded)
    return AWQMI_NULL_POINTER;
  if (n_slots <= 0 || E <= 0) return AWQMI_BAD_SHAPE;
  if (E > AWQMI_MAX_EXPERTS || tile_m <= 0 || tile_m > 4096) return AWQMI_BAD_ARGUMENT;
  const int cap = (int)awqmi_moe_align_capacity(n_slots, E, tile_m);
  if (const int rc = ensure_kernel_attributes()) return rc;
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), (size_t)(MOE_ALIGN_WAVES + 2) * E * sizeof(int),
                     (hipStream_t)stream, topk_ids, n_slots, E, tile_m, cap, sorted_token_ids,
                     expert_ids, num_tokens_post_padded);
  return launch_status();
}

// sorted-token blocks a grouped launch covers: the align capacity, rounded up to whole groups
static int moe_launch_blocks(int n_slots, int E, int tile_m) {
  int nblk = (int)(awqmi_moe_align_capacity(n_slots, E, tile_m) / tile_m);
  // a block that runs holds at least one real slot: a handful of tokens never fills more blocks
  // than it has slots, whatever the expert count (one token with 8 picks of 128 experts: 8
  // blocks, not 121 -- the rest would be workgroups that start, read the padded count and leave)
  if (nblk > n_slots) nblk = n_slots;
  return (nblk + MOE_BLOCK_GROUP_MAX - 1) / MOE_BLOCK_GROUP_MAX * MOE_BLOCK_GROUP_MAX;
}

// Launch shape of a grouped GEMM, shared by the workspace query and the launch itself.
struct MoePlan { int wpl, ncb, nblk, split; };
static MoePlan moe_plan(int n_slots, int E, int K, int N, int tile_m, int split_req) {
  MoePlan pl{};
  const int NW = N / 8;
  pl.wpl = gemv_wpl(N);
  pl.ncb = (NW + 16 * pl.wpl - 1) / (16 * pl.wpl);
  pl.nblk = moe_launch_blocks(n_slots, E, tile_m);
  const int nchunks = K / 128;
  // blocks that will actually run: at most one per tile_m slots plus one per expert touched
  long long live = (n_slots + tile_m - 1) / tile_m;
  const long long touched = n_slots < E ? n_slots : E;
  if (live < touched) live = touched;
  int s = split_req;
  if (s <= 0) {
    if (K % 128 != 0) {
      s = 1;
    } else {
      s = pick_split_k(16, K, N, 128, live);
    }
    if ((size_t)pl.nblk * pl.ncb * sizeof(int) > AWQMI_WS_COUNTER_BYTES) s = 1;
  }
  if (s > nchunks) s = nchunks > 0 ? nchunks : 1;
  pl.split = s;
  return pl;
}

size_t awqmi_moe_gemm_workspace_bytes(int n_slots, int E, int K, int N, int split_k, int tile_m) {
  if (n_slots <= 0 || E <= 0 || K <= 0 || N <= 0 || N % 8 != 0 ||
      (tile_m != 16 && tile_m != 32 && tile_m != 64 && tile_m != 128 && tile_m != 256))
    return 0;
  if (tile_m >= 64) return AWQMI_WS_COUNTER_BYTES;    // the grouped MFMA form needs no partials
  const MoePlan pl = moe_plan(n_slots, E, K, N, tile_m, split_k);
  return AWQMI_WS_COUNTER_BYTES + gemv_partial_bytes(N, pl.split, pl.nblk, tile_m);
}

// Can the w13 GEMM of a block write silu(gate) * up itself?  Needs the paired-column launch
// (two column blocks per workgroup: the gate block and its up block), i.e. no split across
// workgroups, an even chunk count, [gate | up] halves that are whole column blocks, and
// enough blocks that the halved workgroup count still fills the chip.  It pays from about
// eight real rows per 16-row block on (measured on 2048 x 1536 experts, 128 of them: 6 %
// faster at 12 rows per block, 3 - 5 % slower at 2 - 6); below that the separate activation
// kernel is cheaper than the two-waves-per-column-block form of the GEMM.
static bool moe_can_fuse_act(int n_slots, int E, int K, int N) {
  const MoePlan pl = moe_plan(n_slots, E, K, N, 16, 0);
  const long long live_blocks = std::max<long long>((n_slots + 15) / 16, std::min(n_slots, E));
  return pl.wpl == 2 && pl.split == 1 && K % 128 == 0 && (K / 128) % 2 == 0 && N % 512 == 0 &&
         live_blocks * (pl.ncb / 2) >= 256 && n_slots >= 8 * live_blocks;
}

// Same question for a launch that is split in K: the last arrivers of a gate block and its up
// block finish both and apply the activation.
static bool moe_can_fuse_act_split(int n_slots, int E, int K, int N) {
  const MoePlan pl = moe_plan(n_slots, E, K, N, 16, 0);
  return pl.wpl == 2 && pl.split > 1 && N % 512 == 0 && pl.ncb % 2 == 0;
}

static int moe_gemm_impl(const void* x, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                         void* y, const int32_t* sorted_token_ids, const int32_t* expert_ids,
                         const int32_t* num_tokens_post_padded, const float* topk_weights, int n_slots,
                         int a_row_div, int tile_m, int E, int K, int N, int group, int split_k,
                         void* workspace, size_t workspace_bytes, void* stream, bool fuse_act,
                         const MoeRoute* route = nullptr);

int awqmi_moe_gemm_f16(const void* x, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                       void* y, const int32_t* sorted_token_ids, const int32_t* expert_ids,
                       const int32_t* num_tokens_post_padded, const float* topk_weights, int n_slots,
                       int a_row_div, int tile_m, int E, int K, int N, int group, int split_k,
                       void* workspace, size_t workspace_bytes, void* stream) {
  return moe_gemm_impl(x, qweight, scales, qzeros, y, sorted_token_ids, expert_ids, num_tokens_post_padded,
                       topk_weights, n_slots, a_row_div, tile_m, E, K, N, group, split_k, workspace,
                       workspace_bytes, stream, false);
}

static int moe_gemm_impl(const void* x, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                         void* y, const int32_t* sorted_token_ids, const int32_t* expert_ids,
                         const int32_t* num_tokens_post_padded, const float* topk_weights, int n_slots,
                         int a_row_div, int tile_m, int E, int K, int N, int group, int split_k,
                         void* workspace, size_t workspace_bytes, void* stream, bool fuse_act,
                         const MoeRoute* route) {
  // route: the block's routing has not run yet.  The launch takes it along when it is the plain
  // 16-row-block form with G = 128; any other form routes in launches of its own first.
  if (!x || !qweight || !scales || !qzeros || !y || !sorted_token_ids || !expert_ids ||
      !num_tokens_post_padded)
    return AWQMI_NULL_POINTER;
  const int G = norm_group(K, group);
  if (const int rc = check_awq_shape(K, N, G)) return rc;
  if (n_slots <= 0 || E <= 0) return AWQMI_BAD_SHAPE;
  if (a_row_div <= 0 || split_k < 0 || split_k > AWQMI_MAX_SPLIT_K || E > AWQMI_MAX_EXPERTS ||
      (tile_m != 16 && tile_m != 32 && tile_m != 64 && tile_m != 128 && tile_m != 256))
    return AWQMI_BAD_ARGUMENT;
  if (!gemv_tiled_ok(K, G)) return AWQMI_UNSUPPORTED_GROUP;
  if (!aligned16(x) || !aligned16(scales) || !aligned16(qweight) || !aligned16(qzeros) ||
      !aligned16(y))
    return AWQMI_BAD_ALIGN;
  const int NW = N / 8;
  if (tile_m >= 64) {
    // blocks of 64 / 128 slots: the MFMA kernel in its expert-grouped form (no K split)
    if (fuse_act) return AWQMI_BAD_ARGUMENT;
    if (route)
      if (const int rc = moe_route_launches(*route, tile_m, stream)) return rc;
    const size_t x_rows = ((size_t)n_slots + a_row_div - 1) / a_row_div;
    if (x_rows * K * 2 >= (1ull << 32) || (size_t)K * NW * 4 >= (1ull << 32) ||
        (size_t)(K / G) * N * 2 >= (1ull << 32))
      return AWQMI_BAD_SHAPE;
    if (const int rc = ensure_kernel_attributes()) return rc;
    MfmaGemmParams p{};
    p.x = reinterpret_cast<const half_t*>(x);
    p.qw = reinterpret_cast<const uint32_t*>(qweight);
    p.sc = reinterpret_cast<const half_t*>(scales);
    p.qz = reinterpret_cast<const uint32_t*>(qzeros);
    p.y = reinterpret_cast<half_t*>(y);
    p.M = (int)x_rows; p.K = K; p.N = N; p.NW = NW; p.ldw = NW; p.G = G;
    const bool pow2g = (G & (G - 1)) == 0 && G >= 8;
    p.gshift = 0;
    if (pow2g) while ((1 << p.gshift) < G) ++p.gshift;
    p.mt = 1; p.nt = (N + PF_BN - 1) / PF_BN; p.total = p.nt; p.per_xcd = 0;
    p.dp_tiles = 0; p.sk_tiles = 0; p.sk_split = 1;
    p.sorted_ids = sorted_token_ids; p.expert_ids = expert_ids; p.n_post_pad = num_tokens_post_padded;
    p.topk_w = topk_weights; p.n_slots = n_slots; p.a_row_div = a_row_div;
    p.w_stride = (long long)K * NW; p.s_stride = (long long)(K / G) * N; p.z_stride = (long long)(K / G) * NW;
    const int nblk = (int)(awqmi_moe_align_capacity(n_slots, E, tile_m) / tile_m);
    const dim3 grid((unsigned)nblk * p.nt);
    hipStream_t st = (hipStream_t)stream;
    if (tile_m == 64) {
      if (pow2g) hipLaunchKernelGGL((awq_gemm_mfma_kernel<true, 1, 8, true>), grid, dim3(512), PF_LDS_BYTES, st, p);
      else hipLaunchKernelGGL((awq_gemm_mfma_kernel<false, 1, 8, true>), grid, dim3(512), PF_LDS_BYTES, st, p);
    } else if (tile_m == 128) {
      if (pow2g) hipLaunchKernelGGL((awq_gemm_mfma_kernel<true, 2, 8, true>), grid, dim3(512), PF_LDS_BYTES, st, p);
      else hipLaunchKernelGGL((awq_gemm_mfma_kernel<false, 2, 8, true>), grid, dim3(512), PF_LDS_BYTES, st, p);
    } else {
      if (pow2g) hipLaunchKernelGGL((awq_gemm_mfma_kernel<true, 4, 4, true>), grid, dim3(256), PF_LDS_BYTES, st, p);
      else hipLaunchKernelGGL((awq_gemm_mfma_kernel<false, 4, 4, true>), grid, dim3(256), PF_LDS_BYTES, st, p);
    }
    return launch_status();
  }
  const MoePlan pl = moe_plan(n_slots, E, K, N, tile_m, split_k);
  const int wpl = pl.wpl, ncb = pl.ncb, nblk = pl.nblk, split = pl.split;
  // 32-row blocks: one packed word per lane, two column blocks of 128 per workgroup with two waves
  // each (the accumulators of two row blocks then take the registers one row block takes with two
  // words per lane, and two workgroups still fit a CU), the weight ring of four steps in LDS;
  // needs an even chunk count, no K split.  (One 128-column block per workgroup with four K
  // ranges measured 35 - 70 % slower: neighbouring workgroups then fetch the two halves of every
  // 128-byte line.)
  const bool t32_narrow = tile_m == 32 && split == 1 && (K / 128) % 2 == 0 && !variant_on(VAR_MOE_T32_WIDE);
  if (tile_m == 32 && !t32_narrow && wpl != 2) return AWQMI_BAD_SHAPE;   // the wide form needs N % 16 == 0
  if (split > 1) {
    if (!workspace) return AWQMI_NULL_POINTER;
    if (!aligned16(workspace)) return AWQMI_BAD_ALIGN;
    if ((size_t)nblk * ncb * sizeof(int) > AWQMI_WS_COUNTER_BYTES) return AWQMI_BAD_ARGUMENT;
    if (workspace_bytes < AWQMI_WS_COUNTER_BYTES + gemv_partial_bytes(N, split, nblk, tile_m))
      return AWQMI_WORKSPACE_TOO_SMALL;
  }
  GemvParams p{};
  p.x = reinterpret_cast<const half_t*>(x);
  p.qw = reinterpret_cast<const uint32_t*>(qweight);
  p.sc = reinterpret_cast<const half_t*>(scales);
  p.qz = reinterpret_cast<const uint32_t*>(qzeros);
  p.y = reinterpret_cast<half_t*>(y);
  p.cnt = reinterpret_cast<int*>(workspace);
  p.part = workspace ? reinterpret_cast<float*>(static_cast<char*>(workspace) + AWQMI_WS_COUNTER_BYTES)
                     : nullptr;
  p.M = tile_m; p.K = K; p.N = N; p.NW = NW; p.ldw = NW; p.G = G;
  p.split_k = split; p.ncb = ncb;
  p.sorted_ids = sorted_token_ids; p.expert_ids = expert_ids; p.n_post_pad = num_tokens_post_padded;
  p.topk_w = topk_weights; p.n_slots = n_slots; p.a_row_div = a_row_div; p.tile_m = tile_m;
  p.w_stride = (long long)K * NW; p.s_stride = (long long)(K / G) * N; p.z_stride = (long long)(K / G) * NW;
  p.nblk = nblk;
  p.nblk_cap = (int)(awqmi_moe_align_capacity(n_slots, E, tile_m) / tile_m);
  p.ldy = fuse_act ? N / 2 : N;
  const int variant = t_variant;
  // group blocks by XCD once most experts have a full block: runs of 8 from 0.75 blocks per
  // expert on, runs of 32 from 1.5 (measured on 128 experts: 6 % at one block per expert, 15 %
  // at 1.5, 3 - 4 % at 2 - 4 against runs of 8 or none; below 0.75 the order makes no difference)
  p.grp = (long long)n_slots * 2 >= 3LL * tile_m * E ? 32 : ((long long)n_slots * 4 >= 3LL * tile_m * E ? 8 : 1);
  if (E < 16) p.grp = 1;   // a handful of large experts: the plain order measured equal or up to 13 % faster
  if (variant >= 0 && ((variant >> VAR_XCD_RUN_SHIFT) & 7)) p.grp = 1 << (((variant >> VAR_XCD_RUN_SHIFT) & 7) - 1);
  // few chunks of K and no split across workgroups: two column blocks per workgroup, two
  // waves each (three chunks per wave at K = 768 instead of 2 / 2 / 1 / 1)
  // -- as long as the paired launch still fills the chip (blocks that will run: one per expert
  // touched or per 16 slots, whichever is more)
  const long long live_blocks = std::max<long long>((n_slots + 15) / 16, std::min(n_slots, E));
  const bool pair_cols = tile_m == 16 && wpl == 2 && split == 1 && K / 128 <= 8 && (K / 128) % 2 == 0 &&
                         live_blocks * ((ncb + 1) / 2) >= 256 && !variant_on(VAR_NO_PAIR_COLS);
  // fused activation: without a split the paired-column kernel (gate and up block in one
  // workgroup); with a split the ordinary launch whose last arrivers pair the blocks up
  if (fuse_act && (wpl != 2 || tile_m != 16 || ncb % 2 != 0 || N % 512 != 0 ||
                   (split == 1 && (K / 128) % 2 != 0)))
    return AWQMI_BAD_ARGUMENT;
  const bool act_split = fuse_act && split > 1;
  p.act_split = act_split ? 1 : 0;
  const bool act_pair = fuse_act && split == 1;
  const int ncb1 = (NW + 15) / 16;       // column blocks of 128 (one word per lane)
  const bool t32_lds = t32_narrow && (size_t)K * NW * 4 < (1ull << 31) && !variant_on(VAR_NO_LDS_RING);
  const int ncg = t32_narrow ? (ncb1 + 1) / 2 : (act_pair ? ncb / 2 : (pair_cols ? (ncb + 1) / 2 : ncb));
  if (t32_narrow) p.ncb = ncb1;
  // runs of grp slots, dealt to the 8 XCDs in turn; the last deal may be partial
  const long long runs = (long long)(nblk / p.grp) * ncg * split;
  const dim3 grid((unsigned)((runs + 7) / 8 * 8 * p.grp));
  hipStream_t st = (hipStream_t)stream;
  // weight ring of four steps in LDS instead of two in registers, from one full block per
  // expert on (T = 256 ... 1024 of the 128-expert block: 6 - 10 % faster; with fewer rows per
  // expert 1 - 4 % slower, and no gain for the few-block launches once their weights come from
  // HBM rather than from a warm cache)
  const bool ldsq = wpl == 2 && tile_m == 16 && (size_t)K * NW * 4 < (1ull << 31) &&
                    (long long)n_slots >= 16LL * E && !variant_on(VAR_NO_LDS_RING);
  const bool plain_form = !ldsq && !act_pair &&
                          (act_split || (tile_m == 16 && wpl == 2 && !pair_cols && !variant_on(VAR_MOE_RING4)));
  if (route) {
    if (plain_form && G == 128 && moe_route_foldable(route->T, route->E, route->topk, tile_m)) {
      p.r_logits = route->logits; p.r_bias = route->bias;
      p.r_T = route->T; p.r_E = route->E; p.r_topk = route->topk; p.r_renorm = route->renorm;
      p.r_scale = route->scale;
      p.r_ids = route->ids; p.r_wts = route->wts; p.r_sorted = route->sorted; p.r_experts = route->experts;
      p.r_npp = route->npp;
      const bool sig = route->scoring == 1;
#define AWQMI_ROUTE(PERV)                                                                                   \
  do {                                                                                                      \
    if (sig) hipLaunchKernelGGL((awq_gemv_route_kernel<2, PERV, true>), grid, dim3(256), 0, st, p);        \
    else hipLaunchKernelGGL((awq_gemv_route_kernel<2, PERV, false>), grid, dim3(256), 0, st, p);           \
  } while (0)
      if (route->E <= 64) AWQMI_ROUTE(1);
      else if (route->E <= 128) AWQMI_ROUTE(2);
      else AWQMI_ROUTE(4);
#undef AWQMI_ROUTE
      return launch_status();
    }
    if (const int rc = moe_route_launches(*route, tile_m, stream)) return rc;
  }
  if (ldsq && act_pair) launch_gemv<2, 1, true, 4, 2, true, true>(p, grid, st);
  else if (ldsq && pair_cols && !act_split) launch_gemv<2, 1, true, 4, 2, false, true>(p, grid, st);
  else if (ldsq) launch_gemv<2, 1, true, 4, 4, false, true>(p, grid, st);
  else if (act_pair) launch_gemv<2, 1, true, 2, 2, true>(p, grid, st);
  else if (act_split) launch_gemv<2, 1, true, 2>(p, grid, st);
  else if (t32_lds) launch_gemv<1, 2, true, 4, 2, false, true>(p, grid, st);
  else if (t32_narrow) launch_gemv<1, 2, true, 2, 2>(p, grid, st);
  else if (tile_m == 32) launch_gemv<2, 2, true>(p, grid, st);
  else if (wpl == 2 && variant_on(VAR_MOE_RING4)) launch_gemv<2, 1, true, 4>(p, grid, st);
  else if (pair_cols) launch_gemv<2, 1, true, 2, 2>(p, grid, st);
  else if (wpl == 2) launch_gemv<2, 1, true, 2>(p, grid, st);
  else launch_gemv<1, 1, true>(p, grid, st);
  return launch_status();
}

int awqmi_silu_and_mul_f16(const void* in, void* out, int rows, int inter, void* stream) {
  if (!in || !out) return AWQMI_NULL_POINTER;
  if (rows <= 0 || inter <= 0 || inter % 8 != 0) return AWQMI_BAD_SHAPE;
  if (!aligned16(in) || !aligned16(out)) return AWQMI_BAD_ALIGN;
  const size_t n = (size_t)rows * (inter / 8);
  hipLaunchKernelGGL(silu_and_mul_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, reinterpret_cast<const half_t*>(in),
                     reinterpret_cast<half_t*>(out), rows, inter);
  return launch_status();
}

int awqmi_moe_sum_f16(const void* in, void* out, int T, int topk, int H, void* stream) {
  if (!in || !out) return AWQMI_NULL_POINTER;
  if (T <= 0 || topk <= 0 || H <= 0 || H % 8 != 0) return AWQMI_BAD_SHAPE;
  if (!aligned16(in) || !aligned16(out)) return AWQMI_BAD_ALIGN;
  const size_t n = (size_t)T * (H / 8);
  hipLaunchKernelGGL(moe_sum_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, reinterpret_cast<const half_t*>(in),
                     reinterpret_cast<half_t*>(out), T, topk, H);
  return launch_status();
}

namespace {
constexpr int MOE_ALIGN_PARTS_MAX = 64;      // workgroups of the multi-workgroup align
constexpr int MOE_ALIGN_SPLIT_MIN = 16384;   // slots from which it is used (4096 per workgroup)

// Rows per block for the two expert GEMMs of one MoE block: 16 (the skinny kernel) or 64 /
// 128 / 256 (the MFMA kernel's expert-grouped form).  Cost model fitted on measurements over
// three expert shapes (2048/768 x 128 experts, 6144/2560 x 160, 4096/14336 x 8):
//   skinny: flops / (540 TFLOP/s * avg / (avg + 26)), avg = slots per expert;
//   MFMA:   per GEMM blocks * column tiles / 256 CUs rounds (a partial last round counts as
//           at least half) of (K / 64 + overhead) k-tiles at 5.4 ns * (rows + 112) each, plus
//           the separate SiLU pass at 4 TB/s; blocks is the expected block count after
//           padding each expert's run to whole blocks (slots spread evenly over the experts).
// Within 5 % of the best forced block size on 25 points over six expert shapes (fit) and on the
// points of three further shapes it was then checked on.
// The MFMA form also needs every operand under 4 GiB (32-bit buffer offsets).
int moe_pick_tile(int n_slots, int E, int H, int inter, int group) {
  if (variant_on(VAR_MOE_TILE16)) return 16;
  if (!gemv_tiled_ok(H, norm_group(H, group)) || !gemv_tiled_ok(inter, norm_group(inter, group))) return 16;
  if ((size_t)n_slots * std::max(H, inter) * 2 >= (1ull << 32) ||
      (size_t)H * (2 * inter / 8) * 4 >= (1ull << 32) || (size_t)inter * (H / 8) * 4 >= (1ull << 32))
    return 16;
  const int vv = t_variant;
  if (vv >= 0 && ((vv >> VAR_MOE_TILE_SHIFT) & 3)) return 32 << ((vv >> VAR_MOE_TILE_SHIFT) & 3);
  const double avg = (double)n_slots / E;
  // below two 16-row blocks per expert a 64-row block is mostly padding (and the cost terms
  // below, fitted on avg >= 32, do not describe launches of a few blocks)
  if (avg < 32.0) return 16;
  const double flops = 2.0 * n_slots * ((double)H * 2 * inter + (double)inter * H);
  double best = flops / (540e12 * avg / (avg + 26.0));
  int tile = 16;
  for (int bm : {64, 128, 256}) {
    // expected blocks after padding each expert's run: E * sum_j P(count > j * bm), the count
    // of an expert taken as Poisson(avg) (normal tail for j >= 1)
    double per_expert = 1.0 - std::exp(-avg);
    for (int j = 1; j * (double)bm < avg + 6.0 * std::sqrt(avg) + 1.0; ++j)
      per_expert += 0.5 * std::erfc((j * (double)bm + 0.5 - avg) / std::sqrt(2.0 * avg));
    const double blocks = E * per_expert;
    const double kt_s = 5.4e-9 * (bm + 112);
    const int over = bm == 256 ? 6 : 4;
    auto gemm = [&](int K, int N) {
      const double r = blocks * ((N + PF_BN - 1) / PF_BN) / 256.0;
      const double whole = std::floor(r), part = r - whole;
      const double rounds = whole + (part > 0 ? std::max(part, 0.5) : 0.0);
      return rounds * (K / PF_BK + over) * kt_s;
    };
    const double t = gemm(H, 2 * inter) + gemm(inter, H) + 5e-6 + 6.0 * n_slots * inter / 4e12;
    if (t < best) { best = t; tile = bm; }
  }
  return tile;
}

// workspace carve-up of the fused MoE block; every piece starts 256-byte aligned
struct FusedMoeLayout {
  size_t gemm_ws, ids, wts, sorted, experts, npp, h13, act, o, total;
  size_t gemm_ws_bytes;
  int n_slots, cap, tile;
  size_t tab;      // per-part expert counts / first positions of the multi-workgroup align
};
FusedMoeLayout fused_moe_layout(int T, int H, int inter, int E, int topk, int tile) {
  FusedMoeLayout L{};
  auto up = [](size_t v) { return (v + 255) / 256 * 256; };
  L.n_slots = T * topk;
  L.tile = tile;
  L.cap = (int)awqmi_moe_align_capacity(L.n_slots, E, L.tile);
  const size_t g1 = awqmi_moe_gemm_workspace_bytes(L.n_slots, E, H, 2 * inter, 0, L.tile);
  const size_t g2 = awqmi_moe_gemm_workspace_bytes(L.n_slots, E, inter, H, 0, L.tile);
  L.gemm_ws_bytes = g1 > g2 ? g1 : g2;
  size_t off = 0;
  L.gemm_ws = off; off += up(L.gemm_ws_bytes);
  L.ids = off;     off += up((size_t)L.n_slots * 4);
  L.wts = off;     off += up((size_t)L.n_slots * 4);
  L.sorted = off;  off += up((size_t)L.cap * 4);
  L.experts = off; off += up((size_t)(L.cap / L.tile) * 4);
  L.npp = off;     off += 256;
  L.tab = off;     off += up((size_t)MOE_ALIGN_PARTS_MAX * E * 4);
  L.h13 = off;     off += up((size_t)L.n_slots * 2 * inter * 2);
  L.act = off;     off += up((size_t)L.n_slots * inter * 2);
  L.o = off;       off += up((size_t)L.n_slots * H * 2);
  L.total = off;
  return L;
}
}  // namespace

size_t awqmi_fused_moe_workspace_bytes(int T, int H, int inter, int E, int topk) {
  if (T <= 0 || H <= 0 || inter <= 0 || E <= 0 || topk <= 0 || H % 8 != 0 || inter % 8 != 0) return 0;
  if ((long long)T * topk > (1LL << 30)) return 0;
  size_t most = 0;     // the call picks the block rows from the shapes; any choice fits
  for (int tile : {16, 64, 128, 256}) most = std::max(most, fused_moe_layout(T, H, inter, E, topk, tile).total);
  return most;
}

int awqmi_fused_moe_block_rows(int T, int H, int inter, int E, int topk, int group) {
  if (T <= 0 || H <= 0 || inter <= 0 || E <= 0 || H % 8 != 0 || inter % 8 != 0) return 0;
  if (topk <= 0 || topk > E || topk > 64 || E > AWQMI_MAX_EXPERTS || (long long)T * topk > (1LL << 30)) return 0;
  return moe_pick_tile(T * topk, E, H, inter, group);
}

int awqmi_fused_moe_f16(const void* hidden, const float* router_logits, const int32_t* w13_q,
                        const void* w13_s, const int32_t* w13_z, const int32_t* w2_q, const void* w2_s,
                        const int32_t* w2_z, void* out, int T, int H, int inter, int E, int topk,
                        int group, int renormalize, void* workspace, size_t workspace_bytes,
                        void* stream) {
  return awqmi_fused_moe_routed_f16(hidden, router_logits, nullptr, w13_q, w13_s, w13_z, w2_q, w2_s, w2_z, out, T,
                                    H, inter, E, topk, group, 0, renormalize, 1.f, workspace, workspace_bytes,
                                    stream);
}

int awqmi_fused_moe_routed_f16(const void* hidden, const float* router_logits, const float* score_bias,
                               const int32_t* w13_q, const void* w13_s, const int32_t* w13_z,
                               const int32_t* w2_q, const void* w2_s, const int32_t* w2_z, void* out, int T,
                               int H, int inter, int E, int topk, int group, int scoring, int renormalize,
                               float routed_scale, void* workspace, size_t workspace_bytes, void* stream) {
  if (!hidden || !router_logits || !w13_q || !w13_s || !w13_z || !w2_q || !w2_s || !w2_z || !out ||
      !workspace)
    return AWQMI_NULL_POINTER;
  if (T <= 0 || H <= 0 || inter <= 0 || E <= 0 || H % 8 != 0 || inter % 8 != 0) return AWQMI_BAD_SHAPE;
  if (topk <= 0 || topk > E || topk > 64 || E > AWQMI_MAX_EXPERTS || (long long)T * topk > (1LL << 30))
    return AWQMI_BAD_ARGUMENT;
  if ((scoring != 0 && scoring != 1) || (scoring == 0 && score_bias)) return AWQMI_BAD_ARGUMENT;
  if (!aligned16(workspace)) return AWQMI_BAD_ALIGN;
  const int tile = moe_pick_tile(T * topk, E, H, inter, group);
  const FusedMoeLayout L = fused_moe_layout(T, H, inter, E, topk, tile);
  if (workspace_bytes < L.total) return AWQMI_WORKSPACE_TOO_SMALL;
  char* ws = static_cast<char*>(workspace);
  int32_t* ids = reinterpret_cast<int32_t*>(ws + L.ids);
  float* wts = reinterpret_cast<float*>(ws + L.wts);
  int32_t* sorted = reinterpret_cast<int32_t*>(ws + L.sorted);
  int32_t* experts = reinterpret_cast<int32_t*>(ws + L.experts);
  int32_t* npp = reinterpret_cast<int32_t*>(ws + L.npp);
  void* h13 = ws + L.h13;
  void* act = ws + L.act;
  void* o = ws + L.o;
  int st;
  const MoeRoute route{router_logits, score_bias, T, E, topk, scoring, renormalize, routed_scale,
                       ids, wts, sorted, experts, npp};
  // a handful of tokens: the first expert GEMM takes the routing along (one launch less)
  const bool fold = moe_route_foldable(T, E, topk, tile);
  const MoeRoute* pending = fold ? &route : nullptr;
  if (fold) {
    // nothing to launch here
  } else if (L.n_slots < MOE_ALIGN_SPLIT_MIN || variant_on(VAR_ALIGN_ONE_WG)) {
    st = moe_route_launches(route, tile, stream);
    if (st) return st;
  } else {
    st = awqmi_moe_topk_f32(router_logits, score_bias, T, E, topk, scoring, renormalize, routed_scale, ids, wts,
                            stream);
    if (st) return st;
    // long slot lists: count per part, scan, place per part (three launches, many workgroups)
    if (const int rc = ensure_kernel_attributes()) return rc;
    int parts = (L.n_slots + 4095) / 4096;
    if (parts > MOE_ALIGN_PARTS_MAX) parts = MOE_ALIGN_PARTS_MAX;
    const int part = ((L.n_slots + parts - 1) / parts + 63) / 64 * 64;
    parts = (L.n_slots + part - 1) / part;
    int32_t* tab = reinterpret_cast<int32_t*>(ws + L.tab);
    const size_t lds = (size_t)(MOE_ALIGN_WAVES + 2) * E * sizeof(int);
    hipStream_t hs = (hipStream_t)stream;
    hipLaunchKernelGGL(moe_align_count_kernel, dim3(parts), dim3(1024), lds, hs, ids, L.n_slots, E, part, tab);
    hipLaunchKernelGGL(moe_align_scan_kernel, dim3(1), dim3(1024), (size_t)2 * E * sizeof(int), hs, L.n_slots, E,
                       tile, L.cap, parts, tab, sorted, experts, npp);
    hipLaunchKernelGGL(moe_align_place_kernel, dim3(parts), dim3(1024), lds, hs, ids, L.n_slots, E, part, tab,
                       sorted);
    st = launch_status();
    if (st) return st;
  }
  const int Gn = norm_group(H, group);
  if (tile == 16 && gemv_tiled_ok(H, Gn) && !variant_on(VAR_NO_FUSED_ACT) &&
      (moe_can_fuse_act(L.n_slots, E, H, 2 * inter) || moe_can_fuse_act_split(L.n_slots, E, H, 2 * inter))) {
    // the w13 GEMM writes silu(gate) * up itself: in one workgroup per gate / up block pair, or,
    // with few blocks (the launch is split in K), in the last arrivers of such a pair
    st = moe_gemm_impl(hidden, w13_q, w13_s, w13_z, act, sorted, experts, npp, nullptr, L.n_slots, topk, 16, E, H,
                       2 * inter, group, 0, ws + L.gemm_ws, L.gemm_ws_bytes, stream, true, pending);
    if (st) return st;
  } else {
    st = moe_gemm_impl(hidden, w13_q, w13_s, w13_z, h13, sorted, experts, npp, nullptr, L.n_slots, topk,
                       tile, E, H, 2 * inter, group, 0, ws + L.gemm_ws, L.gemm_ws_bytes, stream, false, pending);
    if (st) return st;
    st = awqmi_silu_and_mul_f16(h13, act, L.n_slots, inter, stream);
    if (st) return st;
  }
  st = awqmi_moe_gemm_f16(act, w2_q, w2_s, w2_z, o, sorted, experts, npp, wts, L.n_slots, 1, tile, E, inter, H,
                          group, 0, ws + L.gemm_ws, L.gemm_ws_bytes, stream);
  if (st) return st;
  return awqmi_moe_sum_f16(o, out, T, topk, H, stream);
}

int awqmi_workspace_reset(void* workspace, size_t workspace_bytes, void* stream) {
  if (!workspace) return AWQMI_NULL_POINTER;
  if (!aligned16(workspace)) return AWQMI_BAD_ALIGN;
  if (workspace_bytes < AWQMI_WS_COUNTER_BYTES) return AWQMI_WORKSPACE_TOO_SMALL;
  // a fill kernel rather than a memset node, so that the call behaves the same inside a capture
  hipLaunchKernelGGL(awq_zero_words_kernel, dim3(AWQMI_WS_COUNTER_BYTES / 16 / 256), dim3(256), 0,
                     (hipStream_t)stream, reinterpret_cast<u4v*>(workspace), AWQMI_WS_COUNTER_BYTES / 16);
  return launch_status();
}

// ---- development entry points (include/awq_mi355x_dev.h): the same calls with the launch-rule
// variant as an explicit argument, scoped to the call

int awqmi_dev_gemm_f16(const void* x, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                       void* y, void* workspace, size_t workspace_bytes, int M, int K, int N, int group,
                       int split_k, void* stream, int variant) {
  VariantScope scope(variant);
  return awqmi_gemm_f16(x, qweight, scales, qzeros, y, workspace, workspace_bytes, M, K, N, group, split_k, stream);
}

int awqmi_dev_last_gemm_form(void) { return t_last_gemm_form; }

int awqmi_dev_gemm_timeline_f16(const void* x, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                                void* y, void* workspace, size_t workspace_bytes, int M, int K, int N, int group,
                                int split_k, void* stream, unsigned long long* stamps, size_t stamps_bytes) {
  if (!stamps) return AWQMI_NULL_POINTER;
  if (M <= 0 || M > 16 || K <= 0 || N <= 0) return AWQMI_BAD_SHAPE;     // one dense skinny launch
  const int G = norm_group(K, group);
  if (check_awq_shape(K, N, G) != AWQMI_OK || !gemv_tiled_ok(K, G)) return AWQMI_BAD_SHAPE;
  const int split = split_k > 0 ? split_k : pick_split_k(M, K, N, G, 1, true);
  const size_t wgs = (size_t)((N / 8 + 16 * gemv_wpl(N) - 1) / (16 * gemv_wpl(N))) * split;
  if (stamps_bytes < wgs * 8 * sizeof(unsigned long long)) return AWQMI_WORKSPACE_TOO_SMALL;
  t_trace = stamps;
  const int rc = awqmi_gemm_f16(x, qweight, scales, qzeros, y, workspace, workspace_bytes, M, K, N, group, split_k, stream);
  t_trace = nullptr;
  return rc;
}

static inline int ldw_or(int nw, size_t pitch_words) { return pitch_words >= (size_t)nw ? (int)pitch_words : nw; }

int awqmi_dev_stream_probe(const void* src, void* out, int pattern, int K, int N, int parts, size_t total_bytes,
                           void* stream) {
  if (!src || !out) return AWQMI_NULL_POINTER;
  if (!aligned16(src) || !aligned16(out)) return AWQMI_BAD_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  if (pattern == 0 || pattern == 2) {
    // whole 128-byte lines per column block, whole 128-row chunks, at least one chunk per wave
    if (K <= 0 || N <= 0 || K % 128 != 0 || N % 256 != 0 || parts < 1 || (K / 128) < 4 * parts) return AWQMI_BAD_SHAPE;
    if ((size_t)(N / 256) * parts > 65535u * 4u) return AWQMI_BAD_SHAPE;
    if (pattern == 0)
      hipLaunchKernelGGL((awq_stream_probe_kernel<0>), dim3(N / 256, parts), dim3(256), 0, st,
                         reinterpret_cast<const uint32_t*>(src), reinterpret_cast<uint32_t*>(out), K, ldw_or(N / 8, total_bytes), parts, (size_t)0);
    else
      hipLaunchKernelGGL((awq_stream_probe_kernel<2>), dim3(N / 256, parts), dim3(256), 0, st,
                         reinterpret_cast<const uint32_t*>(src), reinterpret_cast<uint32_t*>(out), K, 32, parts, (size_t)0);
  } else if (pattern == 1) {
    if (total_bytes < (1u << 20) || total_bytes % 1024 != 0) return AWQMI_BAD_SHAPE;
    hipLaunchKernelGGL((awq_stream_probe_kernel<1>), dim3(256), dim3(256), 0, st, reinterpret_cast<const uint32_t*>(src),
                       reinterpret_cast<uint32_t*>(out), 0, 0, 1, total_bytes);
  } else {
    return AWQMI_BAD_ARGUMENT;
  }
  return launch_status();
}

int awqmi_dev_mfma_probe(const void* src, void* out, int shape, int iters, void* stream) {
  if (!src || !out) return AWQMI_NULL_POINTER;
  if (!aligned16(src) || !aligned16(out)) return AWQMI_BAD_ALIGN;
  if (iters <= 0 || (shape != 0 && shape != 1)) return AWQMI_BAD_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  if (shape == 0)
    hipLaunchKernelGGL((awq_mfma_probe_kernel<0>), dim3(256), dim3(256), 0, st, reinterpret_cast<const uint32_t*>(src),
                       reinterpret_cast<float*>(out), iters);
  else
    hipLaunchKernelGGL((awq_mfma_probe_kernel<1>), dim3(256), dim3(256), 0, st, reinterpret_cast<const uint32_t*>(src),
                       reinterpret_cast<float*>(out), iters);
  return launch_status();
}

size_t awqmi_dev_gemm_dense_workspace_bytes(int M, int K, int N) {
  if (M <= 0 || K <= 0 || N <= 0 || K % 64 != 0) return 0;
  const int slab = mfma_slab_rows(M, K);
  if (slab <= 0) return 0;
  size_t part = plan_mfma(slab, K, N, 256).part_bytes;
  if (M % slab) part = std::max(part, plan_mfma(M % slab, K, N, 256).part_bytes);
  return dense_panel_offset(part) + dg_panel_bytes(K, N);
}

int awqmi_dev_moe_gemm_f16(const void* x, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                           void* y, const int32_t* sorted_token_ids, const int32_t* expert_ids,
                           const int32_t* num_tokens_post_padded, const float* topk_weights, int n_slots,
                           int a_row_div, int tile_m, int E, int K, int N, int group, int split_k,
                           void* workspace, size_t workspace_bytes, void* stream, int variant) {
  VariantScope scope(variant);
  return awqmi_moe_gemm_f16(x, qweight, scales, qzeros, y, sorted_token_ids, expert_ids, num_tokens_post_padded,
                            topk_weights, n_slots, a_row_div, tile_m, E, K, N, group, split_k, workspace,
                            workspace_bytes, stream);
}

int awqmi_dev_fused_moe_routed_f16(const void* hidden, const float* router_logits, const float* score_bias,
                                   const int32_t* w13_q, const void* w13_s, const int32_t* w13_z,
                                   const int32_t* w2_q, const void* w2_s, const int32_t* w2_z, void* out, int T,
                                   int H, int inter, int E, int topk, int group, int scoring, int renormalize,
                                   float routed_scale, void* workspace, size_t workspace_bytes, void* stream,
                                   int variant) {
  VariantScope scope(variant);
  return awqmi_fused_moe_routed_f16(hidden, router_logits, score_bias, w13_q, w13_s, w13_z, w2_q, w2_s, w2_z, out,
                                    T, H, inter, E, topk, group, scoring, renormalize, routed_scale, workspace,
                                    workspace_bytes, stream);
}

int awqmi_dev_fused_moe_block_rows(int T, int H, int inter, int E, int topk, int group, int variant) {
  VariantScope scope(variant);
  return awqmi_fused_moe_block_rows(T, H, inter, E, topk, group);
}

}  // extern "C"
