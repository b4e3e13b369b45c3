/* awq_mi355x.h -- C ABI of libawq_mi355x.so: the AWQ W4A16 linear path for AMD MI355X
 * (gfx950), hand-written HIP kernels behind plain pointers and sizes.
 *
 * What it replaces.  The benchmark harness starts a vLLM OpenAI server
 * (reference utils/generate_compose.py:67 image, :85-93 server command) on AWQ checkpoints
 * (reference config.yaml:36,47,51,134); every quantised Linear / fused-MoE layer of that
 * server runs awq_dequantize / awq_gemm / the expert-grouped AWQ GEMM.  That code lives in
 * the docker image, not in the harness repository, so each entry point below cites the
 * harness call site that makes it run plus the operator name it stands in for.
 *
 * Conventions
 *   - All pointers are DEVICE pointers (HIP), row-major, densely packed.
 *   - AutoAWQ "GEMM" layout: qweight int32 [K, N/8], qzeros int32 [K/G, N/8],
 *     scales fp16 [K/G, N]; nibble i of a word at word-column c holds logical column
 *     8c + {0,2,4,6,1,3,5,7}[i].  W[k,n] = fp16((w - z) * s), one rounding.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *   - Every call validates on the host first and launches nothing on error; calls are
 *     asynchronous, never synchronise, never allocate and never keep a pointer, and can be
 *     captured in a HIP graph (grid sizes depend on shapes only).
 *   - Return value: AWQMI_OK or one of the awqmi_status codes below.
 */
#ifndef AWQ_MI355X_H
#define AWQ_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum awqmi_status {
  AWQMI_OK = 0,
  AWQMI_BAD_SHAPE = 1,           /* M/K/N/group relations violated                        */
  AWQMI_BAD_ALIGN = 2,           /* a pointer is not 16-byte aligned                      */
  AWQMI_WORKSPACE_TOO_SMALL = 3, /* workspace_bytes < awqmi_*_workspace_bytes(...)        */
  AWQMI_UNSUPPORTED_GROUP = 4,   /* group size the kernels do not cover                   */
  AWQMI_LAUNCH_FAILED = 5,       /* hipGetLastError() != 0, see awqmi_last_hip_error()    */
  AWQMI_NULL_POINTER = 6,
  AWQMI_BAD_ARGUMENT = 7,        /* split_k / tile_m / topk out of range                  */
  AWQMI_SCRATCH_LIMIT = 8        /* awqmi_gemm_f16_noalloc: needs > AWQMI_STATIC_SCRATCH_BYTES */
} awqmi_status;

#define AWQMI_VERSION 300        /* major*10000 + minor*100 + patch */
#define AWQMI_MOE_TILE_M 16      /* default rows per sorted-token block (32 also accepted)  */
#define AWQMI_MAX_SPLIT_K 64
#define AWQMI_MAX_EXPERTS 1024

/* Optional one-time set-up on the current device: raises the dynamic-LDS limit of the kernels
 * that need it, looks up this GPU's static scratch array (awqmi_gemm_f16_noalloc) and zeroes its
 * arrival counters (synchronously, on the null stream).  Every entry point does its share of
 * this on its first use; call this once per device after loading the library if the first use
 * on that device may sit inside a stream capture.  All set-up state is kept per device (the
 * harness starts one server process per replica and GPU set, reference
 * utils/generate_compose.py:85-100; a process that drives several GPUs makes each one current
 * for its own calls). */
int awqmi_init(void);
int awqmi_version(void);
const char* awqmi_status_string(int status);
/* hipError_t of the last AWQMI_LAUNCH_FAILED on the calling thread (0 if none). */
int awqmi_last_hip_error(void);

/* awq_dequantize(qweight, scales, zeros, split_k_iters, thx, thy) -> fp16 [K, N].
 * Stands in for vLLM's `awq_dequantize` op (taken by AWQLinearMethod.apply for large M);
 * reached from the server started at reference utils/generate_compose.py:85-93.
 * Any group with K % group == 0; N % 8 == 0.  Bit-exact fp16((w - z) * s). */
int awqmi_dequantize_f16(const int32_t* qweight, const void* scales_f16, const int32_t* qzeros,
                         void* out_f16, int K, int N, int group, void* stream);

/* Split-K factor the library would pick for this shape (>= 1). */
int awqmi_gemm_auto_split_k(int M, int K, int N, int group);

/* Bytes of workspace awqmi_gemm_f16 needs for this call (split_k == 0 means "auto").
 * The first AWQMI_WS_COUNTER_BYTES of the workspace are split-K arrival counters: they
 * must be zero before the first call and every call leaves them zero again, so one
 * zero-initialised buffer can be reused call after call on one stream.  Two calls that
 * overlap in time (different streams) need different workspaces. */
#define AWQMI_WS_COUNTER_BYTES 65536
size_t awqmi_gemm_workspace_bytes(int M, int K, int N, int split_k);

/* awq_gemm(input, qweight, scales, qzeros, split_k_iters) -> fp16 [M, N] = X @ W.
 * Stands in for vLLM's `awq_gemm` op (every AWQ Linear at decode and prefill); reached
 * from the server started at reference utils/generate_compose.py:85-93.
 * fp32 accumulation, one final rounding to fp16.  M >= 1; K % group == 0; N % 8 == 0.
 * M <= 32 takes the HBM-bound skinny kernel (split_k honoured, 0 = auto); 33 .. 48 rows take
 * two skinny passes on very wide layers and the MFMA kernel otherwise; larger M the
 * LDS-dequant MFMA kernel (split_k ignored; 64- / 128- / 192-row tiles up to M = 64 / 128 /
 * 192, 256-row tiles above;
 * when the workspace is at least awqmi_gemm_workspace_bytes() a sparsely filled last round
 * of tiles is split in K and a second short kernel sums the partial tiles, otherwise every
 * tile runs on one workgroup).  Shapes outside the fast kernels' tiling (K % 128 != 0, group
 * not in {32, 64, 128*i}) take a slow generic kernel. */
int awqmi_gemm_f16(const void* x_f16, const int32_t* qweight, const void* scales_f16,
                   const int32_t* qzeros, void* y_f16, void* workspace, size_t workspace_bytes,
                   int M, int K, int N, int group, int split_k, void* stream);

/* awqmi_gemm_f16 / awqmi_dequantize_f16 on a qweight whose rows are ldw int32 words apart in
 * memory (ldw == N / 8, or larger and a multiple of 4; the words past N / 8 of a row are never read).  This is
 * the form AWQLinearMethod.process_weights_after_loading hands over: vLLM's quantisation
 * methods re-lay their weights out for their kernels in that hook (reached when the server of
 * reference utils/generate_compose.py:85-93 loads a checkpoint), and this library's re-layout is
 * a row pitch that is not a multiple of eight 128-byte lines -- with such a pitch the skinny
 * kernel streams 12 - 20 % faster (every wave reads one line per row, and rows a multiple of
 * 1 KiB apart put all of a wave's requests on the same address bits 7 - 9).  qzeros and scales
 * stay contiguous.  With ldw == N / 8 these are awqmi_gemm_f16 / awqmi_dequantize_f16. */
int awqmi_gemm_ld_f16(const void* x_f16, const int32_t* qweight, int ldw, const void* scales_f16,
                      const int32_t* qzeros, void* y_f16, void* workspace, size_t workspace_bytes,
                      int M, int K, int N, int group, int split_k, void* stream);
int awqmi_dequantize_ld_f16(const int32_t* qweight, int ldw, const void* scales_f16,
                            const int32_t* qzeros, void* out_f16, int K, int N, int group, void* stream);

/* awqmi_gemm_f16 for callers that cannot allocate or carry a workspace: code under HIP graph
 * capture that has no buffer of its own, tight serving loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the harness or in vLLM's op surface (vLLM's awq_gemm allocates its
 * split-K buffer per call through torch).  Same arguments as awqmi_gemm_ld_f16 minus the
 * workspace (ldw = words between consecutive rows of qweight; 0 or N / 8 for a contiguous tensor, more
 * for the row-padded layout AWQLinearMethod keeps after loading); the split-K arrival counters and fp32 partial tiles live in a static device array
 * of AWQMI_STATIC_SCRATCH_BYTES inside the library (one copy per GPU, held until the process
 * ends), and results are bit-identical to awqmi_gemm_f16 with a zeroed workspace of that many
 * bytes.  The call allocates and frees nothing.
 *   - Rows up to 32 (the skinny kernel): a call whose split-K partial tiles do not fit returns
 *     AWQMI_SCRATCH_LIMIT and launches nothing.  With split_k = 0 every shape fits (at most
 *     8 MiB + the counters); only a large forced split_k on a wide layer does not.
 *   - More rows (the MFMA kernel): when the partial tiles of its K split do not fit, every
 *     tile runs on one workgroup, as awqmi_gemm_f16 does with a workspace of that size.
 *   - All calls on one GPU share that GPU's array: two calls that overlap in time on one GPU
 *     (different streams, or graphs replayed side by side) race on it; serialise them or give
 *     the others awqmi_gemm_f16 with their own workspace.
 *   - The array keeps the last call's partial tiles; only the counters must start at zero.
 *     They are zero when the library is loaded and every call that runs to completion leaves
 *     them so; awqmi_init() zeroes them again (use it after a call that was cut short).
 *   - The device address of the array is looked up on the first call on each GPU (or by
 *     awqmi_init() with that GPU current); the stream must belong to the current device. */
#define AWQMI_STATIC_SCRATCH_BYTES (AWQMI_WS_COUNTER_BYTES + (16u << 20))
int awqmi_gemm_f16_noalloc(const void* x_f16, const int32_t* qweight, int ldw, const void* scales_f16,
                           const int32_t* qzeros, void* y_f16, int M, int K, int N, int group,
                           int split_k, void* stream);

/* Router: softmax over E experts, top-k (ties: lowest expert id), optional renormalise.
 * Stands in for the fused-MoE routing step of the MoE AWQ models at reference
 * config.yaml:36,51,134.  logits fp32 [T, E]; ids int32 [T, topk]; weights fp32 [T, topk]. */
int awqmi_moe_topk_softmax_f32(const float* logits, int T, int E, int topk, int renormalize,
                               int32_t* topk_ids, float* topk_weights, void* stream);

/* Router with the scoring variants of the MoE checkpoints the harness serves
 * (reference config.yaml:36,47,51,134): scoring 0 = softmax (as above; score_bias must be
 * null), scoring 1 = sigmoid: score = sigmoid(logit), experts are chosen by
 * score + score_bias[e] (score_bias fp32 [E] or null), the weight is the score.  Weights are
 * optionally renormalised over the chosen experts, then multiplied by `scale` (a routed
 * scaling factor; 1 for none).  Ties go to the lowest expert id. */
int awqmi_moe_topk_f32(const float* logits, const float* score_bias, int T, int E, int topk, int scoring,
                       int renormalize, float scale, int32_t* topk_ids, float* topk_weights, void* stream);

/* Capacity (entries) of sorted_token_ids for n = T*topk routed slots; expert_ids needs
 * capacity / tile_m entries. */
size_t awqmi_moe_align_capacity(int n_slots, int E, int tile_m);

/* Stable sort of the flat (token, slot) indices by expert; each expert's run is padded to a
 * multiple of tile_m with the sentinel n_slots.  sorted_token_ids[capacity] (tail filled
 * with the sentinel), expert_ids[capacity / tile_m] (tail filled with -1),
 * num_tokens_post_padded[1].  Stands in for the align/sort step of fused MoE (same models).
 * Ids outside [0, E) are dropped (they appear nowhere in the output).  E <= 1024. */
int awqmi_moe_align(const int32_t* topk_ids, int n_slots, int E, int tile_m,
                    int32_t* sorted_token_ids, int32_t* expert_ids,
                    int32_t* num_tokens_post_padded, void* stream);

/* Workspace bytes of one grouped GEMM call (same counter rule as awqmi_gemm_f16). */
size_t awqmi_moe_gemm_workspace_bytes(int n_slots, int E, int K, int N, int split_k, int tile_m);

/* Expert-grouped AWQ GEMM over sorted-token blocks of tile_m rows; the ids must come from
 * awqmi_moe_align with the same tile_m.  tile_m 16 or 32: the skinny kernel (decode-sized
 * batches).  tile_m 64, 128 or 256: the MFMA kernel, for many slots per expert; it takes no
 * split_k or workspace and needs x and each expert's tensors under 4 GiB.
 * For every non-pad entry s = sorted_token_ids[i] in a block owned by expert e:
 *     y[s, :] = (x[s / a_row_div, :] @ W_e) * (topk_weights ? topk_weights[s] : 1)
 * a_row_div = topk for the first GEMM (x is [T, K]), 1 for the second (x is [n_slots, K]).
 * Weights carry a leading expert dimension: qweight [E, K, N/8], scales [E, K/G, N],
 * qzeros [E, K/G, N/8].  y is fp16 [n_slots, N].  Rows of y whose slot was dropped by the
 * align step are not written.  Stands in for the fused-MoE expert GEMMs (same models). */
int awqmi_moe_gemm_f16(const void* x_f16, const int32_t* qweight, const void* scales_f16,
                       const int32_t* qzeros, void* y_f16, const int32_t* sorted_token_ids,
                       const int32_t* expert_ids, const int32_t* num_tokens_post_padded,
                       const float* topk_weights, int n_slots, int a_row_div, int tile_m, int E, int K,
                       int N, int group, int split_k, void* workspace, size_t workspace_bytes,
                       void* stream);

/* out[r, i] = silu(in[r, i]) * in[r, inter + i], in fp16 [rows, 2*inter] ([gate | up]),
 * out fp16 [rows, inter]; fp32 math.  The activation between the two expert GEMMs. */
int awqmi_silu_and_mul_f16(const void* in_f16, void* out_f16, int rows, int inter, void* stream);

/* out[t, :] = sum over the topk slot rows in[t*topk + j, :], fp32 sum, fp16 out. */
int awqmi_moe_sum_f16(const void* in_f16, void* out_f16, int T, int topk, int H, void* stream);

/* One whole AWQ MoE block in one call: softmax + top-k routing, align, grouped w13 GEMM,
 * SiLU(gate) * up, grouped w2 GEMM scaled by the routing weights, sum over each token's
 * slots.  Replaces the sequence fused_topk -> moe_align_block_size -> fused_experts that
 * the AWQ MoE method runs (vLLM model_executor/layers/quantization/awq.py, AWQMoEMethod.apply ->
 * layers/fused_moe/fused_moe.py fused_experts; the harness reaches it through
 * docker-compose.vllm.yml:13-16 with an AWQ MoE checkpoint).
 *   hidden fp16 [T, H]; router_logits fp32 [T, E]; out fp16 [T, H]
 *   w13: qweight int32 [E, H, 2*inter/8], scales fp16 [E, H/G, 2*inter], qzeros int32 [E, H/G, 2*inter/8]
 *        (columns [gate | up]);  w2: [E, inter, H/8], [E, inter/G, H], [E, inter/G, H/8]
 * Every intermediate lives in the workspace (awqmi_fused_moe_workspace_bytes), which must be
 * zero-initialised once; the call itself allocates nothing and is safe to capture in a HIP
 * graph.  H and inter must be multiples of 128 with group in {32, 64, 128 * i}. */
size_t awqmi_fused_moe_workspace_bytes(int T, int H, int inter, int E, int topk);
/* Sorted-token block rows awqmi_fused_moe_f16 uses for these shapes: 16 (skinny kernel) or
 * 64 / 128 / 256 (MFMA kernel, prefill-sized batches).  A query like awqmi_gemm_auto_split_k;
 * 0 for shapes the call would refuse. */
int awqmi_fused_moe_block_rows(int T, int H, int inter, int E, int topk, int group);
int awqmi_fused_moe_f16(const void* hidden_f16, const float* router_logits, const int32_t* w13_qweight,
                        const void* w13_scales_f16, const int32_t* w13_qzeros,
                        const int32_t* w2_qweight, const void* w2_scales_f16, const int32_t* w2_qzeros,
                        void* out_f16, int T, int H, int inter, int E, int topk, int group,
                        int renormalize, void* workspace, size_t workspace_bytes, void* stream);

/* The same block with the routing of awqmi_moe_topk_f32: scoring 0 = softmax, 1 = sigmoid with an
 * optional score-correction bias fp32 [E] in the selection key (NULL for none; not allowed with
 * softmax), weights optionally renormalised and multiplied by routed_scale.  Stands in for the
 * same AWQMoEMethod.apply with scoring_func / e_score_correction_bias / routed_scaling_factor
 * set (the sigmoid-routed MoE checkpoints of reference config.yaml:51).  Workspace as above. */
int awqmi_fused_moe_routed_f16(const void* hidden_f16, const float* router_logits, const float* score_bias,
                               const int32_t* w13_qweight, const void* w13_scales_f16,
                               const int32_t* w13_qzeros, const int32_t* w2_qweight,
                               const void* w2_scales_f16, const int32_t* w2_qzeros, void* out_f16, int T,
                               int H, int inter, int E, int topk, int group, int scoring, int renormalize,
                               float routed_scale, void* workspace, size_t workspace_bytes, void* stream);

/* Zeroes the arrival-counter prefix (AWQMI_WS_COUNTER_BYTES) of a workspace, with a small fill
 * kernel on `stream` (no memset node: safe to capture).  Every call of this library leaves the
 * counters at zero when its kernels run to completion; a binding calls this before it reuses a
 * workspace after anything cut a call short: a launch that failed or was aborted (device
 * error, a destroyed stream or graph, a process that reuses a buffer it did not zero).  No
 * counterpart in vLLM's op surface (its split-K sums need no counters); part of the workspace
 * contract of awqmi_gemm_f16 / awqmi_moe_gemm_f16 / awqmi_fused_moe_f16. */
int awqmi_workspace_reset(void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AWQ_MI355X_H */
