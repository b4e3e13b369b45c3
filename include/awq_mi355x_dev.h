/* awq_mi355x_dev.h -- development entry points of libawq_mi355x.so.
 *
 * Each is an entry point of awq_mi355x.h with one more argument, `variant`, that switches single
 * launch rules of that one call off or forces them (-1 = every default, i.e. exactly the public
 * entry point).  The variant is an argument, not a setting: it lives for the duration of the
 * call on the calling thread and nothing else in the library can observe it, so these are as
 * re-entrant as the calls they wrap.  They exist so that tests can push inputs through kernel
 * forms the default rules would not pick for a small shape, and so that two forms can be timed
 * side by side; bindings have no use for them.  They have no counterpart in the harness or in
 * vLLM's op surface.
 *
 * Bits of `variant` (a value >= 0):
 *   1        one packed word per lane in the skinny kernel for every N
 *   2        MoE launches with the dense kernel's register ring of four steps
 *   4|8|16   v = bits 2..4: runs of 1 << (v - 1) sorted-token blocks per XCD
 *   64       never two column blocks per workgroup
 *   512      64- / 128-row MFMA tiles with four waves instead of eight
 *   1024     the one-call MoE block always runs the separate activation kernel
 *   2048     the one-call MoE block always uses 16-row blocks
 *   4096     every launch keeps the weight ring in registers (no LDS ring)
 *   16384    the align step always runs in one workgroup
 *   1 << 16  v = bits 16..17: the one-call MoE block uses 64 / 128 / 256-row blocks (v = 1 / 2 / 3)
 *   1 << 18  awq_gemm with 17..64 rows: skinny passes wherever they can run
 *   1 << 19  awq_gemm with 17..64 rows: the MFMA kernel wherever it can run
 *   1 << 20  v = bits 20..22: MFMA tiles of 64 v rows (v = 1..4) whatever M is
 *   1 << 23  dense skinny launches never share left-over chunks step by step
 *   1 << 24  the one-call MoE block always routes in a launch of its own (blocks of at most four
 *            tokens otherwise fold the routing into the first expert GEMM)
 *   1 << 25  awq_gemm never takes the dequantise-once form (many-row calls run the fused kernel)
 *   1 << 26  awq_gemm takes the dequantise-once form from 257 rows on, when the workspace holds
 *            awqmi_dev_gemm_dense_workspace_bytes()
 *   1 << 27  expert GEMMs over 32-row sorted-token blocks (tile_m = 32) in the older form with two
 *            packed words per lane and one workgroup per CU (default for tile_m = 32 without a K
 *            split: one word per lane, two 128-column blocks per workgroup, weight ring in LDS, two
 *            workgroups per CU; with 4096 its ring stays in registers)
 * The workspace must be large enough for the form that is forced: the sizes the public queries
 * return cover every variant except a forced MFMA tile size, which silently runs without its K
 * split when the workspace is too small for it.
 */
#ifndef AWQ_MI355X_DEV_H
#define AWQ_MI355X_DEV_H

#include "awq_mi355x.h"

#ifdef __cplusplus
extern "C" {
#endif

int awqmi_dev_gemm_f16(const void* x_f16, const int32_t* qweight, const void* scales_f16,
                       const int32_t* qzeros, void* y_f16, void* workspace, size_t workspace_bytes,
                       int M, int K, int N, int group, int split_k, void* stream, int variant);

/* Kernel family the last awqmi_gemm_* call on the calling thread launched. */
enum {
  AWQMI_FORM_NONE = 0,
  AWQMI_FORM_SKINNY = 1,  /* awq_gemv_kernel: up to 32 rows per pass */
  AWQMI_FORM_FUSED = 2,   /* awq_gemm_mfma_kernel: weights dequantised per tile in LDS */
  AWQMI_FORM_DENSE = 3,   /* awq_dequant_panel_kernel + awq_gemm_dense_kernel */
  AWQMI_FORM_GENERIC = 4  /* any-shape fallback */
};
int awqmi_dev_last_gemm_form(void);

/* Workspace bytes with which a call of this shape can take the dequantise-once form (counters,
 * K-split partial tiles, fp16 panel); 0 when the shape cannot (K % 64 != 0). */
size_t awqmi_dev_gemm_dense_workspace_bytes(int M, int K, int N);

/* Measurement probes (no counterpart anywhere: they exist so that the ceilings the kernels are
 * priced against are measured on the machine).
 * awqmi_dev_stream_probe: a read-only pass with the arithmetic removed.  pattern 0 reads an int32
 * [K, N / 8] matrix the way the skinny GEMM kernel reads qweight (workgroup = 256 columns x one
 * of `parts` K ranges, one 128-byte line per row and 16 lanes, four 32-row steps in flight per
 * wave; K % 128 == 0, N % 256 == 0, K / 128 >= 4 parts; `out` takes (N / 256) * parts * 256 words;
 * total_bytes, when not 0, is the row pitch in words of a row-padded matrix); pattern 2 is pattern 0
 * on a column-block-major copy of the matrix (the K x 128 bytes of every 256-column block contiguous);
 * pattern 1 reads total_bytes linearly (256 workgroups, 1 KiB per wave instruction, 16 KiB in
 * flight per wave; `out` takes 65536 words).
 * awqmi_dev_mfma_probe: 256 workgroups x 4 waves, each a bare loop of fp16 MFMAs over a 128 x 128
 * accumulator tile with two alternating fragment sets taken from `src` (16 MiB of fp16 values);
 * shape 0 = v_mfma_f32_32x32x16_f16, shape 1 = v_mfma_f32_16x16x32_f16; one iteration is 2097152
 * flop per wave; `out` takes 65536 floats. */
int awqmi_dev_stream_probe(const void* src, void* out, int pattern, int K, int N, int parts, size_t total_bytes,
                           void* stream);
int awqmi_dev_mfma_probe(const void* src, void* out, int shape, int iters, void* stream);

/* awqmi_gemm_f16 for one decode-sized call (M <= 16) that also records, per workgroup, seven
 * time stamps of a constant 100 MHz counter at the kernel's phase boundaries (stamps[8 w + k] for
 * workgroup w = part * column_blocks + column_block: 0 start, 1 main loop left, 2 cross-wave sum
 * in LDS done, 3 partial stores acknowledged, 4 arrival counted, 5 last arriver: partials summed,
 * 6 output stored; 3 - 5 only in split-K launches, 5 - 6 only in the finishing workgroup).  The
 * buffer must be zeroed by the caller and hold 8 words per workgroup. */
int awqmi_dev_gemm_timeline_f16(const void* x_f16, const int32_t* qweight, const void* scales_f16,
                                const int32_t* qzeros, void* y_f16, void* workspace, size_t workspace_bytes,
                                int M, int K, int N, int group, int split_k, void* stream,
                                unsigned long long* stamps, size_t stamps_bytes);

int awqmi_dev_moe_gemm_f16(const void* x_f16, const int32_t* qweight, const void* scales_f16,
                           const int32_t* qzeros, void* y_f16, const int32_t* sorted_token_ids,
                           const int32_t* expert_ids, const int32_t* num_tokens_post_padded,
                           const float* topk_weights, int n_slots, int a_row_div, int tile_m, int E, int K,
                           int N, int group, int split_k, void* workspace, size_t workspace_bytes,
                           void* stream, int variant);

int awqmi_dev_fused_moe_routed_f16(const void* hidden_f16, const float* router_logits, const float* score_bias,
                                   const int32_t* w13_qweight, const void* w13_scales_f16,
                                   const int32_t* w13_qzeros, const int32_t* w2_qweight,
                                   const void* w2_scales_f16, const int32_t* w2_qzeros, void* out_f16, int T,
                                   int H, int inter, int E, int topk, int group, int scoring, int renormalize,
                                   float routed_scale, void* workspace, size_t workspace_bytes, void* stream,
                                   int variant);

int awqmi_dev_fused_moe_block_rows(int T, int H, int inter, int E, int topk, int group, int variant);

#ifdef __cplusplus
}
#endif
#endif /* AWQ_MI355X_DEV_H */
