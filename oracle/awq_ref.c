/* Scalar C restatement of the AWQ W4A16 linear path.  TEST INFRASTRUCTURE, NOT PRODUCT.
 *
 * A second, independent derivation of the same closed form as awq_ref.py (its own
 * fp16<->fp32 conversion, its own nibble arithmetic); the two must agree bit for bit
 * before either is trusted.  The reference harness holds no source for this arithmetic:
 * it runs inside docker image vllm/vllm-openai:latest
 * (/root/reference/utils/generate_compose.py:67, server flags :85-93) on the AWQ
 * checkpoints named at /root/reference/config.yaml:36,47,51,134.  Layout: AutoAWQ "GEMM"
 * (qweight [K, N/8], qzeros [K/G, N/8], scales [K/G, N]); nibble i of a packed word holds
 * logical column 8c + P[i], P = {0,2,4,6,1,3,5,7}.
 *
 * Parity status: unpack / dequantize / gemm / moe_align are pinned by the known-answer and
 * brute-force tests in tests/test_oracle.py; nothing here is pinned by a reference-side
 * golden vector because the reference has none for this path.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static const int AWQ_R[8] = {0, 4, 1, 5, 2, 6, 3, 7}; /* logical j -> nibble */

static float h2f(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; ++e; } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* round-to-nearest-even float -> half, subnormals and overflow handled */
static uint16_t f2h(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t absx = x & 0x7FFFFFFFu;
  if (absx >= 0x7F800000u) /* inf / nan */
    return (uint16_t)(sign | 0x7C00u | ((absx > 0x7F800000u) ? 0x200u : 0));
  if (absx >= 0x477FF000u) /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7C00u);
  if (absx < 0x33000001u) /* < 2^-25 (or exactly 2^-25 -> ties to even 0) */
    return sign;
  int e = (int)(absx >> 23) - 127;
  uint32_t m = (absx & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
  int shift = (e >= -14) ? 13 : (13 + (-14 - e)); /* bits to drop */
  uint32_t keep = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (keep & 1u))) ++keep;
  if (e >= -14) {
    /* keep has the implicit bit at position 10 (or 11 after carry) */
    uint32_t hbits = ((uint32_t)(e + 15) << 10) + (keep - 0x400u);
    return (uint16_t)(sign | hbits);
  }
  return (uint16_t)(sign | keep); /* subnormal (carry into normal is automatic) */
}

static inline int nib(uint32_t word, int j) { return (int)((word >> (4 * AWQ_R[j])) & 0xFu); }

void awqref_unpack(const int32_t* words, uint8_t* out, long rows, long cols8) {
  for (long r = 0; r < rows; ++r)
    for (long c = 0; c < cols8; ++c) {
      uint32_t q = (uint32_t)words[r * cols8 + c];
      for (int j = 0; j < 8; ++j) out[(r * cols8 + c) * 8 + j] = (uint8_t)nib(q, j);
    }
}

void awqref_dequantize(const int32_t* qweight, const uint16_t* scales, const int32_t* qzeros,
                       uint16_t* out, long K, long N, long G) {
  long NW = N / 8;
  for (long k = 0; k < K; ++k) {
    long g = k / G;
    for (long c = 0; c < NW; ++c) {
      uint32_t q = (uint32_t)qweight[k * NW + c];
      uint32_t zq = (uint32_t)qzeros[g * NW + c];
      for (int j = 0; j < 8; ++j) {
        float d = (float)(nib(q, j) - nib(zq, j));
        out[k * N + c * 8 + j] = f2h(d * h2f(scales[g * N + c * 8 + j]));
      }
    }
  }
}

/* Y = fp16_rn( sum_k float(x) * float(W) ), accumulation in double (wider than the fp32
 * the product path uses, so it serves as the tolerance anchor). */
void awqref_gemm(const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
                 const int32_t* qzeros, uint16_t* y, double* y_wide, long M, long K, long N,
                 long G) {
  uint16_t* W = (uint16_t*)malloc((size_t)K * N * sizeof(uint16_t));
  awqref_dequantize(qweight, scales, qzeros, W, K, N, G);
  double* acc = (double*)malloc((size_t)N * sizeof(double));
  for (long m = 0; m < M; ++m) {
    for (long n = 0; n < N; ++n) acc[n] = 0.0;
    for (long k = 0; k < K; ++k) {
      double xv = (double)h2f(x[m * K + k]);
      if (xv == 0.0) continue;
      const uint16_t* wr = W + k * N;
      for (long n = 0; n < N; ++n) acc[n] += xv * (double)h2f(wr[n]);
    }
    for (long n = 0; n < N; ++n) {
      if (y) y[m * N + n] = f2h((float)acc[n]);
      if (y_wide) y_wide[m * N + n] = acc[n];
    }
  }
  free(acc);
  free(W);
}

/* Stable counting sort of flat (token, slot) indices by expert; each expert's run padded
 * to a multiple of tile_m with sentinel n.  Returns the padded length. */
long awqref_moe_align(const int32_t* topk_ids, long n, long E, long tile_m, int32_t* sorted_ids,
                      int32_t* expert_ids) {
  long* cnt = (long*)calloc((size_t)E, sizeof(long));
  long* start = (long*)calloc((size_t)E, sizeof(long));
  for (long i = 0; i < n; ++i) cnt[topk_ids[i]]++;
  long pos = 0, blk = 0;
  for (long e = 0; e < E; ++e) {
    start[e] = pos;
    long nb = (cnt[e] + tile_m - 1) / tile_m;
    for (long b = 0; b < nb; ++b) expert_ids[blk++] = (int32_t)e;
    for (long i = 0; i < nb * tile_m; ++i) sorted_ids[pos + i] = (int32_t)n;
    pos += nb * tile_m;
  }
  for (long i = 0; i < n; ++i) sorted_ids[start[topk_ids[i]]++] = (int32_t)i;
  free(cnt);
  free(start);
  return pos;
}

/* exposed for the conversion tests */
uint16_t awqref_f2h(float f) { return f2h(f); }
float awqref_h2f(uint16_t h) { return h2f(h); }
