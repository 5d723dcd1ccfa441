/*
 * CPU oracle in plain C for the W3 path (TEST INFRASTRUCTURE: the checker and the CPU baseline, never shipped or
 * called by the product path).
 *
 * Restates, from the reference (paths relative to its tree):
 *   w3o_codes       hibana/kernels/w3.py:217-229   the unpack: bit b of code[n, k] is bit (4j + b + rot(s)) mod 32 of
 *                                                  word bits*nt + b of lane 4g + t (:12-19, :178-191)
 *   w3o_dequantize  hibana/kernels/w3.py:232-242   level[code] * (float(e4m3 scale) * row_scale[n]), two FP32 products
 *   w3o_moe_layer   hibana/kernels/w3_moe.py:193-214 with an identity activation rounding (weight-only) plus the shared
 *                   expert and combine of hibana/model/flashnext/moe.py:177-192 /
 *                   hibana/kernels/flashnext_fused.py:530-571: per distinct expert, dequantize fc1 and fc2, h1 = bf16(x W13^T),
 *                   h = bf16(silu(gate) * up) or bf16(relu(h1)^2), y = h W2^T in FP32; out = bf16(fma chain over the slots)
 *                   [+ g * bf16(shared)], rounded once more.
 * Pinned by tests/test_oracle_c.py against oracle/w3_format.py (bit-exact) and oracle/layers.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

static float e4m3_to_float(uint8_t b) {
  const int sign = b >> 7, e = (b >> 3) & 15, m = b & 7;
  float v;
  if (e == 0) v = ldexpf((float)m, -9);
  else if (e == 15 && m == 7) v = NAN;
  else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return sign ? -v : v;
}

static float bf16_round(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return f;
  u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
  memcpy(&f, &u, 4);
  return f;
}

static float bf16_bits_to_float(uint16_t h) {
  const uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static uint16_t float_to_bf16_bits(float f) {
  f = bf16_round(f);
  uint32_t u;
  memcpy(&u, &f, 4);
  return (uint16_t)(u >> 16);
}

/* planes uint32 [rows/32, K/128, bits, 32, 4] -> codes uint8 [rows, K] */
void w3o_codes(const uint32_t* planes, int64_t rows, int k, int bits, uint8_t* codes) {
  const int chunks = k / 128;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < rows; n++) {
    const int64_t nb = n / 32;
    const int nt = (int)(n % 32) / 8, g = (int)(n % 8);
    for (int kk = 0; kk < k; kk++) {
      const int kc = kk / 128, s = (kk % 128) / 16, t = (kk % 16) / 4, j = kk % 4;
      const int rot = 16 * (s / 4) + s % 4;
      int code = 0;
      for (int b = 0; b < bits; b++) {
        const int w = bits * nt + b;
        const uint32_t word = planes[(((nb * chunks + kc) * bits + w / 4) * 32 + (4 * g + t)) * 4 + w % 4];
        code |= (int)((word >> ((4 * j + b + rot) % 32)) & 1u) << b;
      }
      codes[n * k + kk] = (uint8_t)code;
    }
  }
}

/* -> float32 [rows, K]; levels: the codebook (8 floats, unused entries zero) */
void w3o_dequantize(const uint32_t* planes, const uint8_t* scales, const float* row_scale, const float* levels, int64_t rows, int k, int bits,
                    float* out) {
  const int chunks = k / 128;
  uint8_t* codes = (uint8_t*)malloc((size_t)rows * k);
  w3o_codes(planes, rows, k, bits, codes);
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < rows; n++) {
    const int64_t nb = n / 32;
    const int nt = (int)(n % 32) / 8;
    for (int grp = 0; grp < k / 32; grp++) {
      const uint8_t byte = scales[((nb * chunks + grp / 4) * 4 + (n % 8) / 2) * 32 + (4 * nt + grp % 4) * 2 + n % 2];
      const float eff = e4m3_to_float(byte) * row_scale[n];
      for (int i = 0; i < 32; i++) out[n * k + grp * 32 + i] = levels[codes[n * k + grp * 32 + i]] * eff;
    }
  }
  free(codes);
}

/* y[r, n] = sum_k a[r, k] * w[n, k], FP32 accumulation in eight interleaved partial sums (vectorizable) */
static void rows_times_matrix(const float* a, int rows, const float* w, int n_out, int k, float* y) {
#pragma omp parallel for schedule(static)
  for (int n = 0; n < n_out; n++) {
    const float* wr = w + (size_t)n * k;
    for (int r = 0; r < rows; r++) {
      const float* ar = a + (size_t)r * k;
      float part[8] = {0};
      for (int kk = 0; kk < k; kk += 8)
        for (int i = 0; i < 8; i++) part[i] += ar[kk + i] * wr[kk + i];
      y[(size_t)r * n_out + n] = ((part[0] + part[4]) + (part[1] + part[5])) + ((part[2] + part[6]) + (part[3] + part[7]));
    }
  }
}

typedef struct {
  const uint32_t* planes13; const uint8_t* scales13; const float* row13;  /* stacked [E, n1, hidden], fc1 rows in fc1_order */
  const uint32_t* planes2; const uint8_t* scales2; const float* row2;     /* stacked [E, hidden, inter] */
  const float* levels13; const float* levels2;
  int experts, base, hidden, inter, gated;
} w3o_experts;

/* Seconds the last w3o_moe_layer call spent unpacking weights (w3o_dequantize), so that a caller that times the whole
 * call also has the matmul-and-the-rest part: total minus this. */
static double unpack_seconds = 0.0;
double w3o_last_unpack_seconds(void) { return unpack_seconds; }
static double now_seconds(void) {
  struct timespec t;
  clock_gettime(CLOCK_MONOTONIC, &t);
  return (double)t.tv_sec + 1e-9 * (double)t.tv_nsec;
}

/* one expert on `rows` gathered activation rows xs [rows, hidden] (float) -> y [rows, hidden] (float) */
static void one_expert(const w3o_experts* ex, int e, const float* xs, int rows, float* y, float* w13, float* w2, float* h1, float* h) {
  const int n1 = ex->gated ? 2 * ex->inter : ex->inter, hd = ex->hidden, it = ex->inter;
  const double t0 = now_seconds();
  w3o_dequantize(ex->planes13 + (size_t)e * n1 / 32 * (hd / 128) * 3 * 128, ex->scales13 + (size_t)e * n1 / 32 * (hd / 128) * 128,
                 ex->row13 + (size_t)e * n1, ex->levels13, n1, hd, 3, w13);
  w3o_dequantize(ex->planes2 + (size_t)e * hd / 32 * (it / 128) * 3 * 128, ex->scales2 + (size_t)e * hd / 32 * (it / 128) * 128,
                 ex->row2 + (size_t)e * hd, ex->levels2, hd, it, 3, w2);
  unpack_seconds += now_seconds() - t0;
  rows_times_matrix(xs, rows, w13, n1, hd, h1);
  for (int r = 0; r < rows; r++)
    for (int c = 0; c < it; c++) {
      float v;
      if (ex->gated) { /* fc1_order: block b of 32 rows = up 16b..16b+15, then gate 16b..16b+15 */
        const int b = c / 16, o = c % 16;
        const float up = bf16_round(h1[(size_t)r * n1 + 32 * b + o]), gate = bf16_round(h1[(size_t)r * n1 + 32 * b + 16 + o]);
        v = gate / (1.0f + expf(-gate)) * up;
      } else {
        const float u = fmaxf(bf16_round(h1[(size_t)r * n1 + c]), 0.0f);
        v = u * u;
      }
      h[(size_t)r * it + c] = bf16_round(v);
    }
  rows_times_matrix(h, rows, w2, hd, it, y);
}

/* x BF16 bits [m, hidden]; ids int32 [m, topk]; weights float [m, topk]; shared: one expert or NULL; gate_vec float [hidden] or NULL;
 * out BF16 bits [m, hidden]. Returns the number of distinct experts run (the shared one not counted). */
int w3o_moe_layer(const w3o_experts* ex, const w3o_experts* shared, const float* gate_vec, const uint16_t* x, const int32_t* ids,
                  const float* weights, int m, int topk, uint16_t* out) {
  const int hd = ex->hidden, it = ex->inter, n1 = ex->gated ? 2 * it : it;
  unpack_seconds = 0.0;
  float* xf = (float*)malloc((size_t)m * hd * 4);
  for (size_t i = 0; i < (size_t)m * hd; i++) xf[i] = bf16_bits_to_float(x[i]);
  float* pairs = (float*)calloc((size_t)m * topk * hd, 4);
  float* w13 = (float*)malloc((size_t)n1 * hd * 4);
  float* w2 = (float*)malloc((size_t)hd * it * 4);
  float* xs = (float*)malloc((size_t)m * topk * hd * 4);
  float* h1 = (float*)malloc((size_t)m * topk * n1 * 4);
  float* h = (float*)malloc((size_t)m * topk * it * 4);
  float* y = (float*)malloc((size_t)m * topk * hd * 4);
  int* which = (int*)malloc((size_t)m * topk * sizeof(int));
  int distinct = 0;
  for (int e = 0; e < ex->experts; e++) { /* ascending expert id; an expert's pairs in ascending pair index */
    int rows = 0;
    for (int q = 0; q < m * topk; q++)
      if (ids[q] - ex->base == e) {
        memcpy(xs + (size_t)rows * hd, xf + (size_t)(q / topk) * hd, (size_t)hd * 4);
        which[rows++] = q;
      }
    if (!rows) continue;
    distinct++;
    one_expert(ex, e, xs, rows, y, w13, w2, h1, h);
    for (int r = 0; r < rows; r++) memcpy(pairs + (size_t)which[r] * hd, y + (size_t)r * hd, (size_t)hd * 4);
  }
  float* sh = NULL;
  if (shared) {
    sh = (float*)malloc((size_t)m * hd * 4);
    float* h1s = (float*)malloc((size_t)m * n1 * 4);
    float* hs = (float*)malloc((size_t)m * it * 4);
    one_expert(shared, 0, xf, m, sh, w13, w2, h1s, hs);
    free(h1s);
    free(hs);
  }
  for (int r = 0; r < m; r++) {
    float g = 1.0f;
    if (shared && gate_vec) {
      double dot = 0;
      for (int c = 0; c < hd; c++) dot += (double)xf[(size_t)r * hd + c] * gate_vec[c];
      g = 1.0f / (1.0f + expf(-(float)dot));
    }
    for (int c = 0; c < hd; c++) {
      float v = 0.0f;
      for (int s = 0; s < topk; s++) {
        const int e = ids[r * topk + s] - ex->base;
        if (e < 0 || e >= ex->experts) continue;
        v = fmaf(weights[r * topk + s], pairs[((size_t)r * topk + s) * hd + c], v);
      }
      if (shared) v = bf16_round(v) + g * bf16_round(sh[(size_t)r * hd + c]);
      out[(size_t)r * hd + c] = float_to_bf16_bits(v);
    }
  }
  free(xf); free(pairs); free(w13); free(w2); free(xs); free(h1); free(h); free(y); free(which); free(sh);
  return distinct;
}

/* dense: y BF16 bits [m, n] = bf16(x W_deq^T) */
void w3o_linear(const uint32_t* planes, const uint8_t* scales, const float* row_scale, const float* levels, int n, int k, int bits,
                const uint16_t* x, int m, uint16_t* y) {
  float* w = (float*)malloc((size_t)n * k * 4);
  float* xf = (float*)malloc((size_t)m * k * 4);
  float* yf = (float*)malloc((size_t)m * n * 4);
  w3o_dequantize(planes, scales, row_scale, levels, n, k, bits, w);
  for (size_t i = 0; i < (size_t)m * k; i++) xf[i] = bf16_bits_to_float(x[i]);
  rows_times_matrix(xf, m, w, n, k, yf);
  for (size_t i = 0; i < (size_t)m * n; i++) y[i] = float_to_bf16_bits(yf[i]);
  free(w); free(xf); free(yf);
}
