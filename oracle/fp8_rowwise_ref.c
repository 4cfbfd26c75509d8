/*
 * Plain-C restatement of the row-wise FP8 GEMM path. TEST INFRASTRUCTURE ONLY: linked by
 * tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg, never by the product.
 *
 * Follows tritonbench/operators/fp8_gemm_rowwise/operator.py:
 *   oracle_quantize_rows   :136-145 (fp32 input; scale = (1 / max(amax, 1e-12)) * 448, clamp,
 *                          round-to-nearest-even cast to e4m3fn, inverse scale = 1/scale)
 *   oracle_gemm            the contract of the callables at :187-217,
 *                          C = bf16((A . B^T) * a_scale * b_scale + bias), accumulated in
 *                          double so it is an independent check of the fp32 torch oracle
 * Built with -ffp-contract=off so every fp32 operation rounds once, as torch's CPU kernels do.
 *
 * Pinned by tests/test_oracle_*.py against the numpy codec, torch's e4m3fn cast and the
 * float64 numpy brute force.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

float oracle_e4m3_decode(uint8_t code) {
  const int s = code >> 7, e = (code >> 3) & 15, m = code & 7;
  float v;
  if (e == 15 && m == 7) return NAN;
  if (e == 0) v = ldexpf((float)m, -9);
  else v = ldexpf((float)(8 + m), e - 10);
  return s ? -v : v;
}

/* fp32 -> e4m3fn, nearest even, NaN past the last finite code (no saturation). */
uint8_t oracle_e4m3_encode(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  const uint8_t sign = (uint8_t)((u >> 24) & 0x80);
  if (isnan(f)) return sign | 0x7f;
  const float a = fabsf(f);
  if (a < 0x1p-6f) return sign | (uint8_t)nearbyintf(a * 512.0f); /* default mode: ties to even */
  if (a > 464.0f || isinf(a)) return sign | 0x7f;
  int e;
  const float fr = frexpf(a, &e);                 /* a = fr * 2^e, fr in [0.5, 1) */
  int q = (int)nearbyintf(fr * 16.0f);            /* 8..16 */
  e -= 1;                                         /* a = (q/8) * 2^e */
  if (q == 16) { q = 8; e += 1; }
  if (e > 8 || (e == 8 && q > 14)) return sign | 0x7f;
  return sign | (uint8_t)(((e + 7) << 3) | (q - 8));
}

void oracle_quantize_rows(const float* x, int64_t rows, int64_t cols, uint8_t* xq, float* inv_scale) {
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    float amax = 0.0f;
    for (int64_t k = 0; k < cols; ++k) {
      const float a = fabsf(xr[k]);
      if (a > amax) amax = a;
    }
    /* torch evaluates `448.0 / tensor` as reciprocal(tensor) * 448.0: two roundings */
    const float recip = 1.0f / (amax > 1e-12f ? amax : 1e-12f);
    const float scale = recip * 448.0f;
    for (int64_t k = 0; k < cols; ++k) {
      float v = xr[k] * scale;
      if (v > 448.0f) v = 448.0f;
      if (v < -448.0f) v = -448.0f;
      xq[r * cols + k] = oracle_e4m3_encode(v);
    }
    inv_scale[r] = 1.0f / scale;
  }
}

static uint16_t bf16_rne(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static float bf16_to_f32(uint16_t h) {
  const uint32_t u = ((uint32_t)h) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* bias may be NULL; c receives bf16 bit patterns. */
void oracle_gemm(const uint8_t* a, const uint8_t* b, const float* a_scale, const float* b_scale,
                 const uint16_t* bias, uint16_t* c, int64_t M, int64_t N, int64_t K) {
  float lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = oracle_e4m3_decode((uint8_t)i);
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    const uint8_t* ar = a + m * K;
    for (int64_t n = 0; n < N; ++n) {
      const uint8_t* br = b + n * K;
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k) acc += (double)lut[ar[k]] * (double)lut[br[k]];
      double v = acc * (double)a_scale[m] * (double)b_scale[n];
      if (bias) v += (double)bf16_to_f32(bias[n]);
      c[m * N + n] = bf16_rne((float)v);
    }
  }
}
