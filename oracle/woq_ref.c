/*
 * CPU port of the reference's optimized WOQ linear arithmetic -- TEST INFRASTRUCTURE ONLY
 * (the timed CPU baseline of bench.py and a second checker for tests; the product never
 * links or loads it).
 *
 * Restates, in plain C with OpenMP over output channels:
 *   - the plain INT4 format: byte j of a row = q[2j] | q[2j+1] << 4
 *     (intel_extension_for_pytorch/quantization/_quantize_utils.py:1184);
 *   - the bf16 kernel's arithmetic (csrc/cpu/aten/utils/woq.h:1495-1581, 3298-3310, 3452):
 *     w = bf16((q - z) * s) with the subtraction and the product in fp32, bf16 x bf16 products
 *     accumulated in fp32, fp32 bias, caller rounds the result;
 *   - the fallback's fp16 regime for M < 5 (woq.h:3511-3613): w = fp16((q - z) * s);
 *   - the optimized fp16 kernel for M < 5 (woq.h:775-951): fp16 fused multiply-adds on integer
 *     weights per K block of 64, the scale applied to the block sum, fp16 accumulators;
 *   - per-row symmetric activation quantization (woq_dynamic_quant.h:1608-1648) and the int8
 *     block sums + fp32 epilogue (woq.h:2172-2186).
 * The reference blocks N by 32 and K by 64 for AVX-512 / AMX; this port keeps the plain
 * [N, K/2] layout and lets the compiler vectorize the K loop, so its speed is a floor for
 * what the hand-tuned kernels reach, not a measurement of them.
 */
#include <immintrin.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline float round_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
  memcpy(&f, &u, 4);
  return f;
}

/* fp32 -> fp16 -> fp32, round to nearest even (F16C) */
static inline float round_f16(float f) {
  return _cvtsh_ss(_cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
}

/* Dequantize one output channel into w[K].  regime 0: fp16-rounded, 1: bf16-rounded, 2: fp32. */
static void dequant_row(const uint8_t* qrow, int64_t K, const float* s_row, const float* z_row,
                        int64_t G, int regime, float* w) {
  for (int64_t k = 0; k < K; ++k) {
    const uint8_t byte = qrow[k >> 1];
    const float q = (float)((k & 1) ? (byte >> 4) : (byte & 0xF));
    const int64_t g = G > 0 ? k / G : 0;
    const float z = z_row ? z_row[g] : 8.0f;
    float v = (q - z) * s_row[g];
    w[k] = regime == 0 ? round_f16(v) : (regime == 1 ? round_bf16(v) : v);
  }
}

/*
 * acc[m, n] = bias[n] + sum_k x[m, k] * w[n, k], x given as bf16 bits, accumulated in fp32.
 * scales / zeros: fp32 [N, KG] (zeros may be NULL: symmetric).  Only channels n0 <= n < n1 are
 * computed (acc is still indexed [m * N + n]), so a caller can time a bounded sample.
 */
void woq_ref_linear_int4(const uint16_t* x, int64_t M, int64_t K, int64_t N, const uint8_t* qw,
                         const float* scales, const float* zeros, int64_t G, const float* bias,
                         int regime, int64_t n0, int64_t n1, float* acc) {
  const int64_t KG = G > 0 ? (K + G - 1) / G : 1;
  const int64_t row_bytes = (K + 1) / 2;
  float* xf = (float*)malloc(sizeof(float) * (size_t)(M * K));
  for (int64_t i = 0; i < M * K; ++i) {
    float v = bf16_to_f32(x[i]);
    xf[i] = regime == 0 ? round_f16(v) : v;
  }
#pragma omp parallel
  {
    float* w = (float*)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(static)
    for (int64_t n = n0; n < n1; ++n) {
      dequant_row(qw + n * row_bytes, K, scales + n * KG, zeros ? zeros + n * KG : NULL, G, regime, w);
      for (int64_t m = 0; m < M; ++m) {
        const float* xr = xf + m * K;
        float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
        int64_t k = 0;
        for (; k + 3 < K; k += 4) {
          s0 += xr[k] * w[k];
          s1 += xr[k + 1] * w[k + 1];
          s2 += xr[k + 2] * w[k + 2];
          s3 += xr[k + 3] * w[k + 3];
        }
        for (; k < K; ++k) s0 += xr[k] * w[k];
        acc[m * N + n] = (s0 + s1) + (s2 + s3) + (bias ? bias[n] : 0.f);
      }
    }
    free(w);
  }
  free(xf);
}

/* double -> fp16 with ONE rounding to nearest even (through a float rounded to odd). */
static inline float round_f16_from_double(double d) {
  float f = (float)d;
  if ((double)f != d) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if (fabs((double)f) > fabs(d)) u -= 1;  /* towards zero */
    u |= 1u;                                /* sticky bit */
    memcpy(&f, &u, 4);
  }
  return round_f16(f);
}

/*
 * The optimized fp16 kernel of the reference for fewer than five rows (GemmMicroKernel<half>,
 * csrc/cpu/aten/utils/woq.h:775-951): activations rounded to fp16; per output and K block of
 * block_k values vc = 0, vc = fma16(x_k, q_k - z, vc) for k ascending, then C = fma16(s, vc, C); C starts
 * at the fp16 bias or 0 and is the fp16 result (returned as float).  fma16 = a * b + c rounded once to
 * fp16: the products and sums of the inner chain are exact in double; the outer fma goes through the
 * double-precision fma, whose own rounding could only matter when |C| exceeds |s * vc| by 2^30.
 */
void woq_ref_linear_int4_fp16_chain(const uint16_t* x, int64_t M, int64_t K, int64_t N, const uint8_t* qw,
                                    const float* scales, const float* zeros, int64_t G, int64_t block_k,
                                    const float* bias, int64_t n0, int64_t n1, float* out) {
  const int64_t KG = G > 0 ? (K + G - 1) / G : 1;
  const int64_t row_bytes = (K + 1) / 2;
  float* xh = (float*)malloc(sizeof(float) * (size_t)(M * K));
  for (int64_t i = 0; i < M * K; ++i) xh[i] = round_f16(bf16_to_f32(x[i]));
#pragma omp parallel for schedule(static)
  for (int64_t n = n0; n < n1; ++n) {
    const uint8_t* qrow = qw + n * row_bytes;
    for (int64_t m = 0; m < M; ++m) {
      const float* xr = xh + m * K;
      float C = bias ? round_f16(bias[n]) : 0.f;
      for (int64_t k0 = 0; k0 < K; k0 += block_k) {
        const int64_t g = G > 0 ? k0 / G : 0;
        const float z = zeros ? round_f16(zeros[n * KG + g]) : 8.0f;
        const float s = round_f16(scales[n * KG + g]);
        float vc = 0.f;
        for (int64_t k = k0; k < k0 + block_k && k < K; ++k) {
          const uint8_t byte = qrow[k >> 1];
          const float w = (float)((k & 1) ? (byte >> 4) : (byte & 0xF)) - z;
          vc = round_f16_from_double((double)xr[k] * (double)w + (double)vc);
        }
        C = round_f16_from_double(fma((double)s, (double)vc, (double)C));
      }
      out[m * N + n] = C;
    }
  }
  free(xh);
}

/* Per-row symmetric int8 quantization: s = max|x| / 127, q = clamp(rint(x / s), -128, 127). */
void woq_ref_quant_per_row(const uint16_t* x, int64_t M, int64_t K, int8_t* q, float* scales) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    float amax = 0.f;
    for (int64_t k = 0; k < K; ++k) amax = fmaxf(amax, fabsf(bf16_to_f32(x[m * K + k])));
    const float s = amax / 127.0f;
    scales[m] = s;
    for (int64_t k = 0; k < K; ++k) {
      float t = s > 0.f ? nearbyintf(bf16_to_f32(x[m * K + k]) / s) : 0.f;
      t = fminf(fmaxf(t, -128.f), 127.f);
      q[m * K + k] = (int8_t)t;
    }
  }
}

/*
 * lowp_mode INT8, per-row activation scales: for each K block of block_k values,
 * qC = sum a_i8 * (q - z) in int32; C += ((float)qC * s_a[m]) * s_w[n, g].  C starts at bias.
 */
void woq_ref_linear_int4_int8(const int8_t* xq, const float* sa, int64_t M, int64_t K, int64_t N,
                              const uint8_t* qw, const float* scales, const float* zeros, int64_t G,
                              int64_t block_k, const float* bias, int64_t n0, int64_t n1, float* acc) {
  const int64_t KG = G > 0 ? (K + G - 1) / G : 1;
  const int64_t row_bytes = (K + 1) / 2;
#pragma omp parallel
  {
    int8_t* b = (int8_t*)malloc((size_t)K);
#pragma omp for schedule(static)
    for (int64_t n = n0; n < n1; ++n) {
      const uint8_t* qrow = qw + n * row_bytes;
      for (int64_t k = 0; k < K; ++k) {
        const uint8_t byte = qrow[k >> 1];
        const int q = (k & 1) ? (byte >> 4) : (byte & 0xF);
        const int64_t g = G > 0 ? k / G : 0;
        const int z = zeros ? (int)zeros[n * KG + g] : 8;
        b[k] = (int8_t)(q - z);
      }
      for (int64_t m = 0; m < M; ++m) {
        float c = bias ? bias[n] : 0.f;
        const int8_t* a = xq + m * K;
        for (int64_t k0 = 0; k0 < K; k0 += block_k) {
          int32_t qc = 0;
          for (int64_t k = k0; k < k0 + block_k; ++k) qc += (int32_t)a[k] * (int32_t)b[k];
          const int64_t g = G > 0 ? k0 / G : 0;
          volatile float t = (float)qc * sa[m];
          volatile float u = t * scales[n * KG + g];
          c = c + u;
        }
        acc[m * N + n] = c;
      }
    }
    free(b);
  }
}
