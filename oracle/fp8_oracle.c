/* CPU oracle for the FP8 mixed-precision linear path, C restatement.  TEST INFRASTRUCTURE ONLY:
 * only tests/, the smoke check and the cpu_baseline leg of the benchmark may load this library.
 *
 * It is a second, independently written implementation of the arithmetic in fp8_oracle.py (the
 * E4M3 encoder here rounds with nearbyintf on a scaled magnitude instead of integer bit
 * tricks, the power-of-two scales come from frexpf / ldexpf instead of exponent-field arithmetic), so the
 * two pin each other bit for bit; both are pinned to torch's float8_e4m3fn cast by tests/test_oracle_pins.py.
 *
 * The reference checkout has no FP8 arithmetic.  The recipe follows the benchmark
 * configuration text (scale = 448/amax, E4M3 cast, fp32 accumulation, bf16 output, 1x128 /
 * 128x128 / 128x1 block geometries); operand roles follow the reference's linear operator
 * (weight [out, in], contraction over the last dim of both operands,
 * hyper_parallel/core/shard/ops/parallel_matmul.py:377-381) and the flat gradient bucket of
 * hyper_parallel/core/hsdp/hsdp_grad_buffer.py:95-108.
 *
 * Build: gcc -O2 -fno-fast-math -ffp-contract=off -fopenmp -shared -fPIC (see Makefile).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define HPO_BLOCK 128
static const float kFp8Max = 448.0f;
static const float kAmaxEps = 1e-12f;

static inline float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

float hpo_e4m3_decode(uint8_t c) {
  int e = (c >> 3) & 0xF, m = c & 7;
  float mag;
  if ((c & 0x7F) == 0x7F) return NAN;
  mag = e ? ldexpf((float)(8 + m), e - 10) : ldexpf((float)m, -9);
  return (c & 0x80) ? -mag : mag;
}

/* Round-to-nearest-even onto the E4M3FN grid, not saturating: |x| >= 464 and NaN -> NaN code. */
uint8_t hpo_e4m3_encode(float x) {
  uint8_t sign = signbit(x) ? 0x80 : 0x00;
  float a = fabsf(x);
  int e, steps;
  float q;
  if (isnan(x) || isinf(x)) return sign | 0x7F;
  if (a < 0.015625f) {                       /* below 2^-6: grid step 2^-9 */
    steps = (int)nearbyintf(a * 512.0f);     /* exact product; 8 lands on the first normal */
    return sign | (uint8_t)steps;
  }
  (void)frexpf(a, &e);                       /* a = f * 2^e, f in [0.5, 1) -> binade 2^(e-1) */
  e -= 1;
  q = nearbyintf(ldexpf(a, 3 - e));          /* in [8, 16]; 16 means carry into next binade */
  steps = (int)q;
  if (steps == 16) { steps = 8; e += 1; }
  if (e > 8 || (e == 8 && steps - 8 > 6)) return sign | 0x7F;
  return sign | (uint8_t)(((e + 7) << 3) | (steps - 8));
}

static inline float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

static inline void scales(float amax, float* scale, float* scale_inv) {
  float amc = amax < kAmaxEps ? kAmaxEps : amax;   /* a NaN amax stays NaN */
  *scale = kFp8Max / amc;
  *scale_inv = amc / kFp8Max;
}

static inline uint8_t cast1(uint16_t xb, float scale) {
  float y = bf16_to_f32(xb) * scale;
  return hpo_e4m3_encode(clampf(y, -kFp8Max, kFp8Max));
}

float hpo_amax_bf16(const uint16_t* x, int64_t n) {
  float am = 0.0f;
  for (int64_t i = 0; i < n; ++i) {
    float a = fabsf(bf16_to_f32(x[i]));
    if (a > am || a != a) am = a;   /* NaN wins and then stays */
  }
  return am;
}

void hpo_quantize_per_tensor(const uint16_t* x, int64_t n, uint8_t* q, float* scale, float* scale_inv) {
  float s, si;
  scales(hpo_amax_bf16(x, n), &s, &si);
  *scale = s;
  *scale_inv = si;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) q[i] = cast1(x[i], s);
}

/* x[rows, cols] -> q[rows, cols], scale/scale_inv[rows, cols/128] */
void hpo_quantize_1x128(const uint16_t* x, int64_t rows, int64_t cols, uint8_t* q, float* scale,
                        float* scale_inv) {
  int64_t groups = rows * (cols / HPO_BLOCK);
#pragma omp parallel for schedule(static)
  for (int64_t g = 0; g < groups; ++g) {
    const uint16_t* p = x + g * HPO_BLOCK;
    float s, si;
    scales(hpo_amax_bf16(p, HPO_BLOCK), &s, &si);
    scale[g] = s;
    scale_inv[g] = si;
    for (int i = 0; i < HPO_BLOCK; ++i) q[g * HPO_BLOCK + i] = cast1(p[i], s);
  }
}

/* w[rows, cols] -> q[rows, cols], scale/scale_inv[rows/128, cols/128] */
void hpo_quantize_128x128(const uint16_t* w, int64_t rows, int64_t cols, uint8_t* q, float* scale,
                          float* scale_inv) {
  int64_t rb = rows / HPO_BLOCK, cb = cols / HPO_BLOCK;
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < rb * cb; ++b) {
    int64_t r0 = (b / cb) * HPO_BLOCK, c0 = (b % cb) * HPO_BLOCK;
    float am = 0.0f, s, si;
    for (int i = 0; i < HPO_BLOCK; ++i) {
      float a = hpo_amax_bf16(w + (r0 + i) * cols + c0, HPO_BLOCK);
      if (a > am || a != a) am = a;   /* NaN wins and then stays */
    }
    scales(am, &s, &si);
    scale[b] = s;
    scale_inv[b] = si;
    for (int i = 0; i < HPO_BLOCK; ++i)
      for (int j = 0; j < HPO_BLOCK; ++j)
        q[(r0 + i) * cols + c0 + j] = cast1(w[(r0 + i) * cols + c0 + j], s);
  }
}

/* x[m, k] -> qt[k, m], scale_t/scale_inv_t[k, m/128]: one scale per 128 consecutive rows of a column */
void hpo_quantize_128x1_t(const uint16_t* x, int64_t m, int64_t k, uint8_t* qt, float* scale_t,
                          float* scale_inv_t) {
  int64_t mb = m / HPO_BLOCK;
#pragma omp parallel for schedule(static)
  for (int64_t col = 0; col < k; ++col) {
    for (int64_t b = 0; b < mb; ++b) {
      float am = 0.0f, s, si;
      for (int i = 0; i < HPO_BLOCK; ++i) {
        float a = fabsf(bf16_to_f32(x[(b * HPO_BLOCK + i) * k + col]));
        if (a > am || a != a) am = a;   /* NaN wins and then stays */
      }
      scales(am, &s, &si);
      scale_t[col * mb + b] = s;
      scale_inv_t[col * mb + b] = si;
      for (int i = 0; i < HPO_BLOCK; ++i)
        qt[col * m + b * HPO_BLOCK + i] = cast1(x[(b * HPO_BLOCK + i) * k + col], s);
    }
  }
}

/* q[rows, cols], scale_inv[rows, cols/128] -> bf16 bits */
void hpo_dequantize_1x128(const uint8_t* q, const float* scale_inv, int64_t rows, int64_t cols,
                          uint16_t* out) {
  int64_t groups = rows * (cols / HPO_BLOCK);
#pragma omp parallel for schedule(static)
  for (int64_t g = 0; g < groups; ++g)
    for (int i = 0; i < HPO_BLOCK; ++i)
      out[g * HPO_BLOCK + i] = f32_to_bf16(hpo_e4m3_decode(q[g * HPO_BLOCK + i]) * scale_inv[g]);
}

/* Scaled GEMM.  a[M,K] codes, sa_inv[M,K/128]; b[N,K] codes, sb_inv is [N/128,K/128]
 * (sb_per_row = 0) or [N,K/128] (sb_per_row = 1).  Per 128-wide k-block: fp32 dot product,
 * times sa_inv*sb_inv, added to the fp32 accumulator, k-blocks ascending.  bias (fp32, may be
 * NULL) is added before the single rounding to bf16.  out_f32 / out_bf16 may each be NULL. */
void hpo_gemm_blockwise(const uint8_t* a, const float* sa_inv, const uint8_t* b, const float* sb_inv,
                        int64_t M, int64_t N, int64_t K, int sb_per_row, const float* bias,
                        float* out_f32, uint16_t* out_bf16) {
  float lut[256];
  int64_t kb_cnt = K / HPO_BLOCK;
  for (int c = 0; c < 256; ++c) lut[c] = hpo_e4m3_decode((uint8_t)c);
#pragma omp parallel
  {
    float* arow = (float*)malloc(sizeof(float) * (size_t)K);
    float* brow = (float*)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
      for (int64_t k = 0; k < K; ++k) brow[k] = lut[b[n * K + k]];
      for (int64_t m = 0; m < M; ++m) {
        float acc = 0.0f;
        for (int64_t k = 0; k < K; ++k) arow[k] = lut[a[m * K + k]];
        for (int64_t kb = 0; kb < kb_cnt; ++kb) {
          float p[8] = {0, 0, 0, 0, 0, 0, 0, 0};
          const float* ap = arow + kb * HPO_BLOCK;
          const float* bp = brow + kb * HPO_BLOCK;
          float part;
          float sb = sb_per_row ? sb_inv[n * kb_cnt + kb] : sb_inv[(n / HPO_BLOCK) * kb_cnt + kb];
          for (int i = 0; i < HPO_BLOCK; i += 8)
            for (int j = 0; j < 8; ++j) p[j] += ap[i + j] * bp[i + j];
          part = ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
          acc += part * (sa_inv[m * kb_cnt + kb] * sb);
        }
        if (bias) acc += bias[n];
        if (out_f32) out_f32[m * N + n] = acc;
        if (out_bf16) out_bf16[m * N + n] = f32_to_bf16(acc);
      }
    }
    free(arow);
    free(brow);
  }
}

/* Power-of-two scales (the optional recipe): scale_inv = the smallest power of two >= max(amax, eps) / 448,
 * found with frexpf instead of the exponent-field arithmetic of the Python form; scale = 1 / scale_inv.
 * NaN and Inf pass through unchanged. */
void hpo_scales_pow2(float amax, float* scale, float* scale_inv) {
  float amc = amax < kAmaxEps ? kAmaxEps : amax;
  float si = amc / kFp8Max;
  if (!isnan(si) && !isinf(si)) {
    int e;
    float f = frexpf(si, &e);            /* si = f * 2^e, f in [0.5, 1) */
    si = (f == 0.5f) ? si : ldexpf(1.0f, e);
  }
  *scale_inv = si;
  *scale = 1.0f / si;
}

/* exp(t) as the SwiGLU kernel defines it, one IEEE fp32 operation per step (no contraction: see the build
 * flags), written with the C library's rounding, scaling and ordered-comparison routines where the Python form
 * uses array operations and exponent-field arithmetic. */
float hpo_exp_spec(float t) {
  volatile float r, p, kk;
  float k;
  if (t < -86.0f) t = -86.0f;            /* (a NaN passes both comparisons and stays) */
  if (t > 89.0f) t = 89.0f;
  k = nearbyintf(t * 1.44269504f);
  kk = k * 0.693359375f;
  r = t - kk;
  kk = k * -2.12194440e-4f;
  r = r - kk;
  p = 1.0f / 720.0f;
  {
    const float c[6] = {1.0f / 120.0f, 1.0f / 24.0f, 1.0f / 6.0f, 0.5f, 1.0f, 1.0f};
    for (int i = 0; i < 6; ++i) {
      p = p * r;
      p = p + c[i];
    }
  }
  p = p * ldexpf(1.0f, (int)k - 1);      /* k - 1 >= -125: a normal number */
  return p * 2.0f;
}

/* act = bf16(bf16(silu(gate)) * up), h[rows, 2 * inter] = gate | up, silu(g) = g / (1 + exp_spec(-g)) */
void hpo_swiglu(const uint16_t* h, int64_t rows, int64_t inter, uint16_t* act) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < inter; ++c) {
      float g = bf16_to_f32(h[r * 2 * inter + c]), u = bf16_to_f32(h[r * 2 * inter + inter + c]);
      volatile float den = 1.0f + hpo_exp_spec(-g);
      volatile float s = g / den;
      float sb = bf16_to_f32(f32_to_bf16(s));
      volatile float prod = sb * u;
      act[r * inter + c] = f32_to_bf16(prod);
    }
}

int hpo_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
