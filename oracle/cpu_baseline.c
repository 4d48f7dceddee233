/*
 * CPU BASELINE - TEST/BENCH INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * C restatement (intrinsics) of the reference's AVX2 dot-product kernels, used only as the
 * "cpu_baseline" leg of the benchmark and checked by the tests against the scalar oracle.
 * These are restated reference kernels, not the Free Pascal binary: FPC is not available
 * and the reference's layer unit is absent from the checkout.
 */
#include <immintrin.h>
#include <stdint.h>
#include <stddef.h>
#include <omp.h>

/* neural/neuralvolume.pas:11960-12078 (AVXDotProduct, AVX2 branch): four ymm accumulators over
 * 32-element strides with vfmadd231ps, combine, 4-wide SSE tail, two HADDPS, scalar remainder. */
float cpu_avx_dot_f32(const float* a, const float* b, int n)
{
  int missed = n & 3, ln = n ^ missed;
  float res = 0;
  if (ln > 0) {
    __m128 x0 = _mm_setzero_ps();
    int big = ln >> 5, i = 0;
    if (big) {
      __m256 y0 = _mm256_setzero_ps(), y1 = y0, y6 = y0, y7 = y0;
      for (int it = 0; it < big; it++, i += 32) {
        y0 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i),      _mm256_loadu_ps(b + i),      y0);
        y1 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 8),  _mm256_loadu_ps(b + i + 8),  y1);
        y6 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 16), _mm256_loadu_ps(b + i + 16), y6);
        y7 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 24), _mm256_loadu_ps(b + i + 24), y7);
      }
      y0 = _mm256_add_ps(_mm256_add_ps(y0, y1), _mm256_add_ps(y6, y7));
      x0 = _mm_add_ps(_mm256_castps256_ps128(y0), _mm256_extractf128_ps(y0, 1));
    }
    for (int it = (ln & 31) >> 2; it > 0; it--, i += 4)
      x0 = _mm_add_ps(x0, _mm_mul_ps(_mm_loadu_ps(a + i), _mm_loadu_ps(b + i)));
    x0 = _mm_hadd_ps(x0, x0); x0 = _mm_hadd_ps(x0, x0);
    res = _mm_cvtss_f32(x0);
  }
  for (int i = ln; i < n; i++) res += a[i] * b[i];
  return res;
}

/* neural/neuralvolume.pas:1780-1882 (AVXDotProductInt8): vpmovsxbd -> vcvtdq2ps -> vfmadd231ps,
 * same skeleton; returns the RAW code sum (scale applied by the caller). */
float cpu_avx_dot_int8(const int8_t* a, const float* b, int n)
{
  int missed = n & 3, ln = n ^ missed;
  float res = 0;
  if (ln > 0) {
    __m128 x0 = _mm_setzero_ps();
    int big = ln >> 5, i = 0;
    if (big) {
      __m256 y0 = _mm256_setzero_ps(), y1 = y0, y6 = y0, y7 = y0;
      for (int it = 0; it < big; it++, i += 32) {
        __m256 w0 = _mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(_mm_loadl_epi64((const __m128i*)(a + i))));
        __m256 w1 = _mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(_mm_loadl_epi64((const __m128i*)(a + i + 8))));
        __m256 w2 = _mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(_mm_loadl_epi64((const __m128i*)(a + i + 16))));
        __m256 w3 = _mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(_mm_loadl_epi64((const __m128i*)(a + i + 24))));
        y0 = _mm256_fmadd_ps(w0, _mm256_loadu_ps(b + i),      y0);
        y1 = _mm256_fmadd_ps(w1, _mm256_loadu_ps(b + i + 8),  y1);
        y6 = _mm256_fmadd_ps(w2, _mm256_loadu_ps(b + i + 16), y6);
        y7 = _mm256_fmadd_ps(w3, _mm256_loadu_ps(b + i + 24), y7);
      }
      y0 = _mm256_add_ps(_mm256_add_ps(y0, y1), _mm256_add_ps(y6, y7));
      x0 = _mm_add_ps(_mm256_castps256_ps128(y0), _mm256_extractf128_ps(y0, 1));
    }
    for (int it = (ln & 31) >> 2; it > 0; it--, i += 4) {
      int32_t four; __builtin_memcpy(&four, a + i, 4);
      __m128 w = _mm_cvtepi32_ps(_mm_cvtepi8_epi32(_mm_cvtsi32_si128(four)));
      x0 = _mm_add_ps(x0, _mm_mul_ps(w, _mm_loadu_ps(b + i)));
    }
    x0 = _mm_hadd_ps(x0, x0); x0 = _mm_hadd_ps(x0, x0);
    res = _mm_cvtss_f32(x0);
  }
  for (int i = ln; i < n; i++) res += (float)a[i] * b[i];
  return res;
}

/* Linear layer over fp32 weights: Out[b*rows+a] = dot(W[a], X[b]) + bias[a]
 * (neural/neuralvolume.pas:12127-12423), output rows split into disjoint contiguous ranges
 * across threads - the intra-layer chunk contract of neural/neuralvolume.pas:519-530. */
void cpu_linear_f32(const float* w, int64_t rows, int cols, const float* x, int n_b,
                    const float* bias, float* y, int threads)
{
#pragma omp parallel for schedule(static) num_threads(threads)
  for (int64_t a = 0; a < rows; a++)
    for (int b = 0; b < n_b; b++)
      y[(int64_t)b * rows + a] = cpu_avx_dot_f32(w + a * cols, x + (int64_t)b * cols, cols) + (bias ? bias[a] : 0.0f);
}

/* Per-row int8 linear layer: Out = dot_int8(codes[a], X[b]) * scale[a] + bias[a]
 * (neural/neuralvolume.pas:12693-12745, DotProductsTiledInt8). */
void cpu_linear_int8(const int8_t* codes, const float* scales, int64_t rows, int cols, const float* x,
                     int n_b, const float* bias, float* y, int threads)
{
#pragma omp parallel for schedule(static) num_threads(threads)
  for (int64_t a = 0; a < rows; a++)
    for (int b = 0; b < n_b; b++)
      y[(int64_t)b * rows + a] = cpu_avx_dot_int8(codes + a * cols, x + (int64_t)b * cols, cols) * scales[a] + (bias ? bias[a] : 0.0f);
}

int cpu_max_threads(void) { return omp_get_max_threads(); }
