// kapy_baseline.cpp — multithreaded CPU implementations of the benchmark workloads, written for speed
// (TEST INFRASTRUCTURE ONLY: they are what the benchmark's cpu_baseline leg times on the host cores).
//
// The checker in kapy_oracle.cpp is written for exactness (fp64, one element at a time) and is a poor
// measure of what the host can do.  These are the same ops as a CPU programmer would write them:
// packed panels and a register-blocked fp32 micro-kernel for the GEMMs, a fused vector loop for
// act(x*s + bias), cache-blocked tiles for the transposes.  AVX-512 forms are picked at run time when
// the host has them; the portable forms compute the same values.  tests/test_oracle_baselines.py
// checks every one of them against the checker, so that the time reported is the time of the right result.
//
// Op semantics as in kapy_oracle.cpp: kapy.matmul with fp32 accumulate (Ops.td:416-439), the fused chain
// extf -> mulf -> addf -> gelu -> fptofp rn of ElementwiseOpToLLVM.cpp:424-1238, ld_global / st_global with
// swapped strides (LdGlobalOpToLLVM.cpp:60-145, StGlobalOpToLLVM.cpp:60-139).
#include <immintrin.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <vector>

#include "kapy_oracle.h"

namespace {

constexpr int MR = 8, NR = 32, KC = 512;
typedef float v16f __attribute__((vector_size(64), aligned(4)));

// C[8 x 32] (+)= Ap[kc x 8] . Bp[kc x 32]; `first` starts from zero instead of C.
#define KO_MICRO_BODY                                                                   \
  v16f acc[MR][2];                                                                      \
  for (int i = 0; i < MR; ++i) {                                                        \
    if (first) {                                                                        \
      acc[i][0] = v16f{};                                                               \
      acc[i][1] = v16f{};                                                               \
    } else {                                                                            \
      acc[i][0] = *(const v16f *)(c + i * ldc);                                         \
      acc[i][1] = *(const v16f *)(c + i * ldc + 16);                                    \
    }                                                                                   \
  }                                                                                     \
  for (int k = 0; k < kc; ++k) {                                                        \
    const v16f b0 = *(const v16f *)(bp + (int64_t)k * NR), b1 = *(const v16f *)(bp + (int64_t)k * NR + 16); \
    for (int i = 0; i < MR; ++i) {                                                      \
      const float a = ap[(int64_t)k * MR + i];                                          \
      acc[i][0] += a * b0;                                                              \
      acc[i][1] += a * b1;                                                              \
    }                                                                                   \
  }                                                                                     \
  for (int i = 0; i < MR; ++i) {                                                        \
    *(v16f *)(c + i * ldc) = acc[i][0];                                                 \
    *(v16f *)(c + i * ldc + 16) = acc[i][1];                                            \
  }

__attribute__((target("avx512f,fma"), optimize("O3", "-ffp-contract=fast"))) void micro_avx512(const float *ap, const float *bp, float *c, int64_t ldc, int kc, bool first) { KO_MICRO_BODY }
__attribute__((target("avx2,fma"), optimize("O3", "-ffp-contract=fast"))) void micro_avx2(const float *ap, const float *bp, float *c, int64_t ldc, int kc, bool first) { KO_MICRO_BODY }
__attribute__((optimize("O3", "-ffp-contract=fast"))) void micro_portable(const float *ap, const float *bp, float *c, int64_t ldc, int kc, bool first) { KO_MICRO_BODY }

typedef void (*micro_fn)(const float *, const float *, float *, int64_t, int, bool);
micro_fn pick_micro() {
  if (__builtin_cpu_supports("avx512f")) return micro_avx512;
  if (__builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma")) return micro_avx2;
  return micro_portable;
}

int64_t elem(const ko_global *g, int64_t i, int64_t j) { return (g->start0 + i) * (int64_t)g->stride0 + (g->start1 + j) * (int64_t)g->stride1; }

// ---- exp on 16 floats: 2^(x log2 e), degree-6 polynomial on the fraction, scaled by scalef ----
__attribute__((target("avx512f,fma"))) inline __m512 exp512(__m512 x) {
  const __m512 t = _mm512_mul_ps(x, _mm512_set1_ps(1.4426950408889634f));
  const __m512 n = _mm512_roundscale_ps(t, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
  const __m512 f = _mm512_sub_ps(t, n);
  __m512 p = _mm512_set1_ps(1.5403530e-4f);
  p = _mm512_fmadd_ps(p, f, _mm512_set1_ps(1.3333558e-3f));
  p = _mm512_fmadd_ps(p, f, _mm512_set1_ps(9.6181291e-3f));
  p = _mm512_fmadd_ps(p, f, _mm512_set1_ps(5.5504109e-2f));
  p = _mm512_fmadd_ps(p, f, _mm512_set1_ps(2.4022651e-1f));
  p = _mm512_fmadd_ps(p, f, _mm512_set1_ps(6.9314718e-1f));
  p = _mm512_fmadd_ps(p, f, _mm512_set1_ps(1.0f));
  return _mm512_scalef_ps(p, n);
}

// y = fptofp_rn(gelu_tanh(extf(x) * s + extf(bias))) over rows [r0, r1), fp16 in and out; cols a multiple of 16.
__attribute__((target("avx512f,avx512bw,f16c,fma"))) void gelu_rows_avx512(const uint16_t *x, const uint16_t *bias, float scale, uint16_t *y, int64_t r0,
                                                                             int64_t r1, int64_t cols, int64_t pitch) {
  const __m512 s = _mm512_set1_ps(scale), k0 = _mm512_set1_ps(0.7978845608028654f), k1 = _mm512_set1_ps(0.044715f);
  const __m512 one = _mm512_set1_ps(1.0f), m2 = _mm512_set1_ps(-2.0f);
  for (int64_t r = r0; r < r1; ++r)
    for (int64_t j = 0; j < cols; j += 16) {
      __m512 v = _mm512_cvtph_ps(_mm256_loadu_si256((const __m256i *)(x + r * pitch + j)));
      const __m512 b = _mm512_cvtph_ps(_mm256_loadu_si256((const __m256i *)(bias + j)));
      v = _mm512_add_ps(_mm512_mul_ps(v, s), b);  // mulf, then addf: two roundings, as the two ops round
      const __m512 v3 = _mm512_mul_ps(_mm512_mul_ps(v, v), v);
      const __m512 u = _mm512_mul_ps(k0, _mm512_fmadd_ps(k1, v3, v));
      // 0.5 v (1 + tanh u) = v / (1 + exp(-2u))
      const __m512 e = exp512(_mm512_mul_ps(m2, u));
      const __m512 g = _mm512_div_ps(v, _mm512_add_ps(one, e));
      _mm256_storeu_si256((__m256i *)(y + r * pitch + j), _mm512_cvtps_ph(g, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
    }
}

void gelu_rows_portable(const uint16_t *x, const uint16_t *bias, float scale, uint16_t *y, int64_t r0, int64_t r1, int64_t cols, int64_t pitch) {
  std::vector<float> b((size_t)cols);
  for (int64_t j = 0; j < cols; ++j) b[j] = (float)ko_f16_to_f64(bias[j]);
  for (int64_t r = r0; r < r1; ++r)
    for (int64_t j = 0; j < cols; ++j) {
      float v = (float)ko_f16_to_f64(x[r * pitch + j]) * scale;
      v += b[j];
      const float u = 0.7978845608028654f * (v + 0.044715f * (v * v * v));
      const float g = v / (1.0f + std::exp(-2.0f * u));
      y[r * pitch + j] = ko_f64_to_f16((double)g, KO_RN);
    }
}

}  // namespace

extern "C" {

// result = cast(lhs . rhs [* row_scale[m] * col_scale[n]]), any operand element types and strides; fp32 accumulate over
// K blocks of 512, the blocks summed in fp64 (so that the whole result can serve as a gate at benchmark sizes).
// *multiply_seconds (if not null) gets the time of the multiplication proper: operands already widened to
// fp32 and packed into panels (the GPU kernels are handed their operands in the layout they want, too),
// result still fp32.
int ko_baseline_gemm(const ko_global *lhs, const ko_global *rhs, const float *row_scale, const float *col_scale, const ko_global *result,
                     double *multiply_seconds) {
  const int64_t M = (int64_t)lhs->end0 - lhs->start0, K = (int64_t)lhs->end1 - lhs->start1, N = (int64_t)rhs->end1 - rhs->start1;
  if ((int64_t)rhs->end0 - rhs->start0 != K || (int64_t)result->end0 - result->start0 != M || (int64_t)result->end1 - result->start1 != N) return -1;
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const int64_t mp = (M + MR - 1) / MR, np = (N + NR - 1) / NR;
  float *ap = (float *)aligned_alloc(64, (size_t)mp * K * MR * sizeof(float));
  float *bp = (float *)aligned_alloc(64, (size_t)np * K * NR * sizeof(float));
  double *c = (double *)aligned_alloc(64, (size_t)mp * MR * np * NR * sizeof(double));
  if (!ap || !bp || !c) {
    free(ap); free(bp); free(c);
    return -2;
  }
  // pack: Ap[panel][k][8 rows], Bp[panel][k][32 columns]; rows / columns past the edge are zero
#pragma omp parallel for schedule(static)
  for (int64_t p = 0; p < mp; ++p)
    for (int64_t k = 0; k < K; ++k)
      for (int i = 0; i < MR; ++i) {
        const int64_t m = p * MR + i;
        ap[(p * K + k) * MR + i] = m < M ? (float)ko_decode(lhs->ptr, lhs->dtype, elem(lhs, m, k)) : 0.f;
      }
#pragma omp parallel for schedule(static)
  for (int64_t p = 0; p < np; ++p)
    for (int64_t k = 0; k < K; ++k)
      for (int j = 0; j < NR; ++j) {
        const int64_t n = p * NR + j;
        bp[(p * K + k) * NR + j] = n < N ? (float)ko_decode(rhs->ptr, rhs->dtype, elem(rhs, k, n)) : 0.f;
      }
  const micro_fn micro = pick_micro();
  const int64_t ldc = np * NR;
  const auto t0 = std::chrono::steady_clock::now();
  for (int64_t k0 = 0; k0 < K; k0 += KC) {
    const int kc = (int)std::min<int64_t>(KC, K - k0);
    // a column panel of B (kc x 32 floats, 64 KiB) stays in a core's L2 while the row panels of A stream past it
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t jp = 0; jp < np; ++jp)
      for (int64_t ip = 0; ip < mp; ++ip) {
        // one K block of an 8 x 32 tile in fp32 registers, the blocks summed in fp64
        alignas(64) float t[MR * NR];
        micro(ap + (ip * K + k0) * MR, bp + (jp * K + k0) * NR, t, NR, kc, true);
        double *cc = c + ip * MR * ldc + jp * NR;
        for (int i = 0; i < MR; ++i)
          for (int j = 0; j < NR; ++j) cc[i * ldc + j] = (k0 == 0 ? 0.0 : cc[i * ldc + j]) + (double)t[i * NR + j];
      }
  }
  const double dt = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
  if (multiply_seconds) *multiply_seconds = dt;
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      double v = c[m * ldc + n];
      if (row_scale && col_scale) v *= (double)(row_scale[m] * col_scale[n]);   // the scale product in fp32, as the checker forms it
      ko_encode(result->ptr, result->dtype, elem(result, m, n), v, KO_RN);
    }
  free(ap); free(bp); free(c);
  return 0;
}

// y[r][j] = f16(gelu_tanh(f32(x[r][j]) * scale + f32(bias[j]))), rows of `pitch` elements, fp32 arithmetic.
int ko_baseline_gelu_f16(const uint16_t *x, const uint16_t *bias, float scale, uint16_t *y, int64_t rows, int64_t cols, int64_t pitch) {
  const bool fast = __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") && __builtin_cpu_supports("f16c") && cols % 16 == 0;
  const int64_t chunk = 8;
#pragma omp parallel for schedule(static)
  for (int64_t r0 = 0; r0 < rows; r0 += chunk) {
    const int64_t r1 = std::min(rows, r0 + chunk);
    if (fast) gelu_rows_avx512(x, bias, scale, y, r0, r1, cols, pitch);
    else gelu_rows_portable(x, bias, scale, y, r0, r1, cols, pitch);
  }
  return 0;
}

// dst[j][i] = src[i][j] for 16-bit elements, both dense row-major; 64 x 64 tiles so that both sides move whole cache lines.
int ko_baseline_transpose16(const uint16_t *src, uint16_t *dst, int64_t rows, int64_t cols) {
  constexpr int64_t T = 64;
  const int64_t tr = (rows + T - 1) / T, tc = (cols + T - 1) / T;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t bi = 0; bi < tr; ++bi)
    for (int64_t bj = 0; bj < tc; ++bj) {
      const int64_t i1 = std::min(rows, bi * T + T), j1 = std::min(cols, bj * T + T);
      for (int64_t j = bj * T; j < j1; ++j)
        for (int64_t i = bi * T; i < i1; ++i) dst[j * rows + i] = src[i * cols + j];
    }
  return 0;
}

// out[b][s][h][:] = in[b][h][s][:] for 16-bit elements: rows of d elements move whole.
int ko_baseline_permute_bhsd_bshd16(const uint16_t *src, uint16_t *dst, int64_t b, int64_t h, int64_t s, int64_t d) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t ib = 0; ib < b; ++ib)
    for (int64_t is = 0; is < s; ++is)
      for (int64_t ih = 0; ih < h; ++ih)
        memcpy(dst + ((ib * s + is) * h + ih) * d, src + ((ib * h + ih) * s + is) * d, (size_t)d * 2);
  return 0;
}

}  // extern "C"
