/*
 * cpu_baseline.c -- OpenMP restatement of the dense contractions, used ONLY as
 * the timed CPU baseline in bench.py and checked against tile_oracle.c in
 * tests/test_cpu_baseline.py.  TEST / MEASUREMENT INFRASTRUCTURE: the shipped
 * library never links or calls it.
 *
 * Same index set and scalar semantics as the reference lowering of
 *   O[n,y,x,co] += I[n, s*y + ky - p, s*x + kx - p, ci] * F[ky,kx,ci,co]
 * (plaidml/op/lib/ops.cc:1342-1456; out-of-range taps are skipped,
 * docs/usage/edsl_ops.rst:24-44), followed by the bias start value
 * (pmlc/dialect/tile/transforms/algebraic_opt.cc:30-75) and ReLU
 * (pmlc/conversion/pxa_to_affine/pxa_to_affine.cc:312-332).  It is NOT the
 * reference's libxsmm JIT path (which cannot be built here); it is a plain
 * cache-friendly loop nest that the compiler vectorises over output channels.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int cpu_baseline_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* fp32 NHWC conv + bias + optional relu; bf16 callers pass bf16-representable fp32 values
 * and round the result themselves. */
void cpu_conv2d_nhwc_f32(const float* in, const float* filt, const float* bias, float* out, int n, int h, int w,
                         int ci, int kh, int kw, int co, int oh, int ow, int stride, int pad, int relu) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < n; ++b) {
    for (int y = 0; y < oh; ++y) {
      float* acc = (float*)malloc(sizeof(float) * co);
      for (int x = 0; x < ow; ++x) {
        for (int c = 0; c < co; ++c) acc[c] = bias ? bias[c] : 0.f;
        for (int ky = 0; ky < kh; ++ky) {
          const int iy = y * stride + ky - pad;
          if (iy < 0 || iy >= h) continue;
          for (int kx = 0; kx < kw; ++kx) {
            const int ix = x * stride + kx - pad;
            if (ix < 0 || ix >= w) continue;
            const float* ip = in + (((size_t)b * h + iy) * w + ix) * ci;
            const float* fp = filt + ((size_t)ky * kw + kx) * ci * co;
            for (int c0 = 0; c0 < ci; ++c0) {
              const float v = ip[c0];
              const float* fr = fp + (size_t)c0 * co;
              for (int c = 0; c < co; ++c) acc[c] += v * fr[c];
            }
          }
        }
        float* op = out + (((size_t)b * oh + y) * ow + x) * co;
        for (int c = 0; c < co; ++c) op[c] = (relu && acc[c] < 0.f) ? 0.f : acc[c];
      }
      free(acc);
    }
  }
}

/* C[m,n] = sum_k A[m,k] * B[k,n], fp32, row-major */
void cpu_gemm_f32(const float* a, const float* b, float* c, int m, int n, int k) {
#pragma omp parallel for schedule(static)
  for (int i = 0; i < m; ++i) {
    float* cr = c + (size_t)i * n;
    memset(cr, 0, sizeof(float) * n);
    for (int p = 0; p < k; ++p) {
      const float v = a[(size_t)i * k + p];
      const float* br = b + (size_t)p * n;
      for (int j = 0; j < n; ++j) cr[j] += v * br[j];
    }
  }
}

/* C[m,n] = sum_k (int32)A[m,k] * (int32)B[k,n] */
void cpu_gemm_i8_i32(const int8_t* a, const int8_t* b, int32_t* c, int m, int n, int k) {
#pragma omp parallel for schedule(static)
  for (int i = 0; i < m; ++i) {
    int32_t* cr = c + (size_t)i * n;
    memset(cr, 0, sizeof(int32_t) * n);
    for (int p = 0; p < k; ++p) {
      const int32_t v = a[(size_t)i * k + p];
      const int8_t* br = b + (size_t)p * n;
      for (int j = 0; j < n; ++j) cr[j] += v * (int32_t)br[j];
    }
  }
}
