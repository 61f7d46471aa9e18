/*
 * oracle_gemm.cpp -- column-major GEMM used by the CPU oracle.  TEST INFRASTRUCTURE ONLY.
 *
 * The reference calls Fortran sgemm/dgemm from MATLAB's libmwblas (Intel MKL) through
 * bits/impl/blashelper.hpp:79-116.  That library is not part of the reference tree, so its
 * published contract is restated here: C <- alpha*op(A)*op(B) + beta*C, column-major, with
 * beta == 0 meaning "C is write-only" (NaNs in C are not propagated).  Summation order
 * inside the product is the library's own and is not pinned by the reference.
 *
 * Built-in kernels are blocked and threaded with OpenMP (the reference's BLAS is the only
 * threaded part of its CPU path).  An ILP64 Fortran gemm can be plugged in instead.
 */
#include "oracle.h"

#include <algorithm>
#include <cstring>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

typedef void (*ext_sgemm_t)(const char*, const char*, const int64_t*, const int64_t*, const int64_t*,
                            const float*, const float*, const int64_t*, const float*, const int64_t*,
                            const float*, float*, const int64_t*);
typedef void (*ext_dgemm_t)(const char*, const char*, const int64_t*, const int64_t*, const int64_t*,
                            const double*, const double*, const int64_t*, const double*, const int64_t*,
                            const double*, double*, const int64_t*);
ext_sgemm_t g_ext_sgemm = nullptr;
ext_dgemm_t g_ext_dgemm = nullptr;

inline bool is_t(char c) { return c == 't' || c == 'T'; }

template <typename T>
void scale_c(int64_t m, int64_t n, T beta, T* c, int64_t ldc) {
  for (int64_t j = 0; j < n; ++j) {
    T* cj = c + j * ldc;
    if (beta == T(0)) {
      std::memset(cj, 0, sizeof(T) * (size_t)m);
    } else if (beta != T(1)) {
      for (int64_t i = 0; i < m; ++i) cj[i] *= beta;
    }
  }
}

/* op(A) = A (m x k, column-major).  C(:,j) += alpha * sum_l A(:,l) * opB(l,j).
   Blocks: 4 columns of C, IB rows, LB reduction steps; the inner loop runs down a column of A. */
template <typename T>
void gemm_n(bool tb, int64_t m, int64_t n, int64_t k, T alpha, const T* a, int64_t lda,
            const T* b, int64_t ldb, T* c, int64_t ldc) {
  const int64_t IB = 512, LB = 128, JB = 4;
  const int64_t nJ = (n + JB - 1) / JB, nI = (m + IB - 1) / IB;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t jb = 0; jb < nJ; ++jb) {
    for (int64_t ib = 0; ib < nI; ++ib) {
      const int64_t j0 = jb * JB, jn = std::min<int64_t>(JB, n - j0);
      const int64_t i0 = ib * IB, in = std::min<int64_t>(IB, m - i0);
      T acc[JB][IB];
      for (int64_t jj = 0; jj < JB; ++jj)
        for (int64_t i = 0; i < in; ++i) acc[jj][i] = T(0);
      for (int64_t l0 = 0; l0 < k; l0 += LB) {
        const int64_t ln = std::min<int64_t>(LB, k - l0);
        for (int64_t l = l0; l < l0 + ln; ++l) {
          const T* al = a + l * lda + i0;
          T bv[JB];
          for (int64_t jj = 0; jj < JB; ++jj) {
            const int64_t j = j0 + (jj < jn ? jj : 0);
            bv[jj] = tb ? b[j + l * ldb] : b[l + j * ldb];
          }
#pragma omp simd
          for (int64_t i = 0; i < in; ++i) {
            const T av = al[i];
            acc[0][i] += av * bv[0];
            acc[1][i] += av * bv[1];
            acc[2][i] += av * bv[2];
            acc[3][i] += av * bv[3];
          }
        }
      }
      for (int64_t jj = 0; jj < jn; ++jj) {
        T* cj = c + (j0 + jj) * ldc + i0;
        for (int64_t i = 0; i < in; ++i) cj[i] += alpha * acc[jj][i];
      }
    }
  }
}

/* op(A) = A' with A stored k x m; op(B) = B stored k x n.  C(i,j) += alpha * <A(:,i), B(:,j)>.
   4 x 4 tiles of dot products, vectorised down the shared reduction axis. */
template <typename T>
void gemm_tn(int64_t m, int64_t n, int64_t k, T alpha, const T* a, int64_t lda, const T* b,
             int64_t ldb, T* c, int64_t ldc) {
  const int64_t TB = 4;
  const int64_t nI = (m + TB - 1) / TB, nJ = (n + TB - 1) / TB;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t jb = 0; jb < nJ; ++jb) {
    for (int64_t ib = 0; ib < nI; ++ib) {
      const int64_t i0 = ib * TB, j0 = jb * TB;
      const int64_t in = std::min<int64_t>(TB, m - i0), jn = std::min<int64_t>(TB, n - j0);
      const T* ap[TB];
      const T* bp[TB];
      for (int64_t t = 0; t < TB; ++t) {
        ap[t] = a + (i0 + (t < in ? t : 0)) * lda;
        bp[t] = b + (j0 + (t < jn ? t : 0)) * ldb;
      }
      T s00 = 0, s01 = 0, s02 = 0, s03 = 0, s10 = 0, s11 = 0, s12 = 0, s13 = 0;
      T s20 = 0, s21 = 0, s22 = 0, s23 = 0, s30 = 0, s31 = 0, s32 = 0, s33 = 0;
#pragma omp simd reduction(+ : s00, s01, s02, s03, s10, s11, s12, s13, s20, s21, s22, s23, s30, s31, s32, s33)
      for (int64_t p = 0; p < k; ++p) {
        const T a0 = ap[0][p], a1 = ap[1][p], a2 = ap[2][p], a3 = ap[3][p];
        const T b0 = bp[0][p], b1 = bp[1][p], b2 = bp[2][p], b3 = bp[3][p];
        s00 += a0 * b0; s01 += a0 * b1; s02 += a0 * b2; s03 += a0 * b3;
        s10 += a1 * b0; s11 += a1 * b1; s12 += a1 * b2; s13 += a1 * b3;
        s20 += a2 * b0; s21 += a2 * b1; s22 += a2 * b2; s23 += a2 * b3;
        s30 += a3 * b0; s31 += a3 * b1; s32 += a3 * b2; s33 += a3 * b3;
      }
      const T s[TB][TB] = {{s00, s01, s02, s03}, {s10, s11, s12, s13},
                           {s20, s21, s22, s23}, {s30, s31, s32, s33}};
      for (int64_t jj = 0; jj < jn; ++jj)
        for (int64_t ii = 0; ii < in; ++ii) c[(i0 + ii) + (j0 + jj) * ldc] += alpha * s[ii][jj];
    }
  }
}

/* Remaining transpose combination (A' * B'), not used by the convolution path; plain loops. */
template <typename T>
void gemm_tt(int64_t m, int64_t n, int64_t k, T alpha, const T* a, int64_t lda, const T* b,
             int64_t ldb, T* c, int64_t ldc) {
  for (int64_t j = 0; j < n; ++j)
    for (int64_t i = 0; i < m; ++i) {
      T s = 0;
      for (int64_t p = 0; p < k; ++p) s += a[p + i * lda] * b[j + p * ldb];
      c[i + j * ldc] += alpha * s;
    }
}

template <typename T>
void gemm_builtin(char ta, char tb, int64_t m, int64_t n, int64_t k, T alpha, const T* a,
                  int64_t lda, const T* b, int64_t ldb, T beta, T* c, int64_t ldc) {
  if (m <= 0 || n <= 0) return;
  scale_c(m, n, beta, c, ldc);
  if (k <= 0 || alpha == T(0)) return;
  if (!is_t(ta)) {
    gemm_n<T>(is_t(tb), m, n, k, alpha, a, lda, b, ldb, c, ldc);
  } else if (!is_t(tb)) {
    gemm_tn<T>(m, n, k, alpha, a, lda, b, ldb, c, ldc);
  } else {
    gemm_tt<T>(m, n, k, alpha, a, lda, b, ldb, c, ldc);
  }
}

}  // namespace

extern "C" {

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void oracle_set_sgemm(void* fn) { g_ext_sgemm = (ext_sgemm_t)fn; }
void oracle_set_dgemm(void* fn) { g_ext_dgemm = (ext_dgemm_t)fn; }

void oracle_gemm_f32(char ta, char tb, int64_t m, int64_t n, int64_t k, float alpha, const float* a,
                     int64_t lda, const float* b, int64_t ldb, float beta, float* c, int64_t ldc) {
  if (g_ext_sgemm) {
    g_ext_sgemm(&ta, &tb, &m, &n, &k, &alpha, a, &lda, b, &ldb, &beta, c, &ldc);
    return;
  }
  gemm_builtin<float>(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
}

void oracle_gemm_f64(char ta, char tb, int64_t m, int64_t n, int64_t k, double alpha,
                     const double* a, int64_t lda, const double* b, int64_t ldb, double beta,
                     double* c, int64_t ldc) {
  if (g_ext_dgemm) {
    g_ext_dgemm(&ta, &tb, &m, &n, &k, &alpha, a, &lda, b, &ldb, &beta, c, &ldc);
    return;
  }
  gemm_builtin<double>(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
}

}  // extern "C"
