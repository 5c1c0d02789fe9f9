// C entry points over the reference's own CPU arithmetic, compiled from the
// reference sources where they lie (never copied): src/my_blas/my_cblas.cpp
// (internal BLAS used when no OpenBLAS is found, CMakeLists.txt:152-161) and the
// header-only include/dlprim/cpu/cpu_ops.hpp.  TEST INFRASTRUCTURE ONLY: used to
// validate the C restatement in dlp_oracle.c; never loaded by the shipped library.
//
// The Convolution2D / InnerProduct operator classes themselves cannot be built
// here without generated files (dlprim/config.hpp from CMake, kernels.cpp from
// build_source.py), so only these two self-contained pieces are compiled.
#include <my_cblas.hpp>
#include <dlprim/cpu/cpu_ops.hpp>
#include <cstddef>

extern "C" {

// dlprim::my_cblas::cblas_sgemm, src/my_blas/my_cblas.cpp:88-103 (row-major)
void ref_cblas_sgemm(int trans_a, int trans_b, int M, int N, int K, float alpha,
                     const float *A, int lda, const float *B, int ldb, float beta, float *C, int ldc)
{
    dlprim::cblas_sgemm(dlprim::CblasRowMajor, trans_a != 0, trans_b != 0, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
}

// dlprim::my_cblas::cblas_saxpy, src/my_blas/my_cblas.cpp:18-22
void ref_cblas_saxpy(int n, float a, float *x, int lx, float *y, int ly)
{
    dlprim::cblas_saxpy(n, a, x, lx, y, ly);
}

// dlprim::cpu::apply_activation<float>, include/dlprim/cpu/cpu_ops.hpp:17-53
void ref_apply_activation(float *p, size_t n, int activation)
{
    dlprim::cpu::apply_activation(p, n, static_cast<dlprim::StandardActivations>(activation));
}

}
