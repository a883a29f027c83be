// TEST INFRASTRUCTURE -- C entry points onto the reference's own templates
// ulmBLAS::gemm (ulmblas/level3/gemm.tcc:13-87), trlsm and trusm, compiled from the reference
// headers where they lie (-I <reference root>) into oracle/_ref/.  This file
// holds no reference code; it only instantiates the three type combinations
// the BLAS interfaces use and hands element strides through unchanged.
#include <complex>
#include <ulmblas/ulmblas.h>
#include <ulmblas/lapack/getf2.h>
#include <ulmblas/lapack/getrf.h>
#include <ulmblas/lapack/laswp.h>

extern "C" {

// dgemm_ / cblas_dgemm arithmetic: everything double.
void ulmref_gemm_d(int m, int n, int k, double alpha, const double *A,
                   int incRowA, int incColA, const double *B, int incRowB,
                   int incColB, double beta, double *C, int incRowC,
                   int incColC)
{
    ulmBLAS::gemm(m, n, k, alpha, false, A, incRowA, incColA, false, B,
                  incRowB, incColB, beta, C, incRowC, incColC);
}

// cblas_sgemm arithmetic: everything float.
void ulmref_gemm_s(int m, int n, int k, float alpha, const float *A,
                   int incRowA, int incColA, const float *B, int incRowB,
                   int incColB, float beta, float *C, int incRowC,
                   int incColC)
{
    ulmBLAS::gemm(m, n, k, alpha, false, A, incRowA, incColA, false, B,
                  incRowB, incColB, beta, C, incRowC, incColC);
}

// sgemm_ arithmetic: float data, double alpha and beta.
void ulmref_gemm_s_f64(int m, int n, int k, double alpha, const float *A,
                       int incRowA, int incColA, const float *B, int incRowB,
                       int incColB, double beta, float *C, int incRowC,
                       int incColC)
{
    ulmBLAS::gemm(m, n, k, alpha, false, A, incRowA, incColA, false, B,
                  incRowB, incColB, beta, C, incRowC, incColC);
}

// Triangular solves: ulmBLAS::trlsm (lower) / ulmBLAS::trusm (upper),
// ulmblas/level3/trlsm.tcc:16-91 and trusm.tcc:18-100, in the three type
// combinations of dtrsm, cblas_strsm and strsm_.
void ulmref_trsm_d(int lower, int m, int n, double alpha, int unit,
                   const double *A, int incRowA, int incColA, double *B,
                   int incRowB, int incColB)
{
    if (lower) {
        ulmBLAS::trlsm(m, n, alpha, false, unit != 0, A, incRowA, incColA, B, incRowB, incColB);
    } else {
        ulmBLAS::trusm(m, n, alpha, false, unit != 0, A, incRowA, incColA, B, incRowB, incColB);
    }
}

void ulmref_trsm_s(int lower, int m, int n, float alpha, int unit,
                   const float *A, int incRowA, int incColA, float *B,
                   int incRowB, int incColB)
{
    if (lower) {
        ulmBLAS::trlsm(m, n, alpha, false, unit != 0, A, incRowA, incColA, B, incRowB, incColB);
    } else {
        ulmBLAS::trusm(m, n, alpha, false, unit != 0, A, incRowA, incColA, B, incRowB, incColB);
    }
}

void ulmref_trsm_s_f64(int lower, int m, int n, double alpha, int unit,
                       const float *A, int incRowA, int incColA, float *B,
                       int incRowB, int incColB)
{
    if (lower) {
        ulmBLAS::trlsm(m, n, alpha, false, unit != 0, A, incRowA, incColA, B, incRowB, incColB);
    } else {
        ulmBLAS::trusm(m, n, alpha, false, unit != 0, A, incRowA, incColA, B, incRowB, incColB);
    }
}

// zgemm_ / cblas_zgemm and cgemm_ / cblas_cgemm arithmetic: complex operands
// and scalars (interleaved re, im), conjugation flags passed through.
void ulmref_gemm_z(int m, int n, int k, const double *alpha, int conjA,
                   const double *A, int incRowA, int incColA, int conjB,
                   const double *B, int incRowB, int incColB,
                   const double *beta, double *C, int incRowC, int incColC)
{
    typedef std::complex<double> Z;
    ulmBLAS::gemm(m, n, k, Z(alpha[0], alpha[1]), conjA != 0, reinterpret_cast<const Z *>(A), incRowA, incColA,
                  conjB != 0, reinterpret_cast<const Z *>(B), incRowB, incColB, Z(beta[0], beta[1]),
                  reinterpret_cast<Z *>(C), incRowC, incColC);
}

void ulmref_gemm_c(int m, int n, int k, const float *alpha, int conjA,
                   const float *A, int incRowA, int incColA, int conjB,
                   const float *B, int incRowB, int incColB, const float *beta,
                   float *C, int incRowC, int incColC)
{
    typedef std::complex<float> Z;
    ulmBLAS::gemm(m, n, k, Z(alpha[0], alpha[1]), conjA != 0, reinterpret_cast<const Z *>(A), incRowA, incColA,
                  conjB != 0, reinterpret_cast<const Z *>(B), incRowB, incColB, Z(beta[0], beta[1]),
                  reinterpret_cast<Z *>(C), incRowC, incColC);
}

// Symmetric rank-k update (sylrk / syurk), symmetric product (sylmm / syumm)
// and triangular product (trlmm / trumm) on element strides, all double.
void ulmref_syrk_d(int lower, int n, int k, double alpha, const double *A,
                   int incRowA, int incColA, double beta, double *C,
                   int incRowC, int incColC)
{
    if (lower) {
        ulmBLAS::sylrk(n, k, alpha, A, incRowA, incColA, beta, C, incRowC, incColC);
    } else {
        ulmBLAS::syurk(n, k, alpha, A, incRowA, incColA, beta, C, incRowC, incColC);
    }
}

// sylr2k / syur2k; the reference reads B on A's strides, so callers pass
// operands whose strides agree.
void ulmref_syr2k_d(int lower, int n, int k, double alpha, const double *A,
                    int incRowA, int incColA, const double *B, int incRowB,
                    int incColB, double beta, double *C, int incRowC,
                    int incColC)
{
    if (lower) {
        ulmBLAS::sylr2k(n, k, alpha, A, incRowA, incColA, B, incRowB, incColB, beta, C, incRowC, incColC);
    } else {
        ulmBLAS::syur2k(n, k, alpha, A, incRowA, incColA, B, incRowB, incColB, beta, C, incRowC, incColC);
    }
}

void ulmref_symm_d(int lower, int m, int n, double alpha, const double *A,
                   int incRowA, int incColA, const double *B, int incRowB,
                   int incColB, double beta, double *C, int incRowC,
                   int incColC)
{
    if (lower) {
        ulmBLAS::sylmm(m, n, alpha, A, incRowA, incColA, B, incRowB, incColB, beta, C, incRowC, incColC);
    } else {
        ulmBLAS::syumm(m, n, alpha, A, incRowA, incColA, B, incRowB, incColB, beta, C, incRowC, incColC);
    }
}

void ulmref_trmm_d(int lower, int m, int n, double alpha, int unit,
                   const double *A, int incRowA, int incColA, double *B,
                   int incRowB, int incColB)
{
    if (lower) {
        ulmBLAS::trlmm(m, n, alpha, false, unit != 0, A, incRowA, incColA, B, incRowB, incColB);
    } else {
        ulmBLAS::trumm(m, n, alpha, false, unit != 0, A, incRowA, incColA, B, incRowB, incColB);
    }
}

// LU: ulmBLAS::getrf (ulmblas/lapack/getrf.tcc:14-75) and ulmBLAS::laswp
// (ulmblas/lapack/laswp.tcc:13-55) on element strides.
int ulmref_getrf_d(int m, int n, double *A, int incRowA, int incColA, int *piv,
                   int incPiv)
{
    return ulmBLAS::getrf(m, n, A, incRowA, incColA, piv, incPiv);
}

int ulmref_getf2_d(int m, int n, double *A, int incRowA, int incColA, int *piv,
                   int incPiv)
{
    return ulmBLAS::getf2(m, n, A, incRowA, incColA, piv, incPiv);
}

void ulmref_laswp_d(int n, double *A, int incRowA, int incColA, int k1, int k2,
                    int *piv, int incPiv)
{
    ulmBLAS::laswp(n, A, incRowA, incColA, k1, k2, piv, incPiv);
}

// Block sizes this build was compiled with (production or USE_TESTPARAM).
void ulmref_blocksize_d(int *out)
{
    out[0] = ulmBLAS::BlockSize<double>::MC;
    out[1] = ulmBLAS::BlockSize<double>::KC;
    out[2] = ulmBLAS::BlockSize<double>::NC;
    out[3] = ulmBLAS::BlockSizeUGemm<double>::MR;
    out[4] = ulmBLAS::BlockSizeUGemm<double>::NR;
}

void ulmref_blocksize_s(int *out)
{
    out[0] = ulmBLAS::BlockSize<float>::MC;
    out[1] = ulmBLAS::BlockSize<float>::KC;
    out[2] = ulmBLAS::BlockSize<float>::NC;
    out[3] = ulmBLAS::BlockSizeUGemm<float>::MR;
    out[4] = ulmBLAS::BlockSizeUGemm<float>::NR;
}

} // extern "C"
