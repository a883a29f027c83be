// TEST INFRASTRUCTURE -- C entry points onto the reference's own template
// ulmBLAS::gemm (ulmblas/level3/gemm.tcc:13-87), compiled from the reference
// headers where they lie (-I <reference root>) into oracle/_ref/.  This file
// holds no reference code; it only instantiates the three type combinations
// the BLAS interfaces use and hands element strides through unchanged.
#include <ulmblas/ulmblas.h>

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
