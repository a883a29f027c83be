/*
 * TEST INFRASTRUCTURE -- CPU restatement of ulmBLAS's GEMM path; see
 * ulm_gemm_oracle.h.  Build with -ffp-contract=off and without -march flags
 * that enable FMA so the roundings match the reference's portable build.
 */
#include "ulm_gemm_oracle.h"

#include <complex.h>
#include <ctype.h>
#include <float.h>
#include <math.h>
#include <stdlib.h>

typedef long idx;

#define ORACLE_MAX_MR 16
#define ORACLE_MAX_NR 16

#define ORACLE_CAT_(a, b) a##b
#define ORACLE_CAT(a, b) ORACLE_CAT_(a, b)

/* all double: dgemm_, cblas_dgemm */
#define T double
#define TAB double
#define TC double
#define SC double
#define ORACLE_SAME_TYPE 1
#define FN(x) ORACLE_CAT(d_, x)
#include "ulm_gemm_frame.inc"
#include "ulm_trsm_frame.inc"
#include "ulm_l3_frame.inc"
#include "ulm_lu_frame.inc"
#undef T
#undef TAB
#undef TC
#undef SC
#undef ORACLE_SAME_TYPE
#undef FN

/* all float: cblas_sgemm (interfaces/blas/C/gemm.cc:295-389 passes float
 * alpha/beta, so the compute type of gemm.tcc:33 is float) */
#define T float
#define TAB float
#define TC float
#define SC float
#define ORACLE_SAME_TYPE 1
#define FN(x) ORACLE_CAT(s_, x)
#include "ulm_gemm_frame.inc"
#include "ulm_trsm_frame.inc"
#include "ulm_l3_frame.inc"
#undef T
#undef TAB
#undef TC
#undef SC
#undef ORACLE_SAME_TYPE
#undef FN

/* float data, double scalars: sgemm_ (interfaces/blas/F77/gemm.cc:33,36 copy
 * alpha and beta into doubles, so the compute type is double and every tile
 * goes through the buffered micro-kernel, ukernel/ugemm.tcc:44-61) */
#define T double
#define TAB float
#define TC float
#define SC double
#define ORACLE_SAME_TYPE 0
#define FN(x) ORACLE_CAT(sd_, x)
#include "ulm_gemm_frame.inc"
#include "ulm_trsm_frame.inc"
#include "ulm_l3_frame.inc"
#undef T
#undef TAB
#undef TC
#undef SC
#undef ORACLE_SAME_TYPE
#undef FN

/* complex double and complex float: zgemm_ / cblas_zgemm and cgemm_ /
 * cblas_cgemm (interfaces/blas/F77/gemm.cc:251-506, interfaces/blas/C/gemm.cc:
 * 140-293, 488-690).  The same frame on complex numbers: the compiler's complex
 * multiply is the one std::complex's operators use, so sums and products round
 * alike.  Only the GEMM frame is instantiated. */
#define T double _Complex
#define TAB double _Complex
#define TC double _Complex
#define SC double _Complex
#define ORACLE_SAME_TYPE 1
#define FN(x) ORACLE_CAT(z_, x)
#include "ulm_gemm_frame.inc"
#undef T
#undef TAB
#undef TC
#undef SC
#undef ORACLE_SAME_TYPE
#undef FN

#define T float _Complex
#define TAB float _Complex
#define TC float _Complex
#define SC float _Complex
#define ORACLE_SAME_TYPE 1
#define FN(x) ORACLE_CAT(c_, x)
#include "ulm_gemm_frame.inc"
#undef T
#undef TAB
#undef TC
#undef SC
#undef ORACLE_SAME_TYPE
#undef FN

/* ulmblas/config/blocksize.h:66-103 */
void ulm_oracle_default_blocksize_d(ulm_oracle_blocksize *bs)
{
    bs->MC = 384; bs->KC = 384; bs->NC = 4096; bs->MR = 4; bs->NR = 4;
}

void ulm_oracle_default_blocksize_s(ulm_oracle_blocksize *bs)
{
    bs->MC = 768; bs->KC = 384; bs->NC = 4096; bs->MR = 8; bs->NR = 4;
}

int ulm_oracle_gemm_d(long m, long n, long k, double alpha, const double *A,
                      long incRowA, long incColA, const double *B,
                      long incRowB, long incColB, double beta, double *C,
                      long incRowC, long incColC,
                      const ulm_oracle_blocksize *bs)
{
    ulm_oracle_blocksize def;
    if (!bs) { ulm_oracle_default_blocksize_d(&def); bs = &def; }
    return d_gemm(m, n, k, alpha, A, incRowA, incColA, B, incRowB, incColB,
                  beta, C, incRowC, incColC, bs);
}

int ulm_oracle_gemm_s(long m, long n, long k, float alpha, const float *A,
                      long incRowA, long incColA, const float *B,
                      long incRowB, long incColB, float beta, float *C,
                      long incRowC, long incColC,
                      const ulm_oracle_blocksize *bs)
{
    ulm_oracle_blocksize def;
    if (!bs) { ulm_oracle_default_blocksize_s(&def); bs = &def; }
    return s_gemm(m, n, k, alpha, A, incRowA, incColA, B, incRowB, incColB,
                  beta, C, incRowC, incColC, bs);
}

int ulm_oracle_gemm_s_f64(long m, long n, long k, double alpha, const float *A,
                          long incRowA, long incColA, const float *B,
                          long incRowB, long incColB, double beta, float *C,
                          long incRowC, long incColC,
                          const ulm_oracle_blocksize *bs)
{
    ulm_oracle_blocksize def;
    if (!bs) { ulm_oracle_default_blocksize_d(&def); bs = &def; }
    return sd_gemm(m, n, k, alpha, A, incRowA, incColA, B, incRowB, incColB,
                   beta, C, incRowC, incColC, bs);
}

/* ulmblas/config/blocksize.h:66-103, the complex rows */
void ulm_oracle_default_blocksize_z(ulm_oracle_blocksize *bs)
{
    bs->MC = 192; bs->KC = 192; bs->NC = 4096; bs->MR = 2; bs->NR = 2;
}

void ulm_oracle_default_blocksize_c(ulm_oracle_blocksize *bs)
{
    bs->MC = 384; bs->KC = 384; bs->NC = 4096; bs->MR = 4; bs->NR = 2;
}

/* ulmBLAS::gemm with conjugation flags (ulmblas/level3/gemm.tcc:13-87): the
 * flags reach gepack_A / gepack_B (:67,74), which store conjugate(x) instead
 * of x (pack/gepack.tcc:21-37,84-100).  Conjugation is exact, so packing a
 * conjugated copy of the operand window fills the same buffers. */
#define ORACLE_COMPLEX_EXPORT(SUF, PRE, R, CONJ, DEFBS)                       \
    static R _Complex *PRE##conj_copy(long rows, long cols, const R _Complex *X, \
                                      long incRow, long incCol)               \
    {                                                                         \
        size_t count = (size_t)(rows > 0 ? rows : 0) * (size_t)(cols > 0 ? cols : 0); \
        R _Complex *Y = (R _Complex *)malloc(sizeof(R _Complex) * (count ? count : 1)); \
        if (!Y) return NULL;                                                  \
        for (long j = 0; j < cols; ++j)                                       \
            for (long i = 0; i < rows; ++i)                                   \
                Y[i + j * rows] = CONJ(X[i * incRow + j * incCol]);           \
        return Y;                                                             \
    }                                                                         \
    int ulm_oracle_gemm_##SUF(long m, long n, long k, const R *alpha,         \
                              int conjA, const R *A, long incRowA,            \
                              long incColA, int conjB, const R *B,            \
                              long incRowB, long incColB, const R *beta,      \
                              R *C, long incRowC, long incColC,               \
                              const ulm_oracle_blocksize *bs)                 \
    {                                                                         \
        ulm_oracle_blocksize def;                                             \
        if (!bs) { DEFBS(&def); bs = &def; }                                  \
        const R _Complex al = alpha[0] + alpha[1] * _Complex_I;               \
        const R _Complex be = beta[0] + beta[1] * _Complex_I;                 \
        const R _Complex *Ac = (const R _Complex *)A;                         \
        const R _Complex *Bc = (const R _Complex *)B;                         \
        R _Complex *Af = NULL, *Bf = NULL;                                    \
        if (conjA && m > 0 && k > 0) {                                        \
            Af = PRE##conj_copy(m, k, Ac, incRowA, incColA);                  \
            if (!Af) return -2;                                               \
            Ac = Af; incRowA = 1; incColA = m;                                \
        }                                                                     \
        if (conjB && k > 0 && n > 0) {                                        \
            Bf = PRE##conj_copy(k, n, Bc, incRowB, incColB);                  \
            if (!Bf) { free(Af); return -2; }                                 \
            Bc = Bf; incRowB = 1; incColB = k;                                \
        }                                                                     \
        int rc = PRE##gemm(m, n, k, al, Ac, incRowA, incColA, Bc, incRowB,    \
                           incColB, be, (R _Complex *)C, incRowC, incColC,    \
                           bs);                                               \
        free(Af);                                                             \
        free(Bf);                                                             \
        return rc;                                                            \
    }
ORACLE_COMPLEX_EXPORT(z, z_, double, conj, ulm_oracle_default_blocksize_z)
ORACLE_COMPLEX_EXPORT(c, c_, float, conjf, ulm_oracle_default_blocksize_c)

static int imax(int a, int b) { return a > b ? a : b; }

/* interfaces/blas/F77/gemm.cc:149-195 (same text for sgemm_ :27-73) */
int ulm_oracle_f77_gemm_info(char transA_, char transB_, int m, int n, int k,
                             int ldA, int ldB, int ldC)
{
    int ta = toupper((unsigned char)transA_);
    int tb = toupper((unsigned char)transB_);
    int transA = (ta == 'T' || ta == 'C');
    int transB = (tb == 'T' || tb == 'C');
    int numRowsA = (!transA) ? m : k;
    int numRowsB = (!transB) ? k : n;

    if (ta != 'N' && ta != 'T' && ta != 'C' && ta != 'R') return 1;
    if (tb != 'N' && tb != 'T' && tb != 'C' && tb != 'R') return 2;
    if (m < 0) return 3;
    if (n < 0) return 4;
    if (k < 0) return 5;
    if (ldA < imax(1, numRowsA)) return 8;
    if (ldB < imax(1, numRowsB)) return 10;
    if (ldC < imax(1, m)) return 13;
    return 0;
}

static int cblas_notrans(int t)
{
    return t == ULM_ORACLE_NO_TRANS || t == ULM_ORACLE_ATLAS_CONJ;
}

static int cblas_trans_valid(int t)
{
    return t == ULM_ORACLE_NO_TRANS || t == ULM_ORACLE_TRANS ||
           t == ULM_ORACLE_ATLAS_CONJ || t == ULM_ORACLE_CONJ_TRANS;
}

/* interfaces/blas/C/gemm.cc:410-466 (same text for cblas_sgemm :314-370) */
int ulm_oracle_cblas_gemm_info(int order, int transA, int transB, int m, int n,
                               int k, int ldA, int ldB, int ldC)
{
    int numRowsA, numRowsB;
    if (order == ULM_ORACLE_COL_MAJOR) {
        numRowsA = cblas_notrans(transA) ? m : k;
        numRowsB = cblas_notrans(transB) ? k : n;
    } else {
        numRowsB = cblas_notrans(transB) ? n : k;
        numRowsA = cblas_notrans(transA) ? k : m;
    }
    if (order != ULM_ORACLE_COL_MAJOR && order != ULM_ORACLE_ROW_MAJOR)
        return 1;
    if (!cblas_trans_valid(transA)) return 2;
    if (!cblas_trans_valid(transB)) return 3;
    if (order == ULM_ORACLE_COL_MAJOR) {
        if (m < 0) return 4;
        if (n < 0) return 5;
        if (k < 0) return 6;
        if (ldA < imax(1, numRowsA)) return 9;
        if (ldB < imax(1, numRowsB)) return 11;
        if (ldC < imax(1, m)) return 14;
    } else {
        if (n < 0) return 4;
        if (m < 0) return 5;
        if (k < 0) return 6;
        if (ldB < imax(1, numRowsB)) return 9;
        if (ldA < imax(1, numRowsA)) return 11;
        if (ldC < imax(1, n)) return 14;
    }
    return 0;
}

/* Strides of op(X) for a column-major X: not transposed (1, ld), transposed
 * (ld, 1) -- interfaces/blas/F77/gemm.cc:204-248. */
static void op_strides(int trans, long ld, long *incRow, long *incCol)
{
    *incRow = trans ? ld : 1;
    *incCol = trans ? 1 : ld;
}

int ulm_oracle_dgemm_f77(char transA_, char transB_, int m, int n, int k,
                         double alpha, const double *A, int ldA,
                         const double *B, int ldB, double beta, double *C,
                         int ldC)
{
    int info = ulm_oracle_f77_gemm_info(transA_, transB_, m, n, k, ldA, ldB,
                                        ldC);
    if (info) return info;
    int ta = toupper((unsigned char)transA_);
    int tb = toupper((unsigned char)transB_);
    long ra, ca, rb, cb;
    op_strides(ta == 'T' || ta == 'C', ldA, &ra, &ca);
    op_strides(tb == 'T' || tb == 'C', ldB, &rb, &cb);
    ulm_oracle_gemm_d(m, n, k, alpha, A, ra, ca, B, rb, cb, beta, C, 1, ldC,
                      NULL);
    return 0;
}

int ulm_oracle_sgemm_f77(char transA_, char transB_, int m, int n, int k,
                         float alpha, const float *A, int ldA, const float *B,
                         int ldB, float beta, float *C, int ldC)
{
    int info = ulm_oracle_f77_gemm_info(transA_, transB_, m, n, k, ldA, ldB,
                                        ldC);
    if (info) return info;
    int ta = toupper((unsigned char)transA_);
    int tb = toupper((unsigned char)transB_);
    long ra, ca, rb, cb;
    op_strides(ta == 'T' || ta == 'C', ldA, &ra, &ca);
    op_strides(tb == 'T' || tb == 'C', ldB, &rb, &cb);
    /* interfaces/blas/F77/gemm.cc:33,36: double alpha = *alpha_ */
    ulm_oracle_gemm_s_f64(m, n, k, (double)alpha, A, ra, ca, B, rb, cb,
                          (double)beta, C, 1, ldC, NULL);
    return 0;
}

/* interfaces/blas/C/gemm.cc:472-484: row-major is computed as the
 * column-major product of the swapped operands, C^T = op(B)^T op(A)^T. */
int ulm_oracle_cblas_dgemm(int order, int transA, int transB, int m, int n,
                           int k, double alpha, const double *A, int ldA,
                           const double *B, int ldB, double beta, double *C,
                           int ldC)
{
    int info = ulm_oracle_cblas_gemm_info(order, transA, transB, m, n, k, ldA,
                                          ldB, ldC);
    if (info) return info;
    long ra, ca, rb, cb;
    if (order == ULM_ORACLE_COL_MAJOR) {
        op_strides(!cblas_notrans(transA), ldA, &ra, &ca);
        op_strides(!cblas_notrans(transB), ldB, &rb, &cb);
        ulm_oracle_gemm_d(m, n, k, alpha, A, ra, ca, B, rb, cb, beta, C, 1,
                          ldC, NULL);
    } else {
        op_strides(!cblas_notrans(transB), ldB, &rb, &cb);
        op_strides(!cblas_notrans(transA), ldA, &ra, &ca);
        ulm_oracle_gemm_d(n, m, k, alpha, B, rb, cb, A, ra, ca, beta, C, 1,
                          ldC, NULL);
    }
    return 0;
}

int ulm_oracle_cblas_sgemm(int order, int transA, int transB, int m, int n,
                           int k, float alpha, const float *A, int ldA,
                           const float *B, int ldB, float beta, float *C,
                           int ldC)
{
    int info = ulm_oracle_cblas_gemm_info(order, transA, transB, m, n, k, ldA,
                                          ldB, ldC);
    if (info) return info;
    long ra, ca, rb, cb;
    if (order == ULM_ORACLE_COL_MAJOR) {
        op_strides(!cblas_notrans(transA), ldA, &ra, &ca);
        op_strides(!cblas_notrans(transB), ldB, &rb, &cb);
        ulm_oracle_gemm_s(m, n, k, alpha, A, ra, ca, B, rb, cb, beta, C, 1,
                          ldC, NULL);
    } else {
        op_strides(!cblas_notrans(transB), ldB, &rb, &cb);
        op_strides(!cblas_notrans(transA), ldA, &ra, &ca);
        ulm_oracle_gemm_s(n, m, k, alpha, B, rb, cb, A, ra, ca, beta, C, 1,
                          ldC, NULL);
    }
    return 0;
}

int ulm_oracle_gemm_samples(int variant, char transA_, char transB_, long m,
                            long n, long k, double alpha, const void *A,
                            long ldA, const void *B, long ldB, double beta,
                            const void *C, long ldC, long nsamples,
                            const long *rows, const long *cols, void *out,
                            double *gauge)
{
    int ta = toupper((unsigned char)transA_);
    int tb = toupper((unsigned char)transB_);
    long ra, ca, rb, cb;
    op_strides(ta == 'T' || ta == 'C', ldA, &ra, &ca);
    op_strides(tb == 'T' || tb == 'C', ldB, &rb, &cb);
    if (variant < 0 || variant > 2) return -1;

    for (long s = 0; s < nsamples; ++s) {
        long i = rows[s], j = cols[s];
        if (i < 0 || i >= m || j < 0 || j >= n) return -3;
        double g = 0.0, c0;
        if (variant == 0) {
            const double *a = (const double *)A + i * ra;
            const double *b = (const double *)B + j * cb;
            c0 = ((const double *)C)[i + j * ldC];
            ((double *)out)[s] =
                d_element(k, alpha, a, ca, b, rb, beta, c0, 384);
            for (long l = 0; l < k; ++l) g += fabs(a[l * ca]) * fabs(b[l * rb]);
        } else {
            const float *a = (const float *)A + i * ra;
            const float *b = (const float *)B + j * cb;
            float c0f = ((const float *)C)[i + j * ldC];
            c0 = c0f;
            if (variant == 1) {
                ((float *)out)[s] = s_element(k, (float)alpha, a, ca, b, rb,
                                              (float)beta, c0f, 384);
            } else {
                ((float *)out)[s] =
                    sd_element(k, alpha, a, ca, b, rb, beta, c0f, 384);
            }
            for (long l = 0; l < k; ++l)
                g += fabs((double)a[l * ca]) * fabs((double)b[l * rb]);
        }
        if (alpha == 0.0 || k == 0) g = 0.0;
        /* the gauge reads c only where the result depends on it */
        gauge[s] = fabs(alpha) * g + (beta == 0.0 ? 0.0 : fabs(beta) * fabs(c0));
    }
    return 0;
}

/* ---------------------------------------------------------------------- *
 * Triangular solve
 * ---------------------------------------------------------------------- */

int ulm_oracle_trsm_d(int lower, long m, long n, double alpha, int unit,
                      const double *A, long incRowA, long incColA, double *B,
                      long incRowB, long incColB,
                      const ulm_oracle_blocksize *bs)
{
    ulm_oracle_blocksize def;
    if (!bs) { ulm_oracle_default_blocksize_d(&def); bs = &def; }
    return d_trsm(lower, m, n, alpha, unit, A, incRowA, incColA, B, incRowB,
                  incColB, bs);
}

int ulm_oracle_trsm_s(int lower, long m, long n, float alpha, int unit,
                      const float *A, long incRowA, long incColA, float *B,
                      long incRowB, long incColB,
                      const ulm_oracle_blocksize *bs)
{
    ulm_oracle_blocksize def;
    if (!bs) { ulm_oracle_default_blocksize_s(&def); bs = &def; }
    return s_trsm(lower, m, n, alpha, unit, A, incRowA, incColA, B, incRowB,
                  incColB, bs);
}

int ulm_oracle_trsm_s_f64(int lower, long m, long n, double alpha, int unit,
                          const float *A, long incRowA, long incColA, float *B,
                          long incRowB, long incColB,
                          const ulm_oracle_blocksize *bs)
{
    ulm_oracle_blocksize def;
    if (!bs) { ulm_oracle_default_blocksize_d(&def); bs = &def; }
    return sd_trsm(lower, m, n, alpha, unit, A, incRowA, incColA, B, incRowB,
                   incColB, bs);
}

/* interfaces/blas/F77/trsm.cc:154-174 (same text for strsm_ :37-57) */
int ulm_oracle_f77_trsm_info(char side_, char upLo_, char transA_, char diag_,
                             int m, int n, int ldA, int ldB)
{
    int sd = toupper((unsigned char)side_);
    int ul = toupper((unsigned char)upLo_);
    int ta = toupper((unsigned char)transA_);
    int dg = toupper((unsigned char)diag_);
    int numRowsA = (sd == 'L') ? m : n;

    if (sd != 'L' && sd != 'R') return 1;
    if (ul != 'L' && ul != 'U') return 2;
    if (ta != 'N' && ta != 'T' && ta != 'C' && ta != 'R') return 3;
    if (dg != 'U' && dg != 'N') return 4;
    if (m < 0) return 5;
    if (n < 0) return 6;
    if (ldA < imax(1, numRowsA)) return 9;
    if (ldB < imax(1, m)) return 11;
    return 0;
}

/* interfaces/blas/C/trsm.cc:400-446 (same text for cblas_strsm) */
int ulm_oracle_cblas_trsm_info(int order, int side, int upLo, int transA,
                               int diag, int m, int n, int ldA, int ldB)
{
    int numRowsA = (side == ULM_ORACLE_LEFT) ? m : n;
    if (order != ULM_ORACLE_COL_MAJOR && order != ULM_ORACLE_ROW_MAJOR)
        return 1;
    if (side != ULM_ORACLE_LEFT && side != ULM_ORACLE_RIGHT) return 2;
    if (upLo != ULM_ORACLE_LOWER && upLo != ULM_ORACLE_UPPER) return 3;
    if (!cblas_trans_valid(transA)) return 4;
    if (diag != ULM_ORACLE_UNIT && diag != ULM_ORACLE_NON_UNIT) return 5;
    if (order == ULM_ORACLE_COL_MAJOR) {
        if (m < 0) return 6;
        if (n < 0) return 7;
        if (ldA < imax(1, numRowsA)) return 10;
        if (ldB < imax(1, m)) return 12;
    } else {
        if (n < 0) return 6;
        if (m < 0) return 7;
        if (ldA < imax(1, numRowsA)) return 10;
        if (ldB < imax(1, n)) return 12;
    }
    return 0;
}

/* The dispatch of interfaces/blas/F77/trsm.cc:183-227 and
 * interfaces/blas/C/trsm.cc:108-152: which solver runs on which strides.
 * left:  op(A) X = alpha B  -- lower/notrans and upper/trans are forward
 *        solves (trlsm), the other two backward (trusm); transposition is a
 *        swap of A's strides.
 * right: X op(A) = alpha B is solved as op(A)^T X^T = alpha B^T: B's strides
 *        swap, m and n swap, and the roles of lower and upper swap. */
#define ORACLE_TRSM_DISPATCH(SOLVE)                                           \
    if (left) {                                                               \
        if (lower) {                                                          \
            if (!trans) return SOLVE(1, m, n, alpha, unit, A, 1, ldA, B, 1, ldB, NULL); \
            return SOLVE(0, m, n, alpha, unit, A, ldA, 1, B, 1, ldB, NULL);   \
        }                                                                     \
        if (!trans) return SOLVE(0, m, n, alpha, unit, A, 1, ldA, B, 1, ldB, NULL); \
        return SOLVE(1, m, n, alpha, unit, A, ldA, 1, B, 1, ldB, NULL);       \
    }                                                                         \
    if (lower) {                                                              \
        if (!trans) return SOLVE(0, n, m, alpha, unit, A, ldA, 1, B, ldB, 1, NULL); \
        return SOLVE(1, n, m, alpha, unit, A, 1, ldA, B, ldB, 1, NULL);       \
    }                                                                         \
    if (!trans) return SOLVE(1, n, m, alpha, unit, A, ldA, 1, B, ldB, 1, NULL); \
    return SOLVE(0, n, m, alpha, unit, A, 1, ldA, B, ldB, 1, NULL);

static int dispatch_trsm_d(int left, int lower, int trans, int unit, int m,
                           int n, double alpha, const double *A, int ldA,
                           double *B, int ldB)
{
    ORACLE_TRSM_DISPATCH(ulm_oracle_trsm_d)
}

static int dispatch_trsm_s(int left, int lower, int trans, int unit, int m,
                           int n, float alpha, const float *A, int ldA,
                           float *B, int ldB)
{
    ORACLE_TRSM_DISPATCH(ulm_oracle_trsm_s)
}

static int dispatch_trsm_s_f64(int left, int lower, int trans, int unit, int m,
                               int n, double alpha, const float *A, int ldA,
                               float *B, int ldB)
{
    ORACLE_TRSM_DISPATCH(ulm_oracle_trsm_s_f64)
}

int ulm_oracle_dtrsm_f77(char side, char upLo, char transA, char diag, int m,
                         int n, double alpha, const double *A, int ldA,
                         double *B, int ldB)
{
    int info = ulm_oracle_f77_trsm_info(side, upLo, transA, diag, m, n, ldA,
                                        ldB);
    if (info) return info;
    int ta = toupper((unsigned char)transA);
    dispatch_trsm_d(toupper((unsigned char)side) == 'L',
                    toupper((unsigned char)upLo) == 'L',
                    ta == 'T' || ta == 'C',
                    toupper((unsigned char)diag) == 'U', m, n, alpha, A, ldA,
                    B, ldB);
    return 0;
}

/* interfaces/blas/F77/trsm.cc:29: double alpha = *alpha_, so strsm_ computes
 * in double on float data. */
int ulm_oracle_strsm_f77(char side, char upLo, char transA, char diag, int m,
                         int n, float alpha, const float *A, int ldA, float *B,
                         int ldB)
{
    int info = ulm_oracle_f77_trsm_info(side, upLo, transA, diag, m, n, ldA,
                                        ldB);
    if (info) return info;
    int ta = toupper((unsigned char)transA);
    dispatch_trsm_s_f64(toupper((unsigned char)side) == 'L',
                        toupper((unsigned char)upLo) == 'L',
                        ta == 'T' || ta == 'C',
                        toupper((unsigned char)diag) == 'U', m, n,
                        (double)alpha, A, ldA, B, ldB);
    return 0;
}

/* interfaces/blas/C/trsm.cc:452-458: row-major swaps side, uplo and m, n. */
int ulm_oracle_cblas_dtrsm(int order, int side, int upLo, int transA, int diag,
                           int m, int n, double alpha, const double *A,
                           int ldA, double *B, int ldB)
{
    int info = ulm_oracle_cblas_trsm_info(order, side, upLo, transA, diag, m,
                                          n, ldA, ldB);
    if (info) return info;
    int left = side == ULM_ORACLE_LEFT, lower = upLo == ULM_ORACLE_LOWER;
    int trans = transA == ULM_ORACLE_TRANS || transA == ULM_ORACLE_CONJ_TRANS;
    if (order == ULM_ORACLE_COL_MAJOR) {
        dispatch_trsm_d(left, lower, trans, diag == ULM_ORACLE_UNIT, m, n,
                        alpha, A, ldA, B, ldB);
    } else {
        dispatch_trsm_d(!left, !lower, trans, diag == ULM_ORACLE_UNIT, n, m,
                        alpha, A, ldA, B, ldB);
    }
    return 0;
}

int ulm_oracle_cblas_strsm(int order, int side, int upLo, int transA, int diag,
                           int m, int n, float alpha, const float *A, int ldA,
                           float *B, int ldB)
{
    int info = ulm_oracle_cblas_trsm_info(order, side, upLo, transA, diag, m,
                                          n, ldA, ldB);
    if (info) return info;
    int left = side == ULM_ORACLE_LEFT, lower = upLo == ULM_ORACLE_LOWER;
    int trans = transA == ULM_ORACLE_TRANS || transA == ULM_ORACLE_CONJ_TRANS;
    if (order == ULM_ORACLE_COL_MAJOR) {
        dispatch_trsm_s(left, lower, trans, diag == ULM_ORACLE_UNIT, m, n,
                        alpha, A, ldA, B, ldB);
    } else {
        dispatch_trsm_s(!left, !lower, trans, diag == ULM_ORACLE_UNIT, n, m,
                        alpha, A, ldA, B, ldB);
    }
    return 0;
}

/* ---------------------------------------------------------------------- *
 * LU factorisation
 * ---------------------------------------------------------------------- */

int ulm_oracle_getrf_d(long m, long n, double *A, long incRowA, long incColA,
                       int *piv, long incPiv, long nb,
                       const ulm_oracle_blocksize *bs)
{
    ulm_oracle_blocksize def;
    if (!bs) { ulm_oracle_default_blocksize_d(&def); bs = &def; }
    if (nb <= 0) nb = 64;     /* ulmblas/lapack/laenv.tcc:29-33 */
    return (int)lu_getrf(m, n, A, incRowA, incColA, piv, incPiv, nb, bs);
}

int ulm_oracle_getf2_d(long m, long n, double *A, long incRowA, long incColA,
                       int *piv, long incPiv)
{
    return (int)lu_getf2(m, n, A, incRowA, incColA, piv, incPiv);
}

void ulm_oracle_laswp_d(long n, double *A, long incRowA, long incColA, long k1,
                        long k2, const int *piv, long incPiv)
{
    lu_laswp(n, A, incRowA, incColA, k1, k2, piv, incPiv);
}

/* interfaces/lapack/C/getrf.cc:7-19: column-major factors the m x n matrix;
 * the row-major branch hands (n, m) and the strides (ldA, 1) to the same
 * routine. */
int ulm_oracle_dgetrf(int order, int m, int n, double *A, int ldA, int *piv)
{
    if (order == ULM_ORACLE_COL_MAJOR) {
        return ulm_oracle_getrf_d(m, n, A, 1, ldA, piv, 1, 0, NULL);
    }
    return ulm_oracle_getrf_d(n, m, A, ldA, 1, piv, 1, 0, NULL);
}

/* interfaces/lapack/C/laswp.cc:7-18 */
void ulm_oracle_dlaswp(int n, double *A, int ldA, int k1, int k2,
                       const int *piv, int incPiv)
{
    lu_laswp(n, A, 1, ldA, k1, k2, piv, incPiv);
}

/* ---------------------------------------------------------------------- *
 * Symmetric rank-k update, symmetric product, triangular product
 * ---------------------------------------------------------------------- */

#define ORACLE_L3_EXPORTS(SUF, PRE, TS, TD, DEFBS)                            \
    int ulm_oracle_syrk_##SUF(int lower, long n, long k, TS alpha,            \
                              const TD *A, long incRowA, long incColA,        \
                              TS beta, TD *C, long incRowC, long incColC,     \
                              const ulm_oracle_blocksize *bs)                 \
    {                                                                         \
        ulm_oracle_blocksize def;                                             \
        if (!bs) { DEFBS(&def); bs = &def; }                                  \
        return PRE##syrk(lower, n, k, alpha, A, incRowA, incColA, beta, C,    \
                         incRowC, incColC, bs);                               \
    }                                                                         \
    int ulm_oracle_syr2k_##SUF(int lower, long n, long k, TS alpha,           \
                               const TD *A, long incRowA, long incColA,       \
                               const TD *B, long incRowB, long incColB,       \
                               TS beta, TD *C, long incRowC, long incColC,    \
                               const ulm_oracle_blocksize *bs)                \
    {                                                                         \
        ulm_oracle_blocksize def;                                             \
        if (!bs) { DEFBS(&def); bs = &def; }                                  \
        return PRE##syr2k(lower, n, k, alpha, A, incRowA, incColA, B,         \
                          incRowB, incColB, beta, C, incRowC, incColC, bs);   \
    }                                                                         \
    int ulm_oracle_symm_##SUF(int lower, long m, long n, TS alpha,            \
                              const TD *A, long incRowA, long incColA,        \
                              const TD *B, long incRowB, long incColB,        \
                              TS beta, TD *C, long incRowC, long incColC,     \
                              const ulm_oracle_blocksize *bs)                 \
    {                                                                         \
        ulm_oracle_blocksize def;                                             \
        if (!bs) { DEFBS(&def); bs = &def; }                                  \
        return PRE##symm(lower, m, n, alpha, A, incRowA, incColA, B, incRowB, \
                         incColB, beta, C, incRowC, incColC, bs);             \
    }                                                                         \
    int ulm_oracle_trmm_##SUF(int lower, long m, long n, TS alpha, int unit,  \
                              const TD *A, long incRowA, long incColA, TD *B, \
                              long incRowB, long incColB,                     \
                              const ulm_oracle_blocksize *bs)                 \
    {                                                                         \
        ulm_oracle_blocksize def;                                             \
        if (!bs) { DEFBS(&def); bs = &def; }                                  \
        return PRE##trmm(lower, m, n, alpha, unit, A, incRowA, incColA, B,    \
                         incRowB, incColB, bs);                               \
    }

ORACLE_L3_EXPORTS(d, d_, double, double, ulm_oracle_default_blocksize_d)
ORACLE_L3_EXPORTS(s, s_, float, float, ulm_oracle_default_blocksize_s)
ORACLE_L3_EXPORTS(s_f64, sd_, double, float, ulm_oracle_default_blocksize_d)

/* interfaces/blas/F77/syrk.cc:114-133 (ssyrk_ :39-58) */
int ulm_oracle_f77_syrk_info(char upLo_, char trans_, int n, int k, int ldA,
                             int ldC)
{
    int ul = toupper((unsigned char)upLo_), tr = toupper((unsigned char)trans_);
    int numRowsA = (tr == 'T' || tr == 'C') ? k : n;
    if (ul != 'L' && ul != 'U') return 1;
    if (tr != 'N' && tr != 'T' && tr != 'C' && tr != 'R') return 2;
    if (n < 0) return 3;
    if (k < 0) return 4;
    if (ldA < imax(1, numRowsA)) return 7;
    if (ldC < imax(1, n)) return 10;
    return 0;
}

/* interfaces/blas/C/syrk.cc:221-250 */
int ulm_oracle_cblas_syrk_info(int order, int upLo, int trans, int n, int k,
                               int ldA, int ldC)
{
    int numRowsA;
    if (order == ULM_ORACLE_COL_MAJOR) {
        numRowsA = cblas_notrans(trans) ? n : k;
    } else {
        numRowsA = cblas_notrans(trans) ? k : n;
    }
    if (order != ULM_ORACLE_COL_MAJOR && order != ULM_ORACLE_ROW_MAJOR)
        return 1;
    if (upLo != ULM_ORACLE_LOWER && upLo != ULM_ORACLE_UPPER) return 2;
    if (!cblas_trans_valid(trans)) return 3;
    if (n < 0) return 4;
    if (k < 0) return 5;
    if (ldA < imax(1, numRowsA)) return 8;
    if (ldC < imax(1, n)) return 11;
    return 0;
}

/* interfaces/blas/F77/syr2k.cc:121-144 (ssyr2k_ :41-64) */
int ulm_oracle_f77_syr2k_info(char upLo_, char trans_, int n, int k, int ldA,
                              int ldB, int ldC)
{
    int ul = toupper((unsigned char)upLo_), tr = toupper((unsigned char)trans_);
    int numRows = (tr == 'T' || tr == 'C') ? k : n;
    if (ul != 'L' && ul != 'U') return 1;
    if (tr != 'N' && tr != 'T' && tr != 'C' && tr != 'R') return 2;
    if (n < 0) return 3;
    if (k < 0) return 4;
    if (ldA < imax(1, numRows)) return 7;
    if (ldB < imax(1, numRows)) return 9;
    if (ldC < imax(1, n)) return 12;
    return 0;
}

/* interfaces/blas/C/syr2k.cc:238-276 */
int ulm_oracle_cblas_syr2k_info(int order, int upLo, int trans, int n, int k,
                                int ldA, int ldB, int ldC)
{
    int numRows;
    if (order == ULM_ORACLE_COL_MAJOR) {
        numRows = cblas_notrans(trans) ? n : k;
    } else {
        numRows = cblas_notrans(trans) ? k : n;
    }
    if (order != ULM_ORACLE_COL_MAJOR && order != ULM_ORACLE_ROW_MAJOR)
        return 1;
    if (upLo != ULM_ORACLE_LOWER && upLo != ULM_ORACLE_UPPER) return 2;
    if (!cblas_trans_valid(trans)) return 3;
    if (n < 0) return 4;
    if (k < 0) return 5;
    if (ldA < imax(1, numRows)) return 8;
    if (ldB < imax(1, numRows)) return 10;
    if (ldC < imax(1, n)) return 13;
    return 0;
}

/* interfaces/blas/F77/symm.cc:119-138 */
int ulm_oracle_f77_symm_info(char side_, char upLo_, int m, int n, int ldA,
                             int ldB, int ldC)
{
    int sd = toupper((unsigned char)side_), ul = toupper((unsigned char)upLo_);
    int numRowsA = (sd == 'L') ? m : n;
    if (sd != 'L' && sd != 'R') return 1;
    if (ul != 'L' && ul != 'U') return 2;
    if (m < 0) return 3;
    if (n < 0) return 4;
    if (ldA < imax(1, numRowsA)) return 7;
    if (ldB < imax(1, m)) return 9;
    if (ldC < imax(1, m)) return 12;
    return 0;
}

/* interfaces/blas/C/symm.cc:261-300 */
int ulm_oracle_cblas_symm_info(int order, int side, int upLo, int m, int n,
                               int ldA, int ldB, int ldC)
{
    int numRowsA = (side == ULM_ORACLE_LEFT) ? m : n;
    if (order != ULM_ORACLE_COL_MAJOR && order != ULM_ORACLE_ROW_MAJOR)
        return 1;
    if (side != ULM_ORACLE_LEFT && side != ULM_ORACLE_RIGHT) return 2;
    if (upLo != ULM_ORACLE_LOWER && upLo != ULM_ORACLE_UPPER) return 3;
    if (order == ULM_ORACLE_COL_MAJOR) {
        if (m < 0) return 4;
        if (n < 0) return 5;
        if (ldA < imax(1, numRowsA)) return 8;
        if (ldB < imax(1, m)) return 10;
        if (ldC < imax(1, m)) return 13;
    } else {
        if (n < 0) return 4;
        if (m < 0) return 5;
        if (ldA < imax(1, numRowsA)) return 8;
        if (ldB < imax(1, n)) return 10;
        if (ldC < imax(1, n)) return 13;
    }
    return 0;
}
