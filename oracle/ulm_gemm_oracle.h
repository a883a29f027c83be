/*
 * TEST INFRASTRUCTURE -- not part of the product.
 *
 * CPU restatement of the GEMM path of michael-lehn/ulmBLAS: the interface
 * layer (argument checks, trans -> stride mapping), the NC/KC/MC frame, panel
 * packing, macro-kernel and the portable micro-kernel.  It exists to check the
 * GPU library and to time a CPU baseline; nothing the product ships may link
 * or call it.  Reference lines are cited per function in the sources.
 *
 * Parity status of every function here: pinned.  The arithmetic is pinned
 * bit-exactly by golden outputs written from a build of the reference's own
 * headers (tests/golden), by that build itself where it is present
 * (oracle/_ref), by the exact-integer known answers of the reference's level-3
 * tester and by a higher-precision brute-force product; the argument checks
 * are pinned by the (call -> info) tables of the reference's error-exit tests.
 */
#ifndef ULM_GEMM_ORACLE_H
#define ULM_GEMM_ORACLE_H 1

#ifdef __cplusplus
extern "C" {
#endif

/* Block sizes; ulmblas/config/blocksize.h:27-103 gives the production values
 * (double 384/384/4096/4/4, float 768/384/4096/8/4) and :11-25 the test
 * override this struct mirrors. */
typedef struct {
    int MC, KC, NC, MR, NR;
} ulm_oracle_blocksize;

enum { ULM_ORACLE_ROW_MAJOR = 101, ULM_ORACLE_COL_MAJOR = 102 };
enum {
    ULM_ORACLE_NO_TRANS = 111,
    ULM_ORACLE_TRANS = 112,
    ULM_ORACLE_CONJ_TRANS = 113,
    ULM_ORACLE_ATLAS_CONJ = 114
};

/* Production block sizes of the three arithmetic variants. */
void ulm_oracle_default_blocksize_d(ulm_oracle_blocksize *bs);
void ulm_oracle_default_blocksize_s(ulm_oracle_blocksize *bs);

/* ulmBLAS::gemm with element strides (ulmblas/level3/gemm.tcc:13-87).
 * bs == NULL selects the production block sizes.  Return 0, or <0 when the
 * block sizes are unusable or scratch memory cannot be had.
 *   _d       all double                         (dgemm_, cblas_dgemm)
 *   _s       all float, float accumulation      (cblas_sgemm)
 *   _s_f64   float data, double alpha/beta and
 *            double accumulation                (sgemm_) */
int ulm_oracle_gemm_d(long m, long n, long k, double alpha, const double *A,
                      long incRowA, long incColA, const double *B,
                      long incRowB, long incColB, double beta, double *C,
                      long incRowC, long incColC,
                      const ulm_oracle_blocksize *bs);
int ulm_oracle_gemm_s(long m, long n, long k, float alpha, const float *A,
                      long incRowA, long incColA, const float *B,
                      long incRowB, long incColB, float beta, float *C,
                      long incRowC, long incColC,
                      const ulm_oracle_blocksize *bs);
int ulm_oracle_gemm_s_f64(long m, long n, long k, double alpha, const float *A,
                          long incRowA, long incColA, const float *B,
                          long incRowB, long incColB, double beta, float *C,
                          long incRowC, long incColC,
                          const ulm_oracle_blocksize *bs);

/* Complex GEMM: ulmBLAS::gemm(m, n, k, alpha, conjA, A, .., conjB, B, .., beta,
 * C, ..) on std::complex<double> (_z) and std::complex<float> (_c), the calls
 * zgemm_ / cgemm_ / cblas_zgemm / cblas_cgemm make.  Matrices and scalars are
 * passed as interleaved (re, im) pairs; strides count complex elements.
 * Default block sizes: MC = KC = 192, MR = NR = 2 (z); MC = KC = 384, MR = 4,
 * NR = 2 (c) (ulmblas/config/blocksize.h:66-103). */
void ulm_oracle_default_blocksize_z(ulm_oracle_blocksize *bs);
void ulm_oracle_default_blocksize_c(ulm_oracle_blocksize *bs);
int ulm_oracle_gemm_z(long m, long n, long k, const double *alpha, int conjA,
                      const double *A, long incRowA, long incColA, int conjB,
                      const double *B, long incRowB, long incColB,
                      const double *beta, double *C, long incRowC,
                      long incColC, const ulm_oracle_blocksize *bs);
int ulm_oracle_gemm_c(long m, long n, long k, const float *alpha, int conjA,
                      const float *A, long incRowA, long incColA, int conjB,
                      const float *B, long incRowB, long incColB,
                      const float *beta, float *C, long incRowC, long incColC,
                      const ulm_oracle_blocksize *bs);

/* Argument checks.  F77: interfaces/blas/F77/gemm.cc:169-195 -> info in
 * {0,1,2,3,4,5,8,10,13}.  CBLAS: interfaces/blas/C/gemm.cc:425-470 -> info in
 * {0,1,2,3,4,5,6,9,11,14} with the row-major swaps. */
int ulm_oracle_f77_gemm_info(char transA, char transB, int m, int n, int k,
                             int ldA, int ldB, int ldC);
int ulm_oracle_cblas_gemm_info(int order, int transA, int transB, int m, int n,
                               int k, int ldA, int ldB, int ldC);

/* The interface functions (interfaces/blas/F77/gemm.cc:10-249,
 * interfaces/blas/C/gemm.cc:9-138, :295-485).  They return the info code and
 * compute only when it is 0 (the reference reports through xerbla and then
 * falls through; all its error-exit tests have zero work). */
int ulm_oracle_dgemm_f77(char transA, char transB, int m, int n, int k,
                         double alpha, const double *A, int ldA,
                         const double *B, int ldB, double beta, double *C,
                         int ldC);
int ulm_oracle_sgemm_f77(char transA, char transB, int m, int n, int k,
                         float alpha, const float *A, int ldA, const float *B,
                         int ldB, float beta, float *C, int ldC);
int ulm_oracle_cblas_dgemm(int order, int transA, int transB, int m, int n,
                           int k, double alpha, const double *A, int ldA,
                           const double *B, int ldB, double beta, double *C,
                           int ldC);
int ulm_oracle_cblas_sgemm(int order, int transA, int transB, int m, int n,
                           int k, float alpha, const float *A, int ldA,
                           const float *B, int ldB, float beta, float *C,
                           int ldC);

/* Sampled elements of C <- alpha*op(A)*op(B) + beta*C for column-major
 * operands: out[s] is the value ulmBLAS would leave at (rows[s], cols[s]),
 * gauge[s] = |alpha|*sum|a||b| + |beta|*|c| (the error scale of DMMCH,
 * test/F77/dblat3.f:2496-2533).  C is read only at the sampled positions.
 * variant: 0 = _d on double data, 1 = _s, 2 = _s_f64 on float data. */
int ulm_oracle_gemm_samples(int variant, char transA, char transB, long m,
                            long n, long k, double alpha, const void *A,
                            long ldA, const void *B, long ldB, double beta,
                            const void *C, long ldC, long nsamples,
                            const long *rows, const long *cols, void *out,
                            double *gauge);

/* ---- triangular solve -------------------------------------------------- */

enum { ULM_ORACLE_UPPER = 121, ULM_ORACLE_LOWER = 122 };
enum { ULM_ORACLE_NON_UNIT = 131, ULM_ORACLE_UNIT = 132 };
enum { ULM_ORACLE_LEFT = 141, ULM_ORACLE_RIGHT = 142 };

/* ulmBLAS::trlsm (lower != 0, ulmblas/level3/trlsm.tcc:16-91) and
 * ulmBLAS::trusm (lower == 0, ulmblas/level3/trusm.tcc:18-100) with element
 * strides: B <- alpha * inv(A) * B for an m x m triangular A and m x n B.
 * Flavours as for gemm (_s_f64 = strsm_: float data, double arithmetic). */
int ulm_oracle_trsm_d(int lower, long m, long n, double alpha, int unit,
                      const double *A, long incRowA, long incColA, double *B,
                      long incRowB, long incColB,
                      const ulm_oracle_blocksize *bs);
int ulm_oracle_trsm_s(int lower, long m, long n, float alpha, int unit,
                      const float *A, long incRowA, long incColA, float *B,
                      long incRowB, long incColB,
                      const ulm_oracle_blocksize *bs);
int ulm_oracle_trsm_s_f64(int lower, long m, long n, double alpha, int unit,
                          const float *A, long incRowA, long incColA, float *B,
                          long incRowB, long incColB,
                          const ulm_oracle_blocksize *bs);

/* Argument checks.  F77: interfaces/blas/F77/trsm.cc:154-174 -> info in
 * {0,1,2,3,4,5,6,9,11}.  CBLAS: interfaces/blas/C/trsm.cc:410-446 -> info in
 * {0,1,2,3,4,5,6,7,10,12} with the row-major swap of m and n. */
int ulm_oracle_f77_trsm_info(char side, char upLo, char transA, char diag,
                             int m, int n, int ldA, int ldB);
int ulm_oracle_cblas_trsm_info(int order, int side, int upLo, int transA,
                               int diag, int m, int n, int ldA, int ldB);

/* The interface functions (interfaces/blas/F77/trsm.cc:10-227,
 * interfaces/blas/C/trsm.cc:9-153, :311-459); return the info code and
 * compute only when it is 0. */
int ulm_oracle_dtrsm_f77(char side, char upLo, char transA, char diag, int m,
                         int n, double alpha, const double *A, int ldA,
                         double *B, int ldB);
int ulm_oracle_strsm_f77(char side, char upLo, char transA, char diag, int m,
                         int n, float alpha, const float *A, int ldA, float *B,
                         int ldB);
int ulm_oracle_cblas_dtrsm(int order, int side, int upLo, int transA, int diag,
                           int m, int n, double alpha, const double *A,
                           int ldA, double *B, int ldB);
int ulm_oracle_cblas_strsm(int order, int side, int upLo, int transA, int diag,
                           int m, int n, float alpha, const float *A, int ldA,
                           float *B, int ldB);

/* ---- symmetric rank-k update, symmetric product, triangular product ---- */

/* ulmBLAS::sylrk / syurk (ulmblas/level3/sylrk.tcc:17-88): the `lower`
 * (else upper) triangle of C <- beta*C + alpha*A*A^T, A n x k on strides.
 * ulmBLAS::sylr2k / syur2k (sylr2k.tcc:15-127): the same triangle of
 * C <- beta*C + alpha*A*B^T + alpha*B*A^T, A and B n x k, each on its own
 * strides (the reference addresses B with A's strides: identical when both
 * leading dimensions agree).
 * ulmBLAS::sylmm / syumm (sylmm.tcc:16-98): C <- beta*C + alpha*A*B, A m x m
 * symmetric with its `lower` (else upper) triangle stored.
 * ulmBLAS::trlmm / trumm (trlmm.tcc:16-88): B <- alpha*A*B, A m x m lower
 * (else upper) triangular.  Flavours _d, _s, _s_f64 as for gemm. */
#define ULM_ORACLE_L3_DECL(SUF, TS, TD)                                       \
    int ulm_oracle_syrk_##SUF(int lower, long n, long k, TS alpha,            \
                              const TD *A, long incRowA, long incColA,        \
                              TS beta, TD *C, long incRowC, long incColC,     \
                              const ulm_oracle_blocksize *bs);                \
    int ulm_oracle_syr2k_##SUF(int lower, long n, long k, TS alpha,           \
                               const TD *A, long incRowA, long incColA,       \
                               const TD *B, long incRowB, long incColB,       \
                               TS beta, TD *C, long incRowC, long incColC,    \
                               const ulm_oracle_blocksize *bs);               \
    int ulm_oracle_symm_##SUF(int lower, long m, long n, TS alpha,            \
                              const TD *A, long incRowA, long incColA,        \
                              const TD *B, long incRowB, long incColB,        \
                              TS beta, TD *C, long incRowC, long incColC,     \
                              const ulm_oracle_blocksize *bs);                \
    int ulm_oracle_trmm_##SUF(int lower, long m, long n, TS alpha, int unit,  \
                              const TD *A, long incRowA, long incColA, TD *B, \
                              long incRowB, long incColB,                     \
                              const ulm_oracle_blocksize *bs);
ULM_ORACLE_L3_DECL(d, double, double)
ULM_ORACLE_L3_DECL(s, float, float)
ULM_ORACLE_L3_DECL(s_f64, double, float)

/* Argument checks of the interfaces (interfaces/blas/F77/syrk.cc:114-133,
 * symm.cc:119-138; interfaces/blas/C/syrk.cc:221-250, symm.cc:261-300; the
 * triangular product checks exactly what the triangular solve checks,
 * F77/trmm.cc:45-64 = trsm.cc, C/trmm.cc:402-437). */
int ulm_oracle_f77_syrk_info(char upLo, char trans, int n, int k, int ldA,
                             int ldC);
int ulm_oracle_cblas_syrk_info(int order, int upLo, int trans, int n, int k,
                               int ldA, int ldC);
int ulm_oracle_f77_syr2k_info(char upLo, char trans, int n, int k, int ldA,
                              int ldB, int ldC);
int ulm_oracle_cblas_syr2k_info(int order, int upLo, int trans, int n, int k,
                                int ldA, int ldB, int ldC);
int ulm_oracle_f77_symm_info(char side, char upLo, int m, int n, int ldA,
                             int ldB, int ldC);
int ulm_oracle_cblas_symm_info(int order, int side, int upLo, int m, int n,
                               int ldA, int ldB, int ldC);

/* ---- LU factorisation (double) ----------------------------------------- */

/* ulmBLAS::getrf (ulmblas/lapack/getrf.tcc:14-75) with element strides;
 * piv[i] = 0-based row exchanged with row i; returns info (0, or j+1 for the
 * first exactly zero pivot).  nb <= 0 selects the reference's block size 64.
 * getf2: the unblocked panel factorisation (ulmblas/lapack/getf2.tcc:15-62);
 * laswp: the row exchanges (ulmblas/lapack/laswp.tcc:13-55). */
int ulm_oracle_getrf_d(long m, long n, double *A, long incRowA, long incColA,
                       int *piv, long incPiv, long nb,
                       const ulm_oracle_blocksize *bs);
int ulm_oracle_getf2_d(long m, long n, double *A, long incRowA, long incColA,
                       int *piv, long incPiv);
void ulm_oracle_laswp_d(long n, double *A, long incRowA, long incColA, long k1,
                        long k2, const int *piv, long incPiv);

/* The interface functions ULMLAPACK(dgetrf) / ULMLAPACK(dlaswp)
 * (interfaces/lapack/C/getrf.cc:7-19, laswp.cc:7-18). */
int ulm_oracle_dgetrf(int order, int m, int n, double *A, int ldA, int *piv);
void ulm_oracle_dlaswp(int n, double *A, int ldA, int k1, int k2,
                       const int *piv, int incPiv);

#ifdef __cplusplus
}
#endif
#endif
