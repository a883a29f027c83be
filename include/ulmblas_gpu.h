/*
 * libulmblas_gpu -- MI355X (gfx950) GEMM behind ulmBLAS's BLAS and CBLAS
 * entry points.
 *
 * Part 1 declares the drop-in symbols: same names, argument meaning and
 * error convention as the reference's interface layer; operands are HOST
 * pointers, the library moves them to the GPU, runs its HIP kernels and
 * copies C back before returning.  Part 2 declares the device-resident entry
 * points (operands already in HBM) that part 1 is built on.
 *
 * All integers are 32-bit `int` as in the reference ABI; matrices are
 * column-major unless cblas_* is told CblasRowMajor.
 */
#ifndef ULMBLAS_GPU_H
#define ULMBLAS_GPU_H 1

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------
 * Part 1: drop-in BLAS / CBLAS symbols (host pointers)
 * --------------------------------------------------------------------- */

/* Constants of the CBLAS interface: interfaces/blas/C/cblas.h.in:17-27. */
enum CBLAS_ORDER { CblasRowMajor = 101, CblasColMajor = 102 };
enum CBLAS_TRANSPOSE {
    CblasNoTrans = 111,
    CblasTrans = 112,
    CblasConjTrans = 113,
    AtlasConj = 114
};
enum CBLAS_UPLO { CblasUpper = 121, CblasLower = 122 };
enum CBLAS_DIAG { CblasNonUnit = 131, CblasUnit = 132 };
enum CBLAS_SIDE { CblasLeft = 141, CblasRight = 142 };

/* Replaces F77BLAS(dgemm), interfaces/blas/F77/gemm.cc:131-249 (declared in
 * interfaces/blas/F77/f77blas.h.in:210-222).  C <- alpha*op(A)*op(B)+beta*C.
 * trans: first character, case-insensitive, 'N'/'R' = as stored, 'T'/'C' =
 * transposed.  Invalid arguments (info 1,2,3,4,5,8,10,13) are reported
 * through xerbla_("DGEMM ", &info) and the call returns without touching C.
 * beta == 0 never reads C; alpha == 0 or k == 0 only scales C. */
void dgemm_(const char *transA, const char *transB, const int *m,
            const int *n, const int *k, const double *alpha, const double *A,
            const int *ldA, const double *B, const int *ldB,
            const double *beta, double *C, const int *ldC);

/* Replaces F77BLAS(sgemm), interfaces/blas/F77/gemm.cc:10-128.  The reference
 * accumulates this entry point in double (:33,36); here the product is
 * accumulated in fp32 on the matrix cores, which stays inside the same
 * k*eps32 error bound. */
void sgemm_(const char *transA, const char *transB, const int *m,
            const int *n, const int *k, const float *alpha, const float *A,
            const int *ldA, const float *B, const int *ldB, const float *beta,
            float *C, const int *ldC);

/* Replaces CBLAS(dgemm), interfaces/blas/C/gemm.cc:391-485 (declared in
 * interfaces/blas/C/cblas.h.in:1186-1199).  Info codes 1,2,3,4,5,6,9,11,14
 * with the row-major swaps, reported through
 * cblas_xerbla(info, "cblas_dgemm", ...).  Row-major is computed as the
 * column-major product of the swapped operands (:478-484). */
void cblas_dgemm(enum CBLAS_ORDER order, enum CBLAS_TRANSPOSE transA,
                 enum CBLAS_TRANSPOSE transB, int m, int n, int k,
                 double alpha, const double *A, int ldA, const double *B,
                 int ldB, double beta, double *C, int ldC);

/* Replaces CBLAS(sgemm), interfaces/blas/C/gemm.cc:295-389. */
void cblas_sgemm(enum CBLAS_ORDER order, enum CBLAS_TRANSPOSE transA,
                 enum CBLAS_TRANSPOSE transB, int m, int n, int k, float alpha,
                 const float *A, int ldA, const float *B, int ldB, float beta,
                 float *C, int ldC);

/* Replace ULMBLAS(dgemm) / ULMBLAS(sgemm), interfaces/blas/C/gemm.cc:75-138
 * and :9-72 (declared in interfaces/blas/C/cblas.h.in:2525-2552): the
 * order-less, unchecked column-major entry points cblas_* forwards to.
 * CblasNoTrans and AtlasConj mean "as stored", anything else transposed. */
void ulmblas_dgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB,
                   int m, int n, int k, double alpha, const double *A, int ldA,
                   const double *B, int ldB, double beta, double *C, int ldC);
void ulmblas_sgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB,
                   int m, int n, int k, float alpha, const float *A, int ldA,
                   const float *B, int ldB, float beta, float *C, int ldC);

/* The same two under the prefix the reference's ATLAS-bench flavour uses
 * (interfaces/blas/C/config/make.atl.inc:4-5), so that bench/l3blastst.c
 * links unchanged. */
void ATL_dgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m,
               int n, int k, double alpha, const double *A, int ldA,
               const double *B, int ldB, double beta, double *C, int ldC);
void ATL_sgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m,
               int n, int k, float alpha, const float *A, int ldA,
               const float *B, int ldB, float beta, float *C, int ldC);

/* Replace F77BLAS(zgemm) / F77BLAS(cgemm), interfaces/blas/F77/gemm.cc:382-506
 * and :251-380: complex C <- alpha*op(A)*op(B) + beta*C, column-major; matrices
 * and the scalars behind alpha / beta are interleaved (re, im) pairs, leading
 * dimensions count complex elements.  trans 'N', 'T', 'C' (conjugate
 * transpose) and 'R' (conjugate, not transposed), as the reference reads them
 * (:270-274); same info codes as dgemm_ (1,2,3,4,5,8,10,13) through
 * xerbla_("ZGEMM ", ..) / ("CGEMM ", ..).  CBLAS / ulmblas_ / ATL_ forms:
 * interfaces/blas/C/gemm.cc:584-690, 488-582 (checked, both storage orders,
 * info as cblas_dgemm) and :219-293, 141-217 (unchecked, column-major;
 * AtlasConj is the 'R' of the F77 form). */
void zgemm_(const char *transA, const char *transB, const int *m, const int *n,
            const int *k, const double *alpha, const double *A, const int *ldA,
            const double *B, const int *ldB, const double *beta, double *C,
            const int *ldC);
void cgemm_(const char *transA, const char *transB, const int *m, const int *n,
            const int *k, const float *alpha, const float *A, const int *ldA,
            const float *B, const int *ldB, const float *beta, float *C,
            const int *ldC);
void cblas_zgemm(enum CBLAS_ORDER order, enum CBLAS_TRANSPOSE transA,
                 enum CBLAS_TRANSPOSE transB, int m, int n, int k,
                 const double *alpha, const double *A, int ldA,
                 const double *B, int ldB, const double *beta, double *C,
                 int ldC);
void cblas_cgemm(enum CBLAS_ORDER order, enum CBLAS_TRANSPOSE transA,
                 enum CBLAS_TRANSPOSE transB, int m, int n, int k,
                 const float *alpha, const float *A, int ldA, const float *B,
                 int ldB, const float *beta, float *C, int ldC);
void ulmblas_zgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB,
                   int m, int n, int k, const double *alpha, const double *A,
                   int ldA, const double *B, int ldB, const double *beta,
                   double *C, int ldC);
void ulmblas_cgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB,
                   int m, int n, int k, const float *alpha, const float *A,
                   int ldA, const float *B, int ldB, const float *beta,
                   float *C, int ldC);
void ATL_zgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m,
               int n, int k, const double *alpha, const double *A, int ldA,
               const double *B, int ldB, const double *beta, double *C,
               int ldC);
void ATL_cgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m,
               int n, int k, const float *alpha, const float *A, int ldA,
               const float *B, int ldB, const float *beta, float *C, int ldC);

/* Replace F77BLAS(dtrsm) / F77BLAS(strsm), interfaces/blas/F77/trsm.cc:120-227
 * and :9-117 (declared in interfaces/blas/F77/f77blas.h.in).  Solves
 * op(A)*X = alpha*B (side 'L') or X*op(A) = alpha*B (side 'R') for X, which
 * overwrites the m x n matrix B; A is triangular (uplo 'U'/'L') of order m
 * (left) or n (right), diag 'U' = unit diagonal that is not read.  Only the
 * named triangle of A is read.  Invalid arguments (info 1,2,3,4,5,6,9,11) go
 * to xerbla_("DTRSM ", &info) and the call returns.  alpha == 0 stores zeros
 * without reading A or B.  The reference's strsm_ computes in double
 * (:29); here the solve runs in fp32. */
void dtrsm_(const char *side, const char *upLo, const char *transA,
            const char *diag, const int *m, const int *n, const double *alpha,
            const double *A, const int *ldA, double *B, const int *ldB);
void strsm_(const char *side, const char *upLo, const char *transA,
            const char *diag, const int *m, const int *n, const float *alpha,
            const float *A, const int *ldA, float *B, const int *ldB);

/* Replace CBLAS(dtrsm) / CBLAS(strsm), interfaces/blas/C/trsm.cc:386-459 and
 * :311-384.  Info codes 1,2,3,4,5,6,7,10,12 through
 * cblas_xerbla(info, "cblas_dtrsm", ""); row-major is solved as the
 * column-major problem with side and uplo flipped and m, n swapped
 * (:454-458). */
void cblas_dtrsm(enum CBLAS_ORDER order, enum CBLAS_SIDE side,
                 enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE transA,
                 enum CBLAS_DIAG diag, int m, int n, double alpha,
                 const double *A, int ldA, double *B, int ldB);
void cblas_strsm(enum CBLAS_ORDER order, enum CBLAS_SIDE side,
                 enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE transA,
                 enum CBLAS_DIAG diag, int m, int n, float alpha,
                 const float *A, int ldA, float *B, int ldB);

/* Replace ULMBLAS(dtrsm) / ULMBLAS(strsm), interfaces/blas/C/trsm.cc:84-153
 * and :9-82: order-less, unchecked, column-major; also under the ATL_ prefix
 * of the reference's ATLAS-bench flavour. */
void ulmblas_dtrsm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo,
                   enum CBLAS_TRANSPOSE transA, enum CBLAS_DIAG diag, int m,
                   int n, double alpha, const double *A, int ldA, double *B,
                   int ldB);
void ulmblas_strsm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo,
                   enum CBLAS_TRANSPOSE transA, enum CBLAS_DIAG diag, int m,
                   int n, float alpha, const float *A, int ldA, float *B,
                   int ldB);
void ATL_dtrsm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo,
               enum CBLAS_TRANSPOSE transA, enum CBLAS_DIAG diag, int m, int n,
               double alpha, const double *A, int ldA, double *B, int ldB);
void ATL_strsm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo,
               enum CBLAS_TRANSPOSE transA, enum CBLAS_DIAG diag, int m, int n,
               float alpha, const float *A, int ldA, float *B, int ldB);

/* Replace F77BLAS(dtrmm) / F77BLAS(strmm), interfaces/blas/F77/trmm.cc:119-230
 * and :9-117, and the CBLAS / ULMBLAS / ATL forms, interfaces/blas/C/trmm.cc:
 * B <- alpha*op(A)*B (side 'L') or alpha*B*op(A) (side 'R'), A triangular.
 * Arguments, checks and info codes are those of the triangular solve above
 * (routine names "DTRMM ", "cblas_dtrmm"); alpha == 0 stores zeros. */
void dtrmm_(const char *side, const char *upLo, const char *transA,
            const char *diag, const int *m, const int *n, const double *alpha,
            const double *A, const int *ldA, double *B, const int *ldB);
void strmm_(const char *side, const char *upLo, const char *transA,
            const char *diag, const int *m, const int *n, const float *alpha,
            const float *A, const int *ldA, float *B, const int *ldB);
void cblas_dtrmm(enum CBLAS_ORDER order, enum CBLAS_SIDE side,
                 enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE transA,
                 enum CBLAS_DIAG diag, int m, int n, double alpha,
                 const double *A, int ldA, double *B, int ldB);
void cblas_strmm(enum CBLAS_ORDER order, enum CBLAS_SIDE side,
                 enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE transA,
                 enum CBLAS_DIAG diag, int m, int n, float alpha,
                 const float *A, int ldA, float *B, int ldB);
void ulmblas_dtrmm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo,
                   enum CBLAS_TRANSPOSE transA, enum CBLAS_DIAG diag, int m,
                   int n, double alpha, const double *A, int ldA, double *B,
                   int ldB);
void ulmblas_strmm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo,
                   enum CBLAS_TRANSPOSE transA, enum CBLAS_DIAG diag, int m,
                   int n, float alpha, const float *A, int ldA, float *B,
                   int ldB);
void ATL_dtrmm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo,
               enum CBLAS_TRANSPOSE transA, enum CBLAS_DIAG diag, int m, int n,
               double alpha, const double *A, int ldA, double *B, int ldB);
void ATL_strmm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo,
               enum CBLAS_TRANSPOSE transA, enum CBLAS_DIAG diag, int m, int n,
               float alpha, const float *A, int ldA, float *B, int ldB);

/* Replace F77BLAS(dsyr2k) / F77BLAS(ssyr2k), interfaces/blas/F77/syr2k.cc:91-165
 * and :11-85 (-> ulmBLAS::sylr2k / syur2k, ulmblas/level3/sylr2k.tcc:15-127):
 * the upLo triangle of C <- alpha*op(A)*op(B)^T + alpha*op(B)*op(A)^T + beta*C.
 * xerbla_ info 1,2,3,4,7,9,12.  CBLAS / ulmblas_ / ATL forms:
 * interfaces/blas/C/syr2k.cc (info 1,2,3,4,5,8,10,13; row-major flips upLo
 * and trans and exchanges A and B, :284-288).  B is read with its own leading
 * dimension; the reference's frame reads it with A's (sylr2k.tcc:66-67), so
 * the two agree exactly when ldA == ldB. */
void dsyr2k_(const char *upLo, const char *trans, const int *n, const int *k,
             const double *alpha, const double *A, const int *ldA,
             const double *B, const int *ldB, const double *beta, double *C,
             const int *ldC);
void ssyr2k_(const char *upLo, const char *trans, const int *n, const int *k,
             const float *alpha, const float *A, const int *ldA, const float *B,
             const int *ldB, const float *beta, float *C, const int *ldC);
void cblas_dsyr2k(enum CBLAS_ORDER order, enum CBLAS_UPLO upLo,
                  enum CBLAS_TRANSPOSE trans, int n, int k, double alpha,
                  const double *A, int ldA, const double *B, int ldB,
                  double beta, double *C, int ldC);
void cblas_ssyr2k(enum CBLAS_ORDER order, enum CBLAS_UPLO upLo,
                  enum CBLAS_TRANSPOSE trans, int n, int k, float alpha,
                  const float *A, int ldA, const float *B, int ldB, float beta,
                  float *C, int ldC);
void ulmblas_dsyr2k(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n,
                    int k, double alpha, const double *A, int ldA,
                    const double *B, int ldB, double beta, double *C, int ldC);
void ulmblas_ssyr2k(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n,
                    int k, float alpha, const float *A, int ldA, const float *B,
                    int ldB, float beta, float *C, int ldC);
void ATL_dsyr2k(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n, int k,
                double alpha, const double *A, int ldA, const double *B,
                int ldB, double beta, double *C, int ldC);
void ATL_ssyr2k(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n, int k,
                float alpha, const float *A, int ldA, const float *B, int ldB,
                float beta, float *C, int ldC);

/* Replace F77BLAS(dsyrk) / F77BLAS(ssyrk), interfaces/blas/F77/syrk.cc:86-157
 * and :11-83: the uplo triangle of C <- alpha*A*A^T + beta*C (trans 'N', A is
 * n x k) or alpha*A^T*A + beta*C (trans 'T'/'C', A is k x n).  The other
 * triangle of C is neither read nor written.  Info codes 1,2,3,4,7,10 through
 * xerbla_("DSYRK ", &info).  alpha == 0 || k == 0 only scales the triangle
 * (beta == 1: untouched, beta == 0: zeros without reading).  CBLAS / ULMBLAS /
 * ATL forms: interfaces/blas/C/syrk.cc (info 1,2,3,4,5,8,11; row-major flips
 * uplo and trans, :258-261). */
void dsyrk_(const char *upLo, const char *trans, const int *n, const int *k,
            const double *alpha, const double *A, const int *ldA,
            const double *beta, double *C, const int *ldC);
void ssyrk_(const char *upLo, const char *trans, const int *n, const int *k,
            const float *alpha, const float *A, const int *ldA,
            const float *beta, float *C, const int *ldC);
void cblas_dsyrk(enum CBLAS_ORDER order, enum CBLAS_UPLO upLo,
                 enum CBLAS_TRANSPOSE trans, int n, int k, double alpha,
                 const double *A, int ldA, double beta, double *C, int ldC);
void cblas_ssyrk(enum CBLAS_ORDER order, enum CBLAS_UPLO upLo,
                 enum CBLAS_TRANSPOSE trans, int n, int k, float alpha,
                 const float *A, int ldA, float beta, float *C, int ldC);
void ulmblas_dsyrk(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n,
                   int k, double alpha, const double *A, int ldA, double beta,
                   double *C, int ldC);
void ulmblas_ssyrk(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n,
                   int k, float alpha, const float *A, int ldA, float beta,
                   float *C, int ldC);
void ATL_dsyrk(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n, int k,
               double alpha, const double *A, int ldA, double beta, double *C,
               int ldC);
void ATL_ssyrk(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n, int k,
               float alpha, const float *A, int ldA, float beta, float *C,
               int ldC);

/* Replace F77BLAS(dsymm) / F77BLAS(ssymm), interfaces/blas/F77/symm.cc:88-159
 * and :11-85: C <- alpha*A*B + beta*C (side 'L', A m x m) or alpha*B*A +
 * beta*C (side 'R', A n x n), A symmetric with its uplo triangle stored (the
 * other one is not read).  Info codes 1,2,3,4,7,9,12 through
 * xerbla_("DSYMM ", &info).  CBLAS / ULMBLAS / ATL forms:
 * interfaces/blas/C/symm.cc (info 1,2,3,4,5,8,10,13; row-major flips side
 * and uplo and swaps m, n, :309-311). */
void dsymm_(const char *side, const char *upLo, const int *m, const int *n,
            const double *alpha, const double *A, const int *ldA,
            const double *B, const int *ldB, const double *beta, double *C,
            const int *ldC);
void ssymm_(const char *side, const char *upLo, const int *m, const int *n,
            const float *alpha, const float *A, const int *ldA, const float *B,
            const int *ldB, const float *beta, float *C, const int *ldC);
void cblas_dsymm(enum CBLAS_ORDER order, enum CBLAS_SIDE side,
                 enum CBLAS_UPLO upLo, int m, int n, double alpha,
                 const double *A, int ldA, const double *B, int ldB,
                 double beta, double *C, int ldC);
void cblas_ssymm(enum CBLAS_ORDER order, enum CBLAS_SIDE side,
                 enum CBLAS_UPLO upLo, int m, int n, float alpha,
                 const float *A, int ldA, const float *B, int ldB, float beta,
                 float *C, int ldC);
void ulmblas_dsymm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, int m, int n,
                   double alpha, const double *A, int ldA, const double *B,
                   int ldB, double beta, double *C, int ldC);
void ulmblas_ssymm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, int m, int n,
                   float alpha, const float *A, int ldA, const float *B,
                   int ldB, float beta, float *C, int ldC);
void ATL_dsymm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, int m, int n,
               double alpha, const double *A, int ldA, const double *B, int ldB,
               double beta, double *C, int ldC);
void ATL_ssymm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, int m, int n,
               float alpha, const float *A, int ldA, const float *B, int ldB,
               float beta, float *C, int ldC);

/* Replaces ULMLAPACK(dgetrf), interfaces/lapack/C/getrf.cc:7-19 (declared in
 * interfaces/lapack/C/clapack.h.in:15-21; the prefix is that of ULMBLAS,
 * interfaces/blas/C/config/make.cblas.inc:11, ATL_ in make.atl.inc:11).
 * LU factorisation with partial pivoting, A = P*L*U in place: L unit lower
 * below the diagonal, U on and above it; piv[i] (0-based) is the row that
 * was exchanged with row i, i < min(m, n).  Returns 0, or j+1 if U(j,j) is
 * exactly zero (first such j; the factorisation is still completed).
 * CblasColMajor factors the m x n matrix with leading dimension ldA.  Any
 * other order does what the reference's row-major branch does: it factors
 * the matrix that has n rows and m columns, element (i, j) at A[i*ldA + j].
 * No argument checks (the reference has none).  If the workgroups of the
 * cooperative panel kernel cannot meet because the GPU holds other work, the
 * matrix is factored again by launches that wait for nobody (same pivots,
 * same bits).  Returns -1, with A and piv as they were, if the GPU could not
 * be used (the text goes to ulmblas_gpu_error_hook). */
int ulmblas_dgetrf(enum CBLAS_ORDER order, int m, int n, double *A, int ldA,
                   int *piv);
int ATL_dgetrf(enum CBLAS_ORDER order, int m, int n, double *A, int ldA,
               int *piv);

/* Replaces ULMLAPACK(dlaswp), interfaces/lapack/C/laswp.cc:7-18: on the
 * column-major matrix A with n columns exchange row i with row
 * piv[i*incPiv] for i = k1 .. k2-1 (0-based, k2 exclusive), in that order,
 * or from k2-1 down to k1 when incPiv < 0. */
void ulmblas_dlaswp(int n, double *A, int ldA, int k1, int k2, int *piv,
                    int incPiv);
void ATL_dlaswp(int n, double *A, int ldA, int k1, int k2, int *piv,
                int incPiv);

/* Error hooks: interfaces/blas/F77/xerbla.cc:6-10 and
 * interfaces/blas/C/xerbla.cc:6-16.  Weak definitions that print
 * "Parameter %d to routine %s was incorrect" to stderr and return; a program
 * (or a test) that defines its own replaces them at link / load time. */
void xerbla_(const char rout[6], const int *info);
void cblas_xerbla(int info, const char *rout, const char *form, ...);
void ulmblas_xerbla(int info, const char *rout, const char *form, ...);

/* ------------------------------------------------------------------------
 * Part 2: device-resident entry points (no counterpart in the reference,
 * which has no device; this is the boundary ulmBLAS::gemm,
 * ulmblas/level3/gemm.tcc:13-87, occupies there)
 * --------------------------------------------------------------------- */

/* Status codes returned by the ulmblas_gpu_* functions. */
enum {
    ULMBLAS_GPU_OK = 0,
    ULMBLAS_GPU_BAD_ARGUMENT = 1, /* negative size, ld too small, bad trans */
    ULMBLAS_GPU_HIP_ERROR = 2,    /* see ulmblas_gpu_last_error() */
    ULMBLAS_GPU_NO_DEVICE = 3,
    /* Not a failure: workgroups that shared a tile of C gave up waiting for
     * one another, and the library recomputed what was missing; the result is
     * complete and the call took longer (see ulmblas_gpu_device_status). */
    ULMBLAS_GPU_RECOVERED = 4
};

/* C <- alpha*op(A)*op(B) + beta*C on column-major operands that already live
 * in device memory.  transA/transB: 0 = as stored, non-zero = transposed.
 * `stream` is a hipStream_t (NULL = the null stream); the call only enqueues
 * work and returns, it does not synchronise and allocates nothing.
 * Semantics are those of ulmBLAS::gemm: m==0 || n==0 writes nothing;
 * alpha==0 || k==0 only scales C (beta==1 leaves it untouched, beta==0 stores
 * zeros without reading); beta==0 never reads C; only the m x n window of C
 * is written; A and B are never written. */
int ulmblas_gpu_dgemm(int transA, int transB, int m, int n, int k,
                      double alpha, const double *dA, int ldA,
                      const double *dB, int ldB, double beta, double *dC,
                      int ldC, void *stream);
int ulmblas_gpu_sgemm(int transA, int transB, int m, int n, int k, float alpha,
                      const float *dA, int ldA, const float *dB, int ldB,
                      float beta, float *dC, int ldC, void *stream);

/* B <- alpha*inv(op(A))*B (right == 0) or alpha*B*inv(op(A)) (right != 0) on
 * column-major operands in device memory; flags are 0 / non-zero.  The
 * device-resident form of ulmBLAS::trlsm / trusm
 * (ulmblas/level3/trlsm.tcc:16-91, trusm.tcc:18-100) that the LU trailing
 * update (ulmblas/lapack/getrf.tcc:59-61) needs.  Enqueues on `stream`,
 * allocates nothing, does not synchronise. */
int ulmblas_gpu_dtrsm(int right, int lower, int transA, int unit, int m, int n,
                      double alpha, const double *dA, int ldA, double *dB,
                      int ldB, void *stream);
int ulmblas_gpu_strsm(int right, int lower, int transA, int unit, int m, int n,
                      float alpha, const float *dA, int ldA, float *dB, int ldB,
                      void *stream);

/* Device-resident forms of the triangular product (ulmBLAS::trlmm / trumm,
 * ulmblas/level3/trlmm.tcc:16-88), the symmetric rank-k update (sylrk /
 * syurk, sylrk.tcc:17-88), the rank-2k update (sylr2k.tcc:15-127) and the
 * symmetric product (sylmm / syumm, sylmm.tcc:16-98); flags are 0 / non-zero, everything is enqueued on
 * `stream`, nothing is allocated.  The symmetric product needs `work`: device
 * memory for min(ka, 2048)^2 elements (ka = m for the left side, n for the
 * right), in which the diagonal blocks of A are completed one after the other;
 * the blocks off the diagonal are read where they are stored. */
int ulmblas_gpu_dtrmm(int right, int lower, int transA, int unit, int m, int n,
                      double alpha, const double *dA, int ldA, double *dB,
                      int ldB, void *stream);
int ulmblas_gpu_strmm(int right, int lower, int transA, int unit, int m, int n,
                      float alpha, const float *dA, int ldA, float *dB, int ldB,
                      void *stream);
int ulmblas_gpu_dsyrk(int lower, int trans, int n, int k, double alpha,
                      const double *dA, int ldA, double beta, double *dC,
                      int ldC, void *stream);
int ulmblas_gpu_ssyrk(int lower, int trans, int n, int k, float alpha,
                      const float *dA, int ldA, float beta, float *dC, int ldC,
                      void *stream);
int ulmblas_gpu_dsyr2k(int lower, int trans, int n, int k, double alpha,
                       const double *dA, int ldA, const double *dB, int ldB,
                       double beta, double *dC, int ldC, void *stream);
int ulmblas_gpu_ssyr2k(int lower, int trans, int n, int k, float alpha,
                       const float *dA, int ldA, const float *dB, int ldB,
                       float beta, float *dC, int ldC, void *stream);
int ulmblas_gpu_dsymm(int right, int lower, int m, int n, double alpha,
                      const double *dA, int ldA, const double *dB, int ldB,
                      double beta, double *dC, int ldC, double *work,
                      void *stream);
int ulmblas_gpu_ssymm(int right, int lower, int m, int n, float alpha,
                      const float *dA, int ldA, const float *dB, int ldB,
                      float beta, float *dC, int ldC, float *work,
                      void *stream);

/* Device-resident complex GEMM: the call of ulmBLAS::gemm with conjugation
 * flags (ulmblas/level3/gemm.tcc:13-87) for column-major complex operands in
 * device memory; enqueued on `stream`, nothing is allocated or synchronised.
 * alpha and beta point to (re, im) pairs in host memory, read before the call
 * returns.  `work`: device memory of ulmblas_gpu_?gemm_worksize(transB, m, n,
 * k) bytes, 16-byte aligned (the real block form of alpha*op(A), 4mk reals,
 * plus op(B) when B is transposed or conjugated). */
long ulmblas_gpu_zgemm_worksize(enum CBLAS_TRANSPOSE transB, int m, int n, int k);
long ulmblas_gpu_cgemm_worksize(enum CBLAS_TRANSPOSE transB, int m, int n, int k);
int ulmblas_gpu_zgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB,
                      int m, int n, int k, const double *alpha,
                      const double *dA, int ldA, const double *dB, int ldB,
                      const double *beta, double *dC, int ldC, void *work,
                      void *stream);
int ulmblas_gpu_cgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB,
                      int m, int n, int k, const float *alpha, const float *dA,
                      int ldA, const float *dB, int ldB, const float *beta,
                      float *dC, int ldC, void *work, void *stream);

/* Device-resident LU (the form ulmBLAS::getrf, ulmblas/lapack/getrf.tcc:14-75,
 * takes when the matrix stays in HBM): column-major dA (m x n, ldA) is
 * overwritten by L and U, dPiv (min(m,n) ints, device) receives the 0-based
 * pivot rows and *dInfo (device) 0, j+1 for the first exactly zero pivot, or
 * -1 if the workgroups of a panel kernel could not meet within their bounded
 * wait.  `work` is device memory of at least ulmblas_gpu_dgetrf_worksize()
 * bytes, 16-byte aligned, used by one factorisation at a time.  Everything is
 * enqueued on `stream`; nothing is allocated, nothing synchronises.  Panels
 * with more rows than the GPU can hold workgroups of the panel kernel at the
 * same time (256 rows each: 65536 rows on an idle MI355X) are factored by
 * three small launches per column instead, at a fraction of the speed. */
long ulmblas_gpu_dgetrf_worksize(void);
int ulmblas_gpu_dgetrf(int m, int n, double *dA, int ldA, int *dPiv,
                       int *dInfo, void *work, void *stream);
/* ulmblas_gpu_dgetrf without the workspace argument, for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The exchange area of the panel kernel lives in a device array inside the
 * library (about 0.5 MiB on every GPU the library runs on, held until the
 * process ends); the call allocates nothing, creates no stream or event and
 * frees nothing.  Same arguments, results and info values as
 * ulmblas_gpu_dgetrf otherwise; m and n at most
 * ULMBLAS_GPU_DGETRF_STATIC_MAX (ULMBLAS_GPU_BAD_ARGUMENT beyond that).
 * All calls on one GPU share the one array: two factorisations that overlap
 * in time on the same GPU (different streams, threads or processes' worth of
 * calls through this symbol) race and give wrong results; calls on one stream,
 * or otherwise ordered one after the other, are safe, and nothing has to be
 * cleared in between. */
#define ULMBLAS_GPU_DGETRF_STATIC_MAX 65536
int ulmblas_gpu_dgetrf_static(int m, int n, double *dA, int ldA, int *dPiv,
                              int *dInfo, void *stream);
/* Row exchanges of ulmblas_dlaswp on device memory (dPiv on the device). */
int ulmblas_gpu_dlaswp(int n, double *dA, int ldA, int k1, int k2,
                       const int *dPiv, int incPiv, void *stream);

/* Selects the workgroup-tile variant the next launches use: 0 = automatic
 * choice from the shape (default), otherwise one of the ids listed by
 * ulmblas_gpu_variant_name().  For tuning and tests; returns
 * ULMBLAS_GPU_BAD_ARGUMENT for an unknown id. */
int ulmblas_gpu_set_variant(int precision /* 'd' or 's' */, int variant);
/* Switches for the library's own tests (no counterpart in the reference):
 *  NARROW_LOADS       value != 0: the 16-byte global loads are not used (they
 *                     are otherwise used by every launch, whatever the
 *                     alignment of A and B beyond that of one element, with
 *                     identical results);
 *  LU_SPIN_LIMIT      polls of one wait of the LU panel kernel for the other
 *                     workgroups before it gives up and the factorisation
 *                     reports info = -1 (negative: the default, 2^24);
 *  SHARED_PIECES      into how many pieces along k a workgroup tile of a
 *                     product may be cut to fill the GPU's last round of
 *                     tiles (default 32: where the estimate says it pays,
 *                     more than 4 only for products of few tiles and long k; 0
 *                     or 1: tiles are never shared; negative: up to -value
 *                     pieces wherever it can be done at all);
 *  SHARED_MUTE        value != 0: workgroups that share a tile do not tell
 *                     each other that their piece is done, so every wait
 *                     runs out (and the launch that follows recomputes what
 *                     the pieces that gave up would have added);
 *  SHARED_SPIN_LIMIT  polls of one such wait (negative: the default, 2^20);
 *  WHOLE_C            1: products whose m or n is no multiple of the tile go
 *                     out as one launch over all of C (tiles that reach past
 *                     the edges load through clamped addresses and mask their
 *                     stores) wherever the variant can do that; 0: never,
 *                     the whole tiles and the strips are launched apart;
 *                     negative (default): whichever the estimate prefers;
 *  LU_SIMPLE_PANELS   value != 0: every panel of an LU factorisation is factored
 *                     by the launches that wait for nobody (three per column),
 *                     which otherwise serve panels with more rows than the
 *                     cooperative panel kernel can hold on the GPU at a time;
 *  TRSM_PARTS         how many blocks of 256 unknowns one launch of the
 *                     triangular solve may take (1 or 2; default 2: a block,
 *                     its share of the next block and that block);
 *  HOST_HEAD          0: the host entry points send A up before anything of B;
 *                     1 (default): large products with beta == 0 send a head
 *                     of op(B)'s columns first and multiply the panels of A
 *                     into it as they land; 2: so does every product that is
 *                     streamed in three or more panels, whatever beta;
 *  TRI_WAY            how a rank-k / rank-2k update of order n is cut up: 0
 *                     (default) by the planner's estimate; 1: the leading
 *                     square of all whole blocks of 256, the rows beyond it as
 *                     a product of their own, the triangle at their end; 2: the
 *                     same with an even number of blocks in the square; 3: the
 *                     any-shape kernel alone over the triangle; 4, 5: as 1, 2
 *                     with the second largest tile (blocks of its order) for
 *                     the square;
 *  FAIL_ALLOC         the next `value` device allocations of the host entry
 *                     points fail (as if the device were out of memory).
 * Every kernel runs to its end whatever is set here. */
enum ULMBLAS_GPU_TEST {
    ULMBLAS_GPU_TEST_NARROW_LOADS = 1,
    ULMBLAS_GPU_TEST_LU_SPIN_LIMIT = 2,
    ULMBLAS_GPU_TEST_SHARED_PIECES = 3,
    ULMBLAS_GPU_TEST_SHARED_MUTE = 4,
    ULMBLAS_GPU_TEST_SHARED_SPIN_LIMIT = 5,
    ULMBLAS_GPU_TEST_FAIL_ALLOC = 6,
    ULMBLAS_GPU_TEST_WHOLE_C = 7,
    ULMBLAS_GPU_TEST_LU_SIMPLE_PANELS = 8,
    ULMBLAS_GPU_TEST_TRSM_PARTS = 9,
    ULMBLAS_GPU_TEST_HOST_HEAD = 10,
    ULMBLAS_GPU_TEST_TRI_WAY = 11
};
int ulmblas_gpu_test_control(int what, long value);
/* How ulmblas_gpu_dgemm / _sgemm (precision 'd' / 's') would launch an
 * m x n x k product with these leading dimensions (reads_c: beta != 0), without
 * launching anything: out[0] the variant id (0: the any-shape kernel alone),
 * out[1] 1 if one launch covers all of C (tiles past the edges included), 0 if
 * whole tiles and strips go out apart, out[2] the number of workgroups that
 * share the tiles of the last round along k (0: none), out[3] how many tiles
 * they share.  For tests and tuning. */
int ulmblas_gpu_plan(int precision, int m, int n, int k, int reads_c, long ldA, long ldB, int out[4]);
/* Workgroups that share a tile of C along k wait for one another, and every
 * such wait is bounded.  On a GPU that a launch has to itself the waits end
 * at once; beside other launches (other streams, other processes) a workgroup
 * may wait for one that is still queued, and give up.  A piece of a tile whose
 * wait ran out is not added to C; every launch that shares tiles is followed,
 * on the same stream, by a second launch that recomputes exactly what is
 * missing, so the C of every entry point of this library is complete when its
 * stream has run, whether or not a wait ran out - only later.
 * ulmblas_gpu_device_status() waits for the device and says whether that has
 * happened to a launch made through the device entry points of part 2 since
 * the last call: ULMBLAS_GPU_OK if not, ULMBLAS_GPU_RECOVERED (and a text in
 * ulmblas_gpu_last_error()) if so; the count is cleared.  The host entry
 * points of part 1 look for themselves before they return and report through
 * ulmblas_gpu_error_hook(routine, ULMBLAS_GPU_RECOVERED, text); their
 * ulmblas_gpu_last_status() stays ULMBLAS_GPU_OK.  Launches recorded into a
 * HIP graph never share tiles. */
int ulmblas_gpu_device_status(void);
/* Name of variant `id` ("128x128x16_w2x2" ...) or NULL past the last one. */
const char *ulmblas_gpu_variant_name(int precision, int id);

/* Text of the last HIP error seen by this thread ("" if none). */
const char *ulmblas_gpu_last_error(void);

/* The BLAS / CBLAS / LAPACK entry points of part 1 return nothing (or, for
 * ulmblas_dgetrf, LAPACK's info), as the reference's do.  When the GPU side of
 * such a call fails (no device, device memory exhausted, a HIP error) the
 * library waits for whatever the call had started, records the status, and
 * calls ulmblas_gpu_error_hook(routine, status, text), whose default prints
 * one line to stderr and returns; like xerbla_ it can be replaced by the
 * program's own definition.  A call that failed before anything was sent to
 * the device (a failed allocation) leaves its output operand untouched.
 * ulmblas_gpu_last_status(): ULMBLAS_GPU_OK or the status of the calling
 * thread's most recent host entry point call. */
void ulmblas_gpu_error_hook(const char *routine, int status, const char *text);
int ulmblas_gpu_last_status(void);

/* Number of times the host entry points of part 1 had to go to the device
 * allocator (their operand buffers are cached between calls). */
long ulmblas_gpu_alloc_count(void);

/* Frees the cached device buffers of the host entry points. */
void ulmblas_gpu_release(void);

#ifdef __cplusplus
}
#endif
#endif /* ULMBLAS_GPU_H */
