// Complex GEMM for MI355X (gfx950): zgemm_ / cgemm_, cblas_zgemm / cblas_cgemm
// and the ulmblas_ / ATL_ forms (interfaces/blas/F77/gemm.cc:251-506,
// interfaces/blas/C/gemm.cc:140-293, 488-690 -> ulmBLAS::gemm with conjugation
// flags, ulmblas/level3/gemm.tcc:13-87, gepack.tcc:21-37).
//
// The reference runs its one GEMM frame on std::complex numbers.  Here the
// complex product is one *real* product on the matrix cores: a column-major
// complex matrix is, read as real numbers, a matrix with twice the rows (real
// and imaginary parts alternate down each column), and
//
//     C~ (2m x n)  =  E (2m x 2k)  *  B~ (2k x n)  +  beta * C~
//
// where C~ and B~ are C and op(B) read as real matrices and E is the real
// 2 x 2 block form of alpha*op(A): the block of element z = x + iy is
// [x -y; y x].  Row 2i of the product is Re(sum_l alpha a_il b_lj), row 2i+1
// its imaginary part, each a plain sum of 2k real products -- the "4M" way of
// multiplying complex matrices, with the 8mnk real flops running in the same
// MFMA kernel as dgemm / sgemm and the result landing interleaved in C with
// the fused beta epilogue.  Preparation is O(mk + kn) work: one kernel builds
// E (transposing / conjugating / scaling by alpha on the way), one more
// materialises op(B) when B is transposed or conjugated; a beta with a
// non-zero imaginary part scales C beforehand.
#include "internal.h"

#include <algorithm>
#include <cctype>
#include <cstdio>

using namespace ulmgpu;

namespace ulmgpu {

int f77_info(const char *transA_, const char *transB_, int m, int n, int k, int ldA, int ldB, int ldC, bool &transA,
             bool &transB);
int cblas_info(int order, int transA, int transB, int m, int n, int k, int ldA, int ldB, int ldC);

// E <- the 2m x 2k real block form of alpha*op(A); op(A) is m x k, A is stored
// with leading dimension ldA (complex elements), transposed and / or
// conjugated as the flags say.  32 x 32 tiles through LDS so that both the
// reads of A and the writes of E run along columns.
template <typename R>
__global__ void embed_kernel(int m, int k, int trans, int conj, R ar, R ai, const R *__restrict__ A, int64_t ldA,
                             R *__restrict__ E, int64_t ldE)
{
    __shared__ R tre[32][33], tim[32][33];
    const int i0 = blockIdx.x * 32, l0 = blockIdx.y * 32;
    for (int r = threadIdx.y; r < 32; r += 8) {
        const int i = trans ? i0 + r : i0 + (int)threadIdx.x;
        const int l = trans ? l0 + (int)threadIdx.x : l0 + r;
        if (i < m && l < k) {
            const R *p = A + 2 * (trans ? (l + (int64_t)i * ldA) : (i + (int64_t)l * ldA));
            const R re = p[0], im = conj ? -p[1] : p[1];
            tre[i - i0][l - l0] = ar * re - ai * im;
            tim[i - i0][l - l0] = ar * im + ai * re;
        }
    }
    __syncthreads();
    for (int r = threadIdx.y; r < 32; r += 8) {
        const int i = i0 + (int)threadIdx.x, l = l0 + r;
        if (i < m && l < k) {
            const R x = tre[threadIdx.x][r], y = tim[threadIdx.x][r];
            R *c0 = E + 2 * (int64_t)i + (int64_t)(2 * l) * ldE;
            R *c1 = c0 + ldE;
            c0[0] = x;
            c0[1] = y;
            c1[0] = -y;
            c1[1] = x;
        }
    }
}

// Out <- op(B) as a compact k x n complex matrix (leading dimension k); B is
// stored transposed and / or conjugated as the flags say.
template <typename R>
__global__ void opcopy_kernel(int k, int n, int trans, int conj, const R *__restrict__ B, int64_t ldB,
                              R *__restrict__ Out)
{
    __shared__ R tre[32][33], tim[32][33];
    const int l0 = blockIdx.x * 32, j0 = blockIdx.y * 32;
    for (int r = threadIdx.y; r < 32; r += 8) {
        const int l = trans ? l0 + r : l0 + (int)threadIdx.x;
        const int j = trans ? j0 + (int)threadIdx.x : j0 + r;
        if (l < k && j < n) {
            const R *p = B + 2 * (trans ? (j + (int64_t)l * ldB) : (l + (int64_t)j * ldB));
            tre[l - l0][j - j0] = p[0];
            tim[l - l0][j - j0] = conj ? -p[1] : p[1];
        }
    }
    __syncthreads();
    for (int r = threadIdx.y; r < 32; r += 8) {
        const int l = l0 + (int)threadIdx.x, j = j0 + r;
        if (l < k && j < n) {
            R *q = Out + 2 * ((int64_t)l + (int64_t)j * k);
            q[0] = tre[threadIdx.x][r];
            q[1] = tim[threadIdx.x][r];
        }
    }
}

// C <- beta*C on the m x n complex window, beta = br + i*bi with bi != 0
template <typename R>
__global__ void cscale_kernel(int m, int n, R br, R bi, R *C, int64_t ldC)
{
    const long total = (long)m * n;
    for (long t = blockIdx.x * (long)blockDim.x + threadIdx.x; t < total; t += (long)gridDim.x * blockDim.x) {
        const long i = t % m, j = t / m;
        R *p = C + 2 * (i + j * ldC);
        const R x = p[0], y = p[1];
        p[0] = x * br - y * bi;
        p[1] = x * bi + y * br;
    }
}

bool t_valid(int t) { return t == CblasNoTrans || t == CblasTrans || t == CblasConjTrans || t == AtlasConj; }
bool t_trans(int t) { return t == CblasTrans || t == CblasConjTrans; }
bool t_conj(int t) { return t == CblasConjTrans || t == AtlasConj; }

template <typename R>
size_t cgemm_worksize(int transB, int m, int n, int k)
{
    size_t bytes = (size_t)4 * std::max(m, 0) * std::max(k, 0) * sizeof(R);
    if (transB != CblasNoTrans) bytes += (size_t)2 * std::max(k, 0) * std::max(n, 0) * sizeof(R);
    return bytes;
}

// C <- alpha*op(A)*op(B) + beta*C on device-resident complex operands
// (interleaved re, im; leading dimensions in complex elements).
template <typename R>
int cgemm_device(int transA, int transB, int m, int n, int k, const R *alpha, const R *dA, int ldA, const R *dB,
                 int ldB, const R *beta, R *dC, int ldC, void *work, hipStream_t stream)
{
    if (!t_valid(transA) || !t_valid(transB)) {
        g_last_error = "invalid transposition flag";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    const bool ta = t_trans(transA), tb = t_trans(transB);
    const int rowsA = ta ? k : m, rowsB = tb ? n : k;
    if (m < 0 || n < 0 || k < 0 || ldA < std::max(1, rowsA) || ldB < std::max(1, rowsB) || ldC < std::max(1, m) ||
        m > (1 << 30) || k > (1 << 30) || ldB > (1 << 30) || ldC > (1 << 30)) {
        g_last_error = "invalid size or leading dimension";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    if (!alpha || !beta) {
        g_last_error = "null scalar";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    const R ar = alpha[0], ai = alpha[1], br = beta[0], bi = beta[1];
    if (m == 0 || n == 0) return ULMBLAS_GPU_OK;
    const bool no_product = (ar == R(0) && ai == R(0)) || k == 0;
    if (!dC || (!no_product && (!dA || !dB || !work))) {
        g_last_error = "null operand or workspace";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    // a complex beta scales C in a pass of its own; a real one rides in the GEMM epilogue
    R beta_real = br;
    if (bi != R(0)) {
        const long total = (long)m * n;
        const unsigned blocks = (unsigned)std::min<long>((total + 255) / 256, 65536);
        hipLaunchKernelGGL(cscale_kernel<R>, dim3(blocks), dim3(256), 0, stream, m, n, br, bi, dC, (int64_t)ldC);
        HIP_TRY(hipGetLastError());
        beta_real = R(1);
    }
    // ulmblas/level3/gemm.tcc:52-55
    if (no_product) {
        if (beta_real == R(1)) return ULMBLAS_GPU_OK;
        return launch_scale<R>(2 * m, n, beta_real, dC, 2 * (int64_t)ldC, stream);
    }
    R *E = static_cast<R *>(work);
    hipLaunchKernelGGL(embed_kernel<R>, dim3((m + 31) / 32, (k + 31) / 32), dim3(32, 8), 0, stream, m, k, ta ? 1 : 0,
                       t_conj(transA) ? 1 : 0, ar, ai, dA, (int64_t)ldA, E, (int64_t)2 * m);
    HIP_TRY(hipGetLastError());
    const R *Bt = dB;
    int ldBt = 2 * ldB;
    if (transB != CblasNoTrans) {
        R *out = E + (size_t)4 * m * k;
        hipLaunchKernelGGL(opcopy_kernel<R>, dim3((k + 31) / 32, (n + 31) / 32), dim3(32, 8), 0, stream, k, n,
                           tb ? 1 : 0, t_conj(transB) ? 1 : 0, dB, (int64_t)ldB, out);
        HIP_TRY(hipGetLastError());
        Bt = out;
        ldBt = 2 * k;
    }
    return gemm_device<R>(false, false, 2 * m, n, 2 * k, R(1), E, 2 * m, Bt, ldBt, beta_real, dC, 2 * ldC, stream);
}

// Host-pointer path: operands go up whole, the product runs, C comes back.
template <typename R>
int cgemm_host(int transA, int transB, int m, int n, int k, const R *alpha, const R *A, int ldA, const R *B, int ldB,
               const R *beta, R *C, int ldC)
{
    if (m <= 0 || n <= 0) return ULMBLAS_GPU_OK;
    const bool no_product = (alpha[0] == R(0) && alpha[1] == R(0)) || k <= 0;
    const bool beta_one = beta[0] == R(1) && beta[1] == R(0), beta_zero = beta[0] == R(0) && beta[1] == R(0);
    if (no_product && beta_one) return ULMBLAS_GPU_OK;
    return with_context([&](HostContext &c) -> int {
    int rc = c.ensure_stream();
    if (rc) return rc;
    typedef R Z[2];
    const size_t zs = sizeof(Z);
    const bool ta = t_trans(transA), tb = t_trans(transB);
    const int rowsA = ta ? k : m, colsA = ta ? m : k, rowsB = tb ? n : k, colsB = tb ? k : n;
    if ((rc = c.reserve(2, (size_t)m * n * zs))) return rc;
    R *dC = static_cast<R *>(c.buf[2]);
    R *dA = nullptr, *dB = nullptr;
    void *work = nullptr;
    // large operands travel through the pinned rings (as windows of real numbers, two per element)
    const int per = (int)(zs / sizeof(R));
    const size_t bytes = ((size_t)rowsA * colsA + (size_t)rowsB * colsB + (size_t)m * n) * zs;
    const bool streamed = streams_transfers(c, bytes, (size_t)std::max(std::max(rowsA, rowsB), m) * zs);
    if (!no_product) {
        // buffer 0: A followed by the workspace; buffer 1: B
        const size_t a_bytes = ((size_t)rowsA * colsA * zs + 255) / 256 * 256;
        if ((rc = c.reserve(0, a_bytes + cgemm_worksize<R>(transB, m, n, k)))) return rc;
        if ((rc = c.reserve(1, (size_t)rowsB * colsB * zs))) return rc;
        dA = static_cast<R *>(c.buf[0]);
        work = static_cast<char *>(c.buf[0]) + a_bytes;
        dB = static_cast<R *>(c.buf[1]);
        if (streamed && (long)m * n >= (8L << 20)) {
            // A goes up and becomes the real block form E once; then C is cut into column panels and
            // for each panel its part of op(B) (and of C when beta != 0) goes up, is brought into the
            // form the product wants, is multiplied and comes back, panels overlapping each other's
            // transfers and kernels as in dgemm_'s streamed path.  A transposed or conjugated B is
            // kept panel by panel on the device, each panel a compact matrix of its own.
            const R ar = alpha[0], ai = alpha[1], br = beta[0], bi = beta[1];
            int panels = (int)std::min<long>(32, std::max<long>(1, ((long)m * n) / (2L << 20)));
            const int nb = ((n + panels - 1) / panels + 255) / 256 * 256;
            panels = (n + nb - 1) / nb;
            if ((rc = c.ensure_events(2 * (size_t)panels + 1))) return rc;
            Pipeline<R> pipe(c);
            pipe.set_free_out(c.out_ring.count());
            if ((rc = pipe.upload(A, (size_t)ldA * per, dA, (size_t)rowsA * per, (size_t)rowsA * per, colsA))) return rc;
            HIP_TRY(hipEventRecord(c.events[2 * panels], c.h2d));
            HIP_TRY(hipStreamWaitEvent(c.stream, c.events[2 * panels], 0));
            R *E = static_cast<R *>(work);
            hipLaunchKernelGGL(embed_kernel<R>, dim3((m + 31) / 32, (k + 31) / 32), dim3(32, 8), 0, c.stream, m, k,
                               ta ? 1 : 0, t_conj(transA) ? 1 : 0, ar, ai, dA, (int64_t)std::max(1, rowsA), E,
                               (int64_t)2 * m);
            HIP_TRY(hipGetLastError());
            for (int p = 0; p < panels; ++p) {
                const int j0 = p * nb, nj = std::min(nb, n - j0);
                R *dBp = dB + (size_t)2 * j0 * k;          // k x nj as stored (no transposition) or nj x k, compact
                if (!tb) {
                    rc = pipe.upload(B + (size_t)2 * j0 * ldB, (size_t)ldB * per, dBp, (size_t)k * per, (size_t)k * per, nj);
                } else {
                    rc = pipe.upload(B + (size_t)2 * j0, (size_t)ldB * per, dBp, (size_t)nj * per, (size_t)nj * per, k);
                }
                if (rc) return rc;
                R *dCp = dC + (size_t)2 * j0 * m;
                R *Cp = C + (size_t)2 * j0 * ldC;
                if (!beta_zero && (rc = pipe.upload(Cp, (size_t)ldC * per, dCp, (size_t)m * per, (size_t)m * per, nj))) return rc;
                hipEvent_t uploaded = c.events[2 * p], computed = c.events[2 * p + 1];
                HIP_TRY(hipEventRecord(uploaded, c.h2d));
                HIP_TRY(hipStreamWaitEvent(c.stream, uploaded, 0));
                R beta_real = br;
                if (bi != R(0)) {        // a complex beta scales C in a pass of its own
                    const long total = (long)m * nj;
                    const unsigned blocks = (unsigned)std::min<long>((total + 255) / 256, 65536);
                    hipLaunchKernelGGL(cscale_kernel<R>, dim3(blocks), dim3(256), 0, c.stream, m, nj, br, bi, dCp, (int64_t)m);
                    HIP_TRY(hipGetLastError());
                    beta_real = R(1);
                }
                const R *Bt = dBp;
                if (transB != CblasNoTrans) {
                    R *out = E + (size_t)4 * m * k + (size_t)2 * j0 * k;
                    hipLaunchKernelGGL(opcopy_kernel<R>, dim3((k + 31) / 32, (nj + 31) / 32), dim3(32, 8), 0, c.stream, k, nj,
                                       tb ? 1 : 0, t_conj(transB) ? 1 : 0, dBp, (int64_t)(tb ? nj : k), out);
                    HIP_TRY(hipGetLastError());
                    Bt = out;
                }
                if ((rc = gemm_device<R>(false, false, 2 * m, nj, 2 * k, R(1), E, 2 * m, Bt, 2 * k, beta_real, dCp, 2 * m,
                                         c.stream))) return rc;
                HIP_TRY(hipEventRecord(computed, c.stream));
                pipe.want_download(dCp, Cp, (size_t)ldC * per, (size_t)m * per, nj, computed);
                if ((rc = pipe.pump(false))) return rc;
            }
            if ((rc = pipe.pump(true))) return rc;
            HIP_TRY(hipStreamSynchronize(c.d2h));
            HIP_TRY(hipStreamSynchronize(c.h2d));
            HIP_TRY(hipStreamSynchronize(c.stream));
            return ULMBLAS_GPU_OK;
        }
        if ((rc = host_upload<R>(c, streamed, A, (size_t)ldA * per, dA, (size_t)rowsA * per, (size_t)rowsA * per,
                                 colsA))) return rc;
        if ((rc = host_upload<R>(c, streamed, B, (size_t)ldB * per, dB, (size_t)rowsB * per, (size_t)rowsB * per,
                                 colsB))) return rc;
    }
    if (!beta_zero) {
        if ((rc = host_upload<R>(c, streamed, C, (size_t)ldC * per, dC, (size_t)m * per, (size_t)m * per, n))) return rc;
    }
    if ((rc = cgemm_device<R>(transA, transB, m, n, k, alpha, dA, std::max(1, rowsA), dB, std::max(1, rowsB), beta, dC,
                              m, work, c.stream))) return rc;
    return host_download<R>(c, streamed, dC, (size_t)m * per, C, (size_t)ldC * per, (size_t)m * per, n);
    });
}

template <typename R>
void cgemm_report(const char *rout, int transA, int transB, int m, int n, int k, const R *alpha, const R *A, int ldA,
                  const R *B, int ldB, const R *beta, R *C, int ldC)
{
    const int rc = cgemm_host<R>(transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
    report_host_status(rout, rc, nullptr);
}

// interfaces/blas/F77/gemm.cc:270-274: 'T' and 'C' transpose, 'C' and 'R' conjugate
int f77_trans(const char *t_)
{
    switch (toupper((unsigned char)*t_)) {
    case 'T': return CblasTrans;
    case 'C': return CblasConjTrans;
    case 'R': return AtlasConj;
    default: return CblasNoTrans;
    }
}

template <typename R>
void f77_cgemm(const char *name6, const char *rout, const char *transA_, const char *transB_, int m, int n, int k,
               const R *alpha, const R *A, int ldA, const R *B, int ldB, const R *beta, R *C, int ldC)
{
    bool ta, tb;
    int info = f77_info(transA_, transB_, m, n, k, ldA, ldB, ldC, ta, tb);
    if (info != 0) {
        xerbla_(name6, &info);
        return;
    }
    cgemm_report<R>(rout, f77_trans(transA_), f77_trans(transB_), m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
}

template <typename R>
void cblas_cgemm_(const char *rout, int order, int transA, int transB, int m, int n, int k, const R *alpha, const R *A,
                  int ldA, const R *B, int ldB, const R *beta, R *C, int ldC)
{
    int info = cblas_info(order, transA, transB, m, n, k, ldA, ldB, ldC);
    if (info != 0) {
        cblas_xerbla(info, rout, "");
        return;
    }
    if (order == CblasColMajor) {
        cgemm_report<R>(rout, transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
    } else {    // interfaces/blas/C/gemm.cc:683-688: C^T = op(B)^T op(A)^T
        cgemm_report<R>(rout, transB, transA, n, m, k, alpha, B, ldB, A, ldA, beta, C, ldC);
    }
}

}  // namespace ulmgpu

extern "C" {

void zgemm_(const char *transA, const char *transB, const int *m, const int *n, const int *k, const double *alpha,
            const double *A, const int *ldA, const double *B, const int *ldB, const double *beta, double *C,
            const int *ldC)
{
    f77_cgemm<double>("ZGEMM ", "zgemm_", transA, transB, *m, *n, *k, alpha, A, *ldA, B, *ldB, beta, C, *ldC);
}

void cgemm_(const char *transA, const char *transB, const int *m, const int *n, const int *k, const float *alpha,
            const float *A, const int *ldA, const float *B, const int *ldB, const float *beta, float *C,
            const int *ldC)
{
    f77_cgemm<float>("CGEMM ", "cgemm_", transA, transB, *m, *n, *k, alpha, A, *ldA, B, *ldB, beta, C, *ldC);
}

void cblas_zgemm(enum CBLAS_ORDER order, enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m, int n, int k,
                 const double *alpha, const double *A, int ldA, const double *B, int ldB, const double *beta,
                 double *C, int ldC)
{
    cblas_cgemm_<double>("cblas_zgemm", order, transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
}

void cblas_cgemm(enum CBLAS_ORDER order, enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m, int n, int k,
                 const float *alpha, const float *A, int ldA, const float *B, int ldB, const float *beta, float *C,
                 int ldC)
{
    cblas_cgemm_<float>("cblas_cgemm", order, transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
}

void ulmblas_zgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m, int n, int k, const double *alpha,
                   const double *A, int ldA, const double *B, int ldB, const double *beta, double *C, int ldC)
{
    cgemm_report<double>("ulmblas_zgemm", transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
}

void ulmblas_cgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m, int n, int k, const float *alpha,
                   const float *A, int ldA, const float *B, int ldB, const float *beta, float *C, int ldC)
{
    cgemm_report<float>("ulmblas_cgemm", transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
}

void ATL_zgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m, int n, int k, const double *alpha,
               const double *A, int ldA, const double *B, int ldB, const double *beta, double *C, int ldC)
{
    cgemm_report<double>("ATL_zgemm", transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
}

void ATL_cgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m, int n, int k, const float *alpha,
               const float *A, int ldA, const float *B, int ldB, const float *beta, float *C, int ldC)
{
    cgemm_report<float>("ATL_cgemm", transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
}

long ulmblas_gpu_zgemm_worksize(enum CBLAS_TRANSPOSE transB, int m, int n, int k)
{
    return (long)cgemm_worksize<double>(transB, m, n, k);
}

long ulmblas_gpu_cgemm_worksize(enum CBLAS_TRANSPOSE transB, int m, int n, int k)
{
    return (long)cgemm_worksize<float>(transB, m, n, k);
}

int ulmblas_gpu_zgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m, int n, int k,
                      const double *alpha, const double *dA, int ldA, const double *dB, int ldB, const double *beta,
                      double *dC, int ldC, void *work, void *stream)
{
    return cgemm_device<double>(transA, transB, m, n, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC, work,
                                static_cast<hipStream_t>(stream));
}

int ulmblas_gpu_cgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m, int n, int k,
                      const float *alpha, const float *dA, int ldA, const float *dB, int ldB, const float *beta,
                      float *dC, int ldC, void *work, void *stream)
{
    return cgemm_device<float>(transA, transB, m, n, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC, work,
                               static_cast<hipStream_t>(stream));
}

}  // extern "C"
