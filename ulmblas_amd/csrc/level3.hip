// Symmetric rank-k update and symmetric matrix product for MI355X (gfx950),
// the operations behind ulmBLAS's dsyrk_ / ssyrk_ / cblas_?syrk
// (interfaces/blas/{F77,C}/syrk.cc -> ulmBLAS::sylrk / syurk,
// ulmblas/level3/sylrk.tcc:17-88) and dsymm_ / ssymm_ / cblas_?symm
// (interfaces/blas/{F77,C}/symm.cc -> ulmBLAS::sylmm / syumm,
// ulmblas/level3/sylmm.tcc:16-98).
//
// In the reference both are the GEMM frame with one twist: sylrk hands the
// blocks below the diagonal to mgemm and the diagonal blocks to a variant
// that masks the write-back (msylrk / usylrk); sylmm packs the blocks of the
// symmetric operand from whichever triangle is stored (sylpack).  The same
// two twists here: the rank-k update is the product op(A) op(A)^T restricted
// to the tiles that meet the triangle -- whole tiles inside it through the
// whole-tile GEMM kernel (tiles off the triangle exit at once), the blocks
// on the diagonal beside them through the any-shape kernel with a triangular
// store predicate; the symmetric product reads the blocks of A off the
// diagonal where they are stored -- as they are, or transposed from the other
// side of the diagonal (what sylpack does element by element,
// ulmblas/level3/pack/sylpack.tcc:10-71) -- and completes only the diagonal
// blocks, one at a time, in a small workspace.
#include "internal.h"

#include <algorithm>
#include <cstring>
#include <cctype>
#include <cstdio>
#include <vector>

using namespace ulmgpu;

namespace ulmgpu {

// ---------------------------------------------------------------------------
// C <- beta*C + alpha*op(A)*op(A)^T on one triangle
// ---------------------------------------------------------------------------
template <typename T>
int syrk_device(bool lower, bool trans, int n, int k, T alpha, const T *dA, int ldA, T beta, T *dC, int ldC,
                hipStream_t stream)
{
    const int rowsA = trans ? k : n;
    if (n < 0 || k < 0 || ldA < std::max(1, rowsA) || ldC < std::max(1, n)) {
        g_last_error = "invalid size or leading dimension";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    // ulmblas/level3/sylrk.tcc:38-45
    if (n == 0 || ((alpha == T(0) || k == 0) && beta == T(1))) return ULMBLAS_GPU_OK;
    if (!dC || (alpha != T(0) && k > 0 && !dA)) {
        g_last_error = "null operand";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    if (alpha == T(0) || k == 0) return launch_scale<T>(n, n, beta, dC, ldC, stream, lower ? 1 : -1);
    // op(A) op(A)^T is the product of op(A) with itself transposed; only the
    // tiles that meet the triangle are computed
    return gemm_tri_device<T>(lower ? 1 : -1, trans, !trans, n, k, alpha, dA, ldA, dA, ldA, beta, dC, ldC, stream);
}

// C <- beta*C + alpha*op(A)*op(B)^T + alpha*op(B)*op(A)^T on one triangle: the
// two sweeps of ulmblas/level3/sylr2k.tcc:58-121 as two triangular products,
// the second with beta = 1.  B is addressed with its own leading dimension
// (the reference uses A's for both operands, sylr2k.tcc:66-67,108-109, which
// agrees with this whenever ldA == ldB).
template <typename T>
int syr2k_device(bool lower, bool trans, int n, int k, T alpha, const T *dA, int ldA, const T *dB, int ldB, T beta,
                 T *dC, int ldC, hipStream_t stream)
{
    const int rows = trans ? k : n;
    if (n < 0 || k < 0 || ldA < std::max(1, rows) || ldB < std::max(1, rows) || ldC < std::max(1, n)) {
        g_last_error = "invalid size or leading dimension";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    // ulmblas/level3/sylr2k.tcc:47-56
    if (n == 0 || ((alpha == T(0) || k == 0) && beta == T(1))) return ULMBLAS_GPU_OK;
    if (!dC || (alpha != T(0) && k > 0 && (!dA || !dB))) {
        g_last_error = "null operand";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    const int tri = lower ? 1 : -1;
    if (alpha == T(0) || k == 0) return launch_scale<T>(n, n, beta, dC, ldC, stream, tri);
    int rc = gemm_tri_device<T>(tri, trans, !trans, n, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC, stream);
    if (rc) return rc;
    return gemm_tri_device<T>(tri, trans, !trans, n, k, alpha, dB, ldB, dA, ldA, T(1), dC, ldC, stream);
}

// ---------------------------------------------------------------------------
// C <- beta*C + alpha*A*B (left) or alpha*B*A (right), A symmetric
// ---------------------------------------------------------------------------

// The symmetric product works on diagonal blocks of this order (the workspace
// holds one of them, completed).  Large enough that the products off the
// diagonal keep k >= 2048 and 2048 rows or columns of C.
constexpr int kSymmBlock = 2048;

// F <- the full symmetric matrix of which A holds the `lower` (else upper)
// triangle; F has leading dimension n.  The other triangle of A is not read.
// (F may be A itself, with ldA == n: no element that is read is ever written
// with another value)
template <typename T>
__global__ void symmetrize_kernel(int n, int lower, const T *A, int64_t ldA, T *F)
{
    __shared__ T tile[32][33];
    // one workgroup per 32 x 32 tile on or below the diagonal of F (bi >= bj)
    const int bi = blockIdx.x, bj = blockIdx.y;
    if (bi < bj) return;
    const int tx = threadIdx.x, ty = threadIdx.y;
    // tile (bi, bj) of the lower triangle of the symmetric matrix S: S(i, j), i >= j, is A(i, j) if lower else A(j, i)
    for (int jj = ty; jj < 32; jj += blockDim.y) {
        const int i = bi * 32 + tx, j = bj * 32 + jj;
        T v = T(0);
        if (i < n && j < n && i >= j) {
            v = lower ? A[i + (int64_t)j * ldA] : A[j + (int64_t)i * ldA];
        }
        tile[jj][tx] = v;
    }
    __syncthreads();
    for (int jj = ty; jj < 32; jj += blockDim.y) {
        const int i = bi * 32 + tx, j = bj * 32 + jj;
        if (i < n && j < n && i >= j) F[i + (int64_t)j * n] = tile[jj][tx];
        // the mirror image: F(j', i') for the transposed tile
        const int mi = bj * 32 + tx, mj = bi * 32 + jj;      // element (mi, mj) = S(mj, mi), mj >= mi wanted strictly
        if (mi < n && mj < n && mj > mi) F[mi + (int64_t)mj * n] = tile[tx][jj];
    }
}

template <typename T>
int symm_device(bool right, bool lower, int m, int n, T alpha, const T *dA, int ldA, const T *dB, int ldB, T beta,
                T *dC, int ldC, T *work, hipStream_t stream)
{
    const int ka = right ? n : m;
    if (m < 0 || n < 0 || ldA < std::max(1, ka) || ldB < std::max(1, m) || ldC < std::max(1, m)) {
        g_last_error = "invalid size or leading dimension";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    // ulmblas/level3/sylmm.tcc:47-54
    if (m == 0 || n == 0 || (alpha == T(0) && beta == T(1))) return ULMBLAS_GPU_OK;
    if (!dC) {
        g_last_error = "null operand";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    if (alpha == T(0)) return launch_scale<T>(m, n, beta, dC, ldC, stream);
    if (!dA || !dB || !work) {
        g_last_error = "null operand or workspace";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    // Block row i of A (left side; block column for the right side) is three pieces: left of the diagonal
    // block, the diagonal block, right of it.  One of the outer two is stored as it is needed, the other
    // is the transpose of what is stored on the other side of the diagonal; the diagonal block (order at
    // most kSymmBlock) is completed in `work`.  Three products per block, each into the same rows
    // (columns) of C: the first one applies beta, the others add.
    for (int r0 = 0; r0 < ka; r0 += kSymmBlock) {
        const int nr = std::min(kSymmBlock, ka - r0), after = ka - r0 - nr;
        const T *diag = dA + r0 + (int64_t)r0 * ldA;
        const int tiles = (nr + 31) / 32;
        hipLaunchKernelGGL(symmetrize_kernel<T>, dim3(tiles, tiles), dim3(32, 8), 0, stream, nr, lower ? 1 : 0, diag,
                           (int64_t)ldA, work);
        HIP_TRY(hipGetLastError());
        int rc;
        if (!right) {
            T *Ci = dC + r0;
            if ((rc = gemm_device<T>(false, false, nr, n, nr, alpha, work, nr, dB + r0, ldB, beta, Ci, ldC, stream))) return rc;
            if (r0 > 0) {       // A(r0.., 0..r0): stored there (lower), or the transpose of A(0..r0, r0..) (upper)
                rc = lower ? gemm_device<T>(false, false, nr, n, r0, alpha, dA + r0, ldA, dB, ldB, T(1), Ci, ldC, stream)
                           : gemm_device<T>(true, false, nr, n, r0, alpha, dA + (int64_t)r0 * ldA, ldA, dB, ldB, T(1), Ci, ldC, stream);
                if (rc) return rc;
            }
            if (after > 0) {    // A(r0.., r0+nr..): the transpose of A(r0+nr.., r0..) (lower), or stored there (upper)
                rc = lower ? gemm_device<T>(true, false, nr, n, after, alpha, diag + nr, ldA, dB + r0 + nr, ldB, T(1), Ci, ldC, stream)
                           : gemm_device<T>(false, false, nr, n, after, alpha, diag + (int64_t)nr * ldA, ldA, dB + r0 + nr, ldB, T(1), Ci, ldC, stream);
                if (rc) return rc;
            }
        } else {
            T *Cj = dC + (int64_t)r0 * ldC;
            if ((rc = gemm_device<T>(false, false, m, nr, nr, alpha, dB + (int64_t)r0 * ldB, ldB, work, nr, beta, Cj, ldC, stream))) return rc;
            if (r0 > 0) {       // A(0..r0, r0..): the transpose of A(r0.., 0..r0) (lower), or stored there (upper)
                rc = lower ? gemm_device<T>(false, true, m, nr, r0, alpha, dB, ldB, dA + r0, ldA, T(1), Cj, ldC, stream)
                           : gemm_device<T>(false, false, m, nr, r0, alpha, dB, ldB, dA + (int64_t)r0 * ldA, ldA, T(1), Cj, ldC, stream);
                if (rc) return rc;
            }
            if (after > 0) {    // A(r0+nr.., r0..): stored there (lower), or the transpose of A(r0.., r0+nr..) (upper)
                rc = lower ? gemm_device<T>(false, false, m, nr, after, alpha, dB + (int64_t)(r0 + nr) * ldB, ldB, diag + nr, ldA, T(1), Cj, ldC, stream)
                           : gemm_device<T>(false, true, m, nr, after, alpha, dB + (int64_t)(r0 + nr) * ldB, ldB, diag + (int64_t)nr * ldA, ldA, T(1), Cj, ldC, stream);
                if (rc) return rc;
            }
        }
    }
    return ULMBLAS_GPU_OK;
}

// ---------------------------------------------------------------------------
// host-pointer entry points
// ---------------------------------------------------------------------------
// B == nullptr: the rank-k update; otherwise the rank-2k update with A and B.
template <typename T>
int syrk_host(bool lower, bool trans, int n, int k, T alpha, const T *A, int ldA, const T *B, int ldB, T beta, T *C,
              int ldC)
{
    if (n <= 0 || ((alpha == T(0) || k <= 0) && beta == T(1))) return ULMBLAS_GPU_OK;
    const bool scale_only = alpha == T(0) || k <= 0;
    return with_context([&](HostContext &c) -> int {
    int rc = c.ensure_stream();
    if (rc) return rc;
    const int rowsA = trans ? k : n, colsA = trans ? n : k;
    if ((rc = c.reserve(2, (size_t)n * n * sizeof(T)))) return rc;
    T *dC = static_cast<T *>(c.buf[2]);
    T *dA = nullptr, *dB = nullptr;
    // large operands go up through the pinned rings (pageable memory at the bus's rate)
    const size_t bytes = ((size_t)rowsA * colsA * (B ? 2 : 1) + (size_t)n * n) * sizeof(T);
    const bool streamed = streams_transfers(c, bytes, (size_t)std::max(rowsA, n) * sizeof(T));
    if (!scale_only) {
        if ((rc = c.reserve(0, (size_t)rowsA * colsA * sizeof(T)))) return rc;
        dA = static_cast<T *>(c.buf[0]);
        if ((rc = host_upload<T>(c, streamed, A, ldA, dA, rowsA, rowsA, colsA))) return rc;
        if (B) {
            if ((rc = c.reserve(1, (size_t)rowsA * colsA * sizeof(T)))) return rc;
            dB = static_cast<T *>(c.buf[1]);
            if ((rc = host_upload<T>(c, streamed, B, ldB, dB, rowsA, rowsA, colsA))) return rc;
        }
    }
    // the whole n x n window travels (its other triangle is carried along untouched);
    // beta == 0 never reads C, so nothing is uploaded then
    if (beta != T(0)) {
        if ((rc = host_upload<T>(c, streamed, C, ldC, dC, n, n, n))) return rc;
    }
    rc = B ? syr2k_device<T>(lower, trans, n, k, alpha, dA, std::max(1, rowsA), dB, std::max(1, rowsA), beta, dC, n,
                             c.stream)
           : syrk_device<T>(lower, trans, n, k, alpha, dA, std::max(1, rowsA), beta, dC, n, c.stream);
    if (rc) return rc;
    // Only the triangle goes back; the other triangle of the caller's C is never written.
    constexpr int kBlock = 256;
    if (streamed && (size_t)n * kBlock * sizeof(T) <= PinnedRing::kChunkBytes) {
        // Blocks of 256 columns of the device's C (contiguous) travel into the pinned buffers, and
        // from there every column's part of the triangle is copied to the caller's C while the next
        // block is on its way.
        if ((rc = c.ensure_events(1))) return rc;
        HIP_TRY(hipEventRecord(c.events[0], c.stream));
        HIP_TRY(hipStreamWaitEvent(c.d2h, c.events[0], 0));
        auto drain = [&](int slot, int j0) -> int {
            HIP_TRY(c.out_ring.wait(slot));
            const int jb = std::min(kBlock, n - j0);
            const T *blk = reinterpret_cast<const T *>(c.out_ring.ptr(slot));
            c.pool->run(jb, [&](int j) {
                const int col = j0 + j;
                const int a = lower ? col : 0, b = lower ? n : col + 1;       // rows [a, b) of this column
                memcpy(C + a + (size_t)col * ldC, blk + a + (size_t)j * n, (size_t)(b - a) * sizeof(T));
            });
            return ULMBLAS_GPU_OK;
        };
        int prev_slot = -1, prev_j0 = 0;
        for (int j0 = 0; j0 < n; j0 += kBlock) {
            const int jb = std::min(kBlock, n - j0);
            int slot;
            HIP_TRY(c.out_ring.acquire(slot));
            HIP_TRY(hipMemcpyAsync(c.out_ring.ptr(slot), dC + (size_t)j0 * n, (size_t)n * jb * sizeof(T),
                                   hipMemcpyDeviceToHost, c.d2h));
            HIP_TRY(c.out_ring.mark(slot, c.d2h));
            if (prev_slot >= 0 && (rc = drain(prev_slot, prev_j0))) return rc;
            prev_slot = slot;
            prev_j0 = j0;
        }
        if (prev_slot >= 0 && (rc = drain(prev_slot, prev_j0))) return rc;
        HIP_TRY(hipStreamSynchronize(c.stream));
        return ULMBLAS_GPU_OK;
    }
    // Per block of 256 columns: the rectangle
    // below (lower) or above (upper) the diagonal block straight into C, the
    // diagonal block through a small host buffer from which its triangle is
    // copied.
    std::vector<T> diag((size_t)kBlock * kBlock);
    for (int j0 = 0; j0 < n; j0 += kBlock) {
        const int jb = std::min(kBlock, n - j0);
        const int r0 = lower ? j0 + jb : 0, rows = lower ? n - r0 : j0;
        if ((rc = copy_window<T>(C + r0 + (size_t)j0 * ldC, (size_t)ldC * sizeof(T), dC + r0 + (size_t)j0 * n,
                                 (size_t)n * sizeof(T), rows, jb, hipMemcpyDeviceToHost, c.stream))) return rc;
        if ((rc = copy_window<T>(diag.data(), (size_t)jb * sizeof(T), dC + j0 + (size_t)j0 * n, (size_t)n * sizeof(T),
                                 jb, jb, hipMemcpyDeviceToHost, c.stream))) return rc;
        HIP_TRY(hipStreamSynchronize(c.stream));
        for (int j = 0; j < jb; ++j) {
            const int a = lower ? j : 0, b = lower ? jb : j + 1;           // rows [a, b) of the block's column j
            std::copy(diag.begin() + (size_t)j * jb + a, diag.begin() + (size_t)j * jb + b,
                      C + (size_t)(j0 + a) + (size_t)(j0 + j) * ldC);
        }
    }
    HIP_TRY(hipStreamSynchronize(c.stream));
    return ULMBLAS_GPU_OK;
    });
}

template <typename T>
int symm_host(bool right, bool lower, int m, int n, T alpha, const T *A, int ldA, const T *B, int ldB, T beta, T *C,
              int ldC)
{
    if (m <= 0 || n <= 0 || (alpha == T(0) && beta == T(1))) return ULMBLAS_GPU_OK;
    const int ka = right ? n : m;
    return with_context([&](HostContext &c) -> int {
    int rc = c.ensure_stream();
    if (rc) return rc;
    if ((rc = c.reserve(2, (size_t)m * n * sizeof(T)))) return rc;
    T *dC = static_cast<T *>(c.buf[2]);
    T *dA = nullptr, *dB = nullptr, *work = nullptr;
    const size_t bytes = ((size_t)ka * ka + 2 * (size_t)m * n) * sizeof(T);
    const bool streamed = streams_transfers(c, bytes, (size_t)std::max(ka, m) * sizeof(T));
    if (alpha != T(0)) {
        // buffer 0: the stored window of A, which is completed in place (the copy is the library's own)
        if ((rc = c.reserve(0, (size_t)ka * ka * sizeof(T)))) return rc;
        if ((rc = c.reserve(1, (size_t)m * n * sizeof(T)))) return rc;
        dA = static_cast<T *>(c.buf[0]);
        work = dA;
        dB = static_cast<T *>(c.buf[1]);
        if (streamed) {
            // A goes up and is completed; then B and C travel in panels that do not depend on
            // each other (columns for the left side; rows for the right side, each panel a compact
            // matrix of its own on the device), every panel up, multiplied and on its way back
            // while its neighbours are at another of the three steps.
            const int span = right ? m : n, other = right ? n : m;
            int panels = (int)std::min<long>(32, std::max<long>(1, ((long)m * n) / (4L << 20)));
            const int per = ((span + panels - 1) / panels + 255) / 256 * 256;
            panels = (span + per - 1) / per;
            if ((rc = c.ensure_events(2 * (size_t)panels + 1))) return rc;
            Pipeline<T> pipe(c);
            pipe.set_free_out(c.out_ring.count());
            if ((rc = pipe.upload(A, ldA, dA, ka, ka, ka))) return rc;
            HIP_TRY(hipEventRecord(c.events[2 * panels], c.h2d));
            HIP_TRY(hipStreamWaitEvent(c.stream, c.events[2 * panels], 0));
            const int tiles = (ka + 31) / 32;
            hipLaunchKernelGGL(symmetrize_kernel<T>, dim3(tiles, tiles), dim3(32, 8), 0, c.stream, ka, lower ? 1 : 0, dA,
                               (int64_t)ka, work);
            HIP_TRY(hipGetLastError());
            for (int p = 0; p < panels; ++p) {
                const int r0 = p * per, nr = std::min(per, span - r0);
                const int pm = right ? nr : m, pn = right ? n : nr;       // the panel of B and of C
                T *dBp = dB + (size_t)r0 * other, *dCp = dC + (size_t)r0 * other;
                const T *Bp = right ? B + r0 : B + (size_t)r0 * ldB;
                T *Cp = right ? C + r0 : C + (size_t)r0 * ldC;
                if ((rc = pipe.upload(Bp, ldB, dBp, pm, pm, pn))) return rc;
                if (beta != T(0) && (rc = pipe.upload(Cp, ldC, dCp, pm, pm, pn))) return rc;
                hipEvent_t uploaded = c.events[2 * p], computed = c.events[2 * p + 1];
                HIP_TRY(hipEventRecord(uploaded, c.h2d));
                HIP_TRY(hipStreamWaitEvent(c.stream, uploaded, 0));
                rc = right ? gemm_device<T>(false, false, pm, pn, n, alpha, dBp, pm, work, ka, beta, dCp, pm, c.stream)
                           : gemm_device<T>(false, false, pm, pn, m, alpha, work, ka, dBp, pm, beta, dCp, pm, c.stream);
                if (rc) return rc;
                HIP_TRY(hipEventRecord(computed, c.stream));
                pipe.want_download(dCp, Cp, ldC, pm, pn, computed);
                if ((rc = pipe.pump(false))) return rc;
            }
            if ((rc = pipe.pump(true))) return rc;
            HIP_TRY(hipStreamSynchronize(c.d2h));
            HIP_TRY(hipStreamSynchronize(c.h2d));
            HIP_TRY(hipStreamSynchronize(c.stream));
            return ULMBLAS_GPU_OK;
        }
        if ((rc = host_upload<T>(c, streamed, A, ldA, dA, ka, ka, ka))) return rc;
        if ((rc = host_upload<T>(c, streamed, B, ldB, dB, m, m, n))) return rc;
    }
    if (beta != T(0)) {
        if ((rc = host_upload<T>(c, streamed, C, ldC, dC, m, m, n))) return rc;
    }
    if (alpha == T(0)) {
        if ((rc = launch_scale<T>(m, n, beta, dC, m, c.stream))) return rc;
    } else {
        const int tiles = (ka + 31) / 32;
        hipLaunchKernelGGL(symmetrize_kernel<T>, dim3(tiles, tiles), dim3(32, 8), 0, c.stream, ka, lower ? 1 : 0, dA,
                           (int64_t)ka, work);
        HIP_TRY(hipGetLastError());
        rc = right ? gemm_device<T>(false, false, m, n, n, alpha, dB, m, work, ka, beta, dC, m, c.stream)
                   : gemm_device<T>(false, false, m, n, m, alpha, work, ka, dB, m, beta, dC, m, c.stream);
        if (rc) return rc;
    }
    return host_download<T>(c, streamed, dC, m, C, ldC, m, n);
    });
}

void report(const char *rout, int rc)
{
    report_host_status(rout, rc, nullptr);
}

bool as_stored(int t) { return t == CblasNoTrans || t == AtlasConj; }
bool trans_valid(int t) { return t == CblasNoTrans || t == CblasTrans || t == AtlasConj || t == CblasConjTrans; }

// interfaces/blas/F77/syrk.cc:114-133
int f77_syrk_info(const char *upLo_, const char *trans_, int n, int k, int ldA, int ldC)
{
    const int ul = toupper((unsigned char)*upLo_), tr = toupper((unsigned char)*trans_);
    const int numRowsA = (tr == 'T' || tr == 'C') ? k : n;
    if (ul != 'L' && ul != 'U') return 1;
    if (tr != 'N' && tr != 'T' && tr != 'C' && tr != 'R') return 2;
    if (n < 0) return 3;
    if (k < 0) return 4;
    if (ldA < std::max(1, numRowsA)) return 7;
    if (ldC < std::max(1, n)) return 10;
    return 0;
}

// interfaces/blas/C/syrk.cc:221-250
int cblas_syrk_info(int order, int upLo, int trans, int n, int k, int ldA, int ldC)
{
    const int numRowsA = (order == CblasColMajor) ? (as_stored(trans) ? n : k) : (as_stored(trans) ? k : n);
    if (order != CblasColMajor && order != CblasRowMajor) return 1;
    if (upLo != CblasLower && upLo != CblasUpper) return 2;
    if (!trans_valid(trans)) return 3;
    if (n < 0) return 4;
    if (k < 0) return 5;
    if (ldA < std::max(1, numRowsA)) return 8;
    if (ldC < std::max(1, n)) return 11;
    return 0;
}

// interfaces/blas/F77/symm.cc:119-138
int f77_symm_info(const char *side_, const char *upLo_, int m, int n, int ldA, int ldB, int ldC)
{
    const int sd = toupper((unsigned char)*side_), ul = toupper((unsigned char)*upLo_);
    const int numRowsA = (sd == 'L') ? m : n;
    if (sd != 'L' && sd != 'R') return 1;
    if (ul != 'L' && ul != 'U') return 2;
    if (m < 0) return 3;
    if (n < 0) return 4;
    if (ldA < std::max(1, numRowsA)) return 7;
    if (ldB < std::max(1, m)) return 9;
    if (ldC < std::max(1, m)) return 12;
    return 0;
}

// interfaces/blas/C/symm.cc:261-300
int cblas_symm_info(int order, int side, int upLo, int m, int n, int ldA, int ldB, int ldC)
{
    const int numRowsA = (side == CblasLeft) ? m : n;
    if (order != CblasColMajor && order != CblasRowMajor) return 1;
    if (side != CblasLeft && side != CblasRight) return 2;
    if (upLo != CblasLower && upLo != CblasUpper) return 3;
    if (order == CblasColMajor) {
        if (m < 0) return 4;
        if (n < 0) return 5;
        if (ldA < std::max(1, numRowsA)) return 8;
        if (ldB < std::max(1, m)) return 10;
        if (ldC < std::max(1, m)) return 13;
    } else {
        if (n < 0) return 4;
        if (m < 0) return 5;
        if (ldA < std::max(1, numRowsA)) return 8;
        if (ldB < std::max(1, n)) return 10;
        if (ldC < std::max(1, n)) return 13;
    }
    return 0;
}

template <typename T>
void f77_syrk(const char *name6, const char *rout, const char *upLo, const char *trans, int n, int k, T alpha,
              const T *A, int ldA, T beta, T *C, int ldC)
{
    int info = f77_syrk_info(upLo, trans, n, k, ldA, ldC);
    if (info != 0) {
        xerbla_(name6, &info);
        return;
    }
    const int tr = toupper((unsigned char)*trans);
    report(rout, syrk_host<T>(toupper((unsigned char)*upLo) == 'L', tr == 'T' || tr == 'C', n, k, alpha, A, ldA, nullptr,
                              0, beta, C, ldC));
}

// interfaces/blas/C/syrk.cc:42-69 (ULMBLAS(dsyrk)): unchecked, column-major
template <typename T>
void ulm_syrk(const char *rout, int upLo, int trans, int n, int k, T alpha, const T *A, int ldA, T beta, T *C, int ldC)
{
    report(rout, syrk_host<T>(upLo == CblasLower, !as_stored(trans), n, k, alpha, A, ldA, nullptr, 0, beta, C, ldC));
}

template <typename T>
void cblas_syrk(const char *rout, int order, int upLo, int trans, int n, int k, T alpha, const T *A, int ldA, T beta,
                T *C, int ldC)
{
    int info = cblas_syrk_info(order, upLo, trans, n, k, ldA, ldC);
    if (info != 0) {
        cblas_xerbla(info, rout, "");
        return;
    }
    if (order != CblasColMajor) {   // interfaces/blas/C/syrk.cc:258-261
        upLo = (upLo == CblasUpper) ? CblasLower : CblasUpper;
        trans = as_stored(trans) ? CblasTrans : CblasNoTrans;
    }
    ulm_syrk<T>(rout, upLo, trans, n, k, alpha, A, ldA, beta, C, ldC);
}

// interfaces/blas/F77/syr2k.cc:121-144
int f77_syr2k_info(const char *upLo_, const char *trans_, int n, int k, int ldA, int ldB, int ldC)
{
    const int ul = toupper((unsigned char)*upLo_), tr = toupper((unsigned char)*trans_);
    const int numRows = (tr == 'T' || tr == 'C') ? k : n;
    if (ul != 'L' && ul != 'U') return 1;
    if (tr != 'N' && tr != 'T' && tr != 'C' && tr != 'R') return 2;
    if (n < 0) return 3;
    if (k < 0) return 4;
    if (ldA < std::max(1, numRows)) return 7;
    if (ldB < std::max(1, numRows)) return 9;
    if (ldC < std::max(1, n)) return 12;
    return 0;
}

// interfaces/blas/C/syr2k.cc:238-276
int cblas_syr2k_info(int order, int upLo, int trans, int n, int k, int ldA, int ldB, int ldC)
{
    const int numRows = (order == CblasColMajor) ? (as_stored(trans) ? n : k) : (as_stored(trans) ? k : n);
    if (order != CblasColMajor && order != CblasRowMajor) return 1;
    if (upLo != CblasLower && upLo != CblasUpper) return 2;
    if (!trans_valid(trans)) return 3;
    if (n < 0) return 4;
    if (k < 0) return 5;
    if (ldA < std::max(1, numRows)) return 8;
    if (ldB < std::max(1, numRows)) return 10;
    if (ldC < std::max(1, n)) return 13;
    return 0;
}

template <typename T>
void f77_syr2k(const char *name6, const char *rout, const char *upLo, const char *trans, int n, int k, T alpha,
               const T *A, int ldA, const T *B, int ldB, T beta, T *C, int ldC)
{
    int info = f77_syr2k_info(upLo, trans, n, k, ldA, ldB, ldC);
    if (info != 0) {
        xerbla_(name6, &info);
        return;
    }
    const int tr = toupper((unsigned char)*trans);
    report(rout, syrk_host<T>(toupper((unsigned char)*upLo) == 'L', tr == 'T' || tr == 'C', n, k, alpha, A, ldA, B, ldB,
                              beta, C, ldC));
}

// interfaces/blas/C/syr2k.cc:44-72 (ULMBLAS(dsyr2k)): unchecked, column-major
template <typename T>
void ulm_syr2k(const char *rout, int upLo, int trans, int n, int k, T alpha, const T *A, int ldA, const T *B, int ldB,
               T beta, T *C, int ldC)
{
    report(rout, syrk_host<T>(upLo == CblasLower, !as_stored(trans), n, k, alpha, A, ldA, B, ldB, beta, C, ldC));
}

template <typename T>
void cblas_syr2k(const char *rout, int order, int upLo, int trans, int n, int k, T alpha, const T *A, int ldA,
                 const T *B, int ldB, T beta, T *C, int ldC)
{
    int info = cblas_syr2k_info(order, upLo, trans, n, k, ldA, ldB, ldC);
    if (info != 0) {
        cblas_xerbla(info, rout, "");
        return;
    }
    if (order == CblasColMajor) {
        ulm_syr2k<T>(rout, upLo, trans, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
    } else {                        // interfaces/blas/C/syr2k.cc:284-288: the operands change places
        upLo = (upLo == CblasUpper) ? CblasLower : CblasUpper;
        trans = as_stored(trans) ? CblasTrans : CblasNoTrans;
        ulm_syr2k<T>(rout, upLo, trans, n, k, alpha, B, ldB, A, ldA, beta, C, ldC);
    }
}

template <typename T>
void f77_symm(const char *name6, const char *rout, const char *side, const char *upLo, int m, int n, T alpha,
              const T *A, int ldA, const T *B, int ldB, T beta, T *C, int ldC)
{
    int info = f77_symm_info(side, upLo, m, n, ldA, ldB, ldC);
    if (info != 0) {
        xerbla_(name6, &info);
        return;
    }
    report(rout, symm_host<T>(toupper((unsigned char)*side) == 'R', toupper((unsigned char)*upLo) == 'L', m, n, alpha,
                              A, ldA, B, ldB, beta, C, ldC));
}

// interfaces/blas/C/symm.cc (ULMBLAS(dsymm)): unchecked, column-major
template <typename T>
void ulm_symm(const char *rout, int side, int upLo, int m, int n, T alpha, const T *A, int ldA, const T *B, int ldB,
              T beta, T *C, int ldC)
{
    report(rout, symm_host<T>(side != CblasLeft, upLo == CblasLower, m, n, alpha, A, ldA, B, ldB, beta, C, ldC));
}

template <typename T>
void cblas_symm(const char *rout, int order, int side, int upLo, int m, int n, T alpha, const T *A, int ldA,
                const T *B, int ldB, T beta, T *C, int ldC)
{
    int info = cblas_symm_info(order, side, upLo, m, n, ldA, ldB, ldC);
    if (info != 0) {
        cblas_xerbla(info, rout, "");
        return;
    }
    if (order == CblasColMajor) {
        ulm_symm<T>(rout, side, upLo, m, n, alpha, A, ldA, B, ldB, beta, C, ldC);
    } else {                        // interfaces/blas/C/symm.cc:309-311
        side = (side == CblasLeft) ? CblasRight : CblasLeft;
        upLo = (upLo == CblasUpper) ? CblasLower : CblasUpper;
        ulm_symm<T>(rout, side, upLo, n, m, alpha, A, ldA, B, ldB, beta, C, ldC);
    }
}

}  // namespace ulmgpu

extern "C" {

void dsyrk_(const char *upLo, const char *trans, const int *n, const int *k, const double *alpha, const double *A,
            const int *ldA, const double *beta, double *C, const int *ldC)
{
    f77_syrk<double>("DSYRK ", "dsyrk_", upLo, trans, *n, *k, *alpha, A, *ldA, *beta, C, *ldC);
}

void ssyrk_(const char *upLo, const char *trans, const int *n, const int *k, const float *alpha, const float *A,
            const int *ldA, const float *beta, float *C, const int *ldC)
{
    f77_syrk<float>("SSYRK ", "ssyrk_", upLo, trans, *n, *k, *alpha, A, *ldA, *beta, C, *ldC);
}

void cblas_dsyrk(enum CBLAS_ORDER order, enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n, int k, double alpha,
                 const double *A, int ldA, double beta, double *C, int ldC)
{
    cblas_syrk<double>("cblas_dsyrk", order, upLo, trans, n, k, alpha, A, ldA, beta, C, ldC);
}

void cblas_ssyrk(enum CBLAS_ORDER order, enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n, int k, float alpha,
                 const float *A, int ldA, float beta, float *C, int ldC)
{
    cblas_syrk<float>("cblas_ssyrk", order, upLo, trans, n, k, alpha, A, ldA, beta, C, ldC);
}

void ulmblas_dsyrk(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n, int k, double alpha, const double *A,
                   int ldA, double beta, double *C, int ldC)
{
    ulm_syrk<double>("ulmblas_dsyrk", upLo, trans, n, k, alpha, A, ldA, beta, C, ldC);
}

void ulmblas_ssyrk(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n, int k, float alpha, const float *A,
                   int ldA, float beta, float *C, int ldC)
{
    ulm_syrk<float>("ulmblas_ssyrk", upLo, trans, n, k, alpha, A, ldA, beta, C, ldC);
}

void ATL_dsyrk(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n, int k, double alpha, const double *A, int ldA,
               double beta, double *C, int ldC)
{
    ulmblas_dsyrk(upLo, trans, n, k, alpha, A, ldA, beta, C, ldC);
}

void ATL_ssyrk(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n, int k, float alpha, const float *A, int ldA,
               float beta, float *C, int ldC)
{
    ulmblas_ssyrk(upLo, trans, n, k, alpha, A, ldA, beta, C, ldC);
}

#define ULM_SYR2K_ENTRY_POINTS(P, T, NAME6)                                                                       \
    void P##syr2k_(const char *upLo, const char *trans, const int *n, const int *k, const T *alpha, const T *A,      \
                   const int *ldA, const T *B, const int *ldB, const T *beta, T *C, const int *ldC)                  \
    {                                                                                                                 \
        f77_syr2k<T>(NAME6, #P "syr2k_", upLo, trans, *n, *k, *alpha, A, *ldA, B, *ldB, *beta, C, *ldC);              \
    }                                                                                                                 \
    void cblas_##P##syr2k(enum CBLAS_ORDER order, enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n, int k,    \
                          T alpha, const T *A, int ldA, const T *B, int ldB, T beta, T *C, int ldC)                  \
    {                                                                                                                 \
        cblas_syr2k<T>("cblas_" #P "syr2k", order, upLo, trans, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);           \
    }                                                                                                                 \
    void ulmblas_##P##syr2k(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n, int k, T alpha, const T *A,     \
                            int ldA, const T *B, int ldB, T beta, T *C, int ldC)                                     \
    {                                                                                                                 \
        ulm_syr2k<T>("ulmblas_" #P "syr2k", upLo, trans, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);                  \
    }                                                                                                                 \
    void ATL_##P##syr2k(enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE trans, int n, int k, T alpha, const T *A,         \
                        int ldA, const T *B, int ldB, T beta, T *C, int ldC)                                         \
    {                                                                                                                 \
        ulm_syr2k<T>("ATL_" #P "syr2k", upLo, trans, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);                      \
    }                                                                                                                 \
    int ulmblas_gpu_##P##syr2k(int lower, int trans, int n, int k, T alpha, const T *dA, int ldA, const T *dB,       \
                               int ldB, T beta, T *dC, int ldC, void *stream)                                        \
    {                                                                                                                 \
        return syr2k_device<T>(lower != 0, trans != 0, n, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC,                  \
                               static_cast<hipStream_t>(stream));                                                     \
    }
ULM_SYR2K_ENTRY_POINTS(d, double, "DSYR2K")
ULM_SYR2K_ENTRY_POINTS(s, float, "SSYR2K")

void dsymm_(const char *side, const char *upLo, const int *m, const int *n, const double *alpha, const double *A,
            const int *ldA, const double *B, const int *ldB, const double *beta, double *C, const int *ldC)
{
    f77_symm<double>("DSYMM ", "dsymm_", side, upLo, *m, *n, *alpha, A, *ldA, B, *ldB, *beta, C, *ldC);
}

void ssymm_(const char *side, const char *upLo, const int *m, const int *n, const float *alpha, const float *A,
            const int *ldA, const float *B, const int *ldB, const float *beta, float *C, const int *ldC)
{
    f77_symm<float>("SSYMM ", "ssymm_", side, upLo, *m, *n, *alpha, A, *ldA, B, *ldB, *beta, C, *ldC);
}

void cblas_dsymm(enum CBLAS_ORDER order, enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, int m, int n, double alpha,
                 const double *A, int ldA, const double *B, int ldB, double beta, double *C, int ldC)
{
    cblas_symm<double>("cblas_dsymm", order, side, upLo, m, n, alpha, A, ldA, B, ldB, beta, C, ldC);
}

void cblas_ssymm(enum CBLAS_ORDER order, enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, int m, int n, float alpha,
                 const float *A, int ldA, const float *B, int ldB, float beta, float *C, int ldC)
{
    cblas_symm<float>("cblas_ssymm", order, side, upLo, m, n, alpha, A, ldA, B, ldB, beta, C, ldC);
}

void ulmblas_dsymm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, int m, int n, double alpha, const double *A, int ldA,
                   const double *B, int ldB, double beta, double *C, int ldC)
{
    ulm_symm<double>("ulmblas_dsymm", side, upLo, m, n, alpha, A, ldA, B, ldB, beta, C, ldC);
}

void ulmblas_ssymm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, int m, int n, float alpha, const float *A, int ldA,
                   const float *B, int ldB, float beta, float *C, int ldC)
{
    ulm_symm<float>("ulmblas_ssymm", side, upLo, m, n, alpha, A, ldA, B, ldB, beta, C, ldC);
}

void ATL_dsymm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, int m, int n, double alpha, const double *A, int ldA,
               const double *B, int ldB, double beta, double *C, int ldC)
{
    ulmblas_dsymm(side, upLo, m, n, alpha, A, ldA, B, ldB, beta, C, ldC);
}

void ATL_ssymm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, int m, int n, float alpha, const float *A, int ldA,
               const float *B, int ldB, float beta, float *C, int ldC)
{
    ulmblas_ssymm(side, upLo, m, n, alpha, A, ldA, B, ldB, beta, C, ldC);
}

int ulmblas_gpu_dsyrk(int lower, int trans, int n, int k, double alpha, const double *dA, int ldA, double beta,
                      double *dC, int ldC, void *stream)
{
    return syrk_device<double>(lower != 0, trans != 0, n, k, alpha, dA, ldA, beta, dC, ldC,
                               static_cast<hipStream_t>(stream));
}

int ulmblas_gpu_ssyrk(int lower, int trans, int n, int k, float alpha, const float *dA, int ldA, float beta, float *dC,
                      int ldC, void *stream)
{
    return syrk_device<float>(lower != 0, trans != 0, n, k, alpha, dA, ldA, beta, dC, ldC,
                              static_cast<hipStream_t>(stream));
}

int ulmblas_gpu_dsymm(int right, int lower, int m, int n, double alpha, const double *dA, int ldA, const double *dB,
                      int ldB, double beta, double *dC, int ldC, double *work, void *stream)
{
    return symm_device<double>(right != 0, lower != 0, m, n, alpha, dA, ldA, dB, ldB, beta, dC, ldC, work,
                               static_cast<hipStream_t>(stream));
}

int ulmblas_gpu_ssymm(int right, int lower, int m, int n, float alpha, const float *dA, int ldA, const float *dB,
                      int ldB, float beta, float *dC, int ldC, float *work, void *stream)
{
    return symm_device<float>(right != 0, lower != 0, m, n, alpha, dA, ldA, dB, ldB, beta, dC, ldC, work,
                              static_cast<hipStream_t>(stream));
}

}  // extern "C"
