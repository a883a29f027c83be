// libulmblas_timer: the timing loop of the benchmark, in C so that the rate
// at which launches are enqueued is that of a C caller of the library and not
// that of an interpreter.  Not part of the drop-in library: it links against
// libulmblas_gpu.so and calls its device entry points like any other program.
//
// The loop is the one the reference's timer runs around its tested routine
// (bench/l3blastst.c:1553-1603): the operands of successive calls rotate
// through `sets` sets of matrices, so that with enough sets no call finds its
// operands in a cache the call before it filled.
#include "../../include/ulmblas_gpu.h"

#include <hip/hip_runtime.h>

extern "C" {

// `reps` calls of ulmblas_gpu_dgemm (precision 'd') or ulmblas_gpu_sgemm ('s')
// on `stream`, call i on operand set i % sets (A[s], B[s], C[s]: device
// pointers, arrays in host memory), after `warm` untimed calls that rotate the
// same way.  *ms receives the time between two events recorded on `stream`
// around the timed calls.  Returns the first non-zero status of a call, or
// ULMBLAS_GPU_HIP_ERROR if an event could not be had.
int ulmblas_timer_gemm(int precision, int transA, int transB, int m, int n, int k, double alpha, double beta,
                       const void *const *A, int ldA, const void *const *B, int ldB, void *const *C, int ldC, int sets,
                       int warm, int reps, void *stream, float *ms)
{
    if (sets < 1 || reps < 1 || warm < 0 || !ms || (precision != 'd' && precision != 's')) return ULMBLAS_GPU_BAD_ARGUMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        if (e0) (void)hipEventDestroy(e0);
        return ULMBLAS_GPU_HIP_ERROR;
    }
    int rc = ULMBLAS_GPU_OK;
    auto call = [&](int i) {
        const int q = i % sets;
        if (precision == 'd')
            return ulmblas_gpu_dgemm(transA, transB, m, n, k, alpha, static_cast<const double *>(A[q]), ldA,
                                     static_cast<const double *>(B[q]), ldB, beta, static_cast<double *>(C[q]), ldC, stream);
        return ulmblas_gpu_sgemm(transA, transB, m, n, k, (float)alpha, static_cast<const float *>(A[q]), ldA,
                                 static_cast<const float *>(B[q]), ldB, (float)beta, static_cast<float *>(C[q]), ldC, stream);
    };
    for (int i = 0; i < warm && rc == ULMBLAS_GPU_OK; ++i) rc = call(i);
    if (rc == ULMBLAS_GPU_OK && hipEventRecord(e0, s) != hipSuccess) rc = ULMBLAS_GPU_HIP_ERROR;
    for (int i = 0; i < reps && rc == ULMBLAS_GPU_OK; ++i) rc = call(warm + i);
    if (rc == ULMBLAS_GPU_OK && (hipEventRecord(e1, s) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
                                 hipEventElapsedTime(ms, e0, e1) != hipSuccess))
        rc = ULMBLAS_GPU_HIP_ERROR;
    if (rc != ULMBLAS_GPU_OK) (void)hipStreamSynchronize(s);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return rc;
}

}  // extern "C"
