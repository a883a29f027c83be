// Default error hooks of the BLAS / CBLAS interfaces, as the reference defines
// them (interfaces/blas/F77/xerbla.cc:6-10, interfaces/blas/C/xerbla.cc:6-16):
// print one line to stderr and return.  They are weak so that a program or a
// test harness that brings its own xerbla_ / cblas_xerbla (the netlib testers
// do: test/F77/dblat3.f:2768-2823, test/C/c_xerbla.c:8-85) takes precedence.
#include "../../include/ulmblas_gpu.h"

#include <cstdio>

extern "C" {

__attribute__((weak)) void xerbla_(const char rout[6], const int *info)
{
    fprintf(stderr, "Parameter %d to routine %.6s was incorrect\n", *info, rout);
}

__attribute__((weak)) void cblas_xerbla(int info, const char *rout, const char *form, ...)
{
    (void)form;
    fprintf(stderr, "Parameter %d to routine %s was incorrect\n", info, rout);
}

__attribute__((weak)) void ulmblas_xerbla(int info, const char *rout, const char *form, ...)
{
    (void)form;
    fprintf(stderr, "Parameter %d to routine %s was incorrect\n", info, rout);
}

// What a host entry point calls when the GPU side of its work failed (no
// device, out of device memory, a HIP error): it has no status to return.
__attribute__((weak)) void ulmblas_gpu_error_hook(const char *routine, int status, const char *text)
{
    fprintf(stderr, "libulmblas_gpu: %s failed (status %d): %s\n", routine, status, text);
}

}  // extern "C"
