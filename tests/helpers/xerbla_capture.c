/* Test helper: recording replacements for the BLAS error hooks, loaded into
 * the global symbol scope so that they take precedence over the library's weak
 * defaults -- what the netlib testers do by linking their own XERBLA
 * (test/F77/dblat3.f:2768-2823, test/C/c_xerbla.c:8-85). */
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

static int g_count = 0;
static int g_info = 0;
static char g_name[64] = "";

void capture_reset(void) { g_count = 0; g_info = 0; g_name[0] = 0; }
int capture_count(void) { return g_count; }
int capture_last_info(void) { return g_info; }
const char *capture_last_name(void) { return g_name; }

void xerbla_(const char rout[6], const int *info)
{
    ++g_count;
    g_info = *info;
    memcpy(g_name, rout, 6);
    g_name[6] = 0;
}

void cblas_xerbla(int info, const char *rout, const char *form, ...)
{
    (void)form;
    ++g_count;
    g_info = info;
    strncpy(g_name, rout, sizeof(g_name) - 1);
}

void ulmblas_xerbla(int info, const char *rout, const char *form, ...)
{
    (void)form;
    ++g_count;
    g_info = info;
    strncpy(g_name, rout, sizeof(g_name) - 1);
}

/* the hook of the host entry points for failures on the GPU side */
static int g_hook_count = 0;
static int g_hook_status = 0;
static char g_hook_routine[64] = "";

void hook_reset(void) { g_hook_count = 0; g_hook_status = 0; g_hook_routine[0] = 0; }
int hook_count(void) { return g_hook_count; }
int hook_last_status(void) { return g_hook_status; }
const char *hook_last_routine(void) { return g_hook_routine; }

void ulmblas_gpu_error_hook(const char *routine, int status, const char *text)
{
    (void)text;
    ++g_hook_count;
    g_hook_status = status;
    strncpy(g_hook_routine, routine, sizeof(g_hook_routine) - 1);
}
