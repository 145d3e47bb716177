// Error reporting, argument checks and the bookkeeping entry points of the
// C ABI.  Kernels and their launchers live in the .hip files.
#include <stdarg.h>
#include <stdio.h>

#include "cmk_launch.hpp"

namespace cmk {

static thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int hip_status(hipError_t e, const char* what) {
  if (e == hipSuccess) return CMK_OK;
  fail((int)e, "%s: %s", what, hipGetErrorString(e));
  return (int)e;
}

int check_desc(const cmk_gemm_desc* d) {
  if (!d) return fail(CMK_ERR_INVALID_ARG, "null descriptor");
  if (d->L < 0 || d->M < 0 || d->N < 0 || d->K < 0)
    return fail(CMK_ERR_INVALID_ARG, "negative dimension (L=%d M=%d N=%d K=%d)", d->L, d->M, d->N,
                d->K);
  if ((d->transA != 0 && d->transA != 1) || (d->transB != 0 && d->transB != 1))
    return fail(CMK_ERR_INVALID_ARG, "transA/transB must be 0 or 1");
  const long long min_lda = d->transA ? d->M : d->K;
  const long long min_ldb = d->transB ? d->K : d->N;
  if (d->lda < min_lda || d->ldb < min_ldb)
    return fail(CMK_ERR_INVALID_ARG, "leading dimension too small (lda=%lld ldb=%lld)", d->lda,
                d->ldb);
  if (d->strideA < 0 || d->strideB < 0)
    return fail(CMK_ERR_INVALID_ARG, "negative batch stride");
  return CMK_OK;
}

int check_grid(long long work_groups) {
  if (work_groups + 8 > 0x7fffffffLL)
    return fail(CMK_ERR_UNSUPPORTED, "problem needs %lld work-groups, more than one grid holds",
                work_groups);
  return CMK_OK;
}

int compute_units() {
  static thread_local int cached_dev = -1, cached_cus = 256;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (dev != cached_dev) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0)
      cached_cus = cus;
    cached_dev = dev;
  }
  return cached_cus;
}

size_t bmm_workspace_bytes(int L, int M, int N, int K);
size_t min_workspace_bytes(int L, int Xext, int Yext, int K);
size_t min_l2_workspace_bytes(int L, int Xext, int Yext, int K);
size_t topk_workspace_bytes(int L, int Xext, int Yext, int K);
size_t topk1d_workspace_bytes(long long n);

}  // namespace cmk

extern "C" size_t cmk_workspace_bytes(int op, int L, int M, int N, int K, int dim) {
  if (L < 0 || M < 0 || N < 0) return 0;
  switch (op) {
    case CMK_OP_BMM:
      return cmk::bmm_workspace_bytes(L, M, N, K);
    case CMK_OP_MIN_BMM:
      if (dim != 1 && dim != 2) return 0;
      return cmk::min_workspace_bytes(L, dim == 2 ? N : M, dim == 2 ? M : N, K);
    case CMK_OP_MIN_BMM_L2:
      if (dim != 1 && dim != 2) return 0;
      return cmk::min_l2_workspace_bytes(L, dim == 2 ? N : M, dim == 2 ? M : N, K);
    case CMK_OP_TOPK_BMM:
      if (dim != 1 && dim != 2) return 0;
      return cmk::topk_workspace_bytes(L, dim == 2 ? N : M, dim == 2 ? M : N, K);
    case CMK_OP_TOPK_1D:
      return cmk::topk1d_workspace_bytes(M);
    default:
      return 0;
  }
}

extern "C" const char* cmk_last_error(void) { return cmk::g_error; }

extern "C" int cmk_abi_version(void) { return CMK_ABI_VERSION; }
