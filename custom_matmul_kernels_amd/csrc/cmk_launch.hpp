// Host-side helpers shared by the translation units of libcmk.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/cmk.h"

namespace cmk {

// Records a message for cmk_last_error() on this thread and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Maps a hipError_t to the ABI's return convention (0 or the positive code).
int hip_status(hipError_t e, const char* what);

// Validates the fields every GEMM-family entry point shares.
int check_desc(const cmk_gemm_desc* d);

// A 1-D grid index must fit the hardware limit.
int check_grid(long long work_groups);

// 16-byte global loads need an aligned base and strides that keep it aligned.
static inline int vec_ok(const void* p, long long ld, long long stride) {
  return ((reinterpret_cast<uintptr_t>(p) & 15) == 0 && (ld & 3) == 0 && (stride & 3) == 0) ? 1 : 0;
}

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Compute units of the current device (cached per device).
int compute_units();

}  // namespace cmk
