// Host-side helpers shared by the translation units of the library.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace dlb {

// Records the thread-local message dlb_last_error() returns and hands `code` back (defined in dlblas_fp8_gemm.hip).
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

// Compute units of the current device (cached per device); -1 if hipGetDevice fails.  *dev_out = device ordinal.
int device_cu_count(int* dev_out);

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline bool misaligned(const void* ptr, size_t a) { return (reinterpret_cast<uintptr_t>(ptr) & (a - 1)) != 0; }

}  // namespace dlb
