// Host-side helpers shared by the source files of libmor_hip.so (not exported).
#pragma once
#include <stdint.h>

// Records the calling thread's error message (printf style) and returns `code`.
__attribute__((visibility("hidden"))) int mor_fail(int code, const char* fmt, ...);
// hipGetLastError() after a launch: 0 or MOR_ERR_LAUNCH with the message recorded.
__attribute__((visibility("hidden"))) int mor_check_launch(const char* what);
// The argument checks common to the entry points that take a tensor and block dims: 0 or MOR_ERR_INVALID_ARGUMENT.
__attribute__((visibility("hidden"))) int mor_validate_shape(const void* input, int64_t rows, int64_t cols, int64_t brows, int64_t bcols);
