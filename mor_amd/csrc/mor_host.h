// Host-side helpers shared by the source files of libmor_hip.so (not exported).
#pragma once

// Records the calling thread's error message (printf style) and returns `code`.
__attribute__((visibility("hidden"))) int mor_fail(int code, const char* fmt, ...);
// hipGetLastError() after a launch: 0 or MOR_ERR_LAUNCH with the message recorded.
__attribute__((visibility("hidden"))) int mor_check_launch(const char* what);
