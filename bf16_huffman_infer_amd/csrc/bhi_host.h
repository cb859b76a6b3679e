// Host-side helpers shared by the C-ABI entry points: error reporting only.
#pragma once
#include <hip/hip_runtime.h>
#include "../../include/bhi.h"

// Records `msg` as the calling thread's last error and returns `code`.
int bhi_fail(int code, const char* msg);

// Fetches the status of the launch just enqueued; 0 or a positive hipError_t.
int bhi_launch_status(const char* what);
