// Host-side plumbing shared by the entry points: error text, launch checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/q8mi.h"

namespace q8mi {

// Records a message for q8mi_last_error() on the calling thread; returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// Picks up the status of the launch just enqueued (what the reference's
// callers do with cudaGetLastError after each launcher).
int check_launch(const char *what);

inline hipStream_t as_stream(void *s) { return static_cast<hipStream_t>(s); }

// Number of compute units of the current device (cached per device).
int device_cu_count();

}  // namespace q8mi
