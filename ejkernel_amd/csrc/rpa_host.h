// Host-side declarations shared by the translation units of librpa_mi355x.so.
#pragma once

#include <hip/hip_runtime.h>

#include "../../include/rpa_mi355x.h"

namespace rpa {

// Each returns RPA_OK or a negative RPA_ERR_* code; all of them only enqueue on `stream`.
int launch_generic(const RpaParams& p, hipStream_t stream);

// Records the calling thread's error message and returns `code`.
int fail(int code, const char* fmt, ...);

}  // namespace rpa
