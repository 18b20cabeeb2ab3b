// Host-side helpers shared by the C-ABI translation units.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>

#include "../../../include/kermac_amd.h"

namespace kmc_host {

// Records a printf-style message for kmc_last_error() on this thread and
// returns `code`, so failures read `return fail(KMC_ERR_..., "...")`.
int fail(int code, const char *format, ...) __attribute__((format(printf, 2, 3)));
int fail_hip(hipError_t error, const char *what);
void clear_error();

// KMC_OK when the device that is current on this thread is a gfx950.
int require_gfx950();

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int ceil_div(int x, int d) { return (x + d - 1) / d; }

}  // namespace kmc_host
