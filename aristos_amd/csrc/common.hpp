// Shared host-side declarations of the library (no device code).
#pragma once
#include <cstdarg>
#include <cstdint>
#include <string>

#include "../../include/kleos_amd.h"

namespace kleos_amd {
// Records a printf-style message for kleos_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
}  // namespace kleos_amd
