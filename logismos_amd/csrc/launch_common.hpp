// Host-side helpers shared by the launchers: status type, rejection messages.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/logismos_decode.h"

namespace lg {

// Writes the reason (if the caller wants one) and returns hipErrorInvalidValue.
inline logismos_status_t reject(char* msg, size_t cap, const char* fmt, ...) {
    if (msg && cap) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(msg, cap, fmt, ap);
        va_end(ap);
    }
    return static_cast<logismos_status_t>(hipErrorInvalidValue);
}

}  // namespace lg
