// Error convention of the library: every fallible host function returns a Status (0 = OK) and
// leaves a message for infmoe_last_error(); nothing aborts or throws across the C ABI.  The
// reference prints and exits instead (plugin/utility.h:13-21,41-47).  Status, fail() and the message
// slot are part of the public plug-in header; this one adds what only the library's own sources use.
#pragma once

#include <hip/hip_runtime_api.h>

#include "../../include/infmoe_sublayer.h"

namespace infmoe {

inline Status hip_fail(hipError_t err, const char* what) {
    return fail(INFMOE_ERR_HIP, "%s: %s", what, hipGetErrorString(err));
}

#define INFMOE_HIP(call)                                                   \
    do {                                                                   \
        hipError_t _e = (call);                                            \
        if (_e != hipSuccess) return ::infmoe::hip_fail(_e, #call);        \
    } while (0)

#define INFMOE_TRY(call)                                                   \
    do {                                                                   \
        ::infmoe::Status _s = (call);                                      \
        if (_s != INFMOE_OK) return _s;                                    \
    } while (0)

inline size_t align_up(size_t v, size_t a = 256) { return (v + a - 1) / a * a; }

}  // namespace infmoe
