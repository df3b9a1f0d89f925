// Host-side helpers of the C ABI: error reporting and argument checks.
#pragma once
#include <hip/hip_runtime.h>
#include <algorithm>
#include <stddef.h>
#include <stdint.h>

#include "../../include/spgt_hip.h"

namespace spgt {

// Records `msg` as the calling thread's last error and returns `code`.
int fail(int code, const char* msg);

// Returns SPGT_OK, or SPGT_ERR_LAUNCH (with the HIP error string recorded) if
// a kernel launch issued by `what` since the last check was rejected.
int check_launch(const char* what);

// Compute units of the current device (cached per device; 256 if the query fails).
int device_cu_count();

// Lets kernel `fn` be launched with up to `bytes` of dynamic LDS on the current device (above 64 KB a kernel has to
// be allowed, per device).  The runtime is asked once per (device, kernel, size class) and the answer remembered;
// false when it refused, in which case the launch that follows fails and check_launch reports it.  A host call,
// not a stream operation: callers that capture graphs make one call outside the capture first.
bool allow_dynamic_lds(const void* fn, size_t bytes);
template <class K>
bool allow_dynamic_lds(K kernel, size_t bytes) {
    return allow_dynamic_lds(reinterpret_cast<const void*>(kernel), bytes);
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }
inline bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

}  // namespace spgt
