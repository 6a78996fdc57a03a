// Optional per-kernel timing with HIP events, for callers that want kernel durations without an
// external profiler.  Off by default; when on, every kernel launch site brackets its launch with
// two events on the launch stream.
#pragma once
#include "rexsc_common.h"

namespace rexsc {

// RAII bracket around one kernel launch: records start in the constructor, stop in the destructor.
// name must be a string literal.  work = algorithmic lane-ops (or bytes) of the launch.
struct ProfScope {
    ProfScope(const char *name, double work, hipStream_t stream);
    ~ProfScope();
    int slot;
    hipStream_t stream;
};

} // namespace rexsc
