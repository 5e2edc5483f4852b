// Optional per-launch timing with HIP events, recorded on the stream the kernels run on.
// Off by default; when on, every kernel launch of the library is bracketed by two events and
// the durations can be collected after the stream has been synchronised.  The reference wraps
// its API calls in Legate profiler ranges instead (cupynumeric/_utils/profiling.py:37-73).
#pragma once

#include <hip/hip_runtime.h>

namespace cpn {

bool profiling_enabled();
// Returns a slot id (>= 0) after recording the start event, or -1 when profiling is off or full.
int profile_begin(const char* label, hipStream_t stream);
void profile_end(int slot, hipStream_t stream);

struct ProfileScope {
  int slot;
  hipStream_t stream;
  ProfileScope(const char* label, hipStream_t s) : slot(profiling_enabled() ? profile_begin(label, s) : -1), stream(s) {}
  ~ProfileScope()
  {
    if (slot >= 0) {
      profile_end(slot, stream);
    }
  }
};

}  // namespace cpn
