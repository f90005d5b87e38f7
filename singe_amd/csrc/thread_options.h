// The calling thread's settings, over the process-wide ones.  The reference keeps its numerical policy per thread
// (singe/src/graph/numerics/mod.rs:44-49: thread_local! NUMERICAL_POLICY) and passes tuning choices in the call
// (singe-kernel/src/cuda/attention/mod.rs:2364-2380); here a thread installs SingeHipThreadOptions, and a size
// query and the launch that follows it on that thread read the same values whatever other threads set.
#pragma once

#include <stdint.h>

#include "singe_hip_attention.h"

namespace singe_hip {

// The thread's options (all fields at "follow the process" when the thread has installed none).
const SingeHipThreadOptions& thread_options();

// A process-wide value, unless the calling thread has set its own.
inline bool effective_relaxed(bool process) {
    const int32_t own = thread_options().relaxed_numerics;
    return own < 0 ? process : own != 0;
}
inline uint32_t effective_count(uint32_t own, uint32_t process) { return own != 0 ? own : process; }

}  // namespace singe_hip
