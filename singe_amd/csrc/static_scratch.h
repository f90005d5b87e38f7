// Address and size of the library's fixed device scratch on the current device (see static_scratch.hip).
#pragma once

#include <stddef.h>

#include "singe_hip_attention.h"  // SINGE_HIP_STATIC_SCRATCH_BYTES: the one place the size is written

namespace singe_hip {

// Returns 0 and the array's device address on the current device, resolving it on the first call there, or
// the negated hipError_t.  Allocates nothing; the first call on a device must not run under stream capture.
int static_scratch(void** pointer, size_t* bytes);

}  // namespace singe_hip
