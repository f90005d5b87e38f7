// Address and size of the library's fixed device scratch on the current device (see static_scratch.hip).
#pragma once

#include <stddef.h>

// 16 MiB per GPU: the paged decode scratch of up to 760 sequences at 32 query / 8 KV heads on 256 compute units
// (the first benchmark decode shape needs 4.7 MB of it).
#ifndef SINGE_HIP_STATIC_SCRATCH_BYTES
#define SINGE_HIP_STATIC_SCRATCH_BYTES (16u << 20)
#endif

namespace singe_hip {

// Returns 0 and the array's device address on the current device, resolving it on the first call there, or
// the negated hipError_t.  Allocates nothing; the first call on a device must not run under stream capture.
int static_scratch(void** pointer, size_t* bytes);

}  // namespace singe_hip
