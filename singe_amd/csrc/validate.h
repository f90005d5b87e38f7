// Checked arithmetic and length checks shared by the entry points; the counterparts of
// singe-kernel/src/utility.rs:4-11 (checked_i32_value, checked_element_count) and :245-266
// (ensure_len_at_least).
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "module.h"
#include "singe_hip_attention.h"

namespace singe_hip {

inline bool fits_i32(uint64_t value) { return value <= 0x7fffffffull; }

inline bool checked_mul(size_t a, size_t b, size_t* out) { return !__builtin_mul_overflow(a, b, out); }
inline bool checked_add(size_t a, size_t b, size_t* out) { return !__builtin_add_overflow(a, b, out); }

inline int32_t ensure_len_at_least(const char* name, size_t actual, size_t minimum) {
    if (actual < minimum) return fail(SINGE_HIP_LENGTH_TOO_SHORT, name, minimum, actual);
    return 0;
}

}  // namespace singe_hip
