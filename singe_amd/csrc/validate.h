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

// fmha_prefill.cpp: the bf16 / f16 matrix-core prefill with the options of the dense op.  sinks [heads] and mask are
// in the element type of the query; any pointer may be null, window negative and softcap 0 when absent.
struct DenseOptions {
    const uint16_t* sinks = nullptr;
    const int32_t* key_lengths = nullptr;
    const uint16_t* mask = nullptr;
    uint64_t mask_strides[4] = {0, 0, 0, 0};
    long long window = -1;
    float softcap = 0.0f;
};
int32_t dense_prefill_with_options(void* stream, bool f16, uint16_t* out, size_t out_len, const uint16_t* query, size_t query_len,
                                   const uint16_t* key, size_t key_len, const uint16_t* value, size_t value_len,
                                   const SingeFmhaPrefillConfig* config, const DenseOptions& options);

}  // namespace singe_hip
