#include "module.h"

#include <dlfcn.h>

#include <atomic>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "singe_hip_attention.h"
#include "static_scratch.h"
#include "thread_options.h"

namespace singe_hip {

const char* const kKernelNames[kKernelCount] = {
    "singe_paged_decode_bf16_d128_g1_b16", "singe_paged_decode_bf16_d128_g2_b16",
    "singe_paged_decode_bf16_d128_g1_any", "singe_paged_decode_bf16_d128_g2_any",
    "singe_paged_decode_combine_bf16",
    "singe_paged_decode_f16_d128_g1_b16", "singe_paged_decode_f16_d128_g2_b16",
    "singe_paged_decode_f16_d128_g1_any", "singe_paged_decode_f16_d128_g2_any",
    "singe_paged_decode_combine_f16",
    "singe_paged_decode_f8kv_wide_d128_b16", "singe_paged_decode_f8kv_wide_d128_any",
    "singe_paged_decode_f8kv_wide_relaxed_d128_b16", "singe_paged_decode_f8kv_wide_relaxed_d128_any",
    "singe_fmha_prefill_bf16_d128_causal", "singe_fmha_prefill_bf16_d128_full",
    "singe_fmha_prefill_f16_d128_causal", "singe_fmha_prefill_f16_d128_full",
    "singe_fmha_prefill_bf16_d128_causal_options", "singe_fmha_prefill_bf16_d128_full_options",
    "singe_fmha_prefill_f16_d128_causal_options", "singe_fmha_prefill_f16_d128_full_options",
    "singe_fmha_prefill_f32_d32", "singe_fmha_prefill_f32_d64", "singe_fmha_prefill_f32_d128", "singe_fmha_prefill_f32_d256",
    "singe_paged_attention_bf16_d128_i32", "singe_paged_attention_bf16_d128_i64",
    "singe_paged_attention_bf16_d128_softcap_i32", "singe_paged_attention_bf16_d128_softcap_i64",
    "singe_paged_attention_bf16_d128_i32_p16", "singe_paged_attention_bf16_d128_i64_p16",
    "singe_paged_attention_bf16_d128_softcap_i32_p16", "singe_paged_attention_bf16_d128_softcap_i64_p16",
    "singe_paged_kv_prefill_bf16_d128", "singe_paged_kv_prefill_bf16_d128_p16",
    "singe_paged_kv_prefill_f16_d128", "singe_paged_kv_prefill_f16_d128_p16",
    "singe_paged_attention_combine_bf16_i32", "singe_paged_attention_combine_bf16_i64",
    "singe_paged_attention_combine_f16_i32", "singe_paged_attention_combine_f16_i64",
    "singe_paged_attention_f16_d128_i32", "singe_paged_attention_f16_d128_i64",
    "singe_paged_attention_f16_d128_softcap_i32", "singe_paged_attention_f16_d128_softcap_i64",
    "singe_paged_attention_f16_d128_i32_p16", "singe_paged_attention_f16_d128_i64_p16",
    "singe_paged_attention_f16_d128_softcap_i32_p16", "singe_paged_attention_f16_d128_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d128_i32", "singe_rotary_paged_attention_bf16_d128_i64",
    "singe_rotary_paged_attention_bf16_d128_i32_p16", "singe_rotary_paged_attention_bf16_d128_i64_p16",
    "singe_splitk_reduce_f32",
    "singe_fmha_decode_splitk_f32_d4", "singe_fmha_decode_splitk_f32_d8", "singe_fmha_decode_splitk_f32_d16",
    "singe_fmha_decode_splitk_f32_d32", "singe_fmha_decode_splitk_f32_d64", "singe_fmha_decode_splitk_f32_d128",
    "singe_fmha_decode_splitk_f32_d256",
    "singe_paged_kv_decode_splitk_f32_d4", "singe_paged_kv_decode_splitk_f32_d8", "singe_paged_kv_decode_splitk_f32_d16",
    "singe_paged_kv_decode_splitk_f32_d32", "singe_paged_kv_decode_splitk_f32_d64", "singe_paged_kv_decode_splitk_f32_d128",
    "singe_paged_kv_decode_splitk_f32_d256",
    "singe_paged_kv_prefill_f32_d4", "singe_paged_kv_prefill_f32_d8", "singe_paged_kv_prefill_f32_d16",
    "singe_paged_kv_prefill_f32_d32", "singe_paged_kv_prefill_f32_d64", "singe_paged_kv_prefill_f32_d128",
    "singe_paged_kv_prefill_f32_d256",
    "singe_fmha_prefill_rows_f32_d4", "singe_fmha_prefill_rows_f32_d8", "singe_fmha_prefill_rows_f32_d16",
    "singe_fmha_prefill_rows_f32_d32", "singe_fmha_prefill_rows_f32_d64", "singe_fmha_prefill_rows_f32_d128",
    "singe_fmha_prefill_rows_f32_d256",
    "singe_rotary_cache_write_f32", "singe_rotary_cache_write_bf16", "singe_rotary_cache_write_f16",
    "singe_paging_indices_i32", "singe_paging_indices_i64",
    "singe_paged_mla_attention_general_f32", "singe_paged_mla_attention_general_bf16", "singe_paged_mla_attention_general_f16",
    "singe_paged_mla_attention_bf16_l512_p64", "singe_paged_mla_attention_f16_l512_p64",
    "singe_paged_mla_attention_combine_bf16", "singe_paged_mla_attention_combine_f16",
    "singe_attention_general_f32_d64", "singe_attention_general_f32_d128", "singe_attention_general_f32_d256",
    "singe_attention_general_bf16_d64", "singe_attention_general_bf16_d128", "singe_attention_general_bf16_d256",
    "singe_attention_general_f16_d64", "singe_attention_general_f16_d128", "singe_attention_general_f16_d256",
    "singe_paged_attention_general_f32_d64", "singe_paged_attention_general_f32_d128", "singe_paged_attention_general_f32_d256",
    "singe_paged_attention_general_bf16_d64", "singe_paged_attention_general_bf16_d128", "singe_paged_attention_general_bf16_d256",
    "singe_paged_attention_general_f16_d64", "singe_paged_attention_general_f16_d128", "singe_paged_attention_general_f16_d256",
    "singe_mfma_ceiling_bf16", "singe_mfma_ceiling_f16",
    "singe_paged_decode_bf16_d64_g1_b16", "singe_paged_decode_bf16_d64_g2_b16",
    "singe_paged_decode_bf16_d64_g1_any", "singe_paged_decode_bf16_d64_g2_any",
    "singe_paged_decode_combine_bf16_d64", "singe_paged_decode_f16_d64_g1_b16",
    "singe_paged_decode_f16_d64_g2_b16", "singe_paged_decode_f16_d64_g1_any",
    "singe_paged_decode_f16_d64_g2_any", "singe_paged_decode_combine_f16_d64",
    "singe_fmha_prefill_bf16_d64_causal", "singe_fmha_prefill_bf16_d64_full",
    "singe_fmha_prefill_f16_d64_causal", "singe_fmha_prefill_f16_d64_full",
    "singe_fmha_prefill_bf16_d64_causal_options", "singe_fmha_prefill_bf16_d64_full_options",
    "singe_fmha_prefill_f16_d64_causal_options", "singe_fmha_prefill_f16_d64_full_options",
    "singe_paged_attention_bf16_d64_i32", "singe_paged_attention_bf16_d64_i64",
    "singe_paged_attention_bf16_d64_softcap_i32", "singe_paged_attention_bf16_d64_softcap_i64",
    "singe_paged_attention_bf16_d64_i32_p16", "singe_paged_attention_bf16_d64_i64_p16",
    "singe_paged_attention_bf16_d64_softcap_i32_p16", "singe_paged_attention_bf16_d64_softcap_i64_p16",
    "singe_paged_kv_prefill_bf16_d64", "singe_paged_kv_prefill_bf16_d64_p16",
    "singe_paged_kv_prefill_f16_d64", "singe_paged_kv_prefill_f16_d64_p16",
    "singe_paged_attention_combine_bf16_d64_i32", "singe_paged_attention_combine_bf16_d64_i64",
    "singe_paged_attention_combine_f16_d64_i32", "singe_paged_attention_combine_f16_d64_i64",
    "singe_paged_attention_f16_d64_i32", "singe_paged_attention_f16_d64_i64",
    "singe_paged_attention_f16_d64_softcap_i32", "singe_paged_attention_f16_d64_softcap_i64",
    "singe_paged_attention_f16_d64_i32_p16", "singe_paged_attention_f16_d64_i64_p16",
    "singe_paged_attention_f16_d64_softcap_i32_p16", "singe_paged_attention_f16_d64_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d64_i32", "singe_rotary_paged_attention_bf16_d64_i64",
    "singe_rotary_paged_attention_bf16_d64_i32_p16", "singe_rotary_paged_attention_bf16_d64_i64_p16",
    "singe_fmha_prefill_bf16_d128_combine", "singe_fmha_prefill_f16_d128_combine",
    "singe_fmha_prefill_bf16_d64_combine", "singe_fmha_prefill_f16_d64_combine",
    "singe_attention_general_f64_d64", "singe_attention_general_f64_d128", "singe_attention_general_f64_d256",
    "singe_paged_attention_general_f64_d64", "singe_paged_attention_general_f64_d128", "singe_paged_attention_general_f64_d256",
    "singe_hbm_stream_read",
    "singe_fmha_prefill_bf16_d32_causal", "singe_fmha_prefill_bf16_d32_full",
    "singe_fmha_prefill_f16_d32_causal", "singe_fmha_prefill_f16_d32_full",
    "singe_fmha_prefill_bf16_d32_causal_options", "singe_fmha_prefill_bf16_d32_full_options",
    "singe_fmha_prefill_f16_d32_causal_options", "singe_fmha_prefill_f16_d32_full_options",
    "singe_fmha_prefill_bf16_d32_combine", "singe_fmha_prefill_f16_d32_combine",
    "singe_paged_attention_bf16_d32_i32", "singe_paged_attention_bf16_d32_i64",
    "singe_paged_attention_bf16_d32_softcap_i32", "singe_paged_attention_bf16_d32_softcap_i64",
    "singe_paged_attention_bf16_d32_i32_p16", "singe_paged_attention_bf16_d32_i64_p16",
    "singe_paged_attention_bf16_d32_softcap_i32_p16", "singe_paged_attention_bf16_d32_softcap_i64_p16",
    "singe_paged_kv_prefill_bf16_d32", "singe_paged_kv_prefill_bf16_d32_p16",
    "singe_paged_kv_prefill_f16_d32", "singe_paged_kv_prefill_f16_d32_p16",
    "singe_paged_attention_combine_bf16_d32_i32", "singe_paged_attention_combine_bf16_d32_i64",
    "singe_paged_attention_combine_f16_d32_i32", "singe_paged_attention_combine_f16_d32_i64",
    "singe_paged_attention_f16_d32_i32", "singe_paged_attention_f16_d32_i64",
    "singe_paged_attention_f16_d32_softcap_i32", "singe_paged_attention_f16_d32_softcap_i64",
    "singe_paged_attention_f16_d32_i32_p16", "singe_paged_attention_f16_d32_i64_p16",
    "singe_paged_attention_f16_d32_softcap_i32_p16", "singe_paged_attention_f16_d32_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d32_i32", "singe_rotary_paged_attention_bf16_d32_i64",
    "singe_rotary_paged_attention_bf16_d32_i32_p16", "singe_rotary_paged_attention_bf16_d32_i64_p16",
    "singe_fmha_prefill_bf16_d96_causal", "singe_fmha_prefill_bf16_d96_full",
    "singe_fmha_prefill_f16_d96_causal", "singe_fmha_prefill_f16_d96_full",
    "singe_fmha_prefill_bf16_d96_causal_options", "singe_fmha_prefill_bf16_d96_full_options",
    "singe_fmha_prefill_f16_d96_causal_options", "singe_fmha_prefill_f16_d96_full_options",
    "singe_fmha_prefill_bf16_d96_combine", "singe_fmha_prefill_f16_d96_combine",
    "singe_paged_attention_bf16_d96_i32", "singe_paged_attention_bf16_d96_i64",
    "singe_paged_attention_bf16_d96_softcap_i32", "singe_paged_attention_bf16_d96_softcap_i64",
    "singe_paged_attention_bf16_d96_i32_p16", "singe_paged_attention_bf16_d96_i64_p16",
    "singe_paged_attention_bf16_d96_softcap_i32_p16", "singe_paged_attention_bf16_d96_softcap_i64_p16",
    "singe_paged_kv_prefill_bf16_d96", "singe_paged_kv_prefill_bf16_d96_p16",
    "singe_paged_kv_prefill_f16_d96", "singe_paged_kv_prefill_f16_d96_p16",
    "singe_paged_attention_combine_bf16_d96_i32", "singe_paged_attention_combine_bf16_d96_i64",
    "singe_paged_attention_combine_f16_d96_i32", "singe_paged_attention_combine_f16_d96_i64",
    "singe_paged_attention_f16_d96_i32", "singe_paged_attention_f16_d96_i64",
    "singe_paged_attention_f16_d96_softcap_i32", "singe_paged_attention_f16_d96_softcap_i64",
    "singe_paged_attention_f16_d96_i32_p16", "singe_paged_attention_f16_d96_i64_p16",
    "singe_paged_attention_f16_d96_softcap_i32_p16", "singe_paged_attention_f16_d96_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d96_i32", "singe_rotary_paged_attention_bf16_d96_i64",
    "singe_rotary_paged_attention_bf16_d96_i32_p16", "singe_rotary_paged_attention_bf16_d96_i64_p16",
    "singe_fmha_prefill_bf16_d16_causal", "singe_fmha_prefill_bf16_d16_full",
    "singe_fmha_prefill_f16_d16_causal", "singe_fmha_prefill_f16_d16_full",
    "singe_fmha_prefill_bf16_d16_causal_options", "singe_fmha_prefill_bf16_d16_full_options",
    "singe_fmha_prefill_f16_d16_causal_options", "singe_fmha_prefill_f16_d16_full_options",
    "singe_fmha_prefill_bf16_d16_combine", "singe_fmha_prefill_f16_d16_combine",
    "singe_paged_attention_bf16_d16_i32", "singe_paged_attention_bf16_d16_i64",
    "singe_paged_attention_bf16_d16_softcap_i32", "singe_paged_attention_bf16_d16_softcap_i64",
    "singe_paged_attention_bf16_d16_i32_p16", "singe_paged_attention_bf16_d16_i64_p16",
    "singe_paged_attention_bf16_d16_softcap_i32_p16", "singe_paged_attention_bf16_d16_softcap_i64_p16",
    "singe_paged_kv_prefill_bf16_d16", "singe_paged_kv_prefill_bf16_d16_p16",
    "singe_paged_kv_prefill_f16_d16", "singe_paged_kv_prefill_f16_d16_p16",
    "singe_paged_attention_combine_bf16_d16_i32", "singe_paged_attention_combine_bf16_d16_i64",
    "singe_paged_attention_combine_f16_d16_i32", "singe_paged_attention_combine_f16_d16_i64",
    "singe_paged_attention_f16_d16_i32", "singe_paged_attention_f16_d16_i64",
    "singe_paged_attention_f16_d16_softcap_i32", "singe_paged_attention_f16_d16_softcap_i64",
    "singe_paged_attention_f16_d16_i32_p16", "singe_paged_attention_f16_d16_i64_p16",
    "singe_paged_attention_f16_d16_softcap_i32_p16", "singe_paged_attention_f16_d16_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d16_i32", "singe_rotary_paged_attention_bf16_d16_i64",
    "singe_rotary_paged_attention_bf16_d16_i32_p16", "singe_rotary_paged_attention_bf16_d16_i64_p16",
    "singe_fmha_prefill_bf16_d48_causal", "singe_fmha_prefill_bf16_d48_full",
    "singe_fmha_prefill_f16_d48_causal", "singe_fmha_prefill_f16_d48_full",
    "singe_fmha_prefill_bf16_d48_causal_options", "singe_fmha_prefill_bf16_d48_full_options",
    "singe_fmha_prefill_f16_d48_causal_options", "singe_fmha_prefill_f16_d48_full_options",
    "singe_fmha_prefill_bf16_d48_combine", "singe_fmha_prefill_f16_d48_combine",
    "singe_paged_attention_bf16_d48_i32", "singe_paged_attention_bf16_d48_i64",
    "singe_paged_attention_bf16_d48_softcap_i32", "singe_paged_attention_bf16_d48_softcap_i64",
    "singe_paged_attention_bf16_d48_i32_p16", "singe_paged_attention_bf16_d48_i64_p16",
    "singe_paged_attention_bf16_d48_softcap_i32_p16", "singe_paged_attention_bf16_d48_softcap_i64_p16",
    "singe_paged_kv_prefill_bf16_d48", "singe_paged_kv_prefill_bf16_d48_p16",
    "singe_paged_kv_prefill_f16_d48", "singe_paged_kv_prefill_f16_d48_p16",
    "singe_paged_attention_combine_bf16_d48_i32", "singe_paged_attention_combine_bf16_d48_i64",
    "singe_paged_attention_combine_f16_d48_i32", "singe_paged_attention_combine_f16_d48_i64",
    "singe_paged_attention_f16_d48_i32", "singe_paged_attention_f16_d48_i64",
    "singe_paged_attention_f16_d48_softcap_i32", "singe_paged_attention_f16_d48_softcap_i64",
    "singe_paged_attention_f16_d48_i32_p16", "singe_paged_attention_f16_d48_i64_p16",
    "singe_paged_attention_f16_d48_softcap_i32_p16", "singe_paged_attention_f16_d48_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d48_i32", "singe_rotary_paged_attention_bf16_d48_i64",
    "singe_rotary_paged_attention_bf16_d48_i32_p16", "singe_rotary_paged_attention_bf16_d48_i64_p16",
    "singe_fmha_prefill_bf16_d80_causal", "singe_fmha_prefill_bf16_d80_full",
    "singe_fmha_prefill_f16_d80_causal", "singe_fmha_prefill_f16_d80_full",
    "singe_fmha_prefill_bf16_d80_causal_options", "singe_fmha_prefill_bf16_d80_full_options",
    "singe_fmha_prefill_f16_d80_causal_options", "singe_fmha_prefill_f16_d80_full_options",
    "singe_fmha_prefill_bf16_d80_combine", "singe_fmha_prefill_f16_d80_combine",
    "singe_paged_attention_bf16_d80_i32", "singe_paged_attention_bf16_d80_i64",
    "singe_paged_attention_bf16_d80_softcap_i32", "singe_paged_attention_bf16_d80_softcap_i64",
    "singe_paged_attention_bf16_d80_i32_p16", "singe_paged_attention_bf16_d80_i64_p16",
    "singe_paged_attention_bf16_d80_softcap_i32_p16", "singe_paged_attention_bf16_d80_softcap_i64_p16",
    "singe_paged_kv_prefill_bf16_d80", "singe_paged_kv_prefill_bf16_d80_p16",
    "singe_paged_kv_prefill_f16_d80", "singe_paged_kv_prefill_f16_d80_p16",
    "singe_paged_attention_combine_bf16_d80_i32", "singe_paged_attention_combine_bf16_d80_i64",
    "singe_paged_attention_combine_f16_d80_i32", "singe_paged_attention_combine_f16_d80_i64",
    "singe_paged_attention_f16_d80_i32", "singe_paged_attention_f16_d80_i64",
    "singe_paged_attention_f16_d80_softcap_i32", "singe_paged_attention_f16_d80_softcap_i64",
    "singe_paged_attention_f16_d80_i32_p16", "singe_paged_attention_f16_d80_i64_p16",
    "singe_paged_attention_f16_d80_softcap_i32_p16", "singe_paged_attention_f16_d80_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d80_i32", "singe_rotary_paged_attention_bf16_d80_i64",
    "singe_rotary_paged_attention_bf16_d80_i32_p16", "singe_rotary_paged_attention_bf16_d80_i64_p16",
    "singe_fmha_prefill_bf16_d112_causal", "singe_fmha_prefill_bf16_d112_full",
    "singe_fmha_prefill_f16_d112_causal", "singe_fmha_prefill_f16_d112_full",
    "singe_fmha_prefill_bf16_d112_causal_options", "singe_fmha_prefill_bf16_d112_full_options",
    "singe_fmha_prefill_f16_d112_causal_options", "singe_fmha_prefill_f16_d112_full_options",
    "singe_fmha_prefill_bf16_d112_combine", "singe_fmha_prefill_f16_d112_combine",
    "singe_paged_attention_bf16_d112_i32", "singe_paged_attention_bf16_d112_i64",
    "singe_paged_attention_bf16_d112_softcap_i32", "singe_paged_attention_bf16_d112_softcap_i64",
    "singe_paged_attention_bf16_d112_i32_p16", "singe_paged_attention_bf16_d112_i64_p16",
    "singe_paged_attention_bf16_d112_softcap_i32_p16", "singe_paged_attention_bf16_d112_softcap_i64_p16",
    "singe_paged_kv_prefill_bf16_d112", "singe_paged_kv_prefill_bf16_d112_p16",
    "singe_paged_kv_prefill_f16_d112", "singe_paged_kv_prefill_f16_d112_p16",
    "singe_paged_attention_combine_bf16_d112_i32", "singe_paged_attention_combine_bf16_d112_i64",
    "singe_paged_attention_combine_f16_d112_i32", "singe_paged_attention_combine_f16_d112_i64",
    "singe_paged_attention_f16_d112_i32", "singe_paged_attention_f16_d112_i64",
    "singe_paged_attention_f16_d112_softcap_i32", "singe_paged_attention_f16_d112_softcap_i64",
    "singe_paged_attention_f16_d112_i32_p16", "singe_paged_attention_f16_d112_i64_p16",
    "singe_paged_attention_f16_d112_softcap_i32_p16", "singe_paged_attention_f16_d112_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d112_i32", "singe_rotary_paged_attention_bf16_d112_i64",
    "singe_rotary_paged_attention_bf16_d112_i32_p16", "singe_rotary_paged_attention_bf16_d112_i64_p16",
    "singe_paged_decode_bf16_wide_d128_b16", "singe_paged_decode_bf16_wide_d128_any",
    "singe_paged_decode_f16_wide_d128_b16", "singe_paged_decode_f16_wide_d128_any",
    "singe_paged_decode_combine_many_bf16", "singe_paged_decode_combine_many_f16",
    "singe_paged_decode_combine_many_bf16_d64", "singe_paged_decode_combine_many_f16_d64",
    "singe_rotary_cache_write_chunks_f32", "singe_rotary_cache_write_chunks_bf16", "singe_rotary_cache_write_chunks_f16",
    "singe_paged_decode_combine_few_bf16", "singe_paged_decode_combine_few_f16",
    "singe_paged_decode_combine_few_bf16_d64", "singe_paged_decode_combine_few_f16_d64",
    "singe_paged_decode_rows_i32", "singe_paged_decode_rows_i64",
    // the fused query rotation beyond bf16 without a cap: per head dimension (128, 64, 32, 96, 16, 48, 80, 112) bf16 with a
    // cap, f16, f16 with a cap, four index / page forms each
    "singe_rotary_paged_attention_bf16_d128_softcap_i32", "singe_rotary_paged_attention_bf16_d128_softcap_i64",
    "singe_rotary_paged_attention_bf16_d128_softcap_i32_p16", "singe_rotary_paged_attention_bf16_d128_softcap_i64_p16",
    "singe_rotary_paged_attention_f16_d128_i32", "singe_rotary_paged_attention_f16_d128_i64",
    "singe_rotary_paged_attention_f16_d128_i32_p16", "singe_rotary_paged_attention_f16_d128_i64_p16",
    "singe_rotary_paged_attention_f16_d128_softcap_i32", "singe_rotary_paged_attention_f16_d128_softcap_i64",
    "singe_rotary_paged_attention_f16_d128_softcap_i32_p16", "singe_rotary_paged_attention_f16_d128_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d64_softcap_i32", "singe_rotary_paged_attention_bf16_d64_softcap_i64",
    "singe_rotary_paged_attention_bf16_d64_softcap_i32_p16", "singe_rotary_paged_attention_bf16_d64_softcap_i64_p16",
    "singe_rotary_paged_attention_f16_d64_i32", "singe_rotary_paged_attention_f16_d64_i64",
    "singe_rotary_paged_attention_f16_d64_i32_p16", "singe_rotary_paged_attention_f16_d64_i64_p16",
    "singe_rotary_paged_attention_f16_d64_softcap_i32", "singe_rotary_paged_attention_f16_d64_softcap_i64",
    "singe_rotary_paged_attention_f16_d64_softcap_i32_p16", "singe_rotary_paged_attention_f16_d64_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d32_softcap_i32", "singe_rotary_paged_attention_bf16_d32_softcap_i64",
    "singe_rotary_paged_attention_bf16_d32_softcap_i32_p16", "singe_rotary_paged_attention_bf16_d32_softcap_i64_p16",
    "singe_rotary_paged_attention_f16_d32_i32", "singe_rotary_paged_attention_f16_d32_i64",
    "singe_rotary_paged_attention_f16_d32_i32_p16", "singe_rotary_paged_attention_f16_d32_i64_p16",
    "singe_rotary_paged_attention_f16_d32_softcap_i32", "singe_rotary_paged_attention_f16_d32_softcap_i64",
    "singe_rotary_paged_attention_f16_d32_softcap_i32_p16", "singe_rotary_paged_attention_f16_d32_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d96_softcap_i32", "singe_rotary_paged_attention_bf16_d96_softcap_i64",
    "singe_rotary_paged_attention_bf16_d96_softcap_i32_p16", "singe_rotary_paged_attention_bf16_d96_softcap_i64_p16",
    "singe_rotary_paged_attention_f16_d96_i32", "singe_rotary_paged_attention_f16_d96_i64",
    "singe_rotary_paged_attention_f16_d96_i32_p16", "singe_rotary_paged_attention_f16_d96_i64_p16",
    "singe_rotary_paged_attention_f16_d96_softcap_i32", "singe_rotary_paged_attention_f16_d96_softcap_i64",
    "singe_rotary_paged_attention_f16_d96_softcap_i32_p16", "singe_rotary_paged_attention_f16_d96_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d16_softcap_i32", "singe_rotary_paged_attention_bf16_d16_softcap_i64",
    "singe_rotary_paged_attention_bf16_d16_softcap_i32_p16", "singe_rotary_paged_attention_bf16_d16_softcap_i64_p16",
    "singe_rotary_paged_attention_f16_d16_i32", "singe_rotary_paged_attention_f16_d16_i64",
    "singe_rotary_paged_attention_f16_d16_i32_p16", "singe_rotary_paged_attention_f16_d16_i64_p16",
    "singe_rotary_paged_attention_f16_d16_softcap_i32", "singe_rotary_paged_attention_f16_d16_softcap_i64",
    "singe_rotary_paged_attention_f16_d16_softcap_i32_p16", "singe_rotary_paged_attention_f16_d16_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d48_softcap_i32", "singe_rotary_paged_attention_bf16_d48_softcap_i64",
    "singe_rotary_paged_attention_bf16_d48_softcap_i32_p16", "singe_rotary_paged_attention_bf16_d48_softcap_i64_p16",
    "singe_rotary_paged_attention_f16_d48_i32", "singe_rotary_paged_attention_f16_d48_i64",
    "singe_rotary_paged_attention_f16_d48_i32_p16", "singe_rotary_paged_attention_f16_d48_i64_p16",
    "singe_rotary_paged_attention_f16_d48_softcap_i32", "singe_rotary_paged_attention_f16_d48_softcap_i64",
    "singe_rotary_paged_attention_f16_d48_softcap_i32_p16", "singe_rotary_paged_attention_f16_d48_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d80_softcap_i32", "singe_rotary_paged_attention_bf16_d80_softcap_i64",
    "singe_rotary_paged_attention_bf16_d80_softcap_i32_p16", "singe_rotary_paged_attention_bf16_d80_softcap_i64_p16",
    "singe_rotary_paged_attention_f16_d80_i32", "singe_rotary_paged_attention_f16_d80_i64",
    "singe_rotary_paged_attention_f16_d80_i32_p16", "singe_rotary_paged_attention_f16_d80_i64_p16",
    "singe_rotary_paged_attention_f16_d80_softcap_i32", "singe_rotary_paged_attention_f16_d80_softcap_i64",
    "singe_rotary_paged_attention_f16_d80_softcap_i32_p16", "singe_rotary_paged_attention_f16_d80_softcap_i64_p16",
    "singe_rotary_paged_attention_bf16_d112_softcap_i32", "singe_rotary_paged_attention_bf16_d112_softcap_i64",
    "singe_rotary_paged_attention_bf16_d112_softcap_i32_p16", "singe_rotary_paged_attention_bf16_d112_softcap_i64_p16",
    "singe_rotary_paged_attention_f16_d112_i32", "singe_rotary_paged_attention_f16_d112_i64",
    "singe_rotary_paged_attention_f16_d112_i32_p16", "singe_rotary_paged_attention_f16_d112_i64_p16",
    "singe_rotary_paged_attention_f16_d112_softcap_i32", "singe_rotary_paged_attention_f16_d112_softcap_i64",
    "singe_rotary_paged_attention_f16_d112_softcap_i32_p16", "singe_rotary_paged_attention_f16_d112_softcap_i64_p16",
    "singe_paged_mla_attention_bf16_any", "singe_paged_mla_attention_f16_any",
    "singe_paged_mla_attention_combine_bf16_any", "singe_paged_mla_attention_combine_f16_any",
    "singe_paged_decode_bf16_d32_g1_b16", "singe_paged_decode_bf16_d32_g2_b16",
    "singe_paged_decode_bf16_d32_g1_any", "singe_paged_decode_bf16_d32_g2_any",
    "singe_paged_decode_combine_bf16_d32", "singe_paged_decode_f16_d32_g1_b16",
    "singe_paged_decode_f16_d32_g2_b16", "singe_paged_decode_f16_d32_g1_any",
    "singe_paged_decode_f16_d32_g2_any", "singe_paged_decode_combine_f16_d32",
    "singe_paged_decode_combine_many_bf16_d32", "singe_paged_decode_combine_many_f16_d32",
    "singe_paged_decode_combine_few_bf16_d32", "singe_paged_decode_combine_few_f16_d32",
    "singe_paged_decode_bf16_d16_g1_b16", "singe_paged_decode_bf16_d16_g2_b16",
    "singe_paged_decode_bf16_d16_g1_any", "singe_paged_decode_bf16_d16_g2_any",
    "singe_paged_decode_combine_bf16_d16", "singe_paged_decode_f16_d16_g1_b16",
    "singe_paged_decode_f16_d16_g2_b16", "singe_paged_decode_f16_d16_g1_any",
    "singe_paged_decode_f16_d16_g2_any", "singe_paged_decode_combine_f16_d16",
    "singe_paged_decode_combine_many_bf16_d16", "singe_paged_decode_combine_many_f16_d16",
    "singe_paged_decode_combine_few_bf16_d16", "singe_paged_decode_combine_few_f16_d16",
    "singe_paged_decode_bf16_d48_g1_b16", "singe_paged_decode_bf16_d48_g2_b16",
    "singe_paged_decode_bf16_d48_g1_any", "singe_paged_decode_bf16_d48_g2_any",
    "singe_paged_decode_combine_bf16_d48", "singe_paged_decode_f16_d48_g1_b16",
    "singe_paged_decode_f16_d48_g2_b16", "singe_paged_decode_f16_d48_g1_any",
    "singe_paged_decode_f16_d48_g2_any", "singe_paged_decode_combine_f16_d48",
    "singe_paged_decode_combine_many_bf16_d48", "singe_paged_decode_combine_many_f16_d48",
    "singe_paged_decode_combine_few_bf16_d48", "singe_paged_decode_combine_few_f16_d48",
    "singe_paged_decode_bf16_d80_g1_b16", "singe_paged_decode_bf16_d80_g2_b16",
    "singe_paged_decode_bf16_d80_g1_any", "singe_paged_decode_bf16_d80_g2_any",
    "singe_paged_decode_combine_bf16_d80", "singe_paged_decode_f16_d80_g1_b16",
    "singe_paged_decode_f16_d80_g2_b16", "singe_paged_decode_f16_d80_g1_any",
    "singe_paged_decode_f16_d80_g2_any", "singe_paged_decode_combine_f16_d80",
    "singe_paged_decode_combine_many_bf16_d80", "singe_paged_decode_combine_many_f16_d80",
    "singe_paged_decode_combine_few_bf16_d80", "singe_paged_decode_combine_few_f16_d80",
    "singe_paged_decode_bf16_d96_g1_b16", "singe_paged_decode_bf16_d96_g2_b16",
    "singe_paged_decode_bf16_d96_g1_any", "singe_paged_decode_bf16_d96_g2_any",
    "singe_paged_decode_combine_bf16_d96", "singe_paged_decode_f16_d96_g1_b16",
    "singe_paged_decode_f16_d96_g2_b16", "singe_paged_decode_f16_d96_g1_any",
    "singe_paged_decode_f16_d96_g2_any", "singe_paged_decode_combine_f16_d96",
    "singe_paged_decode_combine_many_bf16_d96", "singe_paged_decode_combine_many_f16_d96",
    "singe_paged_decode_combine_few_bf16_d96", "singe_paged_decode_combine_few_f16_d96",
    "singe_paged_decode_bf16_d112_g1_b16", "singe_paged_decode_bf16_d112_g2_b16",
    "singe_paged_decode_bf16_d112_g1_any", "singe_paged_decode_bf16_d112_g2_any",
    "singe_paged_decode_combine_bf16_d112", "singe_paged_decode_f16_d112_g1_b16",
    "singe_paged_decode_f16_d112_g2_b16", "singe_paged_decode_f16_d112_g1_any",
    "singe_paged_decode_f16_d112_g2_any", "singe_paged_decode_combine_f16_d112",
    "singe_paged_decode_combine_many_bf16_d112", "singe_paged_decode_combine_many_f16_d112",
    "singe_paged_decode_combine_few_bf16_d112", "singe_paged_decode_combine_few_f16_d112",
    "singe_fmha_prefill_pair_bf16_d128_causal", "singe_fmha_prefill_pair_bf16_d128_full",
    "singe_fmha_prefill_pair_f16_d128_causal", "singe_fmha_prefill_pair_f16_d128_full",
    "singe_fmha_prefill_pair_bf16_d128_causal_ragged", "singe_fmha_prefill_pair_bf16_d128_full_ragged",
    "singe_fmha_prefill_pair_f16_d128_causal_ragged", "singe_fmha_prefill_pair_f16_d128_full_ragged",
    "singe_paged_attention_pair_bf16_d128_i32", "singe_paged_attention_pair_bf16_d128_i64",
    "singe_paged_attention_pair_f16_d128_i32", "singe_paged_attention_pair_f16_d128_i64",
    "singe_rotary_paged_attention_pair_bf16_d128_i32", "singe_rotary_paged_attention_pair_bf16_d128_i64",
    "singe_rotary_paged_attention_pair_f16_d128_i32", "singe_rotary_paged_attention_pair_f16_d128_i64",
    "singe_fmha_prefill_pair_bf16_d64_causal", "singe_fmha_prefill_pair_bf16_d64_full",
    "singe_fmha_prefill_pair_f16_d64_causal", "singe_fmha_prefill_pair_f16_d64_full",
    "singe_fmha_prefill_pair_bf16_d64_causal_ragged", "singe_fmha_prefill_pair_bf16_d64_full_ragged",
    "singe_fmha_prefill_pair_f16_d64_causal_ragged", "singe_fmha_prefill_pair_f16_d64_full_ragged",
    "singe_paged_attention_pair_bf16_d64_i32", "singe_paged_attention_pair_bf16_d64_i64",
    "singe_paged_attention_pair_f16_d64_i32", "singe_paged_attention_pair_f16_d64_i64",
    "singe_rotary_paged_attention_pair_bf16_d64_i32", "singe_rotary_paged_attention_pair_bf16_d64_i64",
    "singe_rotary_paged_attention_pair_f16_d64_i32", "singe_rotary_paged_attention_pair_f16_d64_i64",
    "singe_fmha_prefill_pair_bf16_d96_causal", "singe_fmha_prefill_pair_bf16_d96_full",
    "singe_fmha_prefill_pair_f16_d96_causal", "singe_fmha_prefill_pair_f16_d96_full",
    "singe_fmha_prefill_pair_bf16_d96_causal_ragged", "singe_fmha_prefill_pair_bf16_d96_full_ragged",
    "singe_fmha_prefill_pair_f16_d96_causal_ragged", "singe_fmha_prefill_pair_f16_d96_full_ragged",
    "singe_paged_attention_pair_bf16_d96_i32", "singe_paged_attention_pair_bf16_d96_i64",
    "singe_paged_attention_pair_f16_d96_i32", "singe_paged_attention_pair_f16_d96_i64",
    "singe_rotary_paged_attention_pair_bf16_d96_i32", "singe_rotary_paged_attention_pair_bf16_d96_i64",
    "singe_rotary_paged_attention_pair_f16_d96_i32", "singe_rotary_paged_attention_pair_f16_d96_i64",
    "singe_fmha_prefill_pair_bf16_d112_causal", "singe_fmha_prefill_pair_bf16_d112_full",
    "singe_fmha_prefill_pair_f16_d112_causal", "singe_fmha_prefill_pair_f16_d112_full",
    "singe_fmha_prefill_pair_bf16_d112_causal_ragged", "singe_fmha_prefill_pair_bf16_d112_full_ragged",
    "singe_fmha_prefill_pair_f16_d112_causal_ragged", "singe_fmha_prefill_pair_f16_d112_full_ragged",
    "singe_paged_attention_pair_bf16_d112_i32", "singe_paged_attention_pair_bf16_d112_i64",
    "singe_paged_attention_pair_f16_d112_i32", "singe_paged_attention_pair_f16_d112_i64",
    "singe_rotary_paged_attention_pair_bf16_d112_i32", "singe_rotary_paged_attention_pair_bf16_d112_i64",
    "singe_rotary_paged_attention_pair_f16_d112_i32", "singe_rotary_paged_attention_pair_f16_d112_i64",
    "singe_fmha_prefill_pair_bf16_d80_causal", "singe_fmha_prefill_pair_bf16_d80_full",
    "singe_fmha_prefill_pair_f16_d80_causal", "singe_fmha_prefill_pair_f16_d80_full",
    "singe_fmha_prefill_pair_bf16_d80_causal_ragged", "singe_fmha_prefill_pair_bf16_d80_full_ragged",
    "singe_fmha_prefill_pair_f16_d80_causal_ragged", "singe_fmha_prefill_pair_f16_d80_full_ragged",
    "singe_paged_attention_pair_bf16_d80_i32", "singe_paged_attention_pair_bf16_d80_i64",
    "singe_paged_attention_pair_f16_d80_i32", "singe_paged_attention_pair_f16_d80_i64",
    "singe_rotary_paged_attention_pair_bf16_d80_i32", "singe_rotary_paged_attention_pair_bf16_d80_i64",
    "singe_rotary_paged_attention_pair_f16_d80_i32", "singe_rotary_paged_attention_pair_f16_d80_i64",
    "singe_fmha_prefill_pair_bf16_d48_causal", "singe_fmha_prefill_pair_bf16_d48_full",
    "singe_fmha_prefill_pair_f16_d48_causal", "singe_fmha_prefill_pair_f16_d48_full",
    "singe_fmha_prefill_pair_bf16_d48_causal_ragged", "singe_fmha_prefill_pair_bf16_d48_full_ragged",
    "singe_fmha_prefill_pair_f16_d48_causal_ragged", "singe_fmha_prefill_pair_f16_d48_full_ragged",
    "singe_paged_attention_pair_bf16_d48_i32", "singe_paged_attention_pair_bf16_d48_i64",
    "singe_paged_attention_pair_f16_d48_i32", "singe_paged_attention_pair_f16_d48_i64",
    "singe_rotary_paged_attention_pair_bf16_d48_i32", "singe_rotary_paged_attention_pair_bf16_d48_i64",
    "singe_rotary_paged_attention_pair_f16_d48_i32", "singe_rotary_paged_attention_pair_f16_d48_i64",
    "singe_fmha_prefill_pair_bf16_d32_causal", "singe_fmha_prefill_pair_bf16_d32_full",
    "singe_fmha_prefill_pair_f16_d32_causal", "singe_fmha_prefill_pair_f16_d32_full",
    "singe_fmha_prefill_pair_bf16_d32_causal_ragged", "singe_fmha_prefill_pair_bf16_d32_full_ragged",
    "singe_fmha_prefill_pair_f16_d32_causal_ragged", "singe_fmha_prefill_pair_f16_d32_full_ragged",
    "singe_paged_attention_pair_bf16_d32_i32", "singe_paged_attention_pair_bf16_d32_i64",
    "singe_paged_attention_pair_f16_d32_i32", "singe_paged_attention_pair_f16_d32_i64",
    "singe_rotary_paged_attention_pair_bf16_d32_i32", "singe_rotary_paged_attention_pair_bf16_d32_i64",
    "singe_rotary_paged_attention_pair_f16_d32_i32", "singe_rotary_paged_attention_pair_f16_d32_i64",
    "singe_fmha_prefill_pair_bf16_d16_causal", "singe_fmha_prefill_pair_bf16_d16_full",
    "singe_fmha_prefill_pair_f16_d16_causal", "singe_fmha_prefill_pair_f16_d16_full",
    "singe_fmha_prefill_pair_bf16_d16_causal_ragged", "singe_fmha_prefill_pair_bf16_d16_full_ragged",
    "singe_fmha_prefill_pair_f16_d16_causal_ragged", "singe_fmha_prefill_pair_f16_d16_full_ragged",
    "singe_paged_attention_pair_bf16_d16_i32", "singe_paged_attention_pair_bf16_d16_i64",
    "singe_paged_attention_pair_f16_d16_i32", "singe_paged_attention_pair_f16_d16_i64",
    "singe_rotary_paged_attention_pair_bf16_d16_i32", "singe_rotary_paged_attention_pair_bf16_d16_i64",
    "singe_rotary_paged_attention_pair_f16_d16_i32", "singe_rotary_paged_attention_pair_f16_d16_i64",
};

// The code object is built in parts, one per kernel source (so they compile side by side and a process loads only
// the parts it launches from): singe_attention_gfx950.<part>.hsaco next to the library.  kKernelNames is grouped by
// part; kPartRuns gives the part of each run of consecutive kernels.
const char* const kPartNames[kPartCount] = {
    "paged_decode", "fmha_prefill", "fmha_prefill_f32", "paged_attention", "splitk_reduce", "attention_rows_f32",
    "cache_ops", "latent_attention", "latent_attention_mfma", "general_attention_f32", "general_attention_bf16",
    "general_attention_f16", "mfma_ceiling", "paged_decode_d64", "fmha_prefill_d64", "paged_attention_d64",
    "general_attention_f64", "hbm_stream", "fmha_prefill_d32", "paged_attention_d32", "fmha_prefill_d96", "paged_attention_d96",
    "fmha_prefill_d16", "paged_attention_d16", "fmha_prefill_d48", "paged_attention_d48", "fmha_prefill_d80", "paged_attention_d80",
    "fmha_prefill_d112", "paged_attention_d112", "paged_decode_d32",
    "paged_decode_d16", "paged_decode_d48", "paged_decode_d80", "paged_decode_d96", "paged_decode_d112",
    "fmha_prefill_pair", "paged_attention_pair", "fmha_prefill_pair_d64", "paged_attention_pair_d64",
    "fmha_prefill_pair_d96", "paged_attention_pair_d96",
    "fmha_prefill_pair_d112", "paged_attention_pair_d112",
    "fmha_prefill_pair_d80", "paged_attention_pair_d80",
    "fmha_prefill_pair_d48", "paged_attention_pair_d48",
    "fmha_prefill_pair_d32", "paged_attention_pair_d32",
    "fmha_prefill_pair_d16", "paged_attention_pair_d16",
};

namespace {

struct PartRun {
    int part, kernels;
};
constexpr PartRun kPartRuns[] = {
    {0, 14}, {1, 8}, {2, 4}, {3, 28}, {4, 1}, {5, 28}, {6, 5}, {7, 3}, {8, 4},
    {9, 3}, {10, 3}, {11, 3},  // dense general kernels: f32, bf16, f16
    {9, 3}, {10, 3}, {11, 3},  // paged general kernels
    {12, 2},
    {13, 10}, {14, 8}, {15, 28},  // the head_dim 64 builds
    {1, 2}, {14, 2},              // the dense kernels' merges
    {16, 6},                      // the general kernels on f64
    {17, 1},
    {18, 10}, {19, 28},           // the head_dim 32 builds: dense kernels with their merges, paged kernels
    {20, 10}, {21, 28},           // the head_dim 96 builds
    {22, 10}, {23, 28}, {24, 10}, {25, 28}, {26, 10}, {27, 28}, {28, 10}, {29, 28},  // and those for 16, 48, 80, 112
    {0, 4},                       // the wide decode kernels for bf16 / f16 caches
    {0, 2}, {13, 2},              // the decode merge for rows with many slots, head_dim 128 and 64
    {6, 3},                       // rotate-and-append sixteen bytes at a time
    {0, 2}, {13, 2},              // the decode merge for rows with one or two slots, head_dim 128 and 64
    {6, 2},                       // a decode step in FlashInfer form -> rows for the decode kernels
    {3, 12}, {15, 12}, {19, 12}, {21, 12}, {23, 12}, {25, 12}, {27, 12}, {29, 12},  // the further fused-rotation kernels
    {8, 4},                       // latent attention on the matrix cores at any width it takes
    {30, 14}, {31, 14}, {32, 14}, {33, 14}, {34, 14}, {35, 14},  // the decode kernels and their merges for 32, 16, 48, 80, 96, 112
    {36, 8},                      // the dense prefill with two row tiles a wave (whole key tiles, then a last tile that is not)
    {37, 8},                      // the paged attention op on the same loop, then with a fused query rotation
    {38, 8},                      // the two-tile dense prefill at head_dim 64
    {39, 8},                      // the two-tile paged attention at head_dim 64
    {40, 8}, {41, 8},             // both at head_dim 96
    {42, 8}, {43, 8}, {44, 8}, {45, 8}, {46, 8}, {47, 8}, {48, 8}, {49, 8}, {50, 8}, {51, 8},  // and at 112, 80, 48, 32, 16
};
constexpr int runs_total() {
    int total = 0;
    for (const PartRun& run : kPartRuns) total += run.kernels;
    return total;
}
static_assert(runs_total() == kKernelCount, "every kernel belongs to one part");

}  // namespace

int kernel_part(int kernel) {
    for (const PartRun& run : kPartRuns) {
        if (kernel < run.kernels) return run.part;
        kernel -= run.kernels;
    }
    return 0;
}

namespace {

thread_local SingeHipErrorDetail t_error = {0, "", 0, 0};

constexpr int kMaxDevices = 64;

// A device's kernel handles are published one by one as they are first asked for; a launch reads its handle
// without a lock and takes the mutex only when the handle is not there yet.
struct DeviceModule {
    hipModule_t modules[kPartCount] = {};
    bool loaded[kPartCount] = {};
    std::atomic<hipFunction_t> functions[kKernelCount] = {};
};

std::mutex g_mutex;                               // guards the images, module loading and the publishing of handles
std::vector<unsigned char> g_images[kPartCount];  // copies of the code object's parts
bool g_single_image = false;                      // one code object handed to singe_hip_load holds every kernel (in slot 0)
DeviceModule g_devices[kMaxDevices];

// An archive of parts, as singe_amd/build.py writes it (singe_attention_gfx950.parts): the magic, a version and an
// entry count, then per entry the part's name and where its code object lies in the archive.  All integers little-endian.
constexpr char kArchiveMagic[16] = {'S', 'I', 'N', 'G', 'E', '_', 'H', 'I', 'P', '_', 'P', 'A', 'R', 'T', 'S', '\0'};
constexpr uint32_t kArchiveVersion = 1;
struct ArchiveHeader {
    char magic[16];
    uint32_t version, entries;
};
struct ArchiveEntry {
    char part[48];
    uint64_t offset, bytes;
};
static_assert(sizeof(ArchiveHeader) == 24 && sizeof(ArchiveEntry) == 64, "the archive's layout is fixed");

int part_index(const char* name, size_t limit) {
    for (int part = 0; part < kPartCount; ++part)
        if (std::strlen(kPartNames[part]) < limit && std::strncmp(kPartNames[part], name, limit) == 0) return part;
    return -1;
}

std::string default_image_path(int part) {
    Dl_info info;
    if (dladdr(reinterpret_cast<void*>(&default_image_path), &info) == 0 || info.dli_fname == nullptr) return "";
    std::string path(info.dli_fname);
    size_t slash = path.rfind('/');
    path = slash == std::string::npos ? std::string(".") : path.substr(0, slash);
    return path + "/singe_attention_gfx950." + kPartNames[part] + ".hsaco";
}

bool read_file(const std::string& path, std::vector<unsigned char>& bytes) {
    FILE* file = std::fopen(path.c_str(), "rb");
    if (file == nullptr) return false;
    std::fseek(file, 0, SEEK_END);
    long size = std::ftell(file);
    std::fseek(file, 0, SEEK_SET);
    bool ok = size > 0;
    if (ok) {
        bytes.resize(static_cast<size_t>(size));
        ok = std::fread(bytes.data(), 1, bytes.size(), file) == bytes.size();
    }
    std::fclose(file);
    return ok;
}

// Forgets the handles of one part's kernels (every kernel when part < 0) on every device and unloads the modules.
void drop_modules_locked(int only_part = -1) {
    const HipRuntime* hip = hip_runtime();
    for (DeviceModule& device : g_devices) {
        for (int kernel = 0; kernel < kKernelCount; ++kernel)
            if (only_part < 0 || kernel_part(kernel) == only_part) device.functions[kernel].store(nullptr, std::memory_order_release);
        for (int part = 0; part < kPartCount; ++part) {
            if (only_part >= 0 && part != only_part) continue;
            if (device.loaded[part] && hip != nullptr) hip->hipModuleUnload(device.modules[part]);
            device.modules[part] = nullptr;
            device.loaded[part] = false;
        }
    }
}

// A single code object in place of the parts: everything held so far goes.
void hold_single_image_locked(std::vector<unsigned char>& bytes) {
    drop_modules_locked();
    for (std::vector<unsigned char>& held : g_images) held.clear();
    g_images[0].swap(bytes);
    g_single_image = true;
}

// Takes the parts an archive lists; the archive is checked as a whole before anything held changes.
int32_t hold_archive_locked(const unsigned char* image, size_t bytes) {
    ArchiveHeader header;
    if (bytes < sizeof(header)) return fail(SINGE_HIP_INVALID_LENGTH, "parts archive");
    std::memcpy(&header, image, sizeof(header));
    if (header.version != kArchiveVersion) return fail(SINGE_HIP_INVALID_ARGUMENT, "parts archive version", kArchiveVersion, header.version);
    if (header.entries == 0 || header.entries > static_cast<uint32_t>(kPartCount) ||
        bytes < sizeof(header) + static_cast<size_t>(header.entries) * sizeof(ArchiveEntry))
        return fail(SINGE_HIP_INVALID_LENGTH, "parts archive entries", 1, header.entries);
    std::vector<ArchiveEntry> entries(header.entries);
    std::memcpy(entries.data(), image + sizeof(header), entries.size() * sizeof(ArchiveEntry));
    int parts[kPartCount];
    bool seen[kPartCount] = {};
    for (uint32_t i = 0; i < header.entries; ++i) {
        const ArchiveEntry& entry = entries[i];
        const int part = part_index(entry.part, sizeof(entry.part));
        if (part < 0 || seen[part]) return fail(SINGE_HIP_INVALID_ARGUMENT, "parts archive part name");
        if (entry.bytes == 0 || entry.offset > bytes || entry.bytes > bytes - entry.offset)
            return fail(SINGE_HIP_LENGTH_TOO_SHORT, kPartNames[part], entry.offset + entry.bytes, bytes);
        seen[part] = true;
        parts[i] = part;
    }
    if (g_single_image) {
        drop_modules_locked();
        g_images[0].clear();
        g_single_image = false;
    }
    for (uint32_t i = 0; i < header.entries; ++i) {
        drop_modules_locked(parts[i]);
        g_images[parts[i]].assign(image + entries[i].offset, image + entries[i].offset + entries[i].bytes);
    }
    return 0;
}

int32_t hold_image_locked(std::vector<unsigned char>& bytes) {
    if (bytes.size() >= sizeof(kArchiveMagic) && std::memcmp(bytes.data(), kArchiveMagic, sizeof(kArchiveMagic)) == 0)
        return hold_archive_locked(bytes.data(), bytes.size());
    hold_single_image_locked(bytes);
    return 0;
}

}  // namespace

int32_t fail(int32_t status, const char* name, uint64_t minimum, uint64_t actual) {
    t_error.status = status;
    t_error.name = name;
    t_error.minimum = minimum;
    t_error.actual = actual;
    return status;
}

int32_t fail_hip(hipError_t error, const char* what) { return fail(-static_cast<int32_t>(error), what); }

unsigned compute_units() {
    static std::atomic<unsigned> cached[kMaxDevices] = {};
    const HipRuntime* hip = hip_runtime();
    int device = 0;
    if (hip == nullptr || hip->hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return 256;
    unsigned known = cached[device].load(std::memory_order_relaxed);
    if (known == 0) {
        int count = 0;
        constexpr int kMultiprocessorCount = 63;  // hipDeviceAttributeMultiprocessorCount
        if (hip->hipDeviceGetAttribute(&count, kMultiprocessorCount, device) != hipSuccess || count < 1 || count > 4096)
            count = 256;
        known = static_cast<unsigned>(count);
        cached[device].store(known, std::memory_order_relaxed);  // threads that race here store the same value
    }
    return known;
}

int32_t kernel_function(KernelId kernel, hipFunction_t* function) {
    const HipRuntime* hip = hip_runtime();
    if (hip == nullptr) return fail(SINGE_HIP_RUNTIME_UNAVAILABLE, "libamdhip64");
    int device = 0;
    if (hipError_t error = hip->hipGetDevice(&device)) return fail_hip(error, "hipGetDevice");
    if (device < 0 || device >= kMaxDevices) return fail(SINGE_HIP_UNSUPPORTED_CONFIGURATION, "device index");
    DeviceModule& slot = g_devices[device];
    if (hipFunction_t published = slot.functions[kernel].load(std::memory_order_acquire)) {
        *function = published;
        return 0;
    }
    std::lock_guard<std::mutex> lock(g_mutex);
    const int part = g_single_image ? 0 : kernel_part(kernel);
    if (!slot.loaded[part]) {
        if (g_images[part].empty() && !read_file(default_image_path(part), g_images[part]))
            return fail(SINGE_HIP_KERNEL_NOT_PREPARED, kPartNames[part]);
        if (hipError_t error = hip->hipModuleLoadData(&slot.modules[part], g_images[part].data())) return fail_hip(error, "hipModuleLoadData");
        slot.loaded[part] = true;
    }
    hipFunction_t found = slot.functions[kernel].load(std::memory_order_relaxed);
    if (found == nullptr) {
        if (hipError_t error = hip->hipModuleGetFunction(&found, slot.modules[part], kKernelNames[kernel])) return fail_hip(error, kKernelNames[kernel]);
        slot.functions[kernel].store(found, std::memory_order_release);
    }
    *function = found;
    return 0;
}

}  // namespace singe_hip

namespace {
thread_local SingeHipThreadOptions t_options = {-1, 0, 0, 0, 0, 0};
}  // namespace

namespace singe_hip {
const SingeHipThreadOptions& thread_options() { return t_options; }
}  // namespace singe_hip

using namespace singe_hip;

extern "C" {

int32_t singe_hip_set_thread_options(const SingeHipThreadOptions* options) {
    if (options == nullptr) {
        t_options = SingeHipThreadOptions{-1, 0, 0, 0, 0, 0};
        return 0;
    }
    if (options->relaxed_numerics < -1 || options->relaxed_numerics > 1) return fail(SINGE_HIP_INVALID_ARGUMENT, "relaxed_numerics");
    if (options->paged_attention_splits > 64) return fail(SINGE_HIP_INVALID_ARGUMENT, "paged_attention_splits", 64, options->paged_attention_splits);
    if (options->paged_mla_attention_splits > 64)
        return fail(SINGE_HIP_INVALID_ARGUMENT, "paged_mla_attention_splits", 64, options->paged_mla_attention_splits);
    t_options = *options;
    t_options.has_split_below_blocks = options->has_split_below_blocks != 0;
    return 0;
}

void singe_hip_thread_options(SingeHipThreadOptions* options) {
    if (options != nullptr) *options = t_options;
}


void singe_hip_last_error(SingeHipErrorDetail* detail) {
    if (detail != nullptr) *detail = t_error;
}

const char* singe_hip_status_string(int32_t status) {
    switch (status) {
        case SINGE_HIP_OK: return "ok";
        case SINGE_HIP_INVALID_LENGTH: return "invalid length";
        case SINGE_HIP_LENGTH_TOO_SHORT: return "length too short";
        case SINGE_HIP_LENGTH_EXCEEDS_I32: return "length exceeds i32";
        case SINGE_HIP_SIZE_OVERFLOW: return "size overflow";
        case SINGE_HIP_UNSUPPORTED_WIDTH: return "unsupported width";
        case SINGE_HIP_NULL_POINTER: return "null pointer";
        case SINGE_HIP_KERNEL_NOT_PREPARED: return "kernel specialization has not been prepared";
        case SINGE_HIP_UNSUPPORTED_CONFIGURATION: return "unsupported configuration";
        case SINGE_HIP_INVALID_ARGUMENT: return "invalid argument";
        case SINGE_HIP_RUNTIME_UNAVAILABLE: return "hip runtime unavailable";
        case SINGE_HIP_TUNE_CACHE_MISS: return "tune cache miss";
        case SINGE_HIP_AUTOTUNE_DURING_CAPTURE: return "autotune during stream capture";
        case SINGE_HIP_NO_TUNE_CANDIDATES: return "no tune candidates";
        case SINGE_HIP_NO_SUCCESSFUL_TUNE_CANDIDATES: return "no tune candidate completed";
        case SINGE_HIP_STALE_RECORD: return "stale record";
        default: break;
    }
    if (status < 0) {
        const HipRuntime* hip = hip_runtime();
        if (hip != nullptr) return hip->hipGetErrorString(-status);
        return "hip error";
    }
    return "unknown status";
}

int32_t singe_hip_load(const void* image, size_t bytes) {
    if (image == nullptr) return fail(SINGE_HIP_NULL_POINTER, "image");
    if (bytes == 0) return fail(SINGE_HIP_INVALID_LENGTH, "image");
    std::vector<unsigned char> copy(static_cast<const unsigned char*>(image), static_cast<const unsigned char*>(image) + bytes);
    std::lock_guard<std::mutex> lock(g_mutex);
    return hold_image_locked(copy);
}

int32_t singe_hip_load_part(const char* part, const void* image, size_t bytes) {
    if (part == nullptr) return fail(SINGE_HIP_NULL_POINTER, "part");
    if (image == nullptr) return fail(SINGE_HIP_NULL_POINTER, "image");
    if (bytes == 0) return fail(SINGE_HIP_INVALID_LENGTH, "image");
    const int index = part_index(part, std::strlen(part) + 1);
    if (index < 0) return fail(SINGE_HIP_INVALID_ARGUMENT, "part name");
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_single_image) {  // back from one code object to parts: the other parts are looked for next to the library
        drop_modules_locked();
        g_images[0].clear();
        g_single_image = false;
    }
    drop_modules_locked(index);
    g_images[index].assign(static_cast<const unsigned char*>(image), static_cast<const unsigned char*>(image) + bytes);
    return 0;
}

int32_t singe_hip_load_file(const char* path) {
    if (path == nullptr) return fail(SINGE_HIP_NULL_POINTER, "path");
    std::vector<unsigned char> bytes;
    if (!read_file(path, bytes)) return fail(SINGE_HIP_KERNEL_NOT_PREPARED, "code object file");
    std::lock_guard<std::mutex> lock(g_mutex);
    return hold_image_locked(bytes);
}

void singe_hip_unload(void) {
    std::lock_guard<std::mutex> lock(g_mutex);
    drop_modules_locked();
    for (std::vector<unsigned char>& held : g_images) held.clear();
    g_single_image = false;
}

int32_t singe_hip_kernel(int32_t index, const char** name, const char** part) {
    if (index < 0 || index >= kKernelCount) return fail(SINGE_HIP_INVALID_ARGUMENT, "kernel index");
    if (name != nullptr) *name = kKernelNames[index];
    if (part != nullptr) *part = kPartNames[kernel_part(index)];
    return 0;
}

int32_t singe_hip_prepare(int32_t* count) {
    int32_t found = 0;
    for (int kernel = 0; kernel < kKernelCount; ++kernel) {
        hipFunction_t function = nullptr;
        if (int32_t status = kernel_function(static_cast<KernelId>(kernel), &function)) return status;
        ++found;
    }
    // The fixed scratch of the entry points that allocate nothing: resolve its address on this device now.
    void* scratch = nullptr;
    size_t scratch_bytes = 0;
    if (int status = static_scratch(&scratch, &scratch_bytes)) return fail(status, "hipGetSymbolAddress(static scratch)");
    if (count != nullptr) *count = found;
    return 0;
}

}  // extern "C"
