// The choices the attention kernels leave open, as the reference states them
// (singe/src/backend/cuda/kernel_plan/source/parameters.rs:21-57, 221-230; candidates: attention.rs:113-160), mapped
// to what the gfx950 kernels can vary, and the key a tuning record is stored under.
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include "module.h"
#include "singe_hip_attention.h"
#include "thread_options.h"
#include "validate.h"

using namespace singe_hip;

namespace {

constexpr size_t kWarps = 4, kKeyTile = 64;
// Key splits: a row tile's keys go to at most kMaxShares workgroups (the merge kernels keep a share's weight per
// lane), none with fewer than kShareTiles key tiles where the keys allow it (below that a workgroup's start, its
// paging loads and its partial rows, outweighs what it folds).
constexpr size_t kMaxShares = 64, kShareTiles = 8;
constexpr uint32_t kBuiltMinBlocks = 2;

// 0 = the default (twice the compute units); otherwise split_below_blocks + 1 of the installed parameters.
std::atomic<uint64_t> g_split_below_plus_one{0};
std::atomic<uint64_t> g_stages{1};
std::atomic<uint32_t> g_min_blocks{0};  // 0 = none

size_t default_split_below() { return 2 * static_cast<size_t>(compute_units()); }

bool same(const SingeAttentionParameters& a, const SingeAttentionParameters& b) {
    return a.warps == b.warps && a.key_tile == b.key_tile && a.stages == b.stages && a.split_below_blocks == b.split_below_blocks &&
           (a.has_min_blocks != 0) == (b.has_min_blocks != 0) && (a.has_min_blocks == 0 || a.min_blocks == b.min_blocks);
}

size_t list_candidates(SingeAttentionParameters* out, size_t capacity) {
    SingeAttentionParameters base;
    singe_hip_attention_parameters_default(&base);
    SingeAttentionParameters all[16];
    size_t count = 0;
    auto push = [&](const SingeAttentionParameters& candidate) {
        for (size_t i = 0; i < count; ++i)
            if (same(all[i], candidate)) return;
        all[count++] = candidate;
    };
    push(base);
    // The thresholds the reference tries (64, 0, 256: attention.rs:122), and this device's own: one, two and four
    // workgroups per compute unit.
    const size_t units = compute_units();
    for (size_t below : {static_cast<size_t>(64), static_cast<size_t>(0), static_cast<size_t>(256), units, 2 * units, 4 * units}) {
        SingeAttentionParameters candidate = base;
        candidate.split_below_blocks = below;
        push(candidate);
    }
    SingeAttentionParameters staged = base;
    staged.stages = 2;
    push(staged);
    SingeAttentionParameters bound = base;
    bound.has_min_blocks = 1;
    bound.min_blocks = kBuiltMinBlocks;
    push(bound);
    for (size_t i = 0; i < count && i < capacity; ++i) out[i] = all[i];
    return count;
}

// Rust's Debug of an f32: the shortest digits that read back to the same value, with a fraction always shown.
std::string debug_f32(float value) {
    if (std::isnan(value)) return "NaN";
    if (std::isinf(value)) return value > 0 ? "inf" : "-inf";
    char text[64];
    for (int digits = 1; digits <= 9; ++digits) {
        std::snprintf(text, sizeof text, "%.*e", digits - 1, static_cast<double>(value));
        if (std::strtof(text, nullptr) == value) break;
    }
    // text is d.ddde[+-]xx: split it.
    std::string mantissa(text);
    const size_t e = mantissa.find('e');
    const int exponent = std::atoi(mantissa.c_str() + e + 1);
    mantissa.resize(e);
    const bool negative = mantissa[0] == '-';
    std::string digits;
    for (char c : mantissa)
        if (c >= '0' && c <= '9') digits.push_back(c);
    while (digits.size() > 1 && digits.back() == '0') digits.pop_back();
    std::string out = negative ? "-" : "";
    if (value == 0.0f) return out + "0.0";
    if (exponent >= 16 || exponent < -5) {  // scientific, as Rust prints beyond these magnitudes
        out += digits.substr(0, 1);
        if (digits.size() > 1) out += "." + digits.substr(1);
        return out + "e" + std::to_string(exponent);
    }
    if (exponent < 0) return out + "0." + std::string(static_cast<size_t>(-exponent - 1), '0') + digits;
    if (digits.size() <= static_cast<size_t>(exponent) + 1)
        return out + digits + std::string(static_cast<size_t>(exponent) + 1 - digits.size(), '0') + ".0";
    return out + digits.substr(0, static_cast<size_t>(exponent) + 1) + "." + digits.substr(static_cast<size_t>(exponent) + 1);
}

const char* type_name(int32_t data_type) {
    return data_type == SINGE_HIP_BF16 ? "Bf16" : data_type == SINGE_HIP_F16 ? "F16" : data_type == SINGE_HIP_F64 ? "F64" : "F32";
}

// " <type>[d0, d1, ...][s0, s1, ...]+0" of a contiguous operand; an axis of one element, and every axis of an empty
// operand, addresses with stride 0 (singe/src/layout/mod.rs:32-40).
void operand(std::string& key, const char* type, std::initializer_list<int64_t> dims) {
    int64_t sizes[8], strides[8];
    size_t rank = 0;
    bool empty = false;
    for (int64_t dim : dims) {
        sizes[rank++] = dim;
        empty = empty || dim == 0;
    }
    int64_t stride = 1;
    for (size_t axis = rank; axis-- > 0;) {
        strides[axis] = empty || sizes[axis] == 1 ? 0 : stride;
        stride *= sizes[axis];
    }
    key += " ";
    key += type;
    std::string shape = "[", steps = "[";
    for (size_t axis = 0; axis < rank; ++axis) {
        shape += (axis ? ", " : "") + std::to_string(sizes[axis]);
        steps += (axis ? ", " : "") + std::to_string(strides[axis]);
    }
    key += shape + "]" + steps + "]+0";
}

std::string attributes(bool has_scale, float scale, bool causal, bool has_window, int64_t window, bool has_softcap, float softcap,
                       bool masked, bool sinks, bool key_lengths) {
    auto flag = [](bool value) { return value ? "true" : "false"; };
    std::string text = "ScaledDotProductAttentionAttributes { scale: ";
    text += has_scale ? "Some(" + debug_f32(scale) + ")" : "None";
    text += std::string(", causal: ") + flag(causal) + ", window: ";
    text += has_window ? "Some(" + std::to_string(window) + ")" : "None";
    text += ", softcap: ";
    text += has_softcap ? "Some(" + debug_f32(softcap) + ")" : "None";
    text += std::string(", masked: ") + flag(masked) + ", sinks: " + flag(sinks) + ", key_lengths: " + flag(key_lengths) + " }";
    return text;
}

std::string key_head(const char* label, const std::string& attribute_text) {
    std::string key = "kernel|";
    key += label;
    key += singe_hip_relaxed_numerics() ? "|NumericalPolicy { precision: Relaxed, determinism: Allow }|"
                                        : "|NumericalPolicy { precision: Full, determinism: Allow }|";
    return key + attribute_text;
}

size_t hand_over(const std::string& key, char* buffer, size_t capacity) {
    if (buffer != nullptr && capacity > 0) {
        const size_t n = key.size() < capacity - 1 ? key.size() : capacity - 1;
        std::memcpy(buffer, key.data(), n);
        buffer[n] = '\0';
    }
    return key.size();
}

}  // namespace

namespace singe_hip {

uint32_t attention_key_splits(uint64_t workgroups, uint64_t keys) {
    const SingeHipThreadOptions& own = thread_options();
    const uint64_t installed = g_split_below_plus_one.load(std::memory_order_relaxed);
    const uint64_t below = own.has_split_below_blocks ? own.split_below_blocks : installed == 0 ? default_split_below() : installed - 1;
    if (below == 0 || workgroups == 0 || workgroups >= below || keys <= kShareTiles * kKeyTile) return 1;
    uint64_t wanted = (2 * below + workgroups - 1) / workgroups;
    const uint64_t chunks = (keys + kShareTiles * kKeyTile - 1) / (kShareTiles * kKeyTile);
    wanted = wanted < chunks ? wanted : chunks;
    return static_cast<uint32_t>(wanted > kMaxShares ? kMaxShares : wanted < 1 ? 1 : wanted);
}

}  // namespace singe_hip

extern "C" {

void singe_hip_attention_parameters_default(SingeAttentionParameters* parameters) {
    if (parameters == nullptr) return;
    parameters->warps = kWarps;
    parameters->key_tile = kKeyTile;
    parameters->stages = 1;
    parameters->split_below_blocks = default_split_below();
    parameters->has_min_blocks = 0;
    parameters->min_blocks = 0;
}

int32_t singe_hip_attention_candidates(SingeAttentionParameters* candidates, size_t capacity, size_t* count) {
    if (count == nullptr) return fail(SINGE_HIP_NULL_POINTER, "count");
    if (candidates == nullptr && capacity > 0) return fail(SINGE_HIP_NULL_POINTER, "candidates");
    *count = list_candidates(candidates, capacity);
    return 0;
}

int32_t singe_hip_set_attention_parameters(const SingeAttentionParameters* parameters) {
    if (parameters == nullptr) {
        g_split_below_plus_one.store(0, std::memory_order_relaxed);
        g_stages.store(1, std::memory_order_relaxed);
        g_min_blocks.store(0, std::memory_order_relaxed);
        return 0;
    }
    SingeAttentionParameters taken[16];
    const size_t count = list_candidates(taken, 16);
    for (size_t i = 0; i < count; ++i) {
        if (!same(taken[i], *parameters)) continue;
        g_split_below_plus_one.store(static_cast<uint64_t>(parameters->split_below_blocks) + 1, std::memory_order_relaxed);
        g_stages.store(parameters->stages, std::memory_order_relaxed);
        g_min_blocks.store(parameters->has_min_blocks ? parameters->min_blocks : 0, std::memory_order_relaxed);
        return 0;
    }
    return fail(SINGE_HIP_STALE_RECORD, "attention parameters");
}

void singe_hip_attention_parameters(SingeAttentionParameters* parameters) {
    if (parameters == nullptr) return;
    singe_hip_attention_parameters_default(parameters);
    const uint64_t installed = g_split_below_plus_one.load(std::memory_order_relaxed);
    if (installed != 0) parameters->split_below_blocks = static_cast<size_t>(installed - 1);
    if (thread_options().has_split_below_blocks) parameters->split_below_blocks = static_cast<size_t>(thread_options().split_below_blocks);
    parameters->stages = static_cast<size_t>(g_stages.load(std::memory_order_relaxed));
    const uint32_t bound = g_min_blocks.load(std::memory_order_relaxed);
    parameters->has_min_blocks = bound != 0;
    parameters->min_blocks = bound;
}

size_t singe_hip_paged_attention_parameter_key(const SingePagedAttentionProblem* problem, int32_t data_type, char* buffer,
                                               size_t capacity) {
    if (problem == nullptr) return 0;
    const SingePagedAttentionProblem& p = *problem;
    std::string key = key_head("paged_attention", attributes(p.has_scale != 0, p.scale, p.causal != 0, p.has_window != 0, p.window,
                                                             p.has_softcap != 0, p.softcap, false, false, false));
    const char* element = type_name(data_type);
    const char* index = p.index_type == SINGE_HIP_INDEX_I64 ? "I64" : "I32";
    operand(key, element, {p.tokens, p.heads, p.head_dim});
    operand(key, element, {p.cache_pages, p.page_size, p.kv_heads, p.head_dim});
    operand(key, element, {p.cache_pages, p.page_size, p.kv_heads, p.head_dim});
    operand(key, index, {p.sequences + 1});
    operand(key, index, {p.sequences + 1});
    operand(key, index, {p.page_table});
    operand(key, index, {p.sequences});
    return hand_over(key, buffer, capacity);
}

size_t singe_hip_attention_parameter_key(const SingeAttentionProblem* problem, int32_t masked, int32_t sinks, int32_t key_lengths,
                                         char* buffer, size_t capacity) {
    if (problem == nullptr) return 0;
    const SingeAttentionProblem& p = *problem;
    std::string key = key_head("attention", attributes(p.has_scale != 0, p.scale, p.causal != 0, p.has_window != 0, p.window,
                                                       p.has_softcap != 0, p.softcap, masked != 0, sinks != 0, key_lengths != 0));
    const char* element = type_name(p.data_type);
    operand(key, element, {p.batch, p.heads, p.query_len, p.head_dim});
    operand(key, element, {p.batch, p.kv_heads, p.key_len, p.head_dim});
    operand(key, element, {p.batch, p.kv_heads, p.key_len, p.value_dim});
    // A mask, sinks and key lengths are operands of the key too (attention.rs:241-247): the mask with the axes it
    // broadcasts over as single elements, sinks [heads], key lengths [batch] i32.
    if (masked)
        operand(key, element, {p.mask_strides[0] ? p.batch : 1, p.mask_strides[1] ? p.heads : 1, p.mask_strides[2] ? p.query_len : 1,
                               p.mask_strides[3] ? p.key_len : 1});
    if (sinks) operand(key, element, {p.heads});
    if (key_lengths) operand(key, "I32", {p.batch});
    return hand_over(key, buffer, capacity);
}

}  // extern "C"
