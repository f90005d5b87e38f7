// Shared device helpers for the gfx950 attention kernels: wave64 cross-lane moves, bf16 packing,
// and the small fixed-size vector types the MFMA builtins take.
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

#define SINGE_DEVICE __device__ __forceinline__

constexpr float kLog2e = 1.4426950408889634074f;
constexpr float kLn2 = 0.6931471805599453094f;

// Status word codes, first writer wins (singe/src/backend/kernel_lowering/mod.rs:40-61).
constexpr unsigned int kStatusIndexOutOfBounds = 1u;

SINGE_DEVICE void report_index_error(unsigned int* status) {
    // The status word is null while a stream is being captured
    // (kernel_plan/source/paged_attention.rs:51-54).
    if (status != nullptr) atomicCAS(status, 0u, kStatusIndexOutOfBounds);
}

template <int N, class F>
SINGE_DEVICE void static_for(F&& f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

SINGE_DEVICE float as_float(int bits) { return __builtin_bit_cast(float, bits); }
SINGE_DEVICE int as_int(float value) { return __builtin_bit_cast(int, value); }

// Every lane reads the value held by lane `(lane & ~(WIDTH - 1)) | SOURCE`: a broadcast inside
// aligned groups of WIDTH lanes (WIDTH a power of two up to 16).  Groups of four use a DPP quad
// permute, which the compiler folds into the consuming VALU instruction; wider groups go through
// the LDS crossbar (ds_swizzle) without touching LDS memory.
template <int WIDTH, int SOURCE>
SINGE_DEVICE float group_broadcast(float value) {
    static_assert(WIDTH == 1 || WIDTH == 2 || WIDTH == 4 || WIDTH == 8 || WIDTH == 16, "group width");
    if constexpr (WIDTH <= 4) {
        // Lanes of a quad hold heads 0..WIDTH-1 repeated, so quad position SOURCE has head SOURCE.
        constexpr int sel = SOURCE & 3;
        return as_float(__builtin_amdgcn_update_dpp(0, as_int(value), sel * 0x55, 0xF, 0xF, false));
    } else {
        constexpr int and_mask = 0x1F & ~(WIDTH - 1);
        return as_float(__builtin_amdgcn_ds_swizzle(as_int(value), and_mask | (SOURCE << 5)));
    }
}

SINGE_DEVICE float wave_xor(float value, int mask) { return __shfl_xor(value, mask, 64); }

// bf16 <-> f32.  Widening is a shift (singe-codegen/src/emit/cuda_c/prelude.rs:91-93); narrowing
// rounds to nearest even and quiets NaN (prelude.rs:94-106).
SINGE_DEVICE float bf16_lo(unsigned int packed) { return __builtin_bit_cast(float, packed << 16); }
SINGE_DEVICE float bf16_hi(unsigned int packed) { return __builtin_bit_cast(float, packed & 0xffff0000u); }

SINGE_DEVICE unsigned short f32_to_bf16_bits(float value) {
    unsigned int bits = __builtin_bit_cast(unsigned int, value);
    if ((bits & 0x7fffffffu) > 0x7f800000u) return static_cast<unsigned short>((bits >> 16) | 0x0040u);
    return static_cast<unsigned short>((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
}

SINGE_DEVICE unsigned int pack_bf16x2(float lo, float hi) {
    return static_cast<unsigned int>(f32_to_bf16_bits(lo)) | (static_cast<unsigned int>(f32_to_bf16_bits(hi)) << 16);
}

// 16-byte load of data that is read once: the non-temporal hint keeps it from displacing reusable
// lines in the caches on its way through, which measurably raises streaming read bandwidth.
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
SINGE_DEVICE uint4 stream_load_16(const void* address) {
    const u32x4_t bits = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(address));
    return make_uint4(bits.x, bits.y, bits.z, bits.w);
}

typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
SINGE_DEVICE uint2 stream_load_8(const void* address) {
    const u32x2_t bits = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(address));
    return make_uint2(bits.x, bits.y);
}

// v_permlane16_swap / v_permlane32_swap of a value with a copy of itself: `kept` keeps its even rows
// (its low half for 32) and takes the neighbour's, `taken` the other way round, so kept (op) taken
// combines a lane with its partner 16 (32) lanes away.  Written as inline assembly because the
// compiler's builtin returns the first result twice; the s_nop covers the VALU-write hazard the
// compiler would otherwise pad.
template <int ROWS>
SINGE_DEVICE void swap_with_self(float value, float& kept, float& taken) {
    kept = value;
    taken = value;
    if constexpr (ROWS == 16)
        asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(kept), "+v"(taken));
    else
        asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(kept), "+v"(taken));
}

// max / sum over the four 16-lane groups of a wave: lanes l, l^16, l^32, l^48 end up equal.
SINGE_DEVICE float across_groups_max(float value) {
    float a, b;
    swap_with_self<16>(value, a, b);
    swap_with_self<32>(fmaxf(a, b), a, b);
    return fmaxf(a, b);
}

SINGE_DEVICE float across_groups_sum(float value) {
    float a, b;
    swap_with_self<16>(value, a, b);
    swap_with_self<32>(a + b, a, b);
    return a + b;
}

SINGE_DEVICE float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
SINGE_DEVICE float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
// tanh(x) = 1 - 2 / (e^(2x) + 1): one exponential and one reciprocal; exact at both infinities, absolute error
// about 1e-7 near zero (the subtraction), which a capped score multiplies by the cap.
SINGE_DEVICE float fast_tanh(float x) { return 1.0f - 2.0f * __builtin_amdgcn_rcpf(fast_exp2(x * (2.0f * kLog2e)) + 1.0f); }
