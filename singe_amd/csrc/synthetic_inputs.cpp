// Seeded inputs for benchmarks, made on the host so that any caller, in any language, can make the same tensors from
// the same seed: a measurement aid with no attention in it.  The stream is the splitmix64 sequence the reference uses
// where it wants "one seed, one search everywhere" (singe/src/backend/cuda/tuning/plan.rs:527-543), read as a counter:
// word i of a stream is the mix of seed + (i + 1) * 0x9E3779B97F4A7C15, so any range of a tensor can be made on its own
// and by as many threads as there are.
//
//   normal values   word i gives elements 2 i and 2 i + 1 by Box-Muller on two 24-bit uniforms:
//                   u1 = ((word >> 40) + 1) / 2^24 in (0, 1], u2 = ((word >> 16) & 0xFFFFFF) / 2^24 in [0, 1),
//                   r = sqrt(-2 ln u1), elements r cos(2 pi u2) and r sin(2 pi u2), computed in double and rounded to
//                   float; narrower storage types are rounded from that float.
//   integers        word i gives low + ((word >> 32) * span >> 32) for a value in [low, low + span).
//   a tensor's seed base seed ^ FNV-1a (64 bit) of the tensor's name.
#include <math.h>

#include <cmath>
#include <cstdint>
#include <thread>
#include <vector>

#include "singe_hip_attention.h"

namespace {

inline uint64_t word_at(uint64_t seed, uint64_t index) {
    uint64_t z = seed + (index + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

inline void normal_pair(uint64_t word, float& first, float& second) {
    constexpr double kTwoPi = 6.283185307179586476925286766559;
    constexpr double kUnit = 1.0 / 16777216.0;  // 2^-24
    const double u1 = static_cast<double>((word >> 40) + 1) * kUnit;
    const double u2 = static_cast<double>((word >> 16) & 0xFFFFFFull) * kUnit;
    const double radius = std::sqrt(-2.0 * std::log(u1));
    double sine, cosine;
    sincos(kTwoPi * u2, &sine, &cosine);  // glibc: the values sin() and cos() give, in one pass
    first = static_cast<float>(radius * cosine);
    second = static_cast<float>(radius * sine);
}

void fill_normal(uint64_t seed, uint64_t first_element, float* out, size_t count) {
    size_t done = 0;
    uint64_t element = first_element;
    if (count > 0 && (element & 1)) {  // the second half of a pair
        float a, b;
        normal_pair(word_at(seed, element / 2), a, b);
        out[done++] = b;
        ++element;
    }
    for (; done + 2 <= count; done += 2, element += 2) normal_pair(word_at(seed, element / 2), out[done], out[done + 1]);
    if (done < count) {
        float a, b;
        normal_pair(word_at(seed, element / 2), a, b);
        out[done] = a;
    }
}

}  // namespace

extern "C" uint64_t singe_hip_synthetic_seed(uint64_t base_seed, const char* tensor_name) {
    uint64_t hash = 0xCBF29CE484222325ull;
    if (tensor_name != nullptr)
        for (const unsigned char* p = reinterpret_cast<const unsigned char*>(tensor_name); *p != 0; ++p) {
            hash ^= *p;
            hash *= 0x100000001B3ull;
        }
    return base_seed ^ hash;
}

extern "C" uint64_t singe_hip_synthetic_word(uint64_t seed, uint64_t index) { return word_at(seed, index); }

extern "C" void singe_hip_synthetic_normal_f32(uint64_t seed, uint64_t first_element, float* out, size_t count, uint32_t threads) {
    if (out == nullptr || count == 0) return;
    const size_t workers = threads < 1 ? 1 : threads;
    // Whole pairs per worker, so no two workers compute the same word.
    size_t share = (count + workers - 1) / workers;
    share += share & 1;
    if (workers == 1 || count < 4096) {
        fill_normal(seed, first_element, out, count);
        return;
    }
    // A share starts on an even element of the stream when first_element is even; when it is odd, the first worker
    // takes one element more so that the others still do.
    const size_t lead = first_element & 1;
    std::vector<std::thread> pool;
    size_t begin = 0;
    for (size_t w = 0; w < workers && begin < count; ++w) {
        size_t length = share + (w == 0 ? lead : 0);
        if (length > count - begin) length = count - begin;
        pool.emplace_back(fill_normal, seed, first_element + begin, out + begin, length);
        begin += length;
    }
    for (std::thread& worker : pool) worker.join();
}

extern "C" void singe_hip_synthetic_integers(uint64_t seed, uint64_t first_index, int64_t low, uint64_t span, int64_t* out, size_t count) {
    if (out == nullptr) return;
    for (size_t i = 0; i < count; ++i) {
        const uint64_t high = word_at(seed, first_index + i) >> 32;
        out[i] = low + static_cast<int64_t>((high * (span & 0xFFFFFFFFull)) >> 32);
    }
}

// A permutation of 0 .. count - 1 by Fisher-Yates from the back: step k (k = 0 for the last position) swaps position
// i = count - 1 - k with a position drawn from [0, i] by word k of the stream.
extern "C" void singe_hip_synthetic_permutation(uint64_t seed, int64_t* out, size_t count) {
    if (out == nullptr) return;
    for (size_t i = 0; i < count; ++i) out[i] = static_cast<int64_t>(i);
    for (size_t k = 0; k + 1 < count; ++k) {
        const size_t i = count - 1 - k;
        const uint64_t high = word_at(seed, k) >> 32;
        const size_t j = static_cast<size_t>((high * static_cast<uint64_t>(i + 1)) >> 32);
        const int64_t held = out[i];
        out[i] = out[j];
        out[j] = held;
    }
}
