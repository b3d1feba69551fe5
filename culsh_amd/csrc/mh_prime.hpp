// Arithmetic of the MinHash family (a * x + b) mod p for the two primes the library knows.
//
// The reference hashes modulo 4294967291 = 2^32 - 5 (minhash/hash.cuh:17), which is the default and the
// form every parity statement refers to.  2147483647 = 2^31 - 1 is the other common choice for 32-bit
// MinHash; a context can be switched to it (culsh_ctx_set_minhash_prime).  Both have the form 2^k - c, so
// a 64-bit value folds as hi * 2^k + lo = c * hi + lo (mod p); two folds and one subtraction reduce any
// a * x + b with a, x, b < 2^32.
#pragma once
#include <cstdint>

#include <hip/hip_runtime.h>

namespace culsh_amd {

constexpr int MH_PRIME_2_32_M5 = 0;  // 4294967291, the reference's
constexpr int MH_PRIME_2_31_M1 = 1;  // 2147483647

constexpr uint32_t mh_prime_value(int kind) { return kind == MH_PRIME_2_31_M1 ? 2147483647u : 4294967291u; }

template <int KIND>
struct MhPrime;

template <>
struct MhPrime<MH_PRIME_2_32_M5> {
    static constexpr uint32_t P = 4294967291u;
    // any a, x, b < 2^32
    static __device__ __forceinline__ uint32_t hash(uint32_t a, uint32_t x, uint32_t b) {
        const uint64_t v = static_cast<uint64_t>(a) * x + b;           // < 2^64
        const uint64_t v1 = 5ull * (v >> 32) + (v & 0xFFFFFFFFull);    // < 6 * 2^32
        const uint64_t v2 = 5ull * (v1 >> 32) + (v1 & 0xFFFFFFFFull);  // < 2^32 + 25
        return static_cast<uint32_t>(v2 >= P ? v2 - P : v2);
    }
    // x < 2^25: a * x + b < 2^57, so the first fold leaves less than 2^32 + 5 * 2^25 and a second fold
    // could only add 5 once: it is merged with the final subtraction.
    static __device__ __forceinline__ uint32_t hash_small(uint32_t a, uint32_t x, uint32_t b) {
        const uint64_t v = static_cast<uint64_t>(a) * x + b;
        const uint64_t v1 = 5ull * (v >> 32) + (v & 0xFFFFFFFFull);
        const uint32_t lo = static_cast<uint32_t>(v1);
        return v1 >= P ? lo + 5u : lo;
    }
};

template <>
struct MhPrime<MH_PRIME_2_31_M1> {
    static constexpr uint32_t P = 2147483647u;
    static __device__ __forceinline__ uint32_t hash(uint32_t a, uint32_t x, uint32_t b) {
        const uint64_t v = static_cast<uint64_t>(a) * x + b;           // < 2^64
        const uint64_t v1 = (v >> 31) + (v & 0x7FFFFFFFull);           // < 2^33 + 2^31
        const uint32_t v2 = static_cast<uint32_t>(v1 >> 31) + (static_cast<uint32_t>(v1) & 0x7FFFFFFFu);  // < 2^31 + 5
        return v2 >= P ? v2 - P : v2;
    }
    static __device__ __forceinline__ uint32_t hash_small(uint32_t a, uint32_t x, uint32_t b) { return hash(a, x, b); }
};

}  // namespace culsh_amd
