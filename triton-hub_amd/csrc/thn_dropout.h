// Dropout over a contiguous tensor: y[i] = rand(seed, i) < p ? 0 : x[i] / (1 - p), with rand the uniform float32 that
// Triton's tl.rand(seed, i) returns, so that a seed gives the mask it gives in the reference
// (TritonHub/Layers/dropout.py:12-23; the backward, :56-67, is the same function of the upstream gradient).
//
// tl.rand: the first output word of Philox-4x32 with 10 rounds on counter (i mod 2^32, i div 2^32, 0, 0) and key
// (seed mod 2^32, seed div 2^32), read as int32 v, folded to v < 0 ? -v - 1 : v, converted to float32 and multiplied
// by 4.6566127342e-10.  Every element needs a Philox block of its own (37 32x32-bit multiplications, quarter-rate
// instructions): the kernel is bound by integer arithmetic, not by memory.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#include "thn_device.h"

namespace thn {

struct DropoutArgs {
    const char* x;
    char* out;
    int64_t total_vecs;    // whole 16-byte vectors
    int64_t total_elems;
    int64_t first_offset;  // offset of element 0 (0 for a whole tensor)
    float p;
    uint32_t key_lo, key_hi;
};

__device__ __forceinline__ uint32_t philox_first_word(uint32_t c0, uint32_t c1, uint32_t k0, uint32_t k1) {
    uint32_t c2 = 0u, c3 = 0u;
#pragma unroll
    for (int round = 0; round < 10; ++round) {
        const uint64_t pa = static_cast<uint64_t>(0xD2511F53u) * c0;
        const uint64_t pb = static_cast<uint64_t>(0xCD9E8D57u) * c2;
        const uint32_t n0 = static_cast<uint32_t>(pb >> 32) ^ c1 ^ k0;
        const uint32_t n2 = static_cast<uint32_t>(pa >> 32) ^ c3 ^ k1;
        c1 = static_cast<uint32_t>(pb);
        c3 = static_cast<uint32_t>(pa);
        c0 = n0;
        c2 = n2;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return c0;
}

__device__ __forceinline__ float uniform_from_word(uint32_t w) {
    int32_t v = static_cast<int32_t>(w);
    v ^= v >> 31;                                   // v < 0 ? -v - 1 : v
    return static_cast<float>(v) * 4.6566127342e-10f;
}

__device__ __forceinline__ float dropout_rand(int64_t offset, uint32_t k0, uint32_t k1) {
    const uint64_t o = static_cast<uint64_t>(offset);
    return uniform_from_word(philox_first_word(static_cast<uint32_t>(o), static_cast<uint32_t>(o >> 32), k0, k1));
}

// x / keep for a float32 divisor shared by all elements, correctly rounded like the division it replaces: the
// float64 product of x and the float64 reciprocal of keep is within 2^-52 of the exact quotient, and a quotient of two
// float32 values is never closer than 2^-49 (relative) to a point where float32 rounding changes direction, so
// rounding the product to float32 gives the same value as rounding the quotient itself (infinities, NaN, signed
// zeros, overflow and subnormal results included).  3 instructions per element instead of the 11 of a division.
struct KeepDivisor {
    double rk64;     // float32 storage types
    double keep64;   // float64 storage
};
__device__ __forceinline__ KeepDivisor make_keep_divisor(float keep) {
    return KeepDivisor{1.0 / static_cast<double>(keep), static_cast<double>(keep)};
}
__device__ __forceinline__ float keep_div(float x, const KeepDivisor& d) {
    return static_cast<float>(static_cast<double>(x) * d.rk64);
}
__device__ __forceinline__ double keep_div(double x, const KeepDivisor& d) { return x / d.keep64; }

constexpr int kDropoutBlock = 256;

template <typename T>
__global__ void __launch_bounds__(kDropoutBlock) dropout_flat_kernel(const DropoutArgs a) {
    using C = typename std::conditional<T::kBytes == 8, double, float>::type;
    constexpr int VEC = T::VEC;
    const KeepDivisor keep = make_keep_divisor(1.0f - a.p);        // float32 difference, as the reference's `1 - p`
    const int64_t step = static_cast<int64_t>(gridDim.x) * kDropoutBlock;
    for (int64_t v = static_cast<int64_t>(blockIdx.x) * kDropoutBlock + threadIdx.x; v < a.total_vecs; v += step) {
        const u32x4 raw = ld128u(a.x + v * 16);
        C xf[VEC], of[VEC];
        unpack_as<T>(raw, xf);
        const int64_t e0 = a.first_offset + v * VEC;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float r = dropout_rand(e0 + e, a.key_lo, a.key_hi);
            of[e] = r < a.p ? C(0) : keep_div(xf[e], keep);
        }
        st128u(a.out + v * 16, pack_as<T, C>(of));
    }
    // the tail that does not fill a vector
    const int64_t i = a.total_vecs * VEC + threadIdx.x;
    if (blockIdx.x == 0 && i < a.total_elems) {
        const C x = load_elem<T, C>(a.x, i);
        const float r = dropout_rand(a.first_offset + i, a.key_lo, a.key_hi);
        store_elem<T, C>(a.out, i, r < a.p ? C(0) : keep_div(x, keep));
    }
}

int launch_dropout(int dtype, const DropoutArgs& a, int grid, hipStream_t st);

}  // namespace thn
