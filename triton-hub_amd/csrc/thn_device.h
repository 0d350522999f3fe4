// Device-side building blocks shared by the forward and backward kernels: 128-bit row I/O for the four
// storage types, float32 <-> storage conversion, wave64 DPP reductions and the LDS cross-wave reduction.
// gfx950 (CDNA4) only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace thn {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

enum : int { kF32 = 0, kF16 = 1, kBF16 = 2, kF64 = 3 };

// Bit casts take their operand BY VALUE in a scalar: applying __builtin_bit_cast directly to an element
// of an ext_vector (v[i]) reads element 0 whatever i is with this compiler.
__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

#ifndef THN_NT_LOAD
#define THN_NT_LOAD 1
#endif
#ifndef THN_NT_STORE
#define THN_NT_STORE 1
#endif

__device__ __forceinline__ u32x4 ld128(const void* p) {
#if THN_NT_LOAD
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
#else
    return *reinterpret_cast<const u32x4*>(p);
#endif
}
__device__ __forceinline__ void st128(void* p, u32x4 v) {
#if THN_NT_STORE
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
#else
    *reinterpret_cast<u32x4*>(p) = v;
#endif
}

// The same load without the non-temporal hint: the lines are allocated in the L2 and in the 256 MB memory-side
// cache behind it.  The norm forward reads x this way under the "keep" cache policy (the KEEPX instances of
// norm_fwd_kernel): x is the one tensor of the step that is read again -- by the backward, which needs x to rebuild
// xhat -- and a backward that follows its forward closely then finds a part of x in that cache.  Measured on MI355X,
// bfloat16 16384 x 4096, forward + backward on the same batch, four batches in rotation: RMSNorm 113.8 -> 105.4 us,
// LayerNorm 117.0 -> 109.9 us; 32768 x 8192 (x is twice the cache) 450 -> 434 us.  The forward on its own is 2-3 %
// slower for it (44.1 -> 44.9 us): the streaming loads leave the L2 alone, which is why a forward that no backward
// follows takes the streaming instances.  Everything that is touched once (y, dy, dx; x in the backward) stays
// non-temporal; keeping any of those as well made the step slower again.
__device__ __forceinline__ u32x4 ld128_keep(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ void st128_keep(void* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }

// s_waitcnt vmcnt(0): every vector-memory operation this wave has issued is complete.  Placed once in front
// of the row loop so that the loop is entered with nothing outstanding: the compiler derives the loop's own
// waits from the number of operations in flight on every path into the loop header, and an entry path with
// the prologue's loads still pending makes it wait for more than the loop body needs on every trip.
// The wait alone does not hold the prologue's loads in front of it (the compiler is free to issue them after
// it, and did in the instances whose rows stay inside one wave: their loops then waited for all of the previous
// row's stores at the top of every trip).  So the values the prologue loaded are passed in and pinned: an empty
// asm statement takes each as an operand, which makes the compiler have it in registers at this point.
__device__ __forceinline__ void pin_loaded(float& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin_loaded(u32x4& v) { asm volatile("" : "+v"(v)); }
// The raw bits of a scalar load, held where the statement stands: as pin_loaded, and the compiler may not move it
// across a load or store either (so it stays behind the row's stores when it is written behind them).
__device__ __forceinline__ void hold_loaded_here(uint16_t& v) { asm volatile("" : "+v"(v) : : "memory"); }
__device__ __forceinline__ void hold_loaded_here(uint32_t& v) { asm volatile("" : "+v"(v) : : "memory"); }
__device__ __forceinline__ void hold_loaded_here(uint64_t& v) { asm volatile("" : "+v"(v) : : "memory"); }
template <typename V, int K>
__device__ __forceinline__ void pin_loaded(V (&v)[K]) {
#pragma unroll
    for (int k = 0; k < K; ++k) pin_loaded(v[k]);
}
template <typename... Loaded>
__device__ __forceinline__ void drain_vector_memory(Loaded&... loaded) {
    (pin_loaded(loaded), ...);
    __builtin_amdgcn_s_waitcnt(0x0F70);
}

// 1/sqrt(v) for v > 0: the hardware estimate (v_rsq_f32, about 1 ulp) refined by one Newton step, which
// leaves an error of a fraction of an ulp -- well inside the 1e-6 relative bound on the saved rstd -- in 7
// instructions.  The correctly rounded sqrt followed by a correctly rounded division is about 40, all of them
// on the serial path between a row's reduction and its stores.
__device__ __forceinline__ float rsqrt_refined(float v) {
    const float r = __builtin_amdgcn_rsqf(v);
    const float h = 0.5f * r;
    const float e = fmaf(-v * r, r, 1.0f);       // 1 - v*r^2
    const float refined = fmaf(h, e, r);          // r + r*e/2
    // v == 0 (eps == 0, constant row): +inf, as 1/sqrt(0) is; v == +inf (an infinity in the row): 0, where the
    // step would make inf * 0 = NaN of it
    return (v > 0.0f && v < __builtin_inff()) ? refined : r;
}

// ---------------------------------------------------------------------------------------------------
// Storage traits.  A "vector" is 16 bytes of a row: VEC elements.  unpack() widens a vector to float32,
// pack() narrows with round-to-nearest-even (v_cvt_pk_bf16_f32 / v_cvt_f16_f32 / v_cvt_f64_f32).
// ---------------------------------------------------------------------------------------------------
struct F32 {
    static constexpr bool kWindowIo = true;   // rows that miss the 16-byte path use unaligned 16-byte windows
    static constexpr int kCode = kF32, kBytes = 4, VEC = 4;
    __device__ static __forceinline__ void unpack(u32x4 v, float (&f)[VEC]) {
        uint32_t a = v[0], b = v[1], c = v[2], d = v[3];
        f[0] = as_f32(a); f[1] = as_f32(b); f[2] = as_f32(c); f[3] = as_f32(d);
    }
    __device__ static __forceinline__ u32x4 pack(const float (&f)[VEC]) {
        u32x4 v;
        v[0] = as_u32(f[0]); v[1] = as_u32(f[1]); v[2] = as_u32(f[2]); v[3] = as_u32(f[3]);
        return v;
    }
    using bits_t = uint32_t;
    __device__ static __forceinline__ bits_t load_bits(const void* p, int64_t i) {
        return reinterpret_cast<const uint32_t*>(p)[i];
    }
    __device__ static __forceinline__ float widen(bits_t u) { return as_f32(u); }
    __device__ static __forceinline__ float load1(const void* p, int64_t i) {
        return reinterpret_cast<const float*>(p)[i];
    }
    __device__ static __forceinline__ void store1(void* p, int64_t i, float f) {
        reinterpret_cast<float*>(p)[i] = f;
    }
};

struct F16 {
    static constexpr bool kWindowIo = true;   // rows that miss the 16-byte path use unaligned 16-byte windows
    static constexpr int kCode = kF16, kBytes = 2, VEC = 8;
    __device__ static __forceinline__ void unpack_pair(uint32_t u, float& lo, float& hi) {
        half2_t h = __builtin_bit_cast(half2_t, u);
        lo = static_cast<float>(h[0]);
        hi = static_cast<float>(h[1]);
    }
    __device__ static __forceinline__ void unpack(u32x4 v, float (&f)[VEC]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t u = v[i];
            unpack_pair(u, f[2 * i], f[2 * i + 1]);
        }
    }
    __device__ static __forceinline__ u32x4 pack(const float (&f)[VEC]) {
        u32x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            half2_t h;
            h[0] = static_cast<_Float16>(f[2 * i]);
            h[1] = static_cast<_Float16>(f[2 * i + 1]);
            v[i] = __builtin_bit_cast(uint32_t, h);
        }
        return v;
    }
    using bits_t = uint16_t;
    __device__ static __forceinline__ bits_t load_bits(const void* p, int64_t i) {
        return reinterpret_cast<const uint16_t*>(p)[i];
    }
    __device__ static __forceinline__ float widen(bits_t u) {
        return static_cast<float>(__builtin_bit_cast(_Float16, u));
    }
    __device__ static __forceinline__ float load1(const void* p, int64_t i) {
        return static_cast<float>(reinterpret_cast<const _Float16*>(p)[i]);
    }
    __device__ static __forceinline__ void store1(void* p, int64_t i, float f) {
        reinterpret_cast<_Float16*>(p)[i] = static_cast<_Float16>(f);
    }
};

struct BF16 {
    static constexpr bool kWindowIo = true;   // rows that miss the 16-byte path use unaligned 16-byte windows
    static constexpr int kCode = kBF16, kBytes = 2, VEC = 8;
    __device__ static __forceinline__ void unpack_pair(uint32_t u, float& lo, float& hi) {
        lo = as_f32(u << 16);
        hi = as_f32(u & 0xffff0000u);
    }
    __device__ static __forceinline__ void unpack(u32x4 v, float (&f)[VEC]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t u = v[i];
            unpack_pair(u, f[2 * i], f[2 * i + 1]);
        }
    }
    __device__ static __forceinline__ u32x4 pack(const float (&f)[VEC]) {
        u32x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            bf16x2_t h;
            h[0] = static_cast<__bf16>(f[2 * i]);
            h[1] = static_cast<__bf16>(f[2 * i + 1]);
            v[i] = __builtin_bit_cast(uint32_t, h);
        }
        return v;
    }
    using bits_t = uint16_t;
    __device__ static __forceinline__ bits_t load_bits(const void* p, int64_t i) {
        return reinterpret_cast<const uint16_t*>(p)[i];
    }
    __device__ static __forceinline__ float widen(bits_t u) { return as_f32(static_cast<uint32_t>(u) << 16); }
    __device__ static __forceinline__ float load1(const void* p, int64_t i) {
        return as_f32(static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(p)[i]) << 16);
    }
    __device__ static __forceinline__ void store1(void* p, int64_t i, float f) {
        reinterpret_cast<__bf16*>(p)[i] = static_cast<__bf16>(f);
    }
};

struct F64 {
    static constexpr bool kWindowIo = true;   // rows that miss the 16-byte path use unaligned 16-byte windows
    static constexpr int kCode = kF64, kBytes = 8, VEC = 2;
    __device__ static __forceinline__ void unpack(u32x4 v, float (&f)[VEC]) {
        uint32_t a = v[0], b = v[1], c = v[2], d = v[3];
        uint64_t lo = (static_cast<uint64_t>(b) << 32) | a;
        uint64_t hi = (static_cast<uint64_t>(d) << 32) | c;
        f[0] = static_cast<float>(__builtin_bit_cast(double, lo));
        f[1] = static_cast<float>(__builtin_bit_cast(double, hi));
    }
    __device__ static __forceinline__ u32x4 pack(const float (&f)[VEC]) {
        uint64_t lo = __builtin_bit_cast(uint64_t, static_cast<double>(f[0]));
        uint64_t hi = __builtin_bit_cast(uint64_t, static_cast<double>(f[1]));
        u32x4 v;
        v[0] = static_cast<uint32_t>(lo); v[1] = static_cast<uint32_t>(lo >> 32);
        v[2] = static_cast<uint32_t>(hi); v[3] = static_cast<uint32_t>(hi >> 32);
        return v;
    }
    using bits_t = uint64_t;
    __device__ static __forceinline__ bits_t load_bits(const void* p, int64_t i) {
        return reinterpret_cast<const uint64_t*>(p)[i];
    }
    __device__ static __forceinline__ float widen(bits_t u) {
        return static_cast<float>(__builtin_bit_cast(double, u));
    }
    __device__ static __forceinline__ float load1(const void* p, int64_t i) {
        return static_cast<float>(reinterpret_cast<const double*>(p)[i]);
    }
    __device__ static __forceinline__ void store1(void* p, int64_t i, float f) {
        reinterpret_cast<double*>(p)[i] = static_cast<double>(f);
    }
};

// One element of a weight / bias vector whose storage type is only known at run time (cold paths only).
__device__ __forceinline__ void store_param(void* p, int dtype, int64_t i, float f) {
    switch (dtype) {
        case kF32: F32::store1(p, i, f); break;
        case kF16: F16::store1(p, i, f); break;
        case kBF16: BF16::store1(p, i, f); break;
        default: F64::store1(p, i, f); break;
    }
}

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef u32x4 u32x4_param_unaligned __attribute__((aligned(2)));
typedef u32x2 u32x2_param_unaligned __attribute__((aligned(2)));
typedef uint32_t u32_param_unaligned __attribute__((aligned(2)));

// VEC consecutive parameter elements of storage type WT starting at column c0, widened to float32, fetched
// with the widest loads their size allows.  UNALIGNED false: the 128-bit path guarantees that the chunk is
// naturally aligned (the parameter pointer is 16-byte aligned and c0 is a multiple of VEC).  UNALIGNED true: the
// chunk starts at any element (rows off the 128-bit path: the hardware's unaligned access mode serves the same
// instructions at element-aligned addresses).
template <typename WT, int VEC, bool UNALIGNED = false>
__device__ __forceinline__ void load_param_chunk(const void* p, int c0, float (&out)[VEC]) {
    constexpr int BYTES = VEC * WT::kBytes;
    const char* src = static_cast<const char*>(p) + static_cast<int64_t>(c0) * WT::kBytes;
    if constexpr (BYTES >= 16) {
        constexpr int PIECES = BYTES / 16;
        constexpr int EPP = WT::VEC;            // elements per 16-byte piece
        u32x4 raw[PIECES];
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            if constexpr (UNALIGNED) raw[i] = *reinterpret_cast<const u32x4_param_unaligned*>(src + 16 * i);
            else raw[i] = *reinterpret_cast<const u32x4*>(src + 16 * i);
        }
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            float f[EPP];
            WT::unpack(raw[i], f);
#pragma unroll
            for (int j = 0; j < EPP; ++j) out[i * EPP + j] = f[j];
        }
    } else if constexpr (WT::kBytes == 4) {       // two float32 (VEC == 2)
        u32x2 raw;
        if constexpr (UNALIGNED) raw = *reinterpret_cast<const u32x2_param_unaligned*>(src);
        else raw = *reinterpret_cast<const u32x2*>(src);
        out[0] = as_f32(raw[0]);
        out[1] = as_f32(raw[1]);
    } else {                                      // 16-bit parameters under a wider row type: 4 or 8 bytes
        static_assert(WT::kBytes == 2 && (VEC == 2 || VEC == 4), "chunk shape");
        if constexpr (VEC == 4) {
            u32x2 raw;
            if constexpr (UNALIGNED) raw = *reinterpret_cast<const u32x2_param_unaligned*>(src);
            else raw = *reinterpret_cast<const u32x2*>(src);
            WT::unpack_pair(raw[0], out[0], out[1]);
            WT::unpack_pair(raw[1], out[2], out[3]);
        } else {
            uint32_t raw;
            if constexpr (UNALIGNED) raw = *reinterpret_cast<const u32_param_unaligned*>(src);
            else raw = *reinterpret_cast<const uint32_t*>(src);
            WT::unpack_pair(raw, out[0], out[1]);
        }
    }
}

// The K*VEC weight (or bias) elements of a thread's (clamped) vector slots, widened to float32.  The
// storage type is only known at run time: one uniform branch on it, then independent loads at always valid
// columns.  voff[k] is the slot's byte offset in a row on the 128-bit path (one wide load per slot), its
// vector index on the unaligned path (element loads; columns past the row end read as `fill`).
template <typename WT, int K, int VEC, int ROW_BYTES_PER_ELEM, bool ALIGNED>
__device__ __forceinline__ void load_params_as(float (&out)[K][VEC], const void* p, const int (&voff)[K],
                                               int n_cols, float fill) {
    if constexpr (ALIGNED) {
#pragma unroll
        for (int k = 0; k < K; ++k) load_param_chunk<WT, VEC>(p, voff[k] / ROW_BYTES_PER_ELEM, out[k]);
    } else {
        // Two phases, so that the K*VEC element loads are all in flight before the first one is waited for
        // (interleaved with their conversions they were issued one by one, each waiting for the previous: tens of
        // microseconds at the start of every workgroup).
        typename WT::bits_t raw[K][VEC];
#pragma unroll
        for (int k = 0; k < K; ++k) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const int c = voff[k] * VEC + e;
                raw[k][e] = WT::load_bits(p, c < n_cols ? c : n_cols - 1);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < K; ++k) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) out[k][e] = (voff[k] * VEC + e < n_cols) ? WT::widen(raw[k][e]) : fill;
        }
    }
}

template <int K, int VEC, bool ALIGNED>
__device__ __forceinline__ void load_params_clamped(float (&out)[K][VEC], const void* p, int dtype,
                                                    const int (&voff)[K], int n_cols, float fill) {
    constexpr int RB = 16 / VEC;    // bytes per row element: byte offset / RB = column
    if (p == nullptr) {
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
            for (int e = 0; e < VEC; ++e) out[k][e] = fill;
        return;
    }
    switch (dtype) {
        case kF32: load_params_as<F32, K, VEC, RB, ALIGNED>(out, p, voff, n_cols, fill); break;
        case kF16: load_params_as<F16, K, VEC, RB, ALIGNED>(out, p, voff, n_cols, fill); break;
        case kBF16: load_params_as<BF16, K, VEC, RB, ALIGNED>(out, p, voff, n_cols, fill); break;
        default: load_params_as<F64, K, VEC, RB, ALIGNED>(out, p, voff, n_cols, fill); break;
    }
}

// The same for the overlapped-window slots of rows off the 128-bit path (norm kernels): slot k covers the VEC
// columns that start at byte offset woff[k] of a row, all of them inside the row, at any element.
template <typename WT, int K, int VEC>
__device__ __forceinline__ void load_params_window_as(float (&out)[K][VEC], const void* p, const int (&woff)[K]) {
    constexpr int RB = 16 / VEC;    // bytes per row element: byte offset / RB = column
#pragma unroll
    for (int k = 0; k < K; ++k) load_param_chunk<WT, VEC, true>(p, woff[k] / RB, out[k]);
}

template <int K, int VEC>
__device__ __forceinline__ void load_params_window(float (&out)[K][VEC], const void* p, int dtype, const int (&woff)[K],
                                                   float fill) {
    if (p == nullptr) {
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
            for (int e = 0; e < VEC; ++e) out[k][e] = fill;
        return;
    }
    switch (dtype) {
        case kF32: load_params_window_as<F32, K, VEC>(out, p, woff); break;
        case kF16: load_params_window_as<F16, K, VEC>(out, p, woff); break;
        case kBF16: load_params_window_as<BF16, K, VEC>(out, p, woff); break;
        default: load_params_window_as<F64, K, VEC>(out, p, woff); break;
    }
}

// ---------------------------------------------------------------------------------------------------
// Row I/O for rows that cannot use aligned 128-bit accesses (N not a multiple of VEC, or a pointer or row stride
// that is not a multiple of 16 bytes): the same 16-byte register image is assembled from an unaligned 16-byte
// window (rows of at least one vector) or from element loads with a per-column bound (ElemIo<T>: shorter rows),
// so every other part of the kernels is shared with the 128-bit path.
// ---------------------------------------------------------------------------------------------------
// The same storage type, for rows shorter than one vector (N < VEC): every access is a single element.
template <typename T>
struct ElemIo : T {
    static constexpr bool kWindowIo = false;
};

typedef u32x4 u32x4_unaligned __attribute__((aligned(2)));

// 16-byte accesses at any element-aligned address (the hardware's unaligned access mode, which the HSA stack
// enables; the compiler emits the same global_load_dwordx4 / global_store_dwordx4 as for aligned ones).
__device__ __forceinline__ u32x4 ld128u(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4_unaligned*>(p));
}
// The same load without the non-temporal hint: for data that is read again shortly (it may stay in the caches).
__device__ __forceinline__ u32x4 ld128u_keep(const void* p) { return *reinterpret_cast<const u32x4_unaligned*>(p); }
__device__ __forceinline__ void st128u(void* p, u32x4 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4_unaligned*>(p));
}
// The same store without the hint: for an output that is read again shortly.
__device__ __forceinline__ void st128u_keep(void* p, u32x4 v) { *reinterpret_cast<u32x4_unaligned*>(p) = v; }

// Element accesses with a column bound: for rows shorter than one vector (ElemIo<T>).  Columns past the row end read
// as 0 and are not stored.
template <typename T, bool KEEP = false>
__device__ __forceinline__ u32x4 load_vec_elems(const char* row, int vec, int n_cols) {
    float f[T::VEC];
#pragma unroll
    for (int e = 0; e < T::VEC; ++e) {
        const int c = vec * T::VEC + e;
        const float v = T::load1(row, c < n_cols ? c : n_cols - 1);
        f[e] = c < n_cols ? v : 0.0f;
    }
    return T::pack(f);   // exact: every element came from storage type T
}

template <typename T>
__device__ __forceinline__ void store_vec_elems(char* row, int vec, int n_cols, const float (&f)[T::VEC]) {
#pragma unroll
    for (int e = 0; e < T::VEC; ++e) {
        const int c = vec * T::VEC + e;
        if (c < n_cols) T::store1(row, c, f[e]);
    }
}

// A per-row scalar of storage type T (a saved norm, an upstream gradient of one) that the row loop requests one row
// ahead: load() returns its raw bits, value() widens them.  Between the two the kernel calls hold_loaded_here() at
// the point up to which the value is not needed.  (The bits stay in their own width: a 16-bit value widened to 32
// bits before the hold is one more instruction for the compiler to place early.)
template <typename T>
struct RowScalar {
    using bits_t = typename T::bits_t;
    __device__ static __forceinline__ bits_t load(const void* p, int64_t i) { return T::load_bits(p, i); }
    __device__ static __forceinline__ float value(bits_t raw) { return T::widen(raw); }
};

// Unpacking / packing for kernels whose arithmetic type C is float64 on float64 storage (the float32 traits
// narrow on load).
template <typename T>
__device__ __forceinline__ void unpack_as(u32x4 v, float (&f)[T::VEC]) { T::unpack(v, f); }
template <typename T>
__device__ __forceinline__ void unpack_as(u32x4 v, double (&f)[T::VEC]) {
    static_assert(T::kBytes == 8, "float64 arithmetic is for float64 storage only");
    const uint32_t a = v[0], b = v[1], c = v[2], d = v[3];
    f[0] = __builtin_bit_cast(double, (static_cast<uint64_t>(b) << 32) | a);
    f[1] = __builtin_bit_cast(double, (static_cast<uint64_t>(d) << 32) | c);
}



__device__ __forceinline__ u32x4 pack_f64(const double (&f)[2]) {
    const uint64_t lo = __builtin_bit_cast(uint64_t, f[0]), hi = __builtin_bit_cast(uint64_t, f[1]);
    u32x4 v;
    v[0] = static_cast<uint32_t>(lo); v[1] = static_cast<uint32_t>(lo >> 32);
    v[2] = static_cast<uint32_t>(hi); v[3] = static_cast<uint32_t>(hi >> 32);
    return v;
}

template <typename T, typename C>
__device__ __forceinline__ u32x4 pack_as(const C (&f)[T::VEC]) {
    if constexpr (std::is_same<C, double>::value) return pack_f64(f);
    else return T::pack(f);
}

template <typename T, typename C>
__device__ __forceinline__ C load_elem(const void* p, int64_t i) {
    if constexpr (std::is_same<C, double>::value) return reinterpret_cast<const double*>(p)[i];
    else return T::load1(p, i);
}

template <typename T, typename C>
__device__ __forceinline__ void store_elem(void* p, int64_t i, C v) {
    if constexpr (std::is_same<C, double>::value) reinterpret_cast<double*>(p)[i] = v;
    else T::store1(p, i, v);
}

__device__ __forceinline__ float exp_c(float z) { return __expf(z); }
__device__ __forceinline__ double exp_c(double z) { return exp(z); }


// ---------------------------------------------------------------------------------------------------
// Wave64 all-reduce (sum, or max with OpMax) over aligned groups of W lanes, W in {8, 16, 32, 64}.  The first four steps
// are DPP modifiers fused into v_add_f32 / v_max_f32 (no LDS traffic); the 16- and 32-lane exchanges use the gfx950
// v_permlane16_swap / v_permlane32_swap instructions.  Every lane of a group ends with the group's sum,
// and all lanes of a group add the same values in the same tree, so the result is identical on all of them.
// ---------------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_mov_bits(uint32_t v) {
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) { return as_f32(dpp_mov_bits<CTRL>(as_u32(v))); }
// A float64 travels as its two 32-bit halves, each moved with the same lane pattern.
template <int CTRL>
__device__ __forceinline__ double dpp_mov(double v) {
    const uint64_t u = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = dpp_mov_bits<CTRL>(static_cast<uint32_t>(u));
    const uint32_t hi = dpp_mov_bits<CTRL>(static_cast<uint32_t>(u >> 32));
    return __builtin_bit_cast(double, (static_cast<uint64_t>(hi) << 32) | lo);
}

struct OpSum {
    template <typename V> __device__ static __forceinline__ V apply(V a, V b) { return a + b; }
    template <typename V> __device__ static __forceinline__ V identity() { return V(0); }
};
struct OpMax {
    __device__ static __forceinline__ float apply(float a, float b) { return fmaxf(a, b); }
    __device__ static __forceinline__ double apply(double a, double b) { return fmax(a, b); }
    template <typename V> __device__ static __forceinline__ V identity() { return -static_cast<V>(__builtin_inff()); }
};

// One 32-bit word exchanged with the partner lane 16 (WIDE = false) or 32 (WIDE = true) lanes away: `mine`
// and `theirs` come back in an order that is the same on both partners' sides of the addition tree.
template <bool WIDE>
__device__ __forceinline__ void swap_lanes(uint32_t u, uint32_t& first, uint32_t& second) {
    if constexpr (WIDE) {
        auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        first = r[0]; second = r[1];
    } else {
        auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
        first = r[0]; second = r[1];
    }
}
template <bool WIDE, typename Op>
__device__ __forceinline__ float swap_combine(float v) {
    uint32_t a, b;
    swap_lanes<WIDE>(as_u32(v), a, b);
    return Op::apply(as_f32(a), as_f32(b));
}
template <bool WIDE, typename Op>
__device__ __forceinline__ double swap_combine(double v) {
    const uint64_t u = __builtin_bit_cast(uint64_t, v);
    uint32_t al, bl, ah, bh;
    swap_lanes<WIDE>(static_cast<uint32_t>(u), al, bl);
    swap_lanes<WIDE>(static_cast<uint32_t>(u >> 32), ah, bh);
    const double a = __builtin_bit_cast(double, (static_cast<uint64_t>(ah) << 32) | al);
    const double b = __builtin_bit_cast(double, (static_cast<uint64_t>(bh) << 32) | bl);
    return Op::apply(a, b);
}

template <int W, typename Op = OpSum, typename V = float>
__device__ __forceinline__ V group_allreduce(V v) {
    static_assert(W == 8 || W == 16 || W == 32 || W == 64, "group width");
    v = Op::apply(v, dpp_mov<0xB1>(v));    // quad_perm [1,0,3,2]: lane ^ 1
    v = Op::apply(v, dpp_mov<0x4E>(v));    // quad_perm [2,3,0,1]: lane ^ 2
    v = Op::apply(v, dpp_mov<0x141>(v));   // row_half_mirror: the other quad of each 8 lanes
    if constexpr (W >= 16) v = Op::apply(v, dpp_mov<0x140>(v));   // row_mirror: the other half of each 16 lanes
    if constexpr (W >= 32) v = swap_combine<false, Op>(v);
    if constexpr (W >= 64) v = swap_combine<true, Op>(v);
    return v;
}

// Sum NV values over the TPR threads that share a row.  TPR <= 64: pure register exchange.  TPR > 64: each
// wave publishes its sums in an LDS slot, one workgroup barrier, every thread adds the TPR/64 slots of its
// row in a fixed order.  The slots are double buffered on `phase`, so one barrier per call is enough: a
// slot is rewritten two calls later, and no wave can pass the barrier in between before all have read it.
// All threads of the workgroup must call this together when TPR > 64.
template <int TPR, int G, int NV, typename Op = OpSum, typename V = float>
__device__ __forceinline__ void row_allreduce(V (&v)[NV], V* red, int& phase, int g, int t) {
    constexpr int W = TPR < 64 ? TPR : 64;
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] = group_allreduce<W, Op, V>(v[i]);
    if constexpr (TPR > 64) {
        constexpr int WPR = TPR / 64;
        constexpr int NVP = NV == 3 ? 4 : NV;
        V* slot = red + (((phase & 1) * G + g) * WPR) * NVP;
        const int wv = t >> 6;
        if ((t & 63) == 0) {
#pragma unroll
            for (int i = 0; i < NV; ++i) slot[wv * NVP + i] = v[i];
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NV; ++i) v[i] = Op::template identity<V>();
#pragma unroll
        for (int w = 0; w < WPR; ++w) {
#pragma unroll
            for (int i = 0; i < NV; ++i) v[i] = Op::apply(v[i], slot[w * NVP + i]);
        }
        ++phase;
    }
}

template <int TPR, int G, int NV>
struct RedSmem {
    static constexpr int kFloats = TPR > 64 ? 2 * G * (TPR / 64) * (NV == 3 ? 4 : NV) : 1;
};

}  // namespace thn
