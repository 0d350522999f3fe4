// Element-wise activations, forward and backward: GeLU (exact / tanh), SiLU, ReLU, LeakyReLU, ReLU6, Sigmoid,
// Tanh, Mish, Softplus, Threshold -- the reference's TritonHub/Activations/{gelu,silu,relu,leaky_relu,relu6,
// sigmoid,tanh,mish,softplus,threshold}.py.  Pure streaming: the forward reads x and writes y (2*s bytes per
// element), the backward reads the saved tensor and dy and writes dx (3*s bytes per element).
//
// Arithmetic type, as in the reference: float32 for the kernels that widen on load (gelu.py:20, silu.py:18,
// sigmoid.py:18, tanh.py:18, mish.py:18); the loaded type for the others (relu.py:18, leaky_relu.py:19,
// relu6.py:18, softplus.py:20, threshold.py:19), which for 16-bit storage still means float32 arithmetic with
// one rounding on store (their float32 scalar arguments promote the expression) and for float64 storage means
// float64 -- a ReLU of a float64 tensor returns its input bits.
//
// Where the reference's formula overflows to NaN for large |x| although the function is finite -- tanh as
// (e^x - e^-x)/(e^x + e^-x) (tanh.py:19-21, mish.py:20-22), GeLU's tanh as (e^2u - 1)/(e^2u + 1) (gelu.py:24-25)
// -- the same function is evaluated in a form that cannot overflow; the values agree wherever the reference's
// are finite.
#pragma once

#include <type_traits>

#include "thn_act_math.h"
#include "thn_kernels.h"

namespace thn {

constexpr bool act_uses_loaded_type(int act) {
    return act == kRelu || act == kLeakyRelu || act == kRelu6 || act == kSoftplus || act == kThreshold;
}
// Sigmoid and Tanh save their OUTPUT for the backward (sigmoid.py:81-92, tanh.py:83-94); the others their input.

template <typename T, int ACT>
struct ActCompute {
    using type = typename std::conditional<T::kBytes == 8 && act_uses_loaded_type(ACT), double, float>::type;
};

struct ActArgs {
    const char* x;        // forward: input.  backward: the saved tensor (input, or output for Sigmoid / Tanh)
    const char* g;        // backward: upstream gradient
    char* out;            // y, or dx
    int64_t total_vecs;   // flat kernels: whole 16-byte vectors
    int64_t total_elems;  // flat kernels
    int64_t x_stride_bytes, g_stride_bytes, out_stride_bytes;   // row kernels
    int64_t M, N;         // row kernels
    int lx;               // row kernels: log2 of the threads along a row
    float p0, p1;         // negative_slope | beta, threshold | threshold, value
};

// ---------------------------------------------------------------------------------------------------
// Contiguous tensors: one flat stream of 16-byte vectors.  A persistent grid; every thread owns U vectors per
// grid step (vector v0 + u*BLOCK, so a wave touches contiguous 1 KiB segments), requests the next step's
// vectors before it computes the current ones, and clamps vector slots past the end onto the last vector (they
// recompute and re-store its values), which keeps the loop free of branches around memory operations.
// The last total_elems % VEC elements are handled one by one after the loop.
// ---------------------------------------------------------------------------------------------------
constexpr int kActBlock = 256;

template <typename T, int ACT, bool BWD, int U>
__global__ void __launch_bounds__(kActBlock) act_flat_kernel(const ActArgs a) {
    using C = typename ActCompute<T, ACT>::type;
    constexpr int VEC = T::VEC;
    const C p0 = static_cast<C>(a.p0), p1 = static_cast<C>(a.p1);
    // The forward keeps in the caches the tensor its backward will read again (ld128_keep): the input, or the output
    // for Sigmoid and Tanh; everything else streams.  bf16 16384 x 4096, forward + backward of one batch: SiLU
    // 112.1 -> 106.2 us, ReLU 108.9 -> 106.2 us, float32 Sigmoid 214.0 -> 200.1 us.
    constexpr bool kSavesOutput = ACT == kSigmoid || ACT == kTanh;
    constexpr bool kKeepX = !BWD && !kSavesOutput;
    constexpr bool kKeepOut = !BWD && kSavesOutput;

    if (a.total_vecs > 0) {
        const int64_t step = static_cast<int64_t>(gridDim.x) * kActBlock * U;
        const int64_t last = a.total_vecs - 1;
        int64_t v0 = static_cast<int64_t>(blockIdx.x) * kActBlock * U + threadIdx.x;
        u32x4 cx[U], cg[BWD ? U : 1];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t v = v0 + u * kActBlock;
            const int64_t vc = (v < last ? v : last) * 16;
            cx[u] = kKeepX ? ld128_keep(a.x + vc) : ld128(a.x + vc);
            if constexpr (BWD) cg[u] = ld128(a.g + vc);
        }
        if constexpr (BWD) pin_loaded(cg);
        drain_vector_memory(cx);
        for (int64_t base = static_cast<int64_t>(blockIdx.x) * kActBlock * U; base < a.total_vecs; base += step) {
            const int64_t n0 = v0 + step;
            u32x4 nx[U], ng[BWD ? U : 1];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t v = n0 + u * kActBlock;
                const int64_t vc = (v < last ? v : last) * 16;
                nx[u] = kKeepX ? ld128_keep(a.x + vc) : ld128(a.x + vc);
                if constexpr (BWD) ng[u] = ld128(a.g + vc);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                C xf[VEC], gf[VEC], of[VEC];
                unpack_as<T>(cx[u], xf);
                if constexpr (BWD) unpack_as<T>(cg[u], gf);
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    if constexpr (BWD) of[e] = act_bwd<ACT, C>(xf[e], gf[e], p0, p1);
                    else of[e] = act_fwd<ACT, C>(xf[e], p0, p1);
                }
                const int64_t v = v0 + u * kActBlock;
                if constexpr (kKeepOut) st128_keep(a.out + (v < last ? v : last) * 16, pack_as<T, C>(of));
                else st128(a.out + (v < last ? v : last) * 16, pack_as<T, C>(of));
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                cx[u] = nx[u];
                if constexpr (BWD) cg[u] = ng[u];
            }
            v0 = n0;
        }
    }
    // the tail that does not fill a vector
    const int64_t tail0 = a.total_vecs * VEC;
    const int64_t i = tail0 + threadIdx.x;
    if (blockIdx.x == 0 && i < a.total_elems) {
        const C x = load_elem<T, C>(a.x, i);
        if constexpr (BWD) store_elem<T, C>(a.out, i, act_bwd<ACT, C>(x, load_elem<T, C>(a.g, i), p0, p1));
        else store_elem<T, C>(a.out, i, act_fwd<ACT, C>(x, p0, p1));
    }
}

// ---------------------------------------------------------------------------------------------------
// Strided rows, or pointers that are not 16-byte aligned: the same 16-byte vectors at element-aligned addresses
// (the memory pipeline runs in unaligned access mode), tiled over (rows, vectors of a row).  A workgroup is
// 2^lx threads along the row (consecutive lanes take consecutive vectors) by 256 >> lx rows, so rows of any width
// fill it; every thread takes the same vector slot of U rows per step (all requested before the first is used),
// walks the slots of a row with stride gridDim.x << lx and the rows with stride gridDim.y.  The elements behind
// the last whole vector of a row go one by one, in the thread that owns that slot.
// ---------------------------------------------------------------------------------------------------
template <typename T, int ACT, bool BWD>
__global__ void __launch_bounds__(kActBlock) act_rows_kernel(const ActArgs a) {
    using C = typename ActCompute<T, ACT>::type;
    constexpr int VEC = T::VEC;
    constexpr int U = BWD ? 2 : 4;
    const C p0 = static_cast<C>(a.p0), p1 = static_cast<C>(a.p1);
    const int lx = a.lx;
    const int tx = threadIdx.x & ((1 << lx) - 1);
    const int ty = threadIdx.x >> lx;
    const int64_t rows_per_block = kActBlock >> lx;
    const int64_t slots = (a.N + VEC - 1) / VEC;          // vector slots of a row; the last may be ragged
    const int64_t whole = a.N / VEC;
    const int64_t vstep = static_cast<int64_t>(gridDim.x) << lx;
    for (int64_t row0 = blockIdx.y * rows_per_block * U + ty; row0 < a.M; row0 += gridDim.y * rows_per_block * U) {
        for (int64_t v = (static_cast<int64_t>(blockIdx.x) << lx) + tx; v < slots; v += vstep) {
            u32x4 cx[U], cg[BWD ? U : 1];
            if (v < whole) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int64_t row = row0 + u * rows_per_block;
                    if (row < a.M) {
                        cx[u] = ld128u(a.x + row * a.x_stride_bytes + v * 16);
                        if constexpr (BWD) cg[u] = ld128u(a.g + row * a.g_stride_bytes + v * 16);
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t row = row0 + u * rows_per_block;
                if (row >= a.M) continue;
                char* outr = a.out + row * a.out_stride_bytes;
                if (v < whole) {
                    C xf[VEC], gf[VEC], of[VEC];
                    unpack_as<T>(cx[u], xf);
                    if constexpr (BWD) unpack_as<T>(cg[u], gf);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        if constexpr (BWD) of[e] = act_bwd<ACT, C>(xf[e], gf[e], p0, p1);
                        else of[e] = act_fwd<ACT, C>(xf[e], p0, p1);
                    }
                    st128u(outr + v * 16, pack_as<T, C>(of));
                } else {
                    const char* xr = a.x + row * a.x_stride_bytes;
                    const char* gr = BWD ? a.g + row * a.g_stride_bytes : nullptr;
                    for (int64_t c = v * VEC; c < a.N; ++c) {
                        const C x = load_elem<T, C>(xr, c);
                        if constexpr (BWD) store_elem<T, C>(outr, c, act_bwd<ACT, C>(x, load_elem<T, C>(gr, c), p0, p1));
                        else store_elem<T, C>(outr, c, act_fwd<ACT, C>(x, p0, p1));
                    }
                }
            }
        }
    }
}

}  // namespace thn
