// Softmax / Softmin / LogSoftmax over the last dimension, forward and backward: the reference's
// TritonHub/Activations/softmax.py, softmin.py and logsoftmax.py on the row engine of the norm kernels
// (same decomposition, same branch-free prefetching loop; see thn_kernels.h).
#pragma once

#include <type_traits>

#include "thn_kernels.h"
#include "thn_walk.h"

namespace thn {

struct SoftmaxFwdArgs {
    const char* x;
    char* y;
    int64_t x_stride_bytes;
    int64_t y_stride_bytes;
    int64_t M;
    int n_cols;
    int n_vecs;
    float sign;      // -1: the input is negated on load (Softmin of x = Softmax of -x)
    int line_shift;  // as in FwdArgs (row kernels only)
};

struct SoftmaxBwdArgs {
    const char* y;   // the SAVED OUTPUT of the forward (softmax.py:86-97, logsoftmax.py:93-104)
    const char* dy;
    char* dx;
    int64_t y_stride_bytes;
    int64_t dy_stride_bytes;
    int64_t dx_stride_bytes;
    int64_t M;
    int n_cols;
    int n_vecs;
    float sign;      // -1: the gradient is negated on store (fused Softmin)
    int line_shift;  // as in FwdArgs (row kernels only)
};

// Arithmetic type.  Float32 for 16- and 32-bit storage and for every log-softmax (logsoftmax.py:19, :61-62 widen
// to float32 explicitly).  The reference's softmax / softmin kernels compute in the type they load
// (softmax.py:18-23), so float64 rows are computed in float64.
template <typename T, bool LOG> struct SoftmaxCompute {
    using type = typename std::conditional<T::kBytes == 8 && !LOG, double, float>::type;
};

// The vector slots of one row (slot_place() / slot_load() of thn_kernels.h) for arithmetic type C.  Rows shorter than
// one vector come through element loads, and those of the float32 engine narrow float64 storage on the way, which the
// float64 path must not do.
template <typename T, typename C, int K, bool ALIGNED, bool KEEP = false>
__device__ __forceinline__ void load_slots_as(u32x4 (&dst)[K], const char* base, int64_t stride_bytes, int64_t row,
                                              const int (&voff)[K], int n_cols) {
    if constexpr (ALIGNED || T::kWindowIo || std::is_same<C, float>::value) {
        slot_load_row<T, K, ALIGNED, KEEP>(dst, base, stride_bytes, row, voff, n_cols);
    } else {
        const double* p = reinterpret_cast<const double*>(base + row * stride_bytes);
#pragma unroll
        for (int k = 0; k < K; ++k) {
            double f[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int c = voff[k] * 2 + e;
                const double v = p[c < n_cols ? c : n_cols - 1];
                f[e] = c < n_cols ? v : 0.0;
            }
            dst[k] = pack_f64(f);
        }
    }
}

// Stores one slot.  KEEP: as slot_store() -- the softmax family's forward keeps its output, the backward works from
// the saved y.
template <typename T, bool ALIGNED, bool KEEP = false>
__device__ __forceinline__ void store_slot_as(char* rowp, int voff, int n_cols, const float (&f)[T::VEC]) {
    slot_store<T, ALIGNED, KEEP>(rowp, voff, n_cols, f);
}
template <typename T, bool ALIGNED, bool KEEP = false>
__device__ __forceinline__ void store_slot_as(char* rowp, int voff, int n_cols, const double (&f)[T::VEC]) {
    static_assert(T::kBytes == 8, "float64 arithmetic is for float64 storage only");
    if constexpr (ALIGNED || T::kWindowIo) {
        slot_store_bits<ALIGNED, KEEP>(rowp + voff, pack_f64(f));
    } else {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int c = voff * 2 + e;
            if (c < n_cols) reinterpret_cast<double*>(rowp)[c] = f[e];
        }
    }
}

// Forward (softmax.py:17-23, logsoftmax.py:19-24): z = x - max(x); softmax: exp(z) / sum(exp(z));
// log-softmax: z - log(sum(exp(z))).  One rounding on store.
template <typename T, bool LOG, int K, int TPR, int BLOCK, bool ALIGNED>
__global__ void __launch_bounds__(BLOCK) softmax_fwd_kernel(const SoftmaxFwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int G = BLOCK / TPR;
    static_assert(BLOCK % TPR == 0 && G >= 1, "a workgroup holds whole rows");
    using C = typename SoftmaxCompute<T, LOG>::type;
    __shared__ C red[RedSmem<TPR, G, 1>::kFloats];

    const int tid = threadIdx.x;
    const int g = tid / TPR;
    const int t = tid % TPR;
    int phase = 0;

    const int shift = (ALIGNED && G == 1) ? row_line_shift(a.line_shift, a.x, a.x_stride_bytes, blockIdx.x) : 0;
    // Rows off the 128-bit path: unaligned 16-byte windows, the ragged last one overlapping its neighbour (slot_place()).
    int voff[K], lead[K];
    bool own[K];
#pragma unroll
    for (int k = 0; k < K; ++k) slot_place<T, ALIGNED>(t + k * TPR - shift, a.n_vecs, a.n_cols, voff[k], lead[k], own[k]);
    // element e of slot k counts in the row sums (always true on the 128-bit path)
    auto counts = [&](int k, int e) -> bool { return slot_counts<T, ALIGNED>(voff[k], lead[k], e, a.n_cols); };
    const C sign = static_cast<C>(a.sign);
    const C neg_inf = OpMax::identity<C>();

    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * G;
    const int64_t last_row = a.M - 1;
    int64_t row_raw = static_cast<int64_t>(blockIdx.x) * G + g;
    int64_t row = row_raw < a.M ? row_raw : last_row;
    u32x4 cur[K];
    load_slots_as<T, C, K, ALIGNED>(cur, a.x, a.x_stride_bytes, row, voff, a.n_cols);

    drain_vector_memory(cur);
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * G; base < a.M; base += rows_per_iter) {
        const int64_t nrow_raw = row_raw + rows_per_iter;
        const int64_t nrow = nrow_raw < a.M ? nrow_raw : last_row;
        u32x4 nxt[K];
        load_slots_as<T, C, K, ALIGNED>(nxt, a.x, a.x_stride_bytes, nrow, voff, a.n_cols);

        C xf[K][VEC];
        C m[1] = {neg_inf};
#pragma unroll
        for (int k = 0; k < K; ++k) {
            unpack_as<T>(cur[k], xf[k]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                C v = xf[k][e] * sign;
                if constexpr (!ALIGNED && !T::kWindowIo) v = counts(k, e) ? v : neg_inf;     // past the end of a short row
                xf[k][e] = v;
                m[0] = OpMax::apply(m[0], v);      // clamped and overlapping slots repeat real columns: harmless for a maximum
            }
        }
        row_allreduce<TPR, G, 1, OpMax, C>(m, red, phase, g, t);

        C s[1] = {C(0)};
#pragma unroll
        for (int k = 0; k < K; ++k) {
            C sk = C(0);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const C z = xf[k][e] - m[0];
                const C ez = exp_c(z);              // columns past the row end: exp(-inf) = 0
                xf[k][e] = LOG ? z : ez;
                sk += counts(k, e) ? ez : C(0);
            }
            s[0] += own[k] ? sk : C(0);
        }
        row_allreduce<TPR, G, 1, OpSum, C>(s, red, phase, g, t);
        C scale;
        if constexpr (LOG) scale = logf(s[0]);
        else scale = C(1) / s[0];

        char* yrow = a.y + row * a.y_stride_bytes;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            C yf[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) yf[e] = LOG ? xf[k][e] - scale : xf[k][e] * scale;
            store_slot_as<T, ALIGNED, true>(yrow, voff[k], a.n_cols, yf);
        }

#pragma unroll
        for (int k = 0; k < K; ++k) cur[k] = nxt[k];
        row_raw = nrow_raw;
        row = nrow;
    }
}

// Backward from the saved output y and the upstream gradient g:
//   softmax (softmax.py:57-61):       dx = y*g - y*sum(y*g)
//   log-softmax (logsoftmax.py:61-67): dx = g - exp(y)*sum(g)
template <typename T, bool LOG, int K, int TPR, int BLOCK, bool ALIGNED>
__global__ void __launch_bounds__(BLOCK) softmax_bwd_kernel(const SoftmaxBwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int G = BLOCK / TPR;
    static_assert(BLOCK % TPR == 0 && G >= 1, "a workgroup holds whole rows");
    using C = typename SoftmaxCompute<T, LOG>::type;
    __shared__ C red[RedSmem<TPR, G, 1>::kFloats];

    const int tid = threadIdx.x;
    const int g = tid / TPR;
    const int t = tid % TPR;
    int phase = 0;

    const int shift = (ALIGNED && G == 1) ? row_line_shift(a.line_shift, a.y, a.y_stride_bytes, blockIdx.x) : 0;
    // Rows off the 128-bit path: unaligned 16-byte windows, the ragged last one overlapping its neighbour (slot_place()).
    int voff[K], lead[K];
    bool own[K];
#pragma unroll
    for (int k = 0; k < K; ++k) slot_place<T, ALIGNED>(t + k * TPR - shift, a.n_vecs, a.n_cols, voff[k], lead[k], own[k]);
    // element e of slot k counts in the row sums (always true on the 128-bit path)
    auto counts = [&](int k, int e) -> bool { return slot_counts<T, ALIGNED>(voff[k], lead[k], e, a.n_cols); };

    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * G;
    const int64_t last_row = a.M - 1;
    int64_t row_raw = static_cast<int64_t>(blockIdx.x) * G + g;
    int64_t row = row_raw < a.M ? row_raw : last_row;
    const C sign = static_cast<C>(a.sign);
    u32x4 cy[K], cg[K];
    load_slots_as<T, C, K, ALIGNED>(cy, a.y, a.y_stride_bytes, row, voff, a.n_cols);
    load_slots_as<T, C, K, ALIGNED>(cg, a.dy, a.dy_stride_bytes, row, voff, a.n_cols);

    drain_vector_memory(cy, cg);
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * G; base < a.M; base += rows_per_iter) {
        const int64_t nrow_raw = row_raw + rows_per_iter;
        const int64_t nrow = nrow_raw < a.M ? nrow_raw : last_row;
        u32x4 ny[K], ng[K];
        load_slots_as<T, C, K, ALIGNED>(ny, a.y, a.y_stride_bytes, nrow, voff, a.n_cols);
        load_slots_as<T, C, K, ALIGNED>(ng, a.dy, a.dy_stride_bytes, nrow, voff, a.n_cols);

        C yf[K][VEC], gf[K][VEC];
        C s[1] = {C(0)};
#pragma unroll
        for (int k = 0; k < K; ++k) {
            unpack_as<T>(cy[k], yf[k]);
            unpack_as<T>(cg[k], gf[k]);      // rows shorter than a vector: columns past the row end load as 0
            C sk = C(0);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const C ge = counts(k, e) ? gf[k][e] : C(0);
                if constexpr (LOG) sk += ge;
                else sk = fma(yf[k][e], ge, sk);
            }
            s[0] += own[k] ? sk : C(0);
        }
        row_allreduce<TPR, G, 1, OpSum, C>(s, red, phase, g, t);

        char* dxrow = a.dx + row * a.dx_stride_bytes;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            C dxf[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                C d;
                if constexpr (LOG) d = fma(-exp_c(yf[k][e]), s[0], gf[k][e]);
                else d = yf[k][e] * (gf[k][e] - s[0]);
                dxf[e] = d * sign;
            }
            store_slot_as<T, ALIGNED>(dxrow, voff[k], a.n_cols, dxf);
        }

#pragma unroll
        for (int k = 0; k < K; ++k) { cy[k] = ny[k]; cg[k] = ng[k]; }
        row_raw = nrow_raw;
        row = nrow;
    }
}

// ---------------------------------------------------------------------------------------------------
// Rows wider than 64 KiB (the reference cuts such a row into 64 KiB chunks and normalises each chunk by itself,
// softmax.py:34-40 -- which is not a softmax of the row; here the row is one softmax).  One 1024-thread workgroup
// per row, grid-stride over rows, two walks per row (thn_walk.h); the second comes from the L2 / Infinity Cache.
//   forward:  walk 1 keeps a running maximum m and sum(exp(x - m)) per thread (the sum is rescaled whenever the
//             maximum moves: a few times per thread), combined over the workgroup; walk 2 writes y;
//   backward: walk 1 sum(y*g) (log-softmax: sum(g)); walk 2 writes dx.
// The row sums are accumulated in float64.
// ---------------------------------------------------------------------------------------------------
template <typename T, bool LOG, int kSoftmaxLoopBlock>
__global__ void __launch_bounds__(kSoftmaxLoopBlock) softmax_fwd_loop_kernel(const SoftmaxFwdArgs a) {
    using C = typename SoftmaxCompute<T, LOG>::type;
    __shared__ C red[RedSmem<kSoftmaxLoopBlock, 1, 1>::kFloats];
    __shared__ double red_sum[RedSmem<kSoftmaxLoopBlock, 1, 1>::kFloats];
    int phase = 0, phase_sum = 0;
    const int t = threadIdx.x;
    const C sign = static_cast<C>(a.sign);
    const C neg_inf = OpMax::identity<C>();
    for (int64_t row = blockIdx.x; row < a.M; row += gridDim.x) {
        const char* xrow = a.x + row * a.x_stride_bytes;
        char* yrow = a.y + row * a.y_stride_bytes;
        C m = neg_inf;
        double acc = 0.0;       // tens of thousands of terms per row: float64 sums keep the row total to an ulp
        auto one = [&](C x, C, C) {
            const C v = x * sign;
            if (v > m) {
                acc *= static_cast<double>(exp_c(m - v));          // m = -inf: 0
                m = v;
            }
            acc += v > neg_inf ? static_cast<double>(exp_c(v - m)) : 0.0;   // -inf - -inf must not poison the sum
            return C(0);
        };
        walk_row_vec<T, C, kSoftmaxLoopBlock, 1, false, true, true>(
            xrow, nullptr, nullptr, nullptr, a.n_cols, t,
            [&](const C (&f)[3][T::VEC], C (&)[T::VEC]) {
                C v[T::VEC];
                C vmax = neg_inf;
#pragma unroll
                for (int e = 0; e < T::VEC; ++e) {
                    v[e] = f[0][e] * sign;
                    vmax = OpMax::apply(vmax, v[e]);
                }
                if (vmax > m) {
                    acc *= static_cast<double>(exp_c(m - vmax));
                    m = vmax;
                }
                C part = C(0);
#pragma unroll
                for (int e = 0; e < T::VEC; ++e) part += v[e] > neg_inf ? exp_c(v[e] - m) : C(0);
                acc += static_cast<double>(part);
            },
            one);
        C mx[1] = {m};
        row_allreduce<kSoftmaxLoopBlock, 1, 1, OpMax, C>(mx, red, phase, 0, t);
        double s[1] = {m > neg_inf ? acc * static_cast<double>(exp_c(m - mx[0])) : 0.0};
        row_allreduce<kSoftmaxLoopBlock, 1, 1, OpSum, double>(s, red_sum, phase_sum, 0, t);
        const C row_max = mx[0];
        C scale;
        if constexpr (LOG) scale = static_cast<C>(log(s[0]));
        else scale = static_cast<C>(1.0 / s[0]);
        walk_row<T, C, kSoftmaxLoopBlock, 1, true, false, true>(xrow, nullptr, nullptr, yrow, a.n_cols, t, [&](C x, C, C) {
            const C z = x * sign - row_max;
            if constexpr (LOG) return z - scale;
            else return exp_c(z) * scale;
        });
    }
}

template <typename T, bool LOG, int kSoftmaxLoopBlock>
__global__ void __launch_bounds__(kSoftmaxLoopBlock) softmax_bwd_loop_kernel(const SoftmaxBwdArgs a) {
    using C = typename SoftmaxCompute<T, LOG>::type;
    __shared__ double red_sum[RedSmem<kSoftmaxLoopBlock, 1, 1>::kFloats];
    int phase_sum = 0;
    const int t = threadIdx.x;
    const C sign = static_cast<C>(a.sign);
    for (int64_t row = blockIdx.x; row < a.M; row += gridDim.x) {
        const char* yrow = a.y + row * a.y_stride_bytes;
        const char* grow = a.dy + row * a.dy_stride_bytes;
        char* dxrow = a.dx + row * a.dx_stride_bytes;
        double acc = 0.0;
        walk_row_vec<T, C, kSoftmaxLoopBlock, 2, false, true, true>(
            yrow, grow, nullptr, nullptr, a.n_cols, t,
            [&](const C (&f)[3][T::VEC], C (&)[T::VEC]) {
                C part = C(0);
#pragma unroll
                for (int e = 0; e < T::VEC; ++e) {
                    if constexpr (LOG) part += f[1][e];
                    else part = fma(f[0][e], f[1][e], part);
                }
                acc += static_cast<double>(part);
            },
            [&](C y, C g, C) {
                if constexpr (LOG) acc += static_cast<double>(g);
                else acc = fma(static_cast<double>(y), static_cast<double>(g), acc);
                return C(0);
            });
        double s[1] = {acc};
        row_allreduce<kSoftmaxLoopBlock, 1, 1, OpSum, double>(s, red_sum, phase_sum, 0, t);
        const C total = static_cast<C>(s[0]);
        walk_row<T, C, kSoftmaxLoopBlock, 2, true, false, true>(yrow, grow, nullptr, dxrow, a.n_cols, t, [&](C y, C g, C) {
            C d;
            if constexpr (LOG) d = fma(-exp_c(y), total, g);
            else d = y * (g - total);
            return d * sign;
        });
    }
}

}  // namespace thn
