// Rows SHORTER than one 16-byte vector (1 to 3 float32 columns, 1 to 7 of a 16-bit type) for the softmax and the p-norm /
// normalize families: class scores over a handful of classes, 2- and 3-component vectors.  No vector slot fits such a
// row, and the row kernels' element-wise instances (ElemIo<T>) spend 32 slots of 8 lanes on it.  Here ONE LANE OWNS A
// WHOLE ROW: it loads the row's columns one element at a time (the rows being dense or evenly pitched, the 64 lanes of a
// wave cover one contiguous stretch of memory between them, so every cache line is fetched once), does the row's
// arithmetic in its own registers -- no exchange between lanes at all -- and stores the columns the same way.  J rows
// per lane and step are requested before the first is used; the grid is persistent.  The column count is uniform over
// the launch: the `c < n` tests below are scalar branches, not lane masks.
// Arithmetic as the row kernels (softmax_fwd_kernel / softmax_bwd_kernel, pnorm_fwd_kernel / pnorm_bwd_kernel /
// normalize_bwd_kernel), in float32, with the one rounding on store; float32 / float16 / bfloat16 storage.
#pragma once

#include "thn_dispatch.h"
#include "thn_pnorm.h"
#include "thn_softmax.h"

namespace thn {

constexpr int kTinyBlock = 256;
constexpr int kTinyRows = 4;        // J: rows per lane and step
constexpr int kTinyMaxCols = 7;     // one short of a 16-bit vector: the registers a lane spends on a row and stream

// Row j of this lane in the step that starts at row `base`: consecutive lanes take consecutive rows.
__device__ __forceinline__ int64_t tiny_row(int64_t base, int j, int64_t threads, int64_t last_row) {
    const int64_t r = base + static_cast<int64_t>(j) * threads;
    return r < last_row ? r : last_row;          // rows past the end mirror the last row: same inputs, same bits stored
}

template <typename T, int C>
__device__ __forceinline__ void tiny_load(const char* rowp, int n, float (&f)[C]) {
    static_assert(C <= kTinyMaxCols, "a lane holds at most kTinyMaxCols columns per row and stream");
#pragma unroll
    for (int c = 0; c < C; ++c) {
        f[c] = 0.0f;
        if (c < n) f[c] = T::load1(rowp, c);
    }
}

template <typename T, int C>
__device__ __forceinline__ void tiny_store(char* rowp, int n, const float (&f)[C]) {
#pragma unroll
    for (int c = 0; c < C; ++c) {
        if (c < n) T::store1(rowp, c, f[c]);
    }
}

template <typename T, bool LOGSM>
__global__ void __launch_bounds__(kTinyBlock) softmax_tiny_fwd_kernel(const SoftmaxFwdArgs a) {
    constexpr int C = T::VEC - 1, J = kTinyRows;
    const int n = a.n_cols;
    const int64_t threads = static_cast<int64_t>(gridDim.x) * kTinyBlock;
    const int64_t last_row = a.M - 1;
    const float neg_inf = OpMax::identity<float>();
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kTinyBlock + threadIdx.x; base < a.M; base += J * threads) {
        int64_t row[J];
        float x[J][C];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            row[j] = tiny_row(base, j, threads, last_row);
            tiny_load<T, C>(a.x + row[j] * a.x_stride_bytes, n, x[j]);
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float m = neg_inf;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                x[j][c] = c < n ? x[j][c] * a.sign : neg_inf;
                m = fmaxf(m, x[j][c]);
            }
            float s = 0.0f;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const float z = x[j][c] - m;
                const float ez = exp_c(z);              // columns past the row end: exp(-inf) = 0
                x[j][c] = LOGSM ? z : ez;
                s += ez;
            }
            const float scale = LOGSM ? logf(s) : 1.0f / s;
            float y[C];
#pragma unroll
            for (int c = 0; c < C; ++c) y[c] = LOGSM ? x[j][c] - scale : x[j][c] * scale;
            tiny_store<T, C>(a.y + row[j] * a.y_stride_bytes, n, y);
        }
    }
}

template <typename T, bool LOGSM>
__global__ void __launch_bounds__(kTinyBlock) softmax_tiny_bwd_kernel(const SoftmaxBwdArgs a) {
    constexpr int C = T::VEC - 1, J = kTinyRows;
    const int n = a.n_cols;
    const int64_t threads = static_cast<int64_t>(gridDim.x) * kTinyBlock;
    const int64_t last_row = a.M - 1;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kTinyBlock + threadIdx.x; base < a.M; base += J * threads) {
        int64_t row[J];
        float y[J][C], g[J][C];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            row[j] = tiny_row(base, j, threads, last_row);
            tiny_load<T, C>(a.y + row[j] * a.y_stride_bytes, n, y[j]);
            tiny_load<T, C>(a.dy + row[j] * a.dy_stride_bytes, n, g[j]);       // columns past the row end read as 0
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float s = 0.0f;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                if constexpr (LOGSM) s += g[j][c];
                else s = fmaf(y[j][c], g[j][c], s);
            }
            float dx[C];
#pragma unroll
            for (int c = 0; c < C; ++c) {
                float d;
                if constexpr (LOGSM) d = fmaf(-exp_c(y[j][c]), s, g[j][c]);
                else d = y[j][c] * (g[j][c] - s);
                dx[c] = d * a.sign;
            }
            tiny_store<T, C>(a.dx + row[j] * a.dx_stride_bytes, n, dx);
        }
    }
}

// p-norm family: for tensors whose rows are one folded batch (row r at r * row stride), integer p from 1 to 6.
template <typename T, int MODE, bool NORMALIZE>
__global__ void __launch_bounds__(kTinyBlock) pnorm_tiny_fwd_kernel(const PnormFwdArgs a) {
    constexpr int C = T::VEC - 1, J = kTinyRows;
    const int n = a.n_cols;
    const int64_t threads = static_cast<int64_t>(gridDim.x) * kTinyBlock;
    const int64_t last_row = a.rows - 1;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kTinyBlock + threadIdx.x; base < a.rows; base += J * threads) {
        int64_t row[J];
        float x[J][C];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            row[j] = tiny_row(base, j, threads, last_row);
            tiny_load<T, C>(a.x + row[j] * a.xmap.row_stride_bytes, n, x[j]);   // columns past the row end read as 0
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float s = 0.0f;
#pragma unroll
            for (int c = 0; c < C; ++c) s += norm_term<MODE>(x[j][c], a.p_int);
            const float nrm = fmaxf(norm_root<MODE>(s, a.p_int, a.p), a.eps);
            T::store1(a.norms, row[j], nrm);
            if constexpr (NORMALIZE) {
                const float nr = round_to_storage<T>(nrm);
                const float rn = 1.0f / nr;
                const float nd = residual_divisor(nr);
                float y[C];
#pragma unroll
                for (int c = 0; c < C; ++c) y[c] = div_by_row(x[j][c], nd, rn);
                tiny_store<T, C>(a.y + row[j] * a.ymap.row_stride_bytes, n, y);
            }
        }
    }
}

template <typename T, int MODE>
__global__ void __launch_bounds__(kTinyBlock) pnorm_tiny_bwd_kernel(const PnormBwdArgs a) {
    constexpr int C = T::VEC - 1, J = kTinyRows;
    const int n = a.n_cols;
    const int64_t threads = static_cast<int64_t>(gridDim.x) * kTinyBlock;
    const int64_t last_row = a.rows - 1;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kTinyBlock + threadIdx.x; base < a.rows; base += J * threads) {
        int64_t row[J];
        float x[J][C], c_n[J], c_g[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            row[j] = tiny_row(base, j, threads, last_row);
            tiny_load<T, C>(a.x + row[j] * a.xmap.row_stride_bytes, n, x[j]);
            c_n[j] = MODE == kP1 ? 1.0f : T::load1(a.norms, row[j]);
            c_g[j] = T::load1(a.g, row[j]);
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float den = c_n[j];
            if constexpr (MODE == kPInt) den = pow_small(c_n[j], a.p_int - 1);
            const float rden = 1.0f / den;
            den = residual_divisor(den);
            float d[C];
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const float xv = x[j][c];
                if constexpr (MODE == kP1) d[c] = c_g[j] * sign_of(xv);
                else if constexpr (MODE == kP2) d[c] = div_by_row(c_g[j] * xv, den, rden);
                else d[c] = div_by_row(c_g[j] * sign_of(xv) * pow_small(__builtin_fabsf(xv), a.p_int - 1), den, rden);
            }
            tiny_store<T, C>(a.dx + row[j] * a.dxmap.row_stride_bytes, n, d);
        }
    }
}

template <typename T, int MODE>
__global__ void __launch_bounds__(kTinyBlock) normalize_tiny_bwd_kernel(const NormalizeBwdArgs a) {
    constexpr int C = T::VEC - 1, J = kTinyRows;
    constexpr bool NEED_X = MODE != kP2;
    constexpr bool NEED_Y = MODE != kP1;
    const int n = a.n_cols;
    const int64_t threads = static_cast<int64_t>(gridDim.x) * kTinyBlock;
    const int64_t last_row = a.rows - 1;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kTinyBlock + threadIdx.x; base < a.rows; base += J * threads) {
        int64_t row[J];
        float x[NEED_X ? J : 1][C], y[NEED_Y ? J : 1][C], g[J][C], c_n[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            row[j] = tiny_row(base, j, threads, last_row);
            if constexpr (NEED_X) tiny_load<T, C>(a.x + row[j] * a.xmap.row_stride_bytes, n, x[j]);
            if constexpr (NEED_Y) tiny_load<T, C>(a.y + row[j] * a.ymap.row_stride_bytes, n, y[j]);
            tiny_load<T, C>(a.g + row[j] * a.gmap.row_stride_bytes, n, g[j]);  // columns past the row end read as 0
            c_n[j] = T::load1(a.norms, row[j]);
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float proj = 0.0f;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                if constexpr (MODE == kP1) proj = __builtin_fmaf(x[j][c], g[j][c], proj);
                else proj = __builtin_fmaf(y[j][c], g[j][c], proj);
            }
            const float nrm = c_n[j];
            const float rn = 1.0f / nrm;
            const float nd = residual_divisor(nrm);
            float coef = 0.0f;
            if constexpr (MODE == kP1) coef = proj / (nrm * nrm);
            if constexpr (MODE == kPInt) coef = proj / (pow_small(nrm, a.p_int - 1) * nrm);
            float d[C];
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const float gg = g[j][c];
                if constexpr (MODE == kP2) {
                    d[c] = div_by_row(gg - y[j][c] * proj, nd, rn);
                } else if constexpr (MODE == kP1) {
                    d[c] = div_by_row(gg, nd, rn) - sign_of(x[j][c]) * coef;
                } else {
                    const float xv = x[j][c];
                    d[c] = div_by_row(gg, nd, rn) - sign_of(xv) * pow_small(__builtin_fabsf(xv), a.p_int - 1) * coef;
                }
            }
            tiny_store<T, C>(a.dx + row[j] * a.dxmap.row_stride_bytes, n, d);
        }
    }
}

// Launchers: 0 launched, 1 no such instance, <0 HIP error.  `mode`: kP1 / kP2 / kPInt.
#define THN_DECLARE_TINY_LAUNCHERS(NAME)                                                                        \
    int launch_softmax_tiny_fwd_##NAME(bool is_log, const SoftmaxFwdArgs& a, int grid, hipStream_t st);         \
    int launch_softmax_tiny_bwd_##NAME(bool is_log, const SoftmaxBwdArgs& a, int grid, hipStream_t st);         \
    int launch_pnorm_tiny_fwd_##NAME(int mode, bool normalize, const PnormFwdArgs& a, int grid, hipStream_t st); \
    int launch_pnorm_tiny_bwd_##NAME(int mode, const PnormBwdArgs& a, int grid, hipStream_t st);                \
    int launch_normalize_tiny_bwd_##NAME(int mode, const NormalizeBwdArgs& a, int grid, hipStream_t st);

THN_DECLARE_TINY_LAUNCHERS(f32)
THN_DECLARE_TINY_LAUNCHERS(f16)
THN_DECLARE_TINY_LAUNCHERS(bf16)

#define THN_TINY_MODE_CASE(KERNEL, ARGS_T, MODE_)                                                               \
    if (mode == MODE_) return run_kernel<ARGS_T>(KERNEL<T, MODE_>, a, grid, kTinyBlock, st, nullptr);
#define THN_TINY_FWD_MODE_CASE(MODE_)                                                                           \
    if (mode == MODE_) {                                                                                        \
        return normalize ? run_kernel<PnormFwdArgs>(pnorm_tiny_fwd_kernel<T, MODE_, true>, a, grid, kTinyBlock, st, nullptr)  \
                         : run_kernel<PnormFwdArgs>(pnorm_tiny_fwd_kernel<T, MODE_, false>, a, grid, kTinyBlock, st, nullptr); \
    }

#define THN_DEFINE_TINY_LAUNCHERS(NAME, TYPE)                                                                   \
    int launch_softmax_tiny_fwd_##NAME(bool is_log, const SoftmaxFwdArgs& a, int grid, hipStream_t st) {        \
        using T = TYPE;                                                                                         \
        return is_log ? run_kernel<SoftmaxFwdArgs>(softmax_tiny_fwd_kernel<T, true>, a, grid, kTinyBlock, st, nullptr)   \
                      : run_kernel<SoftmaxFwdArgs>(softmax_tiny_fwd_kernel<T, false>, a, grid, kTinyBlock, st, nullptr); \
    }                                                                                                           \
    int launch_softmax_tiny_bwd_##NAME(bool is_log, const SoftmaxBwdArgs& a, int grid, hipStream_t st) {        \
        using T = TYPE;                                                                                         \
        return is_log ? run_kernel<SoftmaxBwdArgs>(softmax_tiny_bwd_kernel<T, true>, a, grid, kTinyBlock, st, nullptr)   \
                      : run_kernel<SoftmaxBwdArgs>(softmax_tiny_bwd_kernel<T, false>, a, grid, kTinyBlock, st, nullptr); \
    }                                                                                                           \
    int launch_pnorm_tiny_fwd_##NAME(int mode, bool normalize, const PnormFwdArgs& a, int grid, hipStream_t st) { \
        using T = TYPE;                                                                                         \
        THN_TINY_FWD_MODE_CASE(kP1) THN_TINY_FWD_MODE_CASE(kP2) THN_TINY_FWD_MODE_CASE(kPInt)                   \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_pnorm_tiny_bwd_##NAME(int mode, const PnormBwdArgs& a, int grid, hipStream_t st) {               \
        using T = TYPE;                                                                                         \
        THN_TINY_MODE_CASE(pnorm_tiny_bwd_kernel, PnormBwdArgs, kP1)                                            \
        THN_TINY_MODE_CASE(pnorm_tiny_bwd_kernel, PnormBwdArgs, kP2)                                            \
        THN_TINY_MODE_CASE(pnorm_tiny_bwd_kernel, PnormBwdArgs, kPInt)                                          \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_normalize_tiny_bwd_##NAME(int mode, const NormalizeBwdArgs& a, int grid, hipStream_t st) {       \
        using T = TYPE;                                                                                         \
        THN_TINY_MODE_CASE(normalize_tiny_bwd_kernel, NormalizeBwdArgs, kP1)                                    \
        THN_TINY_MODE_CASE(normalize_tiny_bwd_kernel, NormalizeBwdArgs, kP2)                                    \
        THN_TINY_MODE_CASE(normalize_tiny_bwd_kernel, NormalizeBwdArgs, kPInt)                                  \
        return 1;                                                                                               \
    }

}  // namespace thn
