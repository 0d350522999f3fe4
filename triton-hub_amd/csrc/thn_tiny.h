// Rows SHORTER than one 16-byte vector (1 to 3 float32 columns, 1 to 7 of a 16-bit type) for the norm kernels, the softmax
// and the p-norm / normalize families: class scores over a handful of classes, 2- and 3-component vectors.  No vector slot fits such a
// row, and the row kernels' element-wise instances (ElemIo<T>) spend 32 slots of 8 lanes on it.  Here ONE LANE OWNS A
// WHOLE ROW: it loads the row's columns one element at a time (the rows being dense or evenly pitched, the 64 lanes of a
// wave cover one contiguous stretch of memory between them, so every cache line is fetched once), does the row's
// arithmetic in its own registers -- no exchange between lanes at all -- and stores the columns the same way.  J rows
// per lane and step are requested before the first is used; the grid is persistent.  The column count is uniform over
// the launch: the `c < n` tests below are scalar branches, not lane masks.  Dense rows behind aligned pointers go through
// LDS in whole vectors instead (TinyStage below).
// Arithmetic as the row kernels (norm_fwd_kernel / norm_bwd_kernel, softmax_fwd_kernel / softmax_bwd_kernel,
// pnorm_fwd_kernel / pnorm_bwd_kernel / normalize_bwd_kernel), in float32, with the one rounding on store; float32 /
// float16 / bfloat16 storage.
#pragma once

#include "thn_dispatch.h"
#include "thn_pnorm.h"
#include "thn_softmax.h"
#include "thn_staged.h"

namespace thn {

constexpr int kTinyBlock = 256;
constexpr int kTinyRows = 4;        // J: rows per lane and step
constexpr int kTinyMaxCols = 7;     // one short of a 16-bit vector: the registers a lane spends on a row and stream
constexpr int kTinyStageBytes = 1024;   // LDS per wave, stream and batch of 64 rows: 64 x 16 bytes

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

// STAGED: dense rows (row r at r * n elements) behind 16-byte aligned pointers.  The 64 rows of a wave and step are then
// one aligned stretch of 64 * n elements = 4 * n * (bytes per element) vectors: the wave fetches it with one 16-byte load
// per lane, spreads it through LDS, from where every lane picks up the columns of its row, and sends the results back
// the same way -- the memory system sees whole vectors instead of 64 two- or four-byte pieces per instruction (a wave's
// two-byte store is seven partial lines).  The last, incomplete batch of 64 rows of a tensor takes the element accesses.
template <typename T, int C>
struct TinyStage {
    // The wave's stretch of stream `base`, one vector per lane (lanes past its end repeat the last vector).
    __device__ static __forceinline__ u32x4 fetch(const char* base, int64_t row0, int n, int lane, bool keep) {
        const int vecs = 4 * n * T::kBytes;
        const char* p = base + row0 * n * T::kBytes + 16 * (lane < vecs ? lane : vecs - 1);
        return keep ? ld128_keep(p) : ld128(p);
    }
    __device__ static __forceinline__ void spread(u32x4 v, char* lds, int n, int lane, float (&f)[C]) {
        *reinterpret_cast<u32x4*>(lds + 16 * lane) = v;
        wave_sync();
#pragma unroll
        for (int c = 0; c < C; ++c) {
            f[c] = 0.0f;
            if (c < n) f[c] = T::load1(lds, lane * n + c);
        }
    }
    // The lanes' results back through the same LDS (every lane has read its inputs from it: spread() of this batch came
    // before in program order, and a wave executes its LDS instructions in order).
    __device__ static __forceinline__ void collect_store(char* base, int64_t row0, char* lds, int n, int lane,
                                                         const float (&f)[C], bool keep) {
        wave_sync();
#pragma unroll
        for (int c = 0; c < C; ++c) {
            if (c < n) T::store1(lds, lane * n + c, f[c]);
        }
        wave_sync();
        const int vecs = 4 * n * T::kBytes;
        const int l = lane < vecs ? lane : vecs - 1;
        const u32x4 v = *reinterpret_cast<const u32x4*>(lds + 16 * l);
        char* p = base + row0 * n * T::kBytes + 16 * l;
        if (keep) st128_keep(p, v);
        else st128(p, v);
    }
};

// First row of the wave's batch j in the step that starts at `base` for this lane, and whether all 64 rows exist.
__device__ __forceinline__ int64_t tiny_row0(int64_t base, int j, int64_t threads, int lane) {
    return base - lane + static_cast<int64_t>(j) * threads;
}

// One stream of a step: J batches of rows, fetched first (staged: one vector per lane and batch; otherwise the elements
// themselves), handed out batch by batch.
template <typename T, int C, bool STAGED>
struct TinyIn {
    u32x4 v[STAGED ? kTinyRows : 1];
    float f[STAGED ? 1 : kTinyRows][C];
    __device__ __forceinline__ void request(const char* base, int64_t stride_bytes, const int64_t (&row)[kTinyRows],
                                            const int64_t (&row0)[kTinyRows], const bool (&whole)[kTinyRows], int n,
                                            int lane, bool keep = false) {
#pragma unroll
        for (int j = 0; j < kTinyRows; ++j) {
            if constexpr (STAGED) {
                if (whole[j]) v[j] = TinyStage<T, C>::fetch(base, row0[j], n, lane, keep);
            } else {
                tiny_load<T, C>(base + row[j] * stride_bytes, n, f[j]);
            }
        }
    }
    // The columns of this lane's row of batch j (staged: through `lds`; an incomplete batch by element loads).
    __device__ __forceinline__ void take(int j, const char* base, int64_t stride_bytes, int64_t row, bool whole, int n,
                                         int lane, char* lds, float (&out)[C]) {
        if constexpr (STAGED) {
            if (whole) TinyStage<T, C>::spread(v[j], lds, n, lane, out);
            else tiny_load<T, C>(base + row * stride_bytes, n, out);
        } else {
#pragma unroll
            for (int c = 0; c < C; ++c) out[c] = f[j][c];
        }
    }
};

template <typename T, int C, bool STAGED>
__device__ __forceinline__ void tiny_out(char* base, int64_t stride_bytes, int64_t row, int64_t row0, bool whole, int n,
                                         int lane, char* lds, const float (&f)[C], bool keep = false) {
    if constexpr (STAGED) {
        if (whole) {
            TinyStage<T, C>::collect_store(base, row0, lds, n, lane, f, keep);
            return;
        }
    }
    tiny_store<T, C>(base + row * stride_bytes, n, f);
}

// The rows of this lane in one step, the first row of each of its wave's batches, and whether a batch is complete.
#define THN_TINY_STEP_ROWS(M_)                                                                                  \
    int64_t row[J], row0[J];                                                                                    \
    bool whole[J];                                                                                              \
    _Pragma("unroll") for (int j = 0; j < J; ++j) {                                                             \
        row[j] = tiny_row(base, j, threads, last_row);                                                          \
        row0[j] = tiny_row0(base, j, threads, lane);                                                            \
        whole[j] = row0[j] + 64 <= (M_);                                                                        \
    }

template <typename T, bool LOGSM, bool STAGED>
__global__ void __launch_bounds__(kTinyBlock) softmax_tiny_fwd_kernel(const SoftmaxFwdArgs a) {
    constexpr int C = T::VEC - 1, J = kTinyRows;
    __shared__ __align__(16) char stage[STAGED ? (kTinyBlock / 64) * kTinyStageBytes : 16];
    const int n = a.n_cols;
    const int lane = threadIdx.x & 63;
    char* lds = stage + (STAGED ? (threadIdx.x >> 6) * kTinyStageBytes : 0);
    const int64_t threads = static_cast<int64_t>(gridDim.x) * kTinyBlock;
    const int64_t last_row = a.M - 1;
    const float neg_inf = OpMax::identity<float>();
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kTinyBlock + threadIdx.x; base - lane < a.M; base += J * threads) {
        THN_TINY_STEP_ROWS(a.M)
        TinyIn<T, C, STAGED> in;
        in.request(a.x, a.x_stride_bytes, row, row0, whole, n, lane);
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float x[C];
            in.take(j, a.x, a.x_stride_bytes, row[j], whole[j], n, lane, lds, x);
            float m = neg_inf;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                x[c] = c < n ? x[c] * a.sign : neg_inf;
                m = fmaxf(m, x[c]);
            }
            float s = 0.0f;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const float z = x[c] - m;
                const float ez = exp_c(z);              // columns past the row end: exp(-inf) = 0
                x[c] = LOGSM ? z : ez;
                s += ez;
            }
            const float scale = LOGSM ? logf(s) : 1.0f / s;
            float y[C];
#pragma unroll
            for (int c = 0; c < C; ++c) y[c] = LOGSM ? x[c] - scale : x[c] * scale;
            tiny_out<T, C, STAGED>(a.y, a.y_stride_bytes, row[j], row0[j], whole[j], n, lane, lds, y, true);
        }
    }
}

template <typename T, bool LOGSM, bool STAGED>
__global__ void __launch_bounds__(kTinyBlock) softmax_tiny_bwd_kernel(const SoftmaxBwdArgs a) {
    constexpr int C = T::VEC - 1, J = kTinyRows;
    __shared__ __align__(16) char stage[STAGED ? 2 * (kTinyBlock / 64) * kTinyStageBytes : 16];
    const int n = a.n_cols;
    const int lane = threadIdx.x & 63;
    char* lds = stage + (STAGED ? (threadIdx.x >> 6) * 2 * kTinyStageBytes : 0);
    const int64_t threads = static_cast<int64_t>(gridDim.x) * kTinyBlock;
    const int64_t last_row = a.M - 1;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kTinyBlock + threadIdx.x; base - lane < a.M; base += J * threads) {
        THN_TINY_STEP_ROWS(a.M)
        TinyIn<T, C, STAGED> iy, ig;
        iy.request(a.y, a.y_stride_bytes, row, row0, whole, n, lane);
        ig.request(a.dy, a.dy_stride_bytes, row, row0, whole, n, lane);
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float y[C], g[C];
            iy.take(j, a.y, a.y_stride_bytes, row[j], whole[j], n, lane, lds, y);
            ig.take(j, a.dy, a.dy_stride_bytes, row[j], whole[j], n, lane, lds + (STAGED ? kTinyStageBytes : 0), g);
            float s = 0.0f;                              // columns past the row end read as 0
#pragma unroll
            for (int c = 0; c < C; ++c) {
                if constexpr (LOGSM) s += g[c];
                else s = fmaf(y[c], g[c], s);
            }
            float dx[C];
#pragma unroll
            for (int c = 0; c < C; ++c) {
                float d;
                if constexpr (LOGSM) d = fmaf(-exp_c(y[c]), s, g[c]);
                else d = y[c] * (g[c] - s);
                dx[c] = d * a.sign;
            }
            tiny_out<T, C, STAGED>(a.dx, a.dx_stride_bytes, row[j], row0[j], whole[j], n, lane, lds, dx);
        }
    }
}

// p-norm family: for tensors whose rows are one folded batch (row r at r * row stride), integer p from 1 to 6.
template <typename T, int MODE, bool NORMALIZE, bool STAGED>
__global__ void __launch_bounds__(kTinyBlock) pnorm_tiny_fwd_kernel(const PnormFwdArgs a) {
    constexpr int C = T::VEC - 1, J = kTinyRows;
    constexpr bool kKeepY = NORMALIZE && MODE == kP2;      // what the backward reads again stays in the caches
    __shared__ __align__(16) char stage[STAGED ? (kTinyBlock / 64) * kTinyStageBytes : 16];
    const int n = a.n_cols;
    const int lane = threadIdx.x & 63;
    char* lds = stage + (STAGED ? (threadIdx.x >> 6) * kTinyStageBytes : 0);
    const int64_t threads = static_cast<int64_t>(gridDim.x) * kTinyBlock;
    const int64_t last_row = a.rows - 1;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kTinyBlock + threadIdx.x; base - lane < a.rows; base += J * threads) {
        THN_TINY_STEP_ROWS(a.rows)
        TinyIn<T, C, STAGED> in;
        in.request(a.x, a.xmap.row_stride_bytes, row, row0, whole, n, lane, !kKeepY);
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float x[C];
            in.take(j, a.x, a.xmap.row_stride_bytes, row[j], whole[j], n, lane, lds, x);
            float s = 0.0f;                              // columns past the row end read as 0
#pragma unroll
            for (int c = 0; c < C; ++c) s += norm_term<MODE>(x[c], a.p_int);
            const float nrm = fmaxf(norm_root<MODE>(s, a.p_int, a.p), a.eps);
            T::store1(a.norms, row[j], nrm);
            if constexpr (NORMALIZE) {
                const float nr = round_to_storage<T>(nrm);
                const float rn = 1.0f / nr;
                const float nd = residual_divisor(nr);
                float y[C];
#pragma unroll
                for (int c = 0; c < C; ++c) y[c] = div_by_row(x[c], nd, rn);
                tiny_out<T, C, STAGED>(a.y, a.ymap.row_stride_bytes, row[j], row0[j], whole[j], n, lane, lds, y, kKeepY);
            }
        }
    }
}

template <typename T, int MODE, bool STAGED>
__global__ void __launch_bounds__(kTinyBlock) pnorm_tiny_bwd_kernel(const PnormBwdArgs a) {
    constexpr int C = T::VEC - 1, J = kTinyRows;
    __shared__ __align__(16) char stage[STAGED ? (kTinyBlock / 64) * kTinyStageBytes : 16];
    const int n = a.n_cols;
    const int lane = threadIdx.x & 63;
    char* lds = stage + (STAGED ? (threadIdx.x >> 6) * kTinyStageBytes : 0);
    const int64_t threads = static_cast<int64_t>(gridDim.x) * kTinyBlock;
    const int64_t last_row = a.rows - 1;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kTinyBlock + threadIdx.x; base - lane < a.rows; base += J * threads) {
        THN_TINY_STEP_ROWS(a.rows)
        TinyIn<T, C, STAGED> in;
        in.request(a.x, a.xmap.row_stride_bytes, row, row0, whole, n, lane);
        float c_n[J], c_g[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            c_n[j] = MODE == kP1 ? 1.0f : T::load1(a.norms, row[j]);
            c_g[j] = T::load1(a.g, row[j]);
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float x[C];
            in.take(j, a.x, a.xmap.row_stride_bytes, row[j], whole[j], n, lane, lds, x);
            float den = c_n[j];
            if constexpr (MODE == kPInt) den = pow_small(c_n[j], a.p_int - 1);
            const float rden = 1.0f / den;
            den = residual_divisor(den);
            float d[C];
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const float xv = x[c];
                if constexpr (MODE == kP1) d[c] = c_g[j] * sign_of(xv);
                else if constexpr (MODE == kP2) d[c] = div_by_row(c_g[j] * xv, den, rden);
                else d[c] = div_by_row(c_g[j] * sign_of(xv) * pow_small(__builtin_fabsf(xv), a.p_int - 1), den, rden);
            }
            tiny_out<T, C, STAGED>(a.dx, a.dxmap.row_stride_bytes, row[j], row0[j], whole[j], n, lane, lds, d);
        }
    }
}

template <typename T, int MODE, bool STAGED>
__global__ void __launch_bounds__(kTinyBlock) normalize_tiny_bwd_kernel(const NormalizeBwdArgs a) {
    constexpr int C = T::VEC - 1, J = kTinyRows;
    constexpr bool NEED_X = MODE != kP2;
    constexpr bool NEED_Y = MODE != kP1;
    __shared__ __align__(16) char stage[STAGED ? 3 * (kTinyBlock / 64) * kTinyStageBytes : 16];
    const int n = a.n_cols;
    const int lane = threadIdx.x & 63;
    char* lds = stage + (STAGED ? (threadIdx.x >> 6) * 3 * kTinyStageBytes : 0);
    const int64_t threads = static_cast<int64_t>(gridDim.x) * kTinyBlock;
    const int64_t last_row = a.rows - 1;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kTinyBlock + threadIdx.x; base - lane < a.rows; base += J * threads) {
        THN_TINY_STEP_ROWS(a.rows)
        TinyIn<T, C, STAGED> ix, iy, ig;
        if constexpr (NEED_X) ix.request(a.x, a.xmap.row_stride_bytes, row, row0, whole, n, lane);
        if constexpr (NEED_Y) iy.request(a.y, a.ymap.row_stride_bytes, row, row0, whole, n, lane);
        ig.request(a.g, a.gmap.row_stride_bytes, row, row0, whole, n, lane);
        float c_n[J];
#pragma unroll
        for (int j = 0; j < J; ++j) c_n[j] = T::load1(a.norms, row[j]);
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float x[C], y[C], g[C];
            if constexpr (NEED_X) ix.take(j, a.x, a.xmap.row_stride_bytes, row[j], whole[j], n, lane, lds, x);
            if constexpr (NEED_Y) iy.take(j, a.y, a.ymap.row_stride_bytes, row[j], whole[j], n, lane, lds + (STAGED ? kTinyStageBytes : 0), y);
            ig.take(j, a.g, a.gmap.row_stride_bytes, row[j], whole[j], n, lane, lds + (STAGED ? 2 * kTinyStageBytes : 0), g);
            float proj = 0.0f;                           // columns past the row end read as 0
#pragma unroll
            for (int c = 0; c < C; ++c) {
                if constexpr (MODE == kP1) proj = __builtin_fmaf(x[c], g[c], proj);
                else proj = __builtin_fmaf(y[c], g[c], proj);
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
                const float gg = g[c];
                if constexpr (MODE == kP2) {
                    d[c] = div_by_row(gg - y[c] * proj, nd, rn);
                } else if constexpr (MODE == kP1) {
                    d[c] = div_by_row(gg, nd, rn) - sign_of(x[c]) * coef;
                } else {
                    const float xv = x[c];
                    d[c] = div_by_row(gg, nd, rn) - sign_of(xv) * pow_small(__builtin_fabsf(xv), a.p_int - 1) * coef;
                }
            }
            tiny_out<T, C, STAGED>(a.dx, a.dxmap.row_stride_bytes, row[j], row0[j], whole[j], n, lane, lds + (STAGED ? 2 * kTinyStageBytes : 0), d);
        }
    }
}

// LayerNorm / RMSNorm over rows shorter than one vector.  Arithmetic as norm_fwd_kernel / norm_bwd_kernel (LayerNorm:
// mean0, then {sum d, sum d^2} with the delta correction; the backward's {sum u*wdy, sum wdy, sum u}); the weights and
// the bias are launch-uniform values every lane loads once.  dW / dB: per-lane column sums (float64 for float32 rows),
// added up by the workgroup at the end, in a fixed order, into ONE float32 partial row (the second stage is the row
// kernels').
template <typename T, bool LN, bool STAGED>
__global__ void __launch_bounds__(kTinyBlock) norm_tiny_fwd_kernel(const FwdArgs a) {
    constexpr int C = T::VEC - 1, J = kTinyRows;
    __shared__ __align__(16) char stage[STAGED ? (kTinyBlock / 64) * kTinyStageBytes : 16];
    const int n = a.n_cols;
    const int lane = threadIdx.x & 63;
    char* lds = stage + (STAGED ? (threadIdx.x >> 6) * kTinyStageBytes : 0);
    const int64_t threads = static_cast<int64_t>(gridDim.x) * kTinyBlock;
    const int64_t last_row = a.M - 1;
    float wr[1][T::VEC], br[1][T::VEC];
    const int first[1] = {0};
    load_params_clamped<1, T::VEC, false>(wr, a.w, a.w_dtype, first, n, 1.0f);
    load_params_clamped<1, T::VEC, false>(br, LN ? a.b : nullptr, a.w_dtype, first, n, 0.0f);
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kTinyBlock + threadIdx.x; base - lane < a.M; base += J * threads) {
        THN_TINY_STEP_ROWS(a.M)
        TinyIn<T, C, STAGED> in;
        in.request(a.x, a.x_stride_bytes, row, row0, whole, n, lane, a.keep_x != 0);
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float x[C];
            in.take(j, a.x, a.x_stride_bytes, row[j], whole[j], n, lane, lds, x);   // columns past the row end read as 0
            float mean = 0.0f, delta = 0.0f, rstd;
            if constexpr (LN) {
                float s = 0.0f;
#pragma unroll
                for (int c = 0; c < C; ++c) s += x[c];
                const float mean0 = s * a.inv_n;
                float q0 = 0.0f, q1 = 0.0f;
#pragma unroll
                for (int c = 0; c < C; ++c) {
                    const float d = x[c] - mean0;
                    x[c] = d;
                    const float dm = c < n ? d : 0.0f;
                    q0 += dm;
                    q1 = fmaf(dm, dm, q1);
                }
                delta = q0 * a.inv_n;
                const float var = fmaxf(fmaf(-delta, delta, q1 * a.inv_n), 0.0f);
                rstd = rsqrt_refined(var + a.eps);
                mean = mean0 + delta;
            } else {
                float q = 0.0f;
#pragma unroll
                for (int c = 0; c < C; ++c) q = fmaf(x[c], x[c], q);
                rstd = rsqrt_refined(fmaf(q, a.inv_n, a.eps));
            }
            float y[C];
#pragma unroll
            for (int c = 0; c < C; ++c) {
                if constexpr (LN) y[c] = fmaf((x[c] - delta) * rstd, wr[0][c], br[0][c]);
                else y[c] = x[c] * rstd * wr[0][c];
            }
            tiny_out<T, C, STAGED>(a.y, a.y_stride_bytes, row[j], row0[j], whole[j], n, lane, lds, y);
            if constexpr (LN) a.mean[row[j]] = mean;
            a.rstd[row[j]] = rstd;
        }
    }
}

template <typename T, bool LN, bool STAGED>
__global__ void __launch_bounds__(kTinyBlock) norm_tiny_bwd_kernel(const BwdArgs a) {
    constexpr int C = T::VEC - 1, J = kTinyRows;
    using Acc = typename AccType<(T::kBytes >= 4)>::type;
    __shared__ __align__(16) char stage[STAGED ? 2 * (kTinyBlock / 64) * kTinyStageBytes : 16];
    __shared__ Acc totals[2][kTinyBlock][C];             // [dW | dB][thread][column]
    const int n = a.n_cols;
    const int lane = threadIdx.x & 63;
    char* lds = stage + (STAGED ? (threadIdx.x >> 6) * 2 * kTinyStageBytes : 0);
    const int64_t threads = static_cast<int64_t>(gridDim.x) * kTinyBlock;
    const int64_t last_row = a.M - 1;
    float wr[1][T::VEC];
    const int first[1] = {0};
    load_params_clamped<1, T::VEC, false>(wr, a.w, a.w_dtype, first, n, 1.0f);
    Acc dw[C], db[C];
#pragma unroll
    for (int c = 0; c < C; ++c) { dw[c] = Acc(0); db[c] = Acc(0); }
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kTinyBlock + threadIdx.x; base - lane < a.M; base += J * threads) {
        THN_TINY_STEP_ROWS(a.M)
        TinyIn<T, C, STAGED> ix, ig;
        ix.request(a.x, a.x_stride_bytes, row, row0, whole, n, lane);
        ig.request(a.dy, a.dy_stride_bytes, row, row0, whole, n, lane);
        float c_mean[J], c_rstd[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            c_mean[j] = LN ? a.mean[row[j]] : 0.0f;
            c_rstd[j] = a.rstd[row[j]];
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float u[C], g[C], wdy[C];
            ix.take(j, a.x, a.x_stride_bytes, row[j], whole[j], n, lane, lds, u);
            ig.take(j, a.dy, a.dy_stride_bytes, row[j], whole[j], n, lane, lds + (STAGED ? kTinyStageBytes : 0), g);
            float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                if constexpr (LN) u[c] = c < n ? (u[c] - c_mean[j]) * c_rstd[j] : 0.0f;
                else u[c] *= c_rstd[j];
                wdy[c] = wr[0][c] * g[c];                 // columns past the row end: g reads as 0
                s0 = fmaf(u[c], wdy[c], s0);
                if constexpr (LN) {
                    s1 += wdy[c];
                    s2 += u[c];
                }
            }
            float c1, c2 = 0.0f, dlt = 0.0f;
            if constexpr (LN) {
                dlt = s2 * a.inv_n;
                c2 = s1 * a.inv_n;
                c1 = fmaf(-dlt, c2, s0 * a.inv_n);
            } else {
                c1 = s0 * a.inv_n;
            }
            const bool adds = base + static_cast<int64_t>(j) * threads < a.M;      // a row past the end adds nothing to dW / dB
            float dx[C];
#pragma unroll
            for (int c = 0; c < C; ++c) {
                float xhat = u[c];
                if constexpr (LN) xhat -= dlt;
                dx[c] = (wdy[c] - fmaf(xhat, c1, c2)) * c_rstd[j];
                const float gl = adds ? g[c] : 0.0f;
                dw[c] = fma(static_cast<Acc>(gl), static_cast<Acc>(xhat), dw[c]);
                if constexpr (LN) db[c] += static_cast<Acc>(gl);
            }
            tiny_out<T, C, STAGED>(a.dx, a.dx_stride_bytes, row[j], row0[j], whole[j], n, lane, lds, dx);
        }
    }
    // The workgroup's partial row: one thread per column adds the threads' sums in thread order.
    const bool want_dw = a.dw_part != nullptr;
    const bool want_db = LN && a.db_part != nullptr;
#pragma unroll
    for (int c = 0; c < C; ++c) {
        totals[0][threadIdx.x][c] = dw[c];
        totals[1][threadIdx.x][c] = LN ? db[c] : Acc(0);
    }
    __syncthreads();
    if (threadIdx.x < n) {
        Acc sw = Acc(0), sb = Acc(0);
        for (int t = 0; t < kTinyBlock; ++t) {
            sw += totals[0][t][threadIdx.x];
            sb += totals[1][t][threadIdx.x];
        }
        const int64_t off = static_cast<int64_t>(blockIdx.x) * a.part_pitch + threadIdx.x;
        if (want_dw) a.dw_part[off] = static_cast<float>(sw);
        if (want_db) a.db_part[off] = static_cast<float>(sb);
    }
}

// Launchers: 0 launched, 1 no such instance, <0 HIP error.  `mode`: kP1 / kP2 / kPInt; `staged`: every stream is dense
// (row r at r * n elements) behind a 16-byte aligned pointer.
#define THN_DECLARE_TINY_LAUNCHERS(NAME)                                                                        \
    int launch_softmax_tiny_fwd_##NAME(bool is_log, bool staged, const SoftmaxFwdArgs& a, int grid, hipStream_t st); \
    int launch_softmax_tiny_bwd_##NAME(bool is_log, bool staged, const SoftmaxBwdArgs& a, int grid, hipStream_t st); \
    int launch_pnorm_tiny_fwd_##NAME(int mode, bool normalize, bool staged, const PnormFwdArgs& a, int grid, hipStream_t st); \
    int launch_pnorm_tiny_bwd_##NAME(int mode, bool staged, const PnormBwdArgs& a, int grid, hipStream_t st);   \
    int launch_normalize_tiny_bwd_##NAME(int mode, bool staged, const NormalizeBwdArgs& a, int grid, hipStream_t st); \
    int launch_norm_tiny_fwd_##NAME(bool ln, bool staged, const FwdArgs& a, int grid, hipStream_t st);          \
    int launch_norm_tiny_bwd_##NAME(bool ln, bool staged, const BwdArgs& a, int grid, hipStream_t st);

THN_DECLARE_TINY_LAUNCHERS(f32)
THN_DECLARE_TINY_LAUNCHERS(f16)
THN_DECLARE_TINY_LAUNCHERS(bf16)

#define THN_TINY_RUN(ARGS_T, KERNEL, ...)                                                                       \
    (staged ? run_kernel<ARGS_T>(KERNEL<T, __VA_ARGS__, true>, a, grid, kTinyBlock, st, nullptr)                \
            : run_kernel<ARGS_T>(KERNEL<T, __VA_ARGS__, false>, a, grid, kTinyBlock, st, nullptr))
#define THN_TINY_MODE_CASE(KERNEL, ARGS_T, MODE_)                                                               \
    if (mode == MODE_) return THN_TINY_RUN(ARGS_T, KERNEL, MODE_);
#define THN_TINY_FWD_MODE_CASE(MODE_)                                                                           \
    if (mode == MODE_) {                                                                                        \
        return normalize ? THN_TINY_RUN(PnormFwdArgs, pnorm_tiny_fwd_kernel, MODE_, true)                       \
                         : THN_TINY_RUN(PnormFwdArgs, pnorm_tiny_fwd_kernel, MODE_, false);                     \
    }

#define THN_DEFINE_TINY_LAUNCHERS(NAME, TYPE)                                                                   \
    int launch_softmax_tiny_fwd_##NAME(bool is_log, bool staged, const SoftmaxFwdArgs& a, int grid, hipStream_t st) { \
        using T = TYPE;                                                                                         \
        return is_log ? THN_TINY_RUN(SoftmaxFwdArgs, softmax_tiny_fwd_kernel, true)                             \
                      : THN_TINY_RUN(SoftmaxFwdArgs, softmax_tiny_fwd_kernel, false);                           \
    }                                                                                                           \
    int launch_softmax_tiny_bwd_##NAME(bool is_log, bool staged, const SoftmaxBwdArgs& a, int grid, hipStream_t st) { \
        using T = TYPE;                                                                                         \
        return is_log ? THN_TINY_RUN(SoftmaxBwdArgs, softmax_tiny_bwd_kernel, true)                             \
                      : THN_TINY_RUN(SoftmaxBwdArgs, softmax_tiny_bwd_kernel, false);                           \
    }                                                                                                           \
    int launch_pnorm_tiny_fwd_##NAME(int mode, bool normalize, bool staged, const PnormFwdArgs& a, int grid,    \
                                     hipStream_t st) {                                                          \
        using T = TYPE;                                                                                         \
        THN_TINY_FWD_MODE_CASE(kP1) THN_TINY_FWD_MODE_CASE(kP2) THN_TINY_FWD_MODE_CASE(kPInt)                   \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_pnorm_tiny_bwd_##NAME(int mode, bool staged, const PnormBwdArgs& a, int grid, hipStream_t st) {  \
        using T = TYPE;                                                                                         \
        THN_TINY_MODE_CASE(pnorm_tiny_bwd_kernel, PnormBwdArgs, kP1)                                            \
        THN_TINY_MODE_CASE(pnorm_tiny_bwd_kernel, PnormBwdArgs, kP2)                                            \
        THN_TINY_MODE_CASE(pnorm_tiny_bwd_kernel, PnormBwdArgs, kPInt)                                          \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_normalize_tiny_bwd_##NAME(int mode, bool staged, const NormalizeBwdArgs& a, int grid, hipStream_t st) { \
        using T = TYPE;                                                                                         \
        THN_TINY_MODE_CASE(normalize_tiny_bwd_kernel, NormalizeBwdArgs, kP1)                                    \
        THN_TINY_MODE_CASE(normalize_tiny_bwd_kernel, NormalizeBwdArgs, kP2)                                    \
        THN_TINY_MODE_CASE(normalize_tiny_bwd_kernel, NormalizeBwdArgs, kPInt)                                  \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_norm_tiny_fwd_##NAME(bool ln, bool staged, const FwdArgs& a, int grid, hipStream_t st) {         \
        using T = TYPE;                                                                                         \
        return ln ? THN_TINY_RUN(FwdArgs, norm_tiny_fwd_kernel, true) : THN_TINY_RUN(FwdArgs, norm_tiny_fwd_kernel, false); \
    }                                                                                                           \
    int launch_norm_tiny_bwd_##NAME(bool ln, bool staged, const BwdArgs& a, int grid, hipStream_t st) {         \
        using T = TYPE;                                                                                         \
        return ln ? THN_TINY_RUN(BwdArgs, norm_tiny_bwd_kernel, true) : THN_TINY_RUN(BwdArgs, norm_tiny_bwd_kernel, false); \
    }

}  // namespace thn
