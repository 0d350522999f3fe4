// Softmax / Softmin / LogSoftmax over narrow rows (1 to 32 vectors) with the flat lane-to-vector mapping of
// thn_flat.h: lane l of a wave owns vector l % L of row l / L, a wave holds 64 / L whole rows and requests one
// contiguous piece of memory per load / store instruction.  The row kernels of thn_softmax.h give a row 8, 16 or 32
// lanes, so rows of 1, 2 and 4 vectors leave 7/8, 3/4 and half of their lanes idle, and 9 vectors 7 of 16.  A softmax
// needs ONE value per reduction round (the row maximum, the row sum; the backward one sum), which is what the
// segmented ds_bpermute reductions are cheapest at.  Arithmetic as softmax_fwd_kernel / softmax_bwd_kernel, in float32;
// float32 / float16 / bfloat16 rows; ALIGNED = false: rows of at least one vector off the 128-bit path, whose slots are
// unaligned 16-byte windows, the ragged last one overlapping its neighbour (slot_place() in thn_kernels.h).
#pragma once

#include "thn_flat.h"
#include "thn_softmax.h"

namespace thn {

// segment_allreduce with a choice of operation (maximum or sum).  A lane outside every segment (pos = L) keeps its own
// value through the tree and then picks up the total of the segment it mirrors.
template <int LOG, int NV, typename Op>
__device__ __forceinline__ void segment_allreduce_op(float (&v)[NV], int lane, int pos, int L, int first) {
#pragma unroll
    for (int s = 0; s < LOG; ++s) {
        const int d = 1 << s;
        const bool take = pos + d < L;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const float other = lane_read(v[i], lane + d);
            v[i] = take ? Op::apply(v[i], other) : v[i];
        }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] = lane_read(v[i], first);
}

// Byte offset of vector t of a row of L vectors and the number of its leading columns that the slot before it owns
// (0 on the 128-bit path).
template <typename T, bool ALIGNED>
__device__ __forceinline__ void flat_slot(int t, int L, int n_cols, int& voff, int& lead) {
    bool own;
    slot_place<T, ALIGNED>(t, L, n_cols, voff, lead, own);
}

template <typename T, bool LOGSM, int J, int LOG, bool ALIGNED>
__global__ void __launch_bounds__(kFlatBlock) softmax_flat_fwd_kernel(const SoftmaxFwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int W = kFlatBlock / 64;
    const int L = a.n_vecs;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rpw = 64 / L;
    const FlatLane f = flat_lane(lane, L);
    int voff, lead;
    flat_slot<T, ALIGNED>(f.t, L, a.n_cols, voff, lead);
    const float neg_inf = OpMax::identity<float>();

    const int64_t rows_per_block = static_cast<int64_t>(W) * rpw * J;
    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * rows_per_block;
    const int64_t last_row = a.M - 1;
    int64_t row_raw[J], row[J];
    u32x4 cur[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
        row_raw[j] = static_cast<int64_t>(blockIdx.x) * rows_per_block + static_cast<int64_t>(j * W + wave) * rpw + f.r;
        row[j] = row_raw[j] < a.M ? row_raw[j] : last_row;
        cur[j] = slot_load<T, ALIGNED>(a.x + row[j] * a.x_stride_bytes, voff, a.n_cols);
    }
    drain_vector_memory(cur);

    for (int64_t base = static_cast<int64_t>(blockIdx.x) * rows_per_block; base < a.M; base += rows_per_iter) {
        int64_t nrow_raw[J], nrow[J];
        u32x4 nxt[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            nrow_raw[j] = row_raw[j] + rows_per_iter;
            nrow[j] = nrow_raw[j] < a.M ? nrow_raw[j] : last_row;
            nxt[j] = slot_load<T, ALIGNED>(a.x + nrow[j] * a.x_stride_bytes, voff, a.n_cols);
        }
        float xf[J][VEC];
        float m[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            T::unpack(cur[j], xf[j]);
            float mj = neg_inf;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                xf[j][e] *= a.sign;
                mj = fmaxf(mj, xf[j][e]);          // mirror lanes and overlapping windows repeat real columns: harmless for a maximum
            }
            m[j] = mj;
        }
        segment_allreduce_op<LOG, J, OpMax>(m, lane, f.pos, L, f.first);
        float s[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float sk = 0.0f;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float z = xf[j][e] - m[j];
                const float ez = exp_c(z);
                xf[j][e] = LOGSM ? z : ez;
                sk += e >= lead ? ez : 0.0f;          // an overlapping window's leading columns count in the slot before
            }
            s[j] = f.own ? sk : 0.0f;
        }
        segment_allreduce_op<LOG, J, OpSum>(s, lane, f.pos, L, f.first);
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const float scale = LOGSM ? logf(s[j]) : 1.0f / s[j];
            float yf[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) yf[e] = LOGSM ? xf[j][e] - scale : xf[j][e] * scale;
            slot_store<T, ALIGNED, true>(a.y + row[j] * a.y_stride_bytes, voff, a.n_cols, yf);   // the backward works from the saved y
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            cur[j] = nxt[j];
            row_raw[j] = nrow_raw[j];
            row[j] = nrow[j];
        }
    }
}

template <typename T, bool LOGSM, int J, int LOG, bool ALIGNED>
__global__ void __launch_bounds__(kFlatBlock) softmax_flat_bwd_kernel(const SoftmaxBwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int W = kFlatBlock / 64;
    const int L = a.n_vecs;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rpw = 64 / L;
    const FlatLane f = flat_lane(lane, L);
    int voff, lead;
    flat_slot<T, ALIGNED>(f.t, L, a.n_cols, voff, lead);

    const int64_t rows_per_block = static_cast<int64_t>(W) * rpw * J;
    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * rows_per_block;
    const int64_t last_row = a.M - 1;
    int64_t row_raw[J], row[J];
    u32x4 cy[J], cg[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
        row_raw[j] = static_cast<int64_t>(blockIdx.x) * rows_per_block + static_cast<int64_t>(j * W + wave) * rpw + f.r;
        row[j] = row_raw[j] < a.M ? row_raw[j] : last_row;
        cy[j] = slot_load<T, ALIGNED>(a.y + row[j] * a.y_stride_bytes, voff, a.n_cols);
        cg[j] = slot_load<T, ALIGNED>(a.dy + row[j] * a.dy_stride_bytes, voff, a.n_cols);
    }
    drain_vector_memory(cy, cg);

    for (int64_t base = static_cast<int64_t>(blockIdx.x) * rows_per_block; base < a.M; base += rows_per_iter) {
        int64_t nrow_raw[J], nrow[J];
        u32x4 ny[J], ng[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            nrow_raw[j] = row_raw[j] + rows_per_iter;
            nrow[j] = nrow_raw[j] < a.M ? nrow_raw[j] : last_row;
            ny[j] = slot_load<T, ALIGNED>(a.y + nrow[j] * a.y_stride_bytes, voff, a.n_cols);
            ng[j] = slot_load<T, ALIGNED>(a.dy + nrow[j] * a.dy_stride_bytes, voff, a.n_cols);
        }
        float yf[J][VEC], gf[J][VEC];
        float s[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            T::unpack(cy[j], yf[j]);
            T::unpack(cg[j], gf[j]);
            float sk = 0.0f;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float ge = e >= lead ? gf[j][e] : 0.0f;
                if constexpr (LOGSM) sk += ge;
                else sk = fmaf(yf[j][e], ge, sk);
            }
            s[j] = f.own ? sk : 0.0f;
        }
        segment_allreduce_op<LOG, J, OpSum>(s, lane, f.pos, L, f.first);
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float dxf[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float d;
                if constexpr (LOGSM) d = fmaf(-exp_c(yf[j][e]), s[j], gf[j][e]);
                else d = yf[j][e] * (gf[j][e] - s[j]);
                dxf[e] = d * a.sign;
            }
            slot_store<T, ALIGNED>(a.dx + row[j] * a.dx_stride_bytes, voff, a.n_cols, dxf);
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            cy[j] = ny[j];
            cg[j] = ng[j];
            row_raw[j] = nrow_raw[j];
            row[j] = nrow[j];
        }
    }
}

// Launchers: 0 launched, 1 no such instance, <0 HIP error.  `log_steps`: tree steps of the segmented reductions (0 for
// rows of one vector, 2 up to 4 vectors, 4 up to 16, 5 up to 32); `rows_each` = J.
#define THN_DECLARE_SOFTMAX_FLAT_LAUNCHERS(NAME)                                                                \
    int launch_softmax_flat_fwd_##NAME(bool is_log, bool aligned, int rows_each, int log_steps, const SoftmaxFwdArgs& a, \
                                       int grid, hipStream_t st);                                               \
    int launch_softmax_flat_bwd_##NAME(bool is_log, bool aligned, int rows_each, int log_steps, const SoftmaxBwdArgs& a, \
                                       int grid, hipStream_t st);

THN_DECLARE_SOFTMAX_FLAT_LAUNCHERS(f32)
THN_DECLARE_SOFTMAX_FLAT_LAUNCHERS(f16)
THN_DECLARE_SOFTMAX_FLAT_LAUNCHERS(bf16)

#define THN_SOFTMAX_FLAT_CASE(KERNEL, ARGS_T, AL, J_, LOG_)                                                     \
    if (rows_each == J_ && log_steps == LOG_) {                                                                 \
        return is_log ? run_kernel<ARGS_T>(KERNEL<T, true, J_, LOG_, AL>, a, grid, kFlatBlock, st, nullptr)      \
                      : run_kernel<ARGS_T>(KERNEL<T, false, J_, LOG_, AL>, a, grid, kFlatBlock, st, nullptr);    \
    }
#define THN_SOFTMAX_FLAT_FWD_AL(J_, LOG_) THN_SOFTMAX_FLAT_CASE(softmax_flat_fwd_kernel, SoftmaxFwdArgs, true, J_, LOG_)
#define THN_SOFTMAX_FLAT_BWD_AL(J_, LOG_) THN_SOFTMAX_FLAT_CASE(softmax_flat_bwd_kernel, SoftmaxBwdArgs, true, J_, LOG_)
#define THN_SOFTMAX_FLAT_FWD_SC(J_, LOG_) THN_SOFTMAX_FLAT_CASE(softmax_flat_fwd_kernel, SoftmaxFwdArgs, false, J_, LOG_)
#define THN_SOFTMAX_FLAT_BWD_SC(J_, LOG_) THN_SOFTMAX_FLAT_CASE(softmax_flat_bwd_kernel, SoftmaxBwdArgs, false, J_, LOG_)
// X(J, LOG): rows per lane and step x tree steps
#define THN_SOFTMAX_FLAT_SHAPES(X) X(2, 0) X(4, 0) X(2, 2) X(4, 2) X(2, 4) X(4, 4) X(2, 5) X(4, 5)
// off the 128-bit path: two rows per lane only
#define THN_SOFTMAX_FLAT_SHAPES_UNALIGNED(X) X(2, 0) X(2, 2) X(2, 4) X(2, 5)

#define THN_DEFINE_SOFTMAX_FLAT_LAUNCHERS(NAME, TYPE)                                                           \
    int launch_softmax_flat_fwd_##NAME(bool is_log, bool aligned, int rows_each, int log_steps, const SoftmaxFwdArgs& a, \
                                       int grid, hipStream_t st) {                                              \
        using T = TYPE;                                                                                         \
        if (aligned) {                                                                                          \
            THN_SOFTMAX_FLAT_SHAPES(THN_SOFTMAX_FLAT_FWD_AL)                                                    \
        } else {                                                                                                \
            THN_SOFTMAX_FLAT_SHAPES_UNALIGNED(THN_SOFTMAX_FLAT_FWD_SC)                                          \
        }                                                                                                       \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_softmax_flat_bwd_##NAME(bool is_log, bool aligned, int rows_each, int log_steps, const SoftmaxBwdArgs& a, \
                                       int grid, hipStream_t st) {                                              \
        using T = TYPE;                                                                                         \
        if (aligned) {                                                                                          \
            THN_SOFTMAX_FLAT_SHAPES(THN_SOFTMAX_FLAT_BWD_AL)                                                    \
        } else {                                                                                                \
            THN_SOFTMAX_FLAT_SHAPES_UNALIGNED(THN_SOFTMAX_FLAT_BWD_SC)                                          \
        }                                                                                                       \
        return 1;                                                                                               \
    }

}  // namespace thn
