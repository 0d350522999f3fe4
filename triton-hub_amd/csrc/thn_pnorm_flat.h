// Row p-norm and normalize over narrow rows (1 to 32 vectors) with the flat lane-to-vector mapping of thn_flat.h:
// lane l of a wave owns vector l % L of row l / L, a wave holds 64 / L whole rows and requests one contiguous piece of
// memory per load / store instruction; row sums are segmented ds_bpermute reductions (one value per row here: the power
// sum, or the projection of the gradient).  The row kernels of thn_pnorm.h give a row 8, 16 or 32 lanes: rows of 1, 2
// and 4 vectors -- normalising 4-, 8- or 16-component float32 vectors -- leave 7/8, 3/4 and half of their lanes idle.
// Arithmetic as pnorm_fwd_kernel / pnorm_bwd_kernel / normalize_bwd_kernel.  For tensors whose rows are one folded
// batch (row r at r * row stride), float32 / float16 / bfloat16, integer p from 1 to 6; two rows per lane and step.
// ALIGNED = false: rows of at least one vector off the 128-bit path (unaligned 16-byte windows, see thn_softmax_flat.h).
#pragma once

#include "thn_pnorm.h"
#include "thn_softmax_flat.h"

namespace thn {

constexpr int kRowsFlatJ = 2;     // rows per lane and step of these kernels

template <typename T, int MODE, bool NORMALIZE, int LOG, bool ALIGNED>
__global__ void __launch_bounds__(kFlatBlock) pnorm_flat_fwd_kernel(const PnormFwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int W = kFlatBlock / 64;
    constexpr int J = kRowsFlatJ;
    constexpr bool kKeepY = NORMALIZE && MODE == kP2;        // what the backward reads again stays in the caches
    constexpr bool kKeepX = !kKeepY;
    const int L = a.n_vecs;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rpw = 64 / L;
    const FlatLane f = flat_lane(lane, L);
    int voff, lead;
    flat_slot<T, ALIGNED>(f.t, L, a.n_cols, voff, lead);

    const int64_t rows_per_block = static_cast<int64_t>(W) * rpw * J;
    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * rows_per_block;
    const int64_t last_row = a.rows - 1;
    int64_t row_raw[J], row[J];
    u32x4 cur[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
        row_raw[j] = static_cast<int64_t>(blockIdx.x) * rows_per_block + static_cast<int64_t>(j * W + wave) * rpw + f.r;
        row[j] = row_raw[j] < a.rows ? row_raw[j] : last_row;
        cur[j] = slot_load<T, ALIGNED, kKeepX>(a.x + row[j] * a.xmap.row_stride_bytes, voff, a.n_cols);
    }
    drain_vector_memory(cur);

    for (int64_t base = static_cast<int64_t>(blockIdx.x) * rows_per_block; base < a.rows; base += rows_per_iter) {
        int64_t nrow_raw[J], nrow[J];
        u32x4 nxt[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            nrow_raw[j] = row_raw[j] + rows_per_iter;
            nrow[j] = nrow_raw[j] < a.rows ? nrow_raw[j] : last_row;
            nxt[j] = slot_load<T, ALIGNED, kKeepX>(a.x + nrow[j] * a.xmap.row_stride_bytes, voff, a.n_cols);
        }
        float xf[J][VEC];
        float s[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            T::unpack(cur[j], xf[j]);
            float sk = 0.0f;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {      // an overlapping window's leading columns count in the slot before
                const float term = norm_term<MODE>(xf[j][e], a.p_int);
                sk += e >= lead ? term : 0.0f;
            }
            s[j] = f.own ? sk : 0.0f;
        }
        segment_allreduce_op<LOG, J, OpSum>(s, lane, f.pos, L, f.first);
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const float n = fmaxf(norm_root<MODE>(s[j], a.p_int, a.p), a.eps);
            T::store1(a.norms, row[j], n);                // every lane of the row: the same value to the same address
            if constexpr (NORMALIZE) {
                const float nr = round_to_storage<T>(n);
                const float rn = 1.0f / nr;
                const float nd = residual_divisor(nr);
                float yf[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) yf[e] = div_by_row(xf[j][e], nd, rn);
                slot_store<T, ALIGNED, kKeepY>(a.y + row[j] * a.ymap.row_stride_bytes, voff, a.n_cols, yf);
            }
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            cur[j] = nxt[j];
            row_raw[j] = nrow_raw[j];
            row[j] = nrow[j];
        }
    }
}

// Norm backward: element-wise with two per-row scalars, no row sum.
template <typename T, int MODE, bool ALIGNED>
__global__ void __launch_bounds__(kFlatBlock) pnorm_flat_bwd_kernel(const PnormBwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int W = kFlatBlock / 64;
    constexpr int J = kRowsFlatJ;
    const int L = a.n_vecs;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rpw = 64 / L;
    const FlatLane f = flat_lane(lane, L);
    int voff, lead;
    flat_slot<T, ALIGNED>(f.t, L, a.n_cols, voff, lead);

    const int64_t rows_per_block = static_cast<int64_t>(W) * rpw * J;
    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * rows_per_block;
    const int64_t last_row = a.rows - 1;
    int64_t row_raw[J], row[J];
    u32x4 cur[J];
    float c_n[J], c_g[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
        row_raw[j] = static_cast<int64_t>(blockIdx.x) * rows_per_block + static_cast<int64_t>(j * W + wave) * rpw + f.r;
        row[j] = row_raw[j] < a.rows ? row_raw[j] : last_row;
        cur[j] = slot_load<T, ALIGNED>(a.x + row[j] * a.xmap.row_stride_bytes, voff, a.n_cols);
        c_n[j] = MODE == kP1 ? 1.0f : T::load1(a.norms, row[j]);
        c_g[j] = T::load1(a.g, row[j]);
    }
#pragma unroll
    for (int j = 0; j < J; ++j) {
        if constexpr (MODE != kP1) pin_loaded(c_n[j]);
        pin_loaded(c_g[j]);
    }
    drain_vector_memory(cur);

    for (int64_t base = static_cast<int64_t>(blockIdx.x) * rows_per_block; base < a.rows; base += rows_per_iter) {
        int64_t nrow_raw[J], nrow[J];
        u32x4 nxt[J];
        typename RowScalar<T>::bits_t raw_n[J], raw_g[J];     // widened at the end of the step (see pnorm_bwd_kernel)
#pragma unroll
        for (int j = 0; j < J; ++j) {
            nrow_raw[j] = row_raw[j] + rows_per_iter;
            nrow[j] = nrow_raw[j] < a.rows ? nrow_raw[j] : last_row;
            nxt[j] = slot_load<T, ALIGNED>(a.x + nrow[j] * a.xmap.row_stride_bytes, voff, a.n_cols);
            raw_n[j] = MODE == kP1 ? 0 : RowScalar<T>::load(a.norms, nrow[j]);
            raw_g[j] = RowScalar<T>::load(a.g, nrow[j]);
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float den = c_n[j];
            if constexpr (MODE == kPInt) den = pow_small(c_n[j], a.p_int - 1);
            const float rden = 1.0f / den;
            den = residual_divisor(den);
            float xf[VEC], df[VEC];
            T::unpack(cur[j], xf);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float x = xf[e];
                if constexpr (MODE == kP1) df[e] = c_g[j] * sign_of(x);
                else if constexpr (MODE == kP2) df[e] = div_by_row(c_g[j] * x, den, rden);
                else df[e] = div_by_row(c_g[j] * sign_of(x) * pow_small(__builtin_fabsf(x), a.p_int - 1), den, rden);
            }
            slot_store<T, ALIGNED>(a.dx + row[j] * a.dxmap.row_stride_bytes, voff, a.n_cols, df);
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            cur[j] = nxt[j];
            if constexpr (MODE != kP1) {
                hold_loaded_here(raw_n[j]);
                c_n[j] = RowScalar<T>::value(raw_n[j]);
            }
            hold_loaded_here(raw_g[j]);
            c_g[j] = RowScalar<T>::value(raw_g[j]);
            row_raw[j] = nrow_raw[j];
            row[j] = nrow[j];
        }
    }
}

// Normalize backward: one segmented row sum (the projection of the gradient on x or y).
template <typename T, int MODE, int LOG, bool ALIGNED>
__global__ void __launch_bounds__(kFlatBlock) normalize_flat_bwd_kernel(const NormalizeBwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int W = kFlatBlock / 64;
    constexpr int J = kRowsFlatJ;
    constexpr bool NEED_X = MODE != kP2;
    constexpr bool NEED_Y = MODE != kP1;
    const int L = a.n_vecs;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rpw = 64 / L;
    const FlatLane f = flat_lane(lane, L);
    int voff, lead;
    flat_slot<T, ALIGNED>(f.t, L, a.n_cols, voff, lead);

    const int64_t rows_per_block = static_cast<int64_t>(W) * rpw * J;
    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * rows_per_block;
    const int64_t last_row = a.rows - 1;
    int64_t row_raw[J], row[J];
    u32x4 cx[NEED_X ? J : 1], cy[NEED_Y ? J : 1], cg[J];
    float c_n[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
        row_raw[j] = static_cast<int64_t>(blockIdx.x) * rows_per_block + static_cast<int64_t>(j * W + wave) * rpw + f.r;
        row[j] = row_raw[j] < a.rows ? row_raw[j] : last_row;
        if constexpr (NEED_X) cx[j] = slot_load<T, ALIGNED>(a.x + row[j] * a.xmap.row_stride_bytes, voff, a.n_cols);
        if constexpr (NEED_Y) cy[j] = slot_load<T, ALIGNED>(a.y + row[j] * a.ymap.row_stride_bytes, voff, a.n_cols);
        cg[j] = slot_load<T, ALIGNED>(a.g + row[j] * a.gmap.row_stride_bytes, voff, a.n_cols);
        c_n[j] = T::load1(a.norms, row[j]);
    }
#pragma unroll
    for (int j = 0; j < J; ++j) pin_loaded(c_n[j]);
    if constexpr (NEED_X) pin_loaded(cx);
    if constexpr (NEED_Y) pin_loaded(cy);
    drain_vector_memory(cg);

    for (int64_t base = static_cast<int64_t>(blockIdx.x) * rows_per_block; base < a.rows; base += rows_per_iter) {
        int64_t nrow_raw[J], nrow[J];
        u32x4 nx[NEED_X ? J : 1], ny[NEED_Y ? J : 1], ng[J];
        typename RowScalar<T>::bits_t raw_n[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            nrow_raw[j] = row_raw[j] + rows_per_iter;
            nrow[j] = nrow_raw[j] < a.rows ? nrow_raw[j] : last_row;
            if constexpr (NEED_X) nx[j] = slot_load<T, ALIGNED>(a.x + nrow[j] * a.xmap.row_stride_bytes, voff, a.n_cols);
            if constexpr (NEED_Y) ny[j] = slot_load<T, ALIGNED>(a.y + nrow[j] * a.ymap.row_stride_bytes, voff, a.n_cols);
            ng[j] = slot_load<T, ALIGNED>(a.g + nrow[j] * a.gmap.row_stride_bytes, voff, a.n_cols);
            raw_n[j] = RowScalar<T>::load(a.norms, nrow[j]);
        }
        float xf[NEED_X ? J : 1][VEC], yf[NEED_Y ? J : 1][VEC], gf[J][VEC];
        float s[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            if constexpr (NEED_X) T::unpack(cx[j], xf[j]);
            if constexpr (NEED_Y) T::unpack(cy[j], yf[j]);
            T::unpack(cg[j], gf[j]);
            float sk = 0.0f;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float ge = e >= lead ? gf[j][e] : 0.0f;
                if constexpr (MODE == kP1) sk = __builtin_fmaf(xf[j][e], ge, sk);
                else sk = __builtin_fmaf(yf[j][e], ge, sk);
            }
            s[j] = f.own ? sk : 0.0f;
        }
        segment_allreduce_op<LOG, J, OpSum>(s, lane, f.pos, L, f.first);
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const float proj = s[j];
            const float n = c_n[j];
            const float rn = 1.0f / n;
            const float nd = residual_divisor(n);
            float coef = 0.0f;
            if constexpr (MODE == kP1) coef = proj / (n * n);
            if constexpr (MODE == kPInt) coef = proj / (pow_small(n, a.p_int - 1) * n);
            float df[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float gg = gf[j][e];
                if constexpr (MODE == kP2) {
                    df[e] = div_by_row(gg - yf[j][e] * proj, nd, rn);
                } else if constexpr (MODE == kP1) {
                    df[e] = div_by_row(gg, nd, rn) - sign_of(xf[j][e]) * coef;
                } else {
                    const float x = xf[j][e];
                    df[e] = div_by_row(gg, nd, rn) - sign_of(x) * pow_small(__builtin_fabsf(x), a.p_int - 1) * coef;
                }
            }
            slot_store<T, ALIGNED>(a.dx + row[j] * a.dxmap.row_stride_bytes, voff, a.n_cols, df);
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            if constexpr (NEED_X) cx[j] = nx[j];
            if constexpr (NEED_Y) cy[j] = ny[j];
            cg[j] = ng[j];
            hold_loaded_here(raw_n[j]);
            c_n[j] = RowScalar<T>::value(raw_n[j]);
            row_raw[j] = nrow_raw[j];
            row[j] = nrow[j];
        }
    }
}

// Launchers: 0 launched, 1 no such instance, <0 HIP error.  `mode`: kP1 / kP2 / kPInt; `log_steps` as in
// thn_softmax_flat.h.
#define THN_DECLARE_PNORM_FLAT_LAUNCHERS(NAME)                                                                  \
    int launch_pnorm_flat_fwd_##NAME(int mode, bool normalize, bool aligned, int log_steps, const PnormFwdArgs& a, \
                                     int grid, hipStream_t st);                                                 \
    int launch_pnorm_flat_bwd_##NAME(int mode, bool aligned, const PnormBwdArgs& a, int grid, hipStream_t st);  \
    int launch_normalize_flat_bwd_##NAME(int mode, bool aligned, int log_steps, const NormalizeBwdArgs& a, int grid, \
                                         hipStream_t st);

THN_DECLARE_PNORM_FLAT_LAUNCHERS(f32)
THN_DECLARE_PNORM_FLAT_LAUNCHERS(f16)
THN_DECLARE_PNORM_FLAT_LAUNCHERS(bf16)

#define THN_PNORM_FLAT_FWD_CASE(AL, MODE_, LOG_)                                                                \
    if (mode == MODE_ && log_steps == LOG_) {                                                                   \
        return normalize ? run_kernel<PnormFwdArgs>(pnorm_flat_fwd_kernel<T, MODE_, true, LOG_, AL>, a, grid, kFlatBlock, st, nullptr)  \
                         : run_kernel<PnormFwdArgs>(pnorm_flat_fwd_kernel<T, MODE_, false, LOG_, AL>, a, grid, kFlatBlock, st, nullptr); \
    }
#define THN_NORMALIZE_FLAT_BWD_CASE(AL, MODE_, LOG_)                                                            \
    if (mode == MODE_ && log_steps == LOG_) {                                                                   \
        return run_kernel<NormalizeBwdArgs>(normalize_flat_bwd_kernel<T, MODE_, LOG_, AL>, a, grid, kFlatBlock, st, nullptr); \
    }
#define THN_PNORM_FLAT_BWD_CASE(AL, MODE_)                                                                      \
    if (mode == MODE_) return run_kernel<PnormBwdArgs>(pnorm_flat_bwd_kernel<T, MODE_, AL>, a, grid, kFlatBlock, st, nullptr);
#define THN_PNF_FLAT_AL(MODE_, LOG_) THN_PNORM_FLAT_FWD_CASE(true, MODE_, LOG_)
#define THN_PNF_FLAT_SC(MODE_, LOG_) THN_PNORM_FLAT_FWD_CASE(false, MODE_, LOG_)
#define THN_NZB_FLAT_AL(MODE_, LOG_) THN_NORMALIZE_FLAT_BWD_CASE(true, MODE_, LOG_)
#define THN_NZB_FLAT_SC(MODE_, LOG_) THN_NORMALIZE_FLAT_BWD_CASE(false, MODE_, LOG_)
// X(MODE, LOG)
#define THN_PNORM_FLAT_SHAPES(X)                                                                                \
    X(kP1, 0) X(kP1, 2) X(kP1, 4) X(kP1, 5) X(kP2, 0) X(kP2, 2) X(kP2, 4) X(kP2, 5)                             \
    X(kPInt, 0) X(kPInt, 2) X(kPInt, 4) X(kPInt, 5)

#define THN_DEFINE_PNORM_FLAT_LAUNCHERS(NAME, TYPE)                                                             \
    int launch_pnorm_flat_fwd_##NAME(int mode, bool normalize, bool aligned, int log_steps, const PnormFwdArgs& a, \
                                     int grid, hipStream_t st) {                                                \
        using T = TYPE;                                                                                         \
        if (aligned) {                                                                                          \
            THN_PNORM_FLAT_SHAPES(THN_PNF_FLAT_AL)                                                              \
        } else {                                                                                                \
            THN_PNORM_FLAT_SHAPES(THN_PNF_FLAT_SC)                                                              \
        }                                                                                                       \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_pnorm_flat_bwd_##NAME(int mode, bool aligned, const PnormBwdArgs& a, int grid, hipStream_t st) { \
        using T = TYPE;                                                                                         \
        if (aligned) {                                                                                          \
            THN_PNORM_FLAT_BWD_CASE(true, kP1) THN_PNORM_FLAT_BWD_CASE(true, kP2) THN_PNORM_FLAT_BWD_CASE(true, kPInt) \
        } else {                                                                                                \
            THN_PNORM_FLAT_BWD_CASE(false, kP1) THN_PNORM_FLAT_BWD_CASE(false, kP2) THN_PNORM_FLAT_BWD_CASE(false, kPInt) \
        }                                                                                                       \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_normalize_flat_bwd_##NAME(int mode, bool aligned, int log_steps, const NormalizeBwdArgs& a, int grid, \
                                         hipStream_t st) {                                                      \
        using T = TYPE;                                                                                         \
        if (aligned) {                                                                                          \
            THN_PNORM_FLAT_SHAPES(THN_NZB_FLAT_AL)                                                              \
        } else {                                                                                                \
            THN_PNORM_FLAT_SHAPES(THN_NZB_FLAT_SC)                                                              \
        }                                                                                                       \
        return 1;                                                                                               \
    }

}  // namespace thn
