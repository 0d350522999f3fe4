// Norm kernels for narrow rows whose vector count does not fill a power-of-two lane group: the FLAT mapping.
//
// The row kernels of thn_kernels.h give a row 8, 16 or 32 lanes (a power of two, so that the row sums are DPP
// reductions over aligned lane groups).  A row of 9 vectors then leaves 7 of 16 lanes idle, one of 17 vectors 15 of 32:
// up to half of every load and store instruction of a wave re-requests a vector another lane already owns, and the
// pieces a wave requests are separated by the rows' pitch.  Here consecutive lanes own consecutive vectors ACROSS
// rows: lane l of a wave owns vector l % L of row l / L (L = vectors per row, any value from 2 to 32), a wave holds
// 64 / L whole rows, and -- the rows being dense -- every load / store instruction of a wave covers one contiguous
// piece of (64 / L) * L vectors.  At most L - 1 lanes at the top of a wave have no row; they mirror the wave's last
// lane that has one (same address, same inputs, same instructions: the same bits stored twice) and add to no sum.
//
// Row sums are segmented reductions over L consecutive lanes that start anywhere in the wave: a log2(L)-step tree of
// ds_bpermute_b32 exchanges (register-to-register through the LDS crossbar, no LDS memory), in which lane p of a
// segment adds the value of lane p + d while p + d < L, then one more exchange that hands every lane the total that
// has formed in the segment's first lane.  The order of the additions depends on L alone: a row's results are the same
// bits wherever the row sits.
//
// Everything else follows the row kernels: a persistent grid, J independent rows per lane and step with the next J
// requested before the current ones are reduced, no branch around a load or store (rows past the end are clamped
// onto the last row and masked out of dW / dB), float32 arithmetic, the statistics stored by every lane of a row,
// one float32 partial row of dW / dB per workgroup summed in a fixed order.  ALIGNED = false: rows of at least two
// vectors off the 128-bit path, whose slots are unaligned 16-byte windows, the ragged last one overlapping its neighbour
// (slot_place() in thn_kernels.h: the overlapped columns are computed and stored twice, and counted once in every sum).
#pragma once

#include "thn_dispatch.h"

namespace thn {

constexpr int kFlatBlock = 256;        // threads per workgroup of the flat kernels
constexpr int kFlatMaxVecs = 32;       // widest row (in vectors) they take

__device__ __forceinline__ float lane_read(float v, int src_lane) {
    return as_f32(static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(src_lane << 2, static_cast<int>(as_u32(v)))));
}

// Sums NV values over each segment of L consecutive lanes.  `pos`: the lane's position in its segment (L for a lane
// that belongs to none: it adds nothing and nobody reads it); `first`: the first lane of the segment whose total the
// lane wants.  LOG = ceil(log2(L)).
template <int LOG, int NV>
__device__ __forceinline__ void segment_allreduce(float (&v)[NV], int lane, int pos, int L, int first) {
#pragma unroll
    for (int s = 0; s < LOG; ++s) {
        const int d = 1 << s;
        const bool take = pos + d < L;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const float other = lane_read(v[i], lane + d);
            v[i] += take ? other : 0.0f;
        }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] = lane_read(v[i], first);
}

// Where a lane stands: its row within the wave's batch of rows, its vector, its place in the reduction.
struct FlatLane {
    int r, t, pos, first;
    bool own;
};
__device__ __forceinline__ FlatLane flat_lane(int lane, int L) {
    const int rpw = 64 / L;
    FlatLane f;
    f.r = lane / L;
    f.t = lane - f.r * L;
    f.own = f.r < rpw;
    if (!f.own) {          // a lane without a row mirrors the last lane that has one
        f.r = rpw - 1;
        f.t = L - 1;
    }
    f.pos = f.own ? f.t : L;
    f.first = f.r * L;
    return f;
}

// Forward.  Arithmetic as norm_fwd_kernel (LayerNorm: mean0, then {sum d, sum d^2} with the delta correction).
template <typename T, bool LN, int J, int LOG, bool KEEPX, bool ALIGNED>
__global__ void __launch_bounds__(kFlatBlock) norm_flat_fwd_kernel(const FwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int W = kFlatBlock / 64;
    const int L = a.n_vecs;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rpw = 64 / L;
    const FlatLane f = flat_lane(lane, L);
    int voff, lead;
    {
        bool in_row;
        slot_place<T, ALIGNED>(f.t, L, a.n_cols, voff, lead, in_row);
    }

    const int64_t rows_per_block = static_cast<int64_t>(W) * rpw * J;
    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * rows_per_block;
    const int64_t last_row = a.M - 1;
    int64_t row_raw[J], row[J];
    u32x4 cur[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
        row_raw[j] = static_cast<int64_t>(blockIdx.x) * rows_per_block + static_cast<int64_t>(j * W + wave) * rpw + f.r;
        row[j] = row_raw[j] < a.M ? row_raw[j] : last_row;
        cur[j] = slot_load<T, ALIGNED, KEEPX>(a.x + row[j] * a.x_stride_bytes, voff, a.n_cols);
    }
    float wr[1][VEC], br[1][VEC];
    const int pv[1] = {voff};
    slot_params<T, 1, ALIGNED>(wr, a.w, a.w_dtype, pv, a.n_cols, 1.0f);
    if constexpr (LN) slot_params<T, 1, ALIGNED>(br, a.b, a.w_dtype, pv, a.n_cols, 0.0f);
    drain_vector_memory(cur);

    for (int64_t base = static_cast<int64_t>(blockIdx.x) * rows_per_block; base < a.M; base += rows_per_iter) {
        int64_t nrow_raw[J], nrow[J];
        u32x4 nxt[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            nrow_raw[j] = row_raw[j] + rows_per_iter;
            nrow[j] = nrow_raw[j] < a.M ? nrow_raw[j] : last_row;
            nxt[j] = slot_load<T, ALIGNED, KEEPX>(a.x + nrow[j] * a.x_stride_bytes, voff, a.n_cols);
        }
        float xf[J][VEC];
#pragma unroll
        for (int j = 0; j < J; ++j) T::unpack(cur[j], xf[j]);
        float mean[J], rstd[J], delta[J];
        if constexpr (LN) {
            float s[J];
#pragma unroll
            for (int j = 0; j < J; ++j) {
                float sk = 0.0f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) sk += e >= lead ? xf[j][e] : 0.0f;     // overlapped columns count once
                s[j] = f.own ? sk : 0.0f;
            }
            segment_allreduce<LOG, J>(s, lane, f.pos, L, f.first);
            float q[2 * J];
#pragma unroll
            for (int j = 0; j < J; ++j) {
                const float mean0 = s[j] * a.inv_n;
                float q0 = 0.0f, q1 = 0.0f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float d = xf[j][e] - mean0;
                    xf[j][e] = d;
                    const float dm = e >= lead ? d : 0.0f;
                    q0 += dm;
                    q1 = fmaf(dm, dm, q1);
                }
                q[2 * j] = f.own ? q0 : 0.0f;
                q[2 * j + 1] = f.own ? q1 : 0.0f;
                mean[j] = mean0;
            }
            segment_allreduce<LOG, 2 * J>(q, lane, f.pos, L, f.first);
#pragma unroll
            for (int j = 0; j < J; ++j) {
                delta[j] = q[2 * j] * a.inv_n;
                const float var = fmaxf(fmaf(-delta[j], delta[j], q[2 * j + 1] * a.inv_n), 0.0f);
                rstd[j] = rsqrt_refined(var + a.eps);
                mean[j] += delta[j];
            }
        } else {
            float q[J];
#pragma unroll
            for (int j = 0; j < J; ++j) {
                float qk = 0.0f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float xm = e >= lead ? xf[j][e] : 0.0f;
                    qk = fmaf(xm, xm, qk);
                }
                q[j] = f.own ? qk : 0.0f;
            }
            segment_allreduce<LOG, J>(q, lane, f.pos, L, f.first);
#pragma unroll
            for (int j = 0; j < J; ++j) {
                rstd[j] = rsqrt_refined(fmaf(q[j], a.inv_n, a.eps));
                delta[j] = 0.0f;
                mean[j] = 0.0f;
            }
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float yf[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if constexpr (LN) yf[e] = fmaf((xf[j][e] - delta[j]) * rstd[j], wr[0][e], br[0][e]);
                else yf[e] = xf[j][e] * rstd[j] * wr[0][e];
            }
            slot_store<T, ALIGNED>(a.y + row[j] * a.y_stride_bytes, voff, a.n_cols, yf);
            if constexpr (LN) a.mean[row[j]] = mean[j];
            a.rstd[row[j]] = rstd[j];
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            cur[j] = nxt[j];
            row_raw[j] = nrow_raw[j];
            row[j] = nrow[j];
        }
    }
}

// Backward.  Arithmetic as norm_bwd_kernel: one round of {sum u*wdy, sum wdy, sum u}; per-lane column sums of dW / dB
// (float64 for float32 rows), which the workgroup adds up at the end, in a fixed order, into ONE float32 partial row.
template <typename T, bool LN, int J, int LOG, bool ALIGNED>
__global__ void __launch_bounds__(kFlatBlock) norm_flat_bwd_kernel(const BwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int W = kFlatBlock / 64;
    constexpr int NV = LN ? 3 : 1;
    using Acc = typename AccType<(T::kBytes >= 4)>::type;
    __shared__ Acc totals[2][kFlatBlock][VEC];       // [dW | dB][thread][column of the thread's vector]

    const int L = a.n_vecs;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rpw = 64 / L;
    const FlatLane f = flat_lane(lane, L);
    int voff, lead;
    {
        bool in_row;
        slot_place<T, ALIGNED>(f.t, L, a.n_cols, voff, lead, in_row);
    }

    const int64_t rows_per_block = static_cast<int64_t>(W) * rpw * J;
    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * rows_per_block;
    const int64_t last_row = a.M - 1;
    int64_t row_raw[J], row[J];
    u32x4 cx[J], cg[J];
    float c_mean[J], c_rstd[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
        row_raw[j] = static_cast<int64_t>(blockIdx.x) * rows_per_block + static_cast<int64_t>(j * W + wave) * rpw + f.r;
        row[j] = row_raw[j] < a.M ? row_raw[j] : last_row;
        cx[j] = slot_load<T, ALIGNED>(a.x + row[j] * a.x_stride_bytes, voff, a.n_cols);
        cg[j] = slot_load<T, ALIGNED>(a.dy + row[j] * a.dy_stride_bytes, voff, a.n_cols);
        c_mean[j] = LN ? a.mean[row[j]] : 0.0f;
        c_rstd[j] = a.rstd[row[j]];
    }
    float wr[1][VEC];
    const int pv[1] = {voff};
    slot_params<T, 1, ALIGNED>(wr, a.w, a.w_dtype, pv, a.n_cols, 1.0f);
    Acc dw[VEC], db[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) { dw[e] = Acc(0); db[e] = Acc(0); }
#pragma unroll
    for (int j = 0; j < J; ++j) {
        if constexpr (LN) pin_loaded(c_mean[j]);
        pin_loaded(c_rstd[j]);
    }
    drain_vector_memory(cx, cg);

    for (int64_t base = static_cast<int64_t>(blockIdx.x) * rows_per_block; base < a.M; base += rows_per_iter) {
        int64_t nrow_raw[J], nrow[J];
        u32x4 nx[J], ng[J];
        float n_mean[J], n_rstd[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            nrow_raw[j] = row_raw[j] + rows_per_iter;
            nrow[j] = nrow_raw[j] < a.M ? nrow_raw[j] : last_row;
            nx[j] = slot_load<T, ALIGNED>(a.x + nrow[j] * a.x_stride_bytes, voff, a.n_cols);
            ng[j] = slot_load<T, ALIGNED>(a.dy + nrow[j] * a.dy_stride_bytes, voff, a.n_cols);
            n_mean[j] = LN ? a.mean[nrow[j]] : 0.0f;
            n_rstd[j] = a.rstd[nrow[j]];
        }
        float u[J][VEC], gf[J][VEC], wdy[J][VEC];
        float s[NV * J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            T::unpack(cx[j], u[j]);
            T::unpack(cg[j], gf[j]);
            float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if constexpr (LN) u[j][e] = (u[j][e] - c_mean[j]) * c_rstd[j];
                else u[j][e] *= c_rstd[j];
                wdy[j][e] = wr[0][e] * gf[j][e];
                const bool counts = e >= lead;               // overlapped columns count once
                const float wm = counts ? wdy[j][e] : 0.0f;
                s0 = fmaf(u[j][e], wm, s0);
                if constexpr (LN) {
                    s1 += wm;
                    s2 += counts ? u[j][e] : 0.0f;
                }
            }
            s[NV * j] = f.own ? s0 : 0.0f;
            if constexpr (LN) {
                s[NV * j + 1] = f.own ? s1 : 0.0f;
                s[NV * j + 2] = f.own ? s2 : 0.0f;
            }
        }
        segment_allreduce<LOG, NV * J>(s, lane, f.pos, L, f.first);
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float c1, c2 = 0.0f, dlt = 0.0f;
            if constexpr (LN) {
                dlt = s[NV * j + 2] * a.inv_n;
                c2 = s[NV * j + 1] * a.inv_n;
                c1 = fmaf(-dlt, c2, s[NV * j] * a.inv_n);
            } else {
                c1 = s[NV * j] * a.inv_n;
            }
            const bool adds = f.own && row_raw[j] < a.M;       // a mirror lane or a row past the end adds nothing to dW / dB
            float dxf[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float xhat = u[j][e];
                if constexpr (LN) xhat -= dlt;
                dxf[e] = (wdy[j][e] - fmaf(xhat, c1, c2)) * c_rstd[j];
                const float gl = (adds && e >= lead) ? gf[j][e] : 0.0f;
                dw[e] = fma(static_cast<Acc>(gl), static_cast<Acc>(xhat), dw[e]);
                if constexpr (LN) db[e] += static_cast<Acc>(gl);
            }
            slot_store<T, ALIGNED>(a.dx + row[j] * a.dx_stride_bytes, voff, a.n_cols, dxf);
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            cx[j] = nx[j];
            cg[j] = ng[j];
            c_mean[j] = n_mean[j];
            c_rstd[j] = n_rstd[j];
            row_raw[j] = nrow_raw[j];
            row[j] = nrow[j];
        }
    }

    // The workgroup's partial row: column c = t * VEC + e is the sum over the waves, and over the rows of a wave, of
    // the lanes that own vector t -- added by one thread per column in a fixed order (wave, then row).
    const bool want_dw = a.dw_part != nullptr;
    const bool want_db = LN && a.db_part != nullptr;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        totals[0][threadIdx.x][e] = dw[e];
        totals[1][threadIdx.x][e] = LN ? db[e] : Acc(0);
    }
    __syncthreads();
    for (int c = threadIdx.x; c < a.n_cols; c += kFlatBlock) {
        const int t = c / VEC;                                 // the slot that owns column c, and c's place in its window
        const int start = (!ALIGNED && t * VEC > a.n_cols - VEC) ? a.n_cols - VEC : t * VEC;
        const int e = c - start;
        Acc sw = Acc(0), sb = Acc(0);
        for (int w = 0; w < W; ++w) {
            for (int r = 0; r < rpw; ++r) {
                const int src = w * 64 + r * L + t;
                sw += totals[0][src][e];
                sb += totals[1][src][e];
            }
        }
        const int64_t off = static_cast<int64_t>(blockIdx.x) * a.part_pitch + c;
        if (want_dw) a.dw_part[off] = static_cast<float>(sw);
        if (want_db) a.db_part[off] = static_cast<float>(sb);
    }
}

// Launchers: 0 launched (or occupancy written), 1 no such instance, <0 HIP error.  `log_steps` = ceil(log2(L)): 4 or 5
// (rows of up to 16 vectors use the 4-step instances as well); `rows_each` = J.
#define THN_DECLARE_FLAT_LAUNCHERS(NAME)                                                                        \
    int launch_flat_fwd_##NAME(bool ln, bool aligned, int rows_each, int log_steps, const FwdArgs& a, int grid, \
                               hipStream_t st, int* occupancy);                                                 \
    int launch_flat_bwd_##NAME(bool ln, bool aligned, int rows_each, int log_steps, const BwdArgs& a, int grid, \
                               hipStream_t st, int* occupancy);

THN_DECLARE_FLAT_LAUNCHERS(f32)
THN_DECLARE_FLAT_LAUNCHERS(f16)
THN_DECLARE_FLAT_LAUNCHERS(bf16)

#define THN_FLAT_FWD_CASE(AL, J_, LOG_)                                                                         \
    if (rows_each == J_ && log_steps == LOG_) {                                                                 \
        if (a.keep_x) {                                                                                         \
            return ln ? run_kernel<FwdArgs>(norm_flat_fwd_kernel<T, true, J_, LOG_, true, AL>, a, grid, kFlatBlock, st, occupancy)  \
                      : run_kernel<FwdArgs>(norm_flat_fwd_kernel<T, false, J_, LOG_, true, AL>, a, grid, kFlatBlock, st, occupancy); \
        }                                                                                                       \
        return ln ? run_kernel<FwdArgs>(norm_flat_fwd_kernel<T, true, J_, LOG_, false, AL>, a, grid, kFlatBlock, st, occupancy)     \
                  : run_kernel<FwdArgs>(norm_flat_fwd_kernel<T, false, J_, LOG_, false, AL>, a, grid, kFlatBlock, st, occupancy);   \
    }
#define THN_FLAT_BWD_CASE(AL, J_, LOG_)                                                                         \
    if (rows_each == J_ && log_steps == LOG_) {                                                                 \
        return ln ? run_kernel<BwdArgs>(norm_flat_bwd_kernel<T, true, J_, LOG_, AL>, a, grid, kFlatBlock, st, occupancy)   \
                  : run_kernel<BwdArgs>(norm_flat_bwd_kernel<T, false, J_, LOG_, AL>, a, grid, kFlatBlock, st, occupancy);  \
    }
#define THN_FLAT_FWD_AL(J_, LOG_) THN_FLAT_FWD_CASE(true, J_, LOG_)
#define THN_FLAT_FWD_SC(J_, LOG_) THN_FLAT_FWD_CASE(false, J_, LOG_)
#define THN_FLAT_BWD_AL(J_, LOG_) THN_FLAT_BWD_CASE(true, J_, LOG_)
#define THN_FLAT_BWD_SC(J_, LOG_) THN_FLAT_BWD_CASE(false, J_, LOG_)
// X(J, LOG): rows per lane and step x tree steps
#define THN_FLAT_SHAPES(X) X(1, 4) X(2, 4) X(4, 4) X(1, 5) X(2, 5) X(4, 5)
// off the 128-bit path: one or two rows per lane
#define THN_FLAT_SHAPES_UNALIGNED(X) X(1, 4) X(2, 4) X(1, 5) X(2, 5)

#define THN_DEFINE_FLAT_LAUNCHERS(NAME, TYPE)                                                                   \
    int launch_flat_fwd_##NAME(bool ln, bool aligned, int rows_each, int log_steps, const FwdArgs& a, int grid, \
                               hipStream_t st, int* occupancy) {                                                \
        using T = TYPE;                                                                                         \
        if (aligned) {                                                                                          \
            THN_FLAT_SHAPES(THN_FLAT_FWD_AL)                                                                    \
        } else {                                                                                                \
            THN_FLAT_SHAPES_UNALIGNED(THN_FLAT_FWD_SC)                                                          \
        }                                                                                                       \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_flat_bwd_##NAME(bool ln, bool aligned, int rows_each, int log_steps, const BwdArgs& a, int grid, \
                               hipStream_t st, int* occupancy) {                                                \
        using T = TYPE;                                                                                         \
        if (aligned) {                                                                                          \
            THN_FLAT_SHAPES(THN_FLAT_BWD_AL)                                                                    \
        } else {                                                                                                \
            THN_FLAT_SHAPES_UNALIGNED(THN_FLAT_BWD_SC)                                                          \
        }                                                                                                       \
        return 1;                                                                                               \
    }

}  // namespace thn
