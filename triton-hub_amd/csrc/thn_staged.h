// Norm kernels for narrow rows (1 to 32 vectors): a wave stages its rows through LDS and ONE lane (or 2, 4, 8) sums a row.
//
// The row kernels of thn_kernels.h give a row 8, 16 or 32 lanes (a power of two, so that the row sums are DPP
// reductions over aligned lane groups).  A row of 9 vectors then leaves 7 of 16 lanes idle, and a row of 4 or 8 vectors
// makes a wave's request out of 64- or 128-byte pieces, one per row.  Here the two jobs -- moving vectors, summing
// rows -- are dealt to the lanes separately.  Each wave of a workgroup works on batches of R rows of its own:
//   1. flat pass: lane t (of the S = (64 / L) * L lanes that have work) loads vector t % L of rows t / L,
//      t / L + 64 / L, ... (J of them): the rows being dense, every load instruction of the wave covers ONE contiguous
//      piece of S vectors; the vectors are copied into the wave's part of LDS, row after row (pitch L | 1 vectors, so
//      that the rows of consecutive lanes start in different banks);
//   2. statistics pass: lane s reads row s / P back (P lanes share a row when the batch has fewer rows than the wave has
//      lanes: its vectors p, p + P, ...; their sums meet in one to three DPP steps inside a quad or a half row) and
//      sums it serially: no idle lanes, no lane exchange per vector.  The row's constants go to a small table in LDS,
//      and mean / rstd leave for global memory from here, consecutive rows from consecutive lanes;
//   3. flat pass again: every lane picks up the constants of the rows its J vectors belong to, finishes y (or dx)
//      from the vectors it still holds in registers and stores them, again in one contiguous piece per instruction.
//      In the backward the flat pass also adds to the lane's column sums of dW / dB: a lane's column group never
//      changes.
// The next batch is requested before the statistics pass and lands while passes 2 and 3 run.  No workgroup barrier in
// the loop: a wave executes its LDS instructions in order, so what its lanes write is there when its lanes read.
// A row's sums are added in an order that depends on L, J and nothing else: a row gives the same bits wherever it
// sits.  Everything else follows the row kernels: a persistent grid, no branch around a load or store (rows past the
// end are clamped onto the last row and masked out of dW / dB), float32 arithmetic, one float32 partial row of dW / dB
// per workgroup summed in a fixed order.  128-bit path only (N a whole number of vectors, 16-byte aligned rows).
#pragma once

#include "thn_dispatch.h"

namespace thn {

constexpr int kStagedBlock = 256;         // threads per workgroup
constexpr int kStagedGroup = 64;          // threads that share a batch of rows: one wave
constexpr int kStagedMaxVecs = 32;        // widest row (in vectors)
constexpr int kStagedMaxPasses = 4;       // J: flat passes (vectors per lane) per batch
constexpr int kStagedVecs = 1280;         // vectors of one tensor the four waves of a workgroup may hold in LDS (20 KiB:
                                          // the largest batch, 4 passes over rows of 4 vectors, is 320 per wave)

struct StagedGeom {
    int L;        // vectors per row
    int rpp;      // rows a flat pass of the wave covers: 64 / L
    int S;        // lanes with work in the flat passes: rpp * L
    int pitch;    // vectors between rows in LDS (odd)
    int R;        // rows per batch: J * rpp
    int P;        // lanes per row in the statistics pass: 1, 2, 4 or 8, R * P <= 64
    int log_p;
};
__host__ __device__ inline StagedGeom staged_geom(int L, int J) {
    StagedGeom g;
    g.L = L;
    g.rpp = kStagedGroup / L;
    g.S = g.rpp * L;
    g.pitch = L | 1;
    g.R = J * g.rpp;
    g.P = 1;
    g.log_p = 0;
    while (2 * g.P * g.R <= kStagedGroup && g.P < 8) {
        g.P *= 2;
        ++g.log_p;
    }
    return g;
}
// Whether a batch of J flat passes over rows of L vectors fits the kernels' LDS arrays and statistics threads.
__host__ __device__ inline bool staged_fits(int L, int J) {
    if (L < 1 || L > kStagedMaxVecs || J < 1 || J > kStagedMaxPasses) return false;
    const StagedGeom g = staged_geom(L, J);
    return g.R <= kStagedGroup && g.R * g.pitch <= kStagedVecs / (kStagedBlock / kStagedGroup);
}

// The lanes of a wave have written LDS that other lanes of the wave read next.  A wave executes its LDS instructions in
// order, so nothing needs to wait: the fences only keep the compiler from moving the accesses across this point.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Sum over the P consecutive lanes (P = 1, 2, 4, 8, the same for the whole workgroup) that share a row.
__device__ __forceinline__ float few_lanes_allreduce(float v, int P) {
    if (P >= 2) v += dpp_mov<0xB1>(v);     // lane ^ 1
    if (P >= 4) v += dpp_mov<0x4E>(v);     // lane ^ 2
    if (P >= 8) v += dpp_mov<0x141>(v);    // the other quad of each 8 lanes
    return v;
}

// The statistics pass's walk over a row in LDS: calls f(vector, counts) for the vectors sp, sp + P, ... of the row, four
// requested at a time while four remain, then one by one.  A lane whose last index falls past the row (only when P > 1)
// re-reads the row's last vector and is told not to count it.
template <typename F>
__device__ __forceinline__ void walk_row(const u32x4* rowp, int sp, int log_p, int L, int n_steps, F&& f) {
    int i = 0;
    for (; i + 4 <= n_steps; i += 4) {
        u32x4 v4[4];
        bool ok[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int v = sp + ((i + u) << log_p);
            ok[u] = v < L;
            v4[u] = rowp[ok[u] ? v : L - 1];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) f(v4[u], ok[u]);
    }
    for (; i < n_steps; ++i) {
        const int v = sp + (i << log_p);
        const bool ok = v < L;
        f(rowp[ok ? v : L - 1], ok);
    }
}

// The same over two tensors' copies of the row and the float32 weights of its columns, two vectors at a time.
template <int VEC, typename F>
__device__ __forceinline__ void walk_row_pair(const u32x4* xrow, const u32x4* grow, const float* wl, int sp, int log_p, int L,
                                              int n_steps, F&& f) {
    int i = 0;
    for (; i + 2 <= n_steps; i += 2) {
        u32x4 vx[2], vg[2];
        float wf[2][VEC];
        bool ok[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int v = sp + ((i + u) << log_p);
            ok[u] = v < L;
            const int vc = ok[u] ? v : L - 1;
            vx[u] = xrow[vc];
            vg[u] = grow[vc];
#pragma unroll
            for (int e = 0; e < VEC; ++e) wf[u][e] = wl[vc * VEC + e];
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) f(vx[u], vg[u], wf[u], ok[u]);
    }
    for (; i < n_steps; ++i) {
        const int v = sp + (i << log_p);
        const bool ok = v < L;
        const int vc = ok ? v : L - 1;
        float wf[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) wf[e] = wl[vc * VEC + e];
        f(xrow[vc], grow[vc], wf, ok);
    }
}

// Forward.  Arithmetic as norm_fwd_kernel (LayerNorm: mean0, then {sum d, sum d^2} with the delta correction).
template <typename T, bool LN, int J, bool KEEPX>
__global__ void __launch_bounds__(kStagedBlock) norm_staged_fwd_kernel(const FwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int NG = kStagedBlock / kStagedGroup;           // waves per workgroup
    __shared__ u32x4 xs_all[kStagedVecs];
    __shared__ float st_all[2][kStagedBlock][4];              // per row of the batch: mean0, delta, rstd

    const StagedGeom g = staged_geom(a.n_vecs, J);
    const int lane = threadIdx.x & (kStagedGroup - 1), wave = threadIdx.x / kStagedGroup;
    u32x4* xs = xs_all + wave * (kStagedVecs / NG);
    float (*st)[kStagedBlock][4] = reinterpret_cast<float (*)[kStagedBlock][4]>(&st_all[0][wave * kStagedGroup][0]);
    const int tf = lane < g.S ? lane : g.S - 1;                // a thread without work mirrors the last one that has some
    const int fr = tf / g.L, ft = tf - fr * g.L;             // flat passes: row within a pass, vector within the row
    const int voff = ft * 16;
    const int sr_raw = lane >> g.log_p, sp = lane & (g.P - 1); // statistics pass: row within the batch, place among its P threads
    const int sr = sr_raw < g.R ? sr_raw : g.R - 1;
    const int n_steps = (g.L + g.P - 1) >> g.log_p;           // vectors of a row per statistics thread

    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * NG * g.R;
    const int64_t last_row = a.M - 1;
    int64_t base = (static_cast<int64_t>(blockIdx.x) * NG + wave) * g.R;
    u32x4 cur[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
        int64_t r = base + j * g.rpp + fr;
        r = r < a.M ? r : last_row;
        cur[j] = slot_load<T, true, KEEPX>(a.x + r * a.x_stride_bytes, voff, a.n_cols);
    }
    float wr[1][VEC], br[1][VEC];
    const int pv[1] = {voff};
    load_params_clamped<1, VEC, true>(wr, a.w, a.w_dtype, pv, a.n_cols, 1.0f);
    if constexpr (LN) load_params_clamped<1, VEC, true>(br, a.b, a.w_dtype, pv, a.n_cols, 0.0f);
    drain_vector_memory(cur);

    int par = 0;
    for (; base < a.M; base += rows_per_iter) {
#pragma unroll
        for (int j = 0; j < J; ++j) xs[(j * g.rpp + fr) * g.pitch + ft] = cur[j];
        u32x4 nxt[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            int64_t r = base + rows_per_iter + j * g.rpp + fr;
            r = r < a.M ? r : last_row;
            nxt[j] = slot_load<T, true, KEEPX>(a.x + r * a.x_stride_bytes, voff, a.n_cols);
        }
        wave_sync();

        const u32x4* rowp = xs + sr * g.pitch;
        float mean0 = 0.0f, delta = 0.0f, rstd;
        if constexpr (LN) {
            float s = 0.0f;
            walk_row(rowp, sp, g.log_p, g.L, n_steps, [&](u32x4 v, bool counts) {
                float xf[VEC];
                T::unpack(v, xf);
                float sk = 0.0f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) sk += xf[e];
                s += counts ? sk : 0.0f;
            });
            s = few_lanes_allreduce(s, g.P);
            mean0 = s * a.inv_n;
            float q0 = 0.0f, q1 = 0.0f;
            walk_row(rowp, sp, g.log_p, g.L, n_steps, [&](u32x4 v, bool counts) {
                float xf[VEC];
                T::unpack(v, xf);
                float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float d = xf[e] - mean0;
                    a0 += d;
                    a1 = fmaf(d, d, a1);
                }
                q0 += counts ? a0 : 0.0f;
                q1 += counts ? a1 : 0.0f;
            });
            q0 = few_lanes_allreduce(q0, g.P);
            q1 = few_lanes_allreduce(q1, g.P);
            delta = q0 * a.inv_n;
            const float var = fmaxf(fmaf(-delta, delta, q1 * a.inv_n), 0.0f);
            rstd = rsqrt_refined(var + a.eps);
        } else {
            float q = 0.0f;
            walk_row(rowp, sp, g.log_p, g.L, n_steps, [&](u32x4 v, bool counts) {
                float xf[VEC];
                T::unpack(v, xf);
                float qk = 0.0f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) qk = fmaf(xf[e], xf[e], qk);
                q += counts ? qk : 0.0f;
            });
            q = few_lanes_allreduce(q, g.P);
            rstd = rsqrt_refined(fmaf(q, a.inv_n, a.eps));
        }
        st[par][sr][0] = mean0;
        st[par][sr][1] = delta;
        st[par][sr][2] = rstd;
        {
            // A row past the end of the matrix was loaded as a copy of the last row: its statistics are that row's,
            // stored once more to that row's place.
            int64_t r = base + sr;
            r = r < a.M ? r : last_row;
            if constexpr (LN) a.mean[r] = mean0 + delta;
            a.rstd[r] = rstd;
        }
        wave_sync();

#pragma unroll
        for (int j = 0; j < J; ++j) {
            const int rb = j * g.rpp + fr;
            const float m0 = st[par][rb][0], dl = st[par][rb][1], rs = st[par][rb][2];
            float xf[VEC], yf[VEC];
            T::unpack(cur[j], xf);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if constexpr (LN) yf[e] = fmaf(((xf[e] - m0) - dl) * rs, wr[0][e], br[0][e]);
                else yf[e] = xf[e] * rs * wr[0][e];
            }
            int64_t r = base + rb;
            r = r < a.M ? r : last_row;
            slot_store<T, true>(a.y + r * a.y_stride_bytes, voff, a.n_cols, yf);
        }
#pragma unroll
        for (int j = 0; j < J; ++j) cur[j] = nxt[j];
        par ^= 1;
    }
}

// Backward.  Arithmetic as norm_bwd_kernel: {sum u*wdy, sum wdy, sum u} per row in the statistics pass; dx and the
// per-thread column sums of dW / dB (float64 for float32 rows) in the flat pass; the workgroup adds the column sums
// of its threads at the end, in a fixed order, into ONE float32 partial row.
template <typename T, bool LN, int J>
__global__ void __launch_bounds__(kStagedBlock) norm_staged_bwd_kernel(const BwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int NG = kStagedBlock / kStagedGroup;
    using Acc = typename AccType<(T::kBytes >= 4)>::type;
    __shared__ u32x4 xs_all[kStagedVecs];
    __shared__ u32x4 gs_all[kStagedVecs];
    __shared__ float wl[kStagedMaxVecs * VEC];                // the weights as float32
    __shared__ float st_all[2][kStagedBlock][6];              // per row of the batch: rstd, c1, mean, delta', c2
    static_assert(sizeof(Acc) * kStagedBlock * VEC <= sizeof(u32x4) * kStagedVecs, "the column sums reuse xs / gs");

    const StagedGeom g = staged_geom(a.n_vecs, J);
    const int lane = threadIdx.x & (kStagedGroup - 1), wave = threadIdx.x / kStagedGroup;
    u32x4* xs = xs_all + wave * (kStagedVecs / NG);
    u32x4* gs = gs_all + wave * (kStagedVecs / NG);
    float (*st)[kStagedBlock][6] = reinterpret_cast<float (*)[kStagedBlock][6]>(&st_all[0][wave * kStagedGroup][0]);
    const bool works = lane < g.S;
    const int tf = works ? lane : g.S - 1;
    const int fr = tf / g.L, ft = tf - fr * g.L;
    const int voff = ft * 16;
    const int sr_raw = lane >> g.log_p, sp = lane & (g.P - 1);
    const int sr = sr_raw < g.R ? sr_raw : g.R - 1;
    const int n_steps = (g.L + g.P - 1) >> g.log_p;

    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * NG * g.R;
    const int64_t last_row = a.M - 1;
    int64_t base = (static_cast<int64_t>(blockIdx.x) * NG + wave) * g.R;
    u32x4 cx[J], cg[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
        int64_t r = base + j * g.rpp + fr;
        r = r < a.M ? r : last_row;
        cx[j] = slot_load<T, true>(a.x + r * a.x_stride_bytes, voff, a.n_cols);
        cg[j] = slot_load<T, true>(a.dy + r * a.dy_stride_bytes, voff, a.n_cols);
    }
    float c_mean, c_rstd;                                     // of the row this thread sums in the statistics pass
    {
        int64_t r = base + sr;
        r = r < a.M ? r : last_row;
        c_mean = LN ? a.mean[r] : 0.0f;
        c_rstd = a.rstd[r];
    }
    float wr[1][VEC];
    const int pv[1] = {voff};
    load_params_clamped<1, VEC, true>(wr, a.w, a.w_dtype, pv, a.n_cols, 1.0f);
    if (threadIdx.x < g.L) {                                   // (the first L threads of the workgroup own vectors 0 ... L - 1)
#pragma unroll
        for (int e = 0; e < VEC; ++e) wl[threadIdx.x * VEC + e] = wr[0][e];
    }
    __syncthreads();
    Acc dw[VEC], db[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) { dw[e] = Acc(0); db[e] = Acc(0); }
    if constexpr (LN) pin_loaded(c_mean);
    pin_loaded(c_rstd);
    drain_vector_memory(cx, cg);

    int par = 0;
    for (; base < a.M; base += rows_per_iter) {
#pragma unroll
        for (int j = 0; j < J; ++j) {
            xs[(j * g.rpp + fr) * g.pitch + ft] = cx[j];
            gs[(j * g.rpp + fr) * g.pitch + ft] = cg[j];
        }
        u32x4 nx[J], ng[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            int64_t r = base + rows_per_iter + j * g.rpp + fr;
            r = r < a.M ? r : last_row;
            nx[j] = slot_load<T, true>(a.x + r * a.x_stride_bytes, voff, a.n_cols);
            ng[j] = slot_load<T, true>(a.dy + r * a.dy_stride_bytes, voff, a.n_cols);
        }
        float n_mean, n_rstd;
        {
            int64_t r = base + rows_per_iter + sr;
            r = r < a.M ? r : last_row;
            n_mean = LN ? a.mean[r] : 0.0f;
            n_rstd = a.rstd[r];
        }
        wave_sync();

        const u32x4* xrow = xs + sr * g.pitch;
        const u32x4* grow = gs + sr * g.pitch;
        float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f;
        walk_row_pair<VEC>(xrow, grow, wl, sp, g.log_p, g.L, n_steps,
                           [&](u32x4 vx, u32x4 vg, const float (&wf)[VEC], bool counts) {
            float xf[VEC], gf[VEC];
            T::unpack(vx, xf);
            T::unpack(vg, gf);
            float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float uu = LN ? (xf[e] - c_mean) * c_rstd : xf[e] * c_rstd;
                const float wdy = wf[e] * gf[e];
                a0 = fmaf(uu, wdy, a0);
                if constexpr (LN) {
                    a1 += wdy;
                    a2 += uu;
                }
            }
            s0 += counts ? a0 : 0.0f;
            if constexpr (LN) {
                s1 += counts ? a1 : 0.0f;
                s2 += counts ? a2 : 0.0f;
            }
        });
        s0 = few_lanes_allreduce(s0, g.P);
        float c1, c2 = 0.0f, dlt = 0.0f;
        if constexpr (LN) {
            s1 = few_lanes_allreduce(s1, g.P);
            s2 = few_lanes_allreduce(s2, g.P);
            dlt = s2 * a.inv_n;
            c2 = s1 * a.inv_n;
            c1 = fmaf(-dlt, c2, s0 * a.inv_n);
        } else {
            c1 = s0 * a.inv_n;
        }
        st[par][sr][0] = c_rstd;
        st[par][sr][1] = c1;
        if constexpr (LN) {
            st[par][sr][2] = c_mean;
            st[par][sr][3] = dlt;
            st[par][sr][4] = c2;
        }
        wave_sync();

#pragma unroll
        for (int j = 0; j < J; ++j) {
            const int rb = j * g.rpp + fr;
            const float rs = st[par][rb][0], k1 = st[par][rb][1];
            float mn = 0.0f, dl = 0.0f, k2 = 0.0f;
            if constexpr (LN) {
                mn = st[par][rb][2];
                dl = st[par][rb][3];
                k2 = st[par][rb][4];
            }
            const int64_t r_raw = base + rb;
            const int64_t r = r_raw < a.M ? r_raw : last_row;
            const bool adds = works && r_raw < a.M;          // a mirror thread or a row past the end adds nothing to dW / dB
            float xf[VEC], gf[VEC], dxf[VEC];
            T::unpack(cx[j], xf);
            T::unpack(cg[j], gf);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float xhat = LN ? (xf[e] - mn) * rs : xf[e] * rs;
                if constexpr (LN) xhat -= dl;
                const float wdy = wr[0][e] * gf[e];
                dxf[e] = (wdy - fmaf(xhat, k1, k2)) * rs;
                const float gl = adds ? gf[e] : 0.0f;
                dw[e] = fma(static_cast<Acc>(gl), static_cast<Acc>(xhat), dw[e]);
                if constexpr (LN) db[e] += static_cast<Acc>(gl);
            }
            slot_store<T, true>(a.dx + r * a.dx_stride_bytes, voff, a.n_cols, dxf);
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            cx[j] = nx[j];
            cg[j] = ng[j];
        }
        c_mean = n_mean;
        c_rstd = n_rstd;
        par ^= 1;
    }

    // The workgroup's partial row: column c = t * VEC + e is the sum over the threads that own vector t (one per row of a
    // flat pass), added by one thread per column in a fixed order.
    __syncthreads();
    Acc* tw = reinterpret_cast<Acc*>(xs_all);
    Acc* tb = reinterpret_cast<Acc*>(gs_all);
    const bool want_dw = a.dw_part != nullptr;
    const bool want_db = LN && a.db_part != nullptr;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        tw[threadIdx.x * VEC + e] = dw[e];
        tb[threadIdx.x * VEC + e] = LN ? db[e] : Acc(0);
    }
    __syncthreads();
    for (int c = threadIdx.x; c < a.n_cols; c += kStagedBlock) {
        const int t = c / VEC, e = c - t * VEC;
        Acc sw = Acc(0), sb = Acc(0);
        for (int gi = 0; gi < NG; ++gi) {
            for (int r = 0; r < g.rpp; ++r) {
                const int src = gi * kStagedGroup + r * g.L + t;
                sw += tw[src * VEC + e];
                sb += tb[src * VEC + e];
            }
        }
        const int64_t off = static_cast<int64_t>(blockIdx.x) * a.part_pitch + c;
        if (want_dw) a.dw_part[off] = static_cast<float>(sw);
        if (want_db) a.db_part[off] = static_cast<float>(sb);
    }
}

// Launchers: 0 launched (or occupancy written), 1 no such instance, <0 HIP error.  `passes` = J, the flat passes per batch.
#define THN_DECLARE_STAGED_LAUNCHERS(NAME)                                                                      \
    int launch_staged_fwd_##NAME(bool ln, int passes, const FwdArgs& a, int grid, hipStream_t st, int* occupancy); \
    int launch_staged_bwd_##NAME(bool ln, int passes, const BwdArgs& a, int grid, hipStream_t st, int* occupancy);

THN_DECLARE_STAGED_LAUNCHERS(f32)
THN_DECLARE_STAGED_LAUNCHERS(f16)
THN_DECLARE_STAGED_LAUNCHERS(bf16)

#define THN_STAGED_FWD_CASE(J_)                                                                                 \
    if (passes == J_) {                                                                                         \
        if (a.keep_x) {                                                                                         \
            return ln ? run_kernel<FwdArgs>(norm_staged_fwd_kernel<T, true, J_, true>, a, grid, kStagedBlock, st, occupancy)  \
                      : run_kernel<FwdArgs>(norm_staged_fwd_kernel<T, false, J_, true>, a, grid, kStagedBlock, st, occupancy); \
        }                                                                                                       \
        return ln ? run_kernel<FwdArgs>(norm_staged_fwd_kernel<T, true, J_, false>, a, grid, kStagedBlock, st, occupancy)     \
                  : run_kernel<FwdArgs>(norm_staged_fwd_kernel<T, false, J_, false>, a, grid, kStagedBlock, st, occupancy);   \
    }
#define THN_STAGED_BWD_CASE(J_)                                                                                 \
    if (passes == J_) {                                                                                         \
        return ln ? run_kernel<BwdArgs>(norm_staged_bwd_kernel<T, true, J_>, a, grid, kStagedBlock, st, occupancy)   \
                  : run_kernel<BwdArgs>(norm_staged_bwd_kernel<T, false, J_>, a, grid, kStagedBlock, st, occupancy);  \
    }
// flat passes per batch
#define THN_STAGED_PASSES(X) X(1) X(2) X(3) X(4)

#define THN_DEFINE_STAGED_LAUNCHERS(NAME, TYPE)                                                                 \
    int launch_staged_fwd_##NAME(bool ln, int passes, const FwdArgs& a, int grid, hipStream_t st, int* occupancy) { \
        using T = TYPE;                                                                                         \
        THN_STAGED_PASSES(THN_STAGED_FWD_CASE)                                                                  \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_staged_bwd_##NAME(bool ln, int passes, const BwdArgs& a, int grid, hipStream_t st, int* occupancy) { \
        using T = TYPE;                                                                                         \
        THN_STAGED_PASSES(THN_STAGED_BWD_CASE)                                                                  \
        return 1;                                                                                               \
    }

}  // namespace thn
