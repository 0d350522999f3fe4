// The forward and backward row kernels.
//
// Work decomposition (the same for both): a row of N elements is 16-byte "vectors"; TPR threads share a
// row and thread t owns vectors t, t+TPR, ..., t+(K-1)*TPR, so a wave touches contiguous 1 KiB segments.
// A workgroup of BLOCK threads holds G = BLOCK/TPR rows at a time and walks the matrix with a grid stride
// of gridDim.x*G rows (a persistent grid: the whole chip works on one contiguous window of rows at any
// moment).  A row lives in registers between its load and its store: x (and dy) are read from HBM exactly
// once per pass.
//
// The row loop is branch free on the 128-bit path.  The vectors of the NEXT row are requested before the
// current row is reduced, and the hardware returns vector-memory operations in issue order, so the only
// wait in the loop is "all but the newest loads have landed" (s_waitcnt vmcnt(n)); any branch around a load
// or store would force the compiler to wait for everything (vmcnt(0)) and serialise the loop on memory
// latency.  To stay branch free, slots that have no work -- a row past the end in the last grid-stride
// step, a vector slot past the row end when K*TPR > N/VEC -- are CLAMPED onto the last valid row / vector:
// they load, compute and store exactly what the owner of that row / vector does (same inputs, same
// instruction sequence, hence the same bits to the same address), and are only masked out of the row sums
// and of the dW / dB accumulators.
#pragma once

#include <type_traits>

#include "thn_act_math.h"
#include "thn_device.h"

namespace thn {

constexpr int kNoAct = -1;   // ACT of the norm kernels: no activation epilogue

struct FwdArgs {
    const char* x;
    char* y;
    const void* w;      // may be null
    const void* b;      // may be null
    float* mean;        // null for RMSNorm
    float* rstd;
    int64_t x_stride_bytes;
    int64_t y_stride_bytes;
    int64_t M;
    int n_cols;         // N
    int n_vecs;         // ceil(N / VEC)
    int w_dtype;
    float eps;
    float inv_n;
    int line_shift;     // 1: rows are not 128 bytes apart and the launch may use row_line_shift()
    int keep_x;         // host side only: selects the KEEPX instance (thn_norm_set_cache_policy)
};

struct BwdArgs {
    const char* x;
    const char* dy;
    char* dx;
    const void* w;      // may be null
    const void* b;      // may be null; read only by the activation-epilogue instances (to recompute the pre-activation)
    const float* mean;  // null for RMSNorm
    const float* rstd;
    float* dw_part;     // (gridDim.x, part_pitch) float32, may be null
    float* db_part;     // (gridDim.x, part_pitch) float32, may be null
    int64_t x_stride_bytes;
    int64_t dy_stride_bytes;
    int64_t dx_stride_bytes;
    int64_t M;
    int64_t part_pitch; // floats between partial rows
    int n_cols;
    int n_vecs;
    int w_dtype;
    float inv_n;
    int line_shift;     // as in FwdArgs
};

// Rows that are a multiple of 16 but not of 128 bytes apart start in the middle of a 128-byte line, and a wave's
// 1 KiB request then touches nine lines instead of eight (float32 8192 x 6000: 9 % of the kernel).  Where the
// host has checked that it may -- one row per workgroup at a time, the same phase for every row the workgroup
// visits and for every stream, K*TPR - 7 >= n_vecs -- the threads take the vectors `shift` places further left
// (thread t owns vectors t - shift + k*TPR), which puts every request of a wave on line boundaries; the slots that
// fall off the left end are clamped onto vector 0 like those off the right end onto the last one.
__device__ __forceinline__ int row_line_shift(int enabled, const char* base, int64_t stride_bytes, int64_t first_row) {
    if (!enabled) return 0;
    return static_cast<int>(((reinterpret_cast<uintptr_t>(base) + static_cast<uint64_t>(first_row * stride_bytes)) & 127u) >> 4);
}

// Vector slots of the norm kernels.  Three I/O modes, fixed at compile time:
//   ALIGNED                      the 128-bit path: slot v is bytes [16 v, 16 v + 16) of the row;
//   !ALIGNED, T::kWindowIo       rows off that path that hold at least one vector: slot v is the 16-byte window of
//                                VEC columns that starts at column min(v * VEC, N - VEC) -- whole inside the row, at
//                                any element-aligned address.  Only the ragged last slot of a row is moved: its
//                                window ends at the row end and OVERLAPS the slot before it by `lead` columns.  Those
//                                columns are loaded, computed and stored a second time -- the same inputs through the
//                                same instructions, so the same bits to the same bytes as their owner writes -- and
//                                only left out of the row sums and of the dW / dB sums.  No shifting of registers, no
//                                branch around the ragged store: the loop keeps its exact s_waitcnt, like the
//                                128-bit path;
//   !ALIGNED, !T::kWindowIo      rows shorter than one vector (ElemIo<T>): element accesses with a column bound.
// voff is the slot's byte offset in a row in the first two modes and its vector index in the third.
template <typename T, bool ALIGNED, bool KEEP = false>
__device__ __forceinline__ u32x4 slot_load(const char* rowp, int voff, int n_cols) {
    if constexpr (ALIGNED) return KEEP ? ld128_keep(rowp + voff) : ld128(rowp + voff);
    else if constexpr (T::kWindowIo) return KEEP ? ld128u_keep(rowp + voff) : ld128u(rowp + voff);
    else return load_vec_elems<T, KEEP>(rowp, voff, n_cols);
}

template <typename T, int K, bool ALIGNED, bool KEEP = false>
__device__ __forceinline__ void slot_load_row(u32x4 (&dst)[K], const char* base, int64_t stride_bytes, int64_t row,
                                              const int (&voff)[K], int n_cols) {
    const char* p = base + row * stride_bytes;
#pragma unroll
    for (int k = 0; k < K; ++k) dst[k] = slot_load<T, ALIGNED, KEEP>(p, voff[k], n_cols);
}

// The 16 bytes of a slot on the 128-bit path or as an unaligned window.  KEEP: with an ordinary (cache-allocating)
// store instead of a streaming one, for an output that the operator's backward reads again (see ld128_keep).
template <bool ALIGNED, bool KEEP = false>
__device__ __forceinline__ void slot_store_bits(char* p, u32x4 bits) {
    if constexpr (ALIGNED) {
        if constexpr (KEEP) st128_keep(p, bits);
        else st128(p, bits);
    } else {
        if constexpr (KEEP) st128u_keep(p, bits);
        else st128u(p, bits);
    }
}

template <typename T, bool ALIGNED, bool KEEP = false>
__device__ __forceinline__ void slot_store(char* rowp, int voff, int n_cols, const float (&f)[T::VEC]) {
    if constexpr (ALIGNED || T::kWindowIo) slot_store_bits<ALIGNED, KEEP>(rowp + voff, T::pack(f));
    else store_vec_elems<T>(rowp, voff, n_cols, f);
}

// Offset, overlap and ownership of vector slot v of a row (v may lie outside [0, n_vecs): a slot without work is
// clamped onto the nearest one and mirrors it).
template <typename T, bool ALIGNED>
__device__ __forceinline__ void slot_place(int v, int n_vecs, int n_cols, int& voff, int& lead, bool& own) {
    const int vc = v < 0 ? 0 : (v < n_vecs ? v : n_vecs - 1);
    own = v >= 0 && v < n_vecs;
    lead = 0;
    if constexpr (ALIGNED) {
        voff = vc * 16;
    } else if constexpr (T::kWindowIo) {
        const int c0 = vc * T::VEC, last = n_cols - T::VEC;
        const int cw = c0 < last ? c0 : last;
        voff = cw * T::kBytes;
        lead = c0 - cw;
    } else {
        voff = vc;
    }
}

// Whether element e of a slot is a column that this slot owns (and therefore counts in sums).
template <typename T, bool ALIGNED>
__device__ __forceinline__ bool slot_counts(int voff, int lead, int e, int n_cols) {
    if constexpr (ALIGNED) return true;
    else if constexpr (T::kWindowIo) return e >= lead;
    else return voff * T::VEC + e < n_cols;
}

template <typename T, int K, bool ALIGNED>
__device__ __forceinline__ void slot_params(float (&out)[K][T::VEC], const void* p, int dtype, const int (&voff)[K],
                                            int n_cols, float fill) {
    if constexpr (!ALIGNED && T::kWindowIo) load_params_window<K, T::VEC>(out, p, dtype, voff, fill);
    else load_params_clamped<K, T::VEC, ALIGNED>(out, p, dtype, voff, n_cols, fill);
}

// Workgroups of 1024 threads serve the widest rows (more than 24 KiB of x in the backward, 32 KiB in the
// forward) and have 128 registers per thread.  Holding a row as float32 next to the packed next row, the
// parameters and the column accumulators does not always fit there, and a kernel that spills to scratch
// memory loses more than half of its bandwidth.  Instances that would spill run a leaner form of the row loop,
// chosen at compile time from three independent savings, in the order of what they cost in speed:
//   recompute: only the packed 16-byte vectors of the row stay live across a reduction round; every pass
//              unpacks them again (the same instructions on the same inputs, so the same bits);
//   lds_dw:    (backward, 16-bit rows) the dW sums of a thread live in LDS, in slots no other thread touches;
//   !ahead:    the next row is not requested a whole row ahead: vector k of the next row is loaded into the
//              registers of vector k as soon as that one has been stored (4-16 % slower where the row-ahead
//              form fits, so it is the last resort).
// The LayerNorm backward of 16-bit rows wider than 32 KiB runs in 512-thread workgroups instead (5 to 8 vectors
// per thread, 256 registers): its weights and dB sums alone take 80 to 128 registers; it uses the same forms.
struct RowForm {
    bool recompute, ahead, lds_dw;
};
constexpr RowForm kPlainForm{false, true, false};

template <int BYTES, bool LN, int K, int BLOCK, bool FUSED>
constexpr RowForm fwd_form() {
    if (BLOCK < 1024) return kPlainForm;
    if (BYTES == 2 && LN && K == 4) return RowForm{true, true, false};
    if (FUSED && BYTES == 2 && K == 4) return RowForm{true, true, false};
    return kPlainForm;
}

template <int BYTES, bool LN, int K, int BLOCK, bool FUSED>
constexpr RowForm bwd_form() {
    if (BYTES == 2 && LN && K >= 5) return RowForm{true, K <= 6 && !FUSED, true};      // 512-thread workgroups
    if (BLOCK < 1024) return kPlainForm;
    if (BYTES >= 4) {
        if (K == 4) return RowForm{true, !LN, false};
        return (FUSED && LN && K == 3) ? RowForm{true, false, false} : kPlainForm;
    }
    if (K == 1) return kPlainForm;
    if (K == 2) return (LN || FUSED) ? RowForm{true, !(LN && FUSED), false} : kPlainForm;
    return RowForm{true, !LN, true};     // K = 3, 4: rows of more than 32 KiB
}

// Makes the compiler forget what it has derived from the packed vectors, so that the next pass really
// unpacks them again instead of keeping the float32 values of the previous pass in registers.  No instruction.
template <int K>
__device__ __forceinline__ void forget_derived(u32x4 (&v)[K]) {
#pragma unroll
    for (int k = 0; k < K; ++k) asm volatile("" : "+v"(v[k]));
}

// ---------------------------------------------------------------------------------------------------
// Forward.  LayerNorm: mean0 = sum(x)/N; d = x - mean0; delta = sum(d)/N; var = sum(d^2)/N - delta^2;
// rstd = 1/sqrt(var + eps); y = (d - delta)*rstd*w + b; saved mean = mean0 + delta.  The second pass runs
// on registers; carrying delta (the float32 rounding error of mean0) keeps y accurate when |mean| >> std.
// RMSNorm: rstd = 1/sqrt(sum(x^2)/N + eps); y = x*rstd*w.
// ---------------------------------------------------------------------------------------------------
// ACT != kNoAct: y = act(normalise(x)*w + b) -- the activation (one of the parameter-free, input-saving ones of
// thn_act_math.h) is applied to the float32 value before the one rounding on store; nothing else changes.
// KEEPX: x is loaded with ordinary (cache-allocating) loads because the operator's backward reads it again (see
// ld128_keep); false: with streaming loads, for a forward that no backward follows closely.  The two forms differ in
// that hint on the load instructions and in nothing else: same arithmetic, same bits.
template <typename T, bool LN, int K, int TPR, int BLOCK, bool ALIGNED, int ACT = kNoAct, bool KEEPX = true>
__global__ void __launch_bounds__(BLOCK) norm_fwd_kernel(const FwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int G = BLOCK / TPR;
    constexpr bool kKeepX = KEEPX;
    static_assert(BLOCK % TPR == 0 && G >= 1, "a workgroup holds whole rows");
    __shared__ float red[RedSmem<TPR, G, 2>::kFloats];

    const int tid = threadIdx.x;
    const int g = tid / TPR;
    const int t = tid % TPR;
    int phase = 0;

    // Per-slot masks (1 = this thread owns real columns there) and clamped offsets.
    const int shift = (ALIGNED && G == 1) ? row_line_shift(a.line_shift, a.x, a.x_stride_bytes, blockIdx.x) : 0;
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
    u32x4 cur[K];
    slot_load_row<T, K, ALIGNED, kKeepX>(cur, a.x, a.x_stride_bytes, row, voff, a.n_cols);   // first, so it overlaps the params

    // Parameters of the clamped slot, so that a clamped slot reproduces its owner's output bit for bit.
    float wr[K][VEC];
    float br[LN ? K : 1][VEC];
    slot_params<T, K, ALIGNED>(wr, a.w, a.w_dtype, voff, a.n_cols, 1.0f);
    if constexpr (LN) slot_params<T, K, ALIGNED>(br, a.b, a.w_dtype, voff, a.n_cols, 0.0f);

    drain_vector_memory(cur);
    constexpr RowForm kForm = fwd_form<T::kBytes, LN, K, BLOCK, ACT != kNoAct>();
    if constexpr (kForm.recompute) {
        for (int64_t base = static_cast<int64_t>(blockIdx.x) * G; base < a.M; base += rows_per_iter) {
            const int64_t nrow_raw = row_raw + rows_per_iter;
            const int64_t nrow = nrow_raw < a.M ? nrow_raw : last_row;
            const char* nxrow = a.x + nrow * a.x_stride_bytes;
            u32x4 nxt[kForm.ahead ? K : 1];
            if constexpr (kForm.ahead) {
#pragma unroll
                for (int k = 0; k < K; ++k) nxt[k] = slot_load<T, ALIGNED, kKeepX>(nxrow, voff[k], a.n_cols);
            }
            float mean0 = 0.0f, mean = 0.0f, rstd, delta = 0.0f;
            if constexpr (LN) {
                float s[1] = {0.0f};
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    float xf[VEC];
                    T::unpack(cur[k], xf);
                    float sk = 0.0f;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) sk += counts(k, e) ? xf[e] : 0.0f;
                    s[0] += own[k] ? sk : 0.0f;
                }
                row_allreduce<TPR, G, 1>(s, red, phase, g, t);
                forget_derived(cur);
                mean0 = s[0] * a.inv_n;
                float q[2] = {0.0f, 0.0f};
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    float xf[VEC];
                    T::unpack(cur[k], xf);
                    float q0 = 0.0f, q1 = 0.0f;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        float d = xf[e] - mean0;
                        d = counts(k, e) ? d : 0.0f;
                        q0 += d;
                        q1 = fmaf(d, d, q1);
                    }
                    q[0] += own[k] ? q0 : 0.0f;
                    q[1] += own[k] ? q1 : 0.0f;
                }
                row_allreduce<TPR, G, 2>(q, red, phase, g, t);
                forget_derived(cur);
                delta = q[0] * a.inv_n;
                const float var = fmaxf(fmaf(-delta, delta, q[1] * a.inv_n), 0.0f);
                rstd = rsqrt_refined(var + a.eps);
                mean = mean0 + delta;
            } else {
                float q[1] = {0.0f};
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    float xf[VEC];
                    T::unpack(cur[k], xf);
                    float qk = 0.0f;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const float xm = counts(k, e) ? xf[e] : 0.0f;
                        qk = fmaf(xm, xm, qk);
                    }
                    q[0] += own[k] ? qk : 0.0f;
                }
                row_allreduce<TPR, G, 1>(q, red, phase, g, t);
                forget_derived(cur);
                rstd = rsqrt_refined(fmaf(q[0], a.inv_n, a.eps));
            }
            char* yrow = a.y + row * a.y_stride_bytes;
#pragma unroll
            for (int k = 0; k < K; ++k) {
                float xf[VEC], yf[VEC];
                T::unpack(cur[k], xf);
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    if constexpr (LN) {
                        const float d = xf[e] - mean0;       // every column of the slot is stored: none is masked here
                        yf[e] = fmaf((d - delta) * rstd, wr[k][e], br[k][e]);
                    } else {
                        yf[e] = xf[e] * rstd * wr[k][e];
                    }
                    if constexpr (ACT != kNoAct) yf[e] = act_fwd<ACT, float>(yf[e], 0.0f, 0.0f);
                }
                slot_store<T, ALIGNED>(yrow, voff[k], a.n_cols, yf);
                if constexpr (kForm.ahead) cur[k] = nxt[k];
                else cur[k] = slot_load<T, ALIGNED, kKeepX>(nxrow, voff[k], a.n_cols);
            }
            if constexpr (LN) a.mean[row] = mean;
            a.rstd[row] = rstd;
            row_raw = nrow_raw;
            row = nrow;
        }
        return;
    }
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * G; base < a.M; base += rows_per_iter) {
        const int64_t nrow_raw = row_raw + rows_per_iter;
        const int64_t nrow = nrow_raw < a.M ? nrow_raw : last_row;
        u32x4 nxt[K];
        // One row of 4 x 256 vectors per 256-thread workgroup: the previous row's stores are waited for before the next
        // row is requested, so that a workgroup's writes and reads reach memory in turns (bf16 32768 / 65536 rows of
        // 8192: RMSNorm 180.9 / 371.6 -> 175.8 / 363.5 us, LayerNorm 183.5 / 376.6 -> 177.4 / 365.9; float32 16384 x 4096
        // 0.8 % faster; 8192 x 8192 bf16 the same).  Only this shape: one row of 4 x 512 vectors in 512 threads loses
        // 3-5 % with the same wait from 8192 rows on, the other forward shapes +-1 %, and the backward shapes with one
        // row per workgroup lose 2-6 %.
        if constexpr (G == 1 && ALIGNED && K == 4 && BLOCK == 256) __builtin_amdgcn_s_waitcnt(0x0F70);
        slot_load_row<T, K, ALIGNED, kKeepX>(nxt, a.x, a.x_stride_bytes, nrow, voff, a.n_cols);

        float xf[K][VEC];
#pragma unroll
        for (int k = 0; k < K; ++k) T::unpack(cur[k], xf[k]);

        float mean = 0.0f, rstd, delta = 0.0f;
        if constexpr (LN) {
            float s[1] = {0.0f};
#pragma unroll
            for (int k = 0; k < K; ++k) {
                float sk = 0.0f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) sk += counts(k, e) ? xf[k][e] : 0.0f;
                s[0] += own[k] ? sk : 0.0f;
            }
            row_allreduce<TPR, G, 1>(s, red, phase, g, t);
            const float mean0 = s[0] * a.inv_n;
            float q[2] = {0.0f, 0.0f};
#pragma unroll
            for (int k = 0; k < K; ++k) {
                float q0 = 0.0f, q1 = 0.0f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float d = xf[k][e] - mean0;
                    xf[k][e] = d;                                   // kept for the output of every column of the slot
                    const float dm = counts(k, e) ? d : 0.0f;
                    q0 += dm;
                    q1 = fmaf(dm, dm, q1);
                }
                q[0] += own[k] ? q0 : 0.0f;
                q[1] += own[k] ? q1 : 0.0f;
            }
            row_allreduce<TPR, G, 2>(q, red, phase, g, t);
            delta = q[0] * a.inv_n;
            const float var = fmaxf(fmaf(-delta, delta, q[1] * a.inv_n), 0.0f);
            rstd = rsqrt_refined(var + a.eps);
            mean = mean0 + delta;
        } else {
            float q[1] = {0.0f};
#pragma unroll
            for (int k = 0; k < K; ++k) {
                float qk = 0.0f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float xm = counts(k, e) ? xf[k][e] : 0.0f;
                    qk = fmaf(xm, xm, qk);
                }
                q[0] += own[k] ? qk : 0.0f;
            }
            row_allreduce<TPR, G, 1>(q, red, phase, g, t);
            rstd = rsqrt_refined(fmaf(q[0], a.inv_n, a.eps));
        }

        char* yrow = a.y + row * a.y_stride_bytes;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            float yf[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if constexpr (LN) yf[e] = fmaf((xf[k][e] - delta) * rstd, wr[k][e], br[k][e]);
                else yf[e] = xf[k][e] * rstd * wr[k][e];
                if constexpr (ACT != kNoAct) yf[e] = act_fwd<ACT, float>(yf[e], 0.0f, 0.0f);
            }
            slot_store<T, ALIGNED>(yrow, voff[k], a.n_cols, yf);
        }
        // Every thread of the row stores the same two words to the same address (one request per wave): a
        // store under "if (t == 0)" would be a branch, see the note on branches at the top of this file.
        if constexpr (LN) a.mean[row] = mean;
        a.rstd[row] = rstd;

#pragma unroll
        for (int k = 0; k < K; ++k) cur[k] = nxt[k];
        row_raw = nrow_raw;
        row = nrow;
    }
}

// ---------------------------------------------------------------------------------------------------
// Backward.  With m, r the saved float32 mean and rstd of the row:
//   u = (x - m)*r (x*r for RMSNorm); wdy = w*dy; one reduction round of {sum(u*wdy), sum(wdy), sum(u)};
//   LayerNorm: dlt = sum(u)/N (the part of the mean that float32 m could not hold), xhat = u - dlt,
//              c2 = sum(wdy)/N, c1 = sum(u*wdy)/N - dlt*c2  (= sum(xhat*wdy)/N);
//   RMSNorm:   xhat = u, c1 = sum(u*wdy)/N, c2 = 0;
//   dx = (wdy - (xhat*c1 + c2))*r;  dW += dy*xhat;  dB += dy  (per-thread column accumulators).
// After the row loop the G row groups of the workgroup are summed through LDS in a fixed binary tree and the
// workgroup writes ONE float32 partial row of dW (and dB): no atomics, run-to-run deterministic.
// ---------------------------------------------------------------------------------------------------
template <bool WIDE> struct AccType { using type = double; };
template <> struct AccType<false> { using type = float; };

template <int BLOCK, int TPR, int VEC, typename Acc>
__device__ __forceinline__ void combine_groups(Acc (&acc)[VEC], Acc* comb, int g, int t) {
    constexpr int G = BLOCK / TPR;
    constexpr int HALF = BLOCK / 2;
#pragma unroll
    for (int stride = G / 2; stride >= 1; stride >>= 1) {
        if (g >= stride && g < 2 * stride) {
            const int slot = (g - stride) * TPR + t;
#pragma unroll
            for (int e = 0; e < VEC; ++e) comb[e * HALF + slot] = acc[e];
        }
        __syncthreads();
        if (g < stride) {
            const int slot = g * TPR + t;
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] += comb[e * HALF + slot];
        }
        __syncthreads();
    }
}

// One vector slot of a partial row.  The workspace is 16-byte aligned, the partial rows are a multiple of 256
// bytes apart and a slot starts a multiple of VEC floats into its row: 16-byte stores.  They are ordinary
// (cache-allocating) stores: the second stage reads the rows a few microseconds later, and what is written this way
// is still in the memory-side cache then (fp16 4096 x 16384, 16 MiB of partial rows: both stages 81.3 -> 78.5 us;
// bf16 16384 x 4096: step 105.4 -> 104.6 us; as streaming stores the rows went to HBM and came back from there).
// As 4-byte-per-lane stores they had cost the LayerNorm backward 2 us at 4096 columns, in either form.
template <int VEC>
__device__ __forceinline__ void store_partial(float* dst, const float (&f)[VEC]) {
    if constexpr (VEC % 4 == 0) {
#pragma unroll
        for (int e = 0; e < VEC; e += 4) {
            st128_keep(dst + e, u32x4{as_u32(f[e]), as_u32(f[e + 1]), as_u32(f[e + 2]), as_u32(f[e + 3])});
        }
    } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) dst[e] = f[e];
    }
}

// ACT != kNoAct: the forward was y = act(z), z = xhat*w + b.  The pre-activation is not stored: the kernel
// recomputes z from the saved statistics and replaces the upstream gradient by dy * act'(z) before anything else
// uses it.  z needs the corrected xhat, so LayerNorm takes one more reduction round (sum(u) first); the loop is
// still bound by memory.
template <typename T, bool LN, int K, int TPR, int BLOCK, bool ALIGNED, int ACT = kNoAct>
__global__ void __launch_bounds__(BLOCK) norm_bwd_kernel(const BwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int G = BLOCK / TPR;
    constexpr bool FUSED = ACT != kNoAct;
    constexpr int NV = LN ? (FUSED ? 2 : 3) : 1;      // fused LayerNorm: sum(u) has its own round
    static_assert(BLOCK % TPR == 0 && G >= 1, "a workgroup holds whole rows");
    // (fused LayerNorm calls row_allreduce with 1 value, then with 2, once each per row: the two calls always use
    // opposite halves of the double buffer, as in the forward kernel, so their different slot strides never overlap)
    __shared__ float red[RedSmem<TPR, G, NV>::kFloats];
    // Column accumulators: float64 for float32 / float64 rows in workgroups that have the registers (a
    // workgroup adds up to M/gridDim.x rows per column; float32 accumulators lose about 10 ulp of the final
    // float32 dW at a million rows, float64 ones leave only the error the float32 xhat terms carry anyway,
    // about 2^-24 * sqrt(M)).  16-bit rows accumulate in float32: the loop is VALU-latency sensitive (each
    // instruction per element costs about 1 % of the kernel) and the extra digits would not survive a 16-bit
    // dW.  A 1024-thread workgroup has 128 registers per thread and serves rows of 24 KiB and more (few rows
    // per workgroup): float32 too.
    constexpr bool kWideTotals = BLOCK < 1024 && T::kBytes >= 4;
    using Acc = typename AccType<kWideTotals>::type;
    __shared__ Acc comb[G > 1 ? VEC * (BLOCK / 2) : 1];

    const int tid = threadIdx.x;
    const int g = tid / TPR;
    const int t = tid % TPR;
    int phase = 0;

    const int shift = (ALIGNED && G == 1) ? row_line_shift(a.line_shift, a.x, a.x_stride_bytes, blockIdx.x) : 0;
    int voff[K], lead[K];
    bool own[K];
#pragma unroll
    for (int k = 0; k < K; ++k) slot_place<T, ALIGNED>(t + k * TPR - shift, a.n_vecs, a.n_cols, voff[k], lead[k], own[k]);
    // element e of slot k counts in the row sums and in dW / dB (always true on the 128-bit path)
    auto counts = [&](int k, int e) -> bool { return slot_counts<T, ALIGNED>(voff[k], lead[k], e, a.n_cols); };

    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * G;
    const int64_t last_row = a.M - 1;
    int64_t row_raw = static_cast<int64_t>(blockIdx.x) * G + g;
    int64_t row = row_raw < a.M ? row_raw : last_row;
    u32x4 cx[K], cg[K];
    slot_load_row<T, K, ALIGNED>(cx, a.x, a.x_stride_bytes, row, voff, a.n_cols);    // first, so they overlap the params
    slot_load_row<T, K, ALIGNED>(cg, a.dy, a.dy_stride_bytes, row, voff, a.n_cols);
    float c_mean = LN ? a.mean[row] : 0.0f;
    float c_rstd = a.rstd[row];

    // RowForm::lds_dw: the dW sums of a thread (24 or 32 floats) live in LDS, in slots that only this thread
    // touches (no barrier), 16 bytes per access.
    constexpr RowForm kForm = bwd_form<T::kBytes, LN, K, BLOCK, FUSED>();
    constexpr bool kLdsTotals = kForm.lds_dw;
    static_assert(!kLdsTotals || (G == 1 && VEC == 8), "one row per workgroup, eight columns per vector");
    __shared__ f32x4 dw_lds[kLdsTotals ? K * 2 * BLOCK : 1];

    float wr[K][VEC];
    Acc dw[kLdsTotals ? 1 : K][VEC];
    Acc db[LN ? K : 1][VEC];
    slot_params<T, K, ALIGNED>(wr, a.w, a.w_dtype, voff, a.n_cols, 1.0f);
    float br[(FUSED && LN) ? K : 1][VEC];
    if constexpr (FUSED && LN) slot_params<T, K, ALIGNED>(br, a.b, a.w_dtype, voff, a.n_cols, 0.0f);
#pragma unroll
    for (int k = 0; k < K; ++k) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            if constexpr (!kLdsTotals) dw[k][e] = Acc(0);
            if constexpr (LN) db[k][e] = Acc(0);
        }
        if constexpr (kLdsTotals) {
            dw_lds[(2 * k) * BLOCK + tid] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            dw_lds[(2 * k + 1) * BLOCK + tid] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }

    // One grid-stride step.  MASKED is only needed for the last step of a workgroup, where some of its row
    // groups may have run past the end and mirror the last row: they must add nothing to dW / dB.
    auto step = [&](auto masked_tag) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        const int64_t nrow_raw = row_raw + rows_per_iter;
        const int64_t nrow = nrow_raw < a.M ? nrow_raw : last_row;
        u32x4 nx[K], ng[K];
        slot_load_row<T, K, ALIGNED>(nx, a.x, a.x_stride_bytes, nrow, voff, a.n_cols);
        slot_load_row<T, K, ALIGNED>(ng, a.dy, a.dy_stride_bytes, nrow, voff, a.n_cols);
        const float n_mean = LN ? a.mean[nrow] : 0.0f;
        const float n_rstd = a.rstd[nrow];
        const bool live = !MASKED || row_raw < a.M;

        // u, gf, wdy hold every column of a slot as it is needed for dx (also the columns of an overlapped window that
        // the slot does not own); whatever enters a sum goes through counts().
        float u[K][VEC], gf[K][VEC], wdy[K][VEC];
        float s[NV];
#pragma unroll
        for (int i = 0; i < NV; ++i) s[i] = 0.0f;
        float dlt_fused = 0.0f;
        if constexpr (FUSED && LN) {
            // first round: dlt = sum(u)/N, so that z below is built from the corrected xhat
            float su[1] = {0.0f};
#pragma unroll
            for (int k = 0; k < K; ++k) {
                T::unpack(cx[k], u[k]);
                float sk = 0.0f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float v = (u[k][e] - c_mean) * c_rstd;
                    u[k][e] = v;
                    sk += counts(k, e) ? v : 0.0f;
                }
                su[0] += own[k] ? sk : 0.0f;
            }
            row_allreduce<TPR, G, 1>(su, red, phase, g, t);
            dlt_fused = su[0] * a.inv_n;
        }
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if constexpr (!(FUSED && LN)) T::unpack(cx[k], u[k]);
            T::unpack(cg[k], gf[k]);
            float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if constexpr (FUSED && LN) {
                    u[k][e] -= dlt_fused;                               // the corrected xhat
                } else if constexpr (LN) {
                    u[k][e] = (u[k][e] - c_mean) * c_rstd;
                } else {
                    u[k][e] *= c_rstd;
                }
                if constexpr (FUSED) {
                    const float z = LN ? fmaf(u[k][e], wr[k][e], br[k][e]) : u[k][e] * wr[k][e];
                    gf[k][e] = act_bwd<ACT, float>(z, gf[k][e], 0.0f, 0.0f);       // dy * act'(z)
                }
                wdy[k][e] = wr[k][e] * gf[k][e];
                const bool in = counts(k, e);
                const float wdy_in = in ? wdy[k][e] : 0.0f;
                s0 = fmaf(u[k][e], wdy_in, s0);
                if constexpr (LN) {
                    s1 += wdy_in;
                    if constexpr (!FUSED) s2 += in ? u[k][e] : 0.0f;
                }
            }
            s[0] += own[k] ? s0 : 0.0f;
            if constexpr (LN) {
                s[1] += own[k] ? s1 : 0.0f;
                if constexpr (!FUSED) s[2] += own[k] ? s2 : 0.0f;
            }
        }
        row_allreduce<TPR, G, NV>(s, red, phase, g, t);
        float c1, c2 = 0.0f, dlt = 0.0f;
        if constexpr (LN && FUSED) {
            c2 = s[1] * a.inv_n;                   // u already is the corrected xhat
            c1 = s[0] * a.inv_n;
        } else if constexpr (LN) {
            dlt = s[2] * a.inv_n;
            c2 = s[1] * a.inv_n;
            c1 = fmaf(-dlt, c2, s[0] * a.inv_n);
        } else {
            c1 = s[0] * a.inv_n;
        }

        char* dxrow = a.dx + row * a.dx_stride_bytes;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            float dxf[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float xhat = u[k][e];
                if constexpr (LN) xhat -= dlt;
                // subtract first, scale by rstd last: when dx cancels to (almost) nothing -- rstd is huge for a
                // near-constant row -- the rounding error stays relative to the small difference
                dxf[e] = (wdy[k][e] - fmaf(xhat, c1, c2)) * c_rstd;
                const float gl = ((MASKED && !live) || !counts(k, e)) ? 0.0f : gf[k][e];
                dw[k][e] = fma(static_cast<Acc>(gl), static_cast<Acc>(xhat), dw[k][e]);
                if constexpr (LN) db[k][e] += static_cast<Acc>(gl);
            }
            slot_store<T, ALIGNED>(dxrow, voff[k], a.n_cols, dxf);
        }

#pragma unroll
        for (int k = 0; k < K; ++k) { cx[k] = nx[k]; cg[k] = ng[k]; }
        c_mean = n_mean;
        c_rstd = n_rstd;
        row_raw = nrow_raw;
        row = nrow;
    };

    // The same step in the forms of RowForm::recompute: nothing but the packed vectors of the row lives across
    // the reduction rounds.
    auto lean_step = [&](auto masked_tag) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        // Byte offset of vector slot k.  The instance with 8 vectors per thread has no register to spare (it spilled
        // six): it rebuilds the offsets from the lane's position on every row instead of keeping eight of them
        // (the empty asm keeps the compiler from moving that back out of the row loop).
        auto vo = [&](int k) -> int {
            if constexpr (ALIGNED && (K >= 8 || BLOCK == 1024)) {
                int tt = t;
                asm volatile("" : "+v"(tt));
                const int v = tt + k * TPR - shift;
                return (v < 0 ? 0 : (v < a.n_vecs ? v : a.n_vecs - 1)) * 16;
            } else {
                return voff[k];
            }
        };
        const int64_t nrow_raw = row_raw + rows_per_iter;
        const int64_t nrow = nrow_raw < a.M ? nrow_raw : last_row;
        const bool live = !MASKED || row_raw < a.M;
        const char* nxrow = a.x + nrow * a.x_stride_bytes;
        const char* ngrow = a.dy + nrow * a.dy_stride_bytes;
        u32x4 nx[kForm.ahead ? K : 1], ng[kForm.ahead ? K : 1];
        if constexpr (kForm.ahead) {
#pragma unroll
            for (int k = 0; k < K; ++k) nx[k] = slot_load<T, ALIGNED>(nxrow, vo(k), a.n_cols);
#pragma unroll
            for (int k = 0; k < K; ++k) ng[k] = slot_load<T, ALIGNED>(ngrow, vo(k), a.n_cols);
        }
        const float n_mean = LN ? a.mean[nrow] : 0.0f;
        const float n_rstd = a.rstd[nrow];

        // float32 view of vector slot k: u (LayerNorm: before the dlt correction unless `dlt_f` carries it) and
        // the upstream gradient (times act'(z) with an epilogue); every column of the slot, masked nowhere
        auto expand = [&](int k, float dlt_f, bool corrected, float (&u)[VEC], float (&gf)[VEC]) {
            T::unpack(cx[k], u);
            T::unpack(cg[k], gf);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if constexpr (LN) {
                    float v = (u[e] - c_mean) * c_rstd;
                    if constexpr (FUSED) {
                        if (corrected) v -= dlt_f;
                    }
                    u[e] = v;
                } else {
                    u[e] *= c_rstd;
                }
                if constexpr (FUSED) {
                    if (corrected) {
                        const float z = LN ? fmaf(u[e], wr[k][e], br[k][e]) : u[e] * wr[k][e];
                        gf[e] = act_bwd<ACT, float>(z, gf[e], 0.0f, 0.0f);
                    }
                }
            }
        };

        float s[NV];
#pragma unroll
        for (int i = 0; i < NV; ++i) s[i] = 0.0f;
        float dlt_fused = 0.0f;
        if constexpr (FUSED && LN) {
            float su[1] = {0.0f};
#pragma unroll
            for (int k = 0; k < K; ++k) {
                float u[VEC], gf[VEC];
                expand(k, 0.0f, false, u, gf);
                float sk = 0.0f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) sk += counts(k, e) ? u[e] : 0.0f;
                su[0] += own[k] ? sk : 0.0f;
            }
            row_allreduce<TPR, G, 1>(su, red, phase, g, t);
            forget_derived(cx);
            forget_derived(cg);
            dlt_fused = su[0] * a.inv_n;
        }
#pragma unroll
        for (int k = 0; k < K; ++k) {
            float u[VEC], gf[VEC];
            expand(k, dlt_fused, true, u, gf);
            float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const bool in = counts(k, e);
                const float wdy_in = in ? wr[k][e] * gf[e] : 0.0f;
                s0 = fmaf(u[e], wdy_in, s0);
                if constexpr (LN) {
                    s1 += wdy_in;
                    if constexpr (!FUSED) s2 += in ? u[e] : 0.0f;
                }
            }
            s[0] += own[k] ? s0 : 0.0f;
            if constexpr (LN) {
                s[1] += own[k] ? s1 : 0.0f;
                if constexpr (!FUSED) s[2] += own[k] ? s2 : 0.0f;
            }
        }
        row_allreduce<TPR, G, NV>(s, red, phase, g, t);
        forget_derived(cx);
        forget_derived(cg);
        float c1, c2 = 0.0f, dlt = 0.0f;
        if constexpr (LN && FUSED) {
            c2 = s[1] * a.inv_n;
            c1 = s[0] * a.inv_n;
        } else if constexpr (LN) {
            dlt = s[2] * a.inv_n;
            c2 = s[1] * a.inv_n;
            c1 = fmaf(-dlt, c2, s[0] * a.inv_n);
        } else {
            c1 = s[0] * a.inv_n;
        }

        char* dxrow = a.dx + row * a.dx_stride_bytes;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            float u[VEC], gf[VEC], dxf[VEC];
            expand(k, dlt_fused, true, u, gf);
            float tot[kLdsTotals ? VEC : 1];
            if constexpr (kLdsTotals) {
                const f32x4 lo = dw_lds[(2 * k) * BLOCK + tid], hi = dw_lds[(2 * k + 1) * BLOCK + tid];
#pragma unroll
                for (int e = 0; e < 4; ++e) { tot[e] = lo[e]; tot[4 + e] = hi[e]; }
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float wdy = wr[k][e] * gf[e];
                float xhat = u[e];
                if constexpr (LN) xhat -= dlt;
                dxf[e] = (wdy - fmaf(xhat, c1, c2)) * c_rstd;
                const float gl = ((MASKED && !live) || !counts(k, e)) ? 0.0f : gf[e];
                if constexpr (kLdsTotals) tot[e] = fmaf(gl, xhat, tot[e]);
                else dw[k][e] = fma(static_cast<Acc>(gl), static_cast<Acc>(xhat), dw[k][e]);
                if constexpr (LN) db[k][e] += static_cast<Acc>(gl);
            }
            if constexpr (kLdsTotals) {
                dw_lds[(2 * k) * BLOCK + tid] = f32x4{tot[0], tot[1], tot[2], tot[3]};
                dw_lds[(2 * k + 1) * BLOCK + tid] = f32x4{tot[4], tot[5], tot[6], tot[7]};
            }
            slot_store<T, ALIGNED>(dxrow, vo(k), a.n_cols, dxf);
            if constexpr (kForm.ahead) {
                cx[k] = nx[k];
                cg[k] = ng[k];
            } else {
                cx[k] = slot_load<T, ALIGNED>(nxrow, vo(k), a.n_cols);
                cg[k] = slot_load<T, ALIGNED>(ngrow, vo(k), a.n_cols);
            }
        }
        c_mean = n_mean;
        c_rstd = n_rstd;
        row_raw = nrow_raw;
        row = nrow;
    };

    if constexpr (LN) pin_loaded(c_mean);
    drain_vector_memory(cx, cg, c_rstd);
    int64_t base = static_cast<int64_t>(blockIdx.x) * G;
    if constexpr (kForm.recompute) {
        for (; base + G <= a.M; base += rows_per_iter) lean_step(std::false_type{});
        if (base < a.M) lean_step(std::true_type{});
    } else {
        for (; base + G <= a.M; base += rows_per_iter) step(std::false_type{});
        if (base < a.M) step(std::true_type{});
    }

    // Workgroup partial: tree over the G row groups, then group 0 stores its K vectors of VEC floats.
    // Clamped vector slots hold a copy of their owner's sums and are simply not written.
    const bool want_dw = a.dw_part != nullptr;
    const bool want_db = LN && a.db_part != nullptr;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        float dwk[VEC];
        if constexpr (kLdsTotals) {
            const f32x4 lo = dw_lds[(2 * k) * BLOCK + tid], hi = dw_lds[(2 * k + 1) * BLOCK + tid];
#pragma unroll
            for (int e = 0; e < 4; ++e) { dwk[e] = lo[e]; dwk[4 + e] = hi[e]; }
        }
        if constexpr (G > 1) {
            if (want_dw) combine_groups<BLOCK, TPR, VEC, Acc>(dw[k], comb, g, t);
            if constexpr (LN) {
                if (want_db) combine_groups<BLOCK, TPR, VEC, Acc>(db[k], comb, g, t);
            }
        }
        if (g == 0 && own[k]) {
            // The slot's first column: a multiple of VEC floats into the partial row on the 128-bit path (the pitch is a
            // multiple of 64 floats >= n_vecs*VEC, so whole vectors fit and the 16-byte stores are aligned), any column
            // for the overlapped window of a ragged last slot, whose first `lead` columns belong to the slot before it.
            const int col0 = ALIGNED ? (t + k * TPR - shift) * VEC
                                     : (T::kWindowIo ? voff[k] / T::kBytes : voff[k] * VEC);
            const int64_t off = static_cast<int64_t>(blockIdx.x) * a.part_pitch + col0;
            float pw[VEC], pb[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if constexpr (kLdsTotals) pw[e] = dwk[e];
                else pw[e] = static_cast<float>(dw[k][e]);
                pb[e] = LN ? static_cast<float>(db[LN ? k : 0][e]) : 0.0f;
            }
            if (lead[k] == 0) {
                if (want_dw) store_partial<VEC>(a.dw_part + off, pw);
                if (want_db) store_partial<VEC>(a.db_part + off, pb);
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    if (e >= lead[k]) {
                        if (want_dw) a.dw_part[off + e] = pw[e];
                        if (want_db) a.db_part[off + e] = pb[e];
                    }
                }
            }
        }
    }
}

}  // namespace thn
