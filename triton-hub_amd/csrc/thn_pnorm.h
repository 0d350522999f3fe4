// Row p-norm and p-normalisation over the last dimension of a (B, M, K) tensor, forward and backward: the
// reference's TritonHub/Ops/norm.py and normalize.py.  Rows of at most 64 KiB run on the row engine of the norm
// kernels (see thn_kernels.h: 16-byte vectors, TPR threads per row, next row prefetched, branch-free clamped
// slots).  Everything else -- wider rows, a p that is not an integer -- runs on the looping kernels at the end
// of this file.
//
//   norm forward       (norm.py:24-45):        n = max((sum |x|^p)^(1/p), eps), stored in the storage type
//   normalize forward  (normalize.py:27-33):   y = x / n, with n ALREADY ROUNDED to the storage type (the
//                                              reference reads it back from the tensor the norm kernel wrote);
//                                              here one pass does both: x is read once
//   norm backward      (norm.py:83-102):       p=1: g*sign(x);  p=2: g*x/n;  else g*sign(x)*|x|^(p-1) / n^(p-1)
//   normalize backward (normalize.py:81-117):  proj = sum(y*g)  (p=1: sum(x*g));
//                                              p=1: g/n - sign(x)*(proj/(n*n));  p=2: (g - y*proj)/n;
//                                              else g/n - sign(x)*|x|^(p-1) * (proj/(n^(p-1)*n))
// Arithmetic is float32 whatever the storage type (the reference's `dtype` is float32 for anything that is not
// float16 / bfloat16, norm.py:53).
#pragma once

#include <type_traits>

#include "thn_kernels.h"
#include "thn_walk.h"

namespace thn {

// Addressing of the rows of a (B, M, K) tensor with element-contiguous rows.  Row r is (batch r / rows_per_batch,
// row r % rows_per_batch) and sits at batch*batch_stride + row*row_stride.  When every operand of a launch has
// batch_stride == M*row_stride the host folds the batches away (rows_per_batch = B*M, one "batch").
// The row kernels never divide inside their loop: each row group keeps a (batch, row) cursor and advances it by
// the launch-uniform grid stride, split by the host into (step_batch, step_row) -- a division, or a branch
// around one, inside the loop would cost the loop its precise memory waits (see thn_kernels.h).
struct RowMap {
    int64_t batch_stride_bytes;
    int64_t row_stride_bytes;
};

struct RowWalk {
    int64_t rows_per_batch;
    int64_t step_batch;     // (gridDim.x * G) / rows_per_batch
    int64_t step_row;       // (gridDim.x * G) % rows_per_batch
};

struct RowCursor {
    int64_t b, m;
    __device__ __forceinline__ void init(const RowWalk& w, int64_t row) {
        b = row / w.rows_per_batch;
        m = row - b * w.rows_per_batch;
    }
    __device__ __forceinline__ void advance(const RowWalk& w) {
        m += w.step_row;
        b += w.step_batch;
        const bool carry = m >= w.rows_per_batch;
        m -= carry ? w.rows_per_batch : 0;
        b += carry ? 1 : 0;
    }
};

__device__ __forceinline__ int64_t row_offset(const RowMap& map, const RowCursor& c) {
    return c.b * map.batch_stride_bytes + c.m * map.row_stride_bytes;
}

// The cursor of the next row, or of the tensor's last row when the row group has run past the end (slots without
// work mirror the last row).  A select on the two small integers, not on the offsets: selecting between a computed
// offset and a constant makes the compiler branch around the multiplications.
__device__ __forceinline__ RowCursor clamp_cursor(const RowCursor& c, const RowCursor& last, bool in_range) {
    RowCursor r;
    r.b = in_range ? c.b : last.b;
    r.m = in_range ? c.m : last.m;
    return r;
}

// For the looping kernels, which may divide.
__device__ __forceinline__ int64_t row_offset(const RowMap& map, const RowWalk& w, int64_t r) {
    RowCursor c;
    c.init(w, r);
    return row_offset(map, c);
}

enum : int { kP1 = 1, kP2 = 2, kPInt = 3 };   // MODE of the row-engine kernels; kPInt: p in {3, 4, 5, 6}

struct PnormFwdArgs {
    const char* x;
    char* y;            // normalize only
    void* norms;        // (rows,) storage type
    RowMap xmap, ymap;
    RowWalk walk;
    int64_t rows;
    int64_t n_cols64;   // looping kernels
    int n_cols;
    int n_vecs;
    int p_int;          // p when it is an integer in [1, 6], else 0
    float p;
    float eps;
    int line_shift;     // 1: the row kernels may move their vector slots onto 128-byte lines (row_line_shift(), thn_kernels.h)
};

struct PnormBwdArgs {
    const char* x;
    const void* norms;  // (rows,) storage type: the saved output of the forward
    const void* g;      // (rows,) storage type: upstream gradient of the norms
    char* dx;
    RowMap xmap, dxmap;
    RowWalk walk;
    int64_t rows;
    int64_t n_cols64;
    int n_cols;
    int n_vecs;
    int p_int;
    float p;
    int line_shift;     // as in PnormFwdArgs
};

struct NormalizeBwdArgs {
    const char* x;      // read unless p == 2
    const char* y;      // the saved normalised output; read unless p == 1
    const void* norms;
    const char* g;      // upstream gradient of y, (B, M, K)
    char* dx;
    RowMap xmap, ymap, gmap, dxmap;
    RowWalk walk;
    int64_t rows;
    int64_t n_cols64;
    int n_cols;
    int n_vecs;
    int p_int;
    float p;
    int line_shift;     // as in PnormFwdArgs
};

// a^e for a >= 0 and a launch-uniform integer e in [2, 6], without a branch.
__device__ __forceinline__ float pow_small(float a, int e) {
    const float a2 = a * a, a3 = a2 * a, a4 = a2 * a2;
    float r = a2;
    r = e == 3 ? a3 : r;
    r = e == 4 ? a4 : r;
    r = e == 5 ? a4 * a : r;
    r = e == 6 ? a3 * a3 : r;
    return r;
}

__device__ __forceinline__ float sign_of(float x) { return x > 0.0f ? 1.0f : (x < 0.0f ? -1.0f : 0.0f); }

// num / den with the row's correctly rounded reciprocal `rden` = 1/den: one multiplication and one residual
// correction (q + (num - q*den)*rden), which is the correctly rounded quotient except for isolated
// significand patterns, at 3 instructions per element instead of the ~10 of a full division.  |num/den| must
// be representable (true here: every quotient is bounded by the row's norm) and den must not be subnormal
// (then rden is infinite and the quotient is infinite or NaN where exact division would give a huge finite
// number; the norms are clamped from below by eps, so this needs eps = 0 and a row of subnormals).
__device__ __forceinline__ float div_by_row(float num, float den, float rden) {
    const float q = num * rden;
    return __builtin_fmaf(__builtin_fmaf(-q, den, num), rden, q);
}
// The `den` to pass to div_by_row: an infinite divisor (a row whose power sum overflowed) becomes 0, so that the
// residual is num - q*0 instead of the NaN of 0 * inf, and the quotient 0 (NaN for an infinite numerator), as
// the division gives it.
__device__ __forceinline__ float residual_divisor(float den) { return den < __builtin_inff() ? den : 0.0f; }

// x rounded to storage type T and widened again.
template <typename T>
__device__ __forceinline__ float round_to_storage(float f) {
    if constexpr (T::kBytes >= 4) {
        return f;
    } else {
        float tmp[T::VEC];
#pragma unroll
        for (int e = 0; e < T::VEC; ++e) tmp[e] = f;
        const u32x4 v = T::pack(tmp);
        T::unpack(v, tmp);
        return tmp[0];
    }
}

template <int MODE>
__device__ __forceinline__ float norm_term(float x, int p_int) {
    if constexpr (MODE == kP1) return __builtin_fabsf(x);
    else if constexpr (MODE == kP2) return x * x;
    else return pow_small(__builtin_fabsf(x), p_int);
}

// acc^(1/p) for integer p in [3, 6]: the hardware log2 / exp2 give the root to a few float32 ulp, one Newton step
// on r^p = acc (r^p by multiplication) brings it to about 1 ulp, at a tenth of the instructions of powf -- every
// thread of a row evaluates this once per row.
__device__ __forceinline__ float root_small(float acc, int p_int, float p) {
    const float r = __builtin_amdgcn_exp2f(__builtin_amdgcn_logf(acc) / p);
    const float rp1 = pow_small(r, p_int - 1);                     // r^(p-1)
    const float better = r - (rp1 * r - acc) / (p * rp1);
    return acc > 0.0f && acc < 3.0e38f && rp1 > 0.0f ? better : (acc > 0.0f ? powf(acc, 1.0f / p) : 0.0f);
}

template <int MODE>
__device__ __forceinline__ float norm_root(float acc, int p_int, float p) {
    if constexpr (MODE == kP1) return acc;
    else if constexpr (MODE == kP2) return sqrtf(acc);
    else return root_small(acc, p_int, p);
}

// ---------------------------------------------------------------------------------------------------
// Forward on the row engine.  NORMALIZE = false: norms only (x read once: K*s bytes per row).
// NORMALIZE = true: norms and y = x / norms from the registers (x read once, y written once: 2*K*s bytes).
// ---------------------------------------------------------------------------------------------------
template <typename T, int MODE, bool NORMALIZE, int K, int TPR, int BLOCK, bool ALIGNED>
__global__ void __launch_bounds__(BLOCK) pnorm_fwd_kernel(const PnormFwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int G = BLOCK / TPR;
    // What the backward reads again stays in the caches (ld128_keep): the norm's backward and the normalize backward
    // for p = 1 read x, the normalize backward for p = 2 reads y; for the other p it reads both, and x is kept.
    constexpr bool kKeepY = NORMALIZE && MODE == kP2;
    constexpr bool kKeepX = !kKeepY;
    static_assert(BLOCK % TPR == 0 && G >= 1, "a workgroup holds whole rows");
    __shared__ float red[RedSmem<TPR, G, 1>::kFloats];

    const int tid = threadIdx.x;
    const int g = tid / TPR;
    const int t = tid % TPR;
    int phase = 0;

    // the host sets line_shift only when the rows are one folded batch (row r at r * row stride), every row this
    // workgroup visits and every stream start in the same phase of a 128-byte line, and the slots have room
    const int shift = (ALIGNED && G == 1) ? row_line_shift(a.line_shift, a.x, a.xmap.row_stride_bytes, blockIdx.x) : 0;
    // Rows off the 128-bit path: unaligned 16-byte windows, the ragged last one overlapping its neighbour (slot_place()).
    int voff[K], lead[K];
    bool own[K];
#pragma unroll
    for (int k = 0; k < K; ++k) slot_place<T, ALIGNED>(t + k * TPR - shift, a.n_vecs, a.n_cols, voff[k], lead[k], own[k]);
    // element e of slot k counts in the row sum (always true on the 128-bit path)
    auto counts = [&](int k, int e) -> bool { return slot_counts<T, ALIGNED>(voff[k], lead[k], e, a.n_cols); };

    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * G;
    const int64_t last_row = a.rows - 1;
    int64_t row_raw = static_cast<int64_t>(blockIdx.x) * G + g;
    int64_t row = row_raw < a.rows ? row_raw : last_row;
    RowCursor cursor;
    cursor.init(a.walk, row);
    RowCursor last;
    last.init(a.walk, last_row);
    int64_t y_off = NORMALIZE ? row_offset(a.ymap, cursor) : 0;
    u32x4 cur[K];
    slot_load_row<T, K, ALIGNED, kKeepX>(cur, a.x + row_offset(a.xmap, cursor), 0, 0, voff, a.n_cols);

    drain_vector_memory(cur);
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * G; base < a.rows; base += rows_per_iter) {
        const int64_t nrow_raw = row_raw + rows_per_iter;
        const bool more = nrow_raw < a.rows;
        const int64_t nrow = more ? nrow_raw : last_row;
        cursor.advance(a.walk);
        const RowCursor ncur = clamp_cursor(cursor, last, more);
        u32x4 nxt[K];
        slot_load_row<T, K, ALIGNED, kKeepX>(nxt, a.x + row_offset(a.xmap, ncur), 0, 0, voff, a.n_cols);

        float xf[K][VEC];
        float s[1] = {0.0f};
#pragma unroll
        for (int k = 0; k < K; ++k) {
            T::unpack(cur[k], xf[k]);
            float sk = 0.0f;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {          // rows shorter than a vector: absent columns load as 0
                const float term = norm_term<MODE>(xf[k][e], a.p_int);
                sk += counts(k, e) ? term : 0.0f;
            }
            s[0] += own[k] ? sk : 0.0f;
        }
        row_allreduce<TPR, G, 1>(s, red, phase, g, t);
        const float n = fmaxf(norm_root<MODE>(s[0], a.p_int, a.p), a.eps);
        // Every thread of the row stores the same value to the same address (one request per wave).
        T::store1(a.norms, row, n);

        if constexpr (NORMALIZE) {
            const float nr = round_to_storage<T>(n);
            const float rn = 1.0f / nr;
            const float nd = residual_divisor(nr);
            char* yrow = a.y + y_off;
#pragma unroll
            for (int k = 0; k < K; ++k) {
                float yf[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) yf[e] = div_by_row(xf[k][e], nd, rn);
                slot_store<T, ALIGNED, kKeepY>(yrow, voff[k], a.n_cols, yf);
            }
            y_off = row_offset(a.ymap, ncur);
        }

#pragma unroll
        for (int k = 0; k < K; ++k) cur[k] = nxt[k];
        row_raw = nrow_raw;
        row = nrow;
    }
}

// ---------------------------------------------------------------------------------------------------
// Norm backward: element-wise with two per-row scalars; x read once, dx written once (2*K*s bytes per row).
// ---------------------------------------------------------------------------------------------------
template <typename T, int MODE, int K, int TPR, int BLOCK, bool ALIGNED>
__global__ void __launch_bounds__(BLOCK) pnorm_bwd_kernel(const PnormBwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int G = BLOCK / TPR;
    static_assert(BLOCK % TPR == 0 && G >= 1, "a workgroup holds whole rows");

    const int tid = threadIdx.x;
    const int g = tid / TPR;
    const int t = tid % TPR;

    const int shift = (ALIGNED && G == 1) ? row_line_shift(a.line_shift, a.x, a.xmap.row_stride_bytes, blockIdx.x) : 0;
    int voff[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {      // slots off either end repeat their neighbour's vector (same bits)
        int lead;
        bool own;
        slot_place<T, ALIGNED>(t + k * TPR - shift, a.n_vecs, a.n_cols, voff[k], lead, own);
    }

    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * G;
    const int64_t last_row = a.rows - 1;
    int64_t row_raw = static_cast<int64_t>(blockIdx.x) * G + g;
    int64_t row = row_raw < a.rows ? row_raw : last_row;
    RowCursor cursor;
    cursor.init(a.walk, row);
    RowCursor last;
    last.init(a.walk, last_row);
    int64_t dx_off = row_offset(a.dxmap, cursor);
    u32x4 cur[K];
    slot_load_row<T, K, ALIGNED>(cur, a.x + row_offset(a.xmap, cursor), 0, 0, voff, a.n_cols);
    float c_n = MODE == kP1 ? 1.0f : T::load1(a.norms, row);
    float c_g = T::load1(a.g, row);

    if constexpr (MODE != kP1) pin_loaded(c_n);
    drain_vector_memory(cur, c_g);
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * G; base < a.rows; base += rows_per_iter) {
        const int64_t nrow_raw = row_raw + rows_per_iter;
        const bool more = nrow_raw < a.rows;
        const int64_t nrow = more ? nrow_raw : last_row;
        cursor.advance(a.walk);
        const RowCursor ncur = clamp_cursor(cursor, last, more);
        u32x4 nxt[K];
        slot_load_row<T, K, ALIGNED>(nxt, a.x + row_offset(a.xmap, ncur), 0, 0, voff, a.n_cols);
        // The next row's two scalars are requested here as raw bits and widened at the end of the step (hold_loaded_here
        // there keeps the compiler from widening them earlier): loads return in issue order, so an earlier use would
        // wait for the row's vectors in the middle of the step -- or, requested before them, for the previous row's
        // stores before the vectors are even requested.
        typename RowScalar<T>::bits_t raw_n = MODE == kP1 ? 0 : RowScalar<T>::load(a.norms, nrow);
        typename RowScalar<T>::bits_t raw_g = RowScalar<T>::load(a.g, nrow);

        float den = c_n;
        if constexpr (MODE == kPInt) den = pow_small(c_n, a.p_int - 1);     // norms^(p-1), norm.py:86-87
        const float rden = 1.0f / den;
        den = residual_divisor(den);
        char* dxrow = a.dx + dx_off;
        dx_off = row_offset(a.dxmap, ncur);
#pragma unroll
        for (int k = 0; k < K; ++k) {
            float xf[VEC], df[VEC];
            T::unpack(cur[k], xf);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float x = xf[e];
                if constexpr (MODE == kP1) df[e] = c_g * sign_of(x);
                else if constexpr (MODE == kP2) df[e] = div_by_row(c_g * x, den, rden);
                else df[e] = div_by_row(c_g * sign_of(x) * pow_small(__builtin_fabsf(x), a.p_int - 1), den, rden);
            }
            slot_store<T, ALIGNED>(dxrow, voff[k], a.n_cols, df);
        }

#pragma unroll
        for (int k = 0; k < K; ++k) cur[k] = nxt[k];
        if constexpr (MODE != kP1) {
            hold_loaded_here(raw_n);
            c_n = RowScalar<T>::value(raw_n);
        }
        hold_loaded_here(raw_g);
        c_g = RowScalar<T>::value(raw_g);
        row_raw = nrow_raw;
        row = nrow;
    }
}

// ---------------------------------------------------------------------------------------------------
// Normalize backward.  p = 2 reads y and g (3*K*s bytes per row with the dx store), p = 1 reads x and g
// (3*K*s), other p read x, y and g (4*K*s).  One reduction round per row.
// ---------------------------------------------------------------------------------------------------
template <typename T, int MODE, int K, int TPR, int BLOCK, bool ALIGNED>
__global__ void __launch_bounds__(BLOCK) normalize_bwd_kernel(const NormalizeBwdArgs a) {
    constexpr int VEC = T::VEC;
    constexpr int G = BLOCK / TPR;
    constexpr bool NEED_X = MODE != kP2;
    constexpr bool NEED_Y = MODE != kP1;
    static_assert(BLOCK % TPR == 0 && G >= 1, "a workgroup holds whole rows");
    __shared__ float red[RedSmem<TPR, G, 1>::kFloats];

    const int tid = threadIdx.x;
    const int g = tid / TPR;
    const int t = tid % TPR;
    int phase = 0;

    // the host sets line_shift only when the rows are one folded batch (row r at r * row stride), every row this
    // workgroup visits and every stream start in the same phase of a 128-byte line, and the slots have room
    const int shift = (ALIGNED && G == 1) ? row_line_shift(a.line_shift, a.g, a.gmap.row_stride_bytes, blockIdx.x) : 0;
    // Rows off the 128-bit path: unaligned 16-byte windows, the ragged last one overlapping its neighbour (slot_place()).
    int voff[K], lead[K];
    bool own[K];
#pragma unroll
    for (int k = 0; k < K; ++k) slot_place<T, ALIGNED>(t + k * TPR - shift, a.n_vecs, a.n_cols, voff[k], lead[k], own[k]);
    // element e of slot k counts in the row sum (always true on the 128-bit path)
    auto counts = [&](int k, int e) -> bool { return slot_counts<T, ALIGNED>(voff[k], lead[k], e, a.n_cols); };

    const int64_t rows_per_iter = static_cast<int64_t>(gridDim.x) * G;
    const int64_t last_row = a.rows - 1;
    int64_t row_raw = static_cast<int64_t>(blockIdx.x) * G + g;
    int64_t row = row_raw < a.rows ? row_raw : last_row;
    RowCursor cursor;
    cursor.init(a.walk, row);
    RowCursor last;
    last.init(a.walk, last_row);
    int64_t dx_off = row_offset(a.dxmap, cursor);
    u32x4 cx[NEED_X ? K : 1], cy[NEED_Y ? K : 1], cg[K];
    if constexpr (NEED_X) slot_load_row<T, K, ALIGNED>(cx, a.x + row_offset(a.xmap, cursor), 0, 0, voff, a.n_cols);
    if constexpr (NEED_Y) slot_load_row<T, K, ALIGNED>(cy, a.y + row_offset(a.ymap, cursor), 0, 0, voff, a.n_cols);
    slot_load_row<T, K, ALIGNED>(cg, a.g + row_offset(a.gmap, cursor), 0, 0, voff, a.n_cols);
    float c_n = T::load1(a.norms, row);

    if constexpr (NEED_X) pin_loaded(cx);
    if constexpr (NEED_Y) pin_loaded(cy);
    drain_vector_memory(cg, c_n);
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * G; base < a.rows; base += rows_per_iter) {
        const int64_t nrow_raw = row_raw + rows_per_iter;
        const bool more = nrow_raw < a.rows;
        const int64_t nrow = more ? nrow_raw : last_row;
        cursor.advance(a.walk);
        const RowCursor ncur = clamp_cursor(cursor, last, more);
        u32x4 nx[NEED_X ? K : 1], ny[NEED_Y ? K : 1], ng[K];
        if constexpr (NEED_X) slot_load_row<T, K, ALIGNED>(nx, a.x + row_offset(a.xmap, ncur), 0, 0, voff, a.n_cols);
        if constexpr (NEED_Y) slot_load_row<T, K, ALIGNED>(ny, a.y + row_offset(a.ymap, ncur), 0, 0, voff, a.n_cols);
        slot_load_row<T, K, ALIGNED>(ng, a.g + row_offset(a.gmap, ncur), 0, 0, voff, a.n_cols);
        typename RowScalar<T>::bits_t raw_n = RowScalar<T>::load(a.norms, nrow);      // widened at the end of the step, as in pnorm_bwd_kernel

        float xf[NEED_X ? K : 1][VEC], yf[NEED_Y ? K : 1][VEC], gf[K][VEC];
        float s[1] = {0.0f};
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if constexpr (NEED_X) T::unpack(cx[k], xf[k]);
            if constexpr (NEED_Y) T::unpack(cy[k], yf[k]);
            T::unpack(cg[k], gf[k]);
            float sk = 0.0f;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float ge = counts(k, e) ? gf[k][e] : 0.0f;
                if constexpr (MODE == kP1) sk = __builtin_fmaf(xf[k][e], ge, sk);             // normalize.py:92
                else sk = __builtin_fmaf(yf[k][e], ge, sk);                                   // normalize.py:96
            }
            s[0] += own[k] ? sk : 0.0f;
        }
        row_allreduce<TPR, G, 1>(s, red, phase, g, t);
        const float proj = s[0];
        const float n = c_n;
        const float rn = 1.0f / n;
        const float nd = residual_divisor(n);
        float coef = 0.0f;                                                                    // per-row factor of sign(x)*...
        if constexpr (MODE == kP1) coef = proj / (n * n);                                     // normalize.py:106
        if constexpr (MODE == kPInt) coef = proj / (pow_small(n, a.p_int - 1) * n);           // normalize.py:115

        char* dxrow = a.dx + dx_off;
        dx_off = row_offset(a.dxmap, ncur);
#pragma unroll
        for (int k = 0; k < K; ++k) {
            float df[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float gg = gf[k][e];
                if constexpr (MODE == kP2) {
                    df[e] = div_by_row(gg - yf[k][e] * proj, nd, rn);                          // normalize.py:110
                } else if constexpr (MODE == kP1) {
                    df[e] = div_by_row(gg, nd, rn) - sign_of(xf[k][e]) * coef;
                } else {
                    const float x = xf[k][e];
                    df[e] = div_by_row(gg, nd, rn) - sign_of(x) * pow_small(__builtin_fabsf(x), a.p_int - 1) * coef;
                }
            }
            slot_store<T, ALIGNED>(dxrow, voff[k], a.n_cols, df);
        }

#pragma unroll
        for (int k = 0; k < K; ++k) {
            if constexpr (NEED_X) cx[k] = nx[k];
            if constexpr (NEED_Y) cy[k] = ny[k];
            cg[k] = ng[k];
        }
        hold_loaded_here(raw_n);
        c_n = RowScalar<T>::value(raw_n);
        row_raw = nrow_raw;
        row = nrow;
    }
}

// ---------------------------------------------------------------------------------------------------
// Looping kernels: one 256-thread workgroup per row (grid-stride over rows), the row walked as often as the
// formula needs it (the second walk of a row comes from the L2 or the Infinity Cache).  Any row width, any real
// p in [1, 6] (powf or, for 16-bit storage, the hardware log2 / exp2), any alignment.  This is the path of
// rows wider than 64 KiB and of non-integer p.
// The walks are walk_row of thn_walk.h.
// ---------------------------------------------------------------------------------------------------
constexpr int kLoopBlock = 256;

// ax^e for ax >= 0; e_int is e when e is an integer in [0, 6], else -1.  FAST (16-bit storage): a real exponent
// goes through the hardware log2 / exp2, whose relative error of about e * |log2(ax)| * 2^-24 (3e-6 at the ends
// of the float32 range) disappears in the rounding to a 16-bit result; float32 / float64 storage keeps the accurate powf (an
// exponent-splitting exp2(e*log2) on the hardware functions reached 2-4 ulp, too close to the 4 ulp the results
// are held to).
template <bool FAST>
__device__ __forceinline__ float pow_abs_any(float ax, float e, int e_int) {
    if (e_int == 0) return 1.0f;
    if (e_int == 1) return ax;
    if (e_int >= 2 && e_int <= 6) return pow_small(ax, e_int);
    if constexpr (FAST) return __builtin_amdgcn_exp2f(e * __builtin_amdgcn_logf(ax));
    else return powf(ax, e);
}

template <typename T, bool NORMALIZE>
__global__ void __launch_bounds__(kLoopBlock) pnorm_fwd_loop_kernel(const PnormFwdArgs a) {
    __shared__ float red[RedSmem<kLoopBlock, 1, 1>::kFloats];
    int phase = 0;
    const int t = threadIdx.x;
    const int p_int = a.p_int;
    const float p = a.p;
    for (int64_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
        const char* xrow = a.x + row_offset(a.xmap, a.walk, row);
        float s[1] = {0.0f};
        float acc = 0.0f;
        if (p_int == 2) {
            walk_row<T, float, kLoopBlock, 1, false, NORMALIZE>(xrow, nullptr, nullptr, nullptr, a.n_cols64, t, [&](float x, float, float) {
                acc = __builtin_fmaf(x, x, acc);
                return 0.0f;
            });
        } else {
            walk_row<T, float, kLoopBlock, 1, false, NORMALIZE>(xrow, nullptr, nullptr, nullptr, a.n_cols64, t, [&](float x, float, float) {
                acc += pow_abs_any<T::kBytes == 2>(__builtin_fabsf(x), p, p_int > 0 ? p_int : -1);
                return 0.0f;
            });
        }
        s[0] = acc;
        row_allreduce<kLoopBlock, 1, 1>(s, red, phase, 0, t);
        float n = s[0];
        if (p_int == 2) n = sqrtf(n);
        else if (p_int != 1) {
            // 1/p is rounded to float32, and that rounding is multiplied by ln(n) in the power (8 ulp at n = 2e10):
            // one Newton step on r^p = n brings the root back to about an ulp (once per row)
            const float r = powf(n, 1.0f / p);
            const float rp1 = powf(r, p - 1.0f);
            const float better = r - (rp1 * r - n) / (p * rp1);
            n = (r > 0.0f && r < 3.0e38f && rp1 > 0.0f && rp1 < 3.0e38f) ? better : r;
        }
        n = fmaxf(n, a.eps);
        if (t == 0) T::store1(a.norms, row, n);
        if constexpr (NORMALIZE) {
            const float nr = round_to_storage<T>(n);
            char* yrow = a.y + row_offset(a.ymap, a.walk, row);
            walk_row<T, float, kLoopBlock, 1, true>(xrow, nullptr, nullptr, yrow, a.n_cols64, t, [&](float x, float, float) { return x / nr; });
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(kLoopBlock) pnorm_bwd_loop_kernel(const PnormBwdArgs a) {
    const int t = threadIdx.x;
    const int p_int = a.p_int;
    const float pm1 = a.p - 1.0f;
    const int e_int = p_int > 0 ? p_int - 1 : -1;
    for (int64_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
        const char* xrow = a.x + row_offset(a.xmap, a.walk, row);
        char* dxrow = a.dx + row_offset(a.dxmap, a.walk, row);
        const float g = T::load1(a.g, row);
        float den = 1.0f;
        if (p_int != 1) {
            const float n = T::load1(a.norms, row);
            den = p_int == 2 ? n : pow_abs_any<false>(n, pm1, e_int);
        }
        if (p_int == 1) {
            walk_row<T, float, kLoopBlock, 1, true>(xrow, nullptr, nullptr, dxrow, a.n_cols64, t, [&](float x, float, float) { return g * sign_of(x); });
        } else if (p_int == 2) {
            walk_row<T, float, kLoopBlock, 1, true>(xrow, nullptr, nullptr, dxrow, a.n_cols64, t, [&](float x, float, float) { return (g * x) / den; });
        } else {
            walk_row<T, float, kLoopBlock, 1, true>(xrow, nullptr, nullptr, dxrow, a.n_cols64, t, [&](float x, float, float) {
                return (g * sign_of(x) * pow_abs_any<T::kBytes == 2>(__builtin_fabsf(x), pm1, e_int)) / den;
            });
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(kLoopBlock) normalize_bwd_loop_kernel(const NormalizeBwdArgs a) {
    __shared__ float red[RedSmem<kLoopBlock, 1, 1>::kFloats];
    int phase = 0;
    const int t = threadIdx.x;
    const int p_int = a.p_int;
    const float pm1 = a.p - 1.0f;
    const int e_int = p_int > 0 ? p_int - 1 : -1;
    for (int64_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
        const char* xrow = a.x + row_offset(a.xmap, a.walk, row);
        const char* yrow = a.y + row_offset(a.ymap, a.walk, row);
        const char* grow = a.g + row_offset(a.gmap, a.walk, row);
        char* dxrow = a.dx + row_offset(a.dxmap, a.walk, row);
        const float n = T::load1(a.norms, row);
        float s[1] = {0.0f};
        float acc = 0.0f;
        walk_row<T, float, kLoopBlock, 2, false, true>(p_int == 1 ? xrow : yrow, grow, nullptr, nullptr, a.n_cols64, t, [&](float other, float gg, float) {
            acc = __builtin_fmaf(other, gg, acc);
            return 0.0f;
        });
        s[0] = acc;
        row_allreduce<kLoopBlock, 1, 1>(s, red, phase, 0, t);
        const float proj = s[0];
        if (p_int == 2) {
            walk_row<T, float, kLoopBlock, 2, true>(grow, yrow, nullptr, dxrow, a.n_cols64, t, [&](float gg, float y, float) { return (gg - y * proj) / n; });
        } else {
            const float coef = p_int == 1 ? proj / (n * n) : proj / (pow_abs_any<false>(n, pm1, e_int) * n);
            walk_row<T, float, kLoopBlock, 2, true>(grow, xrow, nullptr, dxrow, a.n_cols64, t, [&](float gg, float x, float) {
                return gg / n - sign_of(x) * pow_abs_any<T::kBytes == 2>(__builtin_fabsf(x), pm1, e_int) * coef;
            });
        }
    }
}

}  // namespace thn
