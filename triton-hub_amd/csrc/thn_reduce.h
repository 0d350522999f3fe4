// Second stage of the dW / dB reduction.  Included by exactly one translation unit (thn_api.hip).
#pragma once

#include "thn_device.h"

namespace thn {

// ---------------------------------------------------------------------------------------------------
// Second stage: out[c] = sum over the P partial rows of part[p][c], added in a fixed order in float64 and
// rounded once to the parameter's storage type.  The stage is pure latency (a few MiB, one dependent launch),
// so it is cut for parallelism: a workgroup owns COLS columns (COLS / 4 lanes x float4) and has SLICES row slices,
// slice s adding partial rows s, s + SLICES, ...; the slice sums are then added in slice order through LDS.
// The ORDER of the additions of a column is fixed by SLICES alone, and SLICES is chosen from the column count N
// alone (reduce_slices()): 64 up to 6144 columns, 32 up to 32768, 16 beyond.  So the bits of dW do not depend on
// whether dB is summed in the same launch, nor on the column width of the workgroups, which is chosen for speed:
// 16 columns (every compute unit takes part from N = 4096 on) while the stage moves little; 32 columns (128-byte
// segments of each partial row) from 6144 columns on, and from 4096 on when dW and dB are both summed (twice the
// workgroups and bytes); 64 columns (256-byte segments) from 32768 columns on, where the stage moves 32 MiB and
// more.  Inside a forward + backward step, 32 against 64 columns: fp16 8192 x 6144 89.0 -> 86.6 us, 4096 x 16384
// 113.3 -> 111.8 us, bf16 32768 x 8192 426.6 -> 425.1 us, 4096 x 32768 257.6 -> 258.6 us; against 16 columns the
// longer segments are 2x faster at 16384 columns and more.
// blockIdx.y selects dW (0) or dB (1).
// ---------------------------------------------------------------------------------------------------
struct ReduceArgs {
    const float* part[2];
    void* out[2];
    int64_t pitch;
    int n_cols;
    int n_parts;
    int w_dtype;
};

constexpr int kReduceMidFrom = 6144;
constexpr int kReduceMidFromBoth = 8192;   // columns of dW and dB together
constexpr int kReduceWideFrom = 32768;

// Row slices of the second stage for N columns: fixes the order of the additions, so it depends on N and on nothing else.
inline int reduce_slices(int64_t n_cols) { return n_cols < kReduceMidFrom ? 64 : (n_cols < kReduceWideFrom ? 32 : 16); }

// AHEAD: partial rows a thread requests before it adds the first.  Only the 32-column forms gain from more than one
// (bf16 LayerNorm 16384 x 4096: the stage inside a forward + backward step 4.3 -> 3.7 us with 4 or 8; fp16 8192 x 6000
// 5.1 -> 4.2; fp16 RMSNorm 4096 x 16384 4.9 -> 4.5; with 16 it is back at 4.0 / 4.5-5.1 / 5.0); the 16-column form
// takes 3.6 us with 1, 2 or 4 and 3.9 with 8, the 64-column form moves 64 MiB at 6 TB/s and loses 0.4 us to the
// clamped extras.
template <int COLS, int SLICES, int AHEAD>
__global__ void __launch_bounds__((COLS / 4) * SLICES) reduce_partials_kernel(const ReduceArgs a) {
    __shared__ double acc[SLICES][COLS];
    const int which = blockIdx.y;
    const float* part = a.part[which];
    void* out = a.out[which];
    constexpr int kLanes = COLS / 4;
    const int lane = threadIdx.x % kLanes;
    const int slice = threadIdx.x / kLanes;
    const int col = blockIdx.x * COLS + lane * 4;
    double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
    if (col < a.n_cols) {     // the pitch is a multiple of 64 floats: the whole float4 is inside the row
        // AHEAD loads are requested before the first is used (a loop of one load and one add per trip compiles
        // to a full wait per trip: 4-16 round trips to the memory-side cache, one after the other).
        // Partial rows past the end are clamped onto the last one and add zero, so the order of the additions
        // and with it every bit of the result is that of the plain loop.
        const int last = a.n_parts - 1;
        for (int p0 = slice; p0 < a.n_parts; p0 += AHEAD * SLICES) {
            float4 v[AHEAD];
#pragma unroll
            for (int u = 0; u < AHEAD; ++u) {
                const int p = p0 + u * SLICES;
                v[u] = *reinterpret_cast<const float4*>(part + static_cast<int64_t>(p < last ? p : last) * a.pitch + col);
            }
#pragma unroll
            for (int u = 0; u < AHEAD; ++u) {
                const bool in = p0 + u * SLICES <= last;
                s0 += in ? v[u].x : 0.0f; s1 += in ? v[u].y : 0.0f; s2 += in ? v[u].z : 0.0f; s3 += in ? v[u].w : 0.0f;
            }
        }
    }
    acc[slice][lane * 4 + 0] = s0;
    acc[slice][lane * 4 + 1] = s1;
    acc[slice][lane * 4 + 2] = s2;
    acc[slice][lane * 4 + 3] = s3;
    __syncthreads();
    if (threadIdx.x < COLS) {
        const int c = blockIdx.x * COLS + threadIdx.x;
        if (c < a.n_cols) {
            double s = 0.0;
#pragma unroll
            for (int i = 0; i < SLICES; ++i) s += acc[i][threadIdx.x];
            if (a.w_dtype == kF64) reinterpret_cast<double*>(out)[c] = s;
            else store_param(out, a.w_dtype, c, static_cast<float>(s));
        }
    }
}

}  // namespace thn
