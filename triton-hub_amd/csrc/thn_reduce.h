// Second stage of the dW / dB reduction.  Included by exactly one translation unit (thn_api.hip).
#pragma once

#include "thn_device.h"

namespace thn {

// ---------------------------------------------------------------------------------------------------
// Second stage: out[c] = sum over the P partial rows of part[p][c], added in a fixed order in float64 and
// rounded once to the parameter's storage type.  The stage is pure latency (a few MiB, one dependent launch),
// so it is cut for parallelism: a workgroup owns 16 columns (4 lanes x float4) and has 64 row slices, each
// adding every 64th partial row; the slice sums are then added in slice order through LDS.  N / 16 workgroups:
// every compute unit takes part from N = 4096 on.  From 6144
// columns on the stage moves 6 MiB and more per gradient and wants longer segments of each partial row: 32 columns
// x 32 slices (128-byte segments) up to 32768 columns, 64 columns x 16 slices (256-byte segments) from there on
// (inside a forward + backward step, 32 against 64 columns: fp16 8192 x 6144 89.0 -> 86.6 us, 4096 x 16384
// 113.3 -> 111.8 us, bf16 32768 x 8192 426.6 -> 425.1 us, 4096 x 32768 257.6 -> 258.6 us; against 16 columns the
// longer segments are 2x faster at 16384 columns and more).  With two gradients the stage has twice the workgroups
// and moves twice the bytes: the 32-column form from 4096 columns on (bf16 LayerNorm 16384 x 4096: second stage inside
// the step 4.6 -> 4.2 us; RMSNorm, one gradient, 3.55 -> 4.0 with it and stays at 16 columns).
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

constexpr int kReduceCols = 16;       // columns per workgroup up to kReduceMidFrom columns
constexpr int kReduceColsMid = 32;    // 128-byte segments per partial row, 32 row slices
constexpr int kReduceColsWide = 64;   // 256-byte segments, 16 row slices
constexpr int kReduceMidFrom = 6144;
constexpr int kReduceMidFromBoth = 8192;   // columns of dW and dB together
constexpr int kReduceWideFrom = 32768;
// Partial rows a thread requests before it adds the first.  Only the 32-column form gains from more than one (bf16
// LayerNorm 16384 x 4096: the stage inside a forward + backward step 4.3 -> 3.7 us with 4 or 8; fp16 8192 x 6000
// 5.1 -> 4.2; fp16 RMSNorm 4096 x 16384 4.9 -> 4.5; with 16 it is back at 4.0 / 4.5-5.1 / 5.0); the 16-column form takes
// 3.6 us with 1, 2 or 4 and 3.9 with 8, the 64-column form moves 64 MiB at 6 TB/s and loses 0.4 us to the clamped extras.
constexpr int kReduceAhead = 1, kReduceAheadMid = 4, kReduceAheadWide = 1;

template <int COLS, int AHEAD>
__global__ void __launch_bounds__(256) reduce_partials_kernel(const ReduceArgs a) {
    constexpr int kReduceCols = COLS;
    constexpr int kReduceAheadHere = AHEAD;
    constexpr int kReduceSlices = 1024 / COLS;     // row slices per workgroup (256 threads x float4)
    __shared__ double acc[kReduceSlices][kReduceCols];
    const int which = blockIdx.y;
    const float* part = a.part[which];
    void* out = a.out[which];
    constexpr int kLanes = kReduceCols / 4;
    const int lane = threadIdx.x % kLanes;
    const int slice = threadIdx.x / kLanes;
    const int col = blockIdx.x * kReduceCols + lane * 4;
    double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
    if (col < a.n_cols) {     // the pitch is a multiple of 64 floats: the whole float4 is inside the row
        // AHEAD loads are requested before the first is used (a loop of one load and one add per trip compiles
        // to a full wait per trip: 4-16 round trips to the memory-side cache, one after the other).
        // Partial rows past the end are clamped onto the last one and add zero, so the order of the additions
        // and with it every bit of the result is that of the plain loop.
        const int last = a.n_parts - 1;
        for (int p0 = slice; p0 < a.n_parts; p0 += kReduceAheadHere * kReduceSlices) {
            float4 v[kReduceAheadHere];
#pragma unroll
            for (int u = 0; u < kReduceAheadHere; ++u) {
                const int p = p0 + u * kReduceSlices;
                v[u] = *reinterpret_cast<const float4*>(part + static_cast<int64_t>(p < last ? p : last) * a.pitch + col);
            }
#pragma unroll
            for (int u = 0; u < kReduceAheadHere; ++u) {
                const bool in = p0 + u * kReduceSlices <= last;
                s0 += in ? v[u].x : 0.0f; s1 += in ? v[u].y : 0.0f; s2 += in ? v[u].z : 0.0f; s3 += in ? v[u].w : 0.0f;
            }
        }
    }
    acc[slice][lane * 4 + 0] = s0;
    acc[slice][lane * 4 + 1] = s1;
    acc[slice][lane * 4 + 2] = s2;
    acc[slice][lane * 4 + 3] = s3;
    __syncthreads();
    if (threadIdx.x < kReduceCols) {
        const int c = blockIdx.x * kReduceCols + threadIdx.x;
        if (c < a.n_cols) {
            double s = 0.0;
#pragma unroll
            for (int i = 0; i < kReduceSlices; ++i) s += acc[i][threadIdx.x];
            if (a.w_dtype == kF64) reinterpret_cast<double*>(out)[c] = s;
            else store_param(out, a.w_dtype, c, static_cast<float>(s));
        }
    }
}

}  // namespace thn
