// Second stage of the dW / dB reduction.  Included by exactly one translation unit (thn_api.hip).
#pragma once

#include "thn_device.h"

namespace thn {

// ---------------------------------------------------------------------------------------------------
// Second stage: out[c] = sum over the P partial rows of part[p][c], added in a fixed order in float64 and
// rounded once to the parameter's storage type.  A workgroup owns 64 columns (16 lanes x float4); its 16
// row slices each add every 16th partial row, then slice sums are added in slice order through LDS.
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

__global__ void __launch_bounds__(256) reduce_partials_kernel(const ReduceArgs a) {
    __shared__ double acc[16][64];
    const int which = blockIdx.y;
    const float* part = a.part[which];
    void* out = a.out[which];
    const int lane = threadIdx.x & 15;
    const int slice = threadIdx.x >> 4;
    const int col = blockIdx.x * 64 + lane * 4;
    double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
    if (col < a.n_cols) {     // the pitch is a multiple of 64 floats: the whole float4 is inside the row
        for (int p = slice; p < a.n_parts; p += 16) {
            const float4 v = *reinterpret_cast<const float4*>(part + static_cast<int64_t>(p) * a.pitch + col);
            s0 += v.x; s1 += v.y; s2 += v.z; s3 += v.w;
        }
    }
    acc[slice][lane * 4 + 0] = s0;
    acc[slice][lane * 4 + 1] = s1;
    acc[slice][lane * 4 + 2] = s2;
    acc[slice][lane * 4 + 3] = s3;
    __syncthreads();
    if (threadIdx.x < 64) {
        const int c = blockIdx.x * 64 + threadIdx.x;
        if (c < a.n_cols) {
            double s = 0.0;
#pragma unroll
            for (int i = 0; i < 16; ++i) s += acc[i][threadIdx.x];
            if (a.w_dtype == kF64) reinterpret_cast<double*>(out)[c] = s;
            else store_param(out, a.w_dtype, c, static_cast<float>(s));
        }
    }
}

}  // namespace thn
