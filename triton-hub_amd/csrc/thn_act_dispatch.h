// Run-time (dtype, activation, direction, layout) -> compiled element-wise kernel instance; one translation unit
// per storage type (thn_act_<dtype>.hip).
#pragma once

#include "thn_act.h"
#include "thn_dispatch.h"

namespace thn {

constexpr int kActFwdVecs = 4;   // 16-byte vectors per thread and grid step, forward (one input stream)
// Backward (two input streams): 4 as well, so that a workgroup step covers the same 16 KiB of the tensor in both
// directions -- workgroup w runs on XCD w % 8, and with equal steps (and grids that are multiples of 8) an element is
// differentiated on the XCD that activated it and found in that XCD's L2 (bfloat16 16384 x 4096, forward + backward of
// one batch, 2 -> 4: ReLU 105.3 -> 100.7 us, SiLU 107.3 -> 105.3, float16 Softplus 107.6 -> 104.8, float32 Sigmoid
// 219.8 -> 217.5; ReLU 4096 x 4096 29.9 -> 26.2; the backward by itself gains 1-2 % everywhere).  The three
// activations with the most arithmetic keep 2: their steps lose 1.3-1.7 % with 4 although their backward by itself
// gains as well (GeLU 110.6 -> 112.3 us, tanh GeLU 106.9 -> 108.8, Mish 108.7 -> 110.7; float32 GeLU the same).
constexpr int act_bwd_vecs(int act) { return (act == kGelu || act == kGeluTanh || act == kMish) ? 2 : 4; }
constexpr int kActRowsBwdVecs = 2;   // rows per thread and step of act_rows_kernel's backward (strided or misaligned tensors)

#define THN_ACT_LIST(X)                                                                                  \
    X(kGelu) X(kGeluTanh) X(kSilu) X(kRelu) X(kLeakyRelu) X(kRelu6) X(kSigmoid) X(kTanh) X(kMish)        \
    X(kSoftplus) X(kThreshold)

// Return value: 0 launched, 1 no such activation, <0 HIP error.
#define THN_DECLARE_ACT_LAUNCHER(NAME)                                                                   \
    int launch_act_##NAME(int act, bool bwd, bool flat, const ActArgs& a, dim3 grid, hipStream_t st);

THN_DECLARE_ACT_LAUNCHER(f32)
THN_DECLARE_ACT_LAUNCHER(f16)
THN_DECLARE_ACT_LAUNCHER(bf16)
THN_DECLARE_ACT_LAUNCHER(f64)

inline int run_kernel_grid(void (*kern)(const ActArgs), const ActArgs& a, dim3 grid, hipStream_t st) {
    hipLaunchKernelGGL(kern, grid, dim3(kActBlock), 0, st, a);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

#define THN_ACT_CASE(A)                                                                                  \
    case A:                                                                                              \
        if (flat) {                                                                                      \
            return bwd ? run_kernel_grid(act_flat_kernel<T, A, true, act_bwd_vecs(A)>, a, grid, st)      \
                       : run_kernel_grid(act_flat_kernel<T, A, false, kActFwdVecs>, a, grid, st);        \
        }                                                                                                \
        return bwd ? run_kernel_grid(act_rows_kernel<T, A, true>, a, grid, st)                           \
                   : run_kernel_grid(act_rows_kernel<T, A, false>, a, grid, st);

#define THN_DEFINE_ACT_LAUNCHER(NAME, TYPE)                                                              \
    int launch_act_##NAME(int act, bool bwd, bool flat, const ActArgs& a, dim3 grid, hipStream_t st) {   \
        using T = TYPE;                                                                                  \
        switch (act) {                                                                                   \
            THN_ACT_LIST(THN_ACT_CASE)                                                                   \
            default: return 1;                                                                           \
        }                                                                                                \
    }

}  // namespace thn
