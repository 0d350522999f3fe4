// Run-time (dtype, activation, direction, layout) -> compiled element-wise kernel instance; one translation unit
// per storage type (thn_act_<dtype>.hip).
#pragma once

#include "thn_act.h"
#include "thn_dispatch.h"

namespace thn {

constexpr int kActFwdVecs = 4;   // 16-byte vectors per thread and grid step, forward (one input stream)
constexpr int kActBwdVecs = 2;   // backward (two input streams)

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
            return bwd ? run_kernel_grid(act_flat_kernel<T, A, true, kActBwdVecs>, a, grid, st)          \
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
