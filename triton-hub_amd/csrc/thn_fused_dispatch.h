// Norm kernels with an activation epilogue: run-time (dtype, LayerNorm / RMSNorm, activation, shape) -> compiled
// instance; two translation units per storage type (thn_fused_fwd_<dtype>.hip, thn_fused_bwd_<dtype>.hip).
#pragma once

#include "thn_dispatch.h"

namespace thn {

// Activations that can ride on a norm kernel: parameter free, and their backward needs only the pre-activation.
#define THN_FUSED_ACTS(X) X(kGelu) X(kGeluTanh) X(kSilu) X(kRelu)

// X(K, TPR, BLOCK).  Forward: the fewest threads per row with at most 4 vectors each, as the plain forward.
#define THN_FUSED_FWD_SHAPES(X)                                                      \
    X(1, 8, 256) X(2, 8, 256) X(4, 8, 256) X(4, 16, 256) X(4, 32, 256)               \
    X(3, 64, 256) X(4, 64, 256) X(3, 128, 256) X(4, 128, 256)                        \
    X(3, 256, 256) X(4, 256, 256) X(3, 512, 512) X(4, 512, 512)                      \
    X(3, 1024, 1024) X(4, 1024, 1024)

// Backward: 2 or 3 vectors per thread (the bias and the recomputed pre-activation are live too; the GeLU
// variants are arithmetic-bound, so vector slots without work cost their full share: with 3 as well as 2 a row
// fills at least two thirds of its slots), 512-thread workgroups once a row spans two waves, 4 vectors only
// where 1024 threads cannot cover the row otherwise.
#define THN_FUSED_BWD_SHAPES(X)                                                      \
    X(1, 8, 256) X(2, 8, 256) X(2, 16, 256) X(2, 32, 256) X(2, 64, 256) X(3, 64, 256) \
    X(2, 128, 512) X(3, 128, 512) X(2, 256, 512) X(3, 256, 512) X(2, 512, 512) X(3, 512, 512) \
    X(2, 1024, 1024) X(3, 1024, 1024) X(4, 1024, 1024)

// LayerNorm with an epilogue over 16-bit rows of more than 32 KiB: the 512-thread shapes of the plain LayerNorm
// backward (bias and weight of 40-64 columns in float32 next to the dB sums; 1024 threads spill 48-284 bytes).
#define THN_FUSED_BWD_SHAPES_LN16(X) THN_BWD_SHAPES_LN16(X)

#define THN_DECLARE_FUSED_LAUNCHERS(NAME)                                                                      \
    int launch_fused_fwd_##NAME(bool ln, int act, bool aligned, Shape s, const FwdArgs& a, int grid,           \
                                hipStream_t st, int* occupancy);                                               \
    int launch_fused_bwd_##NAME(bool ln, int act, bool aligned, Shape s, const BwdArgs& a, int grid,           \
                                hipStream_t st, int* occupancy);

THN_DECLARE_FUSED_LAUNCHERS(f32)
THN_DECLARE_FUSED_LAUNCHERS(f16)
THN_DECLARE_FUSED_LAUNCHERS(bf16)
THN_DECLARE_FUSED_LAUNCHERS(f64)

#define THN_FUSED_ACT_CASE(KERNEL, ARGS_T, AL, K_, TPR_, BLOCK_, A)                                           \
    if (act == A) {                                                                                            \
        return ln ? run_kernel<ARGS_T>(KERNEL<T, true, K_, TPR_, BLOCK_, AL, A>, a, grid, BLOCK_, st, occupancy) \
                  : run_kernel<ARGS_T>(KERNEL<T, false, K_, TPR_, BLOCK_, AL, A>, a, grid, BLOCK_, st, occupancy); \
    }
#define THN_FUSED_CASE(KERNEL, ARGS_T, AL, K_, TPR_, BLOCK_)                                                   \
    if (s.k == K_ && s.tpr == TPR_ && s.block == BLOCK_) {                                                     \
        THN_FUSED_ACT_CASE(KERNEL, ARGS_T, AL, K_, TPR_, BLOCK_, kGelu)                                        \
        THN_FUSED_ACT_CASE(KERNEL, ARGS_T, AL, K_, TPR_, BLOCK_, kGeluTanh)                                    \
        THN_FUSED_ACT_CASE(KERNEL, ARGS_T, AL, K_, TPR_, BLOCK_, kSilu)                                        \
        THN_FUSED_ACT_CASE(KERNEL, ARGS_T, AL, K_, TPR_, BLOCK_, kRelu)                                        \
        return 1;                                                                                              \
    }
#define THN_FUSED_ACT_CASE_LN(AL, K_, TPR_, BLOCK_, A)                                                         \
    if (act == A) return run_kernel<BwdArgs>(norm_bwd_kernel<T, true, K_, TPR_, BLOCK_, AL, A>, a, grid, BLOCK_, st, occupancy);
#define THN_FB_AL_LN(K_, TPR_, BLOCK_)                                                                         \
    if (s.k == K_ && s.tpr == TPR_ && s.block == BLOCK_) {                                                     \
        THN_FUSED_ACT_CASE_LN(true, K_, TPR_, BLOCK_, kGelu)                                                   \
        THN_FUSED_ACT_CASE_LN(true, K_, TPR_, BLOCK_, kGeluTanh)                                               \
        THN_FUSED_ACT_CASE_LN(true, K_, TPR_, BLOCK_, kSilu)                                                   \
        THN_FUSED_ACT_CASE_LN(true, K_, TPR_, BLOCK_, kRelu)                                                   \
        return 1;                                                                                              \
    }
// The forward on the 128-bit path has a streaming-x instance next to the one that keeps x for the backward
// (FwdArgs::keep_x); rows off that path always keep x.
#define THN_FUSED_FWD_ACT_CASE(AL, K_, TPR_, BLOCK_, A)                                                        \
    if (act == A) {                                                                                            \
        if (AL && !a.keep_x) {                                                                                 \
            return ln ? run_kernel<FwdArgs>(norm_fwd_kernel<T, true, K_, TPR_, BLOCK_, AL, A, !AL>, a, grid, BLOCK_, st, occupancy) \
                      : run_kernel<FwdArgs>(norm_fwd_kernel<T, false, K_, TPR_, BLOCK_, AL, A, !AL>, a, grid, BLOCK_, st, occupancy); \
        }                                                                                                      \
        return ln ? run_kernel<FwdArgs>(norm_fwd_kernel<T, true, K_, TPR_, BLOCK_, AL, A, true>, a, grid, BLOCK_, st, occupancy) \
                  : run_kernel<FwdArgs>(norm_fwd_kernel<T, false, K_, TPR_, BLOCK_, AL, A, true>, a, grid, BLOCK_, st, occupancy); \
    }
#define THN_FUSED_FWD_CASE(AL, K_, TPR_, BLOCK_)                                                               \
    if (s.k == K_ && s.tpr == TPR_ && s.block == BLOCK_) {                                                     \
        THN_FUSED_FWD_ACT_CASE(AL, K_, TPR_, BLOCK_, kGelu)                                                    \
        THN_FUSED_FWD_ACT_CASE(AL, K_, TPR_, BLOCK_, kGeluTanh)                                                \
        THN_FUSED_FWD_ACT_CASE(AL, K_, TPR_, BLOCK_, kSilu)                                                    \
        THN_FUSED_FWD_ACT_CASE(AL, K_, TPR_, BLOCK_, kRelu)                                                    \
        return 1;                                                                                              \
    }
#define THN_FF_AL(K_, TPR_, BLOCK_) THN_FUSED_FWD_CASE(true, K_, TPR_, BLOCK_)
#define THN_FF_SC(K_, TPR_, BLOCK_) THN_FUSED_FWD_CASE(false, K_, TPR_, BLOCK_)
#define THN_FB_AL(K_, TPR_, BLOCK_) THN_FUSED_CASE(norm_bwd_kernel, BwdArgs, true, K_, TPR_, BLOCK_)
#define THN_FB_SC(K_, TPR_, BLOCK_) THN_FUSED_CASE(norm_bwd_kernel, BwdArgs, false, K_, TPR_, BLOCK_)

#define THN_DEFINE_FUSED_FWD_LAUNCHER(NAME, TYPE)                                                              \
    int launch_fused_fwd_##NAME(bool ln, int act, bool aligned, Shape s, const FwdArgs& a, int grid,           \
                                hipStream_t st, int* occupancy) {                                              \
        using T = TYPE;                                                                                        \
        if (aligned) {                                                                                         \
            THN_FUSED_FWD_SHAPES(THN_FF_AL)                                                                    \
        } else if (a.n_cols >= TYPE::VEC) { \
            THN_SCALAR_SHAPES(THN_FF_SC) \
        } else { \
            using T = ElemIo<TYPE>; \
            THN_FF_SC(4, 8, 256) \
        }                                                                                                      \
        return 1;                                                                                              \
    }

#define THN_DEFINE_FUSED_BWD_LAUNCHER(NAME, TYPE)                                                              \
    int launch_fused_bwd_##NAME(bool ln, int act, bool aligned, Shape s, const BwdArgs& a, int grid,           \
                                hipStream_t st, int* occupancy) {                                              \
        using T = TYPE;                                                                                        \
        if (aligned) {                                                                                         \
            THN_FUSED_BWD_SHAPES(THN_FB_AL)                                                                    \
            if constexpr (TYPE::kBytes == 2) {                                                                 \
                if (ln) {                                                                                      \
                    THN_FUSED_BWD_SHAPES_LN16(THN_FB_AL_LN)                                                    \
                }                                                                                              \
            }                                                                                                  \
        } else if (a.n_cols >= TYPE::VEC) { \
            THN_SCALAR_SHAPES(THN_FB_SC) \
        } else { \
            using T = ElemIo<TYPE>; \
            THN_FB_SC(4, 8, 256) \
        }                                                                                                      \
        return 1;                                                                                              \
    }

}  // namespace thn
