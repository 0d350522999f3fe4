// Run-time (dtype, flavour, shape) -> compiled softmax kernel instance; one translation unit per storage type.
#pragma once

#include "thn_dispatch.h"
#include "thn_softmax.h"

namespace thn {

#define THN_DECLARE_SOFTMAX_LAUNCHERS(NAME)                                                                     \
    int launch_softmax_fwd_##NAME(bool is_log, bool aligned, Shape s, const SoftmaxFwdArgs& a, int grid,        \
                                  hipStream_t st, int* occupancy);                                              \
    int launch_softmax_bwd_##NAME(bool is_log, bool aligned, Shape s, const SoftmaxBwdArgs& a, int grid,        \
                                  hipStream_t st, int* occupancy);                                              \
    int launch_softmax_fwd_loop_##NAME(bool is_log, int block, const SoftmaxFwdArgs& a, int grid, hipStream_t st); \
    int launch_softmax_bwd_loop_##NAME(bool is_log, int block, const SoftmaxBwdArgs& a, int grid, hipStream_t st);

THN_DECLARE_SOFTMAX_LAUNCHERS(f32)
THN_DECLARE_SOFTMAX_LAUNCHERS(f16)
THN_DECLARE_SOFTMAX_LAUNCHERS(bf16)
THN_DECLARE_SOFTMAX_LAUNCHERS(f64)

// Rows of 4 * TPR + 1 to 5 * TPR vectors (a width just above a power of two of vectors, and 5 * 2^k: 1032 ... 1280,
// 2056 ... 2560, 4104 ... 5120, 8200 ... 10240 columns in 16-bit storage): 5 vectors per thread fill 4/5 or more of the
// shape where 3 vectors on twice the threads fill 2/3 to 5/6.
#define THN_SM_SHAPES_FIVE(X) X(5, 32, 256) X(5, 64, 256) X(5, 128, 256) X(5, 256, 256)

#define THN_SM_CASE(KERNEL, ARGS_T, AL, K_, TPR_, BLOCK_)                                                      \
    if (s.k == K_ && s.tpr == TPR_ && s.block == BLOCK_) {                                                     \
        return is_log ? run_kernel<ARGS_T>(KERNEL<T, true, K_, TPR_, BLOCK_, AL>, a, grid, BLOCK_, st, occupancy) \
                      : run_kernel<ARGS_T>(KERNEL<T, false, K_, TPR_, BLOCK_, AL>, a, grid, BLOCK_, st, occupancy); \
    }
#define THN_SMF_AL(K_, TPR_, BLOCK_) THN_SM_CASE(softmax_fwd_kernel, SoftmaxFwdArgs, true, K_, TPR_, BLOCK_)
#define THN_SMF_SC(K_, TPR_, BLOCK_) THN_SM_CASE(softmax_fwd_kernel, SoftmaxFwdArgs, false, K_, TPR_, BLOCK_)
#define THN_SMB_AL(K_, TPR_, BLOCK_) THN_SM_CASE(softmax_bwd_kernel, SoftmaxBwdArgs, true, K_, TPR_, BLOCK_)
#define THN_SMB_SC(K_, TPR_, BLOCK_) THN_SM_CASE(softmax_bwd_kernel, SoftmaxBwdArgs, false, K_, TPR_, BLOCK_)

#define THN_SM_LOOP_CASE(KERNEL, ARGS_T, TYPE, B)                                                               \
    if (block == B) {                                                                                           \
        return is_log ? run_kernel<ARGS_T>(KERNEL<TYPE, true, B>, a, grid, B, st, nullptr)                      \
                      : run_kernel<ARGS_T>(KERNEL<TYPE, false, B>, a, grid, B, st, nullptr);                    \
    }

// Both directions use the forward shape list of the norm kernels (no per-column accumulators to hold), on and off the
// 128-bit path (off it the slots are unaligned 16-byte windows; rows shorter than one vector have one instance).
#define THN_DEFINE_SOFTMAX_LAUNCHERS(NAME, TYPE)                                                                \
    int launch_softmax_fwd_##NAME(bool is_log, bool aligned, Shape s, const SoftmaxFwdArgs& a, int grid,        \
                                  hipStream_t st, int* occupancy) {                                             \
        using T = TYPE;                                                                                         \
        if (aligned) {                                                                                          \
            THN_FWD_SHAPES(THN_SMF_AL)                                                                          \
            THN_FWD_SHAPES_THREE(THN_SMF_AL)                                                                    \
            THN_SM_SHAPES_FIVE(THN_SMF_AL)                                                                      \
        } else if (a.n_cols >= TYPE::VEC) { \
            THN_FWD_SHAPES(THN_SMF_SC) \
            THN_FWD_SHAPES_THREE(THN_SMF_SC) \
            THN_SM_SHAPES_FIVE(THN_SMF_SC) \
        } else { \
            using T = ElemIo<TYPE>; \
            THN_SMF_SC(4, 8, 256) \
        }                                                                                                       \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_softmax_bwd_##NAME(bool is_log, bool aligned, Shape s, const SoftmaxBwdArgs& a, int grid,        \
                                  hipStream_t st, int* occupancy) {                                             \
        using T = TYPE;                                                                                         \
        if (aligned) {                                                                                          \
            THN_FWD_SHAPES(THN_SMB_AL)                                                                          \
            THN_FWD_SHAPES_THREE(THN_SMB_AL)                                                                    \
            THN_SM_SHAPES_FIVE(THN_SMB_AL)                                                                      \
        } else if (a.n_cols >= TYPE::VEC) { \
            THN_FWD_SHAPES(THN_SMB_SC) \
            THN_FWD_SHAPES_THREE(THN_SMB_SC) \
            THN_SM_SHAPES_FIVE(THN_SMB_SC) \
        } else { \
            using T = ElemIo<TYPE>; \
            THN_SMB_SC(4, 8, 256) \
        }                                                                                                       \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_softmax_fwd_loop_##NAME(bool is_log, int block, const SoftmaxFwdArgs& a, int grid, hipStream_t st) { \
        THN_SM_LOOP_CASE(softmax_fwd_loop_kernel, SoftmaxFwdArgs, TYPE, 256)                                    \
        THN_SM_LOOP_CASE(softmax_fwd_loop_kernel, SoftmaxFwdArgs, TYPE, 512)                                    \
        THN_SM_LOOP_CASE(softmax_fwd_loop_kernel, SoftmaxFwdArgs, TYPE, 1024)                                   \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_softmax_bwd_loop_##NAME(bool is_log, int block, const SoftmaxBwdArgs& a, int grid, hipStream_t st) { \
        THN_SM_LOOP_CASE(softmax_bwd_loop_kernel, SoftmaxBwdArgs, TYPE, 256)                                    \
        THN_SM_LOOP_CASE(softmax_bwd_loop_kernel, SoftmaxBwdArgs, TYPE, 512)                                    \
        THN_SM_LOOP_CASE(softmax_bwd_loop_kernel, SoftmaxBwdArgs, TYPE, 1024)                                   \
        return 1;                                                                                               \
    }

}  // namespace thn
