// Run-time (dtype, p mode, shape) -> compiled p-norm / normalize kernel instance; two translation units per
// storage type (thn_pnorm_fwd_<dtype>.hip, thn_pnorm_bwd_<dtype>.hip).
#pragma once

#include "thn_dispatch.h"
#include "thn_pnorm.h"

namespace thn {

// X(K, TPR, BLOCK): the shapes the launch heuristic can reach (fewest threads per row with at most 4, or at
// most 2, vectors each; 3 x 16 and 3 x 32 for rows of 33 to 48 and 65 to 96 vectors, as in the norm and softmax
// families).
#define THN_ROW_SHAPES(X)                                                            \
    X(1, 8, 256) X(2, 8, 256) X(4, 8, 256)                                           \
    X(2, 16, 256) X(3, 16, 256) X(4, 16, 256) X(2, 32, 256) X(3, 32, 256) X(4, 32, 256) \
    X(2, 64, 256) X(3, 64, 256) X(4, 64, 256)                                        \
    X(2, 128, 256) X(3, 128, 256) X(4, 128, 256)                                     \
    X(2, 256, 256) X(3, 256, 256) X(4, 256, 256)                                     \
    X(2, 512, 512) X(3, 512, 512) X(4, 512, 512)                                     \
    X(2, 1024, 1024) X(3, 1024, 1024) X(4, 1024, 1024)

// Forward and normalize backward only: 5 vectors per thread for rows of 4 * TPR + 1 to 5 * TPR vectors, as in the
// softmax family (THN_SM_SHAPES_FIVE).
#define THN_PN_SHAPES_FIVE(X) X(5, 32, 256) X(5, 64, 256) X(5, 128, 256) X(5, 256, 256)

// mode: kP1 / kP2 / kPInt.  task of the looping kernels: 0 norm forward, 1 normalize forward.
#define THN_DECLARE_PNORM_LAUNCHERS(NAME)                                                                       \
    int launch_pnorm_fwd_##NAME(int mode, bool normalize, bool aligned, Shape s, const PnormFwdArgs& a,         \
                                int grid, hipStream_t st, int* occupancy);                                      \
    int launch_pnorm_bwd_##NAME(int mode, bool aligned, Shape s, const PnormBwdArgs& a, int grid,               \
                                hipStream_t st, int* occupancy);                                                \
    int launch_normalize_bwd_##NAME(int mode, bool aligned, Shape s, const NormalizeBwdArgs& a, int grid,       \
                                    hipStream_t st, int* occupancy);                                            \
    int launch_pnorm_fwd_loop_##NAME(bool normalize, const PnormFwdArgs& a, int grid, hipStream_t st);          \
    int launch_pnorm_bwd_loop_##NAME(const PnormBwdArgs& a, int grid, hipStream_t st);                          \
    int launch_normalize_bwd_loop_##NAME(const NormalizeBwdArgs& a, int grid, hipStream_t st);

THN_DECLARE_PNORM_LAUNCHERS(f32)
THN_DECLARE_PNORM_LAUNCHERS(f16)
THN_DECLARE_PNORM_LAUNCHERS(bf16)
THN_DECLARE_PNORM_LAUNCHERS(f64)

#define THN_PN_FWD_CASE(AL, K_, TPR_, BLOCK_)                                                                   \
    if (s.k == K_ && s.tpr == TPR_ && s.block == BLOCK_) {                                                      \
        if (mode == kP1)                                                                                        \
            return normalize ? run_kernel<PnormFwdArgs>(pnorm_fwd_kernel<T, kP1, true, K_, TPR_, BLOCK_, AL>, a, grid, BLOCK_, st, occupancy)   \
                             : run_kernel<PnormFwdArgs>(pnorm_fwd_kernel<T, kP1, false, K_, TPR_, BLOCK_, AL>, a, grid, BLOCK_, st, occupancy); \
        if (mode == kP2)                                                                                        \
            return normalize ? run_kernel<PnormFwdArgs>(pnorm_fwd_kernel<T, kP2, true, K_, TPR_, BLOCK_, AL>, a, grid, BLOCK_, st, occupancy)   \
                             : run_kernel<PnormFwdArgs>(pnorm_fwd_kernel<T, kP2, false, K_, TPR_, BLOCK_, AL>, a, grid, BLOCK_, st, occupancy); \
        return normalize ? run_kernel<PnormFwdArgs>(pnorm_fwd_kernel<T, kPInt, true, K_, TPR_, BLOCK_, AL>, a, grid, BLOCK_, st, occupancy)     \
                         : run_kernel<PnormFwdArgs>(pnorm_fwd_kernel<T, kPInt, false, K_, TPR_, BLOCK_, AL>, a, grid, BLOCK_, st, occupancy);   \
    }
#define THN_PN_BWD_CASE(KERNEL, ARGS_T, AL, K_, TPR_, BLOCK_)                                                   \
    if (s.k == K_ && s.tpr == TPR_ && s.block == BLOCK_) {                                                      \
        if (mode == kP1) return run_kernel<ARGS_T>(KERNEL<T, kP1, K_, TPR_, BLOCK_, AL>, a, grid, BLOCK_, st, occupancy); \
        if (mode == kP2) return run_kernel<ARGS_T>(KERNEL<T, kP2, K_, TPR_, BLOCK_, AL>, a, grid, BLOCK_, st, occupancy); \
        return run_kernel<ARGS_T>(KERNEL<T, kPInt, K_, TPR_, BLOCK_, AL>, a, grid, BLOCK_, st, occupancy);      \
    }
#define THN_PNF_AL(K_, TPR_, BLOCK_) THN_PN_FWD_CASE(true, K_, TPR_, BLOCK_)
#define THN_PNF_SC(K_, TPR_, BLOCK_) THN_PN_FWD_CASE(false, K_, TPR_, BLOCK_)
#define THN_PNB_AL(K_, TPR_, BLOCK_) THN_PN_BWD_CASE(pnorm_bwd_kernel, PnormBwdArgs, true, K_, TPR_, BLOCK_)
#define THN_PNB_SC(K_, TPR_, BLOCK_) THN_PN_BWD_CASE(pnorm_bwd_kernel, PnormBwdArgs, false, K_, TPR_, BLOCK_)
#define THN_NZB_AL(K_, TPR_, BLOCK_) THN_PN_BWD_CASE(normalize_bwd_kernel, NormalizeBwdArgs, true, K_, TPR_, BLOCK_)
#define THN_NZB_SC(K_, TPR_, BLOCK_) THN_PN_BWD_CASE(normalize_bwd_kernel, NormalizeBwdArgs, false, K_, TPR_, BLOCK_)

#define THN_DEFINE_PNORM_FWD_LAUNCHERS(NAME, TYPE)                                                              \
    int launch_pnorm_fwd_##NAME(int mode, bool normalize, bool aligned, Shape s, const PnormFwdArgs& a,         \
                                int grid, hipStream_t st, int* occupancy) {                                     \
        using T = TYPE;                                                                                         \
        if (aligned) {                                                                                          \
            THN_ROW_SHAPES(THN_PNF_AL)                                                                          \
            THN_PN_SHAPES_FIVE(THN_PNF_AL)                                                                      \
        } else if (a.n_cols >= TYPE::VEC) { \
            THN_ROW_SHAPES(THN_PNF_SC) \
            THN_PN_SHAPES_FIVE(THN_PNF_SC) \
        } else { \
            using T = ElemIo<TYPE>; \
            THN_PNF_SC(4, 8, 256) \
        }                                                                                                       \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_pnorm_fwd_loop_##NAME(bool normalize, const PnormFwdArgs& a, int grid, hipStream_t st) {         \
        return normalize ? run_kernel<PnormFwdArgs>(pnorm_fwd_loop_kernel<TYPE, true>, a, grid, kLoopBlock, st, nullptr) \
                         : run_kernel<PnormFwdArgs>(pnorm_fwd_loop_kernel<TYPE, false>, a, grid, kLoopBlock, st, nullptr); \
    }

#define THN_DEFINE_PNORM_BWD_LAUNCHERS(NAME, TYPE)                                                              \
    int launch_pnorm_bwd_##NAME(int mode, bool aligned, Shape s, const PnormBwdArgs& a, int grid,               \
                                hipStream_t st, int* occupancy) {                                               \
        using T = TYPE;                                                                                         \
        if (aligned) {                                                                                          \
            THN_ROW_SHAPES(THN_PNB_AL)                                                                          \
        } else if (a.n_cols >= TYPE::VEC) { \
            THN_ROW_SHAPES(THN_PNB_SC) \
        } else { \
            using T = ElemIo<TYPE>; \
            THN_PNB_SC(4, 8, 256) \
        }                                                                                                       \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_normalize_bwd_##NAME(int mode, bool aligned, Shape s, const NormalizeBwdArgs& a, int grid,       \
                                    hipStream_t st, int* occupancy) {                                           \
        using T = TYPE;                                                                                         \
        if (aligned) {                                                                                          \
            THN_ROW_SHAPES(THN_NZB_AL)                                                                          \
            THN_PN_SHAPES_FIVE(THN_NZB_AL)                                                                      \
        } else if (a.n_cols >= TYPE::VEC) { \
            THN_ROW_SHAPES(THN_NZB_SC) \
            THN_PN_SHAPES_FIVE(THN_NZB_SC) \
        } else { \
            using T = ElemIo<TYPE>; \
            THN_NZB_SC(4, 8, 256) \
        }                                                                                                       \
        return 1;                                                                                               \
    }                                                                                                           \
    int launch_pnorm_bwd_loop_##NAME(const PnormBwdArgs& a, int grid, hipStream_t st) {                         \
        return run_kernel<PnormBwdArgs>(pnorm_bwd_loop_kernel<TYPE>, a, grid, kLoopBlock, st, nullptr);         \
    }                                                                                                           \
    int launch_normalize_bwd_loop_##NAME(const NormalizeBwdArgs& a, int grid, hipStream_t st) {                 \
        return run_kernel<NormalizeBwdArgs>(normalize_bwd_loop_kernel<TYPE>, a, grid, kLoopBlock, st, nullptr); \
    }

}  // namespace thn
