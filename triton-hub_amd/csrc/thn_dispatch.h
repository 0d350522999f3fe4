// Maps a run-time (dtype, flavour, shape) to one compiled kernel instance.  Each storage type has its own
// pair of translation units (thn_fwd_<dtype>.hip, thn_bwd_<dtype>.hip) that expands these lists, so the types compile in parallel.
#pragma once

#include "thn_kernels.h"

namespace thn {

struct Shape {
    int k;       // vectors (16 bytes) per thread
    int tpr;     // threads per row
    int block;   // threads per workgroup
};

// X(K, TPR, BLOCK): shapes of the 128-bit path.
#define THN_FWD_SHAPES(X)                                                            \
    X(1, 8, 256) X(2, 8, 256) X(4, 8, 256)                                           \
    X(1, 16, 256) X(2, 16, 256) X(4, 16, 256)                                        \
    X(1, 32, 256) X(2, 32, 256) X(4, 32, 256)                                        \
    X(1, 64, 256) X(2, 64, 256) X(3, 64, 256) X(4, 64, 256)                          \
    X(1, 128, 256) X(2, 128, 256) X(3, 128, 256) X(4, 128, 256)                      \
    X(1, 256, 256) X(2, 256, 256) X(3, 256, 256) X(4, 256, 256)                      \
    X(1, 512, 512) X(2, 512, 512) X(3, 512, 512) X(4, 512, 512)                      \
    X(1, 1024, 1024) X(2, 1024, 1024) X(3, 1024, 1024) X(4, 1024, 1024)

// Forward only: rows of 3 x 256 vectors two at a time in 512-thread workgroups.  One such row per 256-thread
// workgroup keeps 12 KiB in flight per compute unit and leaves the two reduction rounds of a row uncovered; two
// 256-thread workgroups per compute unit cover them but pay a second set of parameter loads and launch ramps
// (LayerNorm fp16 8192 x 6144 36.6 -> 35.4 us, 32768 x 6144 139.5 -> 136.3 us, bf16 16384 x 5120 58.4 -> 57.3 us,
// float32 16384 x 3072 68.1 -> 65.8 us; 4 x 256 vectors measured the same both ways and stay in 256 threads).
// Rows of 385 to 512 vectors go the same way, 2 x 256 vectors two at a time, instead of 4 x 128 vectors two at a time
// in 256 threads: eight waves per compute unit cover the reduction rounds of each other's rows (bf16 16384 x 4096
// LayerNorm forward 46.2 -> 45.9 us, RMSNorm 44.9 -> 44.65; 0.1-1 % from 8192 rows on in every type; 4 x 128 in 512
// threads, 1 x 512 and, for rows of 1024 vectors, 2 x 512 in 1024 threads measured 1-4 % slower).
#define THN_FWD_SHAPES_TWO_ROWS(X) X(3, 256, 512) X(2, 256, 512)

// Norm forward and backward only: 3 vectors per thread for rows of 33 to 48 and 65 to 96 vectors (widths of 5 * 2^k
// elements and their neighbours), which fill 5/8 of the next power of two of slots and 5/6 of these.  (The same for
// rows of 17 to 24 vectors, 3 x 8, measured 1-8 points slower than the shapes those rows have.)
#define THN_FWD_SHAPES_THREE(X) X(3, 16, 256) X(3, 32, 256)

#define THN_BWD_SHAPES_THREE(X) X(3, 16, 512) X(3, 32, 512)

// Norm forward only: 3 x 64 and 3 x 128 vectors in 512 threads, eight and four rows at a time -- the row groups of the
// backward over the same rows.  Workgroup w runs on XCD w % 8 and each XCD has an L2 of its own, so with the same rows
// per workgroup in both directions row r is normalised and differentiated on the same XCD, and the backward finds in
// that L2 whatever of x its forward left there (the 256-thread shapes put half as many rows in a workgroup and so a
// different XCD under every second row).  bfloat16 LayerNorm, forward + backward of one batch, 4096 x 2560 28.4 ->
// 25.5 us, 4096 x 2800 30.2 -> 27.5, 26214 x 2560 114.1 -> 111.8; float32 4096 x 1280 27.0 -> 24.1; the forward by
// itself is as fast or faster (float32 48770 x 1376 92.2 -> 89.6 us, bfloat16 23967 x 2800 48.9 -> 46.7).  3 x 16 and
// 3 x 32 are the 16-bit LayerNorm backward's shapes for rows of 33 to 48 and 65 to 96 vectors; the forward takes them
// while x fits the eight L2s (plan_launch()).
#define THN_FWD_SHAPES_AS_BACKWARD(X) X(3, 16, 512) X(3, 32, 512) X(3, 64, 512) X(3, 128, 512)

#define THN_BWD_SHAPES_B(X, B)                                                       \
    X(1, 8, B) X(2, 8, B) X(4, 8, B)                                                 \
    X(1, 16, B) X(2, 16, B) X(4, 16, B)                                              \
    X(1, 32, B) X(2, 32, B) X(4, 32, B)                                              \
    X(1, 64, B) X(2, 64, B) X(3, 64, B) X(4, 64, B)                                  \
    X(1, 128, B) X(2, 128, B) X(3, 128, B) X(4, 128, B)                              \
    X(1, 256, B) X(2, 256, B) X(3, 256, B) X(4, 256, B)

#define THN_BWD_SHAPES(X)                                                            \
    THN_BWD_SHAPES_B(X, 256) THN_BWD_SHAPES_B(X, 512)                                \
    X(1, 512, 512) X(2, 512, 512) X(3, 512, 512) X(4, 512, 512)                      \
    X(1, 1024, 1024) X(2, 1024, 1024) X(3, 1024, 1024) X(4, 1024, 1024)

// LayerNorm backward over 16-bit rows of more than 32 KiB: 5 to 8 vectors per thread in 512-thread workgroups,
// which leave a thread 256 registers for the float32 weights and dB sums of its 40 to 64 columns (the dW sums
// live in LDS).  A 1024-thread workgroup has half as many and spills at 4 vectors per thread.
#define THN_BWD_SHAPES_LN16(X) X(5, 512, 512) X(6, 512, 512) X(7, 512, 512) X(8, 512, 512)

// Rows off the 128-bit path (N not a whole number of 16-byte vectors, or a pointer or stride off 16 bytes) run the
// plain norm kernels in the same shapes as rows on it (their slots are 16-byte windows at element-aligned
// addresses, the ragged last one overlapping its neighbour), and so do the softmax and p-norm families.  The norm
// kernels with an activation epilogue keep one shape per row width there: four vectors per thread.
#define THN_SCALAR_SHAPES(X)                                                         \
    X(4, 8, 256) X(4, 16, 256) X(4, 32, 256) X(4, 64, 256) X(4, 128, 256)            \
    X(4, 256, 256) X(4, 512, 512) X(4, 1024, 1024)

// Return value of the launchers: 0 launched (or occupancy written), 1 no such instance, <0 HIP error.
// When `occupancy` is not null the kernel is not launched; *occupancy receives the number of workgroups
// of that instance that fit on one compute unit.
#define THN_DECLARE_LAUNCHERS(NAME)                                                                        \
    int launch_fwd_##NAME(bool ln, bool aligned, Shape s, const FwdArgs& a, int grid, hipStream_t st,      \
                          int* occupancy);                                                                 \
    int launch_bwd_##NAME(bool ln, bool aligned, Shape s, const BwdArgs& a, int grid, hipStream_t st,      \
                          int* occupancy);

THN_DECLARE_LAUNCHERS(f32)
THN_DECLARE_LAUNCHERS(f16)
THN_DECLARE_LAUNCHERS(bf16)
THN_DECLARE_LAUNCHERS(f64)

template <typename Args>
inline int run_kernel(void (*kern)(const Args), const Args& a, int grid, int block, hipStream_t st,
                      int* occupancy) {
    if (occupancy != nullptr) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, block, 0) != hipSuccess) {
            (void)hipGetLastError();
            return -1;
        }
        *occupancy = n;
        return 0;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(block), 0, st, a);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

#define THN_CASE(KERNEL, ARGS_T, AL, K_, TPR_, BLOCK_)                                                     \
    if (s.k == K_ && s.tpr == TPR_ && s.block == BLOCK_) {                                                 \
        return ln ? run_kernel<ARGS_T>(KERNEL<T, true, K_, TPR_, BLOCK_, AL>, a, grid, BLOCK_, st, occupancy) \
                  : run_kernel<ARGS_T>(KERNEL<T, false, K_, TPR_, BLOCK_, AL>, a, grid, BLOCK_, st, occupancy); \
    }

#define THN_DEFINE_FWD_LAUNCHER(NAME, TYPE)                                                                \
    int launch_fwd_##NAME(bool ln, bool aligned, Shape s, const FwdArgs& a, int grid, hipStream_t st,      \
                          int* occupancy) {                                                                \
        using T = TYPE;                                                                                    \
        if (aligned) {                                                                                     \
            THN_FWD_SHAPES(THN_FWD_AL)                                                                     \
            THN_FWD_SHAPES_TWO_ROWS(THN_FWD_AL)                                                            \
            THN_FWD_SHAPES_THREE(THN_FWD_AL)                                                               \
            THN_FWD_SHAPES_AS_BACKWARD(THN_FWD_AL)                                                         \
        } else if (a.n_cols >= TYPE::VEC) {                                                                \
            THN_FWD_SHAPES(THN_FWD_SC)                                                                     \
            THN_FWD_SHAPES_TWO_ROWS(THN_FWD_SC)                                                            \
            THN_FWD_SHAPES_THREE(THN_FWD_SC)                                                               \
            THN_FWD_SHAPES_AS_BACKWARD(THN_FWD_SC)                                                         \
        } else {                                                                                           \
            using T = ElemIo<TYPE>;                                                                        \
            THN_FWD_SC(4, 8, 256)                                                                          \
        }                                                                                                  \
        return 1;                                                                                          \
    }

#define THN_DEFINE_BWD_LAUNCHER(NAME, TYPE)                                                                \
    int launch_bwd_##NAME(bool ln, bool aligned, Shape s, const BwdArgs& a, int grid, hipStream_t st,      \
                          int* occupancy) {                                                                \
        using T = TYPE;                                                                                    \
        if (aligned) {                                                                                     \
            THN_BWD_SHAPES(THN_BWD_AL)                                                                     \
            THN_BWD_SHAPES_THREE(THN_BWD_AL)                                                               \
            if constexpr (TYPE::kBytes == 2) {                                                             \
                if (ln) {                                                                                  \
                    THN_BWD_SHAPES_LN16(THN_BWD_AL_LN)                                                     \
                }                                                                                          \
            }                                                                                              \
        } else if (a.n_cols >= TYPE::VEC) {                                                                \
            THN_BWD_SHAPES(THN_BWD_SC)                                                                     \
            THN_BWD_SHAPES_THREE(THN_BWD_SC)                                                               \
        } else {                                                                                           \
            using T = ElemIo<TYPE>;                                                                        \
            THN_BWD_SC(4, 8, 256)                                                                          \
        }                                                                                                  \
        return 1;                                                                                          \
    }

// The forward has two instances per shape: x kept in the caches for the backward, or streamed (FwdArgs::keep_x).
#define THN_FWD_CASE(AL, K_, TPR_, BLOCK_)                                                                 \
    if (s.k == K_ && s.tpr == TPR_ && s.block == BLOCK_) {                                                 \
        if (a.keep_x) {                                                                                    \
            return ln ? run_kernel<FwdArgs>(norm_fwd_kernel<T, true, K_, TPR_, BLOCK_, AL, kNoAct, true>, a, grid, BLOCK_, st, occupancy) \
                      : run_kernel<FwdArgs>(norm_fwd_kernel<T, false, K_, TPR_, BLOCK_, AL, kNoAct, true>, a, grid, BLOCK_, st, occupancy); \
        }                                                                                                  \
        return ln ? run_kernel<FwdArgs>(norm_fwd_kernel<T, true, K_, TPR_, BLOCK_, AL, kNoAct, false>, a, grid, BLOCK_, st, occupancy) \
                  : run_kernel<FwdArgs>(norm_fwd_kernel<T, false, K_, TPR_, BLOCK_, AL, kNoAct, false>, a, grid, BLOCK_, st, occupancy); \
    }
#define THN_FWD_AL(K_, TPR_, BLOCK_) THN_FWD_CASE(true, K_, TPR_, BLOCK_)
#define THN_FWD_SC(K_, TPR_, BLOCK_) THN_FWD_CASE(false, K_, TPR_, BLOCK_)
#define THN_BWD_AL(K_, TPR_, BLOCK_) THN_CASE(norm_bwd_kernel, BwdArgs, true, K_, TPR_, BLOCK_)
#define THN_BWD_AL_LN(K_, TPR_, BLOCK_)                                                                    \
    if (s.k == K_ && s.tpr == TPR_ && s.block == BLOCK_) {                                                 \
        return run_kernel<BwdArgs>(norm_bwd_kernel<T, true, K_, TPR_, BLOCK_, true>, a, grid, BLOCK_, st, occupancy); \
    }
#define THN_BWD_SC(K_, TPR_, BLOCK_) THN_CASE(norm_bwd_kernel, BwdArgs, false, K_, TPR_, BLOCK_)

}  // namespace thn
