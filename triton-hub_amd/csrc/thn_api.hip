// C ABI of libthnorm.so (declared in include/thnorm.h): argument checks, launch-shape heuristic,
// persistent-grid sizing and kernel dispatch.  No allocation, no synchronisation, no retained pointers.
#include "thnorm.h"

#include <atomic>
#include <initializer_list>
#include <mutex>
#include <unordered_map>

#include "thn_dispatch.h"
#include "thn_flat.h"
#include "thn_staged.h"
#include "thn_fused_dispatch.h"
#include "thn_reduce.h"
#include "thn_act_dispatch.h"
#include "thn_dropout.h"
#include "thn_pnorm_dispatch.h"
#include "thn_softmax_dispatch.h"
#include "thn_softmax_flat.h"
#include "thn_pnorm_flat.h"
#include "thn_tiny.h"

namespace {

using thn::ActArgs;
using thn::BwdArgs;
using thn::FwdArgs;
using thn::NormalizeBwdArgs;
using thn::PnormBwdArgs;
using thn::PnormFwdArgs;
using thn::RowMap;
using thn::Shape;
using thn::SoftmaxBwdArgs;
using thn::SoftmaxFwdArgs;

// `which` throughout this file: the kernel family a launch belongs to.
enum : int {
    kNormFwd = 0, kNormBwd = 1, kSoftmaxFwd = 2, kSoftmaxBwd = 3, kPnormFwd = 4, kPnormBwd = 5, kNormalizeBwd = 6,
    kActFwd = 7, kActBwd = 8, kFusedFwd = 9, kFusedBwd = 10, kFamilies = 11
};

constexpr int kMaxDevices = 64;
constexpr int64_t kMaxRowBytes = 65536;   // the reference's MAX_FUSED_SIZE (layernorm.py:69-72)
constexpr int kMaxBlocksPerCu = 8;

std::atomic<int> g_cu_count[kMaxDevices];

int current_cu_count() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return 0;
    }
    int n = g_cu_count[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            return 0;
        }
        g_cu_count[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

int elem_bytes(int dtype) {
    switch (dtype) {
        case THN_F32: return 4;
        case THN_F16: return 2;
        case THN_BF16: return 2;
        case THN_F64: return 8;
        default: return 0;
    }
}

struct Override {
    std::atomic<int> k{0}, tpr{0}, block{0}, bpc{0};
};
Override g_override[kFamilies];

// Default cache policy of the forward's read of x (thn_norm_set_cache_policy).
std::atomic<int> g_cache_policy{THN_CACHE_KEEP_X};
constexpr int kPolicyFlags = THN_X_KEEP | THN_X_STREAM;

// `ln16`: LayerNorm over 16-bit rows (the two norm backwards have instances of their own for that).
bool shape_compiled(int which, bool aligned, bool ln16, Shape s) {
#define THN_MATCH(K_, TPR_, BLOCK_) if (s.k == K_ && s.tpr == TPR_ && s.block == BLOCK_) return true;
    if (!aligned && (which == kFusedFwd || which == kFusedBwd)) {
        THN_SCALAR_SHAPES(THN_MATCH)
    } else if (!aligned && which == kNormBwd) {
        THN_BWD_SHAPES(THN_MATCH)
        THN_BWD_SHAPES_THREE(THN_MATCH)
    } else if (which == kNormBwd) {
        THN_BWD_SHAPES(THN_MATCH)
        THN_BWD_SHAPES_THREE(THN_MATCH)
        if (ln16) {
            THN_BWD_SHAPES_LN16(THN_MATCH)
        }
    } else if (which == kFusedFwd) {
        THN_FUSED_FWD_SHAPES(THN_MATCH)
    } else if (which == kFusedBwd) {
        THN_FUSED_BWD_SHAPES(THN_MATCH)
        if (ln16) {
            THN_FUSED_BWD_SHAPES_LN16(THN_MATCH)
        }
    } else if (which >= kPnormFwd) {
        THN_ROW_SHAPES(THN_MATCH)
        if (which != kPnormBwd) {
            THN_PN_SHAPES_FIVE(THN_MATCH)
        }
    } else {
        THN_FWD_SHAPES(THN_MATCH)
        if (which == kNormFwd) {
            THN_FWD_SHAPES_TWO_ROWS(THN_MATCH)
            THN_FWD_SHAPES_AS_BACKWARD(THN_MATCH)
        }
        THN_FWD_SHAPES_THREE(THN_MATCH)
        if (which == kSoftmaxFwd || which == kSoftmaxBwd) {
            THN_SM_SHAPES_FIVE(THN_MATCH)
        }
    }
#undef THN_MATCH
    return false;
}

int launch_fwd(int dtype, bool ln, bool aligned, Shape s, const FwdArgs& a, int grid, hipStream_t st, int* occ) {
    switch (dtype) {
        case THN_F32: return thn::launch_fwd_f32(ln, aligned, s, a, grid, st, occ);
        case THN_F16: return thn::launch_fwd_f16(ln, aligned, s, a, grid, st, occ);
        case THN_BF16: return thn::launch_fwd_bf16(ln, aligned, s, a, grid, st, occ);
        default: return thn::launch_fwd_f64(ln, aligned, s, a, grid, st, occ);
    }
}

int launch_bwd(int dtype, bool ln, bool aligned, Shape s, const BwdArgs& a, int grid, hipStream_t st, int* occ) {
    switch (dtype) {
        case THN_F32: return thn::launch_bwd_f32(ln, aligned, s, a, grid, st, occ);
        case THN_F16: return thn::launch_bwd_f16(ln, aligned, s, a, grid, st, occ);
        case THN_BF16: return thn::launch_bwd_bf16(ln, aligned, s, a, grid, st, occ);
        default: return thn::launch_bwd_f64(ln, aligned, s, a, grid, st, occ);
    }
}

int launch_softmax_fwd(int dtype, bool is_log, bool aligned, Shape s, const SoftmaxFwdArgs& a, int grid,
                       hipStream_t st, int* occ) {
    switch (dtype) {
        case THN_F32: return thn::launch_softmax_fwd_f32(is_log, aligned, s, a, grid, st, occ);
        case THN_F16: return thn::launch_softmax_fwd_f16(is_log, aligned, s, a, grid, st, occ);
        case THN_BF16: return thn::launch_softmax_fwd_bf16(is_log, aligned, s, a, grid, st, occ);
        default: return thn::launch_softmax_fwd_f64(is_log, aligned, s, a, grid, st, occ);
    }
}

int launch_softmax_bwd(int dtype, bool is_log, bool aligned, Shape s, const SoftmaxBwdArgs& a, int grid,
                       hipStream_t st, int* occ) {
    switch (dtype) {
        case THN_F32: return thn::launch_softmax_bwd_f32(is_log, aligned, s, a, grid, st, occ);
        case THN_F16: return thn::launch_softmax_bwd_f16(is_log, aligned, s, a, grid, st, occ);
        case THN_BF16: return thn::launch_softmax_bwd_bf16(is_log, aligned, s, a, grid, st, occ);
        default: return thn::launch_softmax_bwd_f64(is_log, aligned, s, a, grid, st, occ);
    }
}

// `variant` of the fused families: bit 0 = LayerNorm, bits 1.. = the activation code.
// Workgroup size and workgroups per compute unit of the looping softmax kernels (rows wider than 64 KiB); the
// launch override of the family (block_threads, blocks_per_cu) replaces them.
void softmax_loop_launch(int which, int* block, int* bpc);

int launch_softmax_fwd_loop(int dtype, bool is_log, int block, const SoftmaxFwdArgs& a, int grid, hipStream_t st) {
    switch (dtype) {
        case THN_F32: return thn::launch_softmax_fwd_loop_f32(is_log, block, a, grid, st);
        case THN_F16: return thn::launch_softmax_fwd_loop_f16(is_log, block, a, grid, st);
        case THN_BF16: return thn::launch_softmax_fwd_loop_bf16(is_log, block, a, grid, st);
        default: return thn::launch_softmax_fwd_loop_f64(is_log, block, a, grid, st);
    }
}

int launch_softmax_bwd_loop(int dtype, bool is_log, int block, const SoftmaxBwdArgs& a, int grid, hipStream_t st) {
    switch (dtype) {
        case THN_F32: return thn::launch_softmax_bwd_loop_f32(is_log, block, a, grid, st);
        case THN_F16: return thn::launch_softmax_bwd_loop_f16(is_log, block, a, grid, st);
        case THN_BF16: return thn::launch_softmax_bwd_loop_bf16(is_log, block, a, grid, st);
        default: return thn::launch_softmax_bwd_loop_f64(is_log, block, a, grid, st);
    }
}

int launch_fused_fwd(int dtype, int variant, bool aligned, Shape s, const FwdArgs& a, int grid, hipStream_t st, int* occ) {
    const bool ln = (variant & 1) != 0;
    const int act = variant >> 1;
    switch (dtype) {
        case THN_F32: return thn::launch_fused_fwd_f32(ln, act, aligned, s, a, grid, st, occ);
        case THN_F16: return thn::launch_fused_fwd_f16(ln, act, aligned, s, a, grid, st, occ);
        case THN_BF16: return thn::launch_fused_fwd_bf16(ln, act, aligned, s, a, grid, st, occ);
        default: return thn::launch_fused_fwd_f64(ln, act, aligned, s, a, grid, st, occ);
    }
}

int launch_fused_bwd(int dtype, int variant, bool aligned, Shape s, const BwdArgs& a, int grid, hipStream_t st, int* occ) {
    const bool ln = (variant & 1) != 0;
    const int act = variant >> 1;
    switch (dtype) {
        case THN_F32: return thn::launch_fused_bwd_f32(ln, act, aligned, s, a, grid, st, occ);
        case THN_F16: return thn::launch_fused_bwd_f16(ln, act, aligned, s, a, grid, st, occ);
        case THN_BF16: return thn::launch_fused_bwd_bf16(ln, act, aligned, s, a, grid, st, occ);
        default: return thn::launch_fused_bwd_f64(ln, act, aligned, s, a, grid, st, occ);
    }
}

// `variant` of the p-norm families: the p mode (thn::kP1 / kP2 / kPInt), plus 4 when the forward also normalises.
int launch_pnorm_fwd(int dtype, int variant, bool aligned, Shape s, const PnormFwdArgs& a, int grid, hipStream_t st,
                     int* occ) {
    const int mode = variant & 3;
    const bool nz = (variant & 4) != 0;
    switch (dtype) {
        case THN_F32: return thn::launch_pnorm_fwd_f32(mode, nz, aligned, s, a, grid, st, occ);
        case THN_F16: return thn::launch_pnorm_fwd_f16(mode, nz, aligned, s, a, grid, st, occ);
        case THN_BF16: return thn::launch_pnorm_fwd_bf16(mode, nz, aligned, s, a, grid, st, occ);
        default: return thn::launch_pnorm_fwd_f64(mode, nz, aligned, s, a, grid, st, occ);
    }
}

int launch_pnorm_bwd(int dtype, int mode, bool aligned, Shape s, const PnormBwdArgs& a, int grid, hipStream_t st,
                     int* occ) {
    switch (dtype) {
        case THN_F32: return thn::launch_pnorm_bwd_f32(mode, aligned, s, a, grid, st, occ);
        case THN_F16: return thn::launch_pnorm_bwd_f16(mode, aligned, s, a, grid, st, occ);
        case THN_BF16: return thn::launch_pnorm_bwd_bf16(mode, aligned, s, a, grid, st, occ);
        default: return thn::launch_pnorm_bwd_f64(mode, aligned, s, a, grid, st, occ);
    }
}

int launch_normalize_bwd(int dtype, int mode, bool aligned, Shape s, const NormalizeBwdArgs& a, int grid,
                         hipStream_t st, int* occ) {
    switch (dtype) {
        case THN_F32: return thn::launch_normalize_bwd_f32(mode, aligned, s, a, grid, st, occ);
        case THN_F16: return thn::launch_normalize_bwd_f16(mode, aligned, s, a, grid, st, occ);
        case THN_BF16: return thn::launch_normalize_bwd_bf16(mode, aligned, s, a, grid, st, occ);
        default: return thn::launch_normalize_bwd_f64(mode, aligned, s, a, grid, st, occ);
    }
}

// Workgroups of one kernel instance that fit on a compute unit; asked of the runtime once per instance.
std::mutex g_occ_mutex;
std::unordered_map<uint64_t, int> g_occ_cache;

// `flavour`: the kernel variant within the family -- 1 for LayerNorm / log-softmax, 0 for RMSNorm / softmax; the
// `variant` described above for the p-norm and epilogue families.
int occupancy(int which, int dtype, int flavour, bool aligned, Shape s) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    const uint64_t key = (static_cast<uint64_t>(dev) << 44) | (static_cast<uint64_t>(which) << 40) |
                         (static_cast<uint64_t>(dtype) << 36) | (static_cast<uint64_t>(flavour) << 32) |
                         (static_cast<uint64_t>(aligned) << 30) | (static_cast<uint64_t>(s.k) << 24) |
                         (static_cast<uint64_t>(s.tpr) << 12) | static_cast<uint64_t>(s.block);
    {
        std::lock_guard<std::mutex> lock(g_occ_mutex);
        auto it = g_occ_cache.find(key);
        if (it != g_occ_cache.end()) return it->second;
    }
    int occ = 0;
    int rc;
    if (which == kNormFwd) {
        FwdArgs dummy{};
        dummy.keep_x = 1;
        dummy.n_cols = 1 << 20;      // the unaligned-window instances, not the ones for rows shorter than a vector
        rc = launch_fwd(dtype, flavour, aligned, s, dummy, 0, nullptr, &occ);
    } else if (which == kNormBwd) {
        BwdArgs dummy{};
        dummy.n_cols = 1 << 20;      // the unaligned-window instances, not the ones for rows shorter than a vector
        rc = launch_bwd(dtype, flavour, aligned, s, dummy, 0, nullptr, &occ);
    } else if (which == kSoftmaxFwd) {
        SoftmaxFwdArgs dummy{};
        dummy.n_cols = 1 << 20;      // the unaligned-window instances, not the ones for rows shorter than a vector
        rc = launch_softmax_fwd(dtype, flavour, aligned, s, dummy, 0, nullptr, &occ);
    } else if (which == kSoftmaxBwd) {
        SoftmaxBwdArgs dummy{};
        dummy.n_cols = 1 << 20;      // the unaligned-window instances, not the ones for rows shorter than a vector
        rc = launch_softmax_bwd(dtype, flavour, aligned, s, dummy, 0, nullptr, &occ);
    } else if (which == kFusedFwd) {
        FwdArgs dummy{};
        dummy.keep_x = 1;
        dummy.n_cols = 1 << 20;      // the unaligned-window instances, not the ones for rows shorter than a vector
        rc = launch_fused_fwd(dtype, flavour, aligned, s, dummy, 0, nullptr, &occ);
    } else if (which == kFusedBwd) {
        BwdArgs dummy{};
        dummy.n_cols = 1 << 20;      // the unaligned-window instances, not the ones for rows shorter than a vector
        rc = launch_fused_bwd(dtype, flavour, aligned, s, dummy, 0, nullptr, &occ);
    } else if (which == kPnormFwd) {
        PnormFwdArgs dummy{};
        dummy.n_cols = 1 << 20;      // the unaligned-window instances, not the ones for rows shorter than a vector
        rc = launch_pnorm_fwd(dtype, flavour, aligned, s, dummy, 0, nullptr, &occ);
    } else if (which == kPnormBwd) {
        PnormBwdArgs dummy{};
        dummy.n_cols = 1 << 20;      // the unaligned-window instances, not the ones for rows shorter than a vector
        rc = launch_pnorm_bwd(dtype, flavour, aligned, s, dummy, 0, nullptr, &occ);
    } else {
        NormalizeBwdArgs dummy{};
        dummy.n_cols = 1 << 20;      // the unaligned-window instances, not the ones for rows shorter than a vector
        rc = launch_normalize_bwd(dtype, flavour, aligned, s, dummy, 0, nullptr, &occ);
    }
    if (rc != 0 || occ <= 0) occ = 1;
    if (occ > kMaxBlocksPerCu) occ = kMaxBlocksPerCu;
    std::lock_guard<std::mutex> lock(g_occ_mutex);
    g_occ_cache[key] = occ;
    return occ;
}

struct Plan {
    Shape s;
    int grid;
    int n_vecs;
    bool aligned;
};

constexpr int kTprList[] = {8, 16, 32, 64, 128, 256, 512, 1024};

// The static replacement of the reference's autotune over num_warps (autotune.py:62-65), fitted to sweeps
// over (vectors per thread, threads per row, workgroup size, workgroups per compute unit) on MI355X at row
// widths from 1 KiB to 64 KiB.  HBM throughput peaks when a compute unit keeps about 1024 (one input stream) to
// 2048 (two) 16-byte loads in flight and falls off by up to 15 % beyond that, so, for every row family: the
// fewest threads per row with at most `kmax` vectors each, and
//   norm forward, softmax forward, p-norm forward / backward: kmax 4, 256-thread workgroups up to 16 KiB rows
//             (the norm forward takes rows of 3 x 256 and, from 8 steps per workgroup on, of 2 x 256 vectors two
//             at a time in 512 threads: plan_launch());
//   norm backward: kmax 3 (x, dy, w, dW, dB are live per element), 4 for rows of at most 2 KiB (they share a
//             wave: the float64 column sums need the instruction-level parallelism) and for rows that 1024
//             threads cannot cover otherwise; 512-thread workgroups once a row spans two waves or more, which
//             also halves the number of partial rows;
//   normalize / epilogue backward (two or three input streams): kmax 2 up to 32 KiB rows; the softmax backward the
//             forward's shape up to 8 KiB rows and kmax 2 from there to 32 KiB.
// A second finding runs through the norm rules of plan_launch(): a compute unit wants eight waves of a row kernel,
// not four.  One 256-thread workgroup per compute unit (one wave per SIMD) leaves a row's arithmetic and reduction
// rounds uncovered -- the 16-bit LayerNorm forward then takes 1.3 us per row at any width -- so the backward of
// narrow rows, the rows that fill most of a 2-vector shape and the 16-bit forward rows of 769 to 1024 vectors run in
// 512-thread workgroups, and one-row-at-a-time workgroups (the line shift) are kept for rows that fill their shape.
// Workgroups per compute unit: one (kDefaultBlocksPerCu), except where default_blocks_per_cu(),
// narrow_row_blocks_per_cu() or the row-count dependent rules in plan_launch() say otherwise.
constexpr int kDefaultBlocksPerCu = 1;

int ceil_div(int a, int b) { return (a + b - 1) / b; }

Shape heuristic_shape(int which, bool aligned, bool ln16, int n_vecs) {
    // LayerNorm backward over 16-bit rows of more than 32 KiB: 512 threads with 5 to 8 vectors each (256 registers
    // per thread) instead of 1024 threads with 3 or 4 (bf16 N = 20480 / 24576 / 28672 / 32768: 122 / 139 / 183 /
    // 203 us -> 112 / 131 / 156 / 187 us for 4096 rows; with a GeLU epilogue N = 20480 / 28672: 286 / 518 -> 218 /
    // 373 us).
    if ((which == kNormBwd || which == kFusedBwd) && aligned && ln16 && n_vecs > 2048) {
        return Shape{ceil_div(n_vecs, 512), 512, 512};
    }
    // (every family but the norm kernels with an activation epilogue takes the same shapes off the 128-bit path as on it)
    const bool same_shapes = which != kFusedFwd && which != kFusedBwd;
    int kmax = (which == kNormBwd && n_vecs > 128) ? 3 : 4;
    // Softmax backward: the forward's shape up to 8 KiB rows -- as many rows per workgroup in both directions, so a row
    // meets the same XCD and its L2 (forward + backward of 2^26 elements: bfloat16 N = 512 / 2048 / 4096 101.2 / 102.7 /
    // 103.3 -> 98.9 / 99.1 / 98.9 us, N = 1792 / 3584 110.2 / 111.0 -> 102.0 / 102.2, N = 4095 122.8 -> 110.6; float32
    // N = 224 / 896 / 1792 216.2 / 216.9 / 217.1 -> 195.8 / 195.5 / 197.4; the backward by itself gains 1-6 % as well);
    // wider rows 2 vectors per thread per stream (bfloat16 N = 8192 98.5 us against 98.9, float32 N = 8192 198.7 / 200.8).
    if (which == kSoftmaxBwd && n_vecs > 512 && n_vecs <= 2048) kmax = 2;
    if (which == kNormalizeBwd && n_vecs <= 2048) kmax = 2;    // two or three input streams
    if (aligned && which == kFusedBwd && n_vecs <= 2048) kmax = n_vecs > 128 ? 3 : 2;   // bias and pre-activation are live too
    Shape s{4, 1024, 1024};
    for (int tpr : kTprList) {
        if (static_cast<int64_t>(tpr) * kmax >= n_vecs) {
            s.tpr = tpr;
            break;
        }
    }
    if (!aligned && !same_shapes) {
        s.k = 4;
        s.block = s.tpr > 256 ? s.tpr : 256;
        return s;
    }
    if (which == kNormBwd && n_vecs > 8 && n_vecs <= 16) s.tpr = 16;      // 256-byte rows: one vector per thread
    s.k = ceil_div(n_vecs, s.tpr);
    // The softmax backward over rows of more than 8 KiB prefers 2 vectors per thread, but a row of 3 * 2^k vectors (or
    // a little less) would leave a quarter to a half of the slots without work: then 3 vectors on half the threads
    // (measured when narrower rows had 2 vectors as well: bf16 N = 1280 / 2560 / 3072: 5.0 / 5.0 / 5.5 -> 6.0 / 6.4 /
    // 6.3 TB/s).
    if (which == kSoftmaxBwd && s.k == 2 && s.tpr >= 128) {
        const int half = s.tpr / 2;
        if (3 * half >= n_vecs) {          // at most three quarters of the 2-vector slots would have work
            s.tpr = half;
            s.k = 3;
        }
    }
    if (s.k == 3 && s.tpr < 64) s.k = 4;     // K = 3 is only compiled for TPR >= 64
    if (which != kNormBwd && which != kFusedBwd) s.block = s.tpr > 256 ? s.tpr : 256;
    else s.block = s.tpr >= 128 ? (s.tpr > 512 ? s.tpr : 512) : 256;
    if (which == kNormFwd && s.k == 3 && s.tpr == 256) s.block = 512;     // THN_FWD_SHAPES_TWO_ROWS
    // The norm backward over rows of up to 16 vectors (one vector per thread): 512-thread workgroups, two per compute
    // unit (forward + backward of 2^26 elements, % of 8 TB/s, RMSNorm / LayerNorm: bf16 N = 96 68.8 / 66.1 ->
    // 75.0 / 72.9, N = 128 75.9 / 74.1 -> 78.3 / 76.3, N = 64 71.1 / 68.1 -> 72.1 / 68.9; float32 N = 64 79.5 / 76.0 ->
    // 80.3 / 78.4).
    if (which == kNormBwd && aligned && n_vecs <= 16 && s.k == 1) s.block = 512;
    return s;
}

// Upper limit of workgroups per compute unit the library picks by itself (the occupancy may allow fewer).
int default_blocks_per_cu(int which, int flavour, int block) {
    // The p-norm families in 256-thread workgroups (rows up to 16 KiB) measured 5-25 % faster with two workgroups
    // per compute unit.
    if (which >= kPnormFwd && which <= kNormalizeBwd && block <= 256) return 2;
    // A GeLU epilogue makes the norm kernels arithmetic-bound (about 30 instruction slots per element): they take
    // as many workgroups per compute unit as their registers allow, up to four.
    if ((which == kFusedFwd || which == kFusedBwd) && ((flavour >> 1) == thn::kGelu || (flavour >> 1) == thn::kGeluTanh)) return 4;
    return kDefaultBlocksPerCu;
}

void softmax_loop_launch(int which, int* block, int* bpc) {
    *block = 1024;      // sweep over {256, 512, 1024} x {1, 2, 4, 8}: 1024 x 2 best or within 2 % of the best at every width
    *bpc = 2;
    const int ob = g_override[which].block.load(), oc = g_override[which].bpc.load();
    if (ob == 256 || ob == 512 || ob == 1024) *block = ob;
    if (oc > 0) *bpc = oc < kMaxBlocksPerCu ? oc : kMaxBlocksPerCu;
}

// Rows of at most 256 bytes: a thread holds one or two vectors, so one workgroup per compute unit keeps too few
// bytes in flight (measured: bf16 N = 64 forward 3.1 TB/s with one workgroup per compute unit, 5.3 TB/s with
// four; backward 4.3 -> 6.1 TB/s with two).  Families with one input stream take 4 workgroups up to 128-byte
// rows and 2 up to 256-byte rows; those with two streams 2 up to 128-byte rows (the norm backward up to 256-byte
// rows, where it runs one vector per thread: bf16 N = 128 5.2 -> 6.1 TB/s).
int narrow_row_blocks_per_cu(int which, int n_vecs, bool ragged16) {
    // 16-bit rows whose width is not a whole number of vectors.  The norm kernels with an activation epilogue run four
    // vectors per thread there whatever the width, and a second workgroup hides the latency of their arithmetic.  The
    // plain norm kernels' overlapped windows cost no more than aligned vectors and lose 5-7 % with a second workgroup (bf16 24564 x 4098 forward 69.1 us with one, 73.4 with two; fp16 8192 x 12289
    // 81.6 / 85.0).  The softmax forward has the same windows, but holds so little per row that rows of more than 128
    // vectors still gain from the second workgroup (bfloat16, 2^26 elements, one / two: N = 1025 74.7 / 57.4 us, 2050
    // 63.9 / 57.4, 5001 63.8 / 60.1) and narrower ones lose (forward + backward, % of 8 TB/s: N = 197 63.1 / 60.7; 300
    // 72.2 / 70.5; 577 67.6 / 65.4; 1023 77.5 / 73.0); the softmax backward is 3-10 % faster with one at every width
    // (N = 1025 71.0 / 76.7 us, 1500 64.7 / 70.0, 2050 67.2 / 73.3, 4098 67.4 / 73.8, 6001 68.6 / 82.2, 8191 68.3 / 79.7);
    // the p-norm family takes two workgroups of 256 threads anyway, and the normalize backward one of 512 threads
    // (rows of more than 512 vectors: N = 4098 70.8 / 77.4 us, 6001 73.0 / 85.4, 8191 68.4 / 80.8).
    const bool fused = which == kFusedFwd || which == kFusedBwd;
    if (ragged16 && n_vecs > 16 && which != kNormFwd && which != kNormBwd && which != kSoftmaxBwd &&
        which != kNormalizeBwd && (fused || n_vecs > 128)) {
        return 2;
    }
    const bool one_stream = which == kNormFwd || which == kSoftmaxFwd || which == kPnormFwd || which == kFusedFwd;
    if (n_vecs <= 8) return one_stream ? 4 : 2;
    if (n_vecs <= 16) return (one_stream || which == kNormBwd) ? 2 : 1;   // norm backward: with one vector per thread
    return 1;
}

// `pitch_bytes`: distance between rows of x when the caller knows it and every row sits at row * pitch (0 otherwise).
int plan_launch(int which, int flavour, bool aligned, int64_t M, int64_t N, int dtype, Plan* out,
                int64_t pitch_bytes = 0) {
    const int bytes = elem_bytes(dtype);
    if (bytes == 0) return THN_E_DTYPE;
    if (M < 0 || N <= 0) return THN_E_SHAPE;
    if (N * bytes > kMaxRowBytes) return THN_E_FEATURE_DIM;
    const int vec_elems = 16 / bytes;
    const int n_vecs = static_cast<int>((N + vec_elems - 1) / vec_elems);
    const int cus = current_cu_count();
    if (cus <= 0) return THN_E_DEVICE;

    // (rows shorter than one vector have a single element-wise instance)
    const bool ln16 = (which == kNormBwd || which == kFusedBwd) && bytes == 2 && (flavour & 1) != 0 && N >= vec_elems;
    Shape s = heuristic_shape(which, aligned, ln16, n_vecs);
    // The norm forward over rows of 385 to 512 vectors: 2 x 256 vectors, two rows at a time in 512 threads
    // (THN_FWD_SHAPES_TWO_ROWS), unless the kernel is so short that the 256-thread shape takes two workgroups per
    // compute unit (below).
    // (off the 128-bit path as well: bfloat16 N = 3357 / 3997 LayerNorm forward 53.0 / 50.7 -> 49.9 / 47.3 us per 2^26
    // elements, RMSNorm 47.6 / 47.3 -> 46.8 / 46.7)
    if (which == kNormFwd && N >= vec_elems && s.k == 4 && s.tpr == 128 && s.block == 256 && n_vecs > 384 &&
        M > 16 * static_cast<int64_t>(cus)) {
        s = Shape{2, 256, 512};
    }
    // Rows that fill 11/16 or more of a 2-vector shape with twice the threads go there instead of 3 vectors per
    // thread: 352 to 384 vectors as 2 x 256 (forward and backward; not the 16-bit LayerNorm forward, which is 0-5 %
    // slower that way), float32 rows of 704 to 768 vectors as 2 x 512.  Forward + backward of 2^26 elements, % of
    // 8 TB/s, RMSNorm / LayerNorm: float32 N = 1408: 78.8 / 78.2 -> 81.0 / 79.8; 1536: 79.2 / 78.6 -> 81.8 / 80.5;
    // 3072: 79.6 / 79.2 -> 82.0 / 80.5; bf16 N = 2816: 76.0 / 73.9 -> 77.2 / 74.5; 3072: 76.0 / 74.2 -> 78.4 / 74.7.
    // Emptier rows lose: float32 N = 1152 forward 92 -> 101 us, bf16 N = 2688 LayerNorm 73.8 -> 70.7 %.
    {
        const bool norm_bwd = which == kNormBwd, norm_fwd = which == kNormFwd;
        const bool ln_fwd16 = norm_fwd && bytes == 2 && (flavour & 1) != 0;
        Shape two = s;
        if (n_vecs >= 352 && n_vecs <= 384 && !ln_fwd16) two = Shape{2, 256, 512};
        if (n_vecs >= 704 && n_vecs <= 768 && bytes == 4) two = Shape{2, 512, 512};
        if ((norm_bwd || (norm_fwd && M > 16 * static_cast<int64_t>(cus))) && aligned && s.k == 3 &&
            shape_compiled(which, aligned, ln16, two)) {
            s = two;
        }
    }
    // The forward over 16-bit rows of 769 to 1024 vectors: one row of 4 x 256 vectors per 256-thread workgroup is one
    // wave per SIMD, and a row's arithmetic and two reduction rounds then set a floor of 1.3 us per row for LayerNorm
    // whatever the width (4608 rows: 25 us at every width from 6400 to 8192 columns).  2 x 512 vectors in 512 threads
    // instead: for rows of up to 896 vectors at every row count, for wider ones up to 32 rows per compute unit (bf16
    // forward, RMSNorm / LayerNorm: 4608 x 6656 19.1 / 24.9 -> 18.9 / 21.0 us, 16384 x 6656 74.9 / 79.9 -> 72.1 / 74.7,
    // 32768 x 7168 158.0 / 157.7 -> 156.9 / 156.1, 4608 x 8192 22.8 / 25.4 -> 22.8 / 23.8; from 16384 rows on the
    // rows of more than 896 vectors are 1-5 % faster as 4 x 256: 16384 x 8192 87.8 / 87.7 against 89.0 / 90.8).
    // Up to 8 rows per compute unit the 256-thread shape takes two workgroups per compute unit (below) and stays.
    // Off the 128-bit path at every row count (bfloat16 N = 7197 / 7997 LayerNorm forward 59.0 / 60.5 -> 56.4 / 50.8 us
    // per 2^26 elements, RMSNorm 53.5 / 48.2 -> 52.3 / 47.6).
    if (which == kNormFwd && N >= vec_elems && bytes == 2 && s.k == 4 && s.tpr == 256 && s.block == 256 &&
        M > 8 * static_cast<int64_t>(cus) && (n_vecs <= 896 || !aligned || M <= 32 * static_cast<int64_t>(cus))) {
        s = Shape{2, 512, 512};
    }
    // The norm backward over narrow rows (17 to 192 vectors, every storage type, on and off the 128-bit path): 2
    // vectors per thread in 512-thread workgroups -- eight waves per compute unit instead of the four of a 256-thread
    // workgroup, which a backward step does not fill a compute unit with, and twice the threads per row of the
    // 4-vector shapes, so that a wave's request is made of fewer, longer pieces (at a pitch that is not a multiple of
    // 128 bytes every piece starts and ends inside a line).  The LayerNorm backward over 16-bit rows of up to 96
    // vectors goes one step further: 1 vector per thread, two workgroups per compute unit.  Forward + backward of
    // 2^26 elements with only the backward's shape changed, % of 8 TB/s, 4 x TPR / 256 -> 2 x TPR / 512 (-> 1 x TPR /
    // 512, two per compute unit): float32 RMSNorm N = 72: 62.4 -> 75.7; 96: 78.2 -> 79.6; 136: 68.8 -> 75.6; 200:
    // 77.3 -> 79.9; 256: 82.0 -> 81.9; 384: 79.0 -> 80.0; 512: 81.9 -> 81.9; bfloat16 RMSNorm N = 200: 65.3 -> 73.4;
    // 256: 74.8 -> 77.3; 640: 65.5 -> 74.4; 1000: 75.1 -> 76.4; bfloat16 LayerNorm N = 160: 59.6 -> 69.2 -> 71.3; 200:
    // 65.0 -> 70.9 -> 72.6; 256: 70.6 -> 74.3 -> 77.0; 384: 66.6 -> 71.4 -> 73.3; 640: 60.4 -> 67.4 -> 70.7 (1 vector per
    // thread and ONE workgroup per compute unit keeps too little under way: 136 columns 52.9, 200 columns 68.0).
    bool narrow_backward_pair = false;
    // (float32 / float64 rows that fill a 4-vector shape exactly stay there: N = 256 on 2^20 rows 75.6 against 74.5)
    const bool fills_four = bytes >= 4 && n_vecs <= 128 && (n_vecs & (n_vecs - 1)) == 0;
    if (which == kNormBwd && N >= vec_elems && n_vecs > 16 && n_vecs <= 192 && !fills_four) {
        const bool one_each = ln16 && n_vecs <= 96;
        const int k = one_each ? 1 : 2;
        int tpr = 16;
        while (k * tpr < n_vecs) tpr *= 2;
        const Shape narrow{k, tpr, 512};
        if (shape_compiled(which, aligned, ln16, narrow)) {
            s = narrow;
            narrow_backward_pair = one_each;
        }
    }
    // The norm forward over narrow rows (17 to 128 vectors) whose pitch is not a multiple of 128 bytes: 2 vectors per
    // thread in 256-thread workgroups, two per compute unit, for the same reason (pieces of a wave's request that
    // start and end inside a line).  Forward + backward of 2^26 elements with only the forward's shape changed,
    // 4 x TPR / 256, one per compute unit -> 2 x TPR / 256, two: bfloat16 RMSNorm N = 200: 66.0 -> 68.0; 248:
    // 70.0 -> 73.3; 456: 71.0 -> 72.1; float32 N = 72: 61.7 -> 63.3; 120: 77.7 -> 79.1; 136: 59.8 -> 61.3; rows on
    // 128-byte lines that fill a 4-vector shape lose that way (float32 N = 256: 82.0 -> 80.4; bfloat16 N = 512:
    // 79.1 -> 77.6) and keep theirs.
    bool narrow_forward_pair = false;
    if (which == kNormFwd && N >= vec_elems && n_vecs > 16 && n_vecs <= 128 && pitch_bytes % 128 != 0) {
        int tpr = 8;
        while (2 * tpr < n_vecs) tpr *= 2;
        const Shape narrow{2, tpr, 256};
        if (shape_compiled(which, aligned, ln16, narrow)) {
            s = narrow;
            narrow_forward_pair = true;
        }
    }
    // Rows of 33 to 48 and of 65 to 96 vectors (5 * 2^k elements and their neighbours: hidden sizes 320, 640 in 16-bit
    // storage, 160, 320 in float32) fill 5/8 to 3/4 of the 2- and 4-vector shapes above and 5/6 or more of a 3-vector
    // shape with the same threads per row.  The forward takes 3 x 16 / 3 x 32 in 256 threads, two workgroups per
    // compute unit, in every storage type; the backward 3 x 16 / 3 x 32 in 512 threads for the 16-bit LayerNorm (whose
    // arithmetic the idle lanes cost most), and 3 x 64 for its rows of 129 to 160 vectors.  Forward + backward of 2^26
    // elements with that one launch changed, % of 8 TB/s -- forward: bfloat16 RMSNorm N = 272 68.6 -> 73.8; 320 74.5 ->
    // 76.7; 544 70.9 -> 75.7; 640 74.5 -> 76.8; float32 N = 136 75.5 -> 78.6; 272 75.9 -> 79.7 (LayerNorm 72.9 -> 77.0);
    // 320 78.4 -> 80.9; rows that fill the 4-vector shape to 3/4 gain nothing and lose nothing (N = 384 bfloat16 76.6 ->
    // 77.0, float32 79.9 -> 79.6).  Backward, LayerNorm: float16 N = 272 56.3 -> 64.7; 320 63.0 -> 70.6; 544 58.4 ->
    // 66.4; 640 66.2 -> 71.3; 768 71.1 -> 73.5; 1152 67.6 -> 71.0; 1280 70.1 -> 71.6; bfloat16 N = 320 69.9 -> 71.7; 544
    // 62.5 -> 69.1; 640 69.1 -> 72.1; 1152 71.7 -> 73.7 (rows of 161 to 192 vectors lose a point that way and keep 2 x 128;
    // the RMSNorm backward gains in float16, +1 to +3.6, and loses in bfloat16, -0.5 to -1.5: left as it is; float32
    // backwards lose 0.5 to 6 points).
    const bool fills_three_16 = n_vecs > 32 && n_vecs <= 48, fills_three_32 = n_vecs > 64 && n_vecs <= 96;
    if (which == kNormFwd && N >= vec_elems && (fills_three_16 || fills_three_32)) {
        const Shape three{3, fills_three_16 ? 16 : 32, 256};
        if (shape_compiled(which, aligned, ln16, three)) {
            s = three;
            narrow_forward_pair = true;
        }
    }
    // The softmax family at the same widths: the forward as the norm forward; the backward over 33 to 48 vectors 3 x 16
    // in 256 threads, one workgroup per compute unit (forward + backward of 2^26 elements, % of 8 TB/s, one launch
    // changed: bfloat16 N = 272 54.6 -> 70.0; 320 61.2 -> 77.2; 384 69.5 -> 79.9; float32 N = 160 64.2 -> 80.3; forward:
    // bfloat16 N = 544 71.5 -> 77.5; 640 76.8 -> 80.8; float32 N = 272 73.2 -> 79.8; the backward over 65 to 96 vectors
    // gains nothing).
    if ((which == kSoftmaxFwd || which == kSoftmaxBwd) && N >= vec_elems && (fills_three_16 || fills_three_32)) {
        const Shape three{3, fills_three_16 ? 16 : 32, 256};
        if ((which == kSoftmaxFwd || fills_three_16) && shape_compiled(which, aligned, ln16, three)) {
            s = three;
            narrow_forward_pair = which == kSoftmaxFwd;
        }
    }
    // The softmax family over rows of 4 * t + 1 to 5 * t vectors, t = 32 ... 256 (THN_SM_SHAPES_FIVE): 5 x t vectors, one
    // workgroup per compute unit on the 128-bit path, instead of 3 x 2t with a third to a sixth of the slots idle.
    // Forward, 2^26 elements: bfloat16 N = 1032 52.7 -> 48.3 us, 1152 50.6 -> 47.3, 2056 59.5 -> 49.0, 2304 50.9 -> 47.5,
    // 4104 62.5 -> 48.2, 4608 51.4 -> 48.2, 5120 50.9 -> 48.1; float32 N = 516 99.0 -> 94.0, 2052 115.0 -> 96.3; off the
    // path N = 2050 56.9 -> 53.4, 4098 58.2 -> 51.7, 5001 60.0 -> 53.9.  The backward follows (the same rows per
    // workgroup: forward + backward N = 1032 113.9 -> 106.1 us, 2056 110.8 -> 105.2, 8200 108.6 -> 103.9, 9216 103.6 ->
    // 101.3, float32 516 220.3 -> 203.5, 1025 214.4 -> 201.5, off the path 5001 127.3 -> 111.1) except where it was
    // measured to lose by itself more than the shared rows gain: rows of more than 4.5 * t vectors on the path (N =
    // 1280, 2560, 5120: 0.2-0.7 %), float32 rows from t = 128 (N = 2052 207.7 -> 217.8 us) and rows just above 4 * t
    // vectors off the path (N = 1025 116.6 -> 118.1).
    if ((which == kSoftmaxFwd || which == kSoftmaxBwd) && N >= vec_elems && n_vecs > 128 && n_vecs <= 1280) {
        int t = 32;
        while (5 * t < n_vecs) t *= 2;
        if (n_vecs > 4 * t) {
            const bool bwd_keeps = (aligned && 2 * n_vecs > 9 * t) || (bytes >= 4 && t >= 128) ||
                                   (!aligned && 8 * n_vecs <= 33 * t);
            const Shape five{5, t, 256};
            if ((which == kSoftmaxFwd || !bwd_keeps) && shape_compiled(which, aligned, ln16, five)) s = five;
        }
    }
    // normalize over the same rows (THN_PN_SHAPES_FIVE): the forward 5 x t vectors, t = 32 ... 128, ONE workgroup per
    // compute unit (2^26 elements, forward: bfloat16 N = 1032 51.8 -> 49.4 us, 2056 57.3 -> 49.6, 4104 61.1 -> 48.2, 5120
    // 48.6 -> 47.0; float32 N = 516 101.4 -> 93.7, 2052 114.8 -> 92.8; off the path N = 4098 56.8 -> 49.3, 5001 59.9 ->
    // 52.6); the 16-bit backward 5 x t as well off the path and, from t = 64, for rows just above 4 * t vectors on it
    // (forward + backward: N = 2056 117.5 -> 110.4 us, 4104 123.9 -> 108.8, 8200 106.7 -> 104.6; off the path N = 1025
    // 124.5 -> 119.7, 4098 118.6 -> 109.8, 5001 133.8 -> 113.8; fuller rows on the path and float32 rows lose 1-5 % in the
    // backward that way).  The p-norm by itself keeps its shapes.
    if ((which == kNormalizeBwd || (which == kPnormFwd && (flavour & 4) != 0)) && N >= vec_elems && n_vecs > 128 &&
        n_vecs <= 1280) {
        int t = 32;
        while (5 * t < n_vecs) t *= 2;
        if (n_vecs > 4 * t) {
            const bool just_above = 8 * n_vecs <= 33 * t;
            const bool bwd_takes = bytes == 2 && (!aligned || (just_above && t >= 64));
            const bool fwd_takes = t <= 128 || (bwd_takes && aligned);
            const Shape five{5, t, 256};
            if ((which == kPnormFwd ? fwd_takes : bwd_takes) && shape_compiled(which, aligned, ln16, five)) s = five;
        }
    }
    // The p-norm / normalize family at the same widths: the forward 3 x 16 / 3 x 32 in every storage type (normalize,
    // 2^26 elements, forward: bfloat16 N = 264 59.2 -> 52.9 us, 272 56.5 -> 52.3, 384 49.2 -> 47.0, 520 58.2 -> 53.6;
    // float32 N = 132 115.0 -> 105.6, 160 96.5 -> 92.4, 260 114.7 -> 107.5, 384 95.8 -> 92.9); the 16-bit normalize
    // backward for rows of 33 to 40 and 65 to 80 vectors, where 2 x 32 / 2 x 64 are five eighths full at most (forward
    // + backward with both: N = 264 132.3 -> 120.2 us, 320 107.6 -> 103.5, 520 126.1 -> 116.7, 576 110.0 -> 103.3, 640
    // 107.1 -> 103.4; fuller rows and float32 rows lose 3-10 % in the backward that way).
    if (which == kPnormFwd && N >= vec_elems && (fills_three_16 || fills_three_32)) {
        const Shape three{3, fills_three_16 ? 16 : 32, 256};
        if (shape_compiled(which, aligned, ln16, three)) s = three;
    }
    if (which == kNormalizeBwd && bytes == 2 && N >= vec_elems &&
        ((n_vecs > 32 && n_vecs <= 40) || (n_vecs > 64 && n_vecs <= 80))) {
        const Shape three{3, n_vecs <= 40 ? 16 : 32, 256};
        if (shape_compiled(which, aligned, ln16, three)) s = three;
    }
    if (which == kNormBwd && ln16 && (fills_three_16 || fills_three_32 || (n_vecs > 128 && n_vecs <= 160))) {
        const Shape three{3, fills_three_16 ? 16 : (fills_three_32 ? 32 : 64), 512};
        if (shape_compiled(which, aligned, ln16, three)) {
            s = three;
            narrow_backward_pair = false;
        }
    }
    // The 16-bit LayerNorm forward over rows of 17 to 96 vectors: the shape with the rows per workgroup of its backward
    // (1 x 32, 3 x 16, 1 x 64, 3 x 32 in 512 threads: 16, 32, 8, 16 rows), two workgroups per compute unit, so that a row
    // stays on its XCD.  2 x 16 / 2 x 32 in 256 threads for rows of 17 to 32 / 49 to 64 vectors at every row count
    // (bfloat16, forward + backward, 16384 rows / 2^26 elements: N = 256 17.2 / 110.2 -> 16.3 / 109.1 us, 448 23.9 / 112.1
    // -> 21.6 / 111.4, 512 24.8 / 110.7 -> 22.4 / 110.2); 3 x 16 / 3 x 32 in 512 threads for 33 to 48 / 65 to 96 vectors
    // while x fits three quarters of the eight L2s (24 MiB): 16384 rows, N = 320 22.6 -> 21.5 us, 384 22.5 -> 21.2, 640
    // 29.0 -> 26.3, 768 31.7 -> 28.9; from 32 MiB on they are 0-4 % slower than in 256 threads (2^24 elements: N = 320
    // 39.3 -> 40.7 us, 640 38.0 -> 39.5; 2^26: 115.5 -> 117.9), so larger batches keep those.
    if (which == kNormFwd && bytes == 2 && (flavour & 1) != 0 && n_vecs > 16 && n_vecs <= 96) {
        const bool three = fills_three_16 || fills_three_32;
        const Shape grouped = fills_three_16 ? Shape{3, 16, 512} : fills_three_32 ? Shape{3, 32, 512}
                            : n_vecs <= 32 ? Shape{2, 16, 256} : Shape{2, 32, 256};
        if ((!three || M * N * bytes <= (24ll << 20)) && shape_compiled(which, aligned, ln16, grouped)) {
            s = grouped;
            narrow_forward_pair = true;
        }
    }
    // The softmax and the normalize forward over 16-bit rows of 769 to 1024 vectors off the 128-bit path: 2 x 512 vectors
    // in 512 threads, one workgroup per compute unit, as the norm forward takes them, instead of 4 x 256 in 256 threads,
    // two per compute unit (bfloat16 N = 8191, forward / forward + backward: softmax 58.8 / 115.2 -> 52.8 / 113.0 us,
    // normalize 58.1 / 115.4 -> 51.0 / 110.3; N = 7001 normalize 57.4 / 122.7 -> 52.6 / 119.8; the p-norm by itself, which
    // writes one value per row, keeps 4 x 256: N = 8191 27.5 us against 30.9).
    bool wide_ragged_forward = false;
    if ((which == kSoftmaxFwd || (which == kPnormFwd && (flavour & 4) != 0)) && !aligned && bytes == 2 && s.k == 4 &&
        s.tpr == 256 && s.block == 256) {
        const Shape wide{2, 512, 512};
        if (shape_compiled(which, aligned, ln16, wide)) {
            s = wide;
            wide_ragged_forward = true;
        }
    }
    // The normalize backward over 16-bit rows of 129 to 191 and 257 to 383 vectors (129 to 144 and 257 to 288 on the
    // 128-bit path): 3 x 64 / 3 x 128 vectors, the shape
    // (and the rows per workgroup) of its forward, instead of 2 x 128 / 2 x 256 -- by itself the kernel is as fast either
    // way on the 128-bit path, but a row then stays on one XCD through forward and backward, and off the path the
    // fuller shape is faster by itself as well.  bfloat16, forward + backward of 2^26 elements: N = 1032 117.3 -> 114.1
    // us, 1152 107.6 -> 103.6, 1280 104.2 -> 103.8, 2304 106.5 -> 103.1, 2560 104.1 -> 103.9; off the path N = 1025
    // 135.9 -> 123.5, 1281 120.1 -> 116.0, 2050 122.9 -> 117.2, 2900 112.7 -> 110.7 (float32 rows lose 1 % that way, and
    // rows that fill the 3-vector shape exactly lose as much: N = 3072 102.1 -> 102.9).  On the path only up to 9/8 of
    // the 2-vector shape's threads (N = 1152, 2304): rows of 5/4 (1280, 2560) gain 0.3 % with a backward that follows
    // its forward and lose 1.8 % with one that does not.
    if (which == kNormalizeBwd && bytes == 2 && N >= vec_elems && s.k == 2 && s.block == 256 &&
        (s.tpr == 128 || s.tpr == 256) && (aligned ? 8 * n_vecs <= 9 * s.tpr : 2 * n_vecs < 3 * s.tpr)) {
        const Shape three{3, s.tpr / 2, 256};
        if (shape_compiled(which, aligned, ln16, three)) s = three;
    }
    // The normalize backward over 16-bit rows of 385 to 512 vectors off the 128-bit path: 4 x 128 vectors two rows at a
    // time instead of one row of 2 x 256 per workgroup (bfloat16, 2^26 elements, N = 3583 / 3999 / 4095: backward 81.7 /
    // 81.5 / 83.5 -> 72.3 / 70.7 / 70.1 us; narrower and wider rows off the path, and every row on it, keep 2 vectors).
    if (which == kNormalizeBwd && !aligned && bytes == 2 && N >= vec_elems && s.k == 2 && s.tpr == 256 && s.block == 256) {
        s = Shape{4, 128, 256};
    }
    // The forward over rows of 257 to 351 vectors, and the 16-bit LayerNorm forward over 129 to 160: 3 x 128 / 3 x 64
    // vectors in 512 threads instead of 256, the backward's rows per workgroup (THN_FWD_SHAPES_AS_BACKWARD; the 16-bit
    // LayerNorm forward over 352 to 384 vectors keeps 3 x 128 in 256 threads, two rows at a time like its backward).
    if (which == kNormFwd && N >= vec_elems && s.k == 3 && s.block == 256 &&
        ((s.tpr == 128 && n_vecs <= 351) || (s.tpr == 64 && bytes == 2 && (flavour & 1) != 0 && n_vecs <= 160))) {
        const Shape grouped{3, s.tpr, 512};
        if (shape_compiled(which, aligned, ln16, grouped)) s = grouped;
    }
    // Rows that start off 128-byte lines: two-row workgroups of 256-thread rows cannot put their requests on line
    // boundaries (the two rows differ in phase, line_shift_ok() below), one-row workgroups can.  Backward: as fast
    // otherwise (fp16 8192 x 6000: 54.8 -> 53.1 us; 8192 x 6016: 52.6 / 52.4 us).  Forward (THN_FWD_SHAPES_TWO_ROWS):
    // float32 16384 x 3000 69.5 -> 67.2 us, 65536 x 3000 290 -> 280 us, bf16 16384 x 6008 71.0 -> 69.1 us.
    // Only the 3-vector shape: one row of 2 x 256 vectors per 256-thread workgroup keeps too little under way (bf16
    // 16384 x 4000, forward + backward: 116.6 us that way, 107.8 as two unshifted rows per workgroup; LayerNorm 128.3 /
    // 117.6; float32 16384 x 2000 114.7 / 106.9).
    if ((which == kNormBwd || which == kFusedBwd || which == kNormFwd) && aligned && pitch_bytes % 128 != 0 && s.tpr >= 256 &&
        s.k == 3 && s.block == 2 * s.tpr && s.k * s.tpr - 7 >= n_vecs) {
        // ... and only rows that fill the shape: a one-row 256-thread workgroup is one wave per SIMD, and with a sixth
        // or more of its slots idle the row's arithmetic is no longer covered (bf16 16384 x 4248, 531 vectors, forward
        // RMSNorm / LayerNorm 55.5 / 62.4 us one row at a time, 48.3 / 50.0 two unshifted rows; 4760 columns 58.2 /
        // 63.2 against 55.8 / 58.5; 5336 columns, 667 vectors, the same both ways; float32 16384 x 2204 55.7 / 57.8
        // against 50.3 / 50.8).  The 16-bit LayerNorm backward likewise up to 704 vectors (16384 x 4248 forward +
        // backward 143.8 -> 131.2 us, 4760: 148.0 -> 139.6, 5336: 153.4 -> 149.3; fp16 8192 x 6000, 750 vectors: 86.7
        // one row at a time, 88.7 two); the other backwards are 1-3 % faster one row at a time at every fill.
        const bool too_empty = (which == kNormFwd && n_vecs <= 640) || (which == kNormBwd && ln16 && n_vecs <= 704);
        Shape one_row = s;
        one_row.block = s.tpr;
        if (!too_empty && shape_compiled(which, aligned, ln16, one_row)) s = one_row;
    }
    const Override& ov = g_override[which];
    Shape cand = s;
    if (ov.k.load() > 0) cand.k = ov.k.load();
    if (ov.tpr.load() > 0) cand.tpr = ov.tpr.load();
    if (ov.block.load() > 0) cand.block = ov.block.load();
    else if (cand.block < cand.tpr) cand.block = cand.tpr;
    if (static_cast<int64_t>(cand.k) * cand.tpr >= n_vecs && cand.block >= cand.tpr &&
        shape_compiled(which, aligned, ln16, cand)) {
        s = cand;
    }
    // rows shorter than one vector have a single element-wise instance per kernel
    if (!aligned && N < vec_elems) s = Shape{4, 8, 256};
    if (!shape_compiled(which, aligned, ln16, s)) return THN_E_SHAPE;

    int bpc = occupancy(which, dtype, flavour, aligned, s);
    int cap = ov.bpc.load();
    if (cap <= 0) {
        cap = default_blocks_per_cu(which, flavour, s.block);
        const int narrow = narrow_row_blocks_per_cu(which, n_vecs, bytes == 2 && N % vec_elems != 0 && !wide_ragged_forward);
        if (narrow > cap) cap = narrow;
        // One input stream and fewer than 1024 vectors per workgroup step (3 vectors per thread in 256-thread
        // workgroups: row widths of 5 * 2^k elements and their neighbours): a second workgroup brings the bytes in
        // flight back to where HBM throughput peaks (bf16 N = 1280, LayerNorm / softmax / normalize forward, 2048 to
        // 32768 rows: 2-10 % faster at every row count; N = 5120 softmax 13.5 / 35.4 / 128.4 -> 11.6 / 34.2 / 125.8 us
        // at 2048 / 8192 / 32768 rows).  The exception is the one-row workgroup at a pitch off 128-byte lines (its
        // vectors are shifted onto line boundaries, see line_shift_ok() below), which gains from the second workgroup
        // only up to 32 rows per compute unit and loses beyond (fp16 N = 6000, LayerNorm forward at 2048 / 4096 /
        // 8192 / 16384 / 32768 rows: 10.7 / 17.7 / 36.1 / 68.5 / 135.2 us with one, 9.3 / 16.8 / 36.1 / 70.7 / 145.0
        // with two; softmax and normalize the same way).
        const bool one_stream = which == kNormFwd || which == kSoftmaxFwd || which == kPnormFwd || which == kFusedFwd;
        const bool shifted_one_row = pitch_bytes % 128 != 0 && s.block == s.tpr;
        // (rows off the 128-bit path alike, except under an activation epilogue, whose one shape there has four vectors
        // per thread: bfloat16 N = 1025 RMSNorm / LayerNorm forward 56.2 / 59.5 -> 49.9 / 53.5 us per 2^26 elements, 2049:
        // 56.8 / 69.2 -> 50.8 / 55.0; float32 N = 513 106.1 / 109.4 -> 96.8 / 97.3)
        if (one_stream && (aligned || which != kFusedFwd) && s.block * s.k < 1024 && n_vecs > 16 && cap < 2 &&
            (!shifted_one_row || M <= 32 * static_cast<int64_t>(cus))) {
            cap = 2;
        }
        // (the normalize forward, which takes two workgroups for every 256-thread shape, follows the same exception:
        // fp16 N = 6000 at 16384 / 32768 rows 74.9 / 151.9 us with two, 73.8 / 145.2 with one)
        if (which == kPnormFwd && (flavour & 4) != 0 && aligned && shifted_one_row && n_vecs > 16 && cap == 2 &&
            M > 32 * static_cast<int64_t>(cus)) {
            cap = 1;
        }
        // The norm forward's 4-vector 256-thread workgroups (rows of 1024 / G vectors, G rows at a time) with at most
        // 8 steps each: a second workgroup per compute unit fills the start and the end of so short a kernel (bf16
        // LayerNorm forward, 4096 rows of 2048 / 4096: 7.2 / 12.1 -> 6.4 / 11.9 us; forward + backward of one batch
        // 21.7 / 35.0 -> 21.0 / 33.8 us).  From 16 steps on the forward by itself is 1-3 % slower with two (16384 x 4096:
        // 46.0 -> 46.5 us), although the backward that follows it on the same batch then runs faster by more than that
        // up to 32 steps (16384 x 4096 forward + backward 109.9 -> 109.4 us, 8192 x 4096 60.7 -> 59.2): with anything
        // else between a layer's forward and its backward only the forward's loss would be left, so one it stays.
        if (which == kNormFwd && aligned && s.k == 4 && s.block == 256 && n_vecs > 16 && cap < 2 &&
            M <= 8 * static_cast<int64_t>(s.block / s.tpr) * cus) {
            cap = 2;
        }
        // The norm forward's two-row workgroups (THN_FWD_SHAPES_TWO_ROWS) with few rows: bf16 N = 5120, 2048 / 4096
        // rows 8.9 / 14.6 -> 8.3 / 14.0 us with two per compute unit; the same from 8192 rows on.
        if (which == kNormFwd && aligned && s.k == 3 && s.tpr == 256 && s.block == 512 && cap < 2 &&
            M <= 24 * static_cast<int64_t>(cus)) {
            cap = 2;
        }
        // The 16-bit LayerNorm forward off the 128-bit path in 4-vector 256-thread workgroups: the masks that keep a row's
        // overlapped columns out of its three sums make it the most arithmetic of the forwards, and a second workgroup
        // covers it (bfloat16 N = 1593: 62.9 -> 51.2 us per 2^26 elements; 3193: 56.6 -> 52.5; RMSNorm and float32 rows
        // are as fast or faster with one).
        if (which == kNormFwd && !aligned && bytes == 2 && (flavour & 1) != 0 && s.k == 4 && s.block == 256 && n_vecs > 16 &&
            cap < 2) {
            cap = 2;
        }
        if ((narrow_forward_pair || narrow_backward_pair) && cap < 2) cap = 2;
        if (which == kPnormFwd && s.k == 5) cap = 1;       // 1280 vectors per workgroup step: see THN_PN_SHAPES_FIVE above
    }
    if (cap < bpc) bpc = cap;
    const int rows_per_block = s.block / s.tpr;
    const int64_t row_blocks = (M + rows_per_block - 1) / rows_per_block;
    int64_t grid_max = static_cast<int64_t>(cus) * bpc;
    // The forward over rows of more than 32 KiB (1024-thread workgroups, one per compute unit, all 16 waves in step):
    // up to four times as many workgroups as the chip holds, handed to the compute units by the dispatcher as they
    // come free, as long as each still gets four rows or more (4096 rows of 64 KiB: RMSNorm bf16 96.5 -> 92.5 us,
    // LayerNorm float32 96.7 -> 92.9; 8192 rows: 194.7 -> 184.9 and 193.4 -> 181.5; up to twice as many for the 16-bit
    // LayerNorm, whose workgroups load two parameter rows first: 96.8 -> 95.1 and 191.2 -> 185.2, with four 97.5).
    // With fewer than four rows each the start of a workgroup costs more than the hand-out gains (2048 rows in 1024
    // workgroups: 46.8 -> 49.8 us; 300 rows one each: 7.5 -> 10.2), and below 12 rows per compute unit nothing is
    // gained (2048 rows in 512 workgroups: 46.8 -> 47.0, LayerNorm 47.7 -> 48.5; 3072 rows in 768: 70.9 -> 70.4);
    // narrower rows measured the same or slower this way at any row count, and the backward would pay for it with
    // more partial rows.
    // Rows of 4 x 1024 vectors only: with 3 vectors per thread the larger grids are 1-6 % slower (float32 3584 x 9080
    // 44.9 -> 47.8 us, 3072 x 10240 42.9 -> 44.0, bf16 3584 x 20480 50.4 -> 51.6).  And only grids that are whole
    // rounds of workgroups, or close to four of them: 3200 rows of 64 KiB in 640 workgroups (two and a half rounds)
    // took 73.9 us against 72.4 in 247.
    if (which == kNormFwd && aligned && s.block == 1024 && s.k == 4 && ov.bpc.load() <= 0 && row_blocks >= 12 * grid_max) {
        const int64_t most = (bytes == 2 && (flavour & 1) != 0) ? 2 : 4;
        int64_t f = row_blocks / (4 * grid_max);
        if (f > most) f = most;
        for (; f > 1; --f) {
            const int64_t iters = (row_blocks + grid_max * f - 1) / (grid_max * f);
            const int64_t g = (row_blocks + iters - 1) / iters;
            if (g % grid_max == 0 || 4 * g >= 15 * grid_max) break;
        }
        if (f > 1) grid_max *= f;
    }
    int64_t grid = row_blocks;
    if (grid > grid_max) {
        const int64_t iters = (row_blocks + grid_max - 1) / grid_max;
        grid = (row_blocks + iters - 1) / iters;      // every workgroup gets the same number of rows (+-1)
    }
    // More than one workgroup per compute unit: a grid between whole multiples of the compute units would leave some
    // of them one workgroup more than others (384 workgroups of 3 row blocks on 256 compute units: half of them work
    // twice as long), so it is rounded up to the next multiple, where the row blocks differ by one at most (bf16
    // RMSNorm forward, 9216 x 1024: 7.16 -> 6.91 us; 2304 x 3072: 6.14 -> 5.78).
    if (grid > cus && grid % cus != 0) {
        const int64_t up = (grid + cus - 1) / cus * cus;
        if (up <= grid_max && up <= row_blocks) grid = up;
    }
    // The backward over so few rows that a full grid visits at most two row blocks per workgroup and its float32
    // partial rows are a quarter or more of the bytes of x, dy and dx: half the workgroups write half the partial
    // rows, and the second stage reads half (bf16, forward + backward of one batch, RMSNorm / LayerNorm: 512 x 4096
    // 14.6 / 17.5 -> 13.7 / 15.5 us, 1024 x 4096 LayerNorm 19.6 -> 18.6, 256 x 8192 16.3 / 22.0 -> 14.7 / 18.7,
    // 512 x 16384 25.8 / 32.7 -> 24.7 / 30.8).  With more row blocks per workgroup, or partial rows that are a smaller
    // part, the lost parallelism costs more (2048 x 4096 LayerNorm 23.7 -> 24.3, 1024 x 8192 26.3 -> 27.5, 4096 x 1024
    // 19.4 -> 20.5 us); a quarter of the workgroups measured the same as half or slower.
    if ((which == kNormBwd || which == kFusedBwd) && ov.bpc.load() <= 0 && grid >= cus && row_blocks <= 2 * grid) {
        // (two gradients for LayerNorm whichever of them the caller asks for: the grid decides which rows meet in a
        // partial row, and dW must not depend on whether dB is requested as well)
        const int64_t n_grads = (flavour & 1) != 0 ? 2 : 1;
        if (grid * 4 * n_grads * 4 >= M * bytes * 3) grid = (grid + 1) / 2;
    }
    out->s = s;
    out->grid = static_cast<int>(grid);
    out->n_vecs = n_vecs;
    out->aligned = aligned;
    return THN_OK;
}

// Persistent grid of the flat and the staged kernels: one workgroup per block of rows up to bpc per compute unit, then
// as many as give every workgroup the same number of steps, rounded up to a whole number per compute unit where that
// stays within both limits.
int64_t narrow_row_grid(int64_t M, int64_t rows_per_block, int cus, int bpc) {
    const int64_t row_blocks = (M + rows_per_block - 1) / rows_per_block;
    const int64_t grid_max = static_cast<int64_t>(cus) * bpc;
    int64_t grid = row_blocks;
    if (grid > grid_max) {
        const int64_t iters = (row_blocks + grid_max - 1) / grid_max;
        grid = (row_blocks + iters - 1) / iters;
        if (grid > cus && grid % cus != 0) {
            const int64_t up = (grid + cus - 1) / cus * cus;
            if (up <= grid_max && up <= row_blocks) grid = up;
        }
    }
    return grid;
}

// ---- the flat mapping for narrow rows (thn_flat.h) ------------------------------------------------------------
struct FlatPlan {
    int rows_each;      // J: independent rows per lane and step
    int log_steps;      // tree steps of the segmented row sums: ceil(log2(vectors per row)), at least 4
    int grid;
    int n_vecs;
};

int launch_flat_fwd(int dtype, bool ln, bool aligned, const FlatPlan& p, const FwdArgs& a, hipStream_t st, int* occ) {
    switch (dtype) {
        case THN_F32: return thn::launch_flat_fwd_f32(ln, aligned, p.rows_each, p.log_steps, a, p.grid, st, occ);
        case THN_F16: return thn::launch_flat_fwd_f16(ln, aligned, p.rows_each, p.log_steps, a, p.grid, st, occ);
        case THN_BF16: return thn::launch_flat_fwd_bf16(ln, aligned, p.rows_each, p.log_steps, a, p.grid, st, occ);
        default: return 1;
    }
}

int launch_flat_bwd(int dtype, bool ln, bool aligned, const FlatPlan& p, const BwdArgs& a, hipStream_t st, int* occ) {
    switch (dtype) {
        case THN_F32: return thn::launch_flat_bwd_f32(ln, aligned, p.rows_each, p.log_steps, a, p.grid, st, occ);
        case THN_F16: return thn::launch_flat_bwd_f16(ln, aligned, p.rows_each, p.log_steps, a, p.grid, st, occ);
        case THN_BF16: return thn::launch_flat_bwd_bf16(ln, aligned, p.rows_each, p.log_steps, a, p.grid, st, occ);
        default: return 1;
    }
}

// Whether a plain norm launch takes the flat mapping by itself.  16-bit rows on the 128-bit path of 3 to 21 vectors
// whose vector count is not a power of two, where the segmented row sums (5 to 6 lane exchanges per value, against 3 to
// 5 DPP steps of the row kernels) cost less than the idle lanes and scattered pieces of the row kernels do -- and less
// than the staged kernels' detour through LDS, which wins for float32 rows (half the elements per vector) and is
// within a point for these (bfloat16 RMSNorm N = 72: flat 112.2 us per forward + backward, staged 116.2, row kernels
// 121).  Forward + backward of 2^26 elements, % of 8 TB/s, row kernels -> flat (same box):
//   RMSNorm (one value per row sum), forward and backward, up to 21 vectors: bfloat16 N = 24: 53.0 -> 73.3; 40: 67.9 ->
//     74.7; 72: 69.7 -> 75.2; 88: 72.1 -> 74.3; 120: 73.8 -> 75.7; 136: 69.3 -> 72.3; 168: 71.5 -> 75.4; from 22 vectors
//     on the row kernels are as fast or faster (bfloat16 N = 200: 73.7 against 73.0);
//   LayerNorm (three values per row in the forward and in the backward): the forward up to 7 vectors (forward alone
//     flat, bfloat16 N = 40: 64.9 -> 71.1; 56: 68.9 -> 71.8; rows of 9 and 10 vectors gain a point in one run and lose
//     one in the next, wider ones lose 1-3), the backward only for rows of 3 vectors (bfloat16 N = 24: 48.7 -> 66.1;
//     from 5 vectors on it is 0-6 points slower than the row kernels' backward: three segmented sums per row).
// The launch override selects the flat kernels explicitly with threads_per_row = the row's vector count (not a power
// of two), block_threads = 0 or 256 and vecs_per_thread = rows per lane and step (1, 2 or 4).
bool flat_by_default(int which, bool ln, int bytes, int n_vecs) {
    if (bytes != 2 || (n_vecs & (n_vecs - 1)) == 0) return false;
    if (which == kNormFwd) return ln ? n_vecs <= 7 : n_vecs <= 21;
    return ln ? n_vecs == 3 : n_vecs <= 21;
}

// Rows off the 128-bit path (a width that is not a whole number of vectors, a pointer or pitch off 16 bytes): the row
// kernels' lane groups are no fuller there than on the path, and the staged kernels do not take such rows, so the flat
// kernels serve more widths than on the path, powers of two included.  Forward + backward of 2^26 elements with ONE of
// the two launches changed from the row kernels to the flat ones, % of 8 TB/s (bfloat16 widths N = 8 (L - 1) + 1 or + 5,
// float32 N = 4 (L - 1) + 1 or + 3):
//   RMSNorm forward: bfloat16 L = 2 17.7 -> 23.8; 4 41.6 -> 47.2; 8 67.6 -> 71.3; 15 70.0 -> 72.5; 21 66.7 -> 67.9; from
//     22 vectors on the same or lower; float32 L = 3 41.9 -> 48.4; 8 71.1 -> 77.2; 16 74.4 -> 76.9; 21 72.4 -> 73.1;
//   RMSNorm backward: every width up to 32 vectors (bfloat16 L = 2 17.7 -> 27.2; 5 53.5 -> 60.1; 9 56.3 -> 66.4; 17
//     58.9 -> 65.5; 24 68.1 -> 70.9; float32 L = 2 22.5 -> 41.1; 4 48.0 -> 64.1; 9 59.7 -> 71.7; 32 67.4 -> 76.7);
//   LayerNorm forward: 16-bit rows up to 12 vectors (L = 2 15.6 -> 20.7; 4 36.9 -> 42.1; 8 62.5 -> 64.9; from 13 on 0-4
//     points lower), float32 rows up to 16 (L = 3 38.1 -> 43.1; 8 67.0 -> 72.6; 16 70.4 -> 73.1);
//   LayerNorm backward: 16-bit rows of up to 6, of 9 to 12 and of 17 to 20 vectors (L = 2 15.6 -> 24.9; 5 46.8 -> 51.2;
//     9 50.6 -> 59.1; 17 53.2 -> 56.3; rows of 7, 8 and 13 to 16 vectors fill the row kernels' lane groups and are 1-5
//     points faster there), float32 rows up to 12 (L = 2 19.9 -> 36.7; 4 43.6 -> 58.4; 9 54.2 -> 67.2; 12 64.1 -> 68.1).
// Both launches changed: bfloat16 RMSNorm N = 9 17.7 -> 44.9; 21 36.1 -> 60.3; 69 56.3 -> 70.6; 129 58.9 -> 69.6; LayerNorm
// N = 9 15.6 -> 38.4; 69 50.6 -> 60.1; float32 RMSNorm N = 5 22.5 -> 71.4; 11 41.9 -> 74.2; 35 59.7 -> 75.0; 125 67.4 ->
// 76.9; LayerNorm N = 5 19.9 -> 53.4; 11 38.1 -> 67.4; 35 54.2 -> 70.7 (the statistics of such rows -- 4 or 8 bytes per
// row and pass next to 18 to 40 bytes of row -- are not in the algorithmic bytes).
bool flat_off_path_by_default(int which, bool ln, int bytes, int n_vecs) {
    if (which == kNormFwd) {
        if (!ln) return n_vecs <= 21;
        return bytes == 2 ? n_vecs <= 12 : n_vecs <= 16;
    }
    if (!ln) return true;
    if (bytes == 2) return n_vecs <= 6 || (n_vecs >= 9 && n_vecs <= 12) || (n_vecs >= 17 && n_vecs <= 20);
    return n_vecs <= 12;
}

bool plan_flat(int which, bool ln, bool aligned, int64_t M, int64_t N, int dtype, FlatPlan* out) {
    const int bytes = elem_bytes(dtype);
    if (bytes == 0 || bytes == 8 || M <= 0) return false;
    const int vec_elems = 16 / bytes;
    // off the 128-bit path: rows of at least one vector (unaligned 16-byte windows, the last one overlapping)
    if (aligned ? N % vec_elems != 0 : N < vec_elems) return false;
    const int n_vecs = static_cast<int>((N + vec_elems - 1) / vec_elems);
    if (n_vecs < 2 || n_vecs > thn::kFlatMaxVecs) return false;
    const Override& ov = g_override[which];
    // rows per lane and step, workgroups per compute unit: two and two measured best or within a point of it at every
    // width (1, 2, 4 x 2, 4, 8); the 16-bit LayerNorm forward (the most registers per row) takes one and four
    int rows_each = 2, bpc = 2;
    if (which == kNormFwd && ln && bytes == 2) {
        rows_each = 1;
        bpc = 4;
    }
    // the 16-bit LayerNorm backward off the 128-bit path: four workgroups (2-5 points over two at 9 to 20 vectors)
    if (which == kNormBwd && ln && bytes == 2 && !aligned) bpc = 4;
    if (ov.tpr.load() > 0 || ov.block.load() > 0 || ov.k.load() > 0) {
        // (a row-kernel shape is forced; on the 128-bit path a power of two is one: there the staged kernels take over)
        if (ov.tpr.load() != n_vecs || (aligned && (n_vecs & (n_vecs - 1)) == 0)) return false;
        if (ov.block.load() > 0 && ov.block.load() != thn::kFlatBlock) return false;
        if (ov.k.load() > 0) rows_each = ov.k.load();
        if (rows_each != 1 && rows_each != 2 && (rows_each != 4 || !aligned)) return false;
    } else if (!(aligned ? flat_by_default(which, ln, bytes, n_vecs) : flat_off_path_by_default(which, ln, bytes, n_vecs))) {
        return false;
    }
    const int cus = current_cu_count();
    if (cus <= 0) return false;
    if (ov.bpc.load() > 0) bpc = ov.bpc.load();
    if (bpc > kMaxBlocksPerCu) bpc = kMaxBlocksPerCu;
    const int64_t rows_per_block = static_cast<int64_t>(thn::kFlatBlock / 64) * (64 / n_vecs) * rows_each;
    const int64_t grid = narrow_row_grid(M, rows_per_block, cus, bpc);
    out->rows_each = rows_each;
    out->log_steps = n_vecs <= 16 ? 4 : 5;
    out->grid = static_cast<int>(grid);
    out->n_vecs = n_vecs;
    return true;
}

// ---- the LDS-staged kernels for narrow rows (thn_staged.h) ------------------------------------------------------
struct StagedPlan {
    int passes;         // J: flat passes (vectors per lane) per batch
    int grid;
    int n_vecs;
};

int launch_staged_fwd(int dtype, bool ln, const StagedPlan& p, const FwdArgs& a, hipStream_t st, int* occ) {
    switch (dtype) {
        case THN_F32: return thn::launch_staged_fwd_f32(ln, p.passes, a, p.grid, st, occ);
        case THN_F16: return thn::launch_staged_fwd_f16(ln, p.passes, a, p.grid, st, occ);
        case THN_BF16: return thn::launch_staged_fwd_bf16(ln, p.passes, a, p.grid, st, occ);
        default: return 1;
    }
}

int launch_staged_bwd(int dtype, bool ln, const StagedPlan& p, const BwdArgs& a, hipStream_t st, int* occ) {
    switch (dtype) {
        case THN_F32: return thn::launch_staged_bwd_f32(ln, p.passes, a, p.grid, st, occ);
        case THN_F16: return thn::launch_staged_bwd_f16(ln, p.passes, a, p.grid, st, occ);
        case THN_BF16: return thn::launch_staged_bwd_bf16(ln, p.passes, a, p.grid, st, occ);
        default: return 1;
    }
}

// Upper limit of workgroups per compute unit of the staged kernels (the workspace bound of the backward counts on it).
constexpr int kStagedBlocksPerCu = 4;

// Whether a plain norm launch over rows of `n_vecs` vectors takes the staged kernels by itself: where forward +
// backward of 2^26 elements measured faster than with the row kernels (same box, % of 8 TB/s, row kernels -> staged):
//   rows of 1, 2 and 4 vectors in every storage type, forward and backward: bfloat16 N = 16 RMSNorm / LayerNorm
//     39.3 / 35.1 -> 72.5 / 65.4; N = 32 63.9 / 60.0 -> 75.7 / 72.4; float32 N = 8 44.2 / 39.2 -> 75.3 / 72.8; N = 16
//     69.3 / 65.3 -> 78.0 / 75.8; rows of 8 vectors, the forward only: bfloat16 N = 64 71.7 / 69.4 -> 77.2 / 74.1;
//     float32 N = 32 73.8 / 71.5 -> 79.9 / 77.7 (wider powers of two fill the row kernels' lane groups: N = 128
//     bfloat16 78.1 against 77.4);
//   float32 rows whose vector count is not a power of two, RMSNorm and LayerNorm, forward and backward: RMSNorm N = 36
//     73.9 -> 79.8; 80 76.6 -> 80.6; 100 76.6 -> 80.6; LayerNorm N = 36 70.0 -> 76.1; 68 64.5 -> 74.5; 100 68.7 -> 76.3;
//     124 71.6 -> 78.2;
//   the 16-bit LayerNorm over rows of 9 and of 17 to 19 vectors, which fill less than 0.6 of the row kernels' 16 and 32
//     lanes: 1 to 2 points (bfloat16 N = 72, one direction changed: backward 66.4 -> 67.2, forward 67.7 -> 68.4; N = 144
//     backward 66.3 -> 67.9; rows that fill more of their lane group stay: N = 96 73.6 against 70.7, N = 200 72.8 against
//     70.2).  (The other 16-bit rows whose vector count is not a power of two: the flat mapping above, or the row
//     kernels.)
// The launch override selects the staged kernels explicitly with block_threads = 64 (a batch belongs to one wave),
// threads_per_row = the row's vector count or 0, and vecs_per_thread = flat passes per batch (1 to 4) or 0.
bool staged_by_default(int which, bool ln, int bytes, int n_vecs) {
    if ((n_vecs & (n_vecs - 1)) == 0) return n_vecs <= 4 || (n_vecs == 8 && which == kNormFwd);
    if (bytes >= 4) return true;
    return ln && (n_vecs == 9 || (n_vecs >= 17 && n_vecs <= 19));
}

bool plan_staged(int which, bool ln, bool aligned, int64_t M, int64_t N, int dtype, StagedPlan* out) {
    const int bytes = elem_bytes(dtype);
    if (!aligned || bytes == 0 || bytes == 8 || M <= 0) return false;
    const int vec_elems = 16 / bytes;
    if (N % vec_elems != 0) return false;
    const int n_vecs = static_cast<int>(N / vec_elems);
    if (n_vecs > thn::kStagedMaxVecs) return false;
    const Override& ov = g_override[which];
    // flat passes per batch and workgroups per compute unit, from a sweep over 1 to 4 passes x 1 to 4 workgroups at 26
    // widths: the forward 2 x 2, the backward 4 x 2 (the 16-bit RMSNorm 2 x 2)
    int passes = 2, bpc = 2;
    if (which == kNormBwd && (ln || bytes >= 4)) passes = 4;
    if (ov.tpr.load() > 0 || ov.block.load() > 0 || ov.k.load() > 0) {
        if (ov.block.load() != thn::kStagedGroup) return false;                  // a row-kernel shape is forced
        if (ov.tpr.load() > 0 && ov.tpr.load() != n_vecs) return false;
        if (ov.k.load() > 0) {
            passes = ov.k.load();
            if (!thn::staged_fits(n_vecs, passes)) return false;
        }
    } else if (!staged_by_default(which, ln, bytes, n_vecs)) {
        return false;
    }
    while (passes > 1 && !thn::staged_fits(n_vecs, passes)) --passes;         // (rows of 2 and 3 vectors: a batch is 64 rows at most)
    const int cus = current_cu_count();
    if (cus <= 0) return false;
    if (ov.bpc.load() > 0) bpc = ov.bpc.load();
    if (bpc > kStagedBlocksPerCu) bpc = kStagedBlocksPerCu;
    const int64_t rows_per_block = static_cast<int64_t>(thn::staged_geom(n_vecs, passes).R) * (thn::kStagedBlock / thn::kStagedGroup);
    const int64_t grid = narrow_row_grid(M, rows_per_block, cus, bpc);
    out->passes = passes;
    out->grid = static_cast<int>(grid);
    out->n_vecs = n_vecs;
    return true;
}

// ---- the flat mapping for narrow rows of the softmax and p-norm families (thn_softmax_flat.h, thn_pnorm_flat.h): kernels
// that reduce ONE value per row and round ---------------------------------------------------------------------------
struct OneSumFlatPlan {
    int rows_each, log_steps, grid, n_vecs;
};

int launch_softmax_flat_fwd(int dtype, bool is_log, bool aligned, const OneSumFlatPlan& p, const SoftmaxFwdArgs& a, hipStream_t st) {
    switch (dtype) {
        case THN_F32: return thn::launch_softmax_flat_fwd_f32(is_log, aligned, p.rows_each, p.log_steps, a, p.grid, st);
        case THN_F16: return thn::launch_softmax_flat_fwd_f16(is_log, aligned, p.rows_each, p.log_steps, a, p.grid, st);
        case THN_BF16: return thn::launch_softmax_flat_fwd_bf16(is_log, aligned, p.rows_each, p.log_steps, a, p.grid, st);
        default: return 1;
    }
}

int launch_softmax_flat_bwd(int dtype, bool is_log, bool aligned, const OneSumFlatPlan& p, const SoftmaxBwdArgs& a, hipStream_t st) {
    switch (dtype) {
        case THN_F32: return thn::launch_softmax_flat_bwd_f32(is_log, aligned, p.rows_each, p.log_steps, a, p.grid, st);
        case THN_F16: return thn::launch_softmax_flat_bwd_f16(is_log, aligned, p.rows_each, p.log_steps, a, p.grid, st);
        case THN_BF16: return thn::launch_softmax_flat_bwd_bf16(is_log, aligned, p.rows_each, p.log_steps, a, p.grid, st);
        default: return 1;
    }
}

// Rows of 1, 2 and 4 vectors and rows of up to 32 vectors whose vector count is not a power of two, in float32 /
// float16 / bfloat16 storage on the 128-bit path: where the row kernels' lane groups (8 lanes at least, a power of two)
// stand half empty or worse.  Softmax forward + backward of 2^26 elements, % of 8 TB/s, row kernels -> flat: bfloat16
// N = 8 17.7 -> 82.4; 16 31.0 -> 80.4; 32 53.1 -> 80.5; 72 59.1 -> 78.1; 96 66.9 -> 79.5; 136 52.5 -> 74.5; 192 69.3 ->
// 76.7; float32 N = 4 20.7 -> 82.9; 16 56.1 -> 84.4; 36 59.7 -> 78.9; 68 53.3 -> 77.4; 96 73.0 -> 82.2 (rows of 8, 16
// and 32 vectors fill their lane groups: 79-86 % with the row kernels); normalize p = 2 alike (bfloat16 K = 8 16 -> 80,
// float32 K = 4 17 -> 76).  The launch override reaches the kernels with threads_per_row = the row's vector count and
// vecs_per_thread = rows per lane and step (2; the softmax kernels 4 as well), and keeps them off with any other shape.
bool plan_one_sum_flat(int which, bool aligned, int64_t M, int64_t N, int dtype, OneSumFlatPlan* out) {
    const int bytes = elem_bytes(dtype);
    if ((bytes != 2 && bytes != 4) || M <= 0) return false;
    const int vec_elems = 16 / bytes;
    // off the 128-bit path: rows of at least one vector (unaligned 16-byte windows, the last one overlapping)
    if (aligned ? N % vec_elems != 0 : N < vec_elems) return false;
    const int n_vecs = static_cast<int>((N + vec_elems - 1) / vec_elems);
    // On the 128-bit path rows of 8, 16 and 32 vectors fill the row kernels' lane groups; off it they are taken here too
    // (softmax / normalize p = 2, row kernels -> flat: bfloat16 N = 127 62.4 / 50.0 -> 74.3 / 74.8; 255 70.1 / 59.4 -> 71.3 /
    // 73.7; float32 N = 31 77.8 / 73.3 -> 80.1 / 80.9; 63 66.4 / 59.3 -> 78.6 / 79.0; bfloat16 N = 63 76.9 / 73.1 -> 73.3 / 73.9).
    if (n_vecs > thn::kFlatMaxVecs || ((n_vecs & (n_vecs - 1)) == 0 && n_vecs > 4 && aligned)) return false;
    const Override& ov = g_override[which];
    // two rows per lane and step, two workgroups per compute unit: best or within a point of it over 2, 4 x 1, 2, 4 at 17
    // widths; the softmax forward over rows of 17 vectors and more (three rows per wave or fewer) takes four workgroups
    // (bfloat16 N = 192 72.1 -> 76.7; float32 N = 96 77.0 -> 82.2; the normalize forward is 1-3 points faster with two:
    // float32 N = 68 / 80 / 96 / 116 75.6 / 79.6 / 79.3 / 78.0 with four, 78.5 / 82.1 / 81.7 / 80.7 with two)
    int rows_each = 2, bpc = (which == kSoftmaxFwd && n_vecs >= 17) ? 4 : 2;
    if (ov.tpr.load() > 0 || ov.block.load() > 0 || ov.k.load() > 0) {
        if (ov.tpr.load() != n_vecs) return false;                                // a row-kernel shape is forced
        if (ov.block.load() > 0 && ov.block.load() != thn::kFlatBlock) return false;
        if (ov.k.load() > 0) rows_each = ov.k.load();
        if (rows_each != 2 && (rows_each != 4 || which >= kPnormFwd || !aligned)) return false;
    }
    const int cus = current_cu_count();
    if (cus <= 0) return false;
    if (ov.bpc.load() > 0) bpc = ov.bpc.load();
    if (bpc > kMaxBlocksPerCu) bpc = kMaxBlocksPerCu;
    const int64_t rows_per_block = static_cast<int64_t>(thn::kFlatBlock / 64) * (64 / n_vecs) * rows_each;
    out->rows_each = rows_each;
    out->log_steps = n_vecs == 1 ? 0 : (n_vecs <= 4 ? 2 : (n_vecs <= 16 ? 4 : 5));
    out->grid = static_cast<int>(narrow_row_grid(M, rows_per_block, cus, bpc));
    out->n_vecs = n_vecs;
    return true;
}

// The p-norm / normalize family over the same narrow rows (thn_pnorm_flat.h): the plan is plan_one_sum_flat's (two rows
// per lane and step only); for tensors whose rows are one folded batch and integer p from 1 to 6.
int launch_pnorm_flat_fwd(int dtype, int mode, bool normalize, bool aligned, const OneSumFlatPlan& p, const thn::PnormFwdArgs& a, hipStream_t st) {
    switch (dtype) {
        case THN_F32: return thn::launch_pnorm_flat_fwd_f32(mode, normalize, aligned, p.log_steps, a, p.grid, st);
        case THN_F16: return thn::launch_pnorm_flat_fwd_f16(mode, normalize, aligned, p.log_steps, a, p.grid, st);
        case THN_BF16: return thn::launch_pnorm_flat_fwd_bf16(mode, normalize, aligned, p.log_steps, a, p.grid, st);
        default: return 1;
    }
}
int launch_pnorm_flat_bwd(int dtype, int mode, bool aligned, const OneSumFlatPlan& p, const thn::PnormBwdArgs& a, hipStream_t st) {
    switch (dtype) {
        case THN_F32: return thn::launch_pnorm_flat_bwd_f32(mode, aligned, a, p.grid, st);
        case THN_F16: return thn::launch_pnorm_flat_bwd_f16(mode, aligned, a, p.grid, st);
        case THN_BF16: return thn::launch_pnorm_flat_bwd_bf16(mode, aligned, a, p.grid, st);
        default: return 1;
    }
}
int launch_normalize_flat_bwd(int dtype, int mode, bool aligned, const OneSumFlatPlan& p, const thn::NormalizeBwdArgs& a, hipStream_t st) {
    switch (dtype) {
        case THN_F32: return thn::launch_normalize_flat_bwd_f32(mode, aligned, p.log_steps, a, p.grid, st);
        case THN_F16: return thn::launch_normalize_flat_bwd_f16(mode, aligned, p.log_steps, a, p.grid, st);
        case THN_BF16: return thn::launch_normalize_flat_bwd_bf16(mode, aligned, p.log_steps, a, p.grid, st);
        default: return 1;
    }
}

// ---- rows shorter than one vector: a lane per row (thn_tiny.h) -------------------------------------------------------
// Softmax and p-norm families, float32 / float16 / bfloat16.  Forward + backward of 2^25 elements, % of 8 TB/s, the row
// kernels' element-wise instance -> a lane per row (element accesses), softmax / normalize p = 2: float32 N = 1 2.4 / 2.5
// -> 66.8 / 44.7; 2 4.5 / 4.6 -> 61.1 / 52.5; 3 6.4 / 6.4 -> 50.7 / 46.5; bfloat16 N = 2 1.0 / 1.0 -> 24.0 / 22.9; 4 1.8 /
// 1.8 -> 26.6 / 25.9; 7 3.0 / 2.9 -> 23.5 / 22.5 (torch's own softmax forward moves its bytes at 44-61 % of the peak in
// float32 and 17-28 % in bfloat16 at these widths).
// A launch override with any shape field set keeps the row kernels' element-wise instance (4 x 8 in 256 threads).
bool tiny_rows(int which, int64_t N, int dtype) {
    const int bytes = elem_bytes(dtype);
    const Override& ov = g_override[which];
    if (ov.k.load() > 0 || ov.tpr.load() > 0 || ov.block.load() > 0) return false;
    return (bytes == 2 || bytes == 4) && N < 16 / bytes;
}
// Dense rows behind aligned pointers go through LDS in whole vectors (TinyStage in thn_tiny.h) from two columns on:
// forward + backward of 2^25 elements, % of 8 TB/s, element accesses -> staged, softmax / normalize p = 2: bfloat16
// N = 2 24.0 / 22.9 -> 34.6 / 35.2; 4 26.6 / 25.9 -> 49.6 / 49.1; 7 23.5 / 22.5 -> 48.8 / 47.3; float32 N = 3 50.7 / 46.5 ->
// 64.5 / 57.0; a single float32 column is one dword per lane already and loses that way (66.8 / 44.7 -> 45.8 / 39.3).
bool tiny_staged(int64_t N) { return N >= 2; }
int tiny_grid(int64_t rows, int cus) {
    const int64_t per_block = static_cast<int64_t>(thn::kTinyBlock) * thn::kTinyRows;
    const int64_t blocks = (rows + per_block - 1) / per_block;
    const int64_t cap = static_cast<int64_t>(cus) * 8;
    return static_cast<int>(blocks < cap ? blocks : cap);
}
#define THN_TINY_SWITCH(CALL_F32, CALL_F16, CALL_BF16)  \
    switch (dtype) {                                    \
        case THN_F32: return CALL_F32;                  \
        case THN_F16: return CALL_F16;                  \
        case THN_BF16: return CALL_BF16;                \
        default: return 1;                              \
    }
int launch_softmax_tiny_fwd(int dtype, bool is_log, bool staged, const SoftmaxFwdArgs& a, int grid, hipStream_t st) {
    THN_TINY_SWITCH(thn::launch_softmax_tiny_fwd_f32(is_log, staged, a, grid, st), thn::launch_softmax_tiny_fwd_f16(is_log, staged, a, grid, st),
                    thn::launch_softmax_tiny_fwd_bf16(is_log, staged, a, grid, st))
}
int launch_softmax_tiny_bwd(int dtype, bool is_log, bool staged, const SoftmaxBwdArgs& a, int grid, hipStream_t st) {
    THN_TINY_SWITCH(thn::launch_softmax_tiny_bwd_f32(is_log, staged, a, grid, st), thn::launch_softmax_tiny_bwd_f16(is_log, staged, a, grid, st),
                    thn::launch_softmax_tiny_bwd_bf16(is_log, staged, a, grid, st))
}
int launch_pnorm_tiny_fwd(int dtype, int mode, bool normalize, bool staged, const thn::PnormFwdArgs& a, int grid, hipStream_t st) {
    THN_TINY_SWITCH(thn::launch_pnorm_tiny_fwd_f32(mode, normalize, staged, a, grid, st), thn::launch_pnorm_tiny_fwd_f16(mode, normalize, staged, a, grid, st),
                    thn::launch_pnorm_tiny_fwd_bf16(mode, normalize, staged, a, grid, st))
}
int launch_pnorm_tiny_bwd(int dtype, int mode, bool staged, const thn::PnormBwdArgs& a, int grid, hipStream_t st) {
    THN_TINY_SWITCH(thn::launch_pnorm_tiny_bwd_f32(mode, staged, a, grid, st), thn::launch_pnorm_tiny_bwd_f16(mode, staged, a, grid, st),
                    thn::launch_pnorm_tiny_bwd_bf16(mode, staged, a, grid, st))
}
int launch_normalize_tiny_bwd(int dtype, int mode, bool staged, const thn::NormalizeBwdArgs& a, int grid, hipStream_t st) {
    THN_TINY_SWITCH(thn::launch_normalize_tiny_bwd_f32(mode, staged, a, grid, st), thn::launch_normalize_tiny_bwd_f16(mode, staged, a, grid, st),
                    thn::launch_normalize_tiny_bwd_bf16(mode, staged, a, grid, st))
}
int launch_norm_tiny_fwd(int dtype, bool ln, bool staged, const FwdArgs& a, int grid, hipStream_t st) {
    THN_TINY_SWITCH(thn::launch_norm_tiny_fwd_f32(ln, staged, a, grid, st), thn::launch_norm_tiny_fwd_f16(ln, staged, a, grid, st),
                    thn::launch_norm_tiny_fwd_bf16(ln, staged, a, grid, st))
}
int launch_norm_tiny_bwd(int dtype, bool ln, bool staged, const BwdArgs& a, int grid, hipStream_t st) {
    THN_TINY_SWITCH(thn::launch_norm_tiny_bwd_f32(ln, staged, a, grid, st), thn::launch_norm_tiny_bwd_f16(ln, staged, a, grid, st),
                    thn::launch_norm_tiny_bwd_bf16(ln, staged, a, grid, st))
}
// The norm backward writes one partial row per workgroup: its grid stays within what thn_norm_bwd_workspace_bytes()
// promises for narrow rows (kStagedBlocksPerCu workgroups per compute unit, at most one per row).
int tiny_bwd_grid(int64_t rows, int cus) {
    const int64_t per_block = static_cast<int64_t>(thn::kTinyBlock) * thn::kTinyRows;
    const int64_t blocks = (rows + per_block - 1) / per_block;
    const int64_t cap = static_cast<int64_t>(cus) * kStagedBlocksPerCu;
    return static_cast<int>(blocks < cap ? blocks : cap);
}
#undef THN_TINY_SWITCH

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The bytes a (rows, row_bytes) operand with the given row pitch spans, as a half-open address range, with the
// pitch and the row width kept for the row-level test below (pitch 0: not a plain stack of rows).
struct ByteRange {
    uintptr_t lo, hi;
    int64_t pitch, row_bytes;
};
ByteRange span_of(const void* p, int64_t rows, int64_t pitch_bytes, int64_t row_bytes) {
    const uintptr_t lo = reinterpret_cast<uintptr_t>(p);
    if (p == nullptr || rows <= 0) return ByteRange{lo, lo, 0, 0};
    return ByteRange{lo, lo + static_cast<uintptr_t>((rows - 1) * pitch_bytes + row_bytes), rows > 1 ? pitch_bytes : 0,
                     row_bytes};
}
// Outputs must not overlap inputs: lanes without work re-load and re-store the last row or vector, so an aliased
// call would store rows transformed twice.  Checked on the host, on the addresses alone: the two address ranges
// must be disjoint, except that two stacks of rows with the SAME pitch may interleave (x = buf[:, :n], y = buf[:, n:]
// of one buffer) as long as no row of one touches a row of the other.
bool overlaps(ByteRange a, ByteRange b) {
    if (!(a.lo < b.hi && b.lo < a.hi)) return false;
    if (a.pitch > 0 && a.pitch == b.pitch) {
        const int64_t p = a.pitch;
        const int64_t d = static_cast<int64_t>((b.lo >= a.lo ? b.lo - a.lo : p - (a.lo - b.lo) % p) % p);   // (b - a) mod p
        // a row of b starts d bytes behind a row of a (and p - d bytes in front of the next one)
        return d < a.row_bytes || p - d < b.row_bytes;
    }
    return true;
}
bool overlaps_any(ByteRange out, std::initializer_list<ByteRange> ins) {
    for (const ByteRange& in : ins) {
        if (overlaps(out, in)) return true;
    }
    return false;
}

// Whether a norm launch may shift its vector slots onto 128-byte lines (row_line_shift() in thn_kernels.h): rows
// that start off a line boundary, one row per workgroup at a time, every row a workgroup visits and every stream
// in the same phase of a line, and room for the up to 7 slots the shift pushes off the left end of the row.
struct RowStream {
    const void* base;
    int64_t stride_bytes;
};
bool line_shift_ok(bool aligned, const Shape& s, int grid, int n_vecs, const RowStream* streams, int n_streams) {
    if (!aligned || s.block != s.tpr || s.k * s.tpr - 7 < n_vecs) return false;
    const int64_t stride = streams[0].stride_bytes;
    if (stride % 128 == 0 || (static_cast<int64_t>(grid) * stride) % 128 != 0) return false;
    const uintptr_t phase = reinterpret_cast<uintptr_t>(streams[0].base) & 127u;
    for (int i = 1; i < n_streams; ++i) {
        if ((reinterpret_cast<uintptr_t>(streams[i].base) & 127u) != phase) return false;
        if ((streams[i].stride_bytes - stride) % 128 != 0) return false;
    }
    return true;
}

int64_t partial_pitch(int64_t N) { return (N + 63) / 64 * 64; }


// One float32 partial row per workgroup and gradient.  The backward launches at most
// cus * max(default, override) workgroups and never more than one per row, whatever shape it picks.
int64_t bwd_workspace_bytes(int which, int flavour, int64_t M, int64_t N, int want_dw, int want_db, int x_dtype) {
    const int bytes = elem_bytes(x_dtype);
    if (bytes == 0) return THN_E_DTYPE;
    if (M < 0 || N <= 0) return THN_E_SHAPE;
    if (N * bytes > kMaxRowBytes) return THN_E_FEATURE_DIM;
    const int n_grads = (want_dw ? 1 : 0) + (want_db ? 1 : 0);
    if (n_grads == 0 || M == 0) return 0;
    const int cus = current_cu_count();
    if (cus <= 0) return THN_E_DEVICE;
    int bpc = default_blocks_per_cu(which, flavour, 512);
    const int vec_elems = 16 / bytes;
    const int n_vecs = static_cast<int>((N + vec_elems - 1) / vec_elems);
    const int narrow = narrow_row_blocks_per_cu(which, n_vecs, bytes == 2 && N % vec_elems != 0);
    if (narrow > bpc) bpc = narrow;
    if (bytes == 2 && n_vecs <= 96 && bpc < 2) bpc = 2;      // the LayerNorm backward over narrow 16-bit rows (plan_launch)
    if (which == kNormBwd && n_vecs <= thn::kStagedMaxVecs && bpc < kStagedBlocksPerCu) bpc = kStagedBlocksPerCu;   // the staged kernels
    const int forced = g_override[which].bpc.load();
    if (forced > bpc) bpc = forced;
    if (bpc > kMaxBlocksPerCu) bpc = kMaxBlocksPerCu;
    int64_t parts = static_cast<int64_t>(cus) * bpc;
    if (parts > M) parts = M;
    return n_grads * parts * partial_pitch(N) * static_cast<int64_t>(sizeof(float));
}

bool fusable(int act) { return act == thn::kGelu || act == thn::kGeluTanh || act == thn::kSilu || act == thn::kRelu; }

// thn_norm_fwd (act == kNoAct) and thn_norm_act_fwd.
int norm_forward(const void* x, int64_t x_row_stride, void* y, int64_t y_row_stride, const void* w, const void* b,
                 float* mean, float* rstd, int64_t M, int64_t N, float eps, int act, int x_dtype, int w_dtype,
                 void* stream) {
    // the caller's choice for this call rides on the storage code (THN_X_KEEP / THN_X_STREAM)
    const int policy_flags = x_dtype & kPolicyFlags;
    if (policy_flags == kPolicyFlags) return THN_E_DTYPE;
    x_dtype &= ~kPolicyFlags;
    const bool keep_x = policy_flags != 0 ? policy_flags == THN_X_KEEP : g_cache_policy.load() == THN_CACHE_KEEP_X;
    const int bytes = elem_bytes(x_dtype);
    if (bytes == 0 || ((w != nullptr || b != nullptr) && elem_bytes(w_dtype) == 0)) return THN_E_DTYPE;
    if (M < 0 || N <= 0) return THN_E_SHAPE;
    if (N * bytes > kMaxRowBytes) return THN_E_FEATURE_DIM;
    if (M == 0) return THN_OK;
    if (x == nullptr || y == nullptr || rstd == nullptr) return THN_E_NULL;
    const bool ln = mean != nullptr;
    if (!ln && b != nullptr) return THN_E_SHAPE;          // RMSNorm has no bias (rmsnorm.py:13-22)
    if (x_row_stride < N || y_row_stride < N) return THN_E_SHAPE;
    if (overlaps(span_of(y, M, y_row_stride * bytes, N * bytes), span_of(x, M, x_row_stride * bytes, N * bytes))) {
        return THN_E_SHAPE;
    }

    const int vec_elems = 16 / bytes;
    const bool aligned = (N % vec_elems) == 0 && aligned16(x) && aligned16(y) && aligned16(w) && aligned16(b) &&
                         (x_row_stride * bytes) % 16 == 0 && (y_row_stride * bytes) % 16 == 0;
    Plan p;
    const bool fused = act != thn::kNoAct;
    if (!fused && tiny_rows(kNormFwd, N, x_dtype)) {        // rows shorter than one vector: a lane per row
        const int cus = current_cu_count();
        if (cus <= 0) return THN_E_DEVICE;
        FwdArgs t{};
        t.x = static_cast<const char*>(x);
        t.y = static_cast<char*>(y);
        t.w = w;
        t.b = b;
        t.mean = mean;
        t.rstd = rstd;
        t.x_stride_bytes = x_row_stride * bytes;
        t.y_stride_bytes = y_row_stride * bytes;
        t.M = M;
        t.n_cols = static_cast<int>(N);
        t.w_dtype = w_dtype;
        t.eps = eps;
        t.inv_n = 1.0f / static_cast<float>(N);
        t.keep_x = keep_x ? 1 : 0;
        const bool dense = tiny_staged(N) && aligned16(x) && aligned16(y) && x_row_stride == N && y_row_stride == N;
        const int lrc = launch_norm_tiny_fwd(x_dtype, ln, dense, t, tiny_grid(M, cus), static_cast<hipStream_t>(stream));
        if (lrc > 0) return THN_E_SHAPE;
        return lrc == 0 ? THN_OK : THN_E_LAUNCH;
    }
    StagedPlan sp;
    FlatPlan fp;
    const bool staged = !fused && plan_staged(kNormFwd, ln, aligned, M, N, x_dtype, &sp);
    const bool flat = !fused && !staged && plan_flat(kNormFwd, ln, aligned, M, N, x_dtype, &fp);
    if (staged) {
        p.n_vecs = sp.n_vecs;
        p.grid = sp.grid;
        p.s = Shape{sp.passes, sp.n_vecs, thn::kStagedBlock};
    } else if (flat) {
        p.n_vecs = fp.n_vecs;
        p.grid = fp.grid;
        p.s = Shape{fp.rows_each, fp.n_vecs, thn::kFlatBlock};
    } else {
        const int rc = plan_launch(fused ? kFusedFwd : kNormFwd, fused ? ((ln ? 1 : 0) | (act << 1)) : (ln ? 1 : 0), aligned, M,
                                   N, x_dtype, &p, x_row_stride * bytes);
        if (rc != THN_OK) return rc;
    }

    FwdArgs a{};
    a.x = static_cast<const char*>(x);
    a.y = static_cast<char*>(y);
    a.w = w;
    a.b = b;
    a.mean = mean;
    a.rstd = rstd;
    a.x_stride_bytes = x_row_stride * bytes;
    a.y_stride_bytes = y_row_stride * bytes;
    a.M = M;
    a.n_cols = static_cast<int>(N);
    a.n_vecs = p.n_vecs;
    a.w_dtype = w_dtype;
    a.eps = eps;
    a.inv_n = 1.0f / static_cast<float>(N);
    const RowStream streams[2] = {{x, a.x_stride_bytes}, {y, a.y_stride_bytes}};
    a.line_shift = line_shift_ok(aligned, p.s, p.grid, p.n_vecs, streams, 2) ? 1 : 0;
    a.keep_x = keep_x ? 1 : 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (flat || staged) a.line_shift = 0;
    const int lrc = staged ? launch_staged_fwd(x_dtype, ln, sp, a, st, nullptr)
                  : flat ? launch_flat_fwd(x_dtype, ln, aligned, fp, a, st, nullptr)
                  : fused ? launch_fused_fwd(x_dtype, (ln ? 1 : 0) | (act << 1), aligned, p.s, a, p.grid, st, nullptr)
                          : launch_fwd(x_dtype, ln, aligned, p.s, a, p.grid, st, nullptr);
    if (lrc > 0) return THN_E_SHAPE;
    return lrc == 0 ? THN_OK : THN_E_LAUNCH;
}

// thn_norm_bwd_dx_partials (act == kNoAct, b unused) and the first stage of thn_norm_act_bwd.
int norm_backward_stage1(const void* x, int64_t x_row_stride, const void* dy, int64_t dy_row_stride, void* dx,
                         int64_t dx_row_stride, const void* w, const void* b, const float* mean, const float* rstd,
                         int want_dw, int want_db, void* workspace, int64_t workspace_bytes, int32_t* num_partials,
                         int64_t M, int64_t N, int act, int x_dtype, int w_dtype, void* stream) {
    const int bytes = elem_bytes(x_dtype);
    if (bytes == 0 || (w != nullptr && elem_bytes(w_dtype) == 0)) return THN_E_DTYPE;
    if (M < 0 || N <= 0) return THN_E_SHAPE;
    if (N * bytes > kMaxRowBytes) return THN_E_FEATURE_DIM;
    if (num_partials != nullptr) *num_partials = 0;
    if (M == 0) return THN_OK;
    if (x == nullptr || dy == nullptr || dx == nullptr || rstd == nullptr) return THN_E_NULL;
    if (x_row_stride < N || dy_row_stride < N || dx_row_stride < N) return THN_E_SHAPE;
    if (overlaps_any(span_of(dx, M, dx_row_stride * bytes, N * bytes),
                     {span_of(x, M, x_row_stride * bytes, N * bytes), span_of(dy, M, dy_row_stride * bytes, N * bytes)})) {
        return THN_E_SHAPE;
    }
    const bool ln = mean != nullptr;
    if (!ln) want_db = 0;
    const int n_grads = (want_dw ? 1 : 0) + (want_db ? 1 : 0);
    if (n_grads > 0 && (workspace == nullptr || num_partials == nullptr)) return THN_E_NULL;
    if (n_grads > 0 && !aligned16(workspace)) return THN_E_WORKSPACE;

    const int vec_elems = 16 / bytes;
    const bool fused = act != thn::kNoAct;
    const bool aligned = (N % vec_elems) == 0 && aligned16(x) && aligned16(dy) && aligned16(dx) && aligned16(w) &&
                         (!fused || aligned16(b)) &&
                         (x_row_stride * bytes) % 16 == 0 && (dy_row_stride * bytes) % 16 == 0 &&
                         (dx_row_stride * bytes) % 16 == 0;
    Plan p;
    const int variant = fused ? ((ln ? 1 : 0) | (act << 1)) : (ln ? 1 : 0);
    StagedPlan sp;
    FlatPlan fp;
    const bool tiny = !fused && tiny_rows(kNormBwd, N, x_dtype);      // rows shorter than one vector: a lane per row
    const bool staged = !fused && !tiny && plan_staged(kNormBwd, ln, aligned, M, N, x_dtype, &sp);
    const bool flat = !fused && !tiny && !staged && plan_flat(kNormBwd, ln, aligned, M, N, x_dtype, &fp);
    if (tiny) {
        const int cus = current_cu_count();
        if (cus <= 0) return THN_E_DEVICE;
        p.n_vecs = 1;
        p.grid = tiny_bwd_grid(M, cus);
        p.s = Shape{thn::kTinyRows, 1, thn::kTinyBlock};
    } else if (staged) {
        p.n_vecs = sp.n_vecs;
        p.grid = sp.grid;
        p.s = Shape{sp.passes, sp.n_vecs, thn::kStagedBlock};
    } else if (flat) {
        p.n_vecs = fp.n_vecs;
        p.grid = fp.grid;
        p.s = Shape{fp.rows_each, fp.n_vecs, thn::kFlatBlock};
    } else {
        const int rc = plan_launch(fused ? kFusedBwd : kNormBwd, variant, aligned, M, N, x_dtype, &p, x_row_stride * bytes);
        if (rc != THN_OK) return rc;
    }
    const int64_t pitch = partial_pitch(N);
    const int64_t need = n_grads * static_cast<int64_t>(p.grid) * pitch * static_cast<int64_t>(sizeof(float));
    if (workspace_bytes < need) return THN_E_WORKSPACE;

    BwdArgs a{};
    a.x = static_cast<const char*>(x);
    a.dy = static_cast<const char*>(dy);
    a.dx = static_cast<char*>(dx);
    a.w = w;
    a.b = fused ? b : nullptr;
    a.mean = mean;
    a.rstd = rstd;
    float* ws = static_cast<float*>(workspace);
    a.dw_part = want_dw ? ws : nullptr;
    a.db_part = want_db ? ws + (want_dw ? static_cast<int64_t>(p.grid) * pitch : 0) : nullptr;
    a.x_stride_bytes = x_row_stride * bytes;
    a.dy_stride_bytes = dy_row_stride * bytes;
    a.dx_stride_bytes = dx_row_stride * bytes;
    a.M = M;
    a.part_pitch = pitch;
    a.n_cols = static_cast<int>(N);
    a.n_vecs = p.n_vecs;
    a.w_dtype = w_dtype;
    a.inv_n = 1.0f / static_cast<float>(N);
    const RowStream streams[3] = {{x, a.x_stride_bytes}, {dy, a.dy_stride_bytes}, {dx, a.dx_stride_bytes}};
    a.line_shift = line_shift_ok(aligned, p.s, p.grid, p.n_vecs, streams, 3) ? 1 : 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (flat || staged || tiny) a.line_shift = 0;
    const bool dense = tiny && tiny_staged(N) && aligned16(x) && aligned16(dy) && aligned16(dx) && x_row_stride == N &&
                       dy_row_stride == N && dx_row_stride == N;
    const int lrc = tiny ? launch_norm_tiny_bwd(x_dtype, ln, dense, a, p.grid, st)
                  : staged ? launch_staged_bwd(x_dtype, ln, sp, a, st, nullptr)
                  : flat ? launch_flat_bwd(x_dtype, ln, aligned, fp, a, st, nullptr)
                  : fused ? launch_fused_bwd(x_dtype, variant, aligned, p.s, a, p.grid, st, nullptr)
                          : launch_bwd(x_dtype, ln, aligned, p.s, a, p.grid, st, nullptr);
    if (lrc > 0) return THN_E_SHAPE;
    if (lrc < 0) return THN_E_LAUNCH;
    if (num_partials != nullptr) *num_partials = p.grid;
    return THN_OK;
}

// ---- row p-norm / normalize ---------------------------------------------------------------------------------
struct RowProblem {
    int bytes;
    int64_t rows;
    int p_int;          // p when it is an integer in [1, 6], else 0
    bool engine;        // rows fit the row engine (at most 64 KiB, integer p); otherwise the looping kernels
    bool aligned;
};

// Common argument checks of the four p-norm entry points.  Returns THN_OK with *done = true when there is
// nothing to launch.
int check_row_problem(int64_t B, int64_t M, int64_t K, float p, int dtype, RowProblem* out, bool* done) {
    *done = false;
    out->bytes = elem_bytes(dtype);
    if (out->bytes == 0) return THN_E_DTYPE;
    if (B < 0 || M < 0 || K <= 0) return THN_E_SHAPE;
    if (!(p >= 1.0f && p <= 6.0f)) return THN_E_SHAPE;          // "p must be in [1, 6]" (Ops/norm.py:148)
    out->rows = B * M;
    if (out->rows == 0) {
        *done = true;
        return THN_OK;
    }
    const int pi = static_cast<int>(p);
    out->p_int = static_cast<float>(pi) == p ? pi : 0;
    out->engine = out->p_int != 0 && K * out->bytes <= kMaxRowBytes;
    out->aligned = (K % (16 / out->bytes)) == 0;
    return THN_OK;
}

// One (B, M, K) operand: fills its row map, folds its alignment into *aligned and clears *uniform when its batch
// stride is not M row strides.  Returns false when the strides cannot be addressed.
bool map_rows(const void* base, int64_t batch_stride, int64_t row_stride, int64_t B, int64_t M, int64_t K,
              int bytes, RowMap* map, bool* aligned, bool* uniform) {
    if (batch_stride < 0 || row_stride < 0 || (M > 1 && row_stride < K)) return false;
    if (M == 1) row_stride = batch_stride;            // one row per batch: the rows are the batches
    else if (B > 1 && batch_stride != M * row_stride) *uniform = false;
    map->batch_stride_bytes = batch_stride * bytes;
    map->row_stride_bytes = row_stride * bytes;
    *aligned = *aligned && aligned16(base) && (map->row_stride_bytes % 16) == 0 &&
               (B == 1 || (map->batch_stride_bytes % 16) == 0);
    return true;
}

// The (batch, row) walk of a launch whose row groups advance by rows_per_iter rows per step.
thn::RowWalk make_walk(bool uniform, int64_t M, int64_t rows, int64_t rows_per_iter) {
    thn::RowWalk w;
    w.rows_per_batch = uniform ? rows : M;
    w.step_batch = rows_per_iter / w.rows_per_batch;
    w.step_row = rows_per_iter % w.rows_per_batch;
    return w;
}

// The span of a (B, M, K) operand with non-negative batch and row strides in elements.
ByteRange span_of_bmk(const void* p, int64_t B, int64_t M, int64_t K, int64_t batch_stride, int64_t row_stride, int bytes) {
    const uintptr_t lo = reinterpret_cast<uintptr_t>(p);
    if (p == nullptr || B <= 0 || M <= 0 || batch_stride < 0 || row_stride < 0) return ByteRange{lo, lo, 0, 0};
    return ByteRange{lo, lo + static_cast<uintptr_t>(((B - 1) * batch_stride + (M - 1) * row_stride + K) * bytes), 0, 0};
}

int mode_of(int p_int) { return p_int == 1 ? thn::kP1 : (p_int == 2 ? thn::kP2 : thn::kPInt); }

int loop_grid(int64_t rows) {
    const int64_t cap = static_cast<int64_t>(current_cu_count()) * 8;
    return static_cast<int>(rows < cap ? rows : cap);
}

int pnorm_forward(const void* x, int64_t x_batch_stride, int64_t x_row_stride, void* y, int64_t y_batch_stride,
                  int64_t y_row_stride, void* norms, int64_t B, int64_t M, int64_t K, float p, float eps, int dtype,
                  bool normalize, void* stream) {
    RowProblem rp;
    bool done;
    const int crc = check_row_problem(B, M, K, p, dtype, &rp, &done);
    if (crc != THN_OK) return crc;
    if (!(eps >= 0.0f)) return THN_E_SHAPE;                      // "eps must be non-negative" (Ops/norm.py:149)
    if (done) return THN_OK;
    if (x == nullptr || norms == nullptr || (normalize && y == nullptr)) return THN_E_NULL;
    if (normalize && overlaps(span_of_bmk(y, B, M, K, y_batch_stride, y_row_stride, rp.bytes),
                              span_of_bmk(x, B, M, K, x_batch_stride, x_row_stride, rp.bytes))) {
        return THN_E_SHAPE;
    }
    if (current_cu_count() <= 0) return THN_E_DEVICE;
    PnormFwdArgs a{};
    bool aligned = rp.aligned, uniform = true;
    if (!map_rows(x, x_batch_stride, x_row_stride, B, M, K, rp.bytes, &a.xmap, &aligned, &uniform)) return THN_E_SHAPE;
    if (normalize && !map_rows(y, y_batch_stride, y_row_stride, B, M, K, rp.bytes, &a.ymap, &aligned, &uniform)) {
        return THN_E_SHAPE;
    }
    a.x = static_cast<const char*>(x);
    a.y = static_cast<char*>(y);
    a.norms = norms;
    a.rows = rp.rows;
    a.n_cols64 = K;
    a.n_cols = static_cast<int>(K < INT32_MAX ? K : INT32_MAX);
    a.p_int = rp.p_int;
    a.p = p;
    a.eps = eps;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int lrc;
    OneSumFlatPlan fp;
    if (rp.engine && uniform && tiny_rows(kPnormFwd, K, dtype)) {
        const int64_t row_bytes = K * rp.bytes;
        const bool dense = tiny_staged(K) && aligned16(x) && a.xmap.row_stride_bytes == row_bytes &&
                           (!normalize || (aligned16(y) && a.ymap.row_stride_bytes == row_bytes));
        lrc = launch_pnorm_tiny_fwd(dtype, mode_of(rp.p_int), normalize, dense, a, tiny_grid(rp.rows, current_cu_count()), st);
    } else if (rp.engine && uniform && plan_one_sum_flat(kPnormFwd, aligned, rp.rows, K, dtype, &fp)) {
        a.n_vecs = fp.n_vecs;
        lrc = launch_pnorm_flat_fwd(dtype, mode_of(rp.p_int), normalize, aligned, fp, a, st);
    } else if (rp.engine) {
        const int variant = mode_of(rp.p_int) | (normalize ? 4 : 0);
        Plan plan;
        const int rc = plan_launch(kPnormFwd, variant, aligned, rp.rows, K, dtype, &plan, uniform ? a.xmap.row_stride_bytes : 0);
        if (rc != THN_OK) return rc;
        a.n_vecs = plan.n_vecs;
        a.walk = make_walk(uniform, M, rp.rows, static_cast<int64_t>(plan.grid) * (plan.s.block / plan.s.tpr));
        // rows of one folded batch sit at r * row stride, which is what the shift's phase test assumes
        const RowStream streams[2] = {{x, a.xmap.row_stride_bytes}, {y, a.ymap.row_stride_bytes}};
        a.line_shift = (uniform && line_shift_ok(aligned, plan.s, plan.grid, plan.n_vecs, streams, normalize ? 2 : 1)) ? 1 : 0;
        lrc = launch_pnorm_fwd(dtype, variant, aligned, plan.s, a, plan.grid, st, nullptr);
    } else {
        const int grid = loop_grid(rp.rows);
        a.walk = make_walk(uniform, M, rp.rows, grid);
        switch (dtype) {
            case THN_F32: lrc = thn::launch_pnorm_fwd_loop_f32(normalize, a, grid, st); break;
            case THN_F16: lrc = thn::launch_pnorm_fwd_loop_f16(normalize, a, grid, st); break;
            case THN_BF16: lrc = thn::launch_pnorm_fwd_loop_bf16(normalize, a, grid, st); break;
            default: lrc = thn::launch_pnorm_fwd_loop_f64(normalize, a, grid, st); break;
        }
    }
    if (lrc > 0) return THN_E_SHAPE;
    return lrc == 0 ? THN_OK : THN_E_LAUNCH;
}

// ---- element-wise activations --------------------------------------------------------------------------------
// Workgroups per compute unit of the flat kernels, from sweeps on MI355X: the selections and the backward passes
// that need one or two instructions per element stream best with one workgroup (2.5 % over two); everything with
// an exponential in it wants two to overlap arithmetic and memory; the exact GeLU on 16-bit storage is bound by
// arithmetic (about 30 instruction slots per element) and takes four.
int act_blocks_per_cu(int act, bool bwd, int bytes) {
    const bool gelu = act == thn::kGelu;
    if (gelu && bytes == 2) return 4;
    const bool heavy_bwd = gelu || act == thn::kGeluTanh || act == thn::kMish || (act == thn::kSilu && bytes == 2);
    if (bwd) return heavy_bwd ? 2 : 1;
    return 2;
}

int act_launch(const void* x, int64_t x_row_stride, const void* g, int64_t g_row_stride, void* out,
               int64_t out_row_stride, int64_t M, int64_t N, int act, float p0, float p1, int dtype, bool bwd,
               void* stream) {
    const int bytes = elem_bytes(dtype);
    if (bytes == 0) return THN_E_DTYPE;
    if (M < 0 || N <= 0 || act < 0 || act >= thn::kNumActs) return THN_E_SHAPE;
    if (M == 0) return THN_OK;
    if (x == nullptr || out == nullptr || (bwd && g == nullptr)) return THN_E_NULL;
    if (M > 1 && (x_row_stride < N || out_row_stride < N || (bwd && g_row_stride < N))) return THN_E_SHAPE;
    if (overlaps_any(span_of(out, M, out_row_stride * bytes, N * bytes),
                     {span_of(x, M, x_row_stride * bytes, N * bytes),
                      span_of(bwd ? g : nullptr, M, g_row_stride * bytes, N * bytes)})) {
        return THN_E_SHAPE;
    }
    const int cus = current_cu_count();
    if (cus <= 0) return THN_E_DEVICE;
    const int which = bwd ? kActBwd : kActFwd;
    const int bpc_override = g_override[which].bpc.load();
    ActArgs a{};
    a.x = static_cast<const char*>(x);
    a.g = static_cast<const char*>(g);
    a.out = static_cast<char*>(out);
    a.p0 = p0;
    a.p1 = p1;
    const bool contiguous = M == 1 || (x_row_stride == N && out_row_stride == N && (!bwd || g_row_stride == N));
    const bool flat = contiguous && aligned16(x) && aligned16(out) && (!bwd || aligned16(g));
    dim3 grid;
    if (flat) {
        const int vec_elems = 16 / bytes;
        a.total_elems = M * N;
        a.total_vecs = a.total_elems / vec_elems;
        const int per_block = thn::kActBlock * (bwd ? thn::act_bwd_vecs(act) : thn::kActFwdVecs);
        const int64_t blocks = (a.total_vecs + per_block - 1) / per_block;
        const int64_t cap = static_cast<int64_t>(cus) * (bpc_override > 0 ? bpc_override : act_blocks_per_cu(act, bwd, bytes));
        int64_t n = blocks < cap ? blocks : cap;
        if (n > 1 && n == cap) {
            const int64_t iters = (blocks + cap - 1) / cap;
            n = (blocks + iters - 1) / iters;           // every workgroup takes the same number of steps
        }
        grid = dim3(static_cast<unsigned>(n < 1 ? 1 : n));
    } else {
        a.M = M;
        a.N = N;
        a.x_stride_bytes = x_row_stride * bytes;
        a.g_stride_bytes = g_row_stride * bytes;
        a.out_stride_bytes = out_row_stride * bytes;
        // Threads along a row: one per vector slot, at most the whole workgroup; a thread takes `vecs` rows per step.
        const int vecs = bwd ? thn::kActRowsBwdVecs : thn::kActFwdVecs;
        const int64_t slots = (N + 16 / bytes - 1) / (16 / bytes);
        int lx = 0;
        while (lx < 8 && (int64_t{1} << lx) < slots) ++lx;
        a.lx = lx;
        const int64_t col_blocks = (slots + (int64_t{1} << lx) - 1) >> lx;
        const int64_t rows_per_block = static_cast<int64_t>(thn::kActBlock >> lx) * vecs;
        const int64_t row_blocks = (M + rows_per_block - 1) / rows_per_block;
        const int64_t cap = static_cast<int64_t>(cus) * (bpc_override > 0 ? bpc_override : 4);
        int64_t gy = row_blocks < cap ? row_blocks : cap;
        if (gy > 65535) gy = 65535;
        int64_t gx = (cap + gy - 1) / gy;           // few rows: spread the slots of a row over workgroups too
        if (gx > col_blocks) gx = col_blocks;
        grid = dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy < 1 ? 1 : gy));
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    int lrc;
    switch (dtype) {
        case THN_F32: lrc = thn::launch_act_f32(act, bwd, flat, a, grid, st); break;
        case THN_F16: lrc = thn::launch_act_f16(act, bwd, flat, a, grid, st); break;
        case THN_BF16: lrc = thn::launch_act_bf16(act, bwd, flat, a, grid, st); break;
        default: lrc = thn::launch_act_f64(act, bwd, flat, a, grid, st); break;
    }
    if (lrc > 0) return THN_E_SHAPE;
    return lrc == 0 ? THN_OK : THN_E_LAUNCH;
}

}  // namespace

extern "C" {

int thn_abi_version(void) { return THN_ABI_VERSION; }

const char* thn_strerror(int status) {
    switch (status) {
        case THN_OK: return "ok";
        case THN_E_DTYPE: return "unknown storage type code";
        case THN_E_FEATURE_DIM: return "This layer norm doesn't support feature dim >= 64KB.";
        case THN_E_NULL: return "a required pointer is null";
        case THN_E_SHAPE: return "bad shape, stride or launch shape";
        case THN_E_WORKSPACE: return "workspace is too small";
        case THN_E_LAUNCH: return "the HIP runtime refused the kernel launch";
        case THN_E_DEVICE: return "no usable current HIP device";
        default: return "unknown status";
    }
}

int thn_norm_set_launch_override(int which, int vecs_per_thread, int threads_per_row, int block_threads,
                                 int blocks_per_cu) {
    if (which < 0 || which >= kFamilies) return THN_E_SHAPE;
    if (vecs_per_thread < 0 || threads_per_row < 0 || block_threads < 0 || blocks_per_cu < 0) return THN_E_SHAPE;
    Override& ov = g_override[which];
    ov.k.store(vecs_per_thread);
    ov.tpr.store(threads_per_row);
    ov.block.store(block_threads);
    ov.bpc.store(blocks_per_cu);
    return THN_OK;
}

int thn_norm_set_cache_policy(int policy) {
    if (policy != THN_CACHE_KEEP_X && policy != THN_CACHE_STREAM_X) return THN_E_SHAPE;
    g_cache_policy.store(policy);
    return THN_OK;
}

int thn_norm_get_cache_policy(void) { return g_cache_policy.load(); }

int thn_norm_query_launch(int which, int is_layernorm, int64_t M, int64_t N, int x_dtype, int32_t shape[5]) {
    if (which < 0 || which >= kFamilies || which == kActFwd || which == kActBwd || shape == nullptr) {
        return THN_E_SHAPE;                                     // the element-wise kernels have no row shape
    }
    const int bytes = elem_bytes(x_dtype);
    if (bytes == 0) return THN_E_DTYPE;
    Plan p;
    const bool aligned = N > 0 && (N % (16 / bytes)) == 0;
    int flavour = is_layernorm != 0 ? 1 : 0;
    if (which >= kPnormFwd && which <= kNormalizeBwd) {
        flavour = thn::kP2 | ((which == kPnormFwd && is_layernorm != 0) ? 4 : 0);      // 4: the forward also normalises
    }
    if (which == kFusedFwd || which == kFusedBwd) {
        if (is_layernorm < 0 || !fusable(is_layernorm >> 1)) return THN_E_SHAPE;
        flavour = is_layernorm;                     // bit 0 = LayerNorm, bits 1.. = activation
    }
    if (N > 0 && N * bytes > kMaxRowBytes && which >= kSoftmaxFwd && which <= kNormalizeBwd) {
        // the looping kernels: one workgroup per row
        const int cus = current_cu_count();
        if (cus <= 0) return THN_E_DEVICE;
        if (M < 0) return THN_E_SHAPE;
        int block = thn::kLoopBlock, grid = loop_grid(M);
        if (which == kSoftmaxFwd || which == kSoftmaxBwd) {
            int bpc;
            softmax_loop_launch(which, &block, &bpc);
            const int64_t cap = static_cast<int64_t>(cus) * bpc;
            grid = static_cast<int>(M < cap ? M : cap);
        }
        shape[0] = thn::kWalkVecs;
        shape[1] = block;
        shape[2] = block;
        shape[3] = grid;
        shape[4] = 0;
        return THN_OK;
    }
    if (which <= kNormalizeBwd && tiny_rows(which, N, x_dtype)) {
        const int tiny_cus = current_cu_count();
        if (tiny_cus <= 0) return THN_E_DEVICE;
        shape[0] = thn::kTinyRows;     // a lane per row: rows per lane and step, ONE lane per row
        shape[1] = 1;
        shape[2] = thn::kTinyBlock;
        shape[3] = which == kNormBwd ? tiny_bwd_grid(M, tiny_cus) : tiny_grid(M, tiny_cus);
        shape[4] = 0;
        return THN_OK;
    }
    OneSumFlatPlan sfp;
    if (which >= kSoftmaxFwd && which <= kNormalizeBwd && plan_one_sum_flat(which, aligned, M, N, x_dtype, &sfp)) {
        shape[0] = sfp.rows_each;      // the flat mapping: rows per lane and step, lanes per row = vectors per row
        shape[1] = sfp.n_vecs;
        shape[2] = thn::kFlatBlock;
        shape[3] = sfp.grid;
        shape[4] = aligned ? 1 : 0;
        return THN_OK;
    }
    StagedPlan sp;
    if ((which == kNormFwd || which == kNormBwd) && plan_staged(which, is_layernorm != 0, aligned, M, N, x_dtype, &sp)) {
        shape[0] = sp.passes;          // the staged kernels: flat passes per batch, vectors per row, a batch per wave
        shape[1] = sp.n_vecs;
        shape[2] = thn::kStagedGroup;
        shape[3] = sp.grid;
        shape[4] = 1;
        return THN_OK;
    }
    FlatPlan fp;
    if ((which == kNormFwd || which == kNormBwd) && plan_flat(which, is_layernorm != 0, aligned, M, N, x_dtype, &fp)) {
        shape[0] = fp.rows_each;       // the flat mapping: rows per lane and step, lanes per row = vectors per row
        shape[1] = fp.n_vecs;
        shape[2] = thn::kFlatBlock;
        shape[3] = fp.grid;
        shape[4] = aligned ? 1 : 0;
        return THN_OK;
    }
    const int rc = plan_launch(which, flavour, aligned, M, N, x_dtype, &p, N * elem_bytes(x_dtype));   // contiguous rows
    if (rc != THN_OK) return rc;
    shape[0] = p.s.k;
    shape[1] = p.s.tpr;
    shape[2] = p.s.block;
    shape[3] = p.grid;
    shape[4] = p.aligned ? 1 : 0;
    return THN_OK;
}

int thn_norm_fwd(const void* x, int64_t x_row_stride, void* y, int64_t y_row_stride, const void* w,
                 const void* b, float* mean, float* rstd, int64_t M, int64_t N, float eps, int x_dtype,
                 int w_dtype, void* stream) {
    return norm_forward(x, x_row_stride, y, y_row_stride, w, b, mean, rstd, M, N, eps, thn::kNoAct, x_dtype, w_dtype,
                        stream);
}

int thn_norm_act_fwd(const void* x, int64_t x_row_stride, void* y, int64_t y_row_stride, const void* w,
                     const void* b, float* mean, float* rstd, int64_t M, int64_t N, float eps, int act,
                     int x_dtype, int w_dtype, void* stream) {
    if (!fusable(act)) return THN_E_SHAPE;
    return norm_forward(x, x_row_stride, y, y_row_stride, w, b, mean, rstd, M, N, eps, act, x_dtype, w_dtype, stream);
}

int thn_norm_act_bwd(const void* x, int64_t x_row_stride, const void* dy, int64_t dy_row_stride, void* dx,
                     int64_t dx_row_stride, const void* w, const void* b, const float* mean, const float* rstd,
                     void* dw, void* db, void* workspace, int64_t workspace_bytes, int64_t M, int64_t N, int act,
                     int x_dtype, int w_dtype, void* stream) {
    if (!fusable(act)) return THN_E_SHAPE;
    if ((dw != nullptr || db != nullptr || b != nullptr) && elem_bytes(w_dtype) == 0) return THN_E_DTYPE;
    if (mean == nullptr && (db != nullptr || b != nullptr)) return THN_E_SHAPE;     // RMSNorm has no bias
    int32_t parts = 0;
    const int rc = norm_backward_stage1(x, x_row_stride, dy, dy_row_stride, dx, dx_row_stride, w, b, mean, rstd,
                                        dw != nullptr, db != nullptr, workspace, workspace_bytes, &parts, M, N, act,
                                        x_dtype, w_dtype, stream);
    if (rc != THN_OK || M == 0 || (dw == nullptr && db == nullptr)) return rc;
    return thn_norm_bwd_reduce_partials(workspace, parts, dw, db, N, w_dtype, stream);
}

int64_t thn_norm_bwd_workspace_bytes(int64_t M, int64_t N, int want_dw, int want_db, int x_dtype) {
    return bwd_workspace_bytes(kNormBwd, 0, M, N, want_dw, want_db, x_dtype);
}

int64_t thn_norm_act_bwd_workspace_bytes(int64_t M, int64_t N, int want_dw, int want_db, int act, int x_dtype) {
    if (!fusable(act)) return THN_E_SHAPE;
    return bwd_workspace_bytes(kFusedBwd, act << 1, M, N, want_dw, want_db, x_dtype);
}

int thn_norm_bwd_dx_partials(const void* x, int64_t x_row_stride, const void* dy, int64_t dy_row_stride,
                             void* dx, int64_t dx_row_stride, const void* w, const float* mean,
                             const float* rstd, int want_dw, int want_db, void* workspace,
                             int64_t workspace_bytes, int32_t* num_partials, int64_t M, int64_t N,
                             int x_dtype, int w_dtype, void* stream) {
    return norm_backward_stage1(x, x_row_stride, dy, dy_row_stride, dx, dx_row_stride, w, nullptr, mean, rstd, want_dw,
                                want_db, workspace, workspace_bytes, num_partials, M, N, thn::kNoAct, x_dtype, w_dtype,
                                stream);
}

// Workspace layout: dW partial rows first (when wanted), dB partial rows after them.  A caller that wants
// only dB passes dw == NULL and the dB rows start at the beginning.
int thn_norm_bwd_reduce_partials(const void* workspace, int32_t num_partials, void* dw, void* db, int64_t N,
                                 int w_dtype, void* stream) {
    if (elem_bytes(w_dtype) == 0) return THN_E_DTYPE;
    if (N <= 0 || num_partials < 0) return THN_E_SHAPE;
    if (dw == nullptr && db == nullptr) return THN_OK;
    if (workspace == nullptr && num_partials > 0) return THN_E_NULL;
    const int64_t pitch = partial_pitch(N);
    const float* ws = static_cast<const float*>(workspace);
    thn::ReduceArgs r{};
    int n = 0;
    if (dw != nullptr) {
        r.part[n] = ws;
        r.out[n] = dw;
        ++n;
    }
    if (db != nullptr) {
        r.part[n] = ws + (dw != nullptr ? static_cast<int64_t>(num_partials) * pitch : 0);
        r.out[n] = db;
        ++n;
    }
    r.pitch = pitch;
    r.n_cols = static_cast<int>(N);
    r.n_parts = num_partials;
    r.w_dtype = w_dtype;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    const auto blocks = [&](int cols) { return dim3(static_cast<unsigned>((N + cols - 1) / cols), static_cast<unsigned>(n)); };
    // The row slices -- the order of the additions -- follow from N alone; the column width of a workgroup is free.
    const int slices = thn::reduce_slices(N);
    if (slices == 16) {
        hipLaunchKernelGGL((thn::reduce_partials_kernel<64, 16, 1>), blocks(64), dim3(256), 0, st, r);
    } else if (slices == 32) {
        hipLaunchKernelGGL((thn::reduce_partials_kernel<32, 32, 4>), blocks(32), dim3(256), 0, st, r);
    } else if (N * n >= thn::kReduceMidFromBoth) {
        hipLaunchKernelGGL((thn::reduce_partials_kernel<32, 64, 4>), blocks(32), dim3(512), 0, st, r);
    } else if (num_partials > 512) {
        // narrow rows whose backward ran four workgroups per compute unit: 16 rows per slice, four requested at a time
        // (1024 partial rows of 3 columns: 10.4 -> 5.3 us; the order of the additions is the slices', whatever is in flight)
        hipLaunchKernelGGL((thn::reduce_partials_kernel<16, 64, 4>), blocks(16), dim3(256), 0, st, r);
    } else {
        hipLaunchKernelGGL((thn::reduce_partials_kernel<16, 64, 1>), blocks(16), dim3(256), 0, st, r);
    }
    return hipGetLastError() == hipSuccess ? THN_OK : THN_E_LAUNCH;
}

int thn_norm_bwd(const void* x, int64_t x_row_stride, const void* dy, int64_t dy_row_stride, void* dx,
                 int64_t dx_row_stride, const void* w, const float* mean, const float* rstd, void* dw,
                 void* db, void* workspace, int64_t workspace_bytes, int64_t M, int64_t N, int x_dtype,
                 int w_dtype, void* stream) {
    if ((dw != nullptr || db != nullptr) && elem_bytes(w_dtype) == 0) return THN_E_DTYPE;
    if (mean == nullptr && db != nullptr) return THN_E_SHAPE;     // RMSNorm has no bias gradient
    int32_t parts = 0;
    const int rc = thn_norm_bwd_dx_partials(x, x_row_stride, dy, dy_row_stride, dx, dx_row_stride, w, mean, rstd,
                                            dw != nullptr, db != nullptr, workspace, workspace_bytes, &parts,
                                            M, N, x_dtype, w_dtype, stream);
    if (rc != THN_OK) return rc;
    // M == 0: no partial rows; the reduction then writes zeros, the sum of an empty set of rows.
    return thn_norm_bwd_reduce_partials(workspace, parts, dw, db, N, w_dtype, stream);
}

// ---- The backward for callers that cannot allocate -----------------------------------------------------------
// The partial rows of the two-stage dW / dB sum live in a fixed array in device memory instead of a workspace the
// caller brings.  Every device the library runs on holds its own copy of the array, at its own address, until the
// process ends.  In host code the array's name is only a handle for hipGetSymbolAddress(): the address the
// kernels are given is the one that call returns for the device that is current, looked up once per device.
constexpr int64_t kStaticWorkspaceBytes = THN_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char g_static_workspace[kStaticWorkspaceBytes];

namespace {
std::mutex g_static_ws_mutex;
void* g_static_ws_ptr[kMaxDevices];          // per device: the device address of g_static_workspace, or null
bool g_static_ws_known[kMaxDevices];

// The address of the array on the current device; null (and *status set) when it cannot be had.
void* static_workspace_of_current_device(hipStream_t stream, int* status) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        *status = THN_E_DEVICE;
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_static_ws_mutex);
    if (!g_static_ws_known[dev]) {
        // The lookup is not a stream operation and must not happen while the caller's stream is being captured
        // into a graph: the first call on a device belongs outside a capture.
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
            (void)hipGetLastError();
            capturing = hipStreamCaptureStatusNone;
        }
        if (capturing != hipStreamCaptureStatusNone) {
            *status = THN_E_DEVICE;
            return nullptr;
        }
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_workspace)) != hipSuccess || ptr == nullptr) {
            (void)hipGetLastError();
            *status = THN_E_DEVICE;
            return nullptr;
        }
        g_static_ws_ptr[dev] = ptr;
        g_static_ws_known[dev] = true;
    }
    return g_static_ws_ptr[dev];
}
}  // namespace

extern "C" int thn_norm_bwd_static_workspace(const void* x, int64_t x_row_stride, const void* dy, int64_t dy_row_stride,
                                              void* dx, int64_t dx_row_stride, const void* w, const float* mean,
                                              const float* rstd, void* dw, void* db, int64_t M, int64_t N, int x_dtype,
                                              int w_dtype, void* stream) {
    // bad arguments are reported as thn_norm_bwd() reports them
    const int64_t upper = thn_norm_bwd_workspace_bytes(M, N, dw != nullptr, db != nullptr, x_dtype);
    if (upper < 0) return static_cast<int>(upper);
    void* ws = nullptr;
    if (upper > 0) {
        int status = THN_OK;
        ws = static_workspace_of_current_device(static_cast<hipStream_t>(stream), &status);
        if (ws == nullptr) return status;
    }
    // The first stage compares what its launch really writes -- one partial row per workgroup of the grid it picks,
    // which can be fewer than the upper bound above -- with the size of the array and returns THN_E_WORKSPACE when
    // that does not fit: the caller must then bring a workspace (thn_norm_bwd()).
    // Every partial row the second stage reads is written in full by the first stage of the same call: nothing in
    // the array has to be cleared between calls.
    return thn_norm_bwd(x, x_row_stride, dy, dy_row_stride, dx, dx_row_stride, w, mean, rstd, dw, db, ws,
                        upper > 0 ? kStaticWorkspaceBytes : 0, M, N, x_dtype, w_dtype, stream);
}

// ---- Softmax / Softmin / LogSoftmax -------------------------------------------------------------------------

int thn_softmax_fwd(const void* x, int64_t x_row_stride, void* y, int64_t y_row_stride, int64_t M, int64_t N,
                    int kind, int dtype, void* stream) {
    const int bytes = elem_bytes(dtype);
    if (bytes == 0) return THN_E_DTYPE;
    if (M < 0 || N <= 0 || N > INT32_MAX || kind < THN_SOFTMAX || kind > THN_LOGSOFTMAX) return THN_E_SHAPE;
    if (M == 0) return THN_OK;
    if (x == nullptr || y == nullptr) return THN_E_NULL;
    if (x_row_stride < N || y_row_stride < N) return THN_E_SHAPE;
    if (overlaps(span_of(y, M, y_row_stride * bytes, N * bytes), span_of(x, M, x_row_stride * bytes, N * bytes))) {
        return THN_E_SHAPE;
    }
    if (N * bytes > kMaxRowBytes) {                 // rows the row engine cannot hold in registers
        const int cus = current_cu_count();
        if (cus <= 0) return THN_E_DEVICE;
        SoftmaxFwdArgs a{};
        a.x = static_cast<const char*>(x);
        a.y = static_cast<char*>(y);
        a.x_stride_bytes = x_row_stride * bytes;
        a.y_stride_bytes = y_row_stride * bytes;
        a.M = M;
        a.n_cols = static_cast<int>(N);
        a.sign = kind == THN_SOFTMIN ? -1.0f : 1.0f;
        int block, bpc;
        softmax_loop_launch(kSoftmaxFwd, &block, &bpc);
        const int64_t cap = static_cast<int64_t>(cus) * bpc;
        const int grid = static_cast<int>(M < cap ? M : cap);
        const int lrc = launch_softmax_fwd_loop(dtype, kind == THN_LOGSOFTMAX, block, a, grid, static_cast<hipStream_t>(stream));
        if (lrc > 0) return THN_E_SHAPE;
        return lrc == 0 ? THN_OK : THN_E_LAUNCH;
    }
    const int vec_elems = 16 / bytes;
    const bool aligned = (N % vec_elems) == 0 && aligned16(x) && aligned16(y) && (x_row_stride * bytes) % 16 == 0 &&
                         (y_row_stride * bytes) % 16 == 0;
    const bool is_log = kind == THN_LOGSOFTMAX;
    if (tiny_rows(kSoftmaxFwd, N, dtype)) {
        const int cus = current_cu_count();
        if (cus <= 0) return THN_E_DEVICE;
        SoftmaxFwdArgs a{};
        a.x = static_cast<const char*>(x);
        a.y = static_cast<char*>(y);
        a.x_stride_bytes = x_row_stride * bytes;
        a.y_stride_bytes = y_row_stride * bytes;
        a.M = M;
        a.n_cols = static_cast<int>(N);
        a.sign = kind == THN_SOFTMIN ? -1.0f : 1.0f;
        const bool dense = tiny_staged(N) && aligned16(x) && aligned16(y) && x_row_stride == N && y_row_stride == N;
        const int lrc = launch_softmax_tiny_fwd(dtype, is_log, dense, a, tiny_grid(M, cus), static_cast<hipStream_t>(stream));
        if (lrc > 0) return THN_E_SHAPE;
        return lrc == 0 ? THN_OK : THN_E_LAUNCH;
    }
    OneSumFlatPlan fp;
    if (plan_one_sum_flat(kSoftmaxFwd, aligned, M, N, dtype, &fp)) {
        SoftmaxFwdArgs a{};
        a.x = static_cast<const char*>(x);
        a.y = static_cast<char*>(y);
        a.x_stride_bytes = x_row_stride * bytes;
        a.y_stride_bytes = y_row_stride * bytes;
        a.M = M;
        a.n_cols = static_cast<int>(N);
        a.n_vecs = fp.n_vecs;
        a.sign = kind == THN_SOFTMIN ? -1.0f : 1.0f;
        const int lrc = launch_softmax_flat_fwd(dtype, is_log, aligned, fp, a, static_cast<hipStream_t>(stream));
        if (lrc > 0) return THN_E_SHAPE;
        return lrc == 0 ? THN_OK : THN_E_LAUNCH;
    }
    Plan p;
    const int rc = plan_launch(kSoftmaxFwd, is_log, aligned, M, N, dtype, &p, x_row_stride * elem_bytes(dtype));
    if (rc != THN_OK) return rc;
    SoftmaxFwdArgs a{};
    a.x = static_cast<const char*>(x);
    a.y = static_cast<char*>(y);
    a.x_stride_bytes = x_row_stride * bytes;
    a.y_stride_bytes = y_row_stride * bytes;
    a.M = M;
    a.n_cols = static_cast<int>(N);
    a.n_vecs = p.n_vecs;
    a.sign = kind == THN_SOFTMIN ? -1.0f : 1.0f;
    const RowStream streams[2] = {{x, a.x_stride_bytes}, {y, a.y_stride_bytes}};
    a.line_shift = line_shift_ok(aligned, p.s, p.grid, p.n_vecs, streams, 2) ? 1 : 0;
    const int lrc = launch_softmax_fwd(dtype, is_log, aligned, p.s, a, p.grid, static_cast<hipStream_t>(stream), nullptr);
    if (lrc > 0) return THN_E_SHAPE;
    return lrc == 0 ? THN_OK : THN_E_LAUNCH;
}

int thn_softmax_bwd(const void* y, int64_t y_row_stride, const void* dy, int64_t dy_row_stride, void* dx,
                    int64_t dx_row_stride, int64_t M, int64_t N, int kind, int dtype, void* stream) {
    const int bytes = elem_bytes(dtype);
    if (bytes == 0) return THN_E_DTYPE;
    if (M < 0 || N <= 0 || N > INT32_MAX || kind < THN_SOFTMAX || kind > THN_LOGSOFTMAX) return THN_E_SHAPE;
    if (M == 0) return THN_OK;
    if (y == nullptr || dy == nullptr || dx == nullptr) return THN_E_NULL;
    if (y_row_stride < N || dy_row_stride < N || dx_row_stride < N) return THN_E_SHAPE;
    if (overlaps_any(span_of(dx, M, dx_row_stride * bytes, N * bytes),
                     {span_of(y, M, y_row_stride * bytes, N * bytes), span_of(dy, M, dy_row_stride * bytes, N * bytes)})) {
        return THN_E_SHAPE;
    }
    if (N * bytes > kMaxRowBytes) {
        const int cus = current_cu_count();
        if (cus <= 0) return THN_E_DEVICE;
        SoftmaxBwdArgs a{};
        a.y = static_cast<const char*>(y);
        a.dy = static_cast<const char*>(dy);
        a.dx = static_cast<char*>(dx);
        a.y_stride_bytes = y_row_stride * bytes;
        a.dy_stride_bytes = dy_row_stride * bytes;
        a.dx_stride_bytes = dx_row_stride * bytes;
        a.M = M;
        a.n_cols = static_cast<int>(N);
        a.sign = kind == THN_SOFTMIN ? -1.0f : 1.0f;
        int block, bpc;
        softmax_loop_launch(kSoftmaxBwd, &block, &bpc);
        const int64_t cap = static_cast<int64_t>(cus) * bpc;
        const int grid = static_cast<int>(M < cap ? M : cap);
        const int lrc = launch_softmax_bwd_loop(dtype, kind == THN_LOGSOFTMAX, block, a, grid, static_cast<hipStream_t>(stream));
        if (lrc > 0) return THN_E_SHAPE;
        return lrc == 0 ? THN_OK : THN_E_LAUNCH;
    }
    const int vec_elems = 16 / bytes;
    const bool aligned = (N % vec_elems) == 0 && aligned16(y) && aligned16(dy) && aligned16(dx) &&
                         (y_row_stride * bytes) % 16 == 0 && (dy_row_stride * bytes) % 16 == 0 &&
                         (dx_row_stride * bytes) % 16 == 0;
    const bool is_log = kind == THN_LOGSOFTMAX;
    if (tiny_rows(kSoftmaxBwd, N, dtype)) {
        const int cus = current_cu_count();
        if (cus <= 0) return THN_E_DEVICE;
        SoftmaxBwdArgs a{};
        a.y = static_cast<const char*>(y);
        a.dy = static_cast<const char*>(dy);
        a.dx = static_cast<char*>(dx);
        a.y_stride_bytes = y_row_stride * bytes;
        a.dy_stride_bytes = dy_row_stride * bytes;
        a.dx_stride_bytes = dx_row_stride * bytes;
        a.M = M;
        a.n_cols = static_cast<int>(N);
        a.sign = kind == THN_SOFTMIN ? -1.0f : 1.0f;
        const bool dense = tiny_staged(N) && aligned16(y) && aligned16(dy) && aligned16(dx) && y_row_stride == N && dy_row_stride == N &&
                           dx_row_stride == N;
        const int lrc = launch_softmax_tiny_bwd(dtype, is_log, dense, a, tiny_grid(M, cus), static_cast<hipStream_t>(stream));
        if (lrc > 0) return THN_E_SHAPE;
        return lrc == 0 ? THN_OK : THN_E_LAUNCH;
    }
    OneSumFlatPlan fp;
    if (plan_one_sum_flat(kSoftmaxBwd, aligned, M, N, dtype, &fp)) {
        SoftmaxBwdArgs a{};
        a.y = static_cast<const char*>(y);
        a.dy = static_cast<const char*>(dy);
        a.dx = static_cast<char*>(dx);
        a.y_stride_bytes = y_row_stride * bytes;
        a.dy_stride_bytes = dy_row_stride * bytes;
        a.dx_stride_bytes = dx_row_stride * bytes;
        a.M = M;
        a.n_cols = static_cast<int>(N);
        a.n_vecs = fp.n_vecs;
        a.sign = kind == THN_SOFTMIN ? -1.0f : 1.0f;
        const int lrc = launch_softmax_flat_bwd(dtype, is_log, aligned, fp, a, static_cast<hipStream_t>(stream));
        if (lrc > 0) return THN_E_SHAPE;
        return lrc == 0 ? THN_OK : THN_E_LAUNCH;
    }
    Plan p;
    const int rc = plan_launch(kSoftmaxBwd, is_log, aligned, M, N, dtype, &p);
    if (rc != THN_OK) return rc;
    SoftmaxBwdArgs a{};
    a.y = static_cast<const char*>(y);
    a.dy = static_cast<const char*>(dy);
    a.dx = static_cast<char*>(dx);
    a.y_stride_bytes = y_row_stride * bytes;
    a.dy_stride_bytes = dy_row_stride * bytes;
    a.dx_stride_bytes = dx_row_stride * bytes;
    a.M = M;
    a.n_cols = static_cast<int>(N);
    a.n_vecs = p.n_vecs;
    a.sign = kind == THN_SOFTMIN ? -1.0f : 1.0f;
    const RowStream streams[3] = {{y, a.y_stride_bytes}, {dy, a.dy_stride_bytes}, {dx, a.dx_stride_bytes}};
    a.line_shift = line_shift_ok(aligned, p.s, p.grid, p.n_vecs, streams, 3) ? 1 : 0;
    const int lrc = launch_softmax_bwd(dtype, is_log, aligned, p.s, a, p.grid, static_cast<hipStream_t>(stream), nullptr);
    if (lrc > 0) return THN_E_SHAPE;
    return lrc == 0 ? THN_OK : THN_E_LAUNCH;
}

int thn_pnorm_fwd(const void* x, int64_t x_batch_stride, int64_t x_row_stride, void* norms, int64_t B, int64_t M,
                  int64_t K, float p, float eps, int dtype, void* stream) {
    return pnorm_forward(x, x_batch_stride, x_row_stride, nullptr, 0, 0, norms, B, M, K, p, eps, dtype, false, stream);
}

int thn_normalize_fwd(const void* x, int64_t x_batch_stride, int64_t x_row_stride, void* y, int64_t y_batch_stride,
                      int64_t y_row_stride, void* norms, int64_t B, int64_t M, int64_t K, float p, float eps,
                      int dtype, void* stream) {
    return pnorm_forward(x, x_batch_stride, x_row_stride, y, y_batch_stride, y_row_stride, norms, B, M, K, p, eps,
                         dtype, true, stream);
}

int thn_pnorm_bwd(const void* x, int64_t x_batch_stride, int64_t x_row_stride, const void* norms, const void* dnorms,
                  void* dx, int64_t dx_batch_stride, int64_t dx_row_stride, int64_t B, int64_t M, int64_t K, float p,
                  int dtype, void* stream) {
    RowProblem rp;
    bool done;
    const int crc = check_row_problem(B, M, K, p, dtype, &rp, &done);
    if (crc != THN_OK) return crc;
    if (done) return THN_OK;
    if (x == nullptr || dnorms == nullptr || dx == nullptr || (norms == nullptr && p != 1.0f)) return THN_E_NULL;
    if (overlaps(span_of_bmk(dx, B, M, K, dx_batch_stride, dx_row_stride, rp.bytes),
                 span_of_bmk(x, B, M, K, x_batch_stride, x_row_stride, rp.bytes))) {
        return THN_E_SHAPE;
    }
    if (current_cu_count() <= 0) return THN_E_DEVICE;
    PnormBwdArgs a{};
    bool aligned = rp.aligned, uniform = true;
    if (!map_rows(x, x_batch_stride, x_row_stride, B, M, K, rp.bytes, &a.xmap, &aligned, &uniform)) return THN_E_SHAPE;
    if (!map_rows(dx, dx_batch_stride, dx_row_stride, B, M, K, rp.bytes, &a.dxmap, &aligned, &uniform)) return THN_E_SHAPE;
    a.x = static_cast<const char*>(x);
    a.norms = norms;
    a.g = dnorms;
    a.dx = static_cast<char*>(dx);
    a.rows = rp.rows;
    a.n_cols64 = K;
    a.n_cols = static_cast<int>(K < INT32_MAX ? K : INT32_MAX);
    a.p_int = rp.p_int;
    a.p = p;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int lrc;
    OneSumFlatPlan fp;
    if (rp.engine && uniform && tiny_rows(kPnormBwd, K, dtype)) {
        const int64_t row_bytes = K * rp.bytes;
        const bool dense = tiny_staged(K) && aligned16(x) && aligned16(dx) && a.xmap.row_stride_bytes == row_bytes &&
                           a.dxmap.row_stride_bytes == row_bytes;
        lrc = launch_pnorm_tiny_bwd(dtype, mode_of(rp.p_int), dense, a, tiny_grid(rp.rows, current_cu_count()), st);
    } else if (rp.engine && uniform && plan_one_sum_flat(kPnormBwd, aligned, rp.rows, K, dtype, &fp)) {
        a.n_vecs = fp.n_vecs;
        lrc = launch_pnorm_flat_bwd(dtype, mode_of(rp.p_int), aligned, fp, a, st);
    } else if (rp.engine) {
        const int mode = mode_of(rp.p_int);
        Plan plan;
        const int rc = plan_launch(kPnormBwd, mode, aligned, rp.rows, K, dtype, &plan);
        if (rc != THN_OK) return rc;
        a.n_vecs = plan.n_vecs;
        a.walk = make_walk(uniform, M, rp.rows, static_cast<int64_t>(plan.grid) * (plan.s.block / plan.s.tpr));
        const RowStream streams[2] = {{x, a.xmap.row_stride_bytes}, {dx, a.dxmap.row_stride_bytes}};
        a.line_shift = (uniform && line_shift_ok(aligned, plan.s, plan.grid, plan.n_vecs, streams, 2)) ? 1 : 0;
        lrc = launch_pnorm_bwd(dtype, mode, aligned, plan.s, a, plan.grid, st, nullptr);
    } else {
        const int grid = loop_grid(rp.rows);
        a.walk = make_walk(uniform, M, rp.rows, grid);
        switch (dtype) {
            case THN_F32: lrc = thn::launch_pnorm_bwd_loop_f32(a, grid, st); break;
            case THN_F16: lrc = thn::launch_pnorm_bwd_loop_f16(a, grid, st); break;
            case THN_BF16: lrc = thn::launch_pnorm_bwd_loop_bf16(a, grid, st); break;
            default: lrc = thn::launch_pnorm_bwd_loop_f64(a, grid, st); break;
        }
    }
    if (lrc > 0) return THN_E_SHAPE;
    return lrc == 0 ? THN_OK : THN_E_LAUNCH;
}

int thn_normalize_bwd(const void* x, int64_t x_batch_stride, int64_t x_row_stride, const void* y,
                      int64_t y_batch_stride, int64_t y_row_stride, const void* norms, const void* dy,
                      int64_t dy_batch_stride, int64_t dy_row_stride, void* dx, int64_t dx_batch_stride,
                      int64_t dx_row_stride, int64_t B, int64_t M, int64_t K, float p, int dtype, void* stream) {
    RowProblem rp;
    bool done;
    const int crc = check_row_problem(B, M, K, p, dtype, &rp, &done);
    if (crc != THN_OK) return crc;
    if (done) return THN_OK;
    const bool need_x = p != 2.0f, need_y = p != 1.0f;
    if (norms == nullptr || dy == nullptr || dx == nullptr || (need_x && x == nullptr) || (need_y && y == nullptr)) {
        return THN_E_NULL;
    }
    if (overlaps_any(span_of_bmk(dx, B, M, K, dx_batch_stride, dx_row_stride, rp.bytes),
                     {span_of_bmk(need_x ? x : nullptr, B, M, K, x_batch_stride, x_row_stride, rp.bytes),
                      span_of_bmk(need_y ? y : nullptr, B, M, K, y_batch_stride, y_row_stride, rp.bytes),
                      span_of_bmk(dy, B, M, K, dy_batch_stride, dy_row_stride, rp.bytes)})) {
        return THN_E_SHAPE;
    }
    if (current_cu_count() <= 0) return THN_E_DEVICE;
    NormalizeBwdArgs a{};
    bool aligned = rp.aligned, uniform = true;
    if (need_x && !map_rows(x, x_batch_stride, x_row_stride, B, M, K, rp.bytes, &a.xmap, &aligned, &uniform)) return THN_E_SHAPE;
    if (need_y && !map_rows(y, y_batch_stride, y_row_stride, B, M, K, rp.bytes, &a.ymap, &aligned, &uniform)) return THN_E_SHAPE;
    if (!map_rows(dy, dy_batch_stride, dy_row_stride, B, M, K, rp.bytes, &a.gmap, &aligned, &uniform)) return THN_E_SHAPE;
    if (!map_rows(dx, dx_batch_stride, dx_row_stride, B, M, K, rp.bytes, &a.dxmap, &aligned, &uniform)) return THN_E_SHAPE;
    a.x = static_cast<const char*>(need_x ? x : dy);         // never dereferenced when not needed
    a.y = static_cast<const char*>(need_y ? y : dy);
    if (!need_x) a.xmap = a.gmap;
    if (!need_y) a.ymap = a.gmap;
    a.norms = norms;
    a.g = static_cast<const char*>(dy);
    a.dx = static_cast<char*>(dx);
    a.rows = rp.rows;
    a.n_cols64 = K;
    a.n_cols = static_cast<int>(K < INT32_MAX ? K : INT32_MAX);
    a.p_int = rp.p_int;
    a.p = p;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int lrc;
    OneSumFlatPlan fp;
    if (rp.engine && uniform && tiny_rows(kNormalizeBwd, K, dtype)) {
        const int64_t row_bytes = K * rp.bytes;
        const bool dense = tiny_staged(K) && (!need_x || (aligned16(x) && a.xmap.row_stride_bytes == row_bytes)) &&
                           (!need_y || (aligned16(y) && a.ymap.row_stride_bytes == row_bytes)) && aligned16(dy) &&
                           a.gmap.row_stride_bytes == row_bytes && aligned16(dx) && a.dxmap.row_stride_bytes == row_bytes;
        lrc = launch_normalize_tiny_bwd(dtype, mode_of(rp.p_int), dense, a, tiny_grid(rp.rows, current_cu_count()), st);
    } else if (rp.engine && uniform && plan_one_sum_flat(kNormalizeBwd, aligned, rp.rows, K, dtype, &fp)) {
        a.n_vecs = fp.n_vecs;
        lrc = launch_normalize_flat_bwd(dtype, mode_of(rp.p_int), aligned, fp, a, st);
    } else if (rp.engine) {
        const int mode = mode_of(rp.p_int);
        Plan plan;
        const int rc = plan_launch(kNormalizeBwd, mode, aligned, rp.rows, K, dtype, &plan);
        if (rc != THN_OK) return rc;
        a.n_vecs = plan.n_vecs;
        a.walk = make_walk(uniform, M, rp.rows, static_cast<int64_t>(plan.grid) * (plan.s.block / plan.s.tpr));
        // (a stream that is not read carries the map of dy: it agrees with dy by construction)
        const RowStream streams[4] = {{a.g, a.gmap.row_stride_bytes}, {a.dx, a.dxmap.row_stride_bytes},
                                      {a.x, a.xmap.row_stride_bytes}, {a.y, a.ymap.row_stride_bytes}};
        a.line_shift = (uniform && line_shift_ok(aligned, plan.s, plan.grid, plan.n_vecs, streams, 4)) ? 1 : 0;
        lrc = launch_normalize_bwd(dtype, mode, aligned, plan.s, a, plan.grid, st, nullptr);
    } else {
        const int grid = loop_grid(rp.rows);
        a.walk = make_walk(uniform, M, rp.rows, grid);
        switch (dtype) {
            case THN_F32: lrc = thn::launch_normalize_bwd_loop_f32(a, grid, st); break;
            case THN_F16: lrc = thn::launch_normalize_bwd_loop_f16(a, grid, st); break;
            case THN_BF16: lrc = thn::launch_normalize_bwd_loop_bf16(a, grid, st); break;
            default: lrc = thn::launch_normalize_bwd_loop_f64(a, grid, st); break;
        }
    }
    if (lrc > 0) return THN_E_SHAPE;
    return lrc == 0 ? THN_OK : THN_E_LAUNCH;
}

int thn_act_fwd(const void* x, int64_t x_row_stride, void* y, int64_t y_row_stride, int64_t M, int64_t N, int act,
                float param0, float param1, int dtype, void* stream) {
    return act_launch(x, x_row_stride, nullptr, 0, y, y_row_stride, M, N, act, param0, param1, dtype, false, stream);
}

int thn_act_bwd(const void* saved, int64_t saved_row_stride, const void* dy, int64_t dy_row_stride, void* dx,
                int64_t dx_row_stride, int64_t M, int64_t N, int act, float param0, float param1, int dtype,
                void* stream) {
    return act_launch(saved, saved_row_stride, dy, dy_row_stride, dx, dx_row_stride, M, N, act, param0, param1, dtype,
                      true, stream);
}

int thn_dropout(const void* x, void* out, int64_t n, int64_t first_offset, float p, uint64_t seed, int dtype,
                void* stream) {
    const int bytes = elem_bytes(dtype);
    if (bytes == 0) return THN_E_DTYPE;
    if (n < 0 || first_offset < 0 || !(p >= 0.0f && p <= 1.0f)) return THN_E_SHAPE;
    if (n == 0) return THN_OK;
    if (x == nullptr || out == nullptr) return THN_E_NULL;
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) % static_cast<uintptr_t>(bytes) != 0) {
        return THN_E_SHAPE;
    }
    const int cus = current_cu_count();
    if (cus <= 0) return THN_E_DEVICE;
    thn::DropoutArgs a{};
    a.x = static_cast<const char*>(x);
    a.out = static_cast<char*>(out);
    a.total_elems = n;
    a.total_vecs = n / (16 / bytes);
    a.first_offset = first_offset;
    a.p = p;
    a.key_lo = static_cast<uint32_t>(seed);
    a.key_hi = static_cast<uint32_t>(seed >> 32);
    // Bound by integer arithmetic: as many waves as a compute unit holds (8 workgroups of 256 threads).
    const int64_t blocks = (a.total_vecs + thn::kDropoutBlock - 1) / thn::kDropoutBlock;
    const int64_t cap = static_cast<int64_t>(cus) * 8;
    const int grid = static_cast<int>(blocks < 1 ? 1 : (blocks < cap ? blocks : cap));
    const int rc = thn::launch_dropout(dtype, a, grid, static_cast<hipStream_t>(stream));
    if (rc > 0) return THN_E_DTYPE;
    return rc == 0 ? THN_OK : THN_E_LAUNCH;
}

}  // extern "C"
