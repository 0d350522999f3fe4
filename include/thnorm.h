/*
 * thnorm.h -- C ABI of libthnorm.so: LayerNorm / RMSNorm, the row reductions next to them (Softmax / Softmin /
 * LogSoftmax, row p-norm / normalize) and the element-wise activations, forward and backward, for AMD MI355X
 * (gfx950).
 *
 * The reference library (TritonHub) has no native boundary: its last host frames before device code are the
 * Python launch sites in TritonHub/Normalization/layernorm.py and rmsnorm.py (and TritonHub/Activations/
 * softmax.py, softmin.py, logsoftmax.py, TritonHub/Ops/norm.py, normalize.py).  Each entry point below
 * replaces one of those launch sites, so a maintainer of the reference can bind it with ctypes in place of
 * the Triton launch.  The citation on every declaration names the launch site (and device code) replaced.
 *
 * Conventions
 *   - Every pointer is a device pointer owned by the caller.  The library allocates nothing, frees nothing,
 *     keeps no pointer after the call returns and never synchronises: kernels are enqueued on `stream`
 *     (a hipStream_t passed as void*; NULL is the default stream) of the CURRENT device.
 *   - Matrices are row-major (M rows, N columns), unit column stride; row strides are in ELEMENTS.
 *   - Storage codes: THN_F32 / THN_F16 / THN_BF16 / THN_F64.  The norm arithmetic is float32 whatever the storage
 *     (a float64 tensor is narrowed on load and widened on store, as the reference does with
 *     `.to(tl.float32)`, layernorm.py:31).  Results are rounded to nearest even on store.
 *   - Return value: THN_OK (0) or a negative THN_E_* code; thn_strerror() names it.  Nothing throws.
 *   - Outputs must not overlap inputs (nor each other), except where an entry point says that it works in place
 *     (thn_dropout).  A call whose output tensor (y, dx) overlaps the address range of one of its input tensors
 *     returns THN_E_SHAPE and launches nothing.  The row kernels keep their loops free of branches by letting a lane without work
 *     re-load, recompute and re-store the last row or the last vector of its row; with y == x or dx == dy such a
 *     lane can read a row that another workgroup has already overwritten and store it transformed twice.  (The
 *     reference's Triton kernels load a whole row before they store it and tolerate in-place use; callers that
 *     relied on that must pass a separate output here.)
 *   - Thread safe.  Process state: a per-device cache of the compute-unit count, of kernel occupancies and of the
 *     address of the static workspace (thn_norm_bwd_static_workspace), filled on first use; the launch-shape
 *     override of thn_norm_set_launch_override(), a process-wide tuning switch that is off unless a caller sets it;
 *     and the default cache policy of thn_norm_set_cache_policy().
 */
#ifndef THNORM_H_
#define THNORM_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define THN_ABI_VERSION 7

enum thn_dtype { THN_F32 = 0, THN_F16 = 1, THN_BF16 = 2, THN_F64 = 3 };

enum thn_status {
    THN_OK = 0,
    THN_E_DTYPE = -1,         /* unknown storage code */
    THN_E_FEATURE_DIM = -2,   /* a row is wider than 64 KiB (the reference's RuntimeError, layernorm.py:71-72) */
    THN_E_NULL = -3,          /* a required pointer is NULL */
    THN_E_SHAPE = -4,         /* M < 0, N <= 0, a row stride smaller than N, or an output that overlaps an input */
    THN_E_WORKSPACE = -5,     /* workspace smaller than thn_norm_bwd_workspace_bytes() asks for, or not 16-byte aligned */
    THN_E_LAUNCH = -6,        /* the HIP runtime refused the launch (hipGetLastError) */
    THN_E_DEVICE = -7         /* no usable current device */
};

/* Version of this ABI (THN_ABI_VERSION of the library that was loaded). */
int thn_abi_version(void);

/* Static description of a status code. */
const char* thn_strerror(int status);

/*
 * Forward: y = normalise(x) [* w] [+ b]; writes the float32 row statistics the backward needs.
 * Replaces `_layernorm_kernel_fwd[(M,)](...)` (layernorm.py:74-86, device code :27-46) when `mean` is not
 * NULL, and `_rmsnorm_kernel_fwd[(M,)](...)` (rmsnorm.py:60-69, device code :24-38) when `mean` is NULL.
 *   LayerNorm: mean = sum(x)/N, rstd = 1/sqrt(sum((x-mean)^2)/N + eps), y = (x-mean)*rstd*w + b
 *   RMSNorm:   rstd = 1/sqrt(sum(x^2)/N + eps),                         y = x*rstd*w        (b must be NULL)
 * w and b may each be NULL (HAS_WEIGHT / HAS_BIAS false in the reference); both use storage `w_dtype`.
 * x and y use storage `x_dtype`.  mean, rstd: (M,) float32.  M == 0 is a no-op.
 * A row's results depend on that row alone and are run-to-run identical.  They do not depend on where the row
 * sits in the tensor when rows are a multiple of 128 bytes apart; at other pitches the order of the row sums
 * (hence the last bit of the results) can depend on the offset of the row's first byte within a 128-byte line,
 * and on nothing else.  The same holds for thn_norm_bwd.
 */
int thn_norm_fwd(const void* x, int64_t x_row_stride,
                 void* y, int64_t y_row_stride,
                 const void* w, const void* b,
                 float* mean, float* rstd,
                 int64_t M, int64_t N, float eps,
                 int x_dtype, int w_dtype, void* stream);

/*
 * Cache policy of the forward's read of x (no counterpart in the reference; Triton chooses for it).  x is the one
 * tensor of a norm step that is read twice: by the forward, and again by the backward, which rebuilds xhat from it.
 *   THN_CACHE_KEEP_X    the forward loads x with ordinary loads, which leave it in the L2 and in the 256 MB
 *                       memory-side cache: a backward that follows its forward closely finds part of x there
 *                       (bfloat16 16384 x 4096: the backward kernel takes 57 us instead of 65); the forward itself is
 *                       2-3 % slower than with streaming loads.  For forward + backward of one batch back to back.
 *   THN_CACHE_STREAM_X  streaming (non-temporal) loads, like every other access of the step.  For inference, and for
 *                       training steps in which so much other work runs between a layer's forward and its backward
 *                       that nothing of x would be left in any cache.
 * Results are bit-identical under both.  thn_norm_set_cache_policy() sets the process-wide default (initially
 * THN_CACHE_KEEP_X) that thn_norm_fwd() and thn_norm_act_fwd() follow; one call can choose for itself by or-ing
 * THN_X_KEEP or THN_X_STREAM into its `x_dtype` argument (THN_BF16 | THN_X_STREAM), which overrides the default for
 * that call and touches no shared state.  The flags are accepted by these two entry points only.
 */
enum thn_cache_policy { THN_CACHE_KEEP_X = 0, THN_CACHE_STREAM_X = 1 };
#define THN_X_KEEP 0x100
#define THN_X_STREAM 0x200
int thn_norm_set_cache_policy(int policy);      /* THN_E_SHAPE for an unknown policy */
int thn_norm_get_cache_policy(void);

/*
 * Bytes of scratch thn_norm_bwd() needs for its per-workgroup partial sums of dW / dB: the counterpart of
 * the reference's `_dw` / `_db` (sm_count, N) float32 buffers (layernorm.py:183-184, rmsnorm.py:147).
 * One partial row per workgroup the backward can launch: depends on the current device's compute-unit count and
 * on the blocks_per_cu override in force (thn_norm_set_launch_override; raising it after this query makes the
 * backward return THN_E_WORKSPACE).  Returns a negative THN_E_* code on bad arguments, 0 when neither gradient is
 * requested.
 */
int64_t thn_norm_bwd_workspace_bytes(int64_t M, int64_t N, int want_dw, int want_db, int x_dtype);

/*
 * Backward: dx for every row, and dW / dB summed over rows, from the SAVED statistics.
 * Replaces `_layernorm_kernel_bwd[(sm_count,)](...)` plus `_dw.sum(0).to(weight.dtype)` /
 * `_db.sum(0).to(bias.dtype)` (layernorm.py:188-208, device code :113-153) when `mean` is not NULL, and
 * `_rmsnorm_kernel_bwd[(sm_count,)](...)` plus `_dw.sum(0)` (rmsnorm.py:150-166, device code :92-122) when
 * `mean` is NULL.
 *   xhat = (x-mean)*rstd (x*rstd for RMSNorm); wdy = w*dy (dy when w is NULL);
 *   c1 = sum(xhat*wdy)/N; c2 = sum(wdy)/N (0 for RMSNorm); dx = (wdy - (xhat*c1 + c2))*rstd;
 *   dW = sum over rows of dy*xhat; dB = sum over rows of dy.
 * dw / db (storage `w_dtype`, (N,)) may each be NULL when that gradient is not wanted; `workspace` may be
 * NULL only when both are and must be 16-byte aligned otherwise (the partial rows are written 16 bytes at a
 * time).  The two-stage sum has a fixed order: results are run-to-run identical.
 */
int thn_norm_bwd(const void* x, int64_t x_row_stride,
                 const void* dy, int64_t dy_row_stride,
                 void* dx, int64_t dx_row_stride,
                 const void* w,
                 const float* mean, const float* rstd,
                 void* dw, void* db,
                 void* workspace, int64_t workspace_bytes,
                 int64_t M, int64_t N,
                 int x_dtype, int w_dtype, void* stream);

/*
 * The two stages of thn_norm_bwd() as separate launches, for callers that time or schedule them apart.
 * Stage 1 replaces the persistent backward kernel alone (layernorm.py:188-206, rmsnorm.py:150-165): it
 * writes dx and `*num_partials` rows of float32 partial sums into `workspace` (dW partials first, then dB
 * partials, each (num_partials, N)).  Stage 2 replaces `_dw.sum(0).to(weight.dtype)` / `_db.sum(0)...`
 * (layernorm.py:207-208, rmsnorm.py:166): it sums the partial rows in a fixed order, in float64, and rounds
 * once to `w_dtype`.  `want_dw` / `want_db` say which partials stage 1 must produce.
 */
int thn_norm_bwd_dx_partials(const void* x, int64_t x_row_stride,
                             const void* dy, int64_t dy_row_stride,
                             void* dx, int64_t dx_row_stride,
                             const void* w,
                             const float* mean, const float* rstd,
                             int want_dw, int want_db,
                             void* workspace, int64_t workspace_bytes, int32_t* num_partials,
                             int64_t M, int64_t N,
                             int x_dtype, int w_dtype, void* stream);

int thn_norm_bwd_reduce_partials(const void* workspace, int32_t num_partials,
                                 void* dw, void* db,
                                 int64_t N, int w_dtype, void* stream);

/*
 * thn_norm_bwd() for callers that cannot allocate device memory or pass a workspace along: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose
 * wrapper allocates its `_dw` / `_db` partial buffers per call, layernorm.py:183-185).  Same arguments and same
 * results, bit for bit, as thn_norm_bwd(); the partial rows of the two-stage dW / dB sum go to a fixed array of
 * THN_STATIC_WORKSPACE_BYTES in device memory that belongs to the library (one copy per GPU, held until the
 * process ends).  The call allocates nothing and frees nothing; the first call on a device looks the array's
 * address up (hipGetSymbolAddress), so make that one call outside a graph capture: a first call on a stream that
 * is being captured returns THN_E_DEVICE.  Problems whose partial rows -- one per workgroup of the grid the
 * backward launches, at most what thn_norm_bwd_workspace_bytes() says -- need more than THN_STATIC_WORKSPACE_BYTES
 * return THN_E_WORKSPACE: bring a workspace and call thn_norm_bwd().  All calls on one GPU share the array: two calls
 * that may run at the same time (different streams, or graph branches) race on it; calls on one stream are safe.
 */
#define THN_STATIC_WORKSPACE_BYTES (16 * 1024 * 1024)
int thn_norm_bwd_static_workspace(const void* x, int64_t x_row_stride,
                                  const void* dy, int64_t dy_row_stride,
                                  void* dx, int64_t dx_row_stride,
                                  const void* w,
                                  const float* mean, const float* rstd,
                                  void* dw, void* db,
                                  int64_t M, int64_t N,
                                  int x_dtype, int w_dtype, void* stream);

/*
 * Softmax, Softmin and LogSoftmax over the last dimension (the row-reduction activations next to the norm
 * path in the reference: TritonHub/Activations/softmax.py, softmin.py, logsoftmax.py).
 *
 * thn_softmax_fwd replaces `_softmax_kernel_fwd[grid](...)` (softmax.py:37-40, device code :11-24),
 * `_softmin_kernel_fwd` (softmin.py:37-40) and `_logsoftmax_kernel_fwd` (logsoftmax.py:39-43, device code
 * :11-24):  z = x - max(x);  THN_SOFTMAX: y = exp(z)/sum(exp(z));  THN_LOGSOFTMAX: y = z - log(sum(exp(z)));
 * THN_SOFTMIN: softmax of -x (the reference negates with a separate tensor op, softmin.py:103; here the
 * sign is applied on load).
 * thn_softmax_bwd replaces `_softmax_kernel_bwd` (softmax.py:79-83, device code :48-62), `_softmin_kernel_bwd`
 * (softmin.py:79-83) and `_logsoftmax_kernel_bwd` (logsoftmax.py:85-90, device code :51-67); `y` is the SAVED
 * OUTPUT of the forward, as in the reference:
 *   THN_SOFTMAX: dx = y*dy - y*sum(y*dy);  THN_SOFTMIN: the negative of that;  THN_LOGSOFTMAX: dx = dy - exp(y)*sum(dy).
 * All tensors share one storage code.  Arithmetic is float32, except softmax / softmin on THN_F64 storage,
 * which run in float64: the reference's softmax kernels compute in the type they load (softmax.py:18-23),
 * its log-softmax kernels widen to float32 (logsoftmax.py:19, :61-62).  There is no row-width limit: a row wider
 * than 64 KiB is one softmax of the whole row, computed by kernels that walk the row twice (the reference splits
 * such a row into 64 KiB chunks and normalises each chunk by itself, softmax.py:34-40).  N must fit in 31 bits.
 * What a row's results can depend on is as stated for thn_norm_fwd.
 */
enum thn_softmax_kind { THN_SOFTMAX = 0, THN_SOFTMIN = 1, THN_LOGSOFTMAX = 2 };

int thn_softmax_fwd(const void* x, int64_t x_row_stride,
                    void* y, int64_t y_row_stride,
                    int64_t M, int64_t N, int kind, int dtype, void* stream);

int thn_softmax_bwd(const void* y, int64_t y_row_stride,
                    const void* dy, int64_t dy_row_stride,
                    void* dx, int64_t dx_row_stride,
                    int64_t M, int64_t N, int kind, int dtype, void* stream);

/*
 * Row p-norm and p-normalisation over the last dimension of a (B, M, K) tensor (the reference's
 * TritonHub/Ops/norm.py and normalize.py).  x, y, dy, dx: element-contiguous rows, batch and row strides in
 * ELEMENTS; norms, dnorms: contiguous (B*M,) vectors.  All tensors share one storage code; arithmetic is
 * float32 (the reference's `dtype` is float32 unless the tensor is float16 / bfloat16, norm.py:53).
 * p is any real number in [1, 6] and eps >= 0 (the reference's constructor assertions, norm.py:148-149), else
 * THN_E_SHAPE.  There is no row-width limit: rows of more than 64 KiB, and p that is not an integer, take a
 * slower looping kernel.
 *
 * thn_pnorm_fwd replaces `_norm_fwd_kernel[grid](...)` (norm.py:56-59, device code :11-45):
 *   norms = max((sum |x|^p)^(1/p), eps), rounded to the storage type.
 * thn_normalize_fwd replaces the two launches of `_normalize_fwd` (normalize.py:47-54: `_norm_fwd_kernel`, then
 *   `_normalize_fwd_kernel`, device code :11-33) by one pass over x: norms as above, y = x / norms with norms
 *   ALREADY ROUNDED to the storage type (the reference reads them back from the tensor the first kernel wrote).
 * thn_pnorm_bwd replaces `_norm_bwd_kernel[grid](...)` (norm.py:120-125, device code :66-102); `norms` is the
 *   saved output of the forward (not read when p == 1, may then be NULL), `dnorms` its upstream gradient:
 *   p=1: dx = g*sign(x);  p=2: dx = g*x/n;  else dx = g*sign(x)*|x|^(p-1) / n^(p-1).
 * thn_normalize_bwd replaces `_normalize_bwd_kernel[grid](...)` (normalize.py:136-141, device code :61-117); y
 *   and norms are the saved outputs of the forward:  proj = sum(y*dy) (p=1: sum(x*dy));
 *   p=1: dx = dy/n - sign(x)*(proj/(n*n));  p=2: dx = (dy - y*proj)/n;
 *   else dx = dy/n - sign(x)*|x|^(p-1)*(proj/(n^(p-1)*n)).   x is not read when p == 2, y not when p == 1
 *   (each may then be NULL).
 */
int thn_pnorm_fwd(const void* x, int64_t x_batch_stride, int64_t x_row_stride,
                  void* norms,
                  int64_t B, int64_t M, int64_t K, float p, float eps, int dtype, void* stream);

int thn_normalize_fwd(const void* x, int64_t x_batch_stride, int64_t x_row_stride,
                      void* y, int64_t y_batch_stride, int64_t y_row_stride,
                      void* norms,
                      int64_t B, int64_t M, int64_t K, float p, float eps, int dtype, void* stream);

int thn_pnorm_bwd(const void* x, int64_t x_batch_stride, int64_t x_row_stride,
                  const void* norms, const void* dnorms,
                  void* dx, int64_t dx_batch_stride, int64_t dx_row_stride,
                  int64_t B, int64_t M, int64_t K, float p, int dtype, void* stream);

int thn_normalize_bwd(const void* x, int64_t x_batch_stride, int64_t x_row_stride,
                      const void* y, int64_t y_batch_stride, int64_t y_row_stride,
                      const void* norms,
                      const void* dy, int64_t dy_batch_stride, int64_t dy_row_stride,
                      void* dx, int64_t dx_batch_stride, int64_t dx_row_stride,
                      int64_t B, int64_t M, int64_t K, float p, int dtype, void* stream);

/*
 * Element-wise activations (the reference's TritonHub/Activations/gelu.py, silu.py, relu.py, leaky_relu.py,
 * relu6.py, sigmoid.py, tanh.py, mish.py, softplus.py, threshold.py).  (M, N) row-major, unit column stride, row
 * strides in ELEMENTS; one storage code for all tensors; no row-width limit.  `out` must not alias an input.
 *
 * thn_act_fwd replaces the `_<name>_kernel_fwd[grid](...)` launches (gelu.py:45, silu.py:35, relu.py:35,
 * leaky_relu.py:36, relu6.py:36, sigmoid.py:35, tanh.py:37, mish.py:39, softplus.py:37, threshold.py:36);
 * thn_act_bwd the `_<name>_kernel_bwd[grid](...)` launches (gelu.py:100, silu.py:76, relu.py:75,
 * leaky_relu.py:78, relu6.py:77, sigmoid.py:75, tanh.py:77, mish.py:85, softplus.py:81, threshold.py:78).
 *   THN_ACT_GELU        y = 0.5*x*(1 + erf(x/sqrt 2));                    dx = dy*(cdf + x*pdf)
 *   THN_ACT_GELU_TANH   y = 0.5*x*(1 + tanh(sqrt(2/pi)*(x + 0.044715 x^3))); dx as gelu.py:71-75
 *   THN_ACT_SILU        y = x*sigmoid(x);                                 dx = dy*(s*(1 + x*(1 - s)))
 *   THN_ACT_RELU        y = x > 0 ? x : 0;                                dx = x > 0 ? dy : 0
 *   THN_ACT_LEAKY_RELU  y = x > 0 ? x : param0*x;                         dx = x > 0 ? dy : param0*dy
 *   THN_ACT_RELU6       y = min(max(x, 0), 6);                            dx = 0 < x < 6 ? dy : 0
 *   THN_ACT_SIGMOID     y = 1/(1 + exp(-x));                              dx = dy*y*(1 - y)      (saved: OUTPUT)
 *   THN_ACT_TANH        y = tanh(x);                                      dx = dy*(1 - y*y)      (saved: OUTPUT)
 *   THN_ACT_MISH        y = x*tanh(softplus(x));                          dx as mish.py:60-66
 *   THN_ACT_SOFTPLUS    y = x*param0 > param1 ? x : log(1 + exp(param0*x))/param0   (param0 = beta, param1 = threshold)
 *                       dx = x*param0 > param1 ? dy : dy/(1 + exp(-param0*x))
 *   THN_ACT_THRESHOLD   y = x > param0 ? x : param1;                      dx = x > param0 ? dy : 0
 * `saved` of thn_act_bwd is what the reference's Function saves: the forward's input, or its OUTPUT for
 * THN_ACT_SIGMOID and THN_ACT_TANH (sigmoid.py:81-92, tanh.py:83-94).
 * Arithmetic is float32, except RELU / LEAKY_RELU / RELU6 / SOFTPLUS / THRESHOLD on THN_F64 storage, which the
 * reference computes in the loaded type (no `.to(tl.float32)`, relu.py:18): float64 there.  Where the
 * reference's tanh-as-exponentials overflows to NaN for large |x| (tanh.py:19-21, mish.py:20-22, gelu.py:24-25)
 * the same function is evaluated in a form that cannot overflow.
 */
enum thn_act {
    THN_ACT_GELU = 0, THN_ACT_GELU_TANH = 1, THN_ACT_SILU = 2, THN_ACT_RELU = 3, THN_ACT_LEAKY_RELU = 4,
    THN_ACT_RELU6 = 5, THN_ACT_SIGMOID = 6, THN_ACT_TANH = 7, THN_ACT_MISH = 8, THN_ACT_SOFTPLUS = 9,
    THN_ACT_THRESHOLD = 10
};

int thn_act_fwd(const void* x, int64_t x_row_stride,
                void* y, int64_t y_row_stride,
                int64_t M, int64_t N, int act, float param0, float param1, int dtype, void* stream);

int thn_act_bwd(const void* saved, int64_t saved_row_stride,
                const void* dy, int64_t dy_row_stride,
                void* dx, int64_t dx_row_stride,
                int64_t M, int64_t N, int act, float param0, float param1, int dtype, void* stream);

/*
 * LayerNorm / RMSNorm with an activation epilogue: y = act(normalise(x)*w + b) in ONE pass over the tensor.
 * The reference has no such operator; its quick start chains the two (README.md:47-48: `x = layernorm(x)`,
 * then `x = gelu(x)`), i.e. `_layernorm_kernel_fwd` (layernorm.py:74-86) followed by `_gelu_kernel_fwd`
 * (gelu.py:45), and in the backward `_gelu_kernel_bwd` (gelu.py:100) followed by `_layernorm_kernel_bwd` plus the
 * partial sums (layernorm.py:188-208).  These two entry points replace each pair by one launch (plus the
 * second-stage reduction): the activation is applied to the float32 value before the single rounding on store,
 * and the backward recomputes the pre-activation z = xhat*w + b from the saved statistics (nothing extra is
 * saved), replaces dy by dy*act'(z) and continues as thn_norm_bwd.  Five passes over the tensor instead of ten.
 * `act`: THN_ACT_GELU, THN_ACT_GELU_TANH, THN_ACT_SILU or THN_ACT_RELU (the parameter-free activations whose
 * backward needs only their input); anything else is THN_E_SHAPE.  All other arguments and the NULL conventions
 * are those of thn_norm_fwd / thn_norm_bwd; the workspace is sized by thn_norm_act_bwd_workspace_bytes (the
 * arithmetic-bound GeLU variants run more workgroups, hence more partial rows, than the plain backward); `b` is the
 * forward's bias (NULL when there is none).  Because the intermediate is never rounded to the storage type, the
 * result is closer to exact arithmetic than the chained operators', not bit-identical to them.
 */
int thn_norm_act_fwd(const void* x, int64_t x_row_stride,
                     void* y, int64_t y_row_stride,
                     const void* w, const void* b,
                     float* mean, float* rstd,
                     int64_t M, int64_t N, float eps, int act,
                     int x_dtype, int w_dtype, void* stream);

int64_t thn_norm_act_bwd_workspace_bytes(int64_t M, int64_t N, int want_dw, int want_db, int act, int x_dtype);

int thn_norm_act_bwd(const void* x, int64_t x_row_stride,
                     const void* dy, int64_t dy_row_stride,
                     void* dx, int64_t dx_row_stride,
                     const void* w, const void* b,
                     const float* mean, const float* rstd,
                     void* dw, void* db,
                     void* workspace, int64_t workspace_bytes,
                     int64_t M, int64_t N, int act,
                     int x_dtype, int w_dtype, void* stream);

/*
 * Dropout over a contiguous tensor of `n` elements (the reference's TritonHub/Layers/dropout.py).  Replaces both
 * `_dropout_kernel_fwd[grid](x, out, M, p, seed, ...)` (dropout.py:43-48, device code :12-23) and
 * `_dropout_kernel_bwd[grid](dout, dx, M, p, seed, ...)` (dropout.py:87-92, device code :56-67), which are the same
 * function: out[i] = rand(seed, i) < p ? 0 : x[i] / (1 - p), in float32 (float64 storage: the float64 quotient by
 * the float32 1 - p), rounded to the storage type.  rand(seed, i) is what Triton's tl.rand(seed, i) returns --
 * Philox-4x32-10 on counter (i, 0, 0, 0) and key (seed), first word, mapped to a float32 in [0, 1) -- so a seed
 * gives the same mask as in the reference, bit for bit.  Element i of the call uses offset first_offset + i (0 for
 * a whole tensor; a caller that splits a tensor into pieces passes each piece's position); offsets of 2^32 and
 * more put their high word into the second counter word, as tl.rand does for 64-bit offsets (the reference's
 * 32-bit `cols` would have wrapped).  0 <= p <= 1.  `x` and `out` need element alignment only and must not overlap
 * partially (out == x, in place, is fine).  The p == 0 / eval-mode / p == 1 shortcuts of dropout.py:29-32 are the
 * caller's.
 */
int thn_dropout(const void* x, void* out, int64_t n, int64_t first_offset, float p, uint64_t seed, int dtype,
                void* stream);

/*
 * Launch-shape control for tuning sweeps (the counterpart of the reference's `triton.autotune` over
 * num_warps, autotune.py:62-65, which this library replaces by a fixed heuristic on N and the dtype).
 * `which`: 0 = norm forward, 1 = norm backward, 2 = softmax forward, 3 = softmax backward, 4 = p-norm /
 * normalize forward, 5 = p-norm backward, 6 = normalize backward, 7 / 8 = element-wise activation forward /
 * backward (only blocks_per_cu applies to them; thn_norm_query_launch does not cover them), 9 / 10 = norm with
 * activation epilogue forward / backward.
 * vecs_per_thread / threads_per_row / block_threads select a compiled kernel shape, blocks_per_cu caps the
 * persistent grid; 0 for any field keeps the heuristic's choice.
 * For the norm forward / backward (0, 1) two more kernel families for rows of at most 32 16-byte vectors (float32 /
 * float16 / bfloat16 rows on the 128-bit path) are selected here as well: a threads_per_row that is not a power of two,
 * with block_threads 0 or 256, selects the flat kernels for rows of exactly that many vectors (lanes are dealt to
 * vectors without gaps, a wave holds 64 / threads_per_row whole rows; vecs_per_thread = rows a lane carries per step:
 * 1, 2 or 4; rows off the 128-bit path -- a width that is not a whole number of vectors, a pointer or pitch off 16
 * bytes -- of 2 to 32 vectors, powers of two included, with 1 or 2); block_threads = 64 selects the staged kernels (a wave copies a batch of rows into LDS and one lane sums a
 * row; threads_per_row = the row's vector count or 0, vecs_per_thread = the batch in passes of the wave over its rows:
 * 1 to 4, or 0 for the default).  Problems such an override does not fit are refused (THN_E_SHAPE); any other
 * override runs the row kernels.
 * The softmax and p-norm families (2 to 6) have flat kernels of their own for rows of 1, 2 and 4 vectors and of up to
 * 32 vectors whose count is not a power of two, taken by default: threads_per_row = the row's vector count (with
 * block_threads 0 or 256 and vecs_per_thread 0, 2 or, softmax only, 4 rows per lane and step) keeps them, any other
 * shape selects the row kernels for such rows too.  Off the 128-bit path (rows of at least one vector) they take 2 rows
 * per lane only.
 * Process-wide; meant for benchmarks, not for concurrent production use.  Returns THN_E_SHAPE when no
 * compiled kernel has that shape.
 */
int thn_norm_set_launch_override(int which, int vecs_per_thread, int threads_per_row, int block_threads,
                                 int blocks_per_cu);

/*
 * What the heuristic (or the override) would launch for this problem: fills shape[0..4] with
 * {vecs_per_thread, threads_per_row, block_threads, grid_blocks, aligned 128-bit path (1) or unaligned-row path (0)}.
 * (the last field is 0 for every kind of kernel when the rows are off the 128-bit path).
 * For the epilogue families (9, 10) `is_layernorm` carries the activation too: bit 0 = LayerNorm, bits 1.. = the
 * thn_act code.  For the p-norm / normalize forward (4) a non-zero `is_layernorm` asks for thn_normalize_fwd's launch
 * (0: thn_pnorm_fwd's; they differ for 16-bit rows of 769 to 1024 vectors off the 128-bit path).  Rows wider than 64 KiB of the softmax and p-norm families report their looping kernels:
 * {vectors per thread and step, block_threads, block_threads, grid_blocks, 0}.  Norm problems that take the flat
 * kernels (narrow 16-bit rows whose vector count is not a power of two; off the 128-bit path narrow rows of any
 * vector count and type) report {rows per lane and step, vectors per row, 256, grid_blocks, 1}: a threads_per_row that
 * is not a power of two identifies them (off the path a flat launch over 8, 16 or 32 vectors with one row per lane
 * reads like the row kernels' 1 x 8, 1 x 16 and 1 x 32 shapes in 256 threads); those that take the staged
 * kernels (rows of 1 to 8 vectors, narrow float32 rows) report {passes per batch, vectors per row, 64, grid_blocks, 1}.
 * Softmax and p-norm problems over rows shorter than one vector report {4, 1, 256, grid_blocks, 0}: four rows per
 * lane and step, ONE lane per row (any launch override with a shape field set selects the row kernels' element-wise
 * instance, 4 x 8 in 256 threads, instead).
 * Softmax and p-norm problems on their flat kernels report {2 or 4, vectors per row, 256, grid_blocks, 1} (a p-norm
 * problem is taken to be a dense (M, N) tensor here; tensors whose batches do not fold run the row kernels).
 */
int thn_norm_query_launch(int which, int is_layernorm, int64_t M, int64_t N, int x_dtype, int32_t shape[5]);

#ifdef __cplusplus
}
#endif
#endif /* THNORM_H_ */
