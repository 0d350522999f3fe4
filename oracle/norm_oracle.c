/*
 * CPU oracle for the LayerNorm / RMSNorm forward + backward path -- TEST INFRASTRUCTURE ONLY.
 *
 * Plain C restatement, with double accumulation, of the reference's device kernels and of its second-stage
 * parameter-gradient sum.  It exists so that full-size cases can be checked in seconds and so that the
 * benchmark has a CPU figure to print next to the GPU one.  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py load the library built from this file; the product library never links it.
 *
 *   thn_oracle_layernorm_fwd  follows TritonHub/Normalization/layernorm.py:31-46
 *   thn_oracle_layernorm_bwd  follows TritonHub/Normalization/layernorm.py:128-153 and :207-208
 *   thn_oracle_rmsnorm_fwd    follows TritonHub/Normalization/rmsnorm.py:28-38
 *   thn_oracle_rmsnorm_bwd    follows TritonHub/Normalization/rmsnorm.py:104-122 and :166
 *
 * Pinned by tests/test_oracle_pins.py: it must agree with oracle/norm_oracle.py (itself pinned against
 * torch's float64 CPU kernels, frozen vectors, finite differences and closed forms) to float64 round-off.
 *
 * Storage codes (same as the product's C ABI): 0 = float32, 1 = float16, 2 = bfloat16, 3 = float64.
 * Inputs x, dy, w, b are read in their storage type and widened exactly to double.  Outputs y, dx, dw, db
 * are written as float64 when out_dtype == 3 (checking mode: nothing is rounded) or narrowed to
 * out_dtype otherwise (timing mode: double -> float -> half/bfloat16, round to nearest even at each step).
 * mean / rstd are always float64 here.  All matrices are dense row-major (M, N).  y and dx may be NULL
 * (statistics-only forward, parameter-gradient-only backward).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

enum { THN_F32 = 0, THN_F16 = 1, THN_BF16 = 2, THN_F64 = 3 };

static inline float bits_to_float(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t float_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline double half_to_double(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {                      /* zero or subnormal: man * 2^-24 */
        double v = ldexp((double)man, -24);
        return sign ? -v : v;
    }
    if (exp == 31) return bits_to_float(sign | 0x7f800000u | (man << 13));
    return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
}

static inline uint16_t float_to_half(float f) {           /* round to nearest even */
    uint32_t u = float_to_bits(f);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t a = u & 0x7fffffffu;
    if (a >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | ((a > 0x7f800000u) ? 0x200u : 0));
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);          /* rounds to >= 65520 -> inf */
    if (a < 0x38800000u) {                                            /* below 2^-14: subnormal half */
        float scaled = bits_to_float(a) * 16777216.0f;                /* * 2^24, exact */
        float r = nearbyintf(scaled);
        return (uint16_t)(sign | (uint32_t)r);
    }
    uint32_t lsb = (a >> 13) & 1u;
    a += 0xfffu + lsb;
    return (uint16_t)(sign | ((a - 0x38000000u) >> 13));
}

static inline uint16_t float_to_bf16(float f) {           /* round to nearest even */
    uint32_t u = float_to_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    uint32_t lsb = (u >> 16) & 1u;
    return (uint16_t)((u + 0x7fffu + lsb) >> 16);
}

static inline double load_elem(const void* p, int64_t i, int dtype) {
    switch (dtype) {
        case THN_F32:  return ((const float*)p)[i];
        case THN_F16:  return half_to_double(((const uint16_t*)p)[i]);
        case THN_BF16: return bits_to_float((uint32_t)((const uint16_t*)p)[i] << 16);
        default:       return ((const double*)p)[i];
    }
}

static inline void store_elem(void* p, int64_t i, int dtype, double v) {
    switch (dtype) {
        case THN_F32:  ((float*)p)[i] = (float)v; break;
        case THN_F16:  ((uint16_t*)p)[i] = float_to_half((float)v); break;
        case THN_BF16: ((uint16_t*)p)[i] = float_to_bf16((float)v); break;
        default:       ((double*)p)[i] = v; break;
    }
}

static int bad_dtype(int d) { return d < 0 || d > 3; }

static double* widen_params(const void* p, int64_t n, int dtype, double fill) {
    double* out = (double*)malloc(sizeof(double) * (size_t)(n > 0 ? n : 1));
    if (!out) return NULL;
    for (int64_t j = 0; j < n; ++j) out[j] = p ? load_elem(p, j, dtype) : fill;
    return out;
}

int thn_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* layernorm.py:31-46 -- mean, biased two-pass variance, rstd, normalise, affine. */
int thn_oracle_layernorm_fwd(const void* x, int x_dtype, const void* w, const void* b, int w_dtype,
                             double eps, int64_t M, int64_t N,
                             void* y, int out_dtype, double* mean, double* rstd) {
    if (bad_dtype(x_dtype) || bad_dtype(w_dtype) || bad_dtype(out_dtype) || M < 0 || N <= 0) return -1;
    double* wd = widen_params(w, N, w_dtype, 1.0);
    double* bd = widen_params(b, N, w_dtype, 0.0);
    if (!wd || !bd) { free(wd); free(bd); return -2; }
#pragma omp parallel
    {
        double* row = (double*)malloc(sizeof(double) * (size_t)N);
#pragma omp for schedule(static)
        for (int64_t r = 0; r < M; ++r) {
            const int64_t base = r * N;
            double s = 0.0;
            for (int64_t j = 0; j < N; ++j) { row[j] = load_elem(x, base + j, x_dtype); s += row[j]; }
            const double mu = s / (double)N;
            double q = 0.0;
            for (int64_t j = 0; j < N; ++j) { const double d = row[j] - mu; q += d * d; }
            const double rs = 1.0 / sqrt(q / (double)N + eps);
            mean[r] = mu;
            rstd[r] = rs;
            if (y)
                for (int64_t j = 0; j < N; ++j)
                    store_elem(y, base + j, out_dtype, (row[j] - mu) * rs * wd[j] + bd[j]);
        }
        free(row);
    }
    free(wd); free(bd);
    return 0;
}

/* rmsnorm.py:28-38 -- mean square, rstd, scale. */
int thn_oracle_rmsnorm_fwd(const void* x, int x_dtype, const void* w, int w_dtype,
                           double eps, int64_t M, int64_t N,
                           void* y, int out_dtype, double* rstd) {
    if (bad_dtype(x_dtype) || bad_dtype(w_dtype) || bad_dtype(out_dtype) || M < 0 || N <= 0) return -1;
    double* wd = widen_params(w, N, w_dtype, 1.0);
    if (!wd) return -2;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < M; ++r) {
        const int64_t base = r * N;
        double q = 0.0;
        for (int64_t j = 0; j < N; ++j) { const double v = load_elem(x, base + j, x_dtype); q += v * v; }
        const double rs = 1.0 / sqrt(q / (double)N + eps);
        rstd[r] = rs;
        if (y)
            for (int64_t j = 0; j < N; ++j)
                store_elem(y, base + j, out_dtype, load_elem(x, base + j, x_dtype) * rs * wd[j]);
    }
    free(wd);
    return 0;
}

/*
 * Shared backward.  layernorm.py:128-153 (mean != NULL) and rmsnorm.py:104-122 (mean == NULL):
 *   xhat = (x - mean) * rstd;  wdy = w * dy;  c1 = sum(xhat*wdy)/N;  c2 = sum(wdy)/N (LayerNorm only);
 *   dx = (wdy - (xhat*c1 + c2)) * rstd;  dW += dy*xhat;  dB += dy.
 * The per-thread partial sums are combined in thread order, the analogue of the reference's
 * (sm_count, N) partial rows followed by .sum(0) (layernorm.py:150-153, :207-208).
 */
static int backward(const void* x, const void* dy, int x_dtype, const void* w, int w_dtype,
                    const double* mean, const double* rstd, int64_t M, int64_t N,
                    void* dx, int out_dtype, void* dw, void* db, int dw_dtype) {
    if (bad_dtype(x_dtype) || bad_dtype(w_dtype) || bad_dtype(out_dtype) || bad_dtype(dw_dtype) || M < 0 || N <= 0)
        return -1;
    double* wd = widen_params(w, N, w_dtype, 1.0);
    if (!wd) return -2;
    int nthreads = thn_oracle_num_threads();
    double* part = (double*)calloc((size_t)nthreads * 2u * (size_t)N, sizeof(double));
    if (!part) { free(wd); return -2; }
#pragma omp parallel
    {
#ifdef _OPENMP
        const int tid = omp_get_thread_num();
#else
        const int tid = 0;
#endif
        double* pdw = part + (size_t)tid * 2u * (size_t)N;
        double* pdb = pdw + N;
        double* xh = (double*)malloc(sizeof(double) * (size_t)N);
        double* g = (double*)malloc(sizeof(double) * (size_t)N);
#pragma omp for schedule(static)
        for (int64_t r = 0; r < M; ++r) {
            const int64_t base = r * N;
            const double mu = mean ? mean[r] : 0.0;
            const double rs = rstd[r];
            double s1 = 0.0, s2 = 0.0;
            for (int64_t j = 0; j < N; ++j) {
                xh[j] = (load_elem(x, base + j, x_dtype) - mu) * rs;
                g[j] = load_elem(dy, base + j, x_dtype);
                const double wdy = wd[j] * g[j];
                s1 += xh[j] * wdy;
                s2 += wdy;
            }
            const double c1 = s1 / (double)N;
            const double c2 = mean ? s2 / (double)N : 0.0;
            for (int64_t j = 0; j < N; ++j) {
                const double wdy = wd[j] * g[j];
                if (dx) store_elem(dx, base + j, out_dtype, (wdy - (xh[j] * c1 + c2)) * rs);
                pdw[j] += g[j] * xh[j];
                pdb[j] += g[j];
            }
        }
        free(xh); free(g);
    }
    for (int64_t j = 0; j < N; ++j) {
        double sw = 0.0, sb = 0.0;
        for (int t = 0; t < nthreads; ++t) {
            sw += part[(size_t)t * 2u * (size_t)N + (size_t)j];
            sb += part[(size_t)t * 2u * (size_t)N + (size_t)N + (size_t)j];
        }
        if (dw) store_elem(dw, j, dw_dtype, sw);
        if (db) store_elem(db, j, dw_dtype, sb);
    }
    free(part); free(wd);
    return 0;
}

int thn_oracle_layernorm_bwd(const void* x, const void* dy, int x_dtype, const void* w, int w_dtype,
                             const double* mean, const double* rstd, int64_t M, int64_t N,
                             void* dx, int out_dtype, void* dw, void* db, int dw_dtype) {
    if (!mean) return -1;
    return backward(x, dy, x_dtype, w, w_dtype, mean, rstd, M, N, dx, out_dtype, dw, db, dw_dtype);
}

int thn_oracle_rmsnorm_bwd(const void* x, const void* dy, int x_dtype, const void* w, int w_dtype,
                           const double* rstd, int64_t M, int64_t N,
                           void* dx, int out_dtype, void* dw, int dw_dtype) {
    return backward(x, dy, x_dtype, w, w_dtype, NULL, rstd, M, N, dx, out_dtype, dw, NULL, dw_dtype);
}
