// One walk of a workgroup over a row of any width and alignment, for the kernels that loop over a row instead of
// holding it in registers (rows wider than 64 KiB, p-norms with a real exponent).
#pragma once

#include "thn_device.h"

namespace thn {

constexpr int kWalkVecs = 4;    // 16-byte vectors per thread and step

// Whole vectors go to fn_vec(f, o): f[i][e] is element e of the vector of stream i, o[e] the value to store when
// STORE; the elements behind the last whole vector go to fn_elem(in0[c], in1[c], in2[c]) one by one (its value is
// stored when STORE).  Arithmetic type C.  Thread t of BLOCK takes vectors t, t + BLOCK, ...: 16-byte accesses at
// element-aligned addresses (the memory pipeline runs in unaligned access mode), kWalkVecs per thread and step, all
// requested before the first is used (PIPE: one step ahead).  KEEP: the row will be walked again, so the loads carry no non-temporal hint.
template <typename T, typename C, int BLOCK, int NIN, bool STORE, bool KEEP = false, bool PIPE = false, typename FnVec,
          typename FnElem>
__device__ __forceinline__ void walk_row_vec(const char* in0, const char* in1, const char* in2, char* out, int64_t n,
                                             int t, FnVec&& fn_vec, FnElem&& fn_elem) {
    constexpr int VEC = T::VEC;
    constexpr int U = kWalkVecs;
    // When every stream of the row sits at the same offset from a 16-byte boundary (rows of one tensor family
    // with equal strides: the usual case), the elements in front of that boundary go one by one and the vectors
    // are aligned: 16-bit rows with an odd element offset otherwise pay about a third of their bandwidth.
    const uintptr_t mis = reinterpret_cast<uintptr_t>(in0) & 15u;
    bool same = (!STORE || (reinterpret_cast<uintptr_t>(out) & 15u) == mis) &&
                (NIN < 2 || (reinterpret_cast<uintptr_t>(in1) & 15u) == mis) &&
                (NIN < 3 || (reinterpret_cast<uintptr_t>(in2) & 15u) == mis);
    int64_t head = same ? static_cast<int64_t>(((16u - mis) & 15u) / T::kBytes) : 0;
    if (head > n) head = n;
    auto one = [&](int64_t c) {
        const C o = fn_elem(load_elem<T, C>(in0, c), NIN > 1 ? load_elem<T, C>(in1, c) : C(0),
                            NIN > 2 ? load_elem<T, C>(in2, c) : C(0));
        if constexpr (STORE) store_elem<T, C>(out, c, o);
    };
    if (t < head) one(t);
    const int64_t skip = head * T::kBytes;
    const char* in[3] = {in0 + skip, NIN > 1 ? in1 + skip : nullptr, NIN > 2 ? in2 + skip : nullptr};
    char* outv = STORE ? out + skip : nullptr;
    const int64_t whole = (n - head) / VEC;
    // PIPE: the vectors of the next step are requested before the current ones are used (softmax: +2-4 %; the
    // p-norm walks with a real exponent lost 20 % with it)
    u32x4 cur[U][NIN];
    auto request = [&](u32x4 (&dst)[U][NIN], int64_t v0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t v = v0 + u * BLOCK;
            if (v < whole) {
#pragma unroll
                for (int i = 0; i < NIN; ++i) dst[u][i] = KEEP ? ld128u_keep(in[i] + v * 16) : ld128u(in[i] + v * 16);
            }
        }
    };
    if constexpr (PIPE) request(cur, t);
    for (int64_t v0 = t; v0 < whole; v0 += BLOCK * U) {
        u32x4 nxt[PIPE ? U : 1][NIN];
        if constexpr (PIPE) request(nxt, v0 + BLOCK * U);
        else request(cur, v0);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t v = v0 + u * BLOCK;
            if (v < whole) {
                C f[3][VEC], o[VEC];
#pragma unroll
                for (int i = 0; i < NIN; ++i) unpack_as<T>(cur[u][i], f[i]);
                fn_vec(f, o);
                if constexpr (STORE) st128u(outv + v * 16, pack_as<T, C>(o));
            }
        }
        if constexpr (PIPE) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (int i = 0; i < NIN; ++i) cur[u][i] = nxt[u][i];
            }
        }
    }
    for (int64_t c = head + whole * VEC + t; c < n; c += BLOCK) one(c);
}

// The element-wise form: fn(in0[c], in1[c], in2[c]) for every column c (absent streams pass 0).
template <typename T, typename C, int BLOCK, int NIN, bool STORE, bool KEEP = false, bool PIPE = false, typename Fn>
__device__ __forceinline__ void walk_row(const char* in0, const char* in1, const char* in2, char* out, int64_t n,
                                         int t, Fn&& fn) {
    constexpr int VEC = T::VEC;
    walk_row_vec<T, C, BLOCK, NIN, STORE, KEEP, PIPE>(
        in0, in1, in2, out, n, t,
        [&](const C (&f)[3][VEC], C (&o)[VEC]) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) o[e] = fn(f[0][e], NIN > 1 ? f[1][e] : C(0), NIN > 2 ? f[2][e] : C(0));
        },
        fn);
}

}  // namespace thn
