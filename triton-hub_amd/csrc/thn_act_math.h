// Element-wise activation formulas, forward and derivative, shared by the streaming activation kernels (thn_act.h)
// and by the activation epilogue of the norm kernels (thn_kernels.h).  Each formula cites the line of the
// reference it restates (TritonHub/Activations/*.py).
#pragma once

#include <type_traits>

#include "thn_device.h"

namespace thn {

enum : int {
    kGelu = 0, kGeluTanh = 1, kSilu = 2, kRelu = 3, kLeakyRelu = 4, kRelu6 = 5, kSigmoid = 6, kTanh = 7, kMish = 8,
    kSoftplus = 9, kThreshold = 10, kNumActs = 11
};

__device__ __forceinline__ float log_c(float z) { return __logf(z); }
__device__ __forceinline__ double log_c(double z) { return log(z); }

// The float32 formulas below are written for the instruction budget of a streaming kernel: at 16-bit storage a
// compute unit must finish an element in about 25 instruction slots to keep up with HBM, and the quarter-rate
// v_exp_f32 / v_log_f32 / v_rcp_f32 cost four slots each.  Quotients use the hardware reciprocal (1 ulp) and a
// multiplication instead of an IEEE division (10 slots); every result stays within a few float32 ulp of the exact
// function, far inside the test tolerances.
__device__ __forceinline__ float rcp_fast(float x) { return __builtin_amdgcn_rcpf(x); }

// tanh(u) = sign(u) * (1 - t)/(1 + t) with t = exp(-2|u|): no overflow for any u.
__device__ __forceinline__ float tanh_safe(float u) {
    const float t = __expf(-2.0f * __builtin_fabsf(u));
    const float r = (1.0f - t) * rcp_fast(1.0f + t);
    return u < 0.0f ? -r : r;
}

__device__ __forceinline__ float sigmoid_f(float x) { return rcp_fast(1.0f + __expf(-x)); }

// The gate of the tanh form of GeLU: 0.5*(1 + tanh(u)) with u = sqrt(2/pi)*(x + 0.044715 x^3) (gelu.py:23-26) is the
// logistic function of 2u, 1/(1 + exp(-2u)).  One exponential and one reciprocal, no cancellation for negative x
// (where 1 + tanh(u) loses every digit), no overflow: exp(-2u) = inf gives 0, exp(-2u) = 0 gives 1.
struct GateParts { float gate, e; };            // e = exp(-2u), gate = 1/(1 + e)
__device__ __forceinline__ GateParts gelu_tanh_gate_parts(float x) {
    const float inner = __builtin_fmaf(0.044715f * x * x, x, x);
    GateParts p;
    p.e = __builtin_amdgcn_exp2f(-2.302208198144325f * inner);                     // -2*sqrt(2/pi)*log2(e)
    p.gate = rcp_fast(1.0f + p.e);
    return p;
}
__device__ __forceinline__ float gelu_tanh_gate(float x) { return gelu_tanh_gate_parts(x).gate; }

// Phi(x) = 0.5*(1 + erf(x/sqrt 2)), the normal distribution function of GeLU, from the complementary error function
// of z = |x|/sqrt 2, in two forms that share t = 1/(1 + z/2) in (0, 1].  Both are branch free, accurate in the
// negative tail (where 1 + erf(..) cancels) and a third of the instructions of the library erff.  Their
// exponentials are base 2 (the hardware's v_exp_f32), so they work on a = z*sqrt(log2 e), a^2 = z^2*log2(e), and the
// factor 1/2 of Phi is folded into the coefficients.
//
// Backward form: erfc(z) = erfcx(z)*exp(-z^2) with erfcx(z) = t*Q(t), Q of degree 10 (fitted for the smallest
// relative error of t*Q(t): 1.1e-8; 1.2e-7 after float32 Horner evaluation; Q(0) = 1/(2 sqrt(pi)), the limit of
// erfcx(z)*z/2).  Its exponential is exp(-x^2/2), the one the normal density needs: GeLU' costs one exponential.
struct NormalParts { float cdf, e; };           // e = exp(-x^2/2)
__device__ __forceinline__ NormalParts normal_parts(float x) {
    const float a = __builtin_fabsf(x) * 0.84932180028801907f;
    const float t = rcp_fast(__builtin_fmaf(0.41627730557884884f, a, 1.0f));
    float q = 0.021176133f;                     // Q/2
    q = __builtin_fmaf(q, t, -0.1154281f);
    q = __builtin_fmaf(q, t, 0.24308807f);
    q = __builtin_fmaf(q, t, -0.22348733f);
    q = __builtin_fmaf(q, t, 0.06354388f);
    q = __builtin_fmaf(q, t, -0.028615918f);
    q = __builtin_fmaf(q, t, 0.046500217f);
    q = __builtin_fmaf(q, t, 0.08768842f);
    q = __builtin_fmaf(q, t, 0.123440295f);
    q = __builtin_fmaf(q, t, 0.14104693f);
    q = __builtin_fmaf(q, t, 0.1410474f);
    NormalParts n;
    n.e = __builtin_amdgcn_exp2f(-a * a);
    const float half_erfc = t * q * n.e;
    n.cdf = x < 0.0f ? half_erfc : 1.0f - half_erfc;
    return n;
}

// Forward form: erfc(z)/2 = t*exp(-z^2 + P(t) - ln 2) (the Chebyshev fit of Numerical Recipes 6.2, relative error
// below 1.5e-7 for every z with the coefficients scaled to base 2): one multiplication fewer than the product form,
// which measured 1-6 % slower in the forward kernels.
__device__ __forceinline__ float normal_cdf(float x) {
    const float a = __builtin_fabsf(x) * 0.84932180028801907f;
    const float t = rcp_fast(__builtin_fmaf(0.41627730557884884f, a, 1.0f));
    float p = 0.2465173f;
    p = __builtin_fmaf(p, t, -1.1861149f);
    p = __builtin_fmaf(p, t, 2.1474745f);
    p = __builtin_fmaf(p, t, -1.6377531f);
    p = __builtin_fmaf(p, t, 0.40232158f);
    p = __builtin_fmaf(p, t, -0.26875687f);
    p = __builtin_fmaf(p, t, 0.13963005f);
    p = __builtin_fmaf(p, t, 0.5397006f);
    p = __builtin_fmaf(p, t, 1.4427292f);
    p = __builtin_fmaf(p, t, -2.8257482f);
    const float half_erfc = t * __builtin_amdgcn_exp2f(__builtin_fmaf(-a, a, p));
    return x < 0.0f ? half_erfc : 1.0f - half_erfc;
}

// Mish needs t = tanh(softplus(x)) with softplus(x) = x > 20 ? x : log(1 + e^x) (mish.py:19-22).  With w = e^x and
// n = w*(w + 2):  tanh(log(1 + w)) = n/(n + 2)  and  1 - t^2 = 4*(n + 1)/(n + 2)^2 : one exponential, one
// reciprocal, no cancellation for very negative x (where log(1 + e^x) rounds to 0 in float32).  Above 20 the
// reference's branch gives tanh(x), which is 1 in float32.
struct MishParts { float t, one_minus_t2, sig; };
__device__ __forceinline__ MishParts mish_parts(float x) {
    const float w = __expf(x < 20.0f ? x : 20.0f);
    const float n = w * (w + 2.0f);
    const float r = rcp_fast(n + 2.0f);
    MishParts m;
    const bool big = x > 20.0f;
    m.t = big ? 1.0f : n * r;
    m.one_minus_t2 = big ? 0.0f : 4.0f * (n + 1.0f) * r * r;
    m.sig = big ? 1.0f : w * rcp_fast(1.0f + w);          // sigmoid(x) = w/(1 + w); 1 in float32 above 20
    return m;
}

template <int ACT, typename C>
__device__ __forceinline__ C act_fwd(C x, C p0, C p1) {
    if constexpr (ACT == kGelu) {
        return x * normal_cdf(x);                                                          // gelu.py:28
    } else if constexpr (ACT == kGeluTanh) {
        return x * gelu_tanh_gate(x);                                                      // gelu.py:23-26
    } else if constexpr (ACT == kSilu) {
        return x * sigmoid_f(x);                                                           // silu.py:19
    } else if constexpr (ACT == kRelu) {
        return x > C(0) ? x : C(0);                                                        // relu.py:19
    } else if constexpr (ACT == kLeakyRelu) {
        return x > C(0) ? x : p0 * x;                                                      // leaky_relu.py:20
    } else if constexpr (ACT == kRelu6) {
        const C r = x > C(0) ? x : C(0);                                                   // relu6.py:19-20
        return r < C(6) ? r : C(6);
    } else if constexpr (ACT == kSigmoid) {
        return sigmoid_f(x);                                                               // sigmoid.py:19
    } else if constexpr (ACT == kTanh) {
        return tanh_safe(x);                                                               // tanh.py:19-21
    } else if constexpr (ACT == kMish) {
        return x * mish_parts(x).t;                                                        // mish.py:19-23
    } else if constexpr (ACT == kSoftplus) {
        if constexpr (std::is_same<C, float>::value) {                                     // softplus.py:21
            // base-2 hardware exponential and logarithm; the factors log2(e)*beta and ln(2)/beta are the same for every
            // element (two multiplications fewer per element than exp and log of base e)
            const float k = p0 * 1.44269504088896341f, inv = 0.69314718055994531f * rcp_fast(p0);
            return x * p0 > p1 ? x : __builtin_amdgcn_logf(1.0f + __builtin_amdgcn_exp2f(k * x)) * inv;
        } else {
            return x * p0 > p1 ? x : log_c(C(1) + exp_c(p0 * x)) / p0;
        }
    } else {
        return x > p0 ? x : p1;                                                            // threshold.py:20
    }
}

// `s` is the saved tensor: the forward's input, or its output for Sigmoid and Tanh.
template <int ACT, typename C>
__device__ __forceinline__ C act_bwd(C s, C g, C p0, C p1) {
    if constexpr (ACT == kGelu) {
        const NormalParts n = normal_parts(s);                                             // gelu.py:77-80
        const float pdf = n.e * 0.39894228040143267794f;
        return g * __builtin_fmaf(s, pdf, n.cdf);
    } else if constexpr (ACT == kGeluTanh) {
        // gelu.py:71-75 with t = tanh(u) = 2*gate - 1: 0.5*(1 + t) = gate, 0.5*(1 - t^2) = 2*gate*(1 - gate)
        const GateParts p = gelu_tanh_gate_parts(s);
        const float gate = p.gate;
        // 1 - gate = e*gate: taken from whichever side does not cancel (e = inf goes with gate = 0 < 0.5)
        const float slope = gate * (gate < 0.5f ? 1.0f - gate : p.e * gate);   // gate*(1 - gate) = sech^2(u)/4
        const float du2 = __builtin_fmaf(3.0f * 0.044715f * 1.59576912160573071f, s * s, 1.59576912160573071f);   // 2*u'
        const float tail = slope == 0.0f ? 0.0f : s * slope * du2;             // exactly 0 once |s| > ~6: no 0 * inf
        return g * (gate + tail);
    } else if constexpr (ACT == kSilu) {
        const float sg = sigmoid_f(s);                                                     // silu.py:56-57
        return g * (sg * (1.0f + s * (1.0f - sg)));
    } else if constexpr (ACT == kRelu) {
        return s > C(0) ? g : C(0);                                                        // relu.py:56
    } else if constexpr (ACT == kLeakyRelu) {
        return s > C(0) ? g : p0 * g;                                                      // leaky_relu.py:59
    } else if constexpr (ACT == kRelu6) {
        const C r = s > C(0) ? g : C(0);                                                   // relu6.py:57-58
        return s < C(6) ? r : C(0);
    } else if constexpr (ACT == kSigmoid) {
        return g * (s * (1.0f - s));                                                       // sigmoid.py:56
    } else if constexpr (ACT == kTanh) {
        return g * (1.0f - s * s);                                                         // tanh.py:58
    } else if constexpr (ACT == kMish) {
        const MishParts m = mish_parts(s);                                                 // mish.py:60-66
        return g * (m.t + s * m.one_minus_t2 * m.sig);
    } else if constexpr (ACT == kSoftplus) {
        if constexpr (std::is_same<C, float>::value) {                                     // softplus.py:62
            const float k = p0 * -1.44269504088896341f;
            return s * p0 > p1 ? g : g * rcp_fast(1.0f + __builtin_amdgcn_exp2f(k * s));
        } else {
            return s * p0 > p1 ? g : g / (C(1) + exp_c(-p0 * s));
        }
    } else {
        return s > p0 ? g : C(0);                                                          // threshold.py:59
    }
}

}  // namespace thn
