// Elementwise operation table: one functor per agmi_op, shared by the map kernels
// (elementwise.hip) and the map-reduce kernels (reduce.hip).
//
// Each functor states its arity and computes one point from its inputs.  Fused derivative
// rules keep the operation order of the reference rule they replace (cited in agmi.h) so
// that results differ from NumPy's only by the last-bit behaviour of transcendental
// functions; the library is compiled with -ffp-contract=off so products and sums are not
// fused into FMAs that NumPy would not perform.
#pragma once

#include <hip/hip_runtime.h>

#include "agmi.h"

namespace agmi {

// math on T in {float, double}.  The long library routines are inlined into the one-rule kernels; a
// translation unit that holds many of them in one kernel (the program interpreter) defines
// AGMI_HEAVY_MATH as `static __device__ __noinline__` before including this file, so that each is one
// function called element by element and its temporaries do not add to the kernel's register budget.
#ifndef AGMI_HEAVY_MATH
#define AGMI_HEAVY_MATH __device__ __forceinline__
#endif
AGMI_HEAVY_MATH float m_exp(float x) { return expf(x); }
AGMI_HEAVY_MATH double m_exp(double x) { return exp(x); }
// exp(d) for d <= 0 (an element minus the logsumexp of its row) to within 1 ulp of expf, without the
// overflow handling: d*log2(e) is split into an integer n and a remainder whose rounding error is
// recovered with fused multiply-adds (log2(e) as a float pair), the hardware exp2 sees |r| <= 1/2,
// and ldexp scales, also into the subnormals.  n is clamped so that d = -inf (and anything whose exp
// underflows) arrives at exp2(-inf) = 0 and d = +inf (a weighted logsumexp whose maximum is infinite is shifted
// by 0, not by its maximum) at inf; a NaN passes through the clamp's other operand into the fma.
AGMI_HEAVY_MATH float exp_of_nonpositive(float d) {
    const float kLog2eHi = 1.44269502162933349609375f, kLog2eLo = 1.92596299112661746e-8f;
    const float n = fminf(fmaxf(rintf(d * kLog2eHi), -160.0f), 160.0f);  // (the upper clamp only matters for d = +inf: inf, not NaN)
    float r = __builtin_fmaf(d, kLog2eHi, -n);
    r = __builtin_fmaf(d, kLog2eLo, r);
    return ldexpf(__builtin_amdgcn_exp2f(r), static_cast<int>(n));
}
AGMI_HEAVY_MATH double exp_of_nonpositive(double d) { return exp(d); }
AGMI_HEAVY_MATH float m_log(float x) { return logf(x); }
AGMI_HEAVY_MATH double m_log(double x) { return log(x); }
AGMI_HEAVY_MATH float m_log1p(float x) { return log1pf(x); }
AGMI_HEAVY_MATH double m_log1p(double x) { return log1p(x); }
AGMI_HEAVY_MATH float m_expm1(float x) { return expm1f(x); }
AGMI_HEAVY_MATH double m_expm1(double x) { return expm1(x); }
AGMI_HEAVY_MATH float m_tanh(float x) { return tanhf(x); }
AGMI_HEAVY_MATH double m_tanh(double x) { return tanh(x); }
AGMI_HEAVY_MATH float m_sinh(float x) { return sinhf(x); }
AGMI_HEAVY_MATH double m_sinh(double x) { return sinh(x); }
AGMI_HEAVY_MATH float m_cosh(float x) { return coshf(x); }
AGMI_HEAVY_MATH double m_cosh(double x) { return cosh(x); }
AGMI_HEAVY_MATH float m_sin(float x) { return sinf(x); }
AGMI_HEAVY_MATH double m_sin(double x) { return sin(x); }
AGMI_HEAVY_MATH float m_cos(float x) { return cosf(x); }
AGMI_HEAVY_MATH double m_cos(double x) { return cos(x); }
__device__ __forceinline__ float m_sqrt(float x) { return sqrtf(x); }
__device__ __forceinline__ double m_sqrt(double x) { return sqrt(x); }
__device__ __forceinline__ float m_abs(float x) { return fabsf(x); }
__device__ __forceinline__ double m_abs(double x) { return fabs(x); }
AGMI_HEAVY_MATH float m_pow(float x, float y) { return powf(x, y); }
AGMI_HEAVY_MATH double m_pow(double x, double y) { return pow(x, y); }

AGMI_HEAVY_MATH float m_exp2(float x) { return exp2f(x); }
AGMI_HEAVY_MATH double m_exp2(double x) { return exp2(x); }
AGMI_HEAVY_MATH float m_log2(float x) { return log2f(x); }
AGMI_HEAVY_MATH double m_log2(double x) { return log2(x); }
AGMI_HEAVY_MATH float m_log10(float x) { return log10f(x); }
AGMI_HEAVY_MATH double m_log10(double x) { return log10(x); }
AGMI_HEAVY_MATH float m_tan(float x) { return tanf(x); }
AGMI_HEAVY_MATH double m_tan(double x) { return tan(x); }
AGMI_HEAVY_MATH float m_asin(float x) { return asinf(x); }
AGMI_HEAVY_MATH double m_asin(double x) { return asin(x); }
AGMI_HEAVY_MATH float m_acos(float x) { return acosf(x); }
AGMI_HEAVY_MATH double m_acos(double x) { return acos(x); }
AGMI_HEAVY_MATH float m_atan(float x) { return atanf(x); }
AGMI_HEAVY_MATH double m_atan(double x) { return atan(x); }
AGMI_HEAVY_MATH float m_asinh(float x) { return asinhf(x); }
AGMI_HEAVY_MATH double m_asinh(double x) { return asinh(x); }
AGMI_HEAVY_MATH float m_acosh(float x) { return acoshf(x); }
AGMI_HEAVY_MATH double m_acosh(double x) { return acosh(x); }
AGMI_HEAVY_MATH float m_atanh(float x) { return atanhf(x); }
AGMI_HEAVY_MATH double m_atanh(double x) { return atanh(x); }
AGMI_HEAVY_MATH float m_atan2(float y, float x) { return atan2f(y, x); }
AGMI_HEAVY_MATH double m_atan2(double y, double x) { return atan2(y, x); }
AGMI_HEAVY_MATH float m_hypot(float x, float y) { return hypotf(x, y); }
AGMI_HEAVY_MATH double m_hypot(double x, double y) { return hypot(x, y); }

// numpy.logaddexp (npy_math: equal operands -> x + log 2; otherwise the larger one plus log1p of
// the exponential of the negative distance; a NaN distance is returned as it is)
template <typename T>
__device__ __forceinline__ T logaddexp_like_numpy(T x, T y) {
    if (x == y) return x + T(0.693147180559945309417232121458176568);
    const T d = x - y;
    if (d > T(0)) return x + m_log1p(m_exp(-d));
    if (d <= T(0)) return y + m_log1p(m_exp(d));
    return d;
}

// numpy.logaddexp2 (npy_math): like logaddexp with exp2 and log1p scaled by log2(e)
template <typename T>
__device__ __forceinline__ T logaddexp2_like_numpy(T x, T y) {
    const T kLog2e = T(1.442695040888963407359924681001892137);
    if (x == y) return x + T(1);
    const T d = x - y;
    if (d > T(0)) return x + kLog2e * m_log1p(m_exp2(-d));
    if (d <= T(0)) return y + kLog2e * m_log1p(m_exp2(d));
    return d;
}

// numpy.remainder for floating point (npy_divmod): fmod, then moved by one divisor when its sign
// differs from the divisor's; an exact multiple gives a zero with the divisor's sign; b == 0 -> NaN.
AGMI_HEAVY_MATH float m_fmod(float a, float b) { return fmodf(a, b); }
AGMI_HEAVY_MATH double m_fmod(double a, double b) { return fmod(a, b); }
__device__ __forceinline__ float m_copysign(float a, float b) { return copysignf(a, b); }
__device__ __forceinline__ double m_copysign(double a, double b) { return copysign(a, b); }
template <typename T>
__device__ __forceinline__ T remainder_like_numpy(T a, T b) {
    T m = m_fmod(a, b);
    if (b == T(0)) return m;
    if (m != T(0)) {
        if ((b < T(0)) != (m < T(0))) m += b;
    } else {
        m = m_copysign(T(0), b);
    }
    return m;
}

// numpy.nan_to_num with its defaults: NaN -> 0, infinities -> the largest finite values
template <typename T>
__device__ __forceinline__ T nan_to_num_like_numpy(T x) {
    const T big = sizeof(T) == 4 ? T(__FLT_MAX__) : T(__DBL_MAX__);
    if (x != x) return T(0);
    if (x > big) return big;
    if (x < -big) return -big;
    return x;
}

// numpy.fmax / fmin: a NaN operand is ignored when the other one is a number
template <typename T>
__device__ __forceinline__ T fmax_like_numpy(T a, T b) {
    return (a >= b || b != b) ? a : b;
}
template <typename T>
__device__ __forceinline__ T fmin_like_numpy(T a, T b) {
    return (a <= b || b != b) ? a : b;
}

// x**y with the exponents NumPy short-cuts (1, 2, 0, -1, 0.5) computed the same exact way.
template <typename T>
__device__ __forceinline__ T pow_like_numpy(T x, T y) {
    if (y == T(2)) return x * x;
    if (y == T(1)) return x;
    if (y == T(0)) return T(1);
    if (y == T(-1)) return T(1) / x;
    if (y == T(0.5)) return m_sqrt(x);
    return m_pow(x, y);
}

// NumPy's maximum/minimum propagate NaN from either operand.
template <typename T>
__device__ __forceinline__ T max_nan(T a, T b) {
    return (a >= b || a != a) ? a : b;
}
template <typename T>
__device__ __forceinline__ T min_nan(T a, T b) {
    return (a <= b || a != a) ? a : b;
}

// ---- accumulators of the reductions (reduce.hip) and of the row reductions inside programs (program.hip) ----
template <typename T>
struct AccSum {
    typedef T type;
    __device__ __forceinline__ static T identity() { return T(0); }
    __device__ __forceinline__ static T lift(T v) { return v; }
    __device__ __forceinline__ static T combine(T a, T b) { return a + b; }
    __device__ __forceinline__ static T finish(T a) { return a; }
    __device__ __forceinline__ static T shfl_xor(T a, int m) { return __shfl_xor(a, m, 64); }
};
template <typename T>
struct AccProd : AccSum<T> {
    __device__ __forceinline__ static T identity() { return T(1); }
    __device__ __forceinline__ static T combine(T a, T b) { return a * b; }
};
template <typename T>
struct AccMax : AccSum<T> {
    __device__ __forceinline__ static T identity() { return -__builtin_huge_val(); }
    __device__ __forceinline__ static T combine(T a, T b) { return max_nan(a, b); }
};
template <typename T>
struct AccMin : AccSum<T> {
    __device__ __forceinline__ static T identity() { return __builtin_huge_val(); }
    __device__ __forceinline__ static T combine(T a, T b) { return min_nan(a, b); }
};

// log-sum-exp as an associative reduction over (m, s) with value = m + log(s),
// s = sum exp(x - m).  Infinite and equal maxima are combined without forming inf - inf.
template <typename T>
struct LsePair {
    T m, s;
};
template <typename T>
struct AccLse {
    typedef LsePair<T> type;
    __device__ __forceinline__ static type identity() { return {T(-__builtin_huge_val()), T(0)}; }
    __device__ __forceinline__ static type lift(T v) { return {v, T(1)}; }
    // value: the larger maximum, and its sum plus the other sum scaled by exp(difference of the maxima).  Written
    // with selects and one exp, not one branch per case: lanes of a wave disagree on which side is larger, and with
    // branches every step of a wave-wide reduction runs both exps one after the other.  Equal maxima (also both
    // infinite) scale by exp(0) = 1 exactly; a NaN maximum gives NaN for both members.
    __device__ __forceinline__ static type combine(type a, type b) {
        const bool a_larger = a.m >= b.m;
        const T hi_m = a_larger ? a.m : b.m, lo_m = a_larger ? b.m : a.m;
        const T hi_s = a_larger ? a.s : b.s, lo_s = a_larger ? b.s : a.s;
        const T d = (a.m == b.m) ? T(0) : lo_m - hi_m;
        const bool ordered = a.m == a.m && b.m == b.m;
        return {ordered ? hi_m : a.m + b.m, ordered ? hi_s + lo_s * m_exp(d) : a.s + b.s};
    }
    __device__ __forceinline__ static T finish(type a) {
        if (a.s == T(0) || a.m == T(__builtin_huge_val())) return a.m;  // all -inf, or a +inf present
        return a.m + m_log(a.s);
    }
    __device__ __forceinline__ static type shfl_xor(type a, int m) {
        return {__shfl_xor(a.m, m, 64), __shfl_xor(a.s, m, 64)};
    }
};


#define AGMI_FUNCTOR(NAME, N_IN, N_OUT, ...)                                      \
    template <typename T>                                                         \
    struct NAME {                                                                 \
        static constexpr int NIN = N_IN;                                          \
        static constexpr int NOUT = N_OUT;                                        \
        __device__ __forceinline__ static void apply(const T *x, T *o) { __VA_ARGS__ } \
    };

AGMI_FUNCTOR(FCopy, 1, 1, o[0] = x[0];)
AGMI_FUNCTOR(FNeg, 1, 1, o[0] = -x[0];)
AGMI_FUNCTOR(FExp, 1, 1, o[0] = m_exp(x[0]);)
AGMI_FUNCTOR(FLog, 1, 1, o[0] = m_log(x[0]);)
AGMI_FUNCTOR(FTanh, 1, 1, o[0] = m_tanh(x[0]);)
AGMI_FUNCTOR(FSinh, 1, 1, o[0] = m_sinh(x[0]);)
AGMI_FUNCTOR(FCosh, 1, 1, o[0] = m_cosh(x[0]);)
AGMI_FUNCTOR(FSin, 1, 1, o[0] = m_sin(x[0]);)
AGMI_FUNCTOR(FCos, 1, 1, o[0] = m_cos(x[0]);)
AGMI_FUNCTOR(FSqrt, 1, 1, o[0] = m_sqrt(x[0]);)
AGMI_FUNCTOR(FSquare, 1, 1, o[0] = x[0] * x[0];)
AGMI_FUNCTOR(FAbs, 1, 1, o[0] = m_abs(x[0]);)
AGMI_FUNCTOR(FSign, 1, 1, o[0] = x[0] > T(0) ? T(1) : (x[0] < T(0) ? T(-1) : x[0]);)
AGMI_FUNCTOR(FReciprocal, 1, 1, o[0] = T(1) / x[0];)
AGMI_FUNCTOR(FLog1p, 1, 1, o[0] = m_log1p(x[0]);)
AGMI_FUNCTOR(FExpm1, 1, 1, o[0] = m_expm1(x[0]);)

AGMI_FUNCTOR(FExp2, 1, 1, o[0] = m_exp2(x[0]);)
AGMI_FUNCTOR(FLog2, 1, 1, o[0] = m_log2(x[0]);)
AGMI_FUNCTOR(FLog10, 1, 1, o[0] = m_log10(x[0]);)
AGMI_FUNCTOR(FTan, 1, 1, o[0] = m_tan(x[0]);)
AGMI_FUNCTOR(FArcsin, 1, 1, o[0] = m_asin(x[0]);)
AGMI_FUNCTOR(FArccos, 1, 1, o[0] = m_acos(x[0]);)
AGMI_FUNCTOR(FArctan, 1, 1, o[0] = m_atan(x[0]);)
AGMI_FUNCTOR(FArcsinh, 1, 1, o[0] = m_asinh(x[0]);)
AGMI_FUNCTOR(FArccosh, 1, 1, o[0] = m_acosh(x[0]);)
AGMI_FUNCTOR(FArctanh, 1, 1, o[0] = m_atanh(x[0]);)

// rounding functions (no derivative, numpy_vjps.py:13-20)
AGMI_FUNCTOR(FFloor, 1, 1, o[0] = floor(x[0]);)
AGMI_FUNCTOR(FCeil, 1, 1, o[0] = ceil(x[0]);)
AGMI_FUNCTOR(FRint, 1, 1, o[0] = rint(x[0]);)
AGMI_FUNCTOR(FTrunc, 1, 1, o[0] = trunc(x[0]);)
AGMI_FUNCTOR(FNanToNum, 1, 1, o[0] = nan_to_num_like_numpy(x[0]);)

AGMI_FUNCTOR(FAdd, 2, 1, o[0] = x[0] + x[1];)
AGMI_FUNCTOR(FSub, 2, 1, o[0] = x[0] - x[1];)
AGMI_FUNCTOR(FMul, 2, 1, o[0] = x[0] * x[1];)
AGMI_FUNCTOR(FDiv, 2, 1, o[0] = x[0] / x[1];)
AGMI_FUNCTOR(FPow, 2, 1, o[0] = pow_like_numpy(x[0], x[1]);)
AGMI_FUNCTOR(FMaximum, 2, 1, o[0] = max_nan(x[0], x[1]);)
AGMI_FUNCTOR(FMinimum, 2, 1, o[0] = min_nan(x[0], x[1]);)

AGMI_FUNCTOR(FFmax, 2, 1, o[0] = fmax_like_numpy(x[0], x[1]);)
AGMI_FUNCTOR(FFmin, 2, 1, o[0] = fmin_like_numpy(x[0], x[1]);)
AGMI_FUNCTOR(FArctan2, 2, 1, o[0] = m_atan2(x[0], x[1]);)
AGMI_FUNCTOR(FHypot, 2, 1, o[0] = m_hypot(x[0], x[1]);)
AGMI_FUNCTOR(FLogaddexp, 2, 1, o[0] = logaddexp_like_numpy(x[0], x[1]);)
AGMI_FUNCTOR(FRemainder, 2, 1, o[0] = remainder_like_numpy(x[0], x[1]);)
AGMI_FUNCTOR(FLogaddexp2, 2, 1, o[0] = logaddexp2_like_numpy(x[0], x[1]);)

AGMI_FUNCTOR(FWhere, 3, 1, o[0] = (x[0] != T(0)) ? x[1] : x[2];)

// (g, x, y): -g * x / y**2
AGMI_FUNCTOR(FDivVjp1, 3, 1, o[0] = ((-x[0]) * x[1]) / (x[2] * x[2]);)
// (g, x): g / cosh(x)**2
AGMI_FUNCTOR(FTanhVjp, 2, 1, T c = m_cosh(x[1]); o[0] = x[0] / (c * c);)
// (g, x, y): g * y * x**where(y, y - 1, 1)
AGMI_FUNCTOR(FPowVjp0, 3, 1, T e = (x[2] != T(0)) ? x[2] - T(1) : T(1);
             o[0] = (x[0] * x[2]) * pow_like_numpy(x[1], e);)
// (g, x, ans): g * log(where(x, x, 1)) * ans
AGMI_FUNCTOR(FPowVjp1, 3, 1, T b = (x[1] != T(0)) ? x[1] : T(1); o[0] = (x[0] * m_log(b)) * x[2];)
// (g, b, x, ans): g * b * exp(x - ans)
AGMI_FUNCTOR(FLseVjp, 4, 1, o[0] = (x[0] * x[1]) * exp_of_nonpositive(x[2] - x[3]);)
// (g, x): -g / x**2
AGMI_FUNCTOR(FReciprocalVjp, 2, 1, o[0] = (-x[0]) / (x[1] * x[1]);)
// (g, x): g * 0.5 * x**-0.5
AGMI_FUNCTOR(FSqrtVjp, 2, 1, o[0] = (x[0] * T(0.5)) * m_pow(x[1], T(-0.5));)
AGMI_FUNCTOR(FSinVjp, 2, 1, o[0] = x[0] * m_cos(x[1]);)
AGMI_FUNCTOR(FCosVjp, 2, 1, o[0] = (-x[0]) * m_sin(x[1]);)
AGMI_FUNCTOR(FSinhVjp, 2, 1, o[0] = x[0] * m_cosh(x[1]);)
AGMI_FUNCTOR(FCoshVjp, 2, 1, o[0] = x[0] * m_sinh(x[1]);)
AGMI_FUNCTOR(FSquareVjp, 2, 1, o[0] = (x[0] * T(2)) * x[1];)
// (g, x, ans): g * where(x, x, 0) / where(ans, ans, 1)
AGMI_FUNCTOR(FAbsVjp, 3, 1, T d = (x[2] != T(0)) ? x[2] : T(1); o[0] = (x[0] * x[1]) / d;)
// (g, x, ans, y): g * ((x == ans) / (1 + (x == y)))
AGMI_FUNCTOR(FChooseVjp, 4, 1, T num = (x[1] == x[2]) ? T(1) : T(0); T den = (x[1] == x[3]) ? T(2) : T(1);
             o[0] = x[0] * (num / den);)
AGMI_FUNCTOR(FLog1pVjp, 2, 1, o[0] = x[0] / (x[1] + T(1));)
AGMI_FUNCTOR(FExpm1Vjp, 2, 1, o[0] = (x[1] + T(1)) * x[0];)
// (g, x, y) -> g / y, -g * x / y**2
AGMI_FUNCTOR(FDivVjpBoth, 3, 2, o[0] = x[0] / x[2]; o[1] = ((-x[0]) * x[1]) / (x[2] * x[2]);)
// (a, x, y): a * x + y, two roundings
AGMI_FUNCTOR(FMulAdd, 3, 1, T t = x[0] * x[1]; o[0] = t + x[2];)
// (x, y): astype(x == y, dtype)
AGMI_FUNCTOR(FEqualAsFloat, 2, 1, o[0] = (x[0] == x[1]) ? T(1) : T(0);)
// (g, x, ans, n): g * astype(x == ans, dtype) / n
AGMI_FUNCTOR(FExtremumVjp, 4, 1, o[0] = (x[0] * ((x[1] == x[2]) ? T(1) : T(0))) / x[3];)

// two rules in one program instruction, each rounded on its own
AGMI_FUNCTOR(FMulMul, 3, 1, T t = x[0] * x[1]; o[0] = t * x[2];)
AGMI_FUNCTOR(FMulSub, 3, 1, T t = x[0] * x[1]; o[0] = t - x[2];)
AGMI_FUNCTOR(FMulRsub, 3, 1, T t = x[0] * x[1]; o[0] = x[2] - t;)
AGMI_FUNCTOR(FAddMul, 3, 1, T t = x[0] + x[1]; o[0] = t * x[2];)
AGMI_FUNCTOR(FSubMul, 3, 1, T t = x[0] - x[1]; o[0] = t * x[2];)
#define AGMI_FOR_EACH_CHAINED_OP(X)   \
    X(AGMI_OP_MUL_MUL, FMulMul)       \
    X(AGMI_OP_MUL_SUB, FMulSub)       \
    X(AGMI_OP_MUL_RSUB, FMulRsub)     \
    X(AGMI_OP_ADD_MUL, FAddMul)       \
    X(AGMI_OP_SUB_MUL, FSubMul)

// X(op enum, functor): the operations with one result (what an elementwise program may contain)
#define AGMI_FOR_EACH_PROGRAM_OP(X)             \
    X(AGMI_OP_COPY, FCopy)                      \
    X(AGMI_OP_NEG, FNeg)                        \
    X(AGMI_OP_EXP, FExp)                        \
    X(AGMI_OP_LOG, FLog)                        \
    X(AGMI_OP_TANH, FTanh)                      \
    X(AGMI_OP_SINH, FSinh)                      \
    X(AGMI_OP_COSH, FCosh)                      \
    X(AGMI_OP_SIN, FSin)                        \
    X(AGMI_OP_COS, FCos)                        \
    X(AGMI_OP_SQRT, FSqrt)                      \
    X(AGMI_OP_SQUARE, FSquare)                  \
    X(AGMI_OP_ABS, FAbs)                        \
    X(AGMI_OP_SIGN, FSign)                      \
    X(AGMI_OP_RECIPROCAL, FReciprocal)          \
    X(AGMI_OP_LOG1P, FLog1p)                    \
    X(AGMI_OP_EXPM1, FExpm1)                    \
    X(AGMI_OP_EXP2, FExp2)                      \
    X(AGMI_OP_LOG2, FLog2)                      \
    X(AGMI_OP_LOG10, FLog10)                    \
    X(AGMI_OP_TAN, FTan)                        \
    X(AGMI_OP_ARCSIN, FArcsin)                  \
    X(AGMI_OP_ARCCOS, FArccos)                  \
    X(AGMI_OP_ARCTAN, FArctan)                  \
    X(AGMI_OP_ARCSINH, FArcsinh)                \
    X(AGMI_OP_ARCCOSH, FArccosh)                \
    X(AGMI_OP_ARCTANH, FArctanh)                \
    X(AGMI_OP_FLOOR, FFloor)                    \
    X(AGMI_OP_CEIL, FCeil)                      \
    X(AGMI_OP_RINT, FRint)                      \
    X(AGMI_OP_TRUNC, FTrunc)                    \
    X(AGMI_OP_ADD, FAdd)                        \
    X(AGMI_OP_SUB, FSub)                        \
    X(AGMI_OP_MUL, FMul)                        \
    X(AGMI_OP_DIV, FDiv)                        \
    X(AGMI_OP_POW, FPow)                        \
    X(AGMI_OP_MAXIMUM, FMaximum)                \
    X(AGMI_OP_MINIMUM, FMinimum)                \
    X(AGMI_OP_FMAX, FFmax)                      \
    X(AGMI_OP_FMIN, FFmin)                      \
    X(AGMI_OP_ARCTAN2, FArctan2)                \
    X(AGMI_OP_HYPOT, FHypot)                    \
    X(AGMI_OP_LOGADDEXP, FLogaddexp)            \
    X(AGMI_OP_REMAINDER, FRemainder)            \
    X(AGMI_OP_LOGADDEXP2, FLogaddexp2)          \
    X(AGMI_OP_NAN_TO_NUM, FNanToNum)            \
    X(AGMI_OP_WHERE, FWhere)                    \
    X(AGMI_OP_DIV_VJP1, FDivVjp1)               \
    X(AGMI_OP_TANH_VJP, FTanhVjp)               \
    X(AGMI_OP_POW_VJP0, FPowVjp0)               \
    X(AGMI_OP_POW_VJP1, FPowVjp1)               \
    X(AGMI_OP_LSE_VJP, FLseVjp)                 \
    X(AGMI_OP_RECIPROCAL_VJP, FReciprocalVjp)   \
    X(AGMI_OP_SQRT_VJP, FSqrtVjp)               \
    X(AGMI_OP_SIN_VJP, FSinVjp)                 \
    X(AGMI_OP_COS_VJP, FCosVjp)                 \
    X(AGMI_OP_SINH_VJP, FSinhVjp)               \
    X(AGMI_OP_COSH_VJP, FCoshVjp)               \
    X(AGMI_OP_SQUARE_VJP, FSquareVjp)           \
    X(AGMI_OP_ABS_VJP, FAbsVjp)                 \
    X(AGMI_OP_CHOOSE_VJP, FChooseVjp)           \
    X(AGMI_OP_LOG1P_VJP, FLog1pVjp)             \
    X(AGMI_OP_EXPM1_VJP, FExpm1Vjp)             \
    X(AGMI_OP_MUL_ADD, FMulAdd)                 \
    X(AGMI_OP_EQUAL_AS_FLOAT, FEqualAsFloat)    \
    X(AGMI_OP_EXTREMUM_VJP, FExtremumVjp)

// every operation of agmi_elementwise
#define AGMI_FOR_EACH_OP(X)        \
    AGMI_FOR_EACH_PROGRAM_OP(X)    \
    X(AGMI_OP_DIV_VJP_BOTH, FDivVjpBoth)

}  // namespace agmi
