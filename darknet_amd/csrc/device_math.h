/*
 * device_math.h - scalar device functions shared by every kernel: the activations and the
 * batch-norm tail, spelled so that they round exactly as the reference's CPU forms do.
 *
 * The reference writes its activations with double literals (`.1*x`, `1./(1. + exp(-x))`,
 * src/activations.h:31-52), so C promotes to double and rounds once on return; the same is
 * done here.  normalize_cpu divides a float numerator by a double denominator
 * (src/blas.c:154); the kernels multiply by the double reciprocal instead, which rounds to
 * the same float except for a ~1e-8 fraction of double-rounding ties.
 */
#ifndef DN_DEVICE_MATH_H
#define DN_DEVICE_MATH_H

#include <hip/hip_runtime.h>

#include "darknet_hip.h"

__device__ __forceinline__ float dn_activate(float x, int a)
{
    const double xd = (double)x;
    switch (a) {
    case DN_LOGISTIC: return (float)(1. / (1. + exp((double)(-x))));
    case DN_RELU: return x * (float)(x > 0);
    case DN_RELIE: return (x > 0) ? x : (float)(.01 * xd);
    case DN_LINEAR: return x;
    case DN_RAMP: return (float)((double)(x * (float)(x > 0)) + .1 * xd);
    case DN_TANH: {
        const double e = exp((double)(2 * x));
        return (float)((e - 1) / (e + 1));
    }
    case DN_PLSE:
        if (x < -4) return (float)(.01 * (double)(x + 4));
        if (x > 4) return (float)(.01 * (double)(x - 4) + 1);
        return (float)(.125 * xd + .5);
    case DN_LEAKY: return (x > 0) ? x : (float)(.1 * xd);
    case DN_ELU: return (float)((double)((float)(x >= 0) * x) + (x < 0) * (exp(xd) - 1));
    case DN_LOGGY: return (float)(2. / (1. + exp((double)(-x))) - 1);
    case DN_STAIR: {
        const int n = (int)floor(xd);
        if (n % 2 == 0) return (float)floor(xd / 2.);
        return (float)((double)(x - n) + floor(xd / 2.));
    }
    case DN_HARDTAN:
        if (x < -1) return -1;
        if (x > 1) return 1;
        return x;
    case DN_LHTAN:
        if (x < 0) return (float)(.001 * xd);
        if (x > 1) return (float)(.001 * (double)(x - 1) + 1);
        return x;
    case DN_SELU:
        return (float)((x >= 0) * 1.0507 * xd + (x < 0) * 1.0507 * 1.6732 * (exp(xd) - 1));
    default: return 0;
    }
}

/* The logistic of the yolo head in single precision: 1 / (1 + exp(-x)) with a correctly rounded
 * float exponential and a hardware reciprocal.  Its distance from the reference's double
 * evaluation rounded to float (src/activations.h:32) stays below 3e-7 absolute over the whole
 * range (the function is bounded by 1 and its slope by 1/4), inside the 1e-6 the yolo planes are
 * held to, at a tenth of the instructions of the double form: that form made the yolo kernel
 * compute-bound at a third of the memory rate. */
__device__ __forceinline__ float dn_logistic_fast(float x)
{
    return __fdividef(1.f, 1.f + expf(-x));
}

/* Compile-time activation for the fused epilogues (the switch folds away). */
template <int A>
__device__ __forceinline__ float dn_activate_t(float x)
{
    return dn_activate(x, A);
}

/* Per-filter constants of the inference batch-norm tail. */
struct dn_bn_row {
    double inv_denom; /* 1 / (sqrt(var) + 1e-6f), in double */
    float mean;
    float scale;
    float bias;
    float pad_;
};

__device__ __forceinline__ dn_bn_row dn_bn_make(int bn, float bias, float scale, float mean,
                                                float var)
{
    dn_bn_row r;
    r.bias = bias;
    r.pad_ = 0.f;
    if (bn) {
        r.inv_denom = 1.0 / (sqrt((double)var) + (double).000001f);
        r.mean = mean;
        r.scale = scale;
    } else {
        r.inv_denom = 1.0;
        r.mean = 0.f;
        r.scale = 1.f;
    }
    return r;
}

/* normalize -> scale -> bias with a rounding to float after each step, as
 * normalize_cpu / scale_bias / add_bias do in sequence (src/batchnorm_layer.c:151-154). */
__device__ __forceinline__ float dn_bn_apply(float acc, const dn_bn_row &r, int bn)
{
    float x = acc;
    if (bn) {
        const float num = __fsub_rn(x, r.mean);
        x = (float)((double)num * r.inv_denom);
        x = __fmul_rn(x, r.scale);
    }
    return __fadd_rn(x, r.bias);
}

/* A double constant as an unevaluated sum of two floats: fmaf(x, hi, x*lo) reproduces
 * (float)((double)x * c) except when the exact product lies within ~2^-48 (relative) of a float
 * rounding boundary, at a third of the instructions of the convert / multiply / convert sequence. */
struct dn_f2 {
    float hi, lo;
};

__host__ __device__ inline dn_f2 dn_split(double c)
{
    dn_f2 r;
    r.hi = (float)c;
    r.lo = (float)(c - (double)r.hi);
    return r;
}

__device__ __forceinline__ float dn_mul_f2(float x, dn_f2 c) { return fmaf(x, c.hi, __fmul_rn(x, c.lo)); }

/* Per-filter constants of the convolution tail in that form, and the tail itself: normalize
 * (src/blas.c:154, as a multiplication by the reciprocal of the double denominator), scale, bias
 * (src/batchnorm_layer.c:151-154), each step rounded to float as the reference's separate passes
 * do, then the activation y > 0 ? y : slope*y (leaky .1, linear 1, relu 0).  Without batch-norm the
 * constants are neutral and change no bit. */
struct dn_tail_row {
    dn_f2 inv;
    float mean, scale, bias;
};

__device__ __forceinline__ dn_tail_row dn_tail_make(int bn, float bias, float scale, float mean, float var)
{
    dn_tail_row r;
    r.bias = bias;
    if (bn) {
        r.inv = dn_split(1.0 / (sqrt((double)var) + (double).000001f));
        r.mean = mean;
        r.scale = scale;
    } else {
        r.inv.hi = 1.f;
        r.inv.lo = 0.f;
        r.mean = 0.f;
        r.scale = 1.f;
    }
    return r;
}

__device__ __forceinline__ float dn_tail(float acc, const dn_tail_row &row, dn_f2 slope)
{
    float x = dn_mul_f2(__fsub_rn(acc, row.mean), row.inv);
    x = __fadd_rn(__fmul_rn(x, row.scale), row.bias);
    return (x > 0) ? x : dn_mul_f2(x, slope);
}

#endif
