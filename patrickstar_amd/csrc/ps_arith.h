// Per-element arithmetic of the optimizer step: step constants and the two arithmetics (operator order, torch formula).
#ifndef PS_ARITH_H
#define PS_ARITH_H

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cmath>
#include <cstdint>
#include <cstring>

#include "ps_adam.h"

namespace {

// ------------------------------------------------------------ device math

enum WdMode { WD_NONE = 0, WD_L2 = 1, WD_DECOUPLED = 2 };
enum Unscale { UNSCALE_NONE = 0, UNSCALE_DIV = 1, UNSCALE_MUL = 2 };
constexpr int UNSCALE_RUNTIME = -1;  // template value: look at StepConsts::unscale (uniform branch)

// Per-launch constants (cpu_adam.cpp:39-46 and the SIMD_SET block at :55-77).
//
// The reference calls the operator once per tensor with the same step number, and
// Adam_Optimizer::IncrementStep (cpu_adam.h:143-162) lets only the FIRST call of a step continue the
// running float product beta^t; every later call of the step evaluates pow.  The two bias-correction
// scalars therefore exist twice: step_size / bc2inv for every call after the first, first_step_size /
// first_bc2inv for the elements of the first call's tensor (FirstCall below says which those are).
struct StepConsts {
    float beta1, beta2, b1m, b2m, bc2inv, eps, step_size, wd_term;
    float first_step_size, first_bc2inv;
    float scale;  // loss scale (UNSCALE_DIV) or its exact reciprocal (UNSCALE_MUL)
    float clip;   // element-wise clamp bound of the fp16 gradients (an fp16-representable value); 0 = off
    int wd_mode;
    int unscale;
};

// binary32 -> nearest binary16 (ties to even), returned as binary32.  Bit-level so that host and
// device agree; inputs here are positive and at most 65504.
__host__ __device__ inline float round_to_half_precision(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t e = (x >> 23) & 0xFFu;
    if (e >= 255 || f == 0.0f) return f;
    // bits of the float mantissa that do not fit: 13 for a normal half, more below 2^-14
    int drop = e >= 113 ? 13 : (13 + (113 - (int)e));
    if (drop >= 25) return 0.0f;
    uint32_t m = (x & 0x7FFFFFu) | 0x800000u;
    uint32_t rem = m & ((1u << drop) - 1u), half = 1u << (drop - 1);
    m >>= drop;
    if (rem > half || (rem == half && (m & 1u))) m += 1;
    // value = m * 2^(e - 150 + drop)
    float r = (float)m;
    int shift = (int)e - 150 + drop;
    uint32_t sbits = (uint32_t)(shift + 127) << 23;
    float scale2;
    memcpy(&scale2, &sbits, 4);
    r = r * scale2;
    return (x >> 31) ? -r : r;
}

// The bound of the reference's element-wise "gradient clipping" (fp16_cpu_adam.py:364-379, GPU
// branch): min(65504, clipping * loss_scale) as a Python float, handed to Tensor.clamp_ on an fp16
// tensor, i.e. narrowed double -> float -> half.  0 when clipping is off.
// For a binary32 gradient tensor (grad_f32) the bound narrows to float only.
__host__ __device__ inline float clamp_bound(double clipping, double loss_scale, bool grad_f32 = false)
{
    if (!(clipping > 0.0)) return 0.0f;
    double c = clipping;
    if (loss_scale > 0.0) c = c * loss_scale;
    if (65504.0 < c) c = 65504.0;
    return grad_f32 ? (float)c : round_to_half_precision((float)c);
}

// A power-of-two scale 2^k with 2^-k a normal float: g/scale == g*(1/scale)
// bit for bit (the quotient is the same exact real number before the single
// rounding), so the 10-instruction IEEE divide can become one multiply.
__host__ __device__ inline bool exact_reciprocal(float s, float* inv)
{
    uint32_t b;
    memcpy(&b, &s, 4);
    uint32_t e = (b >> 23) & 0xFFu;
    if ((b & 0x807FFFFFu) != 0 || e < 1 || e > 253) return false;
    uint32_t r = (254u - e) << 23;
    memcpy(inv, &r, 4);
    return true;
}

// cpu_adam.h:170-174 and cpu_adam.cpp:44: the two scalars that depend on beta^t.
__host__ __device__ inline void bias_scalars(float lr, float beta1_t, float beta2_t, bool bias_correction,
                                             float* step_size, float* bc2inv_out)
{
    float bc1 = 1.0f, bc2inv = 1.0f;
    if (bias_correction) {
        bc1 = 1.0f - beta1_t;
        bc2inv = 1.0f / sqrtf(1.0f - beta2_t);
    }
    *step_size = (-1.0f * lr) / bc1;
    *bc2inv_out = bc2inv;
}

// beta1_t / beta2_t: beta^t of the call(s) the constants are for.  The first call's pair is set to the same
// values; a caller whose step has a first call with another beta^t overwrites it (bias_scalars).
__host__ __device__ inline void finish_consts(StepConsts& c, float lr, float beta1, float beta2,
                                              float eps, float wd, bool adamw, float beta1_t,
                                              float beta2_t, bool bias_correction, float loss_scale, float clip)
{
    c.clip = clip;
    float bc2inv;
    bias_scalars(lr, beta1_t, beta2_t, bias_correction, &c.step_size, &bc2inv);
    c.first_step_size = c.step_size;
    c.first_bc2inv = bc2inv;
    c.beta1 = beta1;
    c.beta2 = beta2;
    c.b1m = 1.0f - beta1;
    c.b2m = 1.0f - beta2;
    c.bc2inv = bc2inv;
    c.eps = eps;
    c.wd_mode = wd > 0.0f ? (adamw ? WD_DECOUPLED : WD_L2) : WD_NONE;
    c.wd_term = adamw ? (-1.0f * lr) * wd : wd;
    c.unscale = UNSCALE_NONE;
    c.scale = 1.0f;
    if (loss_scale > 0.0f) {
        float inv;
        if (exact_reciprocal(loss_scale, &inv)) {
            c.unscale = UNSCALE_MUL;
            c.scale = inv;
        } else {
            c.unscale = UNSCALE_DIV;
            c.scale = loss_scale;
        }
    }
}

// The constants of FP16Adam.torch_adam_update (fp16_cpu_adam.py:245-277,412-413) as torch's GPU
// kernels see them: every Python double is narrowed to float where a kernel takes it as a scalar;
// `tensor / python_scalar` multiplies by the reciprocal formed in binary64 and then narrowed.
// bc1, bc2 are the binary64 bias corrections 1 - beta ** step.
__host__ __device__ inline void torch_consts(StepConsts& c, double lr, double beta1, double beta2,
                                             double eps, double wd, bool adamw, double bc1,
                                             double bc2, double loss_scale, float clip)
{
    c.clip = clip;
    c.beta1 = (float)beta1;          // exp_avg.mul_(beta1)
    c.beta2 = (float)beta2;          // exp_avg_sq.mul_(beta2)
    c.b1m = (float)(1.0 - beta1);    // .add_(grad, alpha=1 - beta1)
    c.b2m = (float)(1.0 - beta2);    // .addcmul_(grad, grad, value=1 - beta2)
    c.bc2inv = (float)(1.0 / sqrt(bc2));  // exp_avg_sq.sqrt() / math.sqrt(bias_correction2)
    c.eps = (float)eps;              // .add_(eps)
    c.step_size = (float)(-(lr / bc1));   // addcdiv_(..., value=-step_size)
    c.first_step_size = c.step_size;      // Python forms these per tensor from the same step: no first-call form
    c.first_bc2inv = c.bc2inv;
    c.wd_mode = wd != 0.0 ? (adamw ? WD_DECOUPLED : WD_L2) : WD_NONE;
    c.wd_term = adamw ? (float)(1.0 - lr * wd)  // data.mul_(1 - lr * weight_decay)
                      : (float)wd;              // grad.add(data, alpha=weight_decay)
    c.unscale = UNSCALE_NONE;
    c.scale = 1.0f;
    if (loss_scale > 0.0) {          // grad.div_(loss_scale)
        c.unscale = UNSCALE_MUL;
        c.scale = (float)(1.0 / loss_scale);
    }
}

// step_size / bc2inv are arguments of their own: the caller picks the first call's pair or the later calls'.
template <int ARITH, int WD, int UNS>
__device__ __forceinline__ void adam_element(const StepConsts& c, float step_size, float bc2inv, float g,
                                             float& p, float& m, float& v)
{
    // element-wise clamp of the fp16 gradient (comparisons, so a NaN stays a NaN like Tensor.clamp_)
    if (c.clip > 0.0f) g = g < -c.clip ? -c.clip : (g > c.clip ? c.clip : g);
    if (UNS == UNSCALE_DIV) g = g / c.scale;
    if (UNS == UNSCALE_MUL) g = g * c.scale;
    if (ARITH == PS_ARITH_OPERATOR) {
        // Adam_Optimizer::Step, cpu_adam.cpp:91-141
        if (WD == WD_L2) g = __builtin_fmaf(p, c.wd_term, g);
        m = m * c.beta1;
        m = __builtin_fmaf(g, c.b1m, m);
        v = v * c.beta2;
        float gg = g * g;
        v = __builtin_fmaf(gg, c.b2m, v);
        float d = __builtin_sqrtf(v);
        d = __builtin_fmaf(d, bc2inv, c.eps);
        float u = m / d;
        if (WD == WD_DECOUPLED) p = __builtin_fmaf(p, c.wd_term, p);
        p = __builtin_fmaf(u, step_size, p);
    } else {
        // FP16Adam.torch_adam_update, fp16_cpu_adam.py:259-277, one torch kernel per line
        if (WD == WD_DECOUPLED) p = p * c.wd_term;             // data.mul_(1 - lr * wd)
        if (WD == WD_L2) g = __builtin_fmaf(p, c.wd_term, g);  // grad.add(data, alpha=wd)
        m = m * c.beta1;                                       // exp_avg.mul_(beta1)
        m = __builtin_fmaf(g, c.b1m, m);                       //   .add_(grad, alpha=1 - beta1)
        v = v * c.beta2;                                       // exp_avg_sq.mul_(beta2)
        float gg = g * g;
        v = __builtin_fmaf(c.b2m, gg, v);                      //   .addcmul_(grad, grad, value=1 - beta2)
        float d = __builtin_sqrtf(v);                          // exp_avg_sq.sqrt()
        d = d * bc2inv;                                        //   / math.sqrt(bias_correction2)
        d = d + c.eps;                                         //   .add_(eps)
        float q = m / d;
        p = __builtin_fmaf(step_size, q, p);                   // data.addcdiv_(exp_avg, denom, value=-step_size)
    }
}

template <int ARITH, int WD, int UNS>
__device__ __forceinline__ void element_any(const StepConsts& c, float step_size, float bc2inv, float g,
                                            float& p, float& m, float& v)
{
    if (UNS != UNSCALE_RUNTIME)
        adam_element<ARITH, WD, UNS>(c, step_size, bc2inv, g, p, m, v);
    else if (c.unscale == UNSCALE_MUL)
        adam_element<ARITH, WD, UNSCALE_MUL>(c, step_size, bc2inv, g, p, m, v);
    else if (c.unscale == UNSCALE_DIV)
        adam_element<ARITH, WD, UNSCALE_DIV>(c, step_size, bc2inv, g, p, m, v);
    else
        adam_element<ARITH, WD, UNSCALE_NONE>(c, step_size, bc2inv, g, p, m, v);
}

// Which elements of a launch belong to the step's first operator call: elements [lo, hi) of chunk
// `chunk` of the launch's batch (-1: none of them).
struct FirstCall {
    int chunk;
    uint64_t lo, hi;
};

__device__ __forceinline__ float half_bits_to_float(uint32_t h)
{
    return __half2float(__ushort_as_half((unsigned short)h));
}

// RNE binary32 -> binary16 of a value that has ALREADY been rounded to binary32.
// The empty asm makes the float opaque at this point: without it the compiler
// folds "convert(fma(a, b, c))" into v_fma_mixlo_f16, which rounds the exact
// fused result straight to fp16 and so differs from RNE(fp32 param) on about
// one element in 10^4 (double-rounding cases).
__device__ __forceinline__ uint32_t float_to_half_bits(float f)
{
    asm("" : "+v"(f));
    return (uint32_t)__half_as_ushort(__float2half_rn(f));
}

}  // namespace

#endif  // PS_ARITH_H
