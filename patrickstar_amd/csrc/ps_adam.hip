// Chunk-wise mixed-precision Adam step for MI355X (gfx950, wave64).
//
// Everything here is HBM-bandwidth bound: 28 bytes move per element per step
// (read fp16 grad + fp32 param/m/v, write fp32 param/m/v + fp16 param) for
// ~20 flops.  No matrix cores are involved.  What the kernels are organised
// around, all of it measured on MI355X:
//   * one pass over the data, in place; per lane one 16-byte access to each
//     fp32 array and one 8-byte access to the fp16 array, so that every wave
//     instruction covers a contiguous span of whole cache lines;
//   * one small tile (256 elements) per single-wave workgroup and a CAP on
//     resident workgroups (9 per CU, enforced by requesting 17 KiB of unused
//     dynamic LDS): the pass touches four arrays for reading and the same four
//     for writing, and HBM efficiency drops when the set of in-flight cache
//     lines gets wide; a narrow, steadily advancing window per array gave
//     6.3 TB/s where the fully occupied machine gave 5.3 TB/s (a plain
//     1-read-1-write copy peaks at 6.2-6.3 TB/s on the same GPU);
//   * chunk descriptors travel in the kernel-argument segment (64 per launch),
//     so a wave's first data load depends on one scalar load, not two;
//   * plain (temporal) loads/stores: non-temporal loads cost 6 % at this
//     operating point (20-25 % with fully occupied CUs), non-temporal stores
//     change nothing.
//
// Arithmetic contract (bit-exact with the explicit-intrinsic body of the
// reference operator, patrickstar/ops/csrc/adam/cpu_adam.cpp:91-141): every
// a*b+c the reference writes as SIMD_FMA is one __builtin_fmaf; every other
// operation is an individually rounded IEEE binary32 op.  The file must be
// compiled with -ffp-contract=off and with correctly rounded fp32 divide and
// sqrt (hipcc's default), denormals preserved.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <memory>
#include <mutex>
#include <unordered_map>

#include "ps_adam.h"

// Build-time tuning knobs of the fused Adam kernels (defaults = measured best).
#ifndef PS_BLOCK
#define PS_BLOCK 64  // threads per workgroup
#endif
#ifndef PS_LANE_ELEMS
#define PS_LANE_ELEMS 4  // elements per lane per vector step (4 or 8)
#endif
#ifndef PS_UNROLL
#define PS_UNROLL 1  // vector steps per lane per tile
#endif
#ifndef PS_MAX_WAVES_PER_EU
#define PS_MAX_WAVES_PER_EU 0  // cap on resident waves per SIMD (0: no cap; the LDS request below does the capping)
#endif
#ifndef PS_LDS_KB
#define PS_LDS_KB 17  // KiB of (unused) dynamic LDS requested per workgroup: caps resident workgroups per CU at floor(160 / PS_LDS_KB) = 9
#endif
#ifndef PS_STREAMING
#define PS_STREAMING 0  // bit 0: non-temporal loads, bit 1: non-temporal stores of chunk payloads (both slower on MI355X)
#endif
#if PS_MAX_WAVES_PER_EU > 0
#define PS_OCCUPANCY __attribute__((amdgpu_waves_per_eu(1, PS_MAX_WAVES_PER_EU)))
#else
#define PS_OCCUPANCY
#endif

namespace {

// ------------------------------------------------------------------ errors

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char* what)
{
    return fail(-(int)e, "%s: %s", what, hipGetErrorString(e));
}

#define PS_HIP(call)                                      \
    do {                                                  \
        hipError_t e_ = (call);                           \
        if (e_ != hipSuccess) return hip_fail(e_, #call); \
    } while (0)

// ------------------------------------------------------- host scalar state
//
// One object per optimizer id: the float scalars the reference keeps in
// Adam_Optimizer (cpu_adam.h:177-197) and their update rules.

struct HostAdam {
    float alpha, beta1, beta2, eps, weight_decay;
    float beta1_t = 1.0f, beta2_t = 1.0f;
    size_t step = 0;
    bool adamw;
    double grad_clamp = -1.0;  // FP16Adam.gradient_clipping; <= 0: off
    int arith = PS_ARITH_OPERATOR;  // arithmetic for chunks updated in place in HBM

    // cpu_adam.h:143-162
    void advance(size_t s, float b1, float b2)
    {
        if (b1 != beta1 || b2 != beta2) {
            step = s;
            beta1 = b1;
            beta2 = b2;
            beta1_t = (float)std::pow((double)b1, (double)s);
            beta2_t = (float)std::pow((double)b2, (double)s);
            return;
        }
        step += 1;
        if (step != s) {
            beta1_t = (float)std::pow((double)beta1, (double)s);
            beta2_t = (float)std::pow((double)beta2, (double)s);
            step = s;
        } else {
            beta1_t = beta1_t * beta1;
            beta2_t = beta2_t * beta2;
        }
    }
    // cpu_adam.h:163-170 (the bias-correction scalars follow in finish_consts)
    void set(float lr, float epsilon, float wd)
    {
        alpha = lr;
        eps = epsilon;
        weight_decay = wd;
    }
};

std::mutex g_registry_mutex;
std::unordered_map<int, std::shared_ptr<HostAdam>> g_registry;

std::shared_ptr<HostAdam> find_opt(int id)
{
    std::lock_guard<std::mutex> lock(g_registry_mutex);
    auto it = g_registry.find(id);
    return it == g_registry.end() ? nullptr : it->second;
}

// ------------------------------------------------------------ device math

enum WdMode { WD_NONE = 0, WD_L2 = 1, WD_DECOUPLED = 2 };
enum Unscale { UNSCALE_NONE = 0, UNSCALE_DIV = 1, UNSCALE_MUL = 2 };
constexpr int UNSCALE_RUNTIME = -1;  // template value: look at StepConsts::unscale (uniform branch)

// Per-launch constants (cpu_adam.cpp:39-46 and the SIMD_SET block at :55-77).
struct StepConsts {
    float beta1, beta2, b1m, b2m, bc2inv, eps, step_size, wd_term;
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
__host__ __device__ inline float clamp_bound(double clipping, double loss_scale)
{
    if (!(clipping > 0.0)) return 0.0f;
    double c = clipping;
    if (loss_scale > 0.0) c = c * loss_scale;
    if (65504.0 < c) c = 65504.0;
    return round_to_half_precision((float)c);
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

__host__ __device__ inline void finish_consts(StepConsts& c, float lr, float beta1, float beta2,
                                              float eps, float wd, bool adamw, float beta1_t,
                                              float beta2_t, bool bias_correction,
                                              float loss_scale, float clip)
{
    c.clip = clip;
    // cpu_adam.h:170-174
    float bc1 = 1.0f, bc2inv = 1.0f;
    if (bias_correction) {
        bc1 = 1.0f - beta1_t;
        bc2inv = 1.0f / sqrtf(1.0f - beta2_t);
    }
    c.beta1 = beta1;
    c.beta2 = beta2;
    c.b1m = 1.0f - beta1;
    c.b2m = 1.0f - beta2;
    c.bc2inv = bc2inv;
    c.eps = eps;
    c.step_size = (-1.0f * lr) / bc1;
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

template <int ARITH, int WD, int UNS>
__device__ __forceinline__ void adam_element(const StepConsts& c, float g, float& p, float& m,
                                             float& v)
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
        d = __builtin_fmaf(d, c.bc2inv, c.eps);
        float u = m / d;
        if (WD == WD_DECOUPLED) p = __builtin_fmaf(p, c.wd_term, p);
        p = __builtin_fmaf(u, c.step_size, p);
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
        d = d * c.bc2inv;                                      //   / math.sqrt(bias_correction2)
        d = d + c.eps;                                         //   .add_(eps)
        float q = m / d;
        p = __builtin_fmaf(c.step_size, q, p);                 // data.addcdiv_(exp_avg, denom, value=-step_size)
    }
}

template <int ARITH, int WD, int UNS>
__device__ __forceinline__ void element_any(const StepConsts& c, float g, float& p, float& m,
                                            float& v)
{
    if (UNS != UNSCALE_RUNTIME)
        adam_element<ARITH, WD, UNS>(c, g, p, m, v);
    else if (c.unscale == UNSCALE_MUL)
        adam_element<ARITH, WD, UNSCALE_MUL>(c, g, p, m, v);
    else if (c.unscale == UNSCALE_DIV)
        adam_element<ARITH, WD, UNSCALE_DIV>(c, g, p, m, v);
    else
        adam_element<ARITH, WD, UNSCALE_NONE>(c, g, p, m, v);
}

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

// ------------------------------------------------------- vector accesses

typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

// Chunk payloads are always device-global memory; saying so keeps the
// compiler from falling back to flat_* instructions for pointers it did not
// see being allocated.
#define PS_GLOBAL __attribute__((address_space(1)))
typedef PS_GLOBAL float4v gfloat4v;
typedef PS_GLOBAL uint4v guint4v;
typedef PS_GLOBAL uint2v guint2v;

__device__ __forceinline__ float4v ld_f4(const float* p)
{
#if PS_STREAMING & 1
    return __builtin_nontemporal_load((const gfloat4v*)(p));
#else
    return *(const gfloat4v*)(p);
#endif
}
__device__ __forceinline__ void st_f4(float* p, float4v v)
{
#if PS_STREAMING & 2
    __builtin_nontemporal_store(v, (gfloat4v*)(p));
#else
    *(gfloat4v*)(p) = v;
#endif
}
__device__ __forceinline__ uint4v ld_u4(const uint16_t* p)
{
#if PS_STREAMING & 1
    return __builtin_nontemporal_load((const guint4v*)(p));
#else
    return *(const guint4v*)(p);
#endif
}
__device__ __forceinline__ void st_u4(uint16_t* p, uint4v v)
{
#if PS_STREAMING & 2
    __builtin_nontemporal_store(v, (guint4v*)(p));
#else
    *(guint4v*)(p) = v;
#endif
}

constexpr int kBlock = PS_BLOCK;
constexpr unsigned kLdsBytes = PS_LDS_KB * 1024u;
// Elements per lane per vector step.  8: one 16-byte access of fp16 and two
// 16-byte accesses per fp32 array.  4: an 8-byte access of fp16 and one
// 16-byte access per fp32 array.
constexpr int kLaneElems = PS_LANE_ELEMS;
constexpr int kUnroll = PS_UNROLL;  // vector steps per lane per tile
constexpr int kTile = kBlock * kLaneElems * kUnroll;
constexpr int kQuads = kLaneElems / 4;  // float4 accesses per fp32 array per step
constexpr int kWords = kLaneElems / 2;  // 32-bit words of fp16 pairs per step
static_assert(kLaneElems == 4 || kLaneElems == 8, "PS_LANE_ELEMS must be 4 or 8");
static_assert(kBlock % 64 == 0 && kBlock >= 64 && kBlock <= 1024, "PS_BLOCK must be whole waves");

// fp16 pairs of one lane and step: 2 or 4 words, moved with one 8- or 16-byte access
struct HalfWords {
    uint32_t w[kWords];
};

__device__ __forceinline__ HalfWords ld_halves(const uint16_t* p)
{
    HalfWords r;
    if (kWords == 4) {
        uint4v t = ld_u4(p);
#pragma unroll
        for (int k = 0; k < kWords; ++k) r.w[k] = t[k];
    } else {
#if PS_STREAMING & 1
        uint2v t = __builtin_nontemporal_load((const guint2v*)(p));
#else
        uint2v t = *(const guint2v*)(p);
#endif
#pragma unroll
        for (int k = 0; k < kWords; ++k) r.w[k] = t[k];
    }
    return r;
}

__device__ __forceinline__ void st_halves(uint16_t* p, const HalfWords& r)
{
    if (kWords == 4) {
        uint4v t;
#pragma unroll
        for (int k = 0; k < kWords; ++k) t[k] = r.w[k];
        st_u4(p, t);
    } else {
        uint2v t;
#pragma unroll
        for (int k = 0; k < kWords; ++k) t[k] = r.w[k];
#if PS_STREAMING & 2
        __builtin_nontemporal_store(t, (guint2v*)(p));
#else
        *(guint2v*)(p) = t;
#endif
    }
}

// The registers of one lane for one tile.
struct LaneTile {
    HalfWords g[kUnroll];
    float4v p[kUnroll][kQuads], m[kUnroll][kQuads], v[kUnroll][kQuads];
    HalfWords h[kUnroll];
};

template <int ARITH, int WD, int UNS>
__device__ __forceinline__ void lane_math(const StepConsts& c, LaneTile& r)
{
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
        for (int w = 0; w < kWords; ++w) {
            uint32_t word = r.g[u].w[w];
            float g0 = half_bits_to_float(word & 0xFFFFu);
            float g1 = half_bits_to_float(word >> 16);
            const int e0 = 2 * w, e1 = 2 * w + 1;
            float p0 = r.p[u][e0 >> 2][e0 & 3], m0 = r.m[u][e0 >> 2][e0 & 3],
                  v0 = r.v[u][e0 >> 2][e0 & 3];
            float p1 = r.p[u][e1 >> 2][e1 & 3], m1 = r.m[u][e1 >> 2][e1 & 3],
                  v1 = r.v[u][e1 >> 2][e1 & 3];
            adam_element<ARITH, WD, UNS>(c, g0, p0, m0, v0);
            adam_element<ARITH, WD, UNS>(c, g1, p1, m1, v1);
            r.p[u][e0 >> 2][e0 & 3] = p0;
            r.m[u][e0 >> 2][e0 & 3] = m0;
            r.v[u][e0 >> 2][e0 & 3] = v0;
            r.p[u][e1 >> 2][e1 & 3] = p1;
            r.m[u][e1 >> 2][e1 & 3] = m1;
            r.v[u][e1 >> 2][e1 & 3] = v1;
            r.h[u].w[w] = float_to_half_bits(p0) | (float_to_half_bits(p1) << 16);
        }
    }
}

// One tile of one chunk, fast path: the whole tile is in range and all four
// bases are 16-byte aligned.  All loads of the tile are issued before the
// first use.  Loads and stores are written once, outside any branch on the
// arithmetic variant.
template <int ARITH, int WD, int UNS>
__device__ __forceinline__ void adam_tile_vec(const StepConsts& c, float* __restrict__ p32,
                                              float* __restrict__ m32, float* __restrict__ v32,
                                              uint16_t* __restrict__ h16, size_t base)
{
    LaneTile r;
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        size_t i = base + ((size_t)u * kBlock + threadIdx.x) * kLaneElems;
        r.g[u] = ld_halves(h16 + i);
#pragma unroll
        for (int q = 0; q < kQuads; ++q) r.p[u][q] = ld_f4(p32 + i + 4 * q);
#pragma unroll
        for (int q = 0; q < kQuads; ++q) r.m[u][q] = ld_f4(m32 + i + 4 * q);
#pragma unroll
        for (int q = 0; q < kQuads; ++q) r.v[u][q] = ld_f4(v32 + i + 4 * q);
    }
    if (UNS != UNSCALE_RUNTIME) {
        lane_math<ARITH, WD, UNS>(c, r);
    } else if (c.unscale == UNSCALE_MUL) {
        lane_math<ARITH, WD, UNSCALE_MUL>(c, r);
    } else if (ARITH == PS_ARITH_OPERATOR && c.unscale == UNSCALE_DIV) {
        lane_math<ARITH, WD, UNSCALE_DIV>(c, r);
    } else {
        lane_math<ARITH, WD, UNSCALE_NONE>(c, r);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        size_t i = base + ((size_t)u * kBlock + threadIdx.x) * kLaneElems;
#pragma unroll
        for (int q = 0; q < kQuads; ++q) st_f4(p32 + i + 4 * q, r.p[u][q]);
#pragma unroll
        for (int q = 0; q < kQuads; ++q) st_f4(m32 + i + 4 * q, r.m[u][q]);
#pragma unroll
        for (int q = 0; q < kQuads; ++q) st_f4(v32 + i + 4 * q, r.v[u][q]);
        st_halves(h16 + i, r.h[u]);
    }
}

// Same elements, one at a time: ragged tile ends and unaligned bases.
template <int ARITH, int WD, int UNS>
__device__ __forceinline__ void adam_tile_scalar(const StepConsts& c, float* p32, float* m32,
                                                 float* v32, uint16_t* h16, size_t base, size_t end)
{
    for (size_t i = base + threadIdx.x; i < end; i += kBlock) {
        float g = half_bits_to_float(h16[i]);
        float p = p32[i], m = m32[i], v = v32[i];
        element_any<ARITH, WD, UNS>(c, g, p, m, v);
        p32[i] = p;
        m32[i] = m;
        v32[i] = v;
        h16[i] = (uint16_t)float_to_half_bits(p);
    }
}

__device__ __forceinline__ bool aligned16(const void* a, const void* b, const void* c,
                                          const void* d)
{
    return (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c | (uintptr_t)d) & 15u) == 0;
}

template <int ARITH, int WD, int UNS>
__device__ __forceinline__ void adam_tile(const StepConsts& c, const ps_chunk& ch, size_t base,
                                          size_t chunk_numel)
{
    size_t end = base + kTile;
    if (end <= chunk_numel && aligned16(ch.param_fp32, ch.exp_avg, ch.exp_avg_sq, ch.param_fp16)) {
        adam_tile_vec<ARITH, WD, UNS>(c, ch.param_fp32, ch.exp_avg, ch.exp_avg_sq, ch.param_fp16,
                                      base);
    } else {
        if (end > chunk_numel) end = chunk_numel;
        adam_tile_scalar<ARITH, WD, UNS>(c, ch.param_fp32, ch.exp_avg, ch.exp_avg_sq,
                                         ch.param_fp16, base, end);
    }
}

// fp16 <- RNE(fp32) for one tile (the restore of a skipped step and the
// stand-alone write-back).
__device__ __forceinline__ void restore_tile(const float* __restrict__ p32,
                                             uint16_t* __restrict__ h16, size_t base,
                                             size_t numel)
{
    size_t end = base + kTile;
    if (end <= numel && ((((uintptr_t)p32 | (uintptr_t)h16) & 15u) == 0)) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            size_t i = base + ((size_t)u * kBlock + threadIdx.x) * kLaneElems;
            float4v a[kQuads];
#pragma unroll
            for (int q = 0; q < kQuads; ++q) a[q] = ld_f4(p32 + i + 4 * q);
            HalfWords out;
#pragma unroll
            for (int w = 0; w < kWords; ++w)
                out.w[w] = float_to_half_bits(a[w >> 1][(2 * w) & 3]) |
                           (float_to_half_bits(a[w >> 1][(2 * w + 1) & 3]) << 16);
            st_halves(h16 + i, out);
        }
    } else {
        if (end > numel) end = numel;
        for (size_t i = base + threadIdx.x; i < end; i += kBlock)
            h16[i] = (uint16_t)float_to_half_bits(p32[i]);
    }
}

// ------------------------------------------------------- chunk-list kernels
//
// Grid: x = tile inside a chunk, y = chunk inside the batch.  Up to kBatch
// descriptors are passed BY VALUE in the kernel-argument segment.

constexpr int kBatch = 64;
struct ChunkBatch {
    ps_chunk c[kBatch];
};
static_assert(sizeof(ps_chunk) == 32 && sizeof(ps_step_state) == 160 && sizeof(ps_scale_record) == 16,
              "layout of the boundary structs");

// Host-decided step: all scalars arrive as kernel arguments and the
// arithmetic variant is a compile-time property of the kernel.
template <int ARITH, int WD, int UNS>
__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    adam_chunks_kernel(ChunkBatch b, size_t chunk_numel, StepConsts c)
{
    adam_tile<ARITH, WD, UNS>(c, b.c[blockIdx.y], (size_t)blockIdx.x * kTile, chunk_numel);
}

struct GatedArgs {
    double lr, eps, wd;  // the Python numbers; the operator's arithmetic narrows them to float
    double grad_clamp;
    int adamw;
    int bias_correction;
};

// Device-decided step: overflow flag, loss scale and beta^t come from the
// device-resident state; a flagged step restores fp16 from fp32 instead.
// The weight-decay form is known to the host; the unscale form depends on
// the device-resident scale and is a uniform branch around the arithmetic.
template <int ARITH, int WD>
__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    adam_chunks_gated_kernel(ChunkBatch b, size_t chunk_numel, GatedArgs ga,
                             const ps_step_state* __restrict__ st)
{
    const ps_chunk& ch = b.c[blockIdx.y];
    const size_t base = (size_t)blockIdx.x * kTile;
    if (st->overflow) {
        restore_tile(ch.param_fp32, ch.param_fp16, base, chunk_numel);
        return;
    }
    StepConsts c;
    const float clip = clamp_bound(ga.grad_clamp, st->cur_scale);
    if (ARITH == PS_ARITH_OPERATOR) {
        // The operator takes its scalars and loss_scale as C floats: the Python numbers narrow (RNE).
        finish_consts(c, (float)ga.lr, st->beta1, st->beta2, (float)ga.eps, (float)ga.wd,
                      ga.adamw != 0, st->beta1_t_next, st->beta2_t_next, ga.bias_correction != 0,
                      (float)st->cur_scale, clip);
    } else {
        const bool bc = ga.bias_correction != 0;
        torch_consts(c, ga.lr, st->beta1_f64, st->beta2_f64, ga.eps, ga.wd, ga.adamw != 0,
                     bc ? st->bias_correction1_next : 1.0, bc ? st->bias_correction2_next : 1.0,
                     st->cur_scale, clip);
    }
    adam_tile<ARITH, WD, UNSCALE_RUNTIME>(c, ch, base, chunk_numel);
}

__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    restore_chunks_kernel(ChunkBatch b, size_t chunk_numel, const ps_step_state* __restrict__ st)
{
    if (st != nullptr && !st->overflow) return;
    const ps_chunk& ch = b.c[blockIdx.y];
    restore_tile(ch.param_fp32, ch.param_fp16, (size_t)blockIdx.x * kTile, chunk_numel);
}

__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    cast_kernel(const float* __restrict__ src, uint16_t* __restrict__ dst, size_t numel,
                size_t n_tiles)
{
    for (size_t t = blockIdx.x; t < n_tiles; t += gridDim.x)
        restore_tile(src, dst, t * (size_t)kTile, numel);
}

// ------------------------------------------------- auxiliary (non-hot) kernels

constexpr int kAuxBlock = 256;

// Flat tensor, any grad dtype, optional fp16 output (adam_update of the operator).
// Element-wise accesses: tensors handed to the operator are views at arbitrary
// element offsets inside a chunk, so no alignment can be assumed.
template <int WD, bool GRAD_HALF>
__global__ void __launch_bounds__(kAuxBlock)
    adam_flat_kernel(StepConsts c, float* p32, const void* grads, float* m32, float* v32,
                     uint16_t* out16, size_t numel)
{
    const uint16_t* gh = static_cast<const uint16_t*>(grads);
    const float* gf = static_cast<const float*>(grads);
    size_t stride = (size_t)gridDim.x * kAuxBlock;
    for (size_t i = (size_t)blockIdx.x * kAuxBlock + threadIdx.x; i < numel; i += stride) {
        float g = GRAD_HALF ? half_bits_to_float(gh[i]) : gf[i];
        float p = p32[i], m = m32[i], v = v32[i];
        element_any<PS_ARITH_OPERATOR, WD, UNSCALE_RUNTIME>(c, g, p, m, v);
        p32[i] = p;
        m32[i] = m;
        v32[i] = v;
        if (out16) out16[i] = (uint16_t)float_to_half_bits(p);
    }
}

// The same operator on a span whose four (five) addresses share one 16-byte phase: single-wave
// workgroups over 256-element tiles with 16-byte accesses, resident-workgroup cap as for the chunk
// kernels.  Gradients are read only; the fp16 output is optional.
template <int WD, bool GRAD_HALF>
__global__ void __launch_bounds__(64)
    adam_flat_vec_kernel(StepConsts c, float* p32, const void* grads, float* m32, float* v32,
                         uint16_t* out16,  // may alias grads (fp16 gradients overwritten by fp16 parameters)
                         size_t n_tiles)
{
    for (size_t t = blockIdx.x; t < n_tiles; t += gridDim.x) {
        const size_t i = (t * 64 + threadIdx.x) * 4;
        float g[4];
        if (GRAD_HALF) {
            uint2v w = *(const guint2v*)(static_cast<const uint16_t*>(grads) + i);
            g[0] = half_bits_to_float(w[0] & 0xFFFFu);
            g[1] = half_bits_to_float(w[0] >> 16);
            g[2] = half_bits_to_float(w[1] & 0xFFFFu);
            g[3] = half_bits_to_float(w[1] >> 16);
        } else {
            float4v gv = ld_f4(static_cast<const float*>(grads) + i);
#pragma unroll
            for (int e = 0; e < 4; ++e) g[e] = gv[e];
        }
        float4v p = ld_f4(p32 + i), m = ld_f4(m32 + i), v = ld_f4(v32 + i);
        uint32_t h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float pe = p[e], me = m[e], ve = v[e];
            element_any<PS_ARITH_OPERATOR, WD, UNSCALE_RUNTIME>(c, g[e], pe, me, ve);
            p[e] = pe;
            m[e] = me;
            v[e] = ve;
            h[e] = float_to_half_bits(pe);
        }
        st_f4(p32 + i, p);
        st_f4(m32 + i, m);
        st_f4(v32 + i, v);
        if (out16 != nullptr) {
            uint2v o;
            o[0] = h[0] | (h[1] << 16);
            o[1] = h[2] | (h[3] << 16);
            *(guint2v*)(out16 + i) = o;
        }
    }
}

// ----------------------------------------------------------- overflow scan
//
// A binary16 value is inf or nan iff its five exponent bits are all set.
// For a 32-bit word holding two halves: mask the exponents, add one unit of
// the lowest exponent bit to each; an all-ones exponent carries into bit 15 /
// bit 31 (the masked low half is at most 0x7C00, so its carry stops at bit 15).

__device__ __forceinline__ uint32_t nonfinite_halves(uint32_t w)
{
    return ((w & 0x7C007C00u) + 0x04000400u) & 0x80008000u;
}

// OR across the block: shuffle butterfly inside each wave, LDS across the
// four waves, then at most one atomic per block (none when nothing was seen).
__device__ __forceinline__ void block_flag_commit(uint32_t hit, uint32_t* flag)
{
    __shared__ uint32_t wave_hit[kAuxBlock / 64];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) hit |= (uint32_t)__shfl_xor((int)hit, off, 64);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) wave_hit[wave] = hit;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t any = 0;
#pragma unroll
        for (int w = 0; w < kAuxBlock / 64; ++w) any |= wave_hit[w];
        if (any) atomicOr(flag, 1u);
    }
}

constexpr int kScanUnroll = 4;
constexpr int kScanTile = kAuxBlock * 8 * kScanUnroll;  // 16-byte loads of 8 halves: 8192 halves = 16 KiB per tile

// One scan tile of a fp16 buffer.
__device__ __forceinline__ uint32_t scan_tile_f16(const uint16_t* __restrict__ h, size_t numel,
                                                  size_t tile)
{
    uint32_t hit = 0;
    const size_t base = tile * (size_t)kScanTile;
    if (base >= numel) return 0;
    if ((((uintptr_t)h) & 15u) == 0 && base + kScanTile <= numel) {
        uint4v w[kScanUnroll];
#pragma unroll
        for (int u = 0; u < kScanUnroll; ++u)
            w[u] = ld_u4(h + base + ((size_t)u * kAuxBlock + threadIdx.x) * 8);
#pragma unroll
        for (int u = 0; u < kScanUnroll; ++u)
            hit |= nonfinite_halves(w[u][0]) | nonfinite_halves(w[u][1]) |
                   nonfinite_halves(w[u][2]) | nonfinite_halves(w[u][3]);
    } else {
        size_t end = base + kScanTile < numel ? base + kScanTile : numel;
        for (size_t i = base + threadIdx.x; i < end; i += kAuxBlock)
            hit |= ((h[i] & 0x7C00u) == 0x7C00u) ? 1u : 0u;
    }
    return hit;
}

__global__ void __launch_bounds__(kAuxBlock)
    scan_f16_kernel(const uint16_t* __restrict__ h, size_t numel, size_t n_tiles,
                    ps_step_state* st)
{
    uint32_t hit = 0;
    for (size_t t = blockIdx.x; t < n_tiles; t += gridDim.x) hit |= scan_tile_f16(h, numel, t);
    block_flag_commit(hit, &st->overflow);
}

__global__ void __launch_bounds__(kAuxBlock)
    scan_f32_kernel(const float* __restrict__ f, size_t numel, ps_step_state* st)
{
    uint32_t hit = 0;
    const uint32_t* w = reinterpret_cast<const uint32_t*>(f);
    size_t stride = (size_t)gridDim.x * kAuxBlock;
    for (size_t i = (size_t)blockIdx.x * kAuxBlock + threadIdx.x; i < numel; i += stride)
        hit |= ((w[i] & 0x7F800000u) == 0x7F800000u) ? 1u : 0u;
    block_flag_commit(hit, &st->overflow);
}

__global__ void __launch_bounds__(kAuxBlock)
    scan_chunks_kernel(ChunkBatch b, size_t chunk_numel, ps_step_state* st)
{
    uint32_t hit = scan_tile_f16(b.c[blockIdx.y].param_fp16, chunk_numel, blockIdx.x);
    block_flag_commit(hit, &st->overflow);
}

// Backward-side producer: copy one gradient into its slot of the fp16 chunk
// (patrickstar/core/hook.py:212-216) and probe it for inf/nan in the same pass
// (loss_scaler.py:133-155), instead of a separate cast + sum + host sync per
// parameter.  Slots start at arbitrary element offsets, so accesses are per
// element.  fp32 gradients are rounded to fp16 (RNE); the probe looks at the
// value that lands in the chunk.
template <bool SRC_HALF>
__global__ void __launch_bounds__(kAuxBlock)
    grad_to_chunk_kernel(const void* __restrict__ src, uint16_t* __restrict__ dst, size_t numel,
                         ps_step_state* st)
{
    const uint16_t* sh = static_cast<const uint16_t*>(src);
    const float* sf = static_cast<const float*>(src);
    uint32_t hit = 0;
    size_t stride = (size_t)gridDim.x * kAuxBlock;
    for (size_t i = (size_t)blockIdx.x * kAuxBlock + threadIdx.x; i < numel; i += stride) {
        uint32_t h = SRC_HALF ? (uint32_t)sh[i] : float_to_half_bits(sf[i]);
        dst[i] = (uint16_t)h;
        hit |= ((h & 0x7C00u) == 0x7C00u) ? 1u : 0u;
    }
    if (st != nullptr) block_flag_commit(hit, &st->overflow);
}

// Vector form of the same copy for long gradients.  The chunk slot sets the grid: 16-byte stores to
// 16-byte aligned addresses of the slot.  A fp16 source is generally at a different phase, so each lane
// loads the two ALIGNED 16-byte source blocks that straddle its output vector and funnel-shifts them by
// S halves in registers; no misaligned memory access is made.  Every 16-byte block that is loaded holds
// at least one element of the gradient, so it lies inside the gradient's allocation.
template <int S>
__device__ __forceinline__ uint4v shift_halves(const uint4v& a, const uint4v& b)
{
    const uint32_t w[8] = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
    constexpr int d = (2 * S) / 4, r = (2 * S) % 4;
    uint4v o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = r ? ((w[i + d] >> 16) | (w[i + d + 1] << 16)) : w[i + d];
    return o;
}

template <int S>
__device__ __forceinline__ uint32_t copy_shifted_f16(const uint16_t* src_al, uint16_t* dst_al,
                                                      size_t n_vec)
{
    uint32_t hit = 0;
    size_t stride = (size_t)gridDim.x * kAuxBlock;
    for (size_t j = (size_t)blockIdx.x * kAuxBlock + threadIdx.x; j < n_vec; j += stride) {
        uint4v a = ld_u4(src_al + 8 * j);
        uint4v b = a;
        if (S != 0) b = ld_u4(src_al + 8 * j + 8);
        uint4v o = shift_halves<S>(a, b);
        hit |= nonfinite_halves(o[0]) | nonfinite_halves(o[1]) | nonfinite_halves(o[2]) |
               nonfinite_halves(o[3]);
        st_u4(dst_al + 8 * j, o);
    }
    return hit;
}

__global__ void __launch_bounds__(kAuxBlock)
    grad_to_chunk_f16_vec_kernel(const uint16_t* __restrict__ src_al, int shift,
                                 uint16_t* __restrict__ dst_al, size_t n_vec, ps_step_state* st)
{
    uint32_t hit = 0;
    switch (shift) {
        case 0: hit = copy_shifted_f16<0>(src_al, dst_al, n_vec); break;
        case 1: hit = copy_shifted_f16<1>(src_al, dst_al, n_vec); break;
        case 2: hit = copy_shifted_f16<2>(src_al, dst_al, n_vec); break;
        case 3: hit = copy_shifted_f16<3>(src_al, dst_al, n_vec); break;
        case 4: hit = copy_shifted_f16<4>(src_al, dst_al, n_vec); break;
        case 5: hit = copy_shifted_f16<5>(src_al, dst_al, n_vec); break;
        case 6: hit = copy_shifted_f16<6>(src_al, dst_al, n_vec); break;
        default: hit = copy_shifted_f16<7>(src_al, dst_al, n_vec); break;
    }
    if (st != nullptr) block_flag_commit(hit, &st->overflow);
}

// fp32 gradients: eight dword-aligned floats per output vector (multi-dword loads need dword alignment only).
typedef float4v __attribute__((aligned(4))) float4v_dword_aligned;
__global__ void __launch_bounds__(kAuxBlock)
    grad_to_chunk_f32_vec_kernel(const float* __restrict__ src, uint16_t* __restrict__ dst_al,
                                 size_t n_vec, ps_step_state* st)
{
    uint32_t hit = 0;
    size_t stride = (size_t)gridDim.x * kAuxBlock;
    for (size_t j = (size_t)blockIdx.x * kAuxBlock + threadIdx.x; j < n_vec; j += stride) {
        float4v x = *(const PS_GLOBAL float4v_dword_aligned*)(src + 8 * j);
        float4v y = *(const PS_GLOBAL float4v_dword_aligned*)(src + 8 * j + 4);
        uint4v o;
        o[0] = float_to_half_bits(x[0]) | (float_to_half_bits(x[1]) << 16);
        o[1] = float_to_half_bits(x[2]) | (float_to_half_bits(x[3]) << 16);
        o[2] = float_to_half_bits(y[0]) | (float_to_half_bits(y[1]) << 16);
        o[3] = float_to_half_bits(y[2]) | (float_to_half_bits(y[3]) << 16);
        hit |= nonfinite_halves(o[0]) | nonfinite_halves(o[1]) | nonfinite_halves(o[2]) |
               nonfinite_halves(o[3]);
        st_u4(dst_al + 8 * j, o);
    }
    if (st != nullptr) block_flag_commit(hit, &st->overflow);
}

// ------------------------------------------------ device-resident step state

__global__ void state_init_kernel(ps_step_state* st, ps_step_state init)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) *st = init;
}

struct SeedArgs {
    int64_t adam_step;
    float beta1, beta2, b1t_next, b2t_next;
    double beta1_f64, beta2_f64, bc1_next, bc2_next;
};

__global__ void state_seed_kernel(ps_step_state* st, SeedArgs a)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        st->adam_step = a.adam_step;
        st->beta1 = a.beta1;
        st->beta2 = a.beta2;
        st->beta1_t_next = a.b1t_next;
        st->beta2_t_next = a.b2t_next;
        st->beta1_f64 = a.beta1_f64;
        st->beta2_f64 = a.beta2_f64;
        st->bias_correction1_next = a.bc1_next;
        st->bias_correction2_next = a.bc2_next;
    }
}

// beta ** n for a non-negative integer n in binary64, by squaring in double-double arithmetic: the
// result is the correctly rounded power except within ~2^-90 of a rounding boundary, which is what
// Python's float ** int (the C library's pow) returns for all but about one step in 10^4; the
// float constants derived from 1 - beta ** n did not differ on any of 1.8 million (beta, n) pairs.
struct TwoDouble {
    double hi, lo;
};
__device__ inline TwoDouble two_double_mul(TwoDouble a, TwoDouble b)
{
    double p = a.hi * b.hi;
    double e = __builtin_fma(a.hi, b.hi, -p);
    e += a.hi * b.lo + a.lo * b.hi;
    double s = p + e;
    return TwoDouble{s, e - (s - p)};
}
__device__ inline double pow_int(double base, int64_t n)
{
    TwoDouble r{1.0, 0.0}, x{base, 0.0};
    while (n > 0) {
        if (n & 1) r = two_double_mul(r, x);
        n >>= 1;
        if (n) x = two_double_mul(x, x);
    }
    return r.hi;
}

__global__ void state_set_scaler_kernel(ps_step_state* st, double cur_scale, int scale_is_int,
                                        int64_t cur_iter, int64_t last_overflow_iter,
                                        int cur_hysteresis)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        st->cur_scale = cur_scale;
        st->scale_is_int = scale_is_int;
        st->cur_iter = cur_iter;
        st->last_overflow_iter = last_overflow_iter;
        st->cur_hysteresis = cur_hysteresis;
    }
}

// DynamicLossScaler.update_scale (loss_scaler.py:158-182), one lane.
__global__ void scaler_update_kernel(ps_step_state* st, int flag_mode, ps_scale_record* log,
                                     int64_t log_capacity)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    ps_step_state s = *st;
    const bool overflow = flag_mode == PS_FLAG_FROM_DEVICE ? (s.overflow != 0) : (flag_mode != 0);
    if (overflow) {
        if (s.delayed_shift == 1 || s.cur_hysteresis == 1) {
            // Python: max(cur_scale / scale_factor, min_scale) -- true division gives a
            // float; max keeps its first argument unless the second is strictly greater.
            double q = s.cur_scale / s.scale_factor;
            if (s.min_scale > q) {
                s.cur_scale = s.min_scale;
                s.scale_is_int = s.min_is_int;
            } else {
                s.cur_scale = q;
                s.scale_is_int = 0;
            }
        } else {
            s.cur_hysteresis -= 1;
        }
        s.last_overflow_iter = s.cur_iter;
        s.skipped_steps += 1;
    } else {
        if (s.consecutive_hysteresis) s.cur_hysteresis = s.delayed_shift;
        if ((s.cur_iter - s.last_overflow_iter) % s.scale_window == 0) {
            if (!s.consecutive_hysteresis) s.cur_hysteresis = s.delayed_shift;
            s.cur_scale = s.cur_scale * s.scale_factor;
            s.scale_is_int = s.scale_is_int && s.factor_is_int;
        }
        // the step ran: state["step"] += 1 and the float running products advance
        s.adam_step += 1;
        s.beta1_t_next = s.beta1_t_next * s.beta1;
        s.beta2_t_next = s.beta2_t_next * s.beta2;
        // fp16_cpu_adam.py:412-413 for the next step
        s.bias_correction1_next = 1.0 - pow_int(s.beta1_f64, s.adam_step + 1);
        s.bias_correction2_next = 1.0 - pow_int(s.beta2_f64, s.adam_step + 1);
    }
    if (log != nullptr && log_capacity > 0) {
        ps_scale_record r;
        r.scale_after = s.cur_scale;
        r.overflow = overflow ? 1u : 0u;
        r.scale_is_int = (uint32_t)s.scale_is_int;
        log[s.cur_iter % log_capacity] = r;
    }
    s.cur_iter += 1;
    s.last_skipped = overflow ? 1u : 0u;
    s.overflow = 0;
    *st = s;
}

// ------------------------------------------------------------ launch helpers

constexpr size_t kMaxGridX = 0x7FFFFFFFull;

unsigned grid_1d(size_t n_blocks)
{
    size_t g = n_blocks < kMaxGridX ? n_blocks : kMaxGridX;
    return (unsigned)(g ? g : 1);
}

// Validated view of a host array of chunk descriptors.
struct ChunkList {
    const ps_chunk* chunks;
    int n_chunks;
    size_t chunk_numel;
    size_t tiles_per_chunk;  // of kTile elements
};

// All descriptors are checked here, before anything is enqueued or any host state advances.
int make_chunk_list(ChunkList& a, const ps_chunk* chunks, int n_chunks, size_t chunk_numel,
                    size_t tile, bool fp16_only = false, const char* what = "chunk")
{
    if (n_chunks < 0) return fail(PS_ERR_BAD_ARG, "n_chunks = %d is negative", n_chunks);
    if (chunks == nullptr && n_chunks > 0) return fail(PS_ERR_BAD_ARG, "chunks is NULL");
    for (int i = 0; i < n_chunks; ++i) {
        const ps_chunk& c = chunks[i];
        if (!c.param_fp16 || (!fp16_only && (!c.param_fp32 || !c.exp_avg || !c.exp_avg_sq)))
            return fail(PS_ERR_BAD_ARG, "%s %d has a NULL payload address", what, i);
    }
    a.chunks = chunks;
    a.n_chunks = n_chunks;
    a.chunk_numel = chunk_numel;
    a.tiles_per_chunk = (chunk_numel + tile - 1) / tile;
    if (a.tiles_per_chunk > kMaxGridX)
        return fail(PS_ERR_BAD_ARG, "chunk_numel = %zu is beyond the launch grid", chunk_numel);
    return 0;
}

// Calls launch(batch, n_in_batch, grid) for every group of up to kBatch chunks.
template <typename F>
int for_each_batch(const ChunkList& a, F launch)
{
    if (a.n_chunks == 0 || a.tiles_per_chunk == 0) return 0;
    for (int first = 0; first < a.n_chunks; first += kBatch) {
        int n = a.n_chunks - first < kBatch ? a.n_chunks - first : kBatch;
        ChunkBatch b;
        memset(&b, 0, sizeof(b));
        for (int i = 0; i < n; ++i) b.c[i] = a.chunks[first + i];
        launch(b, dim3((unsigned)a.tiles_per_chunk, (unsigned)n));
        PS_HIP(hipGetLastError());
    }
    return 0;
}

template <int ARITH, int WD>
void launch_adam_batch_wd(const ChunkBatch& b, dim3 grid, size_t chunk_numel, const StepConsts& c,
                          hipStream_t s)
{
    dim3 block(kBlock);
    if (c.unscale == UNSCALE_MUL)
        hipLaunchKernelGGL((adam_chunks_kernel<ARITH, WD, UNSCALE_MUL>), grid, block, kLdsBytes, s, b, chunk_numel, c);
    else if (ARITH == PS_ARITH_OPERATOR && c.unscale == UNSCALE_DIV)  // the torch formula never divides
        hipLaunchKernelGGL((adam_chunks_kernel<ARITH, WD, UNSCALE_DIV>), grid, block, kLdsBytes, s, b, chunk_numel, c);
    else
        hipLaunchKernelGGL((adam_chunks_kernel<ARITH, WD, UNSCALE_NONE>), grid, block, kLdsBytes, s, b, chunk_numel, c);
}

template <int ARITH>
void launch_adam_batch_arith(const ChunkBatch& b, dim3 grid, size_t chunk_numel,
                             const StepConsts& c, hipStream_t s)
{
    if (c.wd_mode == WD_DECOUPLED)
        launch_adam_batch_wd<ARITH, WD_DECOUPLED>(b, grid, chunk_numel, c, s);
    else if (c.wd_mode == WD_L2)
        launch_adam_batch_wd<ARITH, WD_L2>(b, grid, chunk_numel, c, s);
    else
        launch_adam_batch_wd<ARITH, WD_NONE>(b, grid, chunk_numel, c, s);
}

// `c` must have been built for `arith` (finish_consts / torch_consts).
void launch_adam_batch(int arith, const ChunkBatch& b, dim3 grid, size_t chunk_numel,
                       const StepConsts& c, hipStream_t s)
{
    if (arith == PS_ARITH_TORCH)
        launch_adam_batch_arith<PS_ARITH_TORCH>(b, grid, chunk_numel, c, s);
    else
        launch_adam_batch_arith<PS_ARITH_OPERATOR>(b, grid, chunk_numel, c, s);
}

template <int ARITH>
void launch_gated_batch_arith(const ChunkBatch& b, dim3 grid, size_t chunk_numel,
                              const GatedArgs& ga, const ps_step_state* d_state, hipStream_t s)
{
    dim3 block(kBlock);
    // the operator tests its float weight decay "> 0" (cpu_adam.cpp:42), the torch formula "!= 0"
    const bool decay = ARITH == PS_ARITH_OPERATOR ? (float)ga.wd > 0.0f : ga.wd != 0.0;
    if (decay && ga.adamw)
        hipLaunchKernelGGL((adam_chunks_gated_kernel<ARITH, WD_DECOUPLED>), grid, block, kLdsBytes, s, b, chunk_numel, ga, d_state);
    else if (decay)
        hipLaunchKernelGGL((adam_chunks_gated_kernel<ARITH, WD_L2>), grid, block, kLdsBytes, s, b, chunk_numel, ga, d_state);
    else
        hipLaunchKernelGGL((adam_chunks_gated_kernel<ARITH, WD_NONE>), grid, block, kLdsBytes, s, b, chunk_numel, ga, d_state);
}

void launch_gated_batch(int arith, const ChunkBatch& b, dim3 grid, size_t chunk_numel,
                        const GatedArgs& ga, const ps_step_state* d_state, hipStream_t s)
{
    if (arith == PS_ARITH_TORCH)
        launch_gated_batch_arith<PS_ARITH_TORCH>(b, grid, chunk_numel, ga, d_state, s);
    else
        launch_gated_batch_arith<PS_ARITH_OPERATOR>(b, grid, chunk_numel, ga, d_state, s);
}

// The Python numbers of one step as they cross the boundary.
struct HyperParams {
    double lr, beta1, beta2, eps, wd;
    double loss_scale;  // <= 0: no loss scaler
    bool bias_correction;
};

// Host-decided step, operator arithmetic: narrow like the pybind signature of adam_update
// (float arguments, cpu_adam.cpp:700-712), advance the operator's step scalars, derive the rest.
StepConsts operator_step_consts(HostAdam& o, size_t step, const HyperParams& hp)
{
    o.advance(step, (float)hp.beta1, (float)hp.beta2);
    o.set((float)hp.lr, (float)hp.eps, (float)hp.wd);
    StepConsts c;
    finish_consts(c, o.alpha, o.beta1, o.beta2, o.eps, o.weight_decay, o.adamw, o.beta1_t,
                  o.beta2_t, hp.bias_correction, (float)hp.loss_scale,
                  clamp_bound(o.grad_clamp, hp.loss_scale));
    return c;
}

// Host-decided step, torch arithmetic (fp16_cpu_adam.py:412-413: Python's float ** int is the C
// library's pow).  The operator object is not touched: the reference does not call it here.
StepConsts torch_step_consts(const HostAdam& o, size_t step, const HyperParams& hp)
{
    double bc1 = 1.0, bc2 = 1.0;
    if (hp.bias_correction) {
        bc1 = 1.0 - std::pow(hp.beta1, (double)step);
        bc2 = 1.0 - std::pow(hp.beta2, (double)step);
    }
    StepConsts c;
    torch_consts(c, hp.lr, hp.beta1, hp.beta2, hp.eps, hp.wd, o.adamw, bc1, bc2, hp.loss_scale,
                 clamp_bound(o.grad_clamp, hp.loss_scale));
    return c;
}

GatedArgs gated_args(const HostAdam& o, double lr, double eps, double wd, int bias_correction)
{
    GatedArgs ga;
    ga.lr = lr;
    ga.eps = eps;
    ga.wd = wd;
    ga.grad_clamp = o.grad_clamp;
    ga.adamw = o.adamw ? 1 : 0;
    ga.bias_correction = bias_correction;
    return ga;
}

// ------------------------------------------- host-resident chunks: streaming
//
// Chunks that live in pinned host memory are streamed through caller-owned
// staging buffers in HBM: H2D copies on one side stream, the fused kernel on a
// compute side stream, D2H copies on another side stream, tied together with
// events, so that with two or more staging slots the copy of chunk k+1 and the
// write-back of chunk k-1 overlap the kernel on chunk k.  Nothing blocks the
// host.  The streams and events are created once per device and kept.

constexpr int kMaxSlots = 8;

struct Pipeline {
    bool ready = false;
    hipStream_t h2d = nullptr, compute = nullptr, d2h = nullptr;
    hipEvent_t entry = nullptr;
    hipEvent_t h2d_done[kMaxSlots] = {}, compute_done[kMaxSlots] = {}, d2h_done[kMaxSlots] = {};
    bool slot_used[kMaxSlots] = {};
};

std::mutex g_pipeline_mutex;
std::unordered_map<int, Pipeline> g_pipelines;

int get_pipeline(Pipeline** out)
{
    int dev = 0;
    PS_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_pipeline_mutex);
    Pipeline& p = g_pipelines[dev];
    if (!p.ready) {
        // default priority on purpose
        PS_HIP(hipStreamCreateWithFlags(&p.h2d, hipStreamNonBlocking));
        PS_HIP(hipStreamCreateWithFlags(&p.compute, hipStreamNonBlocking));
        PS_HIP(hipStreamCreateWithFlags(&p.d2h, hipStreamNonBlocking));
        PS_HIP(hipEventCreateWithFlags(&p.entry, hipEventDisableTiming));
        for (int i = 0; i < kMaxSlots; ++i) {
            PS_HIP(hipEventCreateWithFlags(&p.h2d_done[i], hipEventDisableTiming));
            PS_HIP(hipEventCreateWithFlags(&p.compute_done[i], hipEventDisableTiming));
            PS_HIP(hipEventCreateWithFlags(&p.d2h_done[i], hipEventDisableTiming));
        }
        p.ready = true;
    }
    *out = &p;
    return 0;
}

int check_slots(const ps_chunk* staging, int n_slots, bool need_state, bool need_fp16)
{
    if (n_slots < 1 || n_slots > kMaxSlots)
        return fail(PS_ERR_BAD_ARG, "n_slots = %d must be in 1..%d", n_slots, kMaxSlots);
    if (!staging) return fail(PS_ERR_BAD_ARG, "staging is NULL");
    for (int i = 0; i < n_slots; ++i) {
        if ((need_fp16 && !staging[i].param_fp16) ||
            (need_state && (!staging[i].param_fp32 || !staging[i].exp_avg || !staging[i].exp_avg_sq)))
            return fail(PS_ERR_BAD_ARG, "staging slot %d has a NULL buffer", i);
    }
    return 0;
}

// A host-resident chunk position may keep its fp16 payload in HBM (only the optimizer state lives in
// host memory): say for every position whether its fp16 address is device memory.
int fp16_payloads_in_hbm(const ps_chunk* host_chunks, int n, bool* in_hbm, bool* any_on_host)
{
    *any_on_host = false;
    for (int i = 0; i < n; ++i) {
        hipPointerAttribute_t attr;
        hipError_t e = hipPointerGetAttributes(&attr, host_chunks[i].param_fp16);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return fail(PS_ERR_BAD_ARG, "host chunk %d: the fp16 address is neither device nor pinned host memory (%s)",
                        i, hipGetErrorString(e));
        }
        in_hbm[i] = attr.type == hipMemoryTypeDevice;
        if (!in_hbm[i]) *any_on_host = true;
    }
    return 0;
}

}  // namespace

// ====================================================================== ABI

extern "C" {

int ps_abi_version(void) { return PS_ABI_VERSION; }

const char* ps_last_error(void) { return g_err; }

int ps_adam_create(int optimizer_id, float alpha, float beta1, float beta2, float eps,
                   float weight_decay, int adamw_mode, int should_log)
{
    auto o = std::make_shared<HostAdam>();
    o->alpha = alpha;
    o->beta1 = beta1;
    o->beta2 = beta2;
    o->eps = eps;
    o->weight_decay = weight_decay;
    o->adamw = adamw_mode != 0;
    {
        std::lock_guard<std::mutex> lock(g_registry_mutex);
        g_registry[optimizer_id] = o;
    }
    if (should_log) {
        printf("Adam Optimizer #%d is created with gfx950 HIP arithmetic capability.\n",
               optimizer_id);
        printf("Config: alpha=%f, betas=(%f, %f), weight_decay=%f, adam_w=%d\n", alpha, beta1,
               beta2, weight_decay, (int)(adamw_mode != 0));
    }
    return 0;
}

int ps_adam_set_grad_clamp(int optimizer_id, double gradient_clipping)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    o->grad_clamp = gradient_clipping;
    return 0;
}

int ps_adam_set_arithmetic(int optimizer_id, int arithmetic)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    if (arithmetic != PS_ARITH_OPERATOR && arithmetic != PS_ARITH_TORCH)
        return fail(PS_ERR_BAD_ARG, "arithmetic = %d is neither PS_ARITH_OPERATOR nor PS_ARITH_TORCH", arithmetic);
    o->arith = arithmetic;
    return 0;
}

int ps_adam_destroy(int optimizer_id)
{
    std::lock_guard<std::mutex> lock(g_registry_mutex);
    g_registry.erase(optimizer_id);
    return 0;
}

int ps_adam_update(int optimizer_id, size_t step, float lr, float beta1, float beta2, float epsilon,
                   float weight_decay, int bias_correction, float* d_params, const void* d_grads,
                   int grads_are_half, float* d_exp_avg, float* d_exp_avg_sq, size_t numel,
                   float loss_scale, uint16_t* d_param_fp16_out, ps_stream_t stream)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    if (numel > 0 && (!d_params || !d_grads || !d_exp_avg || !d_exp_avg_sq))
        return fail(PS_ERR_BAD_ARG, "ps_adam_update: NULL tensor pointer");
    o->advance(step, beta1, beta2);
    o->set(lr, epsilon, weight_decay);
    if (numel == 0) return 0;
    StepConsts c;
    // the reference clamps gradients in Python before it calls the operator: not here
    finish_consts(c, o->alpha, o->beta1, o->beta2, o->eps, o->weight_decay, o->adamw, o->beta1_t,
                  o->beta2_t, bias_correction != 0, loss_scale, 0.0f);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t gsz = grads_are_half ? 2 : 4;
    const char* gbytes = static_cast<const char*>(d_grads);

    // element-wise pass over [lo, hi)
    auto scalar_span = [&](size_t lo, size_t hi) {
        if (hi <= lo) return;
        const size_t n = hi - lo;
        dim3 grid(grid_1d((n + kAuxBlock - 1) / kAuxBlock)), block(kAuxBlock);
        uint16_t* out = d_param_fp16_out ? d_param_fp16_out + lo : nullptr;
#define PS_FLAT(WD, HALF)                                                                      \
    hipLaunchKernelGGL((adam_flat_kernel<WD, HALF>), grid, block, 0, s, c, d_params + lo,      \
                       static_cast<const void*>(gbytes + lo * gsz), d_exp_avg + lo,            \
                       d_exp_avg_sq + lo, out, n)
        if (grads_are_half) {
            if (c.wd_mode == WD_DECOUPLED) PS_FLAT(WD_DECOUPLED, true);
            else if (c.wd_mode == WD_L2) PS_FLAT(WD_L2, true);
            else PS_FLAT(WD_NONE, true);
        } else {
            if (c.wd_mode == WD_DECOUPLED) PS_FLAT(WD_DECOUPLED, false);
            else if (c.wd_mode == WD_L2) PS_FLAT(WD_L2, false);
            else PS_FLAT(WD_NONE, false);
        }
#undef PS_FLAT
    };

    // Tensors handed to the operator are views at one element offset into the four chunk
    // payloads, so their addresses normally share a phase relative to 16-byte (4-element)
    // boundaries: peel up to 3 leading elements, run whole 256-element tiles with vector
    // accesses, finish the remainder element-wise.
    auto elem_phase = [](const void* a, size_t elem_size) -> int {
        uintptr_t u = reinterpret_cast<uintptr_t>(a);
        if (u % elem_size) return -1;
        return (int)((u / elem_size) & 3u);
    };
    const int ph = elem_phase(d_params, 4);
    bool vec_ok = ph >= 0 && numel >= 4096 && elem_phase(d_exp_avg, 4) == ph &&
                  elem_phase(d_exp_avg_sq, 4) == ph && elem_phase(d_grads, gsz) == ph &&
                  (d_param_fp16_out == nullptr || elem_phase(d_param_fp16_out, 2) == ph);
    if (!vec_ok) {
        scalar_span(0, numel);
    } else {
        const size_t head = (size_t)((4 - ph) & 3);
        const size_t n_tiles = (numel - head) / 256;
        const size_t body_end = head + n_tiles * 256;
        scalar_span(0, head);
        dim3 grid(grid_1d(n_tiles)), block(64);
        uint16_t* out = d_param_fp16_out ? d_param_fp16_out + head : nullptr;
#define PS_FLAT_VEC(WD, HALF)                                                                     \
    hipLaunchKernelGGL((adam_flat_vec_kernel<WD, HALF>), grid, block, kLdsBytes, s, c,            \
                       d_params + head, static_cast<const void*>(gbytes + head * gsz),            \
                       d_exp_avg + head, d_exp_avg_sq + head, out, n_tiles)
        if (grads_are_half) {
            if (c.wd_mode == WD_DECOUPLED) PS_FLAT_VEC(WD_DECOUPLED, true);
            else if (c.wd_mode == WD_L2) PS_FLAT_VEC(WD_L2, true);
            else PS_FLAT_VEC(WD_NONE, true);
        } else {
            if (c.wd_mode == WD_DECOUPLED) PS_FLAT_VEC(WD_DECOUPLED, false);
            else if (c.wd_mode == WD_L2) PS_FLAT_VEC(WD_L2, false);
            else PS_FLAT_VEC(WD_NONE, false);
        }
#undef PS_FLAT_VEC
        scalar_span(body_end, numel);
    }
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_adam_step_chunks(int optimizer_id, size_t step, double lr, double beta1, double beta2,
                        double epsilon, double weight_decay, int bias_correction,
                        const ps_chunk* chunks, int n_chunks, size_t chunk_numel,
                        double loss_scale, ps_stream_t stream)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    ChunkList a;
    if (int rc = make_chunk_list(a, chunks, n_chunks, chunk_numel, kTile)) return rc;
    const HyperParams hp{lr, beta1, beta2, epsilon, weight_decay, loss_scale, bias_correction != 0};
    StepConsts c;
    if (o->arith == PS_ARITH_TORCH)
        c = torch_step_consts(*o, step, hp);
    else
        c = operator_step_consts(*o, step, hp);
    const int arith = o->arith;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return for_each_batch(a, [&](const ChunkBatch& b, dim3 grid) {
        launch_adam_batch(arith, b, grid, chunk_numel, c, s);
    });
}

int ps_adam_step_chunks_gated(int optimizer_id, double lr, double epsilon, double weight_decay,
                              int bias_correction, const ps_chunk* chunks, int n_chunks,
                              size_t chunk_numel, const ps_step_state* d_state,
                              ps_stream_t stream)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    ChunkList a;
    if (int rc = make_chunk_list(a, chunks, n_chunks, chunk_numel, kTile)) return rc;
    const GatedArgs ga = gated_args(*o, lr, epsilon, weight_decay, bias_correction);
    const int arith = o->arith;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return for_each_batch(a, [&](const ChunkBatch& b, dim3 grid) {
        launch_gated_batch(arith, b, grid, chunk_numel, ga, d_state, s);
    });
}

int ps_restore_fp16_chunks(const ps_chunk* chunks, int n_chunks, size_t chunk_numel,
                           const ps_step_state* d_state, ps_stream_t stream)
{
    ChunkList a;
    if (int rc = make_chunk_list(a, chunks, n_chunks, chunk_numel, kTile)) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return for_each_batch(a, [&](const ChunkBatch& b, dim3 grid) {
        hipLaunchKernelGGL(restore_chunks_kernel, grid, dim3(kBlock), 0, s, b, chunk_numel, d_state);
    });
}

int ps_cast_fp32_to_fp16(const float* d_src, uint16_t* d_dst, size_t numel, ps_stream_t stream)
{
    if (numel == 0) return 0;
    if (!d_src || !d_dst) return fail(PS_ERR_BAD_ARG, "ps_cast_fp32_to_fp16: NULL pointer");
    size_t n_tiles = (numel + kTile - 1) / kTile;
    hipLaunchKernelGGL(cast_kernel, dim3(grid_1d(n_tiles)), dim3(kBlock), 0,
                       static_cast<hipStream_t>(stream), d_src, d_dst, numel, n_tiles);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_adam_step_hybrid(int optimizer_id, size_t step, double lr, double beta1, double beta2,
                        double epsilon, double weight_decay, int bias_correction,
                        const ps_chunk* chunks, int n_chunks, const ps_chunk* host_chunks,
                        int n_host_chunks, size_t chunk_numel, const ps_chunk* staging, int n_slots,
                        double loss_scale, const ps_step_state* d_state, ps_stream_t stream)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    ChunkList resident, host;
    if (int rc = make_chunk_list(resident, chunks, n_chunks, chunk_numel, kTile)) return rc;
    if (int rc = make_chunk_list(host, host_chunks, n_host_chunks, chunk_numel, kTile, false, "host chunk")) return rc;
    std::unique_ptr<bool[]> fp16_in_hbm(new bool[n_host_chunks > 0 ? n_host_chunks : 1]);
    if (n_host_chunks > 0) {
        if (int rc = check_slots(staging, n_slots, true, false)) return rc;
        bool any_on_host = false;
        if (int rc = fp16_payloads_in_hbm(host_chunks, n_host_chunks, fp16_in_hbm.get(), &any_on_host)) return rc;
        if (any_on_host)
            if (int rc = check_slots(staging, n_slots, true, true)) return rc;
    }
    // Resident chunks take the optimizer's arithmetic, streamed host chunks the operator's (the
    // reference updates those with the operator).  The operator's step scalars advance once for
    // the whole list, and only if the operator's arithmetic is used at all.
    const int arith = o->arith;
    StepConsts c_resident, c_host;
    const GatedArgs ga = gated_args(*o, lr, epsilon, weight_decay, bias_correction);
    if (d_state == nullptr) {
        const HyperParams hp{lr, beta1, beta2, epsilon, weight_decay, loss_scale, bias_correction != 0};
        if (arith == PS_ARITH_OPERATOR || n_host_chunks > 0) c_host = operator_step_consts(*o, step, hp);
        c_resident = arith == PS_ARITH_TORCH ? torch_step_consts(*o, step, hp) : c_host;
    }
    hipStream_t caller = static_cast<hipStream_t>(stream);
    const bool stream_host = n_host_chunks > 0 && chunk_numel > 0;
    Pipeline* p = nullptr;
    if (stream_host) {
        if (int rc = get_pipeline(&p)) return rc;
        // Everything the caller queued so far (gradients written, the device flag set) comes
        // first; the resident chunks' kernels, queued next, do NOT hold the copies back.
        PS_HIP(hipEventRecord(p->entry, caller));
        PS_HIP(hipStreamWaitEvent(p->h2d, p->entry, 0));
        PS_HIP(hipStreamWaitEvent(p->compute, p->entry, 0));
    }
    int rc = for_each_batch(resident, [&](const ChunkBatch& b, dim3 grid) {
        if (d_state == nullptr)
            launch_adam_batch(arith, b, grid, chunk_numel, c_resident, caller);
        else
            launch_gated_batch(arith, b, grid, chunk_numel, ga, d_state, caller);
    });
    if (rc) return rc;
    if (!stream_host) return 0;

    const size_t b32 = chunk_numel * sizeof(float), b16 = chunk_numel * sizeof(uint16_t);
    for (int i = 0; i < kMaxSlots; ++i) p->slot_used[i] = false;
    for (int k = 0; k < n_host_chunks; ++k) {
        const int s = k % n_slots;
        const ps_chunk& h = host_chunks[k];
        ps_chunk d = staging[s];
        // a fp16 payload that already lives in HBM is read and written in place: 12 instead of
        // 14 bytes per element cross the link in each direction
        const bool stage_fp16 = !fp16_in_hbm[k];
        if (!stage_fp16) d.param_fp16 = h.param_fp16;
        // the slot is free once its previous occupant has been written back
        if (p->slot_used[s]) PS_HIP(hipStreamWaitEvent(p->h2d, p->d2h_done[s], 0));
        if (stage_fp16)
            PS_HIP(hipMemcpyAsync(d.param_fp16, h.param_fp16, b16, hipMemcpyHostToDevice, p->h2d));
        PS_HIP(hipMemcpyAsync(d.param_fp32, h.param_fp32, b32, hipMemcpyHostToDevice, p->h2d));
        PS_HIP(hipMemcpyAsync(d.exp_avg, h.exp_avg, b32, hipMemcpyHostToDevice, p->h2d));
        PS_HIP(hipMemcpyAsync(d.exp_avg_sq, h.exp_avg_sq, b32, hipMemcpyHostToDevice, p->h2d));
        PS_HIP(hipEventRecord(p->h2d_done[s], p->h2d));

        PS_HIP(hipStreamWaitEvent(p->compute, p->h2d_done[s], 0));
        ChunkBatch b;
        memset(&b, 0, sizeof(b));
        b.c[0] = d;
        dim3 grid((unsigned)host.tiles_per_chunk, 1);
        if (d_state == nullptr)
            launch_adam_batch(PS_ARITH_OPERATOR, b, grid, chunk_numel, c_host, p->compute);
        else
            launch_gated_batch(PS_ARITH_OPERATOR, b, grid, chunk_numel, ga, d_state, p->compute);
        PS_HIP(hipGetLastError());
        PS_HIP(hipEventRecord(p->compute_done[s], p->compute));

        PS_HIP(hipStreamWaitEvent(p->d2h, p->compute_done[s], 0));
        // (on a device-skipped step fp32 param / m / v come back unchanged; copying them anyway
        // keeps the host free of any knowledge of the flag)
        if (stage_fp16)
            PS_HIP(hipMemcpyAsync(h.param_fp16, d.param_fp16, b16, hipMemcpyDeviceToHost, p->d2h));
        PS_HIP(hipMemcpyAsync(h.param_fp32, d.param_fp32, b32, hipMemcpyDeviceToHost, p->d2h));
        PS_HIP(hipMemcpyAsync(h.exp_avg, d.exp_avg, b32, hipMemcpyDeviceToHost, p->d2h));
        PS_HIP(hipMemcpyAsync(h.exp_avg_sq, d.exp_avg_sq, b32, hipMemcpyDeviceToHost, p->d2h));
        PS_HIP(hipEventRecord(p->d2h_done[s], p->d2h));
        p->slot_used[s] = true;
    }
    // later work on the caller's stream sees every chunk written back
    for (int s = 0; s < n_slots; ++s)
        if (p->slot_used[s]) PS_HIP(hipStreamWaitEvent(caller, p->d2h_done[s], 0));
    return 0;
}

int ps_overflow_scan_host_chunks(const ps_chunk* host_chunks, int n_chunks, size_t chunk_numel,
                                 const ps_chunk* staging, int n_slots, ps_step_state* d_state,
                                 ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    ChunkList a;
    if (int rc = make_chunk_list(a, host_chunks, n_chunks, chunk_numel, kScanTile, true, "host chunk")) return rc;
    if (n_chunks == 0 || chunk_numel == 0) return 0;
    std::unique_ptr<bool[]> fp16_in_hbm(new bool[n_chunks]);
    bool any_on_host = false;
    if (int rc = fp16_payloads_in_hbm(host_chunks, n_chunks, fp16_in_hbm.get(), &any_on_host)) return rc;
    hipStream_t caller = static_cast<hipStream_t>(stream);
    const size_t b16 = chunk_numel * sizeof(uint16_t);
    const size_t n_tiles = a.tiles_per_chunk;
    // fp16 payloads that live in HBM are probed in place on the caller's stream
    for (int k = 0; k < n_chunks; ++k) {
        if (!fp16_in_hbm[k]) continue;
        hipLaunchKernelGGL(scan_f16_kernel, dim3(grid_1d(n_tiles)), dim3(kAuxBlock), 0, caller,
                           host_chunks[k].param_fp16, chunk_numel, n_tiles, d_state);
        PS_HIP(hipGetLastError());
    }
    if (!any_on_host) return 0;
    if (int rc = check_slots(staging, n_slots, false, true)) return rc;
    Pipeline* p = nullptr;
    if (int rc = get_pipeline(&p)) return rc;
    PS_HIP(hipEventRecord(p->entry, caller));
    PS_HIP(hipStreamWaitEvent(p->h2d, p->entry, 0));
    PS_HIP(hipStreamWaitEvent(p->compute, p->entry, 0));
    for (int i = 0; i < kMaxSlots; ++i) p->slot_used[i] = false;
    int streamed = 0;
    for (int k = 0; k < n_chunks; ++k) {
        if (fp16_in_hbm[k]) continue;
        const int s = streamed++ % n_slots;
        if (p->slot_used[s]) PS_HIP(hipStreamWaitEvent(p->h2d, p->compute_done[s], 0));
        PS_HIP(hipMemcpyAsync(staging[s].param_fp16, host_chunks[k].param_fp16, b16,
                              hipMemcpyHostToDevice, p->h2d));
        PS_HIP(hipEventRecord(p->h2d_done[s], p->h2d));
        PS_HIP(hipStreamWaitEvent(p->compute, p->h2d_done[s], 0));
        hipLaunchKernelGGL(scan_f16_kernel, dim3(grid_1d(n_tiles)), dim3(kAuxBlock), 0, p->compute,
                           staging[s].param_fp16, chunk_numel, n_tiles, d_state);
        PS_HIP(hipGetLastError());
        PS_HIP(hipEventRecord(p->compute_done[s], p->compute));
        p->slot_used[s] = true;
    }
    for (int s = 0; s < n_slots; ++s)
        if (p->slot_used[s]) PS_HIP(hipStreamWaitEvent(caller, p->compute_done[s], 0));
    return 0;
}

int ps_state_init(ps_step_state* d_state, double init_scale, int init_is_int, double scale_factor,
                  int factor_is_int, int64_t scale_window, double min_scale, int min_is_int,
                  int delayed_shift, int consecutive_hysteresis, double beta1, double beta2,
                  ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    if (scale_window <= 0)
        return fail(PS_ERR_BAD_ARG, "scale_window = %lld must be positive", (long long)scale_window);
    ps_step_state s;
    memset(&s, 0, sizeof(s));
    s.cur_scale = init_scale;
    s.scale_is_int = init_is_int != 0;
    s.scale_factor = scale_factor;
    s.factor_is_int = factor_is_int != 0;
    s.min_scale = min_scale;
    s.min_is_int = min_is_int != 0;
    s.cur_iter = 0;
    s.last_overflow_iter = -1;
    s.scale_window = scale_window;
    s.delayed_shift = delayed_shift;
    s.cur_hysteresis = delayed_shift;
    s.consecutive_hysteresis = consecutive_hysteresis != 0;
    s.beta1 = (float)beta1;
    s.beta2 = (float)beta2;
    // Adam_Optimizer starts with beta^t = 1 and step 0; the first update multiplies once.
    s.beta1_t_next = 1.0f * s.beta1;
    s.beta2_t_next = 1.0f * s.beta2;
    s.beta1_f64 = beta1;
    s.beta2_f64 = beta2;
    s.bias_correction1_next = 1.0 - std::pow(beta1, 1.0);
    s.bias_correction2_next = 1.0 - std::pow(beta2, 1.0);
    hipLaunchKernelGGL(state_init_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                       d_state, s);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_state_seed_step(ps_step_state* d_state, int64_t adam_step, double beta1, double beta2,
                       ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    if (adam_step < 0) return fail(PS_ERR_BAD_ARG, "adam_step is negative");
    SeedArgs a;
    a.adam_step = adam_step;
    a.beta1 = (float)beta1;
    a.beta2 = (float)beta2;
    if (adam_step == 0) {
        a.b1t_next = 1.0f * a.beta1;
        a.b2t_next = 1.0f * a.beta2;
    } else {
        // a fresh native object that is first asked for step adam_step + 1 takes the pow branch
        a.b1t_next = (float)std::pow((double)a.beta1, (double)(adam_step + 1));
        a.b2t_next = (float)std::pow((double)a.beta2, (double)(adam_step + 1));
    }
    a.beta1_f64 = beta1;
    a.beta2_f64 = beta2;
    a.bc1_next = 1.0 - std::pow(beta1, (double)(adam_step + 1));
    a.bc2_next = 1.0 - std::pow(beta2, (double)(adam_step + 1));
    hipLaunchKernelGGL(state_seed_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                       d_state, a);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_state_set_scaler(ps_step_state* d_state, double cur_scale, int scale_is_int,
                        int64_t cur_iter, int64_t last_overflow_iter, int cur_hysteresis,
                        ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    hipLaunchKernelGGL(state_set_scaler_kernel, dim3(1), dim3(64), 0,
                       static_cast<hipStream_t>(stream), d_state, cur_scale, scale_is_int, cur_iter,
                       last_overflow_iter, cur_hysteresis);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_overflow_scan(const uint16_t* d_grads_fp16, size_t numel, ps_step_state* d_state,
                     ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    if (numel == 0) return 0;
    if (!d_grads_fp16) return fail(PS_ERR_BAD_ARG, "d_grads_fp16 is NULL");
    size_t n_tiles = (numel + kScanTile - 1) / kScanTile;
    hipLaunchKernelGGL(scan_f16_kernel, dim3(grid_1d(n_tiles)), dim3(kAuxBlock), 0,
                       static_cast<hipStream_t>(stream), d_grads_fp16, numel, n_tiles, d_state);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_overflow_scan_f32(const float* d_grads_fp32, size_t numel, ps_step_state* d_state,
                         ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    if (numel == 0) return 0;
    if (!d_grads_fp32) return fail(PS_ERR_BAD_ARG, "d_grads_fp32 is NULL");
    size_t blocks = (numel + (size_t)kAuxBlock * 16 - 1) / ((size_t)kAuxBlock * 16);
    hipLaunchKernelGGL(scan_f32_kernel, dim3(grid_1d(blocks)), dim3(kAuxBlock), 0,
                       static_cast<hipStream_t>(stream), d_grads_fp32, numel, d_state);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_overflow_scan_chunks(const ps_chunk* chunks, int n_chunks, size_t chunk_numel,
                            ps_step_state* d_state, ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    ChunkList a;
    if (int rc = make_chunk_list(a, chunks, n_chunks, chunk_numel, kScanTile)) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return for_each_batch(a, [&](const ChunkBatch& b, dim3 grid) {
        hipLaunchKernelGGL(scan_chunks_kernel, grid, dim3(kAuxBlock), 0, s, b, chunk_numel, d_state);
    });
}

int ps_grad_to_chunk(const void* d_grad, int grad_is_half, uint16_t* d_slot_fp16, size_t numel,
                     ps_step_state* d_state, ps_stream_t stream)
{
    if (numel == 0) return 0;
    if (!d_grad || !d_slot_fp16) return fail(PS_ERR_BAD_ARG, "ps_grad_to_chunk: NULL pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t esz = grad_is_half ? 2 : 4;
    const char* gbytes = static_cast<const char*>(d_grad);

    auto scalar_span = [&](size_t lo, size_t hi) {
        if (hi <= lo) return;
        const size_t n = hi - lo;
        size_t blocks = (n + (size_t)kAuxBlock * 4 - 1) / ((size_t)kAuxBlock * 4);
        dim3 grid(grid_1d(blocks)), block(kAuxBlock);
        const void* src = gbytes + lo * esz;
        if (grad_is_half)
            hipLaunchKernelGGL(grad_to_chunk_kernel<true>, grid, block, 0, s, src, d_slot_fp16 + lo, n, d_state);
        else
            hipLaunchKernelGGL(grad_to_chunk_kernel<false>, grid, block, 0, s, src, d_slot_fp16 + lo, n, d_state);
    };

    const uintptr_t dst = reinterpret_cast<uintptr_t>(d_slot_fp16);
    const uintptr_t src = reinterpret_cast<uintptr_t>(d_grad);
    const bool addressable = (dst % 2 == 0) && (src % esz == 0);
    if (!addressable || numel < 4096) {
        scalar_span(0, numel);
    } else {
        // elements before the slot's first 16-byte boundary, whole 8-element vectors, remainder
        const size_t head = (size_t)(((16 - dst % 16) % 16) / 2);
        const size_t n_vec = (numel - head) / 8;
        const size_t body_end = head + n_vec * 8;
        scalar_span(0, head);
        size_t blocks = (n_vec + kAuxBlock - 1) / kAuxBlock;
        dim3 grid(grid_1d(blocks)), block(kAuxBlock);
        uint16_t* dst_al = d_slot_fp16 + head;
        if (grad_is_half) {
            const uintptr_t first = src + head * 2;
            const int shift = (int)((first % 16) / 2);
            const uint16_t* src_al = reinterpret_cast<const uint16_t*>(first - (uintptr_t)shift * 2);
            hipLaunchKernelGGL(grad_to_chunk_f16_vec_kernel, grid, block, 0, s, src_al, shift, dst_al, n_vec, d_state);
        } else {
            hipLaunchKernelGGL(grad_to_chunk_f32_vec_kernel, grid, block, 0, s,
                               static_cast<const float*>(d_grad) + head, dst_al, n_vec, d_state);
        }
        scalar_span(body_end, numel);
    }
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_scaler_update(ps_step_state* d_state, int flag_mode, ps_scale_record* d_log,
                     int64_t log_capacity, ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    if (flag_mode < 0 || flag_mode > 2) return fail(PS_ERR_BAD_ARG, "flag_mode = %d", flag_mode);
    if (d_log != nullptr && log_capacity <= 0)
        return fail(PS_ERR_BAD_ARG, "log_capacity must be positive when d_log is given");
    hipLaunchKernelGGL(scaler_update_kernel, dim3(1), dim3(64), 0,
                       static_cast<hipStream_t>(stream), d_state, flag_mode, d_log, log_capacity);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_state_read(const ps_step_state* d_state, ps_step_state* host_out, ps_stream_t stream)
{
    if (!d_state || !host_out) return fail(PS_ERR_BAD_ARG, "ps_state_read: NULL pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    PS_HIP(hipMemcpyAsync(host_out, d_state, sizeof(ps_step_state), hipMemcpyDeviceToHost, s));
    PS_HIP(hipStreamSynchronize(s));
    return 0;
}

}  // extern "C"
