// The kernels: fused chunk-list step (host-decided and device-gated), restore / cast, flat-tensor operator, inf/nan probe, gradient-to-chunk copy, step-state maintenance.
#ifndef PS_KERNELS_H
#define PS_KERNELS_H

#include "ps_tile.h"

namespace {

// ------------------------------------------------------- chunk-list kernels
//
// Grid: x = tile inside a chunk, y = chunk inside the batch.  Up to kBatch
// descriptors are passed BY VALUE in the kernel-argument segment.

constexpr int kBatch = 64;
struct ChunkBatch {
    ps_chunk c[kBatch];
    size_t n[kBatch];  // elements of each chunk the launch covers: the chunk's length, or less when only zeros follow
};
static_assert(sizeof(ps_chunk) == 32 && sizeof(ps_step_state) == 256 && sizeof(ps_scale_record) == 16 &&
                  sizeof(ps_call_pattern) == 32 && sizeof(ps_tensor_call) == 56,
              "layout of the boundary structs");

// Host-decided step: all scalars arrive as kernel arguments and the
// arithmetic variant is a compile-time property of the kernel.
// The span of the step's first operator call, as seen from this workgroup's chunk (empty elsewhere).
__device__ __forceinline__ void first_call_span(const FirstCall& fc, size_t* lo, size_t* hi)
{
    const bool here = fc.chunk == (int)blockIdx.y;
    *lo = here ? (size_t)fc.lo : 0;
    *hi = here ? (size_t)fc.hi : 0;
}

template <int ARITH, int WD, int UNS>
__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    adam_chunks_kernel(ChunkBatch b, StepConsts c, FirstCall fc)
{
    // b.n: the host has already decided whether the zeros behind a chunk's last tensor may be left alone
    const size_t numel = b.n[blockIdx.y];
    const size_t base = (size_t)blockIdx.x * kTile;
    if (base >= numel) return;  // the grid is as wide as the longest chunk of the batch
    size_t lo, hi;
    first_call_span(fc, &lo, &hi);
    adam_tile<ARITH, WD, UNS>(c, b.c[blockIdx.y], base, numel, lo, hi);
}

struct GatedArgs {
    double lr, eps, wd;  // the Python numbers; the operator's arithmetic narrows them to float
    double grad_clamp;
    int64_t n_calls;  // operator calls the reference makes in this step (its tensors); <= 1: the list is one call
    int adamw;
    int bias_correction;
};

// Device-decided step: overflow flag, loss scale and beta^t come from the
// device-resident state; a flagged step restores fp16 from fp32 instead.
// The weight-decay form is known to the host; the unscale form depends on
// the device-resident scale and is a uniform branch around the arithmetic.
// Step constants of a device-decided step, formed by every wave from the device-resident state.
// `with_first_call`: this workgroup's chunk (tensor) holds elements of the step's first operator call; every
// other workgroup is spared the second pair of bias scalars (a divide and a square root per wave).
// What a device-decided step reads from the device-resident state, fetched in one go (a handful of wide scalar
// loads issued together) instead of field by field as the arithmetic gets to them.
struct StateView {
    double cur_scale, beta1_f64, beta2_f64, bc1_next, bc2_next;
    float beta1, beta2, b1t_next, b2t_next, b1t_rest, b2t_rest;
    uint32_t overflow;
};
__device__ __forceinline__ StateView view_state(const ps_step_state* __restrict__ st)
{
    StateView s;
    s.overflow = st->overflow;
    s.cur_scale = st->cur_scale;
    s.beta1 = st->beta1;
    s.beta2 = st->beta2;
    s.b1t_next = st->beta1_t_next;
    s.b2t_next = st->beta2_t_next;
    s.b1t_rest = st->beta1_t_rest;
    s.b2t_rest = st->beta2_t_rest;
    s.beta1_f64 = st->beta1_f64;
    s.beta2_f64 = st->beta2_f64;
    s.bc1_next = st->bias_correction1_next;
    s.bc2_next = st->bias_correction2_next;
    return s;
}

template <int ARITH>
__device__ __forceinline__ StepConsts gated_consts(const GatedArgs& ga, const StateView& st, bool with_first_call)
{
    StepConsts c;
    const float clip = clamp_bound(ga.grad_clamp, st.cur_scale);
    if (ARITH == PS_ARITH_OPERATOR) {
        // The operator takes its scalars and loss_scale as C floats: the Python numbers narrow (RNE).
        // one operator call in the step: everything is that (first) call
        const bool one_call = ga.n_calls <= 1;
        const float b1t = one_call ? st.b1t_next : st.b1t_rest;
        const float b2t = one_call ? st.b2t_next : st.b2t_rest;
        finish_consts(c, (float)ga.lr, st.beta1, st.beta2, (float)ga.eps, (float)ga.wd, ga.adamw != 0, b1t, b2t,
                      ga.bias_correction != 0, (float)st.cur_scale, clip);
        if (with_first_call && !one_call)
            bias_scalars((float)ga.lr, st.b1t_next, st.b2t_next, ga.bias_correction != 0, &c.first_step_size,
                         &c.first_bc2inv);
    } else {
        const bool bc = ga.bias_correction != 0;
        torch_consts(c, ga.lr, st.beta1_f64, st.beta2_f64, ga.eps, ga.wd, ga.adamw != 0, bc ? st.bc1_next : 1.0,
                     bc ? st.bc2_next : 1.0, st.cur_scale, clip);
    }
    return c;
}

// Zeros in all four lists stay zeros under these constants (so the padding behind a chunk's last tensor need not
// be touched): the denominator sqrt(0) * bc2inv + eps is a positive number and nothing multiplies a zero by an
// infinity or a NaN.  With eps == 0 the reference's arithmetic writes 0 / 0 into the padding; then it is computed.
__host__ __device__ inline bool zeros_are_a_fixed_point(const StepConsts& c)
{
    const float s = c.step_size + c.first_step_size + c.bc2inv + c.first_bc2inv + c.wd_term + c.scale + c.beta1 +
                    c.beta2 + c.b1m + c.b2m + c.eps;
    return c.eps > 0.0f && (s - s) == 0.0f;  // every term finite (no NaN, and no infinities: inf - inf is NaN)
}

template <int ARITH, int WD>
__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    adam_chunks_gated_kernel(ChunkBatch b, size_t chunk_numel, GatedArgs ga, FirstCall fc,
                             const ps_step_state* __restrict__ st)
{
    const ps_chunk& ch = b.c[blockIdx.y];
    const size_t base = (size_t)blockIdx.x * kTile;
    size_t numel = b.n[blockIdx.y];  // what lies behind it is zeros in all four lists
    const StateView sv = view_state(st);
    if (sv.overflow) {
        restore_tile(ch.param_fp32, ch.param_fp16, base, numel);  // RNE(0) = 0 is already there
        return;
    }
    const bool here = fc.chunk == (int)blockIdx.y;
    size_t lo, hi;
    first_call_span(fc, &lo, &hi);
    if (base + kTile > numel && numel < chunk_numel) {
        // a tile that reaches into the padding: leave the zeros alone only if they are a fixed point of this step
        if (!zeros_are_a_fixed_point(gated_consts<ARITH>(ga, sv, here))) numel = chunk_numel;
        if (base >= numel) return;
    }
    adam_tile_late_consts<ARITH, WD, UNSCALE_RUNTIME>([&]() { return gated_consts<ARITH>(ga, sv, here); }, ch, base,
                                                      numel, lo, hi);
}

// ------------------------------------------------------- tensor-list kernels
//
// The same tiles over a list of TENSORS of different lengths, for chunk layouts in which a
// parameter's momentum and variance do not sit at the parameter's own offset (the reference packs
// optimizer-state tensors first-fit in parameters() order, patrickstar/core/client.py:282-309, so the
// whole-chunk pass does not apply and the reference loops over tensors, fp16_cpu_adam.py:336-468).
//
// Grid: x = tile inside a tensor, y = tensor inside the batch, exactly like the chunk-list kernels, so that a
// wave reaches its first data load after ONE scalar load of its descriptor.  The host sorts the tensors by length
// and puts tensors of (nearly) the same length into one launch; x runs up to the longest tensor of the batch and
// the few workgroups beyond a shorter tensor's end leave at once.  (A one-dimensional grid over all tiles with a
// tile -> tensor table costs a second dependent scalar load per wave: 4 to 10 % at this kernel's operating point.)
//
// Tensors start at arbitrary element offsets of their chunks.  The tile grid of a tensor is laid over the ADDRESSES
// of its fp32 parameter, not over its element numbers: the up to 255 elements in front of the parameter's first
// 1 KiB boundary form a tile of their own (done element by element), and every later tile is one whole aligned KiB
// of the fp32 parameter (and of every other list that shares the parameter's phase: the fp16 list does in the
// reference's layout).  Wave accesses at a 256-, 512- or 768-byte phase of a KiB measured 6 to 8 % slower than
// aligned ones (all four lists shifted), 2 % with only the fp16 list at a 256-byte phase.  Momentum and variance
// tensors may sit at ANY element phase against their parameter: their 16-byte accesses then go to addresses that are
// only 4-byte aligned (which the hardware serves: 5.7-5.9 TB/s against 6.1 aligned and 3.7 element by element).

constexpr int kTensorBatch = 64;
struct TensorBatch {
    ps_chunk t[kTensorBatch];          // fp32 param, exp_avg, exp_avg_sq, fp16 slot: addresses of the tile grid's origin
    uint64_t numel_head[kTensorBatch]; // low 56 bits: elements from the origin on; high 8 bits: elements in front of it
                                       // (0..255; they are tile 0 of the tensor if there are any)
    int first_call;                    // which tensor of the batch is the step's first operator call; -1: none
};
constexpr uint64_t kNumelMask = (1ull << 56) - 1;

// The elements in front of a tensor's tile grid: indices -head .. -1 relative to the descriptor's addresses.
template <int ARITH, int WD, int UNS>
__device__ __forceinline__ void adam_head(const StepConsts& c, const ps_chunk& t, int head, bool first_call)
{
    const float step_size = first_call ? c.first_step_size : c.step_size;
    const float bc2inv = first_call ? c.first_bc2inv : c.bc2inv;
    for (int j = threadIdx.x; j < head; j += kBlock) {
        const ptrdiff_t i = (ptrdiff_t)j - head;
        float g = half_bits_to_float(t.param_fp16[i]);
        float p = t.param_fp32[i], m = t.exp_avg[i], v = t.exp_avg_sq[i];
        element_any<ARITH, WD, UNS>(c, step_size, bc2inv, g, p, m, v);
        t.param_fp32[i] = p;
        t.exp_avg[i] = m;
        t.exp_avg_sq[i] = v;
        t.param_fp16[i] = (uint16_t)float_to_half_bits(p);
    }
}

template <int ARITH, int WD, int UNS>
__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    adam_tensors_kernel(TensorBatch b, StepConsts c)
{
    const int k = blockIdx.y;
    const uint64_t nh = b.numel_head[k];
    const size_t numel = (size_t)(nh & kNumelMask);
    const int head = (int)(nh >> 56);
    const bool first = k == b.first_call;  // a tensor is one operator call: all of its tiles, or none
    const ptrdiff_t tile = (ptrdiff_t)blockIdx.x - (head ? 1 : 0);
    if (tile < 0) {
        adam_head<ARITH, WD, UNS>(c, b.t[k], head, first);
        return;
    }
    const size_t base = (size_t)tile * kTile;
    if (base >= numel) return;  // the grid is as wide as the longest tensor of the batch
    adam_tile<ARITH, WD, UNS>(c, b.t[k], base, numel, 0, first ? numel : 0);
}

template <int ARITH, int WD>
__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    adam_tensors_gated_kernel(TensorBatch b, GatedArgs ga, const ps_step_state* __restrict__ st)
{
    const int k = blockIdx.y;
    const uint64_t nh = b.numel_head[k];
    const size_t numel = (size_t)(nh & kNumelMask);
    const int head = (int)(nh >> 56);
    const bool first = k == b.first_call;
    const ptrdiff_t tile = (ptrdiff_t)blockIdx.x - (head ? 1 : 0);
    const size_t base = tile < 0 ? 0 : (size_t)tile * kTile;
    if (tile >= 0 && base >= numel) return;
    const StateView sv = view_state(st);
    if (sv.overflow) {
        if (tile < 0) {
            for (int j = threadIdx.x; j < head; j += kBlock)
                b.t[k].param_fp16[(ptrdiff_t)j - head] = (uint16_t)float_to_half_bits(b.t[k].param_fp32[(ptrdiff_t)j - head]);
        } else {
            restore_tile(b.t[k].param_fp32, b.t[k].param_fp16, base, numel);
        }
        return;
    }
    if (tile < 0) {
        adam_head<ARITH, WD, UNSCALE_RUNTIME>(gated_consts<ARITH>(ga, sv, first), b.t[k], head, first);
        return;
    }
    adam_tile_late_consts<ARITH, WD, UNSCALE_RUNTIME>([&]() { return gated_consts<ARITH>(ga, sv, first); }, b.t[k], base,
                                                      numel, 0, first ? numel : 0);
}

// A step whose tensors carry their own step numbers and hyper-parameters: calls that come out with the same constants
// form a class.  One launch takes tensors of ANY class (the launch shape depends on the tensors' lengths only, so a
// list in which every tensor is a class of its own runs like a list with one class); `ClassIndex` says which record
// of the launch's constants each tensor of the batch uses.  What a launch cannot mix is what the kernels are
// compiled for: the arithmetic, the weight-decay form and the way of unscaling.
struct ClassIndex {
    uint16_t k[kTensorBatch];
};

// Host-decided: the constants of up to kLaunchClasses classes travel with the launch (a launch's arguments stay
// under 4 KiB: 2568 bytes of descriptors, 128 of class indices, 24 x 56 of constants).
constexpr int kLaunchClasses = 24;
struct ConstsBatch {
    StepConsts c[kLaunchClasses];
};
static_assert(sizeof(TensorBatch) + sizeof(ClassIndex) + sizeof(ConstsBatch) <= 4096, "kernel arguments of one launch");

// No tensor is "the first call" here: a first call that differs is a class of its own.
template <int ARITH, int WD, int UNS>
__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    adam_tensors_each_kernel(TensorBatch b, ClassIndex ci, ConstsBatch cb)
{
    const int k = blockIdx.y;
    const uint64_t nh = b.numel_head[k];
    const size_t numel = (size_t)(nh & kNumelMask);
    const int head = (int)(nh >> 56);
    const ptrdiff_t tile = (ptrdiff_t)blockIdx.x - (head ? 1 : 0);
    if (tile < 0) {
        adam_head<ARITH, WD, UNS>(cb.c[ci.k[k]], b.t[k], head, false);
        return;
    }
    const size_t base = (size_t)tile * kTile;
    if (base >= numel) return;  // the grid is as wide as the longest tensor of the batch
    adam_tile_late_consts<ARITH, WD, UNS>([&]() { return cb.c[ci.k[k]]; }, b.t[k], base, numel, 0, 0);
}

// The same for tensors whose gradient is binary32 and which have no binary16 copy (PS_TENSOR_GRAD_F32): the
// descriptor's param_fp16 field holds the gradient's address.  Their tile grid starts at the tensor's first element.
template <int ARITH, int WD, int UNS>
__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    adam_tensors_each_f32grad_kernel(TensorBatch b, ClassIndex ci, ConstsBatch cb)
{
    const int k = blockIdx.y;
    const size_t numel = (size_t)(b.numel_head[k] & kNumelMask);
    const size_t base = (size_t)blockIdx.x * kTile;
    if (base >= numel) return;
    const ps_chunk& t = b.t[k];
    adam_tile_f32grad<ARITH, WD, UNS>([&]() { return cb.c[ci.k[k]]; }, t.param_fp32, t.exp_avg, t.exp_avg_sq,
                                      reinterpret_cast<const float*>(t.param_fp16), base, numel);
}

// Device-decided: the constants of every class are formed on the device by plan_consts_kernel (below), one record
// per class in the caller's workspace, before the update kernels run.
struct PlannedConsts {
    StepConsts c;
    float beta1_t, beta2_t;  // the operator object's beta^t after this call (unused by the torch formula)
};
static_assert(sizeof(PlannedConsts) == 64, "one 64-byte record per class in the caller's workspace");

template <int ARITH, int WD>
__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    adam_tensors_planned_kernel(TensorBatch b, ClassIndex ci, const PlannedConsts* __restrict__ consts,
                                const ps_step_state* __restrict__ st)
{
    const int k = blockIdx.y;
    const uint64_t nh = b.numel_head[k];
    const size_t numel = (size_t)(nh & kNumelMask);
    const int head = (int)(nh >> 56);
    const ptrdiff_t tile = (ptrdiff_t)blockIdx.x - (head ? 1 : 0);
    const size_t base = tile < 0 ? 0 : (size_t)tile * kTile;
    if (tile >= 0 && base >= numel) return;
    if (st->overflow) {
        if (tile < 0) {
            for (int j = threadIdx.x; j < head; j += kBlock)
                b.t[k].param_fp16[(ptrdiff_t)j - head] = (uint16_t)float_to_half_bits(b.t[k].param_fp32[(ptrdiff_t)j - head]);
        } else {
            restore_tile(b.t[k].param_fp32, b.t[k].param_fp16, base, numel);
        }
        return;
    }
    if (tile < 0) {
        adam_head<ARITH, WD, UNSCALE_RUNTIME>(consts[ci.k[k]].c, b.t[k], head, false);
        return;
    }
    adam_tile_late_consts<ARITH, WD, UNSCALE_RUNTIME>([&]() { return consts[ci.k[k]].c; }, b.t[k], base, numel, 0, 0);
}

// PS_TENSOR_GRAD_F32 tensors of a device-decided step: a flagged step leaves them alone (there is no fp16 copy to
// restore).
template <int ARITH, int WD>
__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    adam_tensors_planned_f32grad_kernel(TensorBatch b, ClassIndex ci, const PlannedConsts* __restrict__ consts,
                                        const ps_step_state* __restrict__ st)
{
    const int k = blockIdx.y;
    const size_t numel = (size_t)(b.numel_head[k] & kNumelMask);
    const size_t base = (size_t)blockIdx.x * kTile;
    if (base >= numel || st->overflow) return;
    const ps_chunk& t = b.t[k];
    adam_tile_f32grad<ARITH, WD, UNSCALE_RUNTIME>([&]() { return consts[ci.k[k]].c; }, t.param_fp32, t.exp_avg, t.exp_avg_sq,
                                                  reinterpret_cast<const float*>(t.param_fp16), base, numel);
}

__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    restore_chunks_kernel(ChunkBatch b, const ps_step_state* __restrict__ st)
{
    if (st != nullptr && !st->overflow) return;
    const ps_chunk& ch = b.c[blockIdx.y];
    restore_tile(ch.param_fp32, ch.param_fp16, (size_t)blockIdx.x * kTile, b.n[blockIdx.y]);
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
        element_any<PS_ARITH_OPERATOR, WD, UNSCALE_RUNTIME>(c, c.step_size, c.bc2inv, g, p, m, v);
        p32[i] = p;
        m32[i] = m;
        v32[i] = v;
        if (out16) out16[i] = (uint16_t)float_to_half_bits(p);
    }
}

// The same operator with vector accesses: single-wave workgroups over 256-element tiles, one tile per workgroup, the
// resident-workgroup cap and the order "all loads, arithmetic, all stores" of the chunk-list kernels, every variant
// (weight-decay form, unscale form, gradient type, fp16 output or none) a compile-time property so that a wave runs
// straight through.  The tile grid is laid over the ADDRESSES of the fp32 parameter: the pointers are those of the
// parameter's first 1 KiB boundary, so every wave access covers one aligned KiB (tiles at another phase of a KiB
// measured 6 to 8 % slower); the up to 255 elements in front of it (`head`) and the up to 255 behind the last whole
// tile (`tail`) are done element-wise by one extra workgroup of the same launch.  Gradients are read only and must
// share the parameter's 16-byte phase, as must the optional fp16 output.
// STATE_DWORD_ALIGNED: exp_avg / exp_avg_sq sit at another 16-byte phase than the parameter (any element offset).
template <int WD, int UNS, bool GRAD_HALF, bool HAS_OUT, bool STATE_DWORD_ALIGNED>
__global__ void __launch_bounds__(kBlock) PS_OCCUPANCY
    adam_flat_vec_kernel(StepConsts c, float* p32, const void* grads, float* m32, float* v32,
                         uint16_t* out16,  // may alias grads (fp16 gradients overwritten by fp16 parameters)
                         size_t n_tiles, int head, int tail)
{
    static_assert(kBlock == 64 && kLaneElems == 4 && kUnroll == 1, "one wave, one 16-byte access per lane and fp32 array");
    const size_t t = blockIdx.x;
    if (t == n_tiles) {
        for (int j = threadIdx.x; j < head + tail; j += kBlock) {
            const ptrdiff_t i = j < head ? (ptrdiff_t)j - head : (ptrdiff_t)(n_tiles * kTile) + (j - head);
            float g = GRAD_HALF ? half_bits_to_float(static_cast<const uint16_t*>(grads)[i])
                                : static_cast<const float*>(grads)[i];
            float p = p32[i], m = m32[i], v = v32[i];
            adam_element<PS_ARITH_OPERATOR, WD, UNS>(c, c.step_size, c.bc2inv, g, p, m, v);
            p32[i] = p;
            m32[i] = m;
            v32[i] = v;
            if (HAS_OUT) out16[i] = (uint16_t)float_to_half_bits(p);
        }
        return;
    }
    const size_t i = (t * kBlock + threadIdx.x) * 4;
    uint2v w;
    float4v gv;
    if (GRAD_HALF)
        w = *(const guint2v*)(static_cast<const uint16_t*>(grads) + i);
    else
        gv = ld_f4(static_cast<const float*>(grads) + i);
    float4v p = ld_f4(p32 + i), m = ld_f4_as<STATE_DWORD_ALIGNED>(m32 + i), v = ld_f4_as<STATE_DWORD_ALIGNED>(v32 + i);
    float g[4];
    if (GRAD_HALF) {
        g[0] = half_bits_to_float(w[0] & 0xFFFFu);
        g[1] = half_bits_to_float(w[0] >> 16);
        g[2] = half_bits_to_float(w[1] & 0xFFFFu);
        g[3] = half_bits_to_float(w[1] >> 16);
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) g[e] = gv[e];
    }
    uint32_t h[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float pe = p[e], me = m[e], ve = v[e];
        adam_element<PS_ARITH_OPERATOR, WD, UNS>(c, c.step_size, c.bc2inv, g[e], pe, me, ve);
        p[e] = pe;
        m[e] = me;
        v[e] = ve;
        h[e] = float_to_half_bits(pe);
    }
    st_f4(p32 + i, p);
    st_f4_as<STATE_DWORD_ALIGNED>(m32 + i, m);
    st_f4_as<STATE_DWORD_ALIGNED>(v32 + i, v);
    if (HAS_OUT) {
        uint2v o;
        o[0] = h[0] | (h[1] << 16);
        o[1] = h[2] | (h[3] << 16);
        *(guint2v*)(out16 + i) = o;
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
// waves of the block (if it has several), then at most one atomic per block (none when nothing was seen).
template <int BLOCK = kAuxBlock>
__device__ __forceinline__ void block_flag_commit(uint32_t hit, uint32_t* flag)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) hit |= (uint32_t)__shfl_xor((int)hit, off, 64);
    if (BLOCK == 64) {
        if (threadIdx.x == 0 && hit) atomicOr(flag, 1u);
        return;
    }
    __shared__ uint32_t wave_hit[BLOCK / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) wave_hit[wave] = hit;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t any = 0;
#pragma unroll
        for (int w = 0; w < BLOCK / 64; ++w) any |= wave_hit[w];
        if (any) atomicOr(flag, 1u);
    }
}

// Launch shape of the probe kernels that commit to the device flag: threads per workgroup, 16-byte loads per lane,
// and an unused dynamic-LDS request that caps the resident workgroups per CU (0: no cap).
constexpr int kScanBlock = PS_SCAN_BLOCK;
constexpr int kScanUnroll = PS_SCAN_UNROLL;
constexpr int kScanTile = kScanBlock * 8 * kScanUnroll;  // halves per tile
constexpr size_t kScanLdsBytes = (size_t)PS_SCAN_LDS_KB * 1024;
// The two-stage probe keeps one partial word per tile: tiles twice as large, so that the word array stays small, in
// the same single-wave launch shape (probe + reduction over 3.2 GB: 0.490 ms, against 0.512 ms with 256-thread
// workgroups without a cap).
constexpr int kPartialBlock = 64;
constexpr int kPartialUnroll = 16;
constexpr int kPartialTile = kPartialBlock * 8 * kPartialUnroll;  // 8192 halves = 16 KiB per tile

// One scan tile of a fp16 buffer, by a workgroup of BLOCK threads: UNROLL 16-byte loads of 8 halves per lane.
template <int BLOCK, int UNROLL>
__device__ __forceinline__ uint32_t scan_tile_f16(const uint16_t* __restrict__ h, size_t numel,
                                                  size_t tile)
{
    constexpr size_t kTileHalves = (size_t)BLOCK * 8 * UNROLL;
    uint32_t hit = 0;
    const size_t base = tile * kTileHalves;
    if (base >= numel) return 0;
    if ((((uintptr_t)h) & 15u) == 0 && base + kTileHalves <= numel) {
        uint4v w[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            w[u] = ld_u4(h + base + ((size_t)u * BLOCK + threadIdx.x) * 8);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            hit |= nonfinite_halves(w[u][0]) | nonfinite_halves(w[u][1]) |
                   nonfinite_halves(w[u][2]) | nonfinite_halves(w[u][3]);
    } else {
        size_t end = base + kTileHalves < numel ? base + kTileHalves : numel;
        for (size_t i = base + threadIdx.x; i < end; i += BLOCK)
            hit |= ((h[i] & 0x7C00u) == 0x7C00u) ? 1u : 0u;
    }
    return hit;
}

__global__ void __launch_bounds__(kScanBlock)
    scan_f16_kernel(const uint16_t* __restrict__ h, size_t numel, size_t n_tiles,
                    ps_step_state* st)
{
    uint32_t hit = 0;
    for (size_t t = blockIdx.x; t < n_tiles; t += gridDim.x) hit |= scan_tile_f16<kScanBlock, kScanUnroll>(h, numel, t);
    block_flag_commit<kScanBlock>(hit, &st->overflow);
}

// One scan tile of a binary32 buffer (a value is inf or nan iff its eight exponent bits are all set): the same shape,
// UNROLL 16-byte loads of 4 floats per lane.
constexpr int kScanTileF32 = kScanBlock * 4 * kScanUnroll;  // floats per tile

__device__ __forceinline__ uint32_t nonfinite_float(uint32_t w) { return ((w & 0x7F800000u) == 0x7F800000u) ? 1u : 0u; }

template <int BLOCK, int UNROLL>
__device__ __forceinline__ uint32_t scan_tile_f32(const float* __restrict__ f, size_t numel, size_t tile)
{
    constexpr size_t kTileFloats = (size_t)BLOCK * 4 * UNROLL;
    const uint32_t* w32 = reinterpret_cast<const uint32_t*>(f);
    uint32_t hit = 0;
    const size_t base = tile * kTileFloats;
    if (base >= numel) return 0;
    if ((((uintptr_t)f) & 15u) == 0 && base + kTileFloats <= numel) {
        uint4v w[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            w[u] = ld_u4(reinterpret_cast<const uint16_t*>(w32 + base + ((size_t)u * BLOCK + threadIdx.x) * 4));
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            hit |= nonfinite_float(w[u][0]) | nonfinite_float(w[u][1]) | nonfinite_float(w[u][2]) | nonfinite_float(w[u][3]);
    } else {
        size_t end = base + kTileFloats < numel ? base + kTileFloats : numel;
        for (size_t i = base + threadIdx.x; i < end; i += BLOCK) hit |= nonfinite_float(w32[i]);
    }
    return hit;
}

__global__ void __launch_bounds__(kScanBlock)
    scan_f32_kernel(const float* __restrict__ f, size_t numel, size_t n_tiles, ps_step_state* st)
{
    uint32_t hit = 0;
    for (size_t t = blockIdx.x; t < n_tiles; t += gridDim.x) hit |= scan_tile_f32<kScanBlock, kScanUnroll>(f, numel, t);
    block_flag_commit<kScanBlock>(hit, &st->overflow);
}

__global__ void __launch_bounds__(kScanBlock)
    scan_chunks_kernel(ChunkBatch b, ps_step_state* st)
{
    uint32_t hit = scan_tile_f16<kScanBlock, kScanUnroll>(b.c[blockIdx.y].param_fp16, b.n[blockIdx.y], blockIdx.x);
    block_flag_commit<kScanBlock>(hit, &st->overflow);
}

// The same probe without atomics and without a caller-side state: every workgroup leaves the OR over its tile in
// its own word of a partial-result array; a second, small kernel ORs those words into the caller's flag.
__global__ void __launch_bounds__(kPartialBlock)
    scan_chunks_partial_kernel(ChunkBatch b, uint32_t* __restrict__ partial)
{
    static_assert(kPartialBlock == 64, "one wave per workgroup: the shuffle butterfly is the whole reduction");
    uint32_t hit = scan_tile_f16<kPartialBlock, kPartialUnroll>(b.c[blockIdx.y].param_fp16, b.n[blockIdx.y], blockIdx.x);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) hit |= (uint32_t)__shfl_xor((int)hit, off, 64);
    // written unconditionally: the array keeps whatever an earlier call left in it
    if (threadIdx.x == 0) partial[(size_t)blockIdx.y * gridDim.x + blockIdx.x] = hit ? 1u : 0u;
}

constexpr int kReduceBlock = 1024;
__global__ void __launch_bounds__(kReduceBlock)
    scan_reduce_kernel(const uint32_t* __restrict__ partial, size_t n_words, uint32_t* flag)
{
    __shared__ uint32_t wave_hit[kReduceBlock / 64];
    // every workgroup takes one slice of the words; those that find a hit all store the same 1
    const size_t per = (n_words + gridDim.x - 1) / gridDim.x;
    const size_t lo = (size_t)blockIdx.x * per;
    const size_t hi = lo + per < n_words ? lo + per : n_words;
    uint32_t hit = 0;
#pragma unroll 8
    for (size_t i = lo + threadIdx.x; i < hi; i += kReduceBlock) hit |= partial[i];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) hit |= (uint32_t)__shfl_xor((int)hit, off, 64);
    if ((threadIdx.x & 63) == 0) wave_hit[threadIdx.x >> 6] = hit;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t any = 0;
#pragma unroll
        for (int w = 0; w < kReduceBlock / 64; ++w) any |= wave_hit[w];
        if (any) *flag = 1u;  // sticky, like ps_step_state::overflow: only ever set here
    }
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

// Launch shape of the vector copy kernels: threads per workgroup and an unused dynamic-LDS request that caps the
// resident workgroups per CU (0: no cap).
constexpr int kCopyBlock = PS_COPY_BLOCK;
constexpr size_t kCopyLdsBytes = (size_t)PS_COPY_LDS_KB * 1024;

template <int S>
__device__ __forceinline__ uint32_t copy_shifted_f16(const uint16_t* src_al, uint16_t* dst_al,
                                                      size_t n_vec, unsigned body_blocks)
{
    uint32_t hit = 0;
    size_t stride = (size_t)body_blocks * kCopyBlock;
    for (size_t j = (size_t)blockIdx.x * kCopyBlock + threadIdx.x; j < n_vec; j += stride) {
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

// The elements in front of the slot's first 16-byte boundary and behind its last whole vector (at most 7 each), by
// the LAST workgroup of the vector kernels' launch: a gradient costs one launch wherever its slot starts.
struct CopyEdges {
    const void* src;  // the gradient's first element
    uint16_t* dst;    // the slot's first element
    size_t head;      // elements [0, head) and [body_end, numel) go element by element
    size_t body_end, numel;
};

template <bool SRC_HALF>
__device__ __forceinline__ uint32_t copy_edges(const CopyEdges& e)
{
    const uint16_t* sh = static_cast<const uint16_t*>(e.src);
    const float* sf = static_cast<const float*>(e.src);
    const size_t n_edge = e.head + (e.numel - e.body_end);
    uint32_t hit = 0;
    for (size_t j = threadIdx.x; j < n_edge; j += kCopyBlock) {
        const size_t i = j < e.head ? j : e.body_end + (j - e.head);
        uint32_t h = SRC_HALF ? (uint32_t)sh[i] : float_to_half_bits(sf[i]);
        e.dst[i] = (uint16_t)h;
        hit |= ((h & 0x7C00u) == 0x7C00u) ? 1u : 0u;
    }
    return hit;
}

__global__ void __launch_bounds__(kCopyBlock)
    grad_to_chunk_f16_vec_kernel(const uint16_t* __restrict__ src_al, int shift,
                                 uint16_t* __restrict__ dst_al, size_t n_vec, CopyEdges edges, ps_step_state* st)
{
    const unsigned body_blocks = gridDim.x - 1;
    uint32_t hit = 0;
    if (blockIdx.x == body_blocks) {
        hit = copy_edges<true>(edges);
    } else {
        switch (shift) {
            case 0: hit = copy_shifted_f16<0>(src_al, dst_al, n_vec, body_blocks); break;
            case 1: hit = copy_shifted_f16<1>(src_al, dst_al, n_vec, body_blocks); break;
            case 2: hit = copy_shifted_f16<2>(src_al, dst_al, n_vec, body_blocks); break;
            case 3: hit = copy_shifted_f16<3>(src_al, dst_al, n_vec, body_blocks); break;
            case 4: hit = copy_shifted_f16<4>(src_al, dst_al, n_vec, body_blocks); break;
            case 5: hit = copy_shifted_f16<5>(src_al, dst_al, n_vec, body_blocks); break;
            case 6: hit = copy_shifted_f16<6>(src_al, dst_al, n_vec, body_blocks); break;
            default: hit = copy_shifted_f16<7>(src_al, dst_al, n_vec, body_blocks); break;
        }
    }
    if (st != nullptr) block_flag_commit<kCopyBlock>(hit, &st->overflow);
}

// fp32 gradients: eight dword-aligned floats per output vector (multi-dword loads need dword alignment only).
__global__ void __launch_bounds__(kCopyBlock)
    grad_to_chunk_f32_vec_kernel(const float* __restrict__ src, uint16_t* __restrict__ dst_al,
                                 size_t n_vec, CopyEdges edges, ps_step_state* st)
{
    const unsigned body_blocks = gridDim.x - 1;
    uint32_t hit = 0;
    if (blockIdx.x == body_blocks) {
        hit = copy_edges<false>(edges);
    } else {
        size_t stride = (size_t)body_blocks * kCopyBlock;
        for (size_t j = (size_t)blockIdx.x * kCopyBlock + threadIdx.x; j < n_vec; j += stride) {
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
    }
    if (st != nullptr) block_flag_commit<kCopyBlock>(hit, &st->overflow);
}

// ------------------------------------------------ device-resident step state

__global__ void state_init_kernel(ps_step_state* st, ps_step_state init)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) *st = init;
}

struct SeedArgs {
    int64_t adam_step;
    float beta1, beta2, b1t_rest, b2t_rest;
    double beta1_f64, beta2_f64, bc1_next, bc2_next;
    int fresh_operator;
};

__global__ void state_seed_kernel(ps_step_state* st, SeedArgs a)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        // IncrementStep (cpu_adam.h:143-162) for the first call of step adam_step + 1: changed betas restart from
        // pow; else the running product continues only if the object's own step is adam_step
        if (a.fresh_operator) {
            // a new native object (cpu_adam.h:68-86), created with these betas: step 0, beta^t = 1
            st->operator_step = 0;
            st->beta1_t_cur = 1.0f;
            st->beta2_t_cur = 1.0f;
            st->operator_beta1 = a.beta1;
            st->operator_beta2 = a.beta2;
        }
        const bool same_betas = st->operator_beta1 == a.beta1 && st->operator_beta2 == a.beta2;
        const bool follows = same_betas && st->operator_step == a.adam_step;
        st->adam_step = a.adam_step;
        st->beta1 = a.beta1;
        st->beta2 = a.beta2;
        st->beta1_t_next = follows ? st->beta1_t_cur * a.beta1 : a.b1t_rest;
        st->beta2_t_next = follows ? st->beta2_t_cur * a.beta2 : a.b2t_rest;
        st->beta1_t_rest = a.b1t_rest;
        st->beta2_t_rest = a.b2t_rest;
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

// ------------------------------------- per-tensor step numbers: constants of a device-decided step
//
// One distinct call of the step (ps_adam_step_tensors_each): its hyper-parameters, its distance d from the device's
// step counter, and how Adam_Optimizer::IncrementStep (cpu_adam.h:143-162) treats it, which the host can tell from
// the call before it:
//   PLAN_FIRST  the step's first operator call: continues the object's running product if the object, as the last
//               clean step left it, stands at this call's step minus one with the same betas; else pow
//   PLAN_MUL    its step number is the previous call's plus one, same betas: the previous call's beta^t times beta
//   PLAN_POW    anything else: (float)pow((double)beta, step)
//   PLAN_TORCH  the torch formula: 1 - beta ** step in binary64, no operator call
enum { PLAN_POW = 0, PLAN_FIRST = 1, PLAN_MUL = 2, PLAN_TORCH = 3 };
constexpr int32_t PLAN_KIND_MASK = 0xFF;
constexpr int32_t PLAN_GRAD_F32 = 0x100;  // or-ed into PlanClass::mode: the tensors' gradients are binary32 (the clamp bound differs)
struct PlanClass {
    double lr, beta1, beta2, eps, wd;
    int64_t d;     // the call's step number is adam_step + 1 + d
    int32_t mode;  // one of the kinds above, plus PLAN_GRAD_F32
    int32_t prev;  // PLAN_MUL: the class (index in the table) of the call before it
};
constexpr int kPlanBatch = 64;  // one lane per class; 64 x 56 bytes of kernel arguments
struct PlanBatch {
    PlanClass k[kPlanBatch];
};
struct PlanArgs {
    double grad_clamp;
    int64_t last_d;             // of the step's last operator call
    int adamw, bias_correction;
    int first_class, n;         // this launch covers classes [first_class, first_class + n) of the table
    int is_last_launch;         // the launch that leaves the pending record
    int last_operator_class;    // class of the step's last operator call; -1: the step calls the operator for nothing
    float last_beta1, last_beta2;
};

__global__ void __launch_bounds__(64)
    plan_consts_kernel(PlanBatch pb, PlanArgs a, ps_step_state* st, PlannedConsts* table)
{
    __shared__ float b1t_of[kPlanBatch], b2t_of[kPlanBatch];
    const int j = threadIdx.x;
    const int64_t adam_step = st->adam_step;
    const double cur_scale = st->cur_scale;
    const bool bias = a.bias_correction != 0;
    if (j < a.n && (pb.k[j].mode & PLAN_KIND_MASK) != PLAN_MUL) {
        const PlanClass& k = pb.k[j];
        const int kind = k.mode & PLAN_KIND_MASK;
        const float clip = clamp_bound(a.grad_clamp, cur_scale, (k.mode & PLAN_GRAD_F32) != 0);
        const int64_t t = adam_step + 1 + k.d;
        PlannedConsts out;
        if (kind == PLAN_TORCH) {
            torch_consts(out.c, k.lr, k.beta1, k.beta2, k.eps, k.wd, a.adamw != 0, bias ? 1.0 - pow_int(k.beta1, t) : 1.0,
                         bias ? 1.0 - pow_int(k.beta2, t) : 1.0, cur_scale, clip);
            out.beta1_t = out.beta2_t = 0.0f;
        } else {
            const float b1 = (float)k.beta1, b2 = (float)k.beta2;
            const bool follows = kind == PLAN_FIRST && st->operator_beta1 == b1 && st->operator_beta2 == b2 &&
                                 st->operator_step + 1 == t;
            out.beta1_t = follows ? st->beta1_t_cur * b1 : (float)pow_int((double)b1, t);
            out.beta2_t = follows ? st->beta2_t_cur * b2 : (float)pow_int((double)b2, t);
            finish_consts(out.c, (float)k.lr, b1, b2, (float)k.eps, (float)k.wd, a.adamw != 0, out.beta1_t, out.beta2_t,
                          bias, (float)cur_scale, clip);
        }
        b1t_of[j] = out.beta1_t;
        b2t_of[j] = out.beta2_t;
        table[a.first_class + j] = out;
    }
    __syncthreads();
    if (j != 0) return;
    // a call that multiplies needs the call before it: in order, by one lane
    for (int i = 0; i < a.n; ++i) {
        const PlanClass& k = pb.k[i];
        if ((k.mode & PLAN_KIND_MASK) != PLAN_MUL) continue;
        const float clip = clamp_bound(a.grad_clamp, cur_scale, (k.mode & PLAN_GRAD_F32) != 0);
        const int q = k.prev - a.first_class;  // an earlier class: of this launch, or of a launch before it
        const float p1 = q >= 0 ? b1t_of[q] : table[k.prev].beta1_t;
        const float p2 = q >= 0 ? b2t_of[q] : table[k.prev].beta2_t;
        PlannedConsts out;
        const float b1 = (float)k.beta1, b2 = (float)k.beta2;
        out.beta1_t = p1 * b1;
        out.beta2_t = p2 * b2;
        finish_consts(out.c, (float)k.lr, b1, b2, (float)k.eps, (float)k.wd, a.adamw != 0, out.beta1_t, out.beta2_t, bias,
                      (float)cur_scale, clip);
        b1t_of[i] = out.beta1_t;
        b2t_of[i] = out.beta2_t;
        table[a.first_class + i] = out;
    }
    if (!a.is_last_launch) return;
    if (a.last_operator_class < 0) {
        st->pending_operator_step = 0;
        return;
    }
    const int q = a.last_operator_class - a.first_class;
    st->pending_beta1_t = q >= 0 ? b1t_of[q] : table[a.last_operator_class].beta1_t;
    st->pending_beta2_t = q >= 0 ? b2t_of[q] : table[a.last_operator_class].beta2_t;
    st->pending_beta1 = a.last_beta1;
    st->pending_beta2 = a.last_beta2;
    st->pending_operator_step = adam_step + 1 + a.last_d;
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

// DynamicLossScaler.update_scale (loss_scaler.py:158-182), one lane.  `operator_calls`: how many times the
// step that was just queued called the native operator in the reference's terms (its tensors; 0 when every
// chunk took the torch formula): a clean step moves the operator's own step / beta^t state accordingly
// (Adam_Optimizer::IncrementStep, cpu_adam.h:143-162), a skipped step never reaches the operator.
__global__ void scaler_update_kernel(ps_step_state* st, int flag_mode, ps_scale_record* log,
                                     int64_t log_capacity, int64_t operator_calls)
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
        // the step ran: state["step"] += 1
        const int64_t t = s.adam_step + 1;
        s.adam_step = t;
        if (s.pending_operator_step != 0) {
            // a step whose tensors carried their own step numbers and betas: what its last call left
            s.operator_step = s.pending_operator_step;
            s.beta1_t_cur = s.pending_beta1_t;
            s.beta2_t_cur = s.pending_beta2_t;
            s.operator_beta1 = s.pending_beta1;
            s.operator_beta2 = s.pending_beta2;
        } else if (operator_calls >= 1) {
            // what the operator object holds after its last call of step t: the first call's beta^t if it
            // was the only one, else pow(beta, t) from the second call on
            s.beta1_t_cur = operator_calls == 1 ? s.beta1_t_next : s.beta1_t_rest;
            s.beta2_t_cur = operator_calls == 1 ? s.beta2_t_next : s.beta2_t_rest;
            s.operator_step = t;
            s.operator_beta1 = s.beta1;
            s.operator_beta2 = s.beta2;
        }
        // step t + 1: every call after the first evaluates (float)pow((double)beta, t + 1); the first call
        // multiplies the held value by beta if the object's step is t, else it evaluates pow as well
        s.beta1_t_rest = (float)pow_int((double)s.beta1, t + 1);
        s.beta2_t_rest = (float)pow_int((double)s.beta2, t + 1);
        const bool follows = s.operator_step == t && s.operator_beta1 == s.beta1 && s.operator_beta2 == s.beta2;
        s.beta1_t_next = follows ? s.beta1_t_cur * s.beta1 : s.beta1_t_rest;
        s.beta2_t_next = follows ? s.beta2_t_cur * s.beta2 : s.beta2_t_rest;
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
    s.pending_operator_step = 0;
    *st = s;
}

}  // namespace

#endif  // PS_KERNELS_H
