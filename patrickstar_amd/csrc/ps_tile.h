// Vector accesses and the per-workgroup tile: one 256-element tile of one chunk, loaded, updated and stored by one wave.
#ifndef PS_TILE_H
#define PS_TILE_H

#include "ps_arith.h"
#include "ps_config.h"

namespace {

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

// 16 bytes at an address that is only 4-byte aligned (multi-dword global accesses need dword alignment only): for
// momentum / variance tensors that sit at another 16-byte phase than their parameter.
typedef float4v __attribute__((aligned(4))) float4v_dword_aligned;
template <bool DWORD_ALIGNED>
__device__ __forceinline__ float4v ld_f4_as(const float* p)
{
    if (DWORD_ALIGNED) return *(const PS_GLOBAL float4v_dword_aligned*)(p);
    return ld_f4(p);
}
template <bool DWORD_ALIGNED>
__device__ __forceinline__ void st_f4_as(float* p, float4v v)
{
    if (DWORD_ALIGNED)
        *(PS_GLOBAL float4v_dword_aligned*)(p) = v;
    else
        st_f4(p, v);
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
__device__ __forceinline__ void lane_math(const StepConsts& c, float step_size, float bc2inv, LaneTile& r)
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
            adam_element<ARITH, WD, UNS>(c, step_size, bc2inv, g0, p0, m0, v0);
            adam_element<ARITH, WD, UNS>(c, step_size, bc2inv, g1, p1, m1, v1);
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

// One tile of one chunk, fast path: the whole tile is in range, all four
// bases are 16-byte aligned and the whole tile belongs to one operator call
// (step_size / bc2inv are that call's).  All loads of the tile are issued
// before the first use.  Loads and stores are written once, outside any
// branch on the arithmetic variant.
// The loads of one whole, aligned tile: all of them issued back to back, nothing waited for.
// STATE_DWORD_ALIGNED: exp_avg / exp_avg_sq are only 4-byte aligned (the parameter lists are aligned as always).
template <bool STATE_DWORD_ALIGNED = false>
__device__ __forceinline__ void tile_load(LaneTile& r, const float* __restrict__ p32, const float* __restrict__ m32,
                                          const float* __restrict__ v32, const uint16_t* __restrict__ h16, size_t base)
{
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        size_t i = base + ((size_t)u * kBlock + threadIdx.x) * kLaneElems;
        r.g[u] = ld_halves(h16 + i);
#pragma unroll
        for (int q = 0; q < kQuads; ++q) r.p[u][q] = ld_f4(p32 + i + 4 * q);
#pragma unroll
        for (int q = 0; q < kQuads; ++q) r.m[u][q] = ld_f4_as<STATE_DWORD_ALIGNED>(m32 + i + 4 * q);
#pragma unroll
        for (int q = 0; q < kQuads; ++q) r.v[u][q] = ld_f4_as<STATE_DWORD_ALIGNED>(v32 + i + 4 * q);
    }
}

// Arithmetic and stores of a tile whose loads are under way.
template <int ARITH, int WD, int UNS, bool STATE_DWORD_ALIGNED = false>
__device__ __forceinline__ void tile_finish(const StepConsts& c, float step_size, float bc2inv, LaneTile& r,
                                            float* __restrict__ p32, float* __restrict__ m32,
                                            float* __restrict__ v32, uint16_t* __restrict__ h16, size_t base)
{
    if (UNS != UNSCALE_RUNTIME) {
        lane_math<ARITH, WD, UNS>(c, step_size, bc2inv, r);
    } else if (c.unscale == UNSCALE_MUL) {
        lane_math<ARITH, WD, UNSCALE_MUL>(c, step_size, bc2inv, r);
    } else if (ARITH == PS_ARITH_OPERATOR && c.unscale == UNSCALE_DIV) {
        lane_math<ARITH, WD, UNSCALE_DIV>(c, step_size, bc2inv, r);
    } else {
        lane_math<ARITH, WD, UNSCALE_NONE>(c, step_size, bc2inv, r);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        size_t i = base + ((size_t)u * kBlock + threadIdx.x) * kLaneElems;
#pragma unroll
        for (int q = 0; q < kQuads; ++q) st_f4(p32 + i + 4 * q, r.p[u][q]);
#pragma unroll
        for (int q = 0; q < kQuads; ++q) st_f4_as<STATE_DWORD_ALIGNED>(m32 + i + 4 * q, r.m[u][q]);
#pragma unroll
        for (int q = 0; q < kQuads; ++q) st_f4_as<STATE_DWORD_ALIGNED>(v32 + i + 4 * q, r.v[u][q]);
        st_halves(h16 + i, r.h[u]);
    }
}

template <int ARITH, int WD, int UNS, bool STATE_DWORD_ALIGNED = false>
__device__ __forceinline__ void adam_tile_vec(const StepConsts& c, float step_size, float bc2inv,
                                              float* __restrict__ p32, float* __restrict__ m32,
                                              float* __restrict__ v32, uint16_t* __restrict__ h16,
                                              size_t base)
{
    LaneTile r;
    tile_load<STATE_DWORD_ALIGNED>(r, p32, m32, v32, h16, base);
    tile_finish<ARITH, WD, UNS, STATE_DWORD_ALIGNED>(c, step_size, bc2inv, r, p32, m32, v32, h16, base);
}

// Same elements, one at a time: ragged tile ends, unaligned bases and tiles that an operator call's
// boundary runs through (elements [first_lo, first_hi) take the first call's scalars).
template <int ARITH, int WD, int UNS>
__device__ __forceinline__ void adam_tile_scalar(const StepConsts& c, float* p32, float* m32,
                                                 float* v32, uint16_t* h16, size_t base, size_t end,
                                                 size_t first_lo, size_t first_hi)
{
    for (size_t i = base + threadIdx.x; i < end; i += kBlock) {
        float g = half_bits_to_float(h16[i]);
        float p = p32[i], m = m32[i], v = v32[i];
        const bool first = i >= first_lo && i < first_hi;
        element_any<ARITH, WD, UNS>(c, first ? c.first_step_size : c.step_size,
                                    first ? c.first_bc2inv : c.bc2inv, g, p, m, v);
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

// How a whole tile of this chunk / tensor can be accessed: all four lists 16-byte aligned; or the two parameter
// lists aligned (fp32 to 16 bytes, fp16 to the 8 or 16 bytes of its access) and momentum / variance, which sit at
// another phase, only to the 4 bytes of an element; or element by element.
enum { TILE_ALIGNED = 0, TILE_STATE_DWORD_ALIGNED = 1, TILE_ELEMENTWISE = 2 };
__device__ __forceinline__ int tile_access(const ps_chunk& ch)
{
    if (aligned16(ch.param_fp32, ch.exp_avg, ch.exp_avg_sq, ch.param_fp16)) return TILE_ALIGNED;
    const uintptr_t half_mask = kWords == 4 ? 15u : 7u;
    if ((((uintptr_t)ch.param_fp32) & 15u) == 0 && (((uintptr_t)ch.param_fp16) & half_mask) == 0 &&
        ((((uintptr_t)ch.exp_avg) | ((uintptr_t)ch.exp_avg_sq)) & 3u) == 0)
        return TILE_STATE_DWORD_ALIGNED;
    return TILE_ELEMENTWISE;
}

// first_lo .. first_hi: the elements of THIS chunk that the step's first operator call covers
// (first_hi <= first_lo: none).  Whole tiles inside or outside that span are uniform and keep the vector
// path; the at most two tiles that its ends run through go element by element.
// The same with the step constants still to be formed (a device-decided step builds them from the device-resident
// state): `make_consts()` is called AFTER the tile's loads have been issued, so that the scalar loads and the
// divisions and square roots behind the constants run in the shadow of the data loads instead of in front of them.
template <int ARITH, int WD, int UNS, typename MakeConsts>
__device__ __forceinline__ void adam_tile_late_consts(MakeConsts make_consts, const ps_chunk& ch, size_t base,
                                                      size_t chunk_numel, size_t first_lo, size_t first_hi)
{
    size_t end = base + kTile;
    const size_t last = end < chunk_numel ? end : chunk_numel;
    const bool inside = base >= first_lo && last <= first_hi;
    const bool cut = !inside && base < first_hi && last > first_lo;
    const int access = (!cut && end <= chunk_numel) ? tile_access(ch) : TILE_ELEMENTWISE;
    if (access == TILE_ALIGNED) {
        LaneTile r;
        tile_load(r, ch.param_fp32, ch.exp_avg, ch.exp_avg_sq, ch.param_fp16, base);
        const StepConsts c = make_consts();
        tile_finish<ARITH, WD, UNS>(c, inside ? c.first_step_size : c.step_size, inside ? c.first_bc2inv : c.bc2inv, r,
                                    ch.param_fp32, ch.exp_avg, ch.exp_avg_sq, ch.param_fp16, base);
    } else if (access == TILE_STATE_DWORD_ALIGNED) {
        LaneTile r;
        tile_load<true>(r, ch.param_fp32, ch.exp_avg, ch.exp_avg_sq, ch.param_fp16, base);
        const StepConsts c = make_consts();
        tile_finish<ARITH, WD, UNS, true>(c, inside ? c.first_step_size : c.step_size, inside ? c.first_bc2inv : c.bc2inv,
                                          r, ch.param_fp32, ch.exp_avg, ch.exp_avg_sq, ch.param_fp16, base);
    } else {
        const StepConsts c = make_consts();
        adam_tile_scalar<ARITH, WD, UNS>(c, ch.param_fp32, ch.exp_avg, ch.exp_avg_sq, ch.param_fp16, base, last,
                                         first_lo, first_hi);
    }
}

template <int ARITH, int WD, int UNS>
__device__ __forceinline__ void adam_tile(const StepConsts& c, const ps_chunk& ch, size_t base,
                                          size_t chunk_numel, size_t first_lo, size_t first_hi)
{
    size_t end = base + kTile;
    const size_t last = end < chunk_numel ? end : chunk_numel;  // one past the tile's last element
    const bool inside = base >= first_lo && last <= first_hi;
    const bool cut = !inside && base < first_hi && last > first_lo;
    const int access = (!cut && end <= chunk_numel) ? tile_access(ch) : TILE_ELEMENTWISE;
    if (access == TILE_ALIGNED) {
        adam_tile_vec<ARITH, WD, UNS>(c, inside ? c.first_step_size : c.step_size,
                                      inside ? c.first_bc2inv : c.bc2inv, ch.param_fp32, ch.exp_avg,
                                      ch.exp_avg_sq, ch.param_fp16, base);
    } else if (access == TILE_STATE_DWORD_ALIGNED) {
        adam_tile_vec<ARITH, WD, UNS, true>(c, inside ? c.first_step_size : c.step_size,
                                            inside ? c.first_bc2inv : c.bc2inv, ch.param_fp32, ch.exp_avg,
                                            ch.exp_avg_sq, ch.param_fp16, base);
    } else {
        adam_tile_scalar<ARITH, WD, UNS>(c, ch.param_fp32, ch.exp_avg, ch.exp_avg_sq,
                                         ch.param_fp16, base, last, first_lo, first_hi);
    }
}

// One tile of a tensor whose gradient is binary32 and which has no binary16 copy (a parameter that PyTorch manages
// itself, fp16_cpu_adam.py:345-353,459-460): `g32` is only read.  Whole tiles with all four addresses 16-byte
// aligned take one 16-byte access per lane and array, everything else goes element by element.  As in
// adam_tile_late_consts the constants are formed after the loads have been issued.
template <int ARITH, int WD, int UNS, typename MakeConsts>
__device__ __forceinline__ void adam_tile_f32grad(MakeConsts make_consts, float* __restrict__ p32, float* __restrict__ m32,
                                                  float* __restrict__ v32, const float* __restrict__ g32, size_t base,
                                                  size_t numel)
{
    const size_t end = base + kTile;
    if (end <= numel && aligned16(p32, m32, v32, g32)) {
        float4v g[kUnroll][kQuads], p[kUnroll][kQuads], m[kUnroll][kQuads], v[kUnroll][kQuads];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const size_t i = base + ((size_t)u * kBlock + threadIdx.x) * kLaneElems;
#pragma unroll
            for (int q = 0; q < kQuads; ++q) {
                g[u][q] = ld_f4(g32 + i + 4 * q);
                p[u][q] = ld_f4(p32 + i + 4 * q);
                m[u][q] = ld_f4(m32 + i + 4 * q);
                v[u][q] = ld_f4(v32 + i + 4 * q);
            }
        }
        const StepConsts c = make_consts();
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const size_t i = base + ((size_t)u * kBlock + threadIdx.x) * kLaneElems;
#pragma unroll
            for (int q = 0; q < kQuads; ++q) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float pe = p[u][q][e], me = m[u][q][e], ve = v[u][q][e];
                    element_any<ARITH, WD, UNS>(c, c.step_size, c.bc2inv, g[u][q][e], pe, me, ve);
                    p[u][q][e] = pe;
                    m[u][q][e] = me;
                    v[u][q][e] = ve;
                }
                st_f4(p32 + i + 4 * q, p[u][q]);
                st_f4(m32 + i + 4 * q, m[u][q]);
                st_f4(v32 + i + 4 * q, v[u][q]);
            }
        }
    } else {
        const StepConsts c = make_consts();
        const size_t last = end < numel ? end : numel;
        for (size_t i = base + threadIdx.x; i < last; i += kBlock) {
            float p = p32[i], m = m32[i], v = v32[i];
            element_any<ARITH, WD, UNS>(c, c.step_size, c.bc2inv, g32[i], p, m, v);
            p32[i] = p;
            m32[i] = m;
            v32[i] = v;
        }
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

}  // namespace

#endif  // PS_TILE_H
