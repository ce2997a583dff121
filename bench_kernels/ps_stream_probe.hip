// MEASUREMENT INSTRUMENT, not part of the optimizer library.
//
// Plain streaming kernels in the launch shape of the fused Adam kernel (single-wave workgroups over
// 256-element tiles, 16-byte accesses per lane, a cap on resident workgroups per CU through an
// unused dynamic-LDS request; 1, 2, 4 or 8 tiles per workgroup), used by `bench.py --mode ceiling` to measure what this GPU's memory
// system delivers for
//   - a pure read stream,
//   - a pure write stream,
//   - one read stream copied into one write stream (1 : 1),
//   - the optimizer step's own access pattern with its arithmetic removed: four arrays (three
//     binary32, one binary16) read and written in place, 28 bytes per element,
// on the same buffers the step runs on.  Built into bench_kernels/libps_stream_probe.so by bench.py
// (build_stream_probe) when `--mode ceiling` first needs it; nothing in the package loads it.
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));
#define PROBE_GLOBAL __attribute__((address_space(1)))

constexpr int kWave = 64;
constexpr int kTileFloats = 256;  // 1 KiB of binary32 per wave instruction

// Every workgroup is one wave and moves U tiles of 256 elements per array (tile t of workgroup b is tile b * U + t:
// U KiB of contiguous binary32 per array); all loads of a workgroup are issued before their first use.
//
// `sink` is never written in practice (no float stream holds the all-ones pattern in all four of a lane's words at
// once); the data-dependent store keeps the loads alive.
template <int U>
__global__ void __launch_bounds__(kWave) read_kernel(const float* __restrict__ src, uint32_t* sink)
{
    const size_t i = (((size_t)blockIdx.x * U) * kWave + threadIdx.x) * 4;
    f4 a[U];
#pragma unroll
    for (int u = 0; u < U; ++u) a[u] = *(const PROBE_GLOBAL f4*)(src + i + (size_t)u * kTileFloats);
    uint32_t x = 0xFFFFFFFFu;
#pragma unroll
    for (int u = 0; u < U; ++u)
        x &= __float_as_uint(a[u][0]) & __float_as_uint(a[u][1]) & __float_as_uint(a[u][2]) & __float_as_uint(a[u][3]);
    if (x == 0xFFFFFFFFu) *sink = x;
}

template <int U>
__global__ void __launch_bounds__(kWave) write_kernel(float* __restrict__ dst, float value)
{
    const size_t i = (((size_t)blockIdx.x * U) * kWave + threadIdx.x) * 4;
    f4 a = {value, value, value, value};
#pragma unroll
    for (int u = 0; u < U; ++u) *(PROBE_GLOBAL f4*)(dst + i + (size_t)u * kTileFloats) = a;
}

template <int U>
__global__ void __launch_bounds__(kWave) copy_kernel(const float* __restrict__ src, float* __restrict__ dst)
{
    const size_t i = (((size_t)blockIdx.x * U) * kWave + threadIdx.x) * 4;
    f4 a[U];
#pragma unroll
    for (int u = 0; u < U; ++u) a[u] = *(const PROBE_GLOBAL f4*)(src + i + (size_t)u * kTileFloats);
#pragma unroll
    for (int u = 0; u < U; ++u) *(PROBE_GLOBAL f4*)(dst + i + (size_t)u * kTileFloats) = a[u];
}

// The step's access pattern: per lane and tile one 16-byte load of each binary32 array and one 8-byte load of
// the binary16 array, a few flops, the same four stores.
template <int U>
__global__ void __launch_bounds__(kWave) update4_kernel(float* p, float* m, float* v, uint16_t* h, float s)
{
    const size_t i = (((size_t)blockIdx.x * U) * kWave + threadIdx.x) * 4;
    u2 g[U];
    f4 a[U], b[U], c[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const size_t j = i + (size_t)u * kTileFloats;
        g[u] = *(const PROBE_GLOBAL u2*)(h + j);
        a[u] = *(const PROBE_GLOBAL f4*)(p + j);
        b[u] = *(const PROBE_GLOBAL f4*)(m + j);
        c[u] = *(const PROBE_GLOBAL f4*)(v + j);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        a[u] = a[u] * s + b[u];
        b[u] = b[u] * s + c[u];
        c[u] = c[u] * s + a[u];
        g[u][0] ^= 0x00010001u;
        g[u][1] ^= 0x00010001u;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const size_t j = i + (size_t)u * kTileFloats;
        *(PROBE_GLOBAL f4*)(p + j) = a[u];
        *(PROBE_GLOBAL f4*)(m + j) = b[u];
        *(PROBE_GLOBAL f4*)(v + j) = c[u];
        *(PROBE_GLOBAL u2*)(h + j) = g[u];
    }
}

int check(size_t n_floats, int tiles_per_wg, int lds_kb, unsigned* grid)
{
    if (tiles_per_wg != 1 && tiles_per_wg != 2 && tiles_per_wg != 4 && tiles_per_wg != 8) return -5;
    const size_t per_wg = (size_t)kTileFloats * tiles_per_wg;
    if (n_floats == 0 || n_floats % per_wg != 0) return -1;  // whole workgroups only: the kernels have no tail path
    if (n_floats / per_wg > 0x7FFFFFFFull) return -2;
    if (lds_kb < 0 || lds_kb > 64) return -3;
    *grid = (unsigned)(n_floats / per_wg);
    return 0;
}

int launched()
{
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

#define PROBE_LAUNCH(KERNEL, ...)                                                                              \
    do {                                                                                                       \
        const dim3 g(grid), b(kWave);                                                                          \
        const size_t lds = (size_t)lds_kb * 1024;                                                              \
        hipStream_t s = static_cast<hipStream_t>(stream);                                                      \
        switch (tiles_per_wg) {                                                                                \
            case 1: hipLaunchKernelGGL(KERNEL<1>, g, b, lds, s, __VA_ARGS__); break;                           \
            case 2: hipLaunchKernelGGL(KERNEL<2>, g, b, lds, s, __VA_ARGS__); break;                           \
            case 4: hipLaunchKernelGGL(KERNEL<4>, g, b, lds, s, __VA_ARGS__); break;                           \
            default: hipLaunchKernelGGL(KERNEL<8>, g, b, lds, s, __VA_ARGS__); break;                          \
        }                                                                                                      \
    } while (0)

}  // namespace

// All sizes in ELEMENTS of binary32 (for update4: elements of every array), multiples of 256 * tiles_per_wg.
// 16-byte aligned device addresses.  tiles_per_wg: 1, 2, 4 or 8.  lds_kb: KiB of unused dynamic LDS requested per
// workgroup (caps resident workgroups per CU at floor(160 / lds_kb); 0: no cap).  Every call only enqueues on
// `stream`.  Returns 0, or a negative code for a size / launch problem.
extern "C" {

int ps_probe_read(const float* d_src, size_t n_floats, uint32_t* d_sink, int tiles_per_wg, int lds_kb, void* stream)
{
    unsigned grid;
    if (int rc = check(n_floats, tiles_per_wg, lds_kb, &grid)) return rc;
    PROBE_LAUNCH(read_kernel, d_src, d_sink);
    return launched();
}

int ps_probe_write(float* d_dst, size_t n_floats, float value, int tiles_per_wg, int lds_kb, void* stream)
{
    unsigned grid;
    if (int rc = check(n_floats, tiles_per_wg, lds_kb, &grid)) return rc;
    PROBE_LAUNCH(write_kernel, d_dst, value);
    return launched();
}

int ps_probe_copy(const float* d_src, float* d_dst, size_t n_floats, int tiles_per_wg, int lds_kb, void* stream)
{
    unsigned grid;
    if (int rc = check(n_floats, tiles_per_wg, lds_kb, &grid)) return rc;
    PROBE_LAUNCH(copy_kernel, d_src, d_dst);
    return launched();
}

int ps_probe_update4(float* d_p, float* d_m, float* d_v, uint16_t* d_h, size_t numel, int tiles_per_wg, int lds_kb,
                     void* stream)
{
    unsigned grid;
    if (int rc = check(numel, tiles_per_wg, lds_kb, &grid)) return rc;
    PROBE_LAUNCH(update4_kernel, d_p, d_m, d_v, d_h, 0.5f);
    return launched();
}

}  // extern "C"
