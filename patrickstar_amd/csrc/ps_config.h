// Build-time tuning knobs of the fused Adam kernels (defaults = measured best on MI355X).
#ifndef PS_CONFIG_H
#define PS_CONFIG_H

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
// Launch shape of the inf/nan probe kernels (pure read streams).  Measured on 3.2 GB of fp16 payloads: single-wave
// workgroups with 8 loads per lane and 6 resident workgroups per CU read 6.85 TB/s; 256 threads x 4 loads, uncapped,
// 6.29 TB/s.
#ifndef PS_SCAN_BLOCK
#define PS_SCAN_BLOCK 64  // threads per workgroup (64 or a multiple of it)
#endif
#ifndef PS_SCAN_UNROLL
#define PS_SCAN_UNROLL 8  // 16-byte loads per lane per tile
#endif
#ifndef PS_SCAN_LDS_KB
#define PS_SCAN_LDS_KB 26  // KiB of unused dynamic LDS per workgroup (0: no cap on resident workgroups)
#endif
// Launch shape of the backward-side gradient copy's vector kernels (one gradient tensor into its chunk slot).  Swept over
// 64 / 128 / 256 threads x 0 / 13 / 17 / 26 KiB on 64 Mi-, 10 Mi- and 2.5 Mi-element gradients: nothing beats 256 threads
// without a cap (fp16 40 us, fp32 71 us for 64 Mi elements; caps only slow single-wave workgroups down).
#ifndef PS_COPY_BLOCK
#define PS_COPY_BLOCK 256  // threads per workgroup
#endif
#ifndef PS_COPY_LDS_KB
#define PS_COPY_LDS_KB 0  // KiB of unused dynamic LDS per workgroup (0: no cap on resident workgroups)
#endif
#if PS_MAX_WAVES_PER_EU > 0
#define PS_OCCUPANCY __attribute__((amdgpu_waves_per_eu(1, PS_MAX_WAVES_PER_EU)))
#else
#define PS_OCCUPANCY
#endif

#endif  // PS_CONFIG_H
