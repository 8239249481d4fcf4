// Shared device helpers for the gfx950 kernels of libterrace_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "terrace_hip.h"

namespace terrace {

constexpr int kWave = 64;        // CDNA wavefront width
constexpr int kBlock = 256;      // default workgroup: 4 waves
constexpr int kWavesPerBlock = kBlock / kWave;

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }
__device__ __forceinline__ int wave_in_block() { return threadIdx.x >> 6; }

__device__ __forceinline__ uint64_t lanes_below(int lane) { return (1ull << lane) - 1ull; }

// Wave-private LDS words that lanes of one wave exchange values through.  The pointer carries the LDS address
// space in its type: a volatile access through a generic pointer is left as a flat instruction by the compiler,
// through one of these it is a ds_read / ds_write.
typedef __attribute__((address_space(3))) volatile int32_t lds_i32;
typedef __attribute__((address_space(3))) volatile float lds_f32;

// Value held by `src_lane` (uniform across the wave).
__device__ __forceinline__ int read_lane(int v, int src_lane) {
    return __builtin_amdgcn_readlane(v, src_lane);
}

// Butterfly exchange with lane ^ mask.  Distances 1 and 2 use DPP quad permutes, 4, 8 and 16 a
// ds_swizzle in bit mode (and-mask 0x1F, xor-mask the distance), 32 a ds_bpermute.
template <int MASK>
__device__ __forceinline__ int xchg_xor_i(int v) {
    if constexpr (MASK == 1) {
        return __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xF, 0xF, false);   // quad_perm [1,0,3,2]
    } else if constexpr (MASK == 2) {
        return __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xF, 0xF, false);   // quad_perm [2,3,0,1]
    } else if constexpr (MASK == 4) {
        return __builtin_amdgcn_ds_swizzle(v, 0x101F);                     // bit mode: xor 4
    } else if constexpr (MASK == 8) {
        return __builtin_amdgcn_ds_swizzle(v, 0x201F);                     // bit mode: xor 8
    } else if constexpr (MASK == 16) {
        return __builtin_amdgcn_ds_swizzle(v, 0x401F);                     // bit mode: xor 16
    } else {
        return __shfl_xor(v, 32, kWave);
    }
}
template <int MASK>
__device__ __forceinline__ float xchg_xor_f(float v) {
    return __int_as_float(xchg_xor_i<MASK>(__float_as_int(v)));
}

// Wave-wide inclusive/exclusive helpers over ints (used for small scans).
__device__ __forceinline__ int wave_inclusive_scan(int v) {
    const int lane = lane_id();
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        int o = __shfl_up(v, d, kWave);
        if (lane >= d) v += o;
    }
    return v;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x0040u;        // quiet NaN
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;                          // nearest even
}

// e4m3 "fn" (bias 7, no infinities) -> fp32, exact.
__device__ __forceinline__ float e4m3_to_f32(uint32_t c) {
    const uint32_t sign = (c & 0x80u) << 24;
    const uint32_t e = (c >> 3) & 0xFu, m = c & 0x7u;
    float mag = e ? __uint_as_float(((e + 120u) << 23) | (m << 20)) : (float)m * 0x1p-9f;
    if (e == 0xFu && m == 0x7u) mag = __uint_as_float(0x7FC00000u);
    return __uint_as_float(__float_as_uint(mag) | sign);
}

// A row-width argument of the C ABI may carry a pitch (TERRACE_ROW_PITCHED): `width` bytes of data every `pitch`
// bytes.  Packed rows have pitch == width.
struct RowGeom {
    int64_t width, pitch;
    bool pitched() const { return pitch != width; }
};
inline RowGeom row_geom(int64_t row_bytes) {
    RowGeom g{row_bytes & 0xFFFFFFFFll, row_bytes >> 32};
    if (g.pitch == 0) g.pitch = g.width;
    return g;
}
// Pitched rows move through the kilobyte-sliced kernels only: 16-byte-multiple widths on a whole number of
// kilobytes.  (The buffers must also be 16-byte aligned; the launchers check that.)
inline bool row_geom_ok(const RowGeom &g) {
    if (g.width < 0 || g.pitch < g.width) return false;
    return !g.pitched() || (g.width % 16 == 0 && g.pitch % 1024 == 0);
}

inline int check_launch() { return hipGetLastError() == hipSuccess ? TERRACE_OK : TERRACE_ELAUNCH; }

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace terrace
