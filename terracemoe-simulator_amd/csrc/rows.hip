// Row movers: the HBM-bound kernels of the dispatch/combine path.
//
//   copy_kernel                   y = x                           (streaming-copy roofline probe)
//   scatter_rows_{sliced,aligned} dst[pos[r*fan+f]] = src[r]      (Hop-A pack, Hop-B arrival: a source
//                                                                  row is read once and written fan times)
//   gather_rows_{sliced,flat}     out[i] = src[idx[i]] or zeros   (expert-order regroup, capacity padding)
//   combine_kernel                out[i] = sum_j w[i,j]*src[idx[i,j]] in fp32, one rounding at the end
//   planes_kernel                 wire containers: row = a | b | c | zero pad, and the inverse split
//
// Rows that are multiples of 16 bytes move as one 16-byte vector per lane in one-wave workgroups whose
// stores each cover one aligned kilobyte of the destination.  Other widths take scatter_rows_kernel /
// gather_rows_kernel: 256-thread workgroups split into sub-groups of 64/128/256 lanes, a sub-group
// owning one row at a time with 8/4/2/1-byte lanes.  Nothing here is a contraction: no MFMA, no LDS.
#include "common.hpp"

namespace terrace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename V>
__device__ __forceinline__ V ld_stream(const V *p) { return __builtin_nontemporal_load(p); }
template <typename V>
__device__ __forceinline__ void st_stream(V *p, V v) { __builtin_nontemporal_store(v, p); }

template <typename V>
__device__ __forceinline__ V zero_of() { return V(0); }
template <>
__device__ __forceinline__ u32x4 zero_of<u32x4>() { return u32x4{0u, 0u, 0u, 0u}; }

// ---------------------------------------------------------------------------------------------
// streaming copy
// ---------------------------------------------------------------------------------------------
template <typename V, int UNROLL>
__global__ __launch_bounds__(kBlock) void copy_kernel(const V *__restrict__ x, V *__restrict__ y, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * kBlock * UNROLL;
    for (int64_t base = (int64_t)blockIdx.x * kBlock * UNROLL + threadIdx.x; base < n; base += stride) {
        V v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int64_t i = base + (int64_t)u * kBlock;
            if (i < n) v[u] = ld_stream(x + i);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int64_t i = base + (int64_t)u * kBlock;
            if (i < n) st_stream(y + i, v[u]);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// resident waves per CU
// ---------------------------------------------------------------------------------------------
// A one-wave mover uses no LDS and few registers, so a CU would hold 32 of its waves.  The scatters (one read,
// several writes per wave) and the combine of eight rows per output row stream faster with fewer: the memory system
// then sees fewer interleaved streams per CU.  A launch asks for that by reserving dynamic LDS that no kernel
// touches: a CU has 160 KB, and a reservation of 160 KB / n per one-wave workgroup keeps at most n of them resident.
// Launch time relative to no reservation, rows of 2-14 KB, 0.25-2 GB per launch:
//   scatter  fan 1: 24 waves 0.99-1.00, 16 waves 1.04-1.13, 12 waves 1.4  -> no cap (the gathers, likewise one
//            read and one write per wave, lose 19 % at 16 waves)
//            fan 2: 20 waves 0.975 on the arrival's positions (0.99 on a random permutation, where 16 give 0.975)
//            fan 4: 16 waves 0.95 on the pack's positions, 0.975 on a random permutation; fan 8: 0.91
//   combine  8 rows per output row, bf16 / f16 / f32, launches that read 0.5 GB or more: 12 waves 0.95-0.98,
//            16 waves 0.99; launches the 256 MB memory-side cache holds lose up to 40 % at 12 waves, and so do 2 or
//            4 rows per output row at any size (fewer loads in flight per wave: 12 waves 1.06-1.4) and fp8 rows,
//            whose scale loads want the waves (12 waves 1.05), and so does a table of mostly dead entries (the
//            two-level combine on the general branch's table: 1.75) -> capped only where it gains
// While such a launch runs, its waves hold most of a CU's LDS: a kernel that another stream runs beside it and that
// needs LDS gets a CU's share only as mover waves retire (each lives a few microseconds).
constexpr size_t kLdsPerCu = 160 * 1024;
constexpr size_t lds_for_waves(int waves) { return (kLdsPerCu / (size_t)waves) & ~(size_t)511; }
constexpr size_t kLdsScatterFan2 = lds_for_waves(20);
constexpr size_t kLdsScatterFanN = lds_for_waves(16);
constexpr size_t kLdsCombine8 = lds_for_waves(12);
constexpr int64_t kCombineCapFromBytes = (int64_t)512 << 20;
static_assert(kLdsScatterFan2 == 8192 && kLdsScatterFanN == 10240 && kLdsCombine8 == 13312, "LDS reservations");

// ---------------------------------------------------------------------------------------------
// stream probes: what this part sustains for the traffic mixes the row movers are made of, measured
// with the movers' own launch shape (one-wave workgroups, one 16-byte vector per lane, streaming
// loads and stores).  They carry no result anybody uses; the benchmark times them beside the movers.
// ---------------------------------------------------------------------------------------------
// read only: a wave reads eight kilobytes, one from each eighth of the source (one kilobyte per one-wave workgroup
// would measure the rate workgroups can be launched at, not the memory); what is read decides a store that never
// happens for the data the benchmark feeds (all-zero words), so the loads cannot be dropped
__global__ __launch_bounds__(kWave) void probe_read_kernel(const u32x4 *__restrict__ x, u32x4 *__restrict__ y,
                                                           int64_t eighth_vecs) {
    const int64_t g = (int64_t)blockIdx.x * kWave + threadIdx.x;
    u32x4 v = ld_stream(x + g);
#pragma unroll
    for (int j = 1; j < 8; ++j) v ^= ld_stream(x + j * eighth_vecs + g);
    if (v[0] == 0x7E57AB1Eu && v[3] == 0x5EED5EEDu) st_stream(y + g, v);
}

// write only: one aligned 4 KB block per 256-lane workgroup (the fastest pure-write shape on this part)
__global__ __launch_bounds__(kBlock) void probe_write_kernel(u32x4 *__restrict__ y) {
    const int64_t g = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    st_stream(y + g, u32x4{(uint32_t)g, 1u, 2u, 3u});
}

// eight contiguous streams of bf16 summed into one in fp32: the combine's 8:1 read:write mix, its arithmetic
// and its cap on resident waves, with no row ids and no table
__global__ __launch_bounds__(kWave) void probe_sum8_kernel(const u32x4 *__restrict__ x, u32x4 *__restrict__ y,
                                                           int64_t n_vecs) {
    const int64_t g = (int64_t)blockIdx.x * kWave + threadIdx.x;
    u32x4 raw[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) raw[j] = ld_stream(x + j * n_vecs + g);
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[2 * i] = __fadd_rn(acc[2 * i], __fmul_rn(__uint_as_float(raw[j][i] << 16), 0.125f));
            acc[2 * i + 1] = __fadd_rn(acc[2 * i + 1], __fmul_rn(__uint_as_float(raw[j][i] & 0xFFFF0000u), 0.125f));
        }
    }
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (f32_to_bf16_bits(acc[2 * i]) & 0xFFFFu) | (f32_to_bf16_bits(acc[2 * i + 1]) << 16);
    st_stream(y + g, o);
}

// copy in the movers' shape: one wave per kilobyte
__global__ __launch_bounds__(kWave) void probe_copy_kernel(const u32x4 *__restrict__ x, u32x4 *__restrict__ y) {
    const int64_t g = (int64_t)blockIdx.x * kWave + threadIdx.x;
    st_stream(y + g, ld_stream(x + g));
}

// `nbytes` is what the probe writes (reads, for the read-only one): a positive multiple of 8192, both
// pointers 16-byte aligned; the 8:1 sum reads 8 * nbytes from `x`.
int launch_stream_probe(int kind, const void *x, void *y, size_t nbytes, hipStream_t s) {
    if (nbytes == 0) return TERRACE_OK;
    if (nbytes % 8192 || (((uintptr_t)x | (uintptr_t)y) & 15) || !y) return TERRACE_EINVAL;
    const int64_t vecs = (int64_t)(nbytes / 16);
    if (vecs / kWave > ((int64_t)1 << 31) - 1) return TERRACE_EINVAL;
    const unsigned waves = (unsigned)(vecs / kWave);
    switch (kind) {
        case TERRACE_PROBE_READ:
            if (!x) return TERRACE_EINVAL;
            probe_read_kernel<<<waves / 8, kWave, 0, s>>>((const u32x4 *)x, (u32x4 *)y, vecs / 8);
            break;
        case TERRACE_PROBE_WRITE:
            probe_write_kernel<<<(unsigned)(vecs / kBlock), kBlock, 0, s>>>((u32x4 *)y);
            break;
        case TERRACE_PROBE_SUM8:
            if (!x) return TERRACE_EINVAL;
            probe_sum8_kernel<<<waves, kWave, nbytes * 8 >= (size_t)kCombineCapFromBytes ? kLdsCombine8 : 0, s>>>(
                (const u32x4 *)x, (u32x4 *)y, vecs);
            break;
        case TERRACE_PROBE_COPY:
            if (!x) return TERRACE_EINVAL;
            probe_copy_kernel<<<waves, kWave, 0, s>>>((const u32x4 *)x, (u32x4 *)y);
            break;
        default: return TERRACE_EINVAL;
    }
    return check_launch();
}

// Row ids a caller hands in are never trusted with an address: an id is used only if it lies in [0, bound),
// which one unsigned compare decides ((uint64_t)id < (uint64_t)bound is false for negative ids too).  An id
// outside is a dead entry -- a zero row for a gather, no contribution for the combine, a copy not made for a
// scatter.  The stage operators bound the planes their own index kernels wrote all the same.
__device__ __forceinline__ bool row_in(int64_t id, int64_t bound) { return (uint64_t)id < (uint64_t)bound; }

// ---------------------------------------------------------------------------------------------
// scatter: one read, fan writes
// ---------------------------------------------------------------------------------------------
template <typename V, int VPT, typename I>
__global__ __launch_bounds__(kBlock) void scatter_rows_kernel(const V *__restrict__ src, V *__restrict__ dst,
                                                              const I *__restrict__ pos, int64_t n_src,
                                                              int fan, int64_t row_vecs, int tpr_log2,
                                                              int64_t n_dst) {
    const int tpr = 1 << tpr_log2;
    const int sub = __builtin_amdgcn_readfirstlane(threadIdx.x >> tpr_log2);
    const int lane = threadIdx.x & (tpr - 1);
    const int64_t row = (int64_t)blockIdx.x * (kBlock >> tpr_log2) + sub;
    if (row >= n_src) return;
    const V *s = src + row * row_vecs;
    const I *p = pos + row * fan;
    for (int64_t base = lane; base < row_vecs; base += (int64_t)tpr * VPT) {
        V v[VPT];
#pragma unroll
        for (int u = 0; u < VPT; ++u) {
            const int64_t i = base + (int64_t)u * tpr;
            if (i < row_vecs) v[u] = ld_stream(s + i);
        }
        for (int f = 0; f < fan; ++f) {
            const int64_t d = p[f];
            if (!row_in(d, n_dst)) continue;
            V *o = dst + d * row_vecs;
#pragma unroll
            for (int u = 0; u < VPT; ++u) {
                const int64_t i = base + (int64_t)u * tpr;
                if (i < row_vecs) st_stream(o + i, v[u]);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// gather: out[i] = src[idx[i]], zero row when idx[i] < 0
// ---------------------------------------------------------------------------------------------
template <typename V, int VPT, typename I>
__global__ __launch_bounds__(kBlock) void gather_rows_kernel(const V *__restrict__ src, V *__restrict__ out,
                                                             const I *__restrict__ idx, int64_t n_out,
                                                             int64_t row_vecs, int tpr_log2, int64_t n_src) {
    const int tpr = 1 << tpr_log2;
    const int sub = __builtin_amdgcn_readfirstlane(threadIdx.x >> tpr_log2);
    const int lane = threadIdx.x & (tpr - 1);
    const int64_t row = (int64_t)blockIdx.x * (kBlock >> tpr_log2) + sub;
    if (row >= n_out) return;
    const int64_t from = (int64_t)idx[row];
    V *o = out + row * row_vecs;
    if (!row_in(from, n_src)) {
        for (int64_t i = lane; i < row_vecs; i += tpr) st_stream(o + i, zero_of<V>());
        return;
    }
    const V *s = src + from * row_vecs;
    for (int64_t base = lane; base < row_vecs; base += (int64_t)tpr * VPT) {
        V v[VPT];
#pragma unroll
        for (int u = 0; u < VPT; ++u) {
            const int64_t i = base + (int64_t)u * tpr;
            if (i < row_vecs) v[u] = ld_stream(s + i);
        }
#pragma unroll
        for (int u = 0; u < VPT; ++u) {
            const int64_t i = base + (int64_t)u * tpr;
            if (i < row_vecs) st_stream(o + i, v[u]);
        }
    }
}

// Workgroups are handed to the 8 XCDs round-robin by linear id, and each XCD has an L2 of its own.
// Where neighbouring chunks of a row share cache lines (rows that are not whole 128-byte lines, or fp8
// rows whose block scales sit in one line), the `run` chunks of a row are therefore given ids that are
// 8 apart, so one XCD fetches the shared lines once.  Ids are taken in blocks of 8*run: linear id
// y*8 + x inside a block works on logical chunk x*run + y; a ragged last block keeps its order.
constexpr uint32_t kXcds = 8;
__device__ __forceinline__ uint32_t xcd_swizzle(uint32_t id, uint32_t run, uint32_t total) {
    if (run == 0) return id;
    const uint32_t block = kXcds * run;
    const uint32_t base = id / block * block;
    if (base + block > total) return id;
    const uint32_t in = id - base;
    return base + (in % kXcds) * run + in / kXcds;
}

// Sliced forms for 16-byte vectors: a workgroup is one wave, every lane moves exactly one vector, and
// each wave's store covers one 1 KB-aligned kilobyte of the destination.  Many one-wave workgroups
// keep loads and stores of different rows interleaved in the memory pipeline, which streams
// measurably faster than fewer workgroups that load a whole row and then store it; and because
// consecutive workgroups run on different XCDs (each with an L2 of its own), a store that ends inside
// a 128-byte line would leave that line half-written in two L2s -- so chunks are cut on destination
// kilobyte boundaries, not at multiples of 64 vectors from the row start.

// Gather: the destination is one flat run of n_out*row_vecs vectors; `head` is the number of vectors
// between the kilobyte boundary at or below `out` and `out` itself.
template <typename I>
__global__ __launch_bounds__(kWave) void gather_rows_flat_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ out,
                                                                 const I *__restrict__ idx, int64_t total_vecs,
                                                                 int64_t row_vecs, int head, uint32_t run,
                                                                 int64_t n_src) {
    const uint32_t chunk = xcd_swizzle(blockIdx.x, run, gridDim.x);
    const int64_t first = (int64_t)chunk * kWave - head;                 // wave-uniform, may be < 0 in chunk 0
    const int64_t g = first + threadIdx.x;
    if (g < 0 || g >= total_vecs) return;
    int64_t row, i;
    if (row_vecs >= kWave) {
        const int64_t f0 = first < 0 ? 0 : first;
        row = f0 / row_vecs;                                             // one division per wave
        i = g - row * row_vecs;
        if (i >= row_vecs) {                                             // at most one row boundary inside a wave
            i -= row_vecs;
            ++row;
        }
    } else {
        row = g / row_vecs;
        i = g - row * row_vecs;
    }
    const int64_t from = (int64_t)idx[row];
    u32x4 v = zero_of<u32x4>();
    if (row_in(from, n_src)) v = ld_stream(src + from * row_vecs + i);
    st_stream(out + g, v);
}

// Gather, rows that are whole kilobytes on a kilobyte-aligned destination: blockIdx.x = row * slices + slice.
// `row_vecs` is the distance between rows (the pitch), `live_vecs` <= row_vecs what a row holds; the last slice of
// a row whose width is not a whole number of kilobytes has idle lanes and touches nothing beyond the width.
template <typename I>
__global__ __launch_bounds__(kWave) void gather_rows_sliced_kernel(const u32x4 *__restrict__ src,
                                                                   u32x4 *__restrict__ out, const I *__restrict__ idx,
                                                                   int64_t row_vecs, int64_t live_vecs, uint32_t slices,
                                                                   int64_t n_src) {
    const uint32_t row = blockIdx.x / slices;
    const uint32_t slice = blockIdx.x - row * slices;
    const int64_t i = (int64_t)slice * kWave + threadIdx.x;
    if (i >= live_vecs) return;
    const int64_t from = (int64_t)idx[row];
    u32x4 v = zero_of<u32x4>();
    if (row_in(from, n_src)) v = ld_stream(src + from * row_vecs + i);
    st_stream(out + (int64_t)row * row_vecs + i, v);
}

// Scatter, rows that are whole kilobytes on a kilobyte-aligned destination: load once, store fan times.
template <typename I>
__global__ __launch_bounds__(kWave) void scatter_rows_sliced_kernel(const u32x4 *__restrict__ src,
                                                                    u32x4 *__restrict__ dst, const I *__restrict__ pos,
                                                                    int fan, int64_t row_vecs, int64_t live_vecs,
                                                                    uint32_t slices, int64_t n_dst) {
    const uint32_t row = blockIdx.x / slices;
    const uint32_t slice = blockIdx.x - row * slices;
    const int64_t i = (int64_t)slice * kWave + threadIdx.x;
    if (i >= live_vecs) return;
    const u32x4 v = ld_stream(src + (int64_t)row * row_vecs + i);
    const I *p = pos + (int64_t)row * fan;
    for (int f = 0; f < fan; ++f) {
        const int64_t d = p[f];
        if (row_in(d, n_dst)) st_stream(dst + d * row_vecs + i, v);
    }
}

// The same with exactly two copies: both positions are fetched by one scalar load issued beside the row load, and
// one wait for the row stands before both stores, so nothing separates them.  Measured against the loop above at
// fan 2: arrival scatter 0.470 -> 0.468 ms at 16384 tokens x 14 KB rows, 0.542 -> 0.531 ms at 65536 x 4 KB.  The same
// treatment of four copies is 7-9 % SLOWER than the loop (whose stores go out a scalar load apart), so fan 4 keeps it.
template <typename I>
__global__ __launch_bounds__(kWave) void scatter_rows_sliced_fan2_kernel(const u32x4 *__restrict__ src,
                                                                         u32x4 *__restrict__ dst,
                                                                         const I *__restrict__ pos, int64_t row_vecs,
                                                                         int64_t live_vecs, uint32_t slices,
                                                                         int64_t n_dst) {
    const uint32_t row = blockIdx.x / slices;
    const uint32_t slice = blockIdx.x - row * slices;
    const int64_t i = (int64_t)slice * kWave + threadIdx.x;
    if (i >= live_vecs) return;
    const u32x4 v = ld_stream(src + (int64_t)row * row_vecs + i);
    const I *p = pos + (int64_t)row * 2;
    const int64_t d0 = (int64_t)p[0], d1 = (int64_t)p[1];
    asm volatile("" ::"v"(v));           // the one wait for the row, ahead of the branches around the stores
    if (row_in(d0, n_dst)) st_stream(dst + d0 * row_vecs + i, v);
    if (row_in(d1, n_dst)) st_stream(dst + d1 * row_vecs + i, v);
}

// Scatter, any other 16-byte-multiple row width: every copy is cut on its own destination's kilobyte
// boundaries, so the window of source vectors a wave needs shifts from copy to copy and is loaded
// again for each (the re-loads hit in cache: HBM still sees each source row once).
template <typename I>
__global__ __launch_bounds__(kWave) void scatter_rows_aligned_kernel(const u32x4 *__restrict__ src,
                                                                     u32x4 *__restrict__ dst, const I *__restrict__ pos,
                                                                     int fan, int64_t row_vecs, uint32_t chunks,
                                                                     int head, int64_t n_dst) {
    const uint32_t id = xcd_swizzle(blockIdx.x, chunks, gridDim.x);     // a row's chunks re-read each other's lines
    const uint32_t row = id / chunks;
    const int64_t c = id - row * chunks;
    const u32x4 *s = src + (int64_t)row * row_vecs;
    const I *p = pos + (int64_t)row * fan;
    for (int f = 0; f < fan; ++f) {
        const int64_t d = p[f];
        if (!row_in(d, n_dst)) continue;
        const int64_t base = d * row_vecs;
        const int64_t i = c * kWave - ((base + head) & (kWave - 1)) + threadIdx.x;
        if (i >= 0 && i < row_vecs) st_stream(dst + base + i, s[i]);
    }
}

// ---------------------------------------------------------------------------------------------
// combine
// ---------------------------------------------------------------------------------------------
// One chunk = 16 bytes of a source row: 4 fp32, 8 bf16/f16 or 16 e4m3 values.
template <int SRC>
struct Chunk;
template <>
struct Chunk<TERRACE_F32> { static constexpr int N = 4; };
template <>
struct Chunk<TERRACE_BF16> { static constexpr int N = 8; };
template <>
struct Chunk<TERRACE_F16> { static constexpr int N = 8; };
template <>
struct Chunk<TERRACE_FP8_E4M3_B128> { static constexpr int N = 16; };

template <int SRC>
__device__ __forceinline__ void decode_chunk(u32x4 raw, float *f) {
    if constexpr (SRC == TERRACE_F32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(raw[i]);
    } else if constexpr (SRC == TERRACE_BF16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(raw[i] << 16);
            f[2 * i + 1] = __uint_as_float(raw[i] & 0xFFFF0000u);
        }
    } else if constexpr (SRC == TERRACE_F16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __half2float(__ushort_as_half((unsigned short)(raw[i] & 0xFFFFu)));
            f[2 * i + 1] = __half2float(__ushort_as_half((unsigned short)(raw[i] >> 16)));
        }
    } else {
        // gfx950's packed fp8 conversion reads OCP e4m3 ("fn": bias 7, no infinities)
        typedef float f32x2 __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)raw[i], false);
            const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)raw[i], true);
            f[4 * i] = lo[0];
            f[4 * i + 1] = lo[1];
            f[4 * i + 2] = hi[0];
            f[4 * i + 3] = hi[1];
        }
    }
}

__device__ __forceinline__ float load_weight(const void *w, int w_dtype, int64_t i) {
    if (w_dtype == TERRACE_F32) return ((const float *)w)[i];
    const uint32_t b = ((const uint16_t *)w)[i];
    if (w_dtype == TERRACE_BF16) return bf16_bits_to_f32(b);
    return __half2float(__ushort_as_half((unsigned short)b));
}

template <int OUT, int N>
__device__ __forceinline__ void store_chunk(void *out_row, int64_t first_elem, const float *acc) {
    if constexpr (OUT == TERRACE_F32) {
        u32x4 *o = (u32x4 *)((float *)out_row + first_elem);
#pragma unroll
        for (int v = 0; v < N / 4; ++v) {
            u32x4 t;
#pragma unroll
            for (int i = 0; i < 4; ++i) t[i] = __float_as_uint(acc[4 * v + i]);
            st_stream(o + v, t);
        }
    } else {
        uint32_t packed[N / 2];
#pragma unroll
        for (int i = 0; i < N / 2; ++i) {
            uint32_t lo, hi;
            if constexpr (OUT == TERRACE_BF16) {
                lo = f32_to_bf16_bits(acc[2 * i]);
                hi = f32_to_bf16_bits(acc[2 * i + 1]);
            } else {
                lo = __half_as_ushort(__float2half_rn(acc[2 * i]));
                hi = __half_as_ushort(__float2half_rn(acc[2 * i + 1]));
            }
            packed[i] = (lo & 0xFFFFu) | (hi << 16);
        }
        uint16_t *o16 = (uint16_t *)out_row + first_elem;
        if constexpr (N == 4) {
            st_stream((u32x2 *)o16, u32x2{packed[0], packed[1]});
        } else {
#pragma unroll
            for (int v = 0; v < N / 8; ++v)
                st_stream((u32x4 *)o16 + v, u32x4{packed[4 * v], packed[4 * v + 1], packed[4 * v + 2], packed[4 * v + 3]});
        }
    }
}

// Vector path: rows are 16-byte aligned multiples of 16 bytes.  One thread owns one 16-byte chunk of
// one output row: blockIdx.x = row * slices + slice, chunk = slice * blockDim.x + threadIdx.x.
//
// Everything a batch of source rows needs that is the same for the whole wave -- the row ids and
// the weights -- is fetched first through addresses the compiler can prove uniform (scalar loads; 16-bit
// weights are read as the aligned dword that holds them).  The batch's row loads are then issued back to
// back with nothing between them that waits on memory, and only the accumulation that follows consumes
// them in order.  A dead entry (idx outside [0, n_src)) touches no memory: its load sits behind a branch that
// is uniform over the wave (the ids are), which costs nothing measurable against a select around a dummy load.
constexpr int kWNone = -1;

template <int WD>
__device__ __forceinline__ float uniform_weight(const void *w, int64_t i) {
    if constexpr (WD == TERRACE_F32) {
        return ((const float *)w)[i];
    } else {
        const uint32_t pair = ((const uint32_t *)w)[i >> 1];
        const uint32_t bits = (i & 1) ? (pair >> 16) : (pair & 0xFFFFu);
        if constexpr (WD == TERRACE_BF16) return __uint_as_float(bits << 16);
        else return __half2float(__ushort_as_half((unsigned short)bits));
    }
}

// One batch of exactly B source rows, no guards: B uniform index (and weight) fetches, B row loads
// issued back to back, then the in-order accumulation.
template <int SRC, int WD, int B>
__device__ __forceinline__ void combine_batch(float *acc, const uint8_t *__restrict__ src, int64_t src_row_bytes,
                                              const int64_t *__restrict__ idx_at, const void *__restrict__ w,
                                              int64_t w_at, int64_t hidden, int64_t c, int64_t n_src) {
    constexpr int N = Chunk<SRC>::N;
    int64_t from[B];
    float wj[B];
#pragma unroll
    for (int jj = 0; jj < B; ++jj) {
        from[jj] = idx_at[jj];
        if constexpr (WD != kWNone) wj[jj] = uniform_weight<WD>(w, w_at + jj);
        else wj[jj] = 1.0f;
    }
    u32x4 raw[B];
    float sc[B];
#pragma unroll
    for (int jj = 0; jj < B; ++jj) {
        raw[jj] = zero_of<u32x4>();
        sc[jj] = SRC == TERRACE_FP8_E4M3_B128 ? 0.0f : 1.0f;
        if (row_in(from[jj], n_src)) {                       // wave-uniform: a dead entry touches no memory at all
            const uint8_t *s = src + from[jj] * src_row_bytes;
            raw[jj] = ld_stream((const u32x4 *)s + c);
            if constexpr (SRC == TERRACE_FP8_E4M3_B128) sc[jj] = *(const float *)(s + hidden + 4 * (c * N / 128));
        }
    }
#pragma unroll
    for (int jj = 0; jj < B; ++jj) {
        const bool live = row_in(from[jj], n_src);
        const u32x4 r = raw[jj];
        const float scale = sc[jj], weight = live ? wj[jj] : 0.0f;
        float f[N];
        decode_chunk<SRC>(r, f);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            float x = f[i];
            if constexpr (SRC == TERRACE_FP8_E4M3_B128) x = __fmul_rn(x, scale);
            if constexpr (WD != kWNone) x = __fmul_rn(x, weight);
            acc[i] = __fadd_rn(acc[i], x);
        }
    }
}

template <int SRC, int OUT, int WD>
__device__ __forceinline__ void combine_row_chunk(const uint8_t *__restrict__ src, int64_t src_row_bytes,
                                                  const int64_t *__restrict__ idx_row, const void *__restrict__ w,
                                                  int64_t w_base, int fan, int64_t hidden, int64_t c,
                                                  uint8_t *__restrict__ out_row, int64_t n_src) {
    constexpr int N = Chunk<SRC>::N;
    float acc[N];
#pragma unroll
    for (int i = 0; i < N; ++i) acc[i] = 0.0f;
    int j = 0;
    for (; j + 8 <= fan; j += 8) combine_batch<SRC, WD, 8>(acc, src, src_row_bytes, idx_row + j, w, w_base + j, hidden, c, n_src);
    if (j + 4 <= fan) {
        combine_batch<SRC, WD, 4>(acc, src, src_row_bytes, idx_row + j, w, w_base + j, hidden, c, n_src);
        j += 4;
    }
    if (j + 2 <= fan) {
        combine_batch<SRC, WD, 2>(acc, src, src_row_bytes, idx_row + j, w, w_base + j, hidden, c, n_src);
        j += 2;
    }
    if (j < fan) combine_batch<SRC, WD, 1>(acc, src, src_row_bytes, idx_row + j, w, w_base + j, hidden, c, n_src);
    store_chunk<OUT, N>(out_row, c * N, acc);
}

template <int SRC, int OUT>
__global__ __launch_bounds__(kBlock) void combine_kernel(const uint8_t *__restrict__ src, int64_t src_row_bytes,
                                                         const int64_t *__restrict__ idx, const void *__restrict__ w,
                                                         int w_dtype, int64_t n_out, int fan, int64_t hidden,
                                                         uint8_t *__restrict__ out, int64_t out_row_bytes,
                                                         int slices, uint32_t run, int64_t n_src) {
    constexpr int N = Chunk<SRC>::N;
    const uint32_t id = xcd_swizzle(blockIdx.x, run, gridDim.x);
    const int64_t row = id / slices;
    const int64_t c = (int64_t)(id - row * slices) * blockDim.x + threadIdx.x;
    if (c >= hidden / N) return;
    const int64_t *idx_row = idx + row * fan;
    uint8_t *out_row = out + row * out_row_bytes;
#define TERRACE_COMBINE_BODY(WD) \
    combine_row_chunk<SRC, OUT, WD>(src, src_row_bytes, idx_row, w, row * fan, fan, hidden, c, out_row, n_src)
    if (!w) TERRACE_COMBINE_BODY(kWNone);
    else if (w_dtype == TERRACE_F32) TERRACE_COMBINE_BODY(TERRACE_F32);
    else if (w_dtype == TERRACE_BF16) TERRACE_COMBINE_BODY(TERRACE_BF16);
    else TERRACE_COMBINE_BODY(TERRACE_F16);
#undef TERRACE_COMBINE_BODY
}

// Two levels in one pass: out[t] = round_OUT( sum_m f32( round_SRC( sum_i src[inner[outer[t, m], i]] ) ) ), both sums in
// fp32 in table order, entries outside their range skipped.  This is, bit for bit, combine(src, inner) rounded to the
// source dtype followed by combine(that, outer) -- the reference's two index_add levels
// (terrace/ta2a_dispatch.py:483-494) -- without the [n_rows, H] plane between them ever reaching memory.  The inner
// table is Q ids wide; a wave works on 8 / Q outer entries at a time, so about eight row loads are in flight.
template <int SRC>
__device__ __forceinline__ float round_to_src(float x) {
    if constexpr (SRC == TERRACE_F32) return x;
    else if constexpr (SRC == TERRACE_BF16) return __uint_as_float(f32_to_bf16_bits(x) << 16);
    else return __half2float(__float2half_rn(x));
}

template <int SRC, int OUT, int Q>
__global__ __launch_bounds__(kBlock) void combine2_kernel(const uint8_t *__restrict__ src, int64_t src_row_bytes,
                                                          const int64_t *__restrict__ inner, int64_t n_rows,
                                                          const int64_t *__restrict__ outer, int fan_outer,
                                                          int64_t hidden, uint8_t *__restrict__ out,
                                                          int64_t out_row_bytes, int slices, int64_t n_src) {
    constexpr int N = Chunk<SRC>::N;
    constexpr int MB = 8 / Q;
    const int64_t t = blockIdx.x / slices;
    const int64_t c = (int64_t)(blockIdx.x - t * slices) * blockDim.x + threadIdx.x;
    if (c >= hidden / N) return;
    float total[N];
#pragma unroll
    for (int i = 0; i < N; ++i) total[i] = 0.0f;
    const int64_t *outer_row = outer + t * fan_outer;
    for (int m0 = 0; m0 < fan_outer; m0 += MB) {
        int64_t r[MB], from[MB][Q];
#pragma unroll
        for (int b = 0; b < MB; ++b) r[b] = m0 + b < fan_outer ? outer_row[m0 + b] : -1;
#pragma unroll
        for (int b = 0; b < MB; ++b) {
#pragma unroll
            for (int i = 0; i < Q; ++i) from[b][i] = -1;
            if (row_in(r[b], n_rows)) {
#pragma unroll
                for (int i = 0; i < Q; ++i) from[b][i] = inner[r[b] * Q + i];
            }
        }
        u32x4 raw[MB][Q];
#pragma unroll
        for (int b = 0; b < MB; ++b) {
#pragma unroll
            for (int i = 0; i < Q; ++i) {
                raw[b][i] = zero_of<u32x4>();
                if (row_in(from[b][i], n_src))               // wave-uniform: a dead entry touches no memory
                    raw[b][i] = ld_stream((const u32x4 *)(src + from[b][i] * src_row_bytes) + c);
            }
        }
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            if (!row_in(r[b], n_rows)) continue;             // wave-uniform
            float acc[N];
#pragma unroll
            for (int i = 0; i < N; ++i) acc[i] = 0.0f;
#pragma unroll
            for (int i = 0; i < Q; ++i) {
                float f[N];
                decode_chunk<SRC>(raw[b][i], f);             // a dead entry decodes to +0.0, which changes no sum
#pragma unroll
                for (int e = 0; e < N; ++e) acc[e] = __fadd_rn(acc[e], f[e]);
            }
#pragma unroll
            for (int e = 0; e < N; ++e) total[e] = __fadd_rn(total[e], round_to_src<SRC>(acc[e]));
        }
    }
    store_chunk<OUT, N>(out + t * out_row_bytes, c * N, total);
}

// Element path: any hidden, any alignment.
__device__ __forceinline__ float load_elem(const uint8_t *row, int src_dtype, int64_t e, int64_t hidden) {
    switch (src_dtype) {
        case TERRACE_F32: return ((const float *)row)[e];
        case TERRACE_BF16: return bf16_bits_to_f32(((const uint16_t *)row)[e]);
        case TERRACE_F16: return __half2float(__ushort_as_half(((const uint16_t *)row)[e]));
        default: {
            float sc;
            const uint8_t *sp = row + hidden + 4 * (e / 128);
            uint32_t bits = sp[0] | (sp[1] << 8) | (sp[2] << 16) | ((uint32_t)sp[3] << 24);
            sc = __uint_as_float(bits);
            return __fmul_rn(e4m3_to_f32(row[e]), sc);
        }
    }
}

__global__ __launch_bounds__(kBlock) void combine_elem_kernel(const uint8_t *__restrict__ src, int src_dtype,
                                                              int64_t src_row_bytes, const int64_t *__restrict__ idx,
                                                              const void *__restrict__ w, int w_dtype, int64_t n_out,
                                                              int fan, int64_t hidden, uint8_t *__restrict__ out,
                                                              int out_dtype, int64_t n_src) {
    for (int64_t row = blockIdx.x; row < n_out; row += gridDim.x) {
        for (int64_t e = threadIdx.x; e < hidden; e += kBlock) {
            float acc = 0.0f;
            for (int j = 0; j < fan; ++j) {
                const int64_t from = idx[row * fan + j];
                if (!row_in(from, n_src)) continue;
                float x = load_elem(src + from * src_row_bytes, src_dtype, e, hidden);
                if (w) x = __fmul_rn(x, load_weight(w, w_dtype, row * fan + j));
                acc = __fadd_rn(acc, x);
            }
            if (out_dtype == TERRACE_F32) ((float *)out)[row * hidden + e] = acc;
            else if (out_dtype == TERRACE_BF16) ((uint16_t *)out)[row * hidden + e] = (uint16_t)f32_to_bf16_bits(acc);
            else ((uint16_t *)out)[row * hidden + e] = __half_as_ushort(__float2half_rn(acc));
        }
    }
}

// ---------------------------------------------------------------------------------------------
// wire containers: out row = a | b | c | zero pad, and the inverse split
// (the int64-word rows of the reference's terrace/ta2a_pack.py:319-336,398-414,474-497)
// ---------------------------------------------------------------------------------------------
struct Planes {
    const uint8_t *src[3];
    uint8_t *dst[3];
    int64_t bytes[3];       // per-row width of each plane (0 = absent)
};

template <typename V, bool PACK>
__global__ __launch_bounds__(kBlock) void planes_kernel(Planes pl, uint8_t *__restrict__ packed, int64_t row_bytes,
                                                        int64_t n_rows) {
    const int64_t vecs = row_bytes / (int64_t)sizeof(V);
    const int64_t a = pl.bytes[0], ab = a + pl.bytes[1], abc = ab + pl.bytes[2];
    for (int64_t g = (int64_t)blockIdx.x * kBlock + threadIdx.x; g < n_rows * vecs;
         g += (int64_t)gridDim.x * kBlock) {
        const int64_t row = g / vecs, off = (g - row * vecs) * (int64_t)sizeof(V);
        V *cell = (V *)(packed + row * row_bytes + off);
        int which = -1;
        int64_t inner = 0;
        if (off < a) { which = 0; inner = off; }
        else if (off < ab) { which = 1; inner = off - a; }
        else if (off < abc) { which = 2; inner = off - ab; }
        if constexpr (PACK) {
            *cell = which < 0 ? zero_of<V>() : *(const V *)(pl.src[which] + row * pl.bytes[which] + inner);
        } else {
            if (which >= 0 && pl.dst[which]) *(V *)(pl.dst[which] + row * pl.bytes[which] + inner) = *cell;
        }
    }
}

template <bool PACK>
static int launch_planes(const Planes &pl, void *packed, int64_t row_bytes, int64_t n_rows, hipStream_t s) {
    if (n_rows <= 0 || row_bytes <= 0) return TERRACE_OK;
    uintptr_t bits = (uintptr_t)packed | (uintptr_t)row_bytes;
    for (int i = 0; i < 3; ++i) {
        if (!pl.bytes[i]) continue;
        bits |= (uintptr_t)pl.bytes[i] | (uintptr_t)(PACK ? (const void *)pl.src[i] : (const void *)pl.dst[i]);
    }
    int64_t blocks;
#define TERRACE_PLANES(V)                                                          \
    blocks = (n_rows * (row_bytes / (int64_t)sizeof(V)) + kBlock - 1) / kBlock;    \
    if (blocks > ((int64_t)1 << 22)) blocks = (int64_t)1 << 22;                    \
    planes_kernel<V, PACK><<<(unsigned)blocks, kBlock, 0, s>>>(pl, (uint8_t *)packed, row_bytes, n_rows)
    if ((bits & 15) == 0) { TERRACE_PLANES(u32x4); }
    else if ((bits & 7) == 0) { TERRACE_PLANES(u32x2); }
    else if ((bits & 3) == 0) { TERRACE_PLANES(uint32_t); }
    else if ((bits & 1) == 0) { TERRACE_PLANES(uint16_t); }
    else { TERRACE_PLANES(uint8_t); }
#undef TERRACE_PLANES
    return check_launch();
}

int launch_pack_planes(const void *a, int64_t a_bytes, const void *b, int64_t b_bytes, const void *c, int64_t c_bytes,
                       int64_t n_rows, int64_t row_bytes, void *out, hipStream_t s) {
    Planes pl{{(const uint8_t *)a, (const uint8_t *)b, (const uint8_t *)c}, {nullptr, nullptr, nullptr},
              {a ? a_bytes : 0, b ? b_bytes : 0, c ? c_bytes : 0}};
    return launch_planes<true>(pl, out, row_bytes, n_rows, s);
}

int launch_unpack_planes(const void *packed, int64_t row_bytes, int64_t n_rows, void *a, int64_t a_bytes, void *b,
                         int64_t b_bytes, void *c, int64_t c_bytes, hipStream_t s) {
    Planes pl{{nullptr, nullptr, nullptr}, {(uint8_t *)a, (uint8_t *)b, (uint8_t *)c}, {a_bytes, b_bytes, c_bytes}};
    return launch_planes<false>(pl, (void *)packed, row_bytes, n_rows, s);
}

__global__ __launch_bounds__(kBlock) void index_chain_kernel(const int64_t *__restrict__ table, int64_t n_table,
                                                             const int64_t *__restrict__ idx, int64_t n,
                                                             int64_t *__restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int64_t a = idx[i];
    out[i] = row_in(a, n_table) ? table[a] : -1;
}

__global__ __launch_bounds__(kBlock) void index_chain2_kernel(const int64_t *__restrict__ outer, int64_t n_outer,
                                                              const int64_t *__restrict__ inner, int64_t n_inner,
                                                              const int64_t *__restrict__ idx, int64_t n,
                                                              int64_t *__restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    int64_t a = idx[i];
    a = row_in(a, n_inner) ? inner[a] : -1;
    out[i] = row_in(a, n_outer) ? outer[a] : -1;
}

__global__ void send_splits_kernel(const int64_t *__restrict__ node_counts, int world, int rpn, int my_local,
                                   int64_t *__restrict__ send) {
    for (int i = threadIdx.x; i < world; i += blockDim.x)
        send[i] = (i % rpn == my_local) ? node_counts[i / rpn] : 0;
}

// ---------------------------------------------------------------------------------------------
// host-side launch helpers
// ---------------------------------------------------------------------------------------------
// One sub-group per row and no grid-stride loop: many short workgroups stream measurably
// faster on this part than a resident grid walking the rows.
constexpr int64_t kMaxGridRows = (int64_t)1 << 30;   // keeps every launch below HIP's 2^31 - 1 blocks
constexpr int64_t kMaxBlocks = ((int64_t)1 << 31) - 1;

static unsigned grid_for(int64_t n_rows, int rows_per_block) {
    const int64_t need = (n_rows + rows_per_block - 1) / rows_per_block;
    return (unsigned)(need < 1 ? 1 : need);
}

// Lanes per row: enough that a lane holds about 4 vectors, at least one wave, at most the block.
static int tpr_log2_for(int64_t row_vecs) {
    int l = 6;
    while (l < 8 && ((int64_t)4 << l) < row_vecs) ++l;
    return l;
}

static int vec_bytes_for(int64_t row_bytes, const void *a, const void *b) {
    const uintptr_t bits = (uintptr_t)row_bytes | (uintptr_t)a | (uintptr_t)b;
    if ((bits & 15) == 0) return 16;
    if ((bits & 7) == 0) return 8;
    if ((bits & 3) == 0) return 4;
    if ((bits & 1) == 0) return 2;
    return 1;
}

template <typename V, typename I>
static void launch_scatter_t(const void *src, void *dst, const I *pos, int64_t n_src, int fan,
                             int64_t row_vecs, int64_t n_dst, hipStream_t s) {
    const int l = tpr_log2_for(row_vecs);
    const int rpi = kBlock >> l;
    const unsigned grid = grid_for(n_src, rpi);
    if (row_vecs > ((int64_t)2 << l))
        scatter_rows_kernel<V, 4, I><<<grid, kBlock, 0, s>>>((const V *)src, (V *)dst, pos, n_src, fan, row_vecs, l, n_dst);
    else if (row_vecs > ((int64_t)1 << l))
        scatter_rows_kernel<V, 2, I><<<grid, kBlock, 0, s>>>((const V *)src, (V *)dst, pos, n_src, fan, row_vecs, l, n_dst);
    else
        scatter_rows_kernel<V, 1, I><<<grid, kBlock, 0, s>>>((const V *)src, (V *)dst, pos, n_src, fan, row_vecs, l, n_dst);
}

template <typename I>
int launch_scatter_rows(const void *src, void *dst, const I *pos, int64_t n_src, int fan, int64_t row_bytes,
                        int64_t n_dst, hipStream_t s) {
    const RowGeom geom = row_geom(row_bytes);
    if (!row_geom_ok(geom)) return TERRACE_EINVAL;
    if (n_src <= 0 || geom.width <= 0 || fan <= 0) return TERRACE_OK;
    if (n_src > kMaxGridRows) return TERRACE_EINVAL;
    if (geom.pitched()) {        // rows on a kilobyte pitch: the sliced kernel, idle lanes past the width
        const int64_t slices = (geom.width / 16 + kWave - 1) / kWave;
        if ((((uintptr_t)src | (uintptr_t)dst) & 15) || n_src * slices > kMaxBlocks) return TERRACE_EINVAL;
        if (fan == 2)
            scatter_rows_sliced_fan2_kernel<I><<<(unsigned)(n_src * slices), kWave, kLdsScatterFan2, s>>>(
                (const u32x4 *)src, (u32x4 *)dst, pos, geom.pitch / 16, geom.width / 16, (uint32_t)slices, n_dst);
        else
            scatter_rows_sliced_kernel<I><<<(unsigned)(n_src * slices), kWave, fan > 2 ? kLdsScatterFanN : 0, s>>>(
                (const u32x4 *)src, (u32x4 *)dst, pos, fan, geom.pitch / 16, geom.width / 16, (uint32_t)slices, n_dst);
        return check_launch();
    }
    switch (vec_bytes_for(row_bytes, src, dst)) {
        case 16: {
            const int64_t rv = row_bytes / 16;
            const int head = (int)(((uintptr_t)dst >> 4) & (kWave - 1));
            if (rv % kWave == 0 && head == 0 && n_src * (rv / kWave) <= kMaxBlocks) {
                if (fan == 2)
                    scatter_rows_sliced_fan2_kernel<I><<<(unsigned)(n_src * (rv / kWave)), kWave, kLdsScatterFan2, s>>>(
                        (const u32x4 *)src, (u32x4 *)dst, pos, rv, rv, (uint32_t)(rv / kWave), n_dst);
                else
                    scatter_rows_sliced_kernel<I><<<(unsigned)(n_src * (rv / kWave)), kWave, fan > 2 ? kLdsScatterFanN : 0,
                                                 s>>>(
                        (const u32x4 *)src, (u32x4 *)dst, pos, fan, rv, rv, (uint32_t)(rv / kWave), n_dst);
            } else {
                const int64_t chunks = (rv + 2 * kWave - 2) / kWave;      // most kilobytes one copy can touch
                if (n_src * chunks <= kMaxBlocks)
                    scatter_rows_aligned_kernel<I><<<(unsigned)(n_src * chunks), kWave, 0, s>>>(
                        (const u32x4 *)src, (u32x4 *)dst, pos, fan, rv, (uint32_t)chunks, head, n_dst);
                else
                    launch_scatter_t<u32x4, I>(src, dst, pos, n_src, fan, rv, n_dst, s);
            }
            break;
        }
        case 8: launch_scatter_t<u32x2, I>(src, dst, pos, n_src, fan, row_bytes / 8, n_dst, s); break;
        case 4: launch_scatter_t<uint32_t, I>(src, dst, pos, n_src, fan, row_bytes / 4, n_dst, s); break;
        case 2: launch_scatter_t<uint16_t, I>(src, dst, pos, n_src, fan, row_bytes / 2, n_dst, s); break;
        default: launch_scatter_t<uint8_t, I>(src, dst, pos, n_src, fan, row_bytes, n_dst, s); break;
    }
    return check_launch();
}
template int launch_scatter_rows<int32_t>(const void *, void *, const int32_t *, int64_t, int, int64_t, int64_t,
                                          hipStream_t);
template int launch_scatter_rows<int64_t>(const void *, void *, const int64_t *, int64_t, int, int64_t, int64_t,
                                          hipStream_t);

template <typename V, typename I>
static void launch_gather_t(const void *src, void *out, const I *idx, int64_t n_out, int64_t row_vecs,
                            int64_t n_src, hipStream_t s) {
    const int l = tpr_log2_for(row_vecs);
    const int rpi = kBlock >> l;
    const unsigned grid = grid_for(n_out, rpi);
    if (row_vecs > ((int64_t)2 << l))
        gather_rows_kernel<V, 4, I><<<grid, kBlock, 0, s>>>((const V *)src, (V *)out, idx, n_out, row_vecs, l, n_src);
    else if (row_vecs > ((int64_t)1 << l))
        gather_rows_kernel<V, 2, I><<<grid, kBlock, 0, s>>>((const V *)src, (V *)out, idx, n_out, row_vecs, l, n_src);
    else
        gather_rows_kernel<V, 1, I><<<grid, kBlock, 0, s>>>((const V *)src, (V *)out, idx, n_out, row_vecs, l, n_src);
}

template <typename I>
static bool launch_gather_sliced(const void *src, void *out, const I *idx, int64_t n_out, int64_t row_vecs,
                                 int64_t n_src, hipStream_t s) {
    const int head = (int)(((uintptr_t)out >> 4) & (kWave - 1));
    const int64_t total = n_out * row_vecs;
    const int64_t blocks = (total + head + kWave - 1) / kWave;
    if (blocks > kMaxBlocks) return false;
    if (row_vecs % kWave == 0 && head == 0) {
        gather_rows_sliced_kernel<I><<<(unsigned)blocks, kWave, 0, s>>>((const u32x4 *)src, (u32x4 *)out, idx, row_vecs,
                                                                       row_vecs, (uint32_t)(row_vecs / kWave), n_src);
        return true;
    }
    // rows that are not whole lines: a row's chunks share lines on the source side
    const uint32_t run = (row_vecs % 8) ? (uint32_t)((row_vecs + kWave - 1) / kWave) : 0u;
    gather_rows_flat_kernel<I><<<(unsigned)blocks, kWave, 0, s>>>((const u32x4 *)src, (u32x4 *)out, idx, total, row_vecs,
                                                                 head, run, n_src);
    return true;
}

template <typename I>
int launch_gather_rows(const void *src, void *out, const I *idx, int64_t n_out, int64_t row_bytes, int64_t n_src,
                       hipStream_t s) {
    const RowGeom geom = row_geom(row_bytes);
    if (!row_geom_ok(geom)) return TERRACE_EINVAL;
    if (n_out <= 0 || geom.width <= 0) return TERRACE_OK;
    if (n_out > kMaxGridRows) return TERRACE_EINVAL;
    if (geom.pitched()) {
        const int64_t slices = (geom.width / 16 + kWave - 1) / kWave;
        if ((((uintptr_t)src | (uintptr_t)out) & 15) || n_out * slices > kMaxBlocks) return TERRACE_EINVAL;
        gather_rows_sliced_kernel<I><<<(unsigned)(n_out * slices), kWave, 0, s>>>(
            (const u32x4 *)src, (u32x4 *)out, idx, geom.pitch / 16, geom.width / 16, (uint32_t)slices, n_src);
        return check_launch();
    }
    switch (vec_bytes_for(row_bytes, src, out)) {
        case 16:
            if (!launch_gather_sliced<I>(src, out, idx, n_out, row_bytes / 16, n_src, s))
                launch_gather_t<u32x4, I>(src, out, idx, n_out, row_bytes / 16, n_src, s);
            break;
        case 8: launch_gather_t<u32x2, I>(src, out, idx, n_out, row_bytes / 8, n_src, s); break;
        case 4: launch_gather_t<uint32_t, I>(src, out, idx, n_out, row_bytes / 4, n_src, s); break;
        case 2: launch_gather_t<uint16_t, I>(src, out, idx, n_out, row_bytes / 2, n_src, s); break;
        default: launch_gather_t<uint8_t, I>(src, out, idx, n_out, row_bytes, n_src, s); break;
    }
    return check_launch();
}
template int launch_gather_rows<int32_t>(const void *, void *, const int32_t *, int64_t, int64_t, int64_t, hipStream_t);
template int launch_gather_rows<int64_t>(const void *, void *, const int64_t *, int64_t, int64_t, int64_t, hipStream_t);

__global__ __launch_bounds__(kBlock) void zero_bytes_kernel(uint8_t *__restrict__ p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) p[i] = 0;
}

static int64_t dtype_row_bytes(int dtype, int64_t hidden) {
    switch (dtype) {
        case TERRACE_F32: return hidden * 4;
        case TERRACE_BF16:
        case TERRACE_F16: return hidden * 2;
        case TERRACE_FP8_E4M3_B128: return hidden + 4 * (hidden / 128);
        default: return -1;
    }
}

template <int SRC, int OUT>
static void launch_combine_so(const void *src, int64_t n_src, const int64_t *idx, const void *w, int w_dtype,
                              int64_t n_out, int fan, int64_t hidden, void *out, int64_t src_pitch, hipStream_t s) {
    const int64_t chunks = hidden / Chunk<SRC>::N;
    const int64_t srb = src_pitch, orb = dtype_row_bytes(OUT, hidden);
    // one wave per workgroup when a row is a whole number of waves' worth of chunks (a workgroup
    // spanning a whole misaligned row, which would keep split cache lines inside one L2, measured
    // slower than this at the fp8 row shape)
    const bool one_wave = chunks % kWave == 0 && n_out * (chunks / kWave) <= kMaxBlocks;
    const int bt = one_wave ? kWave : kBlock;
    const int slices = (int)((chunks + bt - 1) / bt);
    const unsigned grid = (unsigned)(n_out * slices);
    // source rows that are not whole lines (and fp8 rows, whose scales share a line): one XCD per output row
    const uint32_t run = (srb % 128 || SRC == TERRACE_FP8_E4M3_B128) && slices > 1 ? (uint32_t)slices : 0u;
    // (a table with fewer source rows than three quarters of its entries is taken to be mostly dead entries -- a
    // source row of this path belongs to one entry -- and keeps all its waves)
    const bool cap = one_wave && SRC != TERRACE_FP8_E4M3_B128 && fan >= 8 &&
                     n_out * fan * srb >= kCombineCapFromBytes && n_src * 4 >= n_out * fan * 3;
    combine_kernel<SRC, OUT><<<grid, bt, cap ? kLdsCombine8 : 0, s>>>(
        (const uint8_t *)src, srb, idx, w, w_dtype, n_out, fan, hidden, (uint8_t *)out, orb, slices, run, n_src);
}

template <int SRC>
static void launch_combine_s(const void *src, int64_t n_src, const int64_t *idx, const void *w, int w_dtype,
                             int64_t n_out, int fan, int64_t hidden, void *out, int out_dtype, int64_t src_pitch,
                             hipStream_t s) {
    if (out_dtype == TERRACE_F32) launch_combine_so<SRC, TERRACE_F32>(src, n_src, idx, w, w_dtype, n_out, fan, hidden, out, src_pitch, s);
    else if (out_dtype == TERRACE_BF16) launch_combine_so<SRC, TERRACE_BF16>(src, n_src, idx, w, w_dtype, n_out, fan, hidden, out, src_pitch, s);
    else launch_combine_so<SRC, TERRACE_F16>(src, n_src, idx, w, w_dtype, n_out, fan, hidden, out, src_pitch, s);
}

// `src_pitch`: bytes between source rows, 0 for rows back to back.
int launch_combine(const void *src, int64_t n_src, int src_dtype, const int64_t *idx, const void *w, int w_dtype,
                   int64_t n_out, int fan, int64_t hidden, void *out, int out_dtype, int64_t src_pitch,
                   hipStream_t s) {
    if (n_out <= 0 || hidden <= 0) return TERRACE_OK;
    if (n_out * ((hidden + 1023) / 1024 + 1) > kMaxGridRows) return TERRACE_EINVAL;
    const int64_t width = dtype_row_bytes(src_dtype, hidden), orb = dtype_row_bytes(out_dtype, hidden);
    if (src_pitch == 0) src_pitch = width;
    if (src_pitch < width) return TERRACE_EINVAL;
    const int64_t srb = src_pitch;
    if (n_src <= 0) {           // no source rows: every entry is dead and every sum empty; no kernel needs to look
        zero_bytes_kernel<<<1024, kBlock, 0, s>>>((uint8_t *)out, n_out * orb);
        return check_launch();
    }
    const int n = src_dtype == TERRACE_F32 ? 4 : (src_dtype == TERRACE_FP8_E4M3_B128 ? 16 : 8);
    const bool vec = hidden % n == 0 && ((uintptr_t)src & 15) == 0 && ((uintptr_t)out & 15) == 0 &&
                     srb % 16 == 0 && orb % 16 == 0 && ((uintptr_t)w & 3) == 0;   // weights are read as dwords
    if (!vec) {
        const int grid = (int)(n_out > 4096 ? 4096 : n_out);
        combine_elem_kernel<<<grid, kBlock, 0, s>>>((const uint8_t *)src, src_dtype, srb, idx, w, w_dtype, n_out, fan,
                                                    hidden, (uint8_t *)out, out_dtype, n_src);
        return check_launch();
    }
    switch (src_dtype) {
        case TERRACE_F32: launch_combine_s<TERRACE_F32>(src, n_src, idx, w, w_dtype, n_out, fan, hidden, out, out_dtype, srb, s); break;
        case TERRACE_BF16: launch_combine_s<TERRACE_BF16>(src, n_src, idx, w, w_dtype, n_out, fan, hidden, out, out_dtype, srb, s); break;
        case TERRACE_F16: launch_combine_s<TERRACE_F16>(src, n_src, idx, w, w_dtype, n_out, fan, hidden, out, out_dtype, srb, s); break;
        default: launch_combine_s<TERRACE_FP8_E4M3_B128>(src, n_src, idx, w, w_dtype, n_out, fan, hidden, out, out_dtype, srb, s); break;
    }
    return check_launch();
}

template <int SRC, int OUT>
static int launch_combine2_so(const void *src, int64_t n_src, const int64_t *inner, int64_t n_rows, int fan_inner,
                              const int64_t *outer, int64_t n_out, int fan_outer, int64_t hidden, void *out,
                              hipStream_t s) {
    const int64_t chunks = hidden / Chunk<SRC>::N;
    const int64_t srb = dtype_row_bytes(SRC, hidden), orb = dtype_row_bytes(OUT, hidden);
    const bool one_wave = chunks % kWave == 0 && n_out * (chunks / kWave) <= kMaxBlocks;
    const int bt = one_wave ? kWave : kBlock;
    const int slices = (int)((chunks + bt - 1) / bt);
    const unsigned grid = (unsigned)(n_out * slices);
    // no cap on resident waves here: 12 waves per CU measured equal on the dense tables of the quota branch and
    // 1.75x slower on the general branch's, whose entries are mostly dead (few loads in flight per wave)
#define TERRACE_C2(Q)                                                                                              \
    combine2_kernel<SRC, OUT, Q><<<grid, bt, 0, s>>>((const uint8_t *)src, srb, inner, n_rows, outer, fan_outer, hidden, \
                                                     (uint8_t *)out, orb, slices, n_src)
    switch (fan_inner) {
        case 1: TERRACE_C2(1); break;
        case 2: TERRACE_C2(2); break;
        case 4: TERRACE_C2(4); break;
        case 8: TERRACE_C2(8); break;
        default: return TERRACE_EINVAL;
    }
#undef TERRACE_C2
    return check_launch();
}

// Vector path only: float rows (f32 / bf16 / f16) that are 16-byte multiples on 16-byte-aligned buffers, inner
// tables 1, 2, 4 or 8 ids wide.  Anything else returns TERRACE_EINVAL and the caller runs the two levels one by one.
int launch_combine2(const void *src, int64_t n_src, int src_dtype, const int64_t *inner, int64_t n_rows, int fan_inner,
                    const int64_t *outer, int64_t n_out, int fan_outer, int64_t hidden, void *out, int out_dtype,
                    hipStream_t s) {
    if (n_out <= 0 || hidden <= 0) return TERRACE_OK;
    if (src_dtype != TERRACE_F32 && src_dtype != TERRACE_BF16 && src_dtype != TERRACE_F16) return TERRACE_EINVAL;
    if (out_dtype != TERRACE_F32 && out_dtype != TERRACE_BF16 && out_dtype != TERRACE_F16) return TERRACE_EINVAL;
    if (fan_outer <= 0 || n_rows < 0 || n_src < 0) return TERRACE_EINVAL;
    if (n_out * ((hidden + 1023) / 1024 + 1) > kMaxGridRows) return TERRACE_EINVAL;
    const int64_t srb = dtype_row_bytes(src_dtype, hidden), orb = dtype_row_bytes(out_dtype, hidden);
    const int n = src_dtype == TERRACE_F32 ? 4 : 8;
    if (hidden % n || ((uintptr_t)src & 15) || ((uintptr_t)out & 15) || srb % 16 || orb % 16) return TERRACE_EINVAL;
    if ((!inner && n_rows > 0) || !outer || !out || (!src && n_src > 0)) return TERRACE_EINVAL;
#define TERRACE_C2O(S)                                                                                             \
    (out_dtype == TERRACE_F32    ? launch_combine2_so<S, TERRACE_F32>(src, n_src, inner, n_rows, fan_inner, outer, n_out, fan_outer, hidden, out, s) \
     : out_dtype == TERRACE_BF16 ? launch_combine2_so<S, TERRACE_BF16>(src, n_src, inner, n_rows, fan_inner, outer, n_out, fan_outer, hidden, out, s) \
                                 : launch_combine2_so<S, TERRACE_F16>(src, n_src, inner, n_rows, fan_inner, outer, n_out, fan_outer, hidden, out, s))
    if (src_dtype == TERRACE_F32) return TERRACE_C2O(TERRACE_F32);
    if (src_dtype == TERRACE_BF16) return TERRACE_C2O(TERRACE_BF16);
    return TERRACE_C2O(TERRACE_F16);
#undef TERRACE_C2O
}

int launch_copy(const void *x, void *y, size_t nbytes, hipStream_t s) {
    if (nbytes == 0) return TERRACE_OK;
    const uintptr_t bits = (uintptr_t)x | (uintptr_t)y | (uintptr_t)nbytes;
    if ((bits & 15) == 0) {
        const int64_t n = (int64_t)(nbytes / 16);
        const int64_t blocks = (n + kBlock - 1) / kBlock;
        copy_kernel<u32x4, 1><<<(unsigned)blocks, kBlock, 0, s>>>((const u32x4 *)x, (u32x4 *)y, n);
    } else {
        const int64_t n = (int64_t)nbytes;
        int64_t blocks = (n + kBlock * 4 - 1) / (kBlock * 4);
        if (blocks > 256 * 16) blocks = 256 * 16;
        copy_kernel<uint8_t, 4><<<(int)blocks, kBlock, 0, s>>>((const uint8_t *)x, (uint8_t *)y, n);
    }
    return check_launch();
}

int launch_index_chain(const int64_t *table, int64_t n_table, const int64_t *idx, int64_t n, int64_t *out,
                       hipStream_t s) {
    if (n <= 0) return TERRACE_OK;
    index_chain_kernel<<<(int)((n + kBlock - 1) / kBlock), kBlock, 0, s>>>(table, n_table, idx, n, out);
    return check_launch();
}

int launch_index_chain2(const int64_t *outer, int64_t n_outer, const int64_t *inner, int64_t n_inner,
                        const int64_t *idx, int64_t n, int64_t *out, hipStream_t s) {
    if (n <= 0) return TERRACE_OK;
    index_chain2_kernel<<<(int)((n + kBlock - 1) / kBlock), kBlock, 0, s>>>(outer, n_outer, inner, n_inner, idx, n,
                                                                           out);
    return check_launch();
}

int launch_send_splits(const int64_t *node_counts, int world, int rpn, int my_local, int64_t *send, hipStream_t s) {
    send_splits_kernel<<<1, 256, 0, s>>>(node_counts, world, rpn, my_local, send);
    return check_launch();
}

}  // namespace terrace
