// Shared pieces of the counting-sort index build (sort.hip, pack.hip).
#pragma once

#include "common.hpp"

namespace terrace {

constexpr int kMaxBuckets = 2048;
constexpr int kScanThreads = 1024;

// A "unit" is the contiguous run of items one wave owns: chunks * 64 of them.  The count and rank kernels
// run `wpb` waves (units) per workgroup.
//
// Two ways from counts to cursors:
//   direct  the count kernel leaves, per unit, the exclusive prefix of the counts inside its workgroup and, per
//           workgroup, the workgroup's totals (blocktot, bucket-major); every rank workgroup then adds up the
//           totals of all buckets before its own and of the workgroups before itself -- n_buckets * n_blocks
//           words from L2 -- and no launch stands between count and rank;
//   scan    the count kernel leaves plain per-unit counts and a one-workgroup scan launch turns the whole table
//           into cursors (tables too large for every workgroup to re-read).
// And for inputs one workgroup can hold (kSoloMaxItems): no count launch at all -- the rank workgroup counts its
// waves' units in LDS first (`solo`).
struct Units {
    int64_t n_items;
    int chunks;       // 64-item chunks per unit: 1, 4 or 16, growing with the item count
    int n_units;
    int n_buckets;
    int wpb;          // waves per workgroup of the count / rank kernels (4 or 16)
    int n_blocks;     // their grid
    int direct;       // 1: no scan launch (see above)
    int solo = 0;     // 1: one workgroup holds every item and the rank launch counts for itself (no count launch)
};

constexpr int kDirectMaxBuckets = 256;
constexpr int64_t kSoloMaxItems = 1024;  // 16 waves x 64 items
constexpr int kDirectMaxWords = 16384;   // n_buckets * n_blocks a rank workgroup may re-read

Units make_units(int64_t n_items, int n_buckets);
// Fills wpb / n_blocks / direct from n_units and n_buckets.
void finish_units(Units &u);
size_t units_table_bytes(const Units &u);
// Words of the table region: [n_units * n_buckets] counts or prefixes, then start[n_buckets + 1], then (direct)
// blocktot[n_buckets * n_blocks], then census[n_blocks * 4] (the send side's per-workgroup guard quantities).
__host__ __device__ inline int64_t units_start_at(const Units &u) { return (int64_t)u.n_units * u.n_buckets; }
__host__ __device__ inline int64_t units_blocktot_at(const Units &u) { return units_start_at(u) + u.n_buckets + 1; }
__host__ __device__ inline int64_t units_census_at(const Units &u) {
    return units_blocktot_at(u) + (int64_t)u.n_buckets * u.n_blocks;
}

// What the one workgroup of a sort that holds every bucket's total and offset publishes for the caller, each
// plane optional: the histogram as int64 and / or float32, the exclusive offsets, and min(count, capacity).
struct TableOut {
    int64_t *hist_i64 = nullptr;
    float *hist_f32 = nullptr;
    int64_t *offsets_i64 = nullptr;
    int64_t *kept_i64 = nullptr;
    int64_t capacity = INT64_MAX;
    __device__ __forceinline__ void put(int b, int32_t count, int32_t offset) const {
        if (hist_i64) hist_i64[b] = count;
        if (hist_f32) hist_f32[b] = (float)count;
        if (offsets_i64) offsets_i64[b] = offset;
        if (kept_i64) kept_i64[b] = count < capacity ? count : capacity;
    }
};

// Scan path: exclusive prefix over the bucket-major count table table[b * n_units + unit], in place; also
// start[b] (n_buckets + 1 int32 right after the table), the optional histogram / offsets planes
// and a zeroed status block.
void launch_scan(const Units &u, int32_t *table, const TableOut &out, int32_t *status, hipStream_t s);

constexpr int kSortBlockMax = 1024;      // 16 waves: the widest count / rank workgroup

// Direct path, rank side: called by every thread of a workgroup (any whole number of waves) before it places
// anything of count workgroup `me`.  From the workgroup totals the count kernel left it derives, into LDS,
//   start[b]  first place of bucket b (n_buckets + 1 entries, the last one the item total),
//   base[b]   first place of the items of bucket b that count workgroup `me` holds,
// using tot[n_buckets] as scratch; with `publish` it also writes start[] after the table and fills the caller's
// planes (`out`) (exactly one workgroup of a launch does).  A unit's cursor is then
// base[b] + table[b * n_units + unit].
__device__ __forceinline__ void direct_block_base(const Units &u, int32_t *__restrict__ table, int me, bool publish,
                                                  lds_i32 *tot, lds_i32 *base, lds_i32 *start, const TableOut &out) {
    const int lane = lane_id(), w = wave_in_block(), nw = (int)(blockDim.x >> 6);
    const int32_t *blocktot = table + units_blocktot_at(u);
    for (int b = w; b < u.n_buckets; b += nw) {            // one wave per bucket: no two waves share a word
        int t = 0, before = 0;
        for (int blk = lane; blk < u.n_blocks; blk += kWave) {
            const int v = blocktot[(int64_t)b * u.n_blocks + blk];
            t += v;
            before += blk < me ? v : 0;
        }
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
            t += __shfl_xor(t, d, kWave);
            before += __shfl_xor(before, d, kWave);
        }
        if (lane == 0) {
            tot[b] = t;
            base[b] = before;
        }
    }
    __syncthreads();
    if (w == 0) {
        int carry = 0;
        for (int b0 = 0; b0 < u.n_buckets; b0 += kWave) {
            const int b = b0 + lane;
            const int v = b < u.n_buckets ? tot[b] : 0;
            const int incl = wave_inclusive_scan(v);
            if (b < u.n_buckets) {
                start[b] = carry + incl - v;
                base[b] = base[b] + carry + incl - v;
            }
            carry += __shfl(incl, kWave - 1, kWave);
        }
        if (lane == 0) start[u.n_buckets] = carry;
    }
    __syncthreads();
    if (publish) {
        int32_t *start_out = table + units_start_at(u);
        for (int b = threadIdx.x; b <= u.n_buckets; b += blockDim.x) {
            const int32_t s0 = start[b];
            start_out[b] = s0;
            if (b == u.n_buckets) break;
            out.put(b, tot[b], s0);
        }
    }
}

// Direct path, count side: called by every thread of a count workgroup once the per-bucket counts of its u.wpb
// units sit in LDS (counts[unit_in_block * n_buckets + b], units past the end hold zeros) and a __syncthreads() has
// passed.  Writes each unit's exclusive prefix inside the workgroup and the workgroup's totals.
__device__ __forceinline__ void direct_block_counts(const Units &u, int32_t *__restrict__ table, lds_i32 *counts) {
    const int nw = u.wpb, me = (int)blockIdx.x;
    int32_t *blocktot = table + units_blocktot_at(u);
    for (int i = threadIdx.x; i < nw * u.n_buckets; i += blockDim.x) {
        const int ww = i / u.n_buckets, b = i - ww * u.n_buckets;
        int run = 0;
        for (int x = 0; x < ww; ++x) run += counts[x * u.n_buckets + b];
        const int un = me * nw + ww;
        if (un < u.n_units) table[(int64_t)b * u.n_units + un] = run;
        if (ww == nw - 1) blocktot[(int64_t)b * u.n_blocks + me] = run + counts[ww * u.n_buckets + b];
    }
}

// n_dst / n_src bound the row ids the movers accept: an id outside [0, bound) is a dead entry.
template <typename I>
int launch_scatter_rows(const void *src, void *dst, const I *pos, int64_t n_src, int fan, int64_t row_bytes,
                        int64_t n_dst, hipStream_t s);
template <typename I>
int launch_gather_rows(const void *src, void *out, const I *idx, int64_t n_out, int64_t row_bytes, int64_t n_src,
                       hipStream_t s);

// Send side with a token's node set in one 64-bit word (n_nodes <= 64, k <= 16, a count table small enough for
// the direct path); returns false when the geometry is outside that and the caller must take the (token, run)-item
// path.
bool k2_token_path_applies(int64_t T, int k, int n_nodes);
size_t k2_token_workspace(int64_t T, int k, int n_nodes, int groups_m);
// Where run_k2_token leaves the [T, groups_m] int32 send-row positions inside its workspace.
const int32_t *k2_token_positions(const void *ws, int64_t T, int k, int n_nodes);
int run_k2_token(const void *hidden, const int64_t *expert_idx, const void *gates, int64_t T, int64_t row_bytes,
                 int gate_bytes, int k, int slots, int n_nodes, int n_experts, int groups_m, void *payload,
                 int64_t *mask, void *gate_rows, int64_t *u_src, int64_t *node_counts, int64_t *u_node,
                 int64_t *inverse, int64_t *node_offsets, int64_t *pair_table, int64_t *sort_order,
                 int64_t *token_rows, void *gate_sorted, int64_t *pair_src, int64_t *combine_table, int32_t *status,
                 void *ws, int64_t mask_pitch, int64_t gate_pitch, int gate_pad, hipStream_t s);

}  // namespace terrace
