// Index build: stable counting sorts over small key ranges, without atomics.
//
// All three index stages of the path are the same object -- "put items in stable ascending
// order of a key with few distinct values":
//   send side   item = (token, run)   key = destination node      (plan + Hop-A wire planes)
//   arrival     item = (row, slot i)  key = owner card            (Hop-B arrival chain)
//   expert card item = received row   key = local expert          (expert-order regroup)
// Unordered atomic cursors cannot give a stable order, so placement is
//   dest = start[key] + (items with that key in earlier units) + (rank inside the unit),
// built in two launches (three for very large tables):
//   count  each wave owns a contiguous "unit" of items and histograms it in wave-private LDS; the workgroup
//          leaves each unit's prefix inside the workgroup and the workgroup's totals;
//   rank   each workgroup adds up the totals before it (a few KB from L2), each wave replays its unit, ranks
//          items with wave ballots, and emits the outputs.
//   (scan  tables too large for every rank workgroup to re-read: one workgroup turns the plain [unit][bucket]
//          counts into exclusive cursors between the two.)
// Up to 1024 items the rank launch is one workgroup that counts for itself, and no count launch runs.
// The row payload itself is moved afterwards by the scatter/gather kernels of rows.hip.
#include "sort.hpp"

namespace terrace {

void finish_units(Units &u) {
    // direct: 16-wave workgroups keep the number of workgroup totals a rank workgroup re-reads small; up to 16
    // units are one such workgroup, which then needs no count launch (solo).  Per sort at 512 items: 5.6 us against
    // 4.6 + 6.4 as count + rank; larger inputs in one workgroup (2048 items as four chunks per wave: 8.9 us
    // against 4.0 + 6.4) gain too little to be worth one CU writing every output plane.
    u.wpb = (u.n_units >= 64 || u.n_units <= 16) ? 16 : 4;
    u.n_blocks = (u.n_units + u.wpb - 1) / u.wpb;
    u.direct = u.n_buckets <= kDirectMaxBuckets && (int64_t)u.n_buckets * u.n_blocks <= kDirectMaxWords;
    if (!u.direct) {
        u.wpb = 4;
        u.n_blocks = (u.n_units + u.wpb - 1) / u.wpb;
    }
    u.solo = u.direct && u.n_blocks == 1 && u.n_items <= kSoloMaxItems;
}

Units make_units(int64_t n_items, int n_buckets) {
    Units u;
    u.n_items = n_items;
    u.n_buckets = n_buckets;
    // Unit size.  A chunk more per wave costs the count and rank passes about 1 us; more units cost the direct
    // path more workgroup totals to re-read and the scan path a larger table (16K entries 5.5 us, 64K entries
    // 12 us).  One chunk per wave up to 4096 units, then four, then sixteen (at 262144 items one chunk per wave
    // measured 8 us a step better than four, arrival and regroup together; at 524288 items one and four measured the
    // same); when even that leaves a table the scan path must take, the scan path's own limits (16K / 64K entries)
    // choose.
    u.chunks = 16;
    for (int c : {1, 4}) {
        if ((n_items + 64 * c - 1) / (64 * c) <= 4096) {
            u.chunks = c;
            break;
        }
    }
    u.n_units = (int)((n_items + 64 * u.chunks - 1) / (64 * u.chunks));
    if (u.n_units < 1) u.n_units = 1;
    finish_units(u);
    if (!u.direct) {
        u.chunks = 16;
        const int64_t limit[] = {16384, 65536};
        const int choice[] = {1, 4};
        for (int i = 0; i < 2; ++i) {
            if ((n_items + 64 * choice[i] - 1) / (64 * choice[i]) * n_buckets <= limit[i]) {
                u.chunks = choice[i];
                break;
            }
        }
        u.n_units = (int)((n_items + 64 * u.chunks - 1) / (64 * u.chunks));
        if (u.n_units < 1) u.n_units = 1;
        finish_units(u);
    }
    return u;
}

size_t units_table_bytes(const Units &u) {
    const size_t words = (size_t)u.n_units * u.n_buckets + u.n_buckets + 1 +
                         (u.direct ? (size_t)u.n_buckets * u.n_blocks + 4 * (size_t)u.n_blocks : 0);
    return align_up(words * sizeof(int32_t), 256);
}

// ---------------------------------------------------------------------------------------------
// key functors: return the bucket of an item, clamped into range; *bad is set for ids outside it
// ---------------------------------------------------------------------------------------------
struct KeyAffine {           // bucket = (plane[item] - sub) / div
    const int64_t *plane;
    int64_t sub;
    int div;
    int n_buckets;
    // the plane may be a [rows, width] table sitting inside wider rows (a wire container): item
    // r*width + i is then at plane[r*pitch + i]
    int width = 1;
    int64_t pitch = 1;
    // a value outside [sub, sub + n_buckets*div): false = contained in bucket 0 (a sort must place every item),
    // true = not an item at all (a histogram must not count it); reported as TERRACE_FAULT_ID_RANGE either way
    bool drop_bad = false;
    // fetch() is one unconditional load (the kernels issue every chunk's fetch before any key is
    // used, so the loads overlap); bucket() turns the fetched value into the key
    __device__ __forceinline__ int64_t fetch(int64_t item) const {
        const uint32_t r = (uint32_t)item / (uint32_t)width;            // items are below 2^31
        const int64_t at = pitch == width ? item : (int64_t)r * pitch + (int64_t)((uint32_t)item - r * (uint32_t)width);
        return plane[at];
    }
    __device__ __forceinline__ int bucket(int64_t, int64_t fetched, bool *bad) const {
        const int64_t v = fetched - sub;
        const bool out = v < 0 || v >= (int64_t)n_buckets * div;
        if (out) *bad = true;
        return out ? (drop_bad ? -1 : 0) : (int)((uint32_t)v / (uint32_t)div);
    }
};

// A token's k expert ids and their nodes, in registers when k <= KMAX (KMAX > 0), else re-read
// through L1.  Padding entries hold INT_MAX so they rank after every real id.  An id is narrowed only after its
// 64-bit value has been bounded: a negative one becomes -1 and one beyond the int range INT_MAX - 1, so neither
// can alias a valid expert and both are reported as out of range by whoever tests the id.
__device__ __forceinline__ int narrow_id(int64_t x) {
    return x < 0 ? -1 : (x > 0x7FFFFFFE ? 0x7FFFFFFE : (int)x);
}

template <int KMAX>
struct RowIds {
    int v[KMAX > 0 ? KMAX : 1];
    int nd[KMAX > 0 ? KMAX : 1];
    const int64_t *row;
    int k, slots;
    __device__ __forceinline__ void load(const int64_t *r, int k_, int slots_) {
        row = r;
        k = k_;
        slots = slots_;
        if constexpr (KMAX > 0) {
#pragma unroll
            for (int j = 0; j < KMAX; ++j) {
                v[j] = j < k ? narrow_id(r[j]) : 0x7FFFFFFF;
                nd[j] = j < k ? (v[j] < 0 ? -1 : v[j] / slots) : 0x7FFFFFFF;
            }
        }
    }
    __device__ __forceinline__ int at(int j) const {
        if constexpr (KMAX > 0) return v[j];
        else return narrow_id(row[j]);
    }
    __device__ __forceinline__ int node(int j) const {
        if constexpr (KMAX > 0) return nd[j];
        else {
            const int e = narrow_id(row[j]);
            return e < 0 ? -1 : e / slots;
        }
    }
};

// Ascending rank of column j inside the row by (id, column): equal ids keep their column order, so the ranks of a
// row are always a permutation of 0..k-1.
template <int KMAX>
__device__ __forceinline__ int rank_in_row(const RowIds<KMAX> &ids, int j) {
    const int e = ids.at(j);
    int r = 0;
    if constexpr (KMAX > 0) {
#pragma unroll
        for (int i = 0; i < KMAX; ++i) r += (ids.v[i] < e || (ids.v[i] == e && i < j)) ? 1 : 0;
    } else {
        for (int i = 0; i < ids.k; ++i) {
            const int o = ids.at(i);
            r += (o < e || (o == e && i < j)) ? 1 : 0;
        }
    }
    return r;
}

// Column of the element whose ascending rank inside the row is `want`.
template <int KMAX>
__device__ __forceinline__ int column_with_rank(const RowIds<KMAX> &ids, int want) {
    int found = -1;
    if constexpr (KMAX > 0) {
#pragma unroll
        for (int j = 0; j < KMAX; ++j)
            if (j < ids.k && rank_in_row(ids, j) == want) found = j;
    } else {
        for (int j = 0; j < ids.k; ++j)
            if (rank_in_row(ids, j) == want) found = j;
    }
    return found;
}

template <int KMAX>
__device__ __forceinline__ int node_of_column(const RowIds<KMAX> &ids, int col) {
    int n = -1;
    if constexpr (KMAX > 0) {
#pragma unroll
        for (int j = 0; j < KMAX; ++j)
            if (j == col) n = ids.nd[j];
    } else {
        if (col >= 0) n = ids.node(col);
    }
    return n;
}

template <int KMAX>
struct KeyRun {              // item = t*M + m  ->  node of the m-th run of token t's ascending row
    const int64_t *expert_idx;
    int k, groups_m, quota, slots, n_nodes;
    __device__ __forceinline__ int64_t fetch(int64_t) const { return 0; }
    __device__ __forceinline__ int bucket(int64_t item, int64_t, bool *bad) const {
        const int64_t t = item / groups_m;
        const int m = (int)(item - t * groups_m);
        RowIds<KMAX> ids;
        ids.load(expert_idx + t * k, k, slots);
        const int col = column_with_rank(ids, m * quota);
        const int n = node_of_column(ids, col);
        if (col < 0 || n < 0 || n >= n_nodes) {
            *bad = true;
            return 0;
        }
        return n;
    }
};

// An emitter that loads nothing of its own.
struct NoPre {};

// General plan with more nodes than one mask word holds: item = (token, column); an item counts only when it is the
// first column of its token on its node, so each occupied (token, node) pair is one item, keyed by the node.
// Items enumerate token-major, hence pairs of one node come out in ascending token order
// (terrace/ta2a.py:205-253: the (node ascending, token ascending) rows of the general branch).
struct KeyFirstOnNode {
    const int64_t *expert_idx;
    int k, slots, n_nodes, n_experts;
    __device__ __forceinline__ int64_t fetch(int64_t item) const { return expert_idx[item]; }
    // -1: not an item (a later column on a node the token already touches, or an id out of range)
    __device__ __forceinline__ int bucket(int64_t item, int64_t e, bool *bad) const {
        if (e < 0 || e >= n_experts) {
            *bad = true;
            return -1;
        }
        const int node = (int)(e / slots);
        const int64_t t = item / k;
        const int j = (int)(item - t * k);
        const int64_t *row = expert_idx + t * k;
        for (int i = 0; i < j; ++i) {
            const int64_t o = row[i];
            if (o >= 0 && o < n_experts && (int)(o / slots) == node) return -1;
        }
        return node;
    }
};

struct EmitPlanWide {
    const int64_t *expert_idx;
    int k, slots, n_experts;
    int64_t *u_src, *u_node, *inverse;
    static constexpr bool kTallies = false;
    static constexpr bool kFills = false;
    typedef NoPre Pre;
    __device__ __forceinline__ Pre fetch(int64_t) const { return Pre{}; }
    __device__ __forceinline__ int operator()(int64_t item, int node, int32_t row, int64_t, Pre, const int32_t *,
                                              int *) const {
        const int64_t t = item / k;
        const int j = (int)(item - t * k);
        u_src[row] = t;
        u_node[row] = node;
        const int64_t *ids = expert_idx + t * k;
        for (int i = j; i < k; ++i) {                  // every column of the token on this node rides this row
            const int64_t o = ids[i];
            if (o >= 0 && o < n_experts && (int)(o / slots) == node) inverse[t * k + i] = row;
        }
        return 0;
    }
};

__global__ __launch_bounds__(kBlock) void mark_bad_ids_kernel(const int64_t *__restrict__ expert_idx, int64_t n,
                                                              int n_experts, int64_t *__restrict__ inverse) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int64_t e = expert_idx[i];
    if (e < 0 || e >= n_experts) inverse[i] = -1;
}

// Lanes of the wave that hold the same key as this one (valid lanes only): one ballot per key bit
// instead of one pass per distinct key.
__device__ __forceinline__ uint64_t same_key_lanes(int key, bool valid, int key_bits) {
    uint64_t peers = __ballot(valid);
    for (int b = 0; b < key_bits; ++b) {
        const bool bit = (key >> b) & 1;
        const uint64_t set = __ballot(valid && bit);
        peers &= bit ? set : ~set;
    }
    return peers;
}

__device__ __forceinline__ int bits_for(int n_buckets) { return n_buckets <= 1 ? 0 : 32 - __builtin_clz(n_buckets - 1); }

// ---------------------------------------------------------------------------------------------
// count: table is bucket-major, table[b * n_units + unit]
// ---------------------------------------------------------------------------------------------
template <typename KeyFn, int CH>
__global__ __launch_bounds__(kSortBlockMax) void count_kernel(KeyFn key_of, Units u, int32_t *__restrict__ table,
                                                              int32_t *__restrict__ status) {
    extern __shared__ int32_t lds[];
    const int lane = lane_id();
    const int w = wave_in_block();
    lds_i32 *hist = (lds_i32 *)lds + w * u.n_buckets;
    const int unit = blockIdx.x * u.wpb + w;
    const bool active = unit < u.n_units;           // an idle wave of the last workgroup still holds zero counts
    if (!active && !u.direct) return;
    for (int b = lane; b < u.n_buckets; b += kWave) hist[b] = 0;
    __builtin_amdgcn_wave_barrier();
    if (active) {
        const int key_bits = bits_for(u.n_buckets);
        const int64_t first = (int64_t)unit * CH * kWave;
        int64_t fetched[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) {       // every chunk's load is issued before any key is computed
            const int64_t item = first + (int64_t)c * kWave + lane;
            fetched[c] = key_of.fetch(item < u.n_items ? item : u.n_items - 1);
        }
        int keys[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int64_t item = first + (int64_t)c * kWave + lane;
            bool bad = false;
            const int key = key_of.bucket(item < u.n_items ? item : u.n_items - 1, fetched[c], &bad);
            keys[c] = item < u.n_items ? key : -1;
        }
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int key = keys[c];
            const bool valid = key >= 0;
            const uint64_t peers = same_key_lanes(key, valid, key_bits);
            // the lowest lane of each key adds the key's count: distinct keys, distinct words
            if (valid && lane == __builtin_ctzll(peers)) hist[key] = hist[key] + __popcll(peers);
            __builtin_amdgcn_wave_barrier();
        }
    }
    if (!u.direct) {
        for (int b = lane; b < u.n_buckets; b += kWave) table[(int64_t)b * u.n_units + unit] = hist[b];
        return;
    }
    // the rank launch accumulates into the status block; nothing but this launch is ordered before it
    if (status && blockIdx.x == 0 && threadIdx.x < TERRACE_STATUS_WORDS) status[threadIdx.x] = 0;
    __syncthreads();
    direct_block_counts(u, table, (lds_i32 *)lds);
}

// ---------------------------------------------------------------------------------------------
// scan: exclusive prefix over the bucket-major table, in place (staged through LDS when it
// fits).  Also writes start[b] (n_buckets+1 int32 after the table), the caller's histogram and
// offsets planes, and zeroes the status block.
// ---------------------------------------------------------------------------------------------
// Each of the 16 waves owns a contiguous span (a multiple of 256 entries) and walks it 256
// entries at a time, 16 bytes per lane, so every access is a fully coalesced 1 KB.
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ i32x4 load4_guarded(const int32_t *t, int64_t i, int64_t n) {
    if (i + 3 < n) return *(const i32x4 *)(t + i);
    i32x4 v = {0, 0, 0, 0};
    if (i < n) v[0] = t[i];
    if (i + 1 < n) v[1] = t[i + 1];
    if (i + 2 < n) v[2] = t[i + 2];
    return v;
}

__global__ __launch_bounds__(kScanThreads) void scan_kernel(Units u, int32_t *__restrict__ table, TableOut out,
        int32_t *__restrict__ status) {
    constexpr int kWaves = kScanThreads / kWave;
    __shared__ int32_t wave_tot[kWaves];
    __shared__ int32_t grand_total;
    const int tid = threadIdx.x, lane = lane_id(), w = tid >> 6;
    const int64_t n = (int64_t)u.n_units * u.n_buckets;
    int32_t *start = table + n;
    if (status && tid < TERRACE_STATUS_WORDS) status[tid] = 0;
    const int64_t span = ((n + kWaves - 1) / kWaves + 255) / 256 * 256;
    const int64_t lo = w * span, hi = lo + span < n ? lo + span : n;
    i32x4 acc = {0, 0, 0, 0};
    for (int64_t base = lo; base < hi; base += 256) acc += load4_guarded(table, base + lane * 4, hi);
    int32_t sum = acc[0] + acc[1] + acc[2] + acc[3];
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) sum += __shfl_xor(sum, d, kWave);
    if (lane == 0) wave_tot[w] = sum;
    __syncthreads();
    if (tid < kWave) {
        const int32_t t = tid < kWaves ? wave_tot[tid] : 0;
        const int32_t ti = wave_inclusive_scan(t);
        if (tid < kWaves) wave_tot[tid] = ti - t;
        if (tid == kWaves - 1) grand_total = ti;
    }
    __syncthreads();
    int32_t carry = wave_tot[w];
    for (int64_t base = lo; base < hi; base += 256) {
        const int64_t i = base + lane * 4;
        const i32x4 c = load4_guarded(table, i, hi);
        const int32_t s4 = c[0] + c[1] + c[2] + c[3];
        const int32_t incl = wave_inclusive_scan(s4);
        i32x4 o;
        o[0] = carry + incl - s4;
        o[1] = o[0] + c[0];
        o[2] = o[1] + c[1];
        o[3] = o[2] + c[2];
        if (i + 3 < hi) {
            *(i32x4 *)(table + i) = o;
        } else {
            if (i < hi) table[i] = o[0];
            if (i + 1 < hi) table[i + 1] = o[1];
            if (i + 2 < hi) table[i + 2] = o[2];
        }
        carry += __shfl(incl, kWave - 1, kWave);
    }
    __syncthreads();
    for (int b = tid; b <= u.n_buckets; b += kScanThreads) {
        const int32_t s0 = b < u.n_buckets ? table[(int64_t)b * u.n_units] : grand_total;
        start[b] = s0;
        if (b == u.n_buckets) break;
        const int32_t s1 = b + 1 < u.n_buckets ? table[(int64_t)(b + 1) * u.n_units] : grand_total;
        out.put(b, s1 - s0, s0);
    }
}

// Tables of up to 64K entries (every geometry make_units produces unless the bucket count itself is
// huge): the same walk as scan_kernel -- each of the 16 waves owns a contiguous span and covers it 256
// entries (one coalesced kilobyte) at a time -- but a wave first takes its whole span into registers,
// all loads issued at once, and scans it there: one memory round trip in, one out.
constexpr int kScanRegVecs = 16;                 // 16 x 256 entries per wave

__global__ __launch_bounds__(kScanThreads) void scan_registers_kernel(Units u, int32_t *__restrict__ table, TableOut out,
        int32_t *__restrict__ status) {
    constexpr int kWaves = kScanThreads / kWave;
    __shared__ int32_t wave_tot[kWaves];
    __shared__ int32_t grand_total;
    const int tid = threadIdx.x, lane = lane_id(), w = tid >> 6;
    const int64_t n = (int64_t)u.n_units * u.n_buckets;
    int32_t *start = table + n;
    if (status && tid < TERRACE_STATUS_WORDS) status[tid] = 0;
    const int64_t span = ((n + kWaves - 1) / kWaves + 255) / 256 * 256;            // <= kScanRegVecs * 256
    const int64_t lo = w * span, hi = lo + span < n ? lo + span : n;
    i32x4 v[kScanRegVecs];
    int32_t s4[kScanRegVecs];
#pragma unroll
    for (int c = 0; c < kScanRegVecs; ++c) {
        const int64_t i = lo + c * 256 + lane * 4;
        v[c] = i32x4{0, 0, 0, 0};
        if (lo + c * 256 < hi) v[c] = load4_guarded(table, i, hi);
    }
    int32_t sum = 0;
#pragma unroll
    for (int c = 0; c < kScanRegVecs; ++c) {
        s4[c] = v[c][0] + v[c][1] + v[c][2] + v[c][3];
        sum += s4[c];
    }
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) sum += __shfl_xor(sum, d, kWave);
    if (lane == 0) wave_tot[w] = sum;
    __syncthreads();
    if (tid < kWave) {
        const int32_t t = tid < kWaves ? wave_tot[tid] : 0;
        const int32_t ti = wave_inclusive_scan(t);
        if (tid < kWaves) wave_tot[tid] = ti - t;
        if (tid == kWaves - 1) grand_total = ti;
    }
    __syncthreads();
    int32_t carry = wave_tot[w];
#pragma unroll
    for (int c = 0; c < kScanRegVecs; ++c) {
        if (lo + c * 256 < hi) {                                                  // wave-uniform
            const int64_t i = lo + c * 256 + lane * 4;
            const int32_t incl = wave_inclusive_scan(s4[c]);
            i32x4 o;
            o[0] = carry + incl - s4[c];
            o[1] = o[0] + v[c][0];
            o[2] = o[1] + v[c][1];
            o[3] = o[2] + v[c][2];
            if (i + 3 < hi) {
                *(i32x4 *)(table + i) = o;
            } else {
                if (i < hi) table[i] = o[0];
                if (i + 1 < hi) table[i + 1] = o[1];
                if (i + 2 < hi) table[i + 2] = o[2];
            }
            carry += __shfl(incl, kWave - 1, kWave);
        }
    }
    __syncthreads();
    for (int b = tid; b <= u.n_buckets; b += kScanThreads) {
        const int32_t s0 = b < u.n_buckets ? table[(int64_t)b * u.n_units] : grand_total;
        start[b] = s0;
        if (b == u.n_buckets) break;
        const int32_t s1 = b + 1 < u.n_buckets ? table[(int64_t)(b + 1) * u.n_units] : grand_total;
        out.put(b, s1 - s0, s0);
    }
}

void launch_scan(const Units &u, int32_t *table, const TableOut &out, int32_t *status, hipStream_t s) {
    const int64_t n = (int64_t)u.n_units * u.n_buckets;
    if (n <= (int64_t)kScanThreads * kScanRegVecs * 4)
        scan_registers_kernel<<<1, kScanThreads, 0, s>>>(u, table, out, status);
    else
        scan_kernel<<<1, kScanThreads, 0, s>>>(u, table, out, status);
}

// ---------------------------------------------------------------------------------------------
// rank
// ---------------------------------------------------------------------------------------------
template <typename KeyFn, typename EmitFn, int CH>
__global__ __launch_bounds__(kSortBlockMax) void rank_kernel(KeyFn key_of, EmitFn emit, Units u,
                                                             int32_t *__restrict__ table, TableOut out,
                                                             int32_t *__restrict__ status) {
    extern __shared__ int32_t lds[];
    const int lane = lane_id();
    const int w = wave_in_block();
    lds_i32 *cursor = (lds_i32 *)lds + w * u.n_buckets;
    const int unit = blockIdx.x * u.wpb + w;
    const bool active = unit < u.n_units;
    if (!active && !u.direct) return;
    const int key_bits = bits_for(u.n_buckets);
    const int64_t first = (int64_t)unit * CH * kWave;
    int fault = 0;
    // phase 1: every chunk's key load and the emitter's own input loads, all issued before any is used
    int64_t fetched[CH];
    typename EmitFn::Pre pre[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int64_t item = first + (int64_t)c * kWave + lane;
        const int64_t safe = item < u.n_items ? item : u.n_items - 1;
        fetched[c] = key_of.fetch(safe);
        pre[c] = emit.fetch(safe);
    }
    const int32_t *start = table + units_start_at(u);
    int keys[CH];
    if (u.solo) {
        // The whole input is this one workgroup's, and no count launch ran: each wave counts its own unit into its
        // row of LDS, the rows become prefixes over the waves, the totals are scanned, and the status block -- which
        // the count launch clears otherwise -- is cleared here, fenced, ahead of the barriers every later atomic
        // sits behind.
        lds_i32 *rows = (lds_i32 *)lds;
        lds_i32 *tot = rows + u.wpb * u.n_buckets, *lstart = tot + 2 * u.n_buckets;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int64_t item = first + (int64_t)c * kWave + lane;
            bool bad = false;
            const int key = key_of.bucket(item < u.n_items ? item : u.n_items - 1, fetched[c], &bad);
            keys[c] = item < u.n_items ? key : -1;
            if (bad && item < u.n_items) fault |= TERRACE_FAULT_ID_RANGE;
        }
        for (int b = lane; b < u.n_buckets; b += kWave) cursor[b] = 0;
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int key = keys[c];
            const bool valid = key >= 0;
            const uint64_t peers = same_key_lanes(key, valid, key_bits);
            if (valid && lane == __builtin_ctzll(peers)) cursor[key] = cursor[key] + __popcll(peers);
            __builtin_amdgcn_wave_barrier();
        }
        if (status && threadIdx.x < TERRACE_STATUS_WORDS) {
            status[threadIdx.x] = 0;
            __threadfence();
        }
        __syncthreads();
        for (int b = threadIdx.x; b < u.n_buckets; b += blockDim.x) {
            int run = 0;
            for (int x = 0; x < u.wpb; ++x) {
                const int v = rows[x * u.n_buckets + b];
                rows[x * u.n_buckets + b] = run;
                run += v;
            }
            tot[b] = run;
        }
        __syncthreads();
        if (w == 0) {
            int carry = 0;
            for (int b0 = 0; b0 < u.n_buckets; b0 += kWave) {
                const int b = b0 + lane;
                const int v = b < u.n_buckets ? tot[b] : 0;
                const int incl = wave_inclusive_scan(v);
                if (b < u.n_buckets) lstart[b] = carry + incl - v;
                carry += __shfl(incl, kWave - 1, kWave);
            }
            if (lane == 0) lstart[u.n_buckets] = carry;
        }
        __syncthreads();
        int32_t *start_out = table + units_start_at(u);
        for (int b = threadIdx.x; b <= u.n_buckets; b += blockDim.x) {
            const int32_t s0 = lstart[b];
            start_out[b] = s0;
            if (b < u.n_buckets) out.put(b, tot[b], s0);
        }
        if (!active) return;
        for (int b = lane; b < u.n_buckets; b += kWave) cursor[b] = cursor[b] + lstart[b];
        start = (const int32_t *)lstart;
    } else if (u.direct) {
        // this unit's prefixes inside its workgroup: loaded now, with the keys, so that the only memory round trip
        // of the kernel is the one the workgroup totals below share with them
        constexpr int kTabRegs = kDirectMaxBuckets / kWave;
        int32_t tab[kTabRegs];
#pragma unroll
        for (int i = 0; i < kTabRegs; ++i) {
            const int b = lane + i * kWave;
            tab[i] = (active && b < u.n_buckets) ? table[(int64_t)b * u.n_units + unit] : 0;
        }
        lds_i32 *shared = (lds_i32 *)lds + u.wpb * u.n_buckets;          // tot, base, start
        lds_i32 *base = shared + u.n_buckets, *lstart = base + u.n_buckets;
        direct_block_base(u, table, (int)blockIdx.x, blockIdx.x == 0, shared, base, lstart, out);
        if (!active) return;
#pragma unroll
        for (int i = 0; i < kTabRegs; ++i) {
            const int b = lane + i * kWave;
            if (b < u.n_buckets) cursor[b] = base[b] + tab[i];
        }
        start = (const int32_t *)lstart;
    } else {
        for (int b = lane; b < u.n_buckets; b += kWave) cursor[b] = table[(int64_t)b * u.n_units + unit];
    }
    if (!u.solo) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int64_t item = first + (int64_t)c * kWave + lane;
            bool bad = false;
            const int key = key_of.bucket(item < u.n_items ? item : u.n_items - 1, fetched[c], &bad);
            keys[c] = item < u.n_items ? key : -1;
            if (bad && item < u.n_items) fault |= TERRACE_FAULT_ID_RANGE;
        }
    }
    __builtin_amdgcn_wave_barrier();
    int tally[2] = {0, 0};
    // phase 2: places, in registers
    int32_t dests[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int key = keys[c];
        const bool valid = key >= 0;
        const uint64_t peers = same_key_lanes(key, valid, key_bits);
        const int32_t base = valid ? cursor[key] : 0;
        dests[c] = base + __popcll(peers & lanes_below(lane));
        __builtin_amdgcn_wave_barrier();
        if (valid && lane == __builtin_ctzll(peers)) cursor[key] = base + __popcll(peers);
        __builtin_amdgcn_wave_barrier();
    }
    // phase 3: outputs
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int64_t item = first + (int64_t)c * kWave + lane;
        if (keys[c] >= 0) fault |= emit(item, keys[c], dests[c], fetched[c], pre[c], start, tally);
    }
    if constexpr (EmitFn::kFills) emit.fill(unit, u.n_units, lane, start);
    if (!status) return;
    if (fault) atomicOr(&status[0], fault);
    if (EmitFn::kTallies) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            int v = tally[i];
#pragma unroll
            for (int d = 1; d < kWave; d <<= 1) v += __shfl_xor(v, d, kWave);
            if (lane == 0 && v) atomicAdd(&status[1 + i], v);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// emit functors
// ---------------------------------------------------------------------------------------------
// An emitter's fetch(item) loads what it needs beyond the key (issued with the key loads); its call
// operator gets the key's fetched value and that Pre back and only computes and stores.
struct EmitOrder {           // plain stable argsort: order[dest] = item
    int64_t *order;
    static constexpr bool kTallies = false;
    static constexpr bool kFills = false;
    typedef NoPre Pre;
    __device__ __forceinline__ Pre fetch(int64_t) const { return Pre{}; }
    __device__ __forceinline__ int operator()(int64_t item, int, int32_t dest, int64_t, Pre, const int32_t *,
                                              int *) const {
        order[dest] = item;
        return 0;
    }
};

struct EmitNothing {
    static constexpr bool kTallies = false;
    static constexpr bool kFills = false;
    typedef NoPre Pre;
    __device__ __forceinline__ Pre fetch(int64_t) const { return Pre{}; }
    __device__ __forceinline__ int operator()(int64_t, int, int32_t, int64_t, Pre, const int32_t *, int *) const {
        return 0;
    }
};

struct EmitArrival {         // terrace/ops/__init__.py:287-299
    const int64_t *rslot;    // [R, quota] at row pitch slot_pitch (int64 elements)
    const void *rgate;       // [R, quota] at row pitch gate_pitch (gate elements)
    int gate_bytes, quota;
    int64_t slot_pitch, gate_pitch;
    void *gate_pairs;
    int64_t *r_idx, *slot_idx, *pair_pos;
    int32_t *pos32;
    int64_t *meta;           // Hop-B container [P, 2]: word 0 the slot id, word 1 the gate then zeros; or NULL
    const int64_t *tags_in;  // [P] a caller's tag per pair, carried to the pair's place: tags_out[dest] = tags_in[p]
    int64_t *tags_out;
    static constexpr bool kTallies = false;
    static constexpr bool kFills = false;
    struct Pre { uint32_t gbits; int64_t tag; };
    __device__ __forceinline__ Pre fetch(int64_t p) const {
        Pre pre{0u, -1};
        if (rgate) {
            const uint32_t r = (uint32_t)p / (uint32_t)quota;
            const int64_t at = (int64_t)r * gate_pitch + (int64_t)((uint32_t)p - r * (uint32_t)quota);
            pre.gbits = gate_bytes == 4 ? ((const uint32_t *)rgate)[at] : (uint32_t)((const uint16_t *)rgate)[at];
        }
        if (tags_in) pre.tag = tags_in[p];
        return pre;
    }
    // `slot` is the value the key was computed from: rslot[r, i]
    __device__ __forceinline__ int operator()(int64_t p, int, int32_t dest, int64_t slot, Pre pre, const int32_t *,
                                              int *) const {
        if (tags_out) tags_out[dest] = pre.tag;
        r_idx[dest] = (int64_t)((uint32_t)p / (uint32_t)quota);
        if (slot_idx) slot_idx[dest] = slot;
        if (rgate && gate_pairs) {
            if (gate_bytes == 4) ((uint32_t *)gate_pairs)[dest] = pre.gbits;
            else ((uint16_t *)gate_pairs)[dest] = (uint16_t)pre.gbits;
        }
        if (meta) {
            meta[2 * (int64_t)dest] = slot;
            meta[2 * (int64_t)dest + 1] = (int64_t)(uint64_t)pre.gbits;
        }
        pos32[p] = dest;
        if (pair_pos) pair_pos[p] = dest;
        return 0;
    }
};

struct EmitHopB {            // arrival + expert-order regroup in one placement (all of the node's slots local)
    const void *rgate;       // [R, quota] at row pitch gate_pitch (gate elements), or NULL
    int gate_bytes, quota;
    int64_t gate_pitch;
    int64_t capacity;        // < 0: drop-less
    int64_t *place;          // [P]: where pair p sits in the expert-order buffer, -1 = dropped
    uint8_t *kept;           // [P]
    int64_t *pair_of_place;  // [places]: the pair behind each place
    void *permuted_gate;     // [places]
    int32_t *pos32;          // [P]: `place` for the row mover
    const int64_t *tags_in;  // [P] a caller's tag per pair: place_by_tag[tags_in[p]] = place of p (-1 dropped)
    int64_t *place_by_tag;
    int64_t n_tags;
    static constexpr bool kTallies = false;
    static constexpr bool kFills = false;
    struct Pre { uint32_t gbits; int64_t tag; };
    __device__ __forceinline__ Pre fetch(int64_t p) const {
        Pre pre{0u, -1};
        if (rgate) {
            const uint32_t r = (uint32_t)p / (uint32_t)quota;
            const int64_t at = (int64_t)r * gate_pitch + (int64_t)((uint32_t)p - r * (uint32_t)quota);
            pre.gbits = gate_bytes == 4 ? ((const uint32_t *)rgate)[at] : (uint32_t)((const uint16_t *)rgate)[at];
        }
        if (tags_in) pre.tag = tags_in[p];
        return pre;
    }
    __device__ __forceinline__ int operator()(int64_t p, int key, int32_t dest, int64_t, Pre pre,
                                              const int32_t *start, int *) const {
        int64_t d = dest;
        bool keep = true;
        if (capacity >= 0) {
            const int64_t rank = dest - start[key];
            keep = rank < capacity;
            d = keep ? key * capacity + rank : -1;
        }
        pos32[p] = (int32_t)d;
        if (place) place[p] = d;
        if (kept) kept[p] = keep ? 1 : 0;
        if (place_by_tag && (uint64_t)pre.tag < (uint64_t)n_tags) place_by_tag[pre.tag] = d;
        if (keep) {
            if (pair_of_place) pair_of_place[d] = p;
            if (rgate && permuted_gate) {
                if (gate_bytes == 4) ((uint32_t *)permuted_gate)[d] = pre.gbits;
                else ((uint16_t *)permuted_gate)[d] = (uint16_t)pre.gbits;
            }
        }
        return 0;
    }
};

// The places of a capacity layout that hold no row: zero rows, zero gates, no pair.  blockIdx.x = x * chunks + c
// looks after places [c * pad_rows, (c + 1) * pad_rows) of expert x and leaves at once when they are all in use;
// the first workgroup of an expert also writes kept_per_expert.
constexpr int kPadRows = 16;             // the most places one workgroup looks after (the launcher picks pad_rows)
template <typename V>
__global__ __launch_bounds__(kBlock) void zero_pad_kernel(const int32_t *__restrict__ start, int epr, int64_t capacity,
                                                          int chunks, int pad_rows, V *__restrict__ rows, int64_t row_vecs,
                                                          int64_t live_vecs,
                                                          void *__restrict__ gate_plane, int gate_bytes,
                                                          int64_t *__restrict__ pair_of_place,
                                                          int64_t *__restrict__ kept_per_expert) {
    const int x = blockIdx.x / chunks, c = blockIdx.x - x * chunks;
    const int64_t count = start[x + 1] - start[x];
    const int64_t used = count < capacity ? count : capacity;
    if (c == 0 && threadIdx.x == 0 && kept_per_expert) kept_per_expert[x] = used;
    int64_t lo = (int64_t)c * pad_rows, hi = lo + pad_rows;
    if (lo < used) lo = used;
    if (hi > capacity) hi = capacity;
    if (lo >= hi) return;
    const int64_t first = x * capacity + lo, n = hi - lo;
    for (int64_t i = threadIdx.x; i < n; i += kBlock) {
        if (pair_of_place) pair_of_place[first + i] = -1;
        if (gate_plane) {
            if (gate_bytes == 4) ((uint32_t *)gate_plane)[first + i] = 0u;
            else ((uint16_t *)gate_plane)[first + i] = (uint16_t)0;
        }
    }
    if (!rows) return;
    V *o = rows + first * row_vecs;
    V z;
    __builtin_memset(&z, 0, sizeof(V));
    if (live_vecs == row_vecs) {
        for (int64_t i = threadIdx.x; i < n * row_vecs; i += kBlock) __builtin_nontemporal_store(z, o + i);
    } else {                     // rows on a pitch: only the width of each row is written
        for (int64_t i = threadIdx.x; i < n * live_vecs; i += kBlock) {
            const int64_t r = i / live_vecs;
            __builtin_nontemporal_store(z, o + r * row_vecs + (i - r * live_vecs));
        }
    }
}

struct EmitPairs {           // terrace/ta2a_fwd.py:605-628, general branch: pairs come as (row, slot) lists
    const int64_t *r_in, *slot_in;
    const void *rgate;       // sparse plane [R, gate_width]
    int gate_bytes, gate_width;
    int64_t R;
    void *gate_pairs;
    int64_t *r_idx, *slot_idx, *ordo;
    int32_t *src32;          // source row of each output place (-1: row id out of range)
    static constexpr bool kTallies = false;
    static constexpr bool kFills = false;
    struct Pre { int64_t r; };
    __device__ __forceinline__ Pre fetch(int64_t p) const { return Pre{r_in[p]}; }
    __device__ __forceinline__ int operator()(int64_t p, int, int32_t dest, int64_t sl, Pre pre, const int32_t *,
                                              int *) const {
        const int64_t r = pre.r;
        const bool ok = r >= 0 && r < R;
        r_idx[dest] = r;
        slot_idx[dest] = sl;
        if (ordo) ordo[dest] = p;
        src32[dest] = ok ? (int32_t)r : -1;
        if (rgate) {
            const bool gok = ok && sl >= 0 && sl < gate_width;
            const int64_t cell = r * gate_width + sl;
            if (gate_bytes == 4) ((uint32_t *)gate_pairs)[dest] = gok ? ((const uint32_t *)rgate)[cell] : 0u;
            else ((uint16_t *)gate_pairs)[dest] = gok ? ((const uint16_t *)rgate)[cell] : (uint16_t)0;
        }
        return ok ? 0 : TERRACE_FAULT_ID_RANGE;
    }
};

struct EmitRegroup {         // terrace/ta2a_fwd.py:641-646 (+ capacity cut)
    int64_t capacity;        // < 0: drop-less
    int64_t *order, *dest_out;
    uint8_t *kept;
    int32_t *order32;
    const int64_t *tags_in;  // [P] a caller's tag per row: place_by_tag[tags_in[p]] = place of row p (-1 dropped)
    int64_t *place_by_tag;
    int64_t n_tags;
    const void *gate_in;     // drop-less layout only: the row's gate goes to its place from here; with a capacity
    void *gate_out;          // the padded plane is gathered per place afterwards (its padding places are zeros)
    int gate_bytes;
    int64_t gate_pitch;
    int32_t *gidx;           // capacity layout only: the source row of every place, -1 for a padding place
    int epr;
    static constexpr bool kTallies = false;
    static constexpr bool kFills = true;
    // The padding places of the capacity layout, shared out over the launch's units: place d = x*capacity + r is
    // padding when r is past expert x's count (the kept places are written by the rows that take them).
    __device__ __forceinline__ void fill(int unit, int n_units, int lane, const int32_t *start) const {
        if (capacity < 0 || !gidx) return;
        const int64_t places = (int64_t)epr * capacity;
        const int64_t per = (places + n_units - 1) / n_units;
        const int64_t lo = (int64_t)unit * per, hi = lo + per < places ? lo + per : places;
        for (int64_t d = lo + lane; d < hi; d += kWave) {
            const uint32_t x = (uint32_t)d / (uint32_t)capacity;          // places < 2^31
            const int64_t r = d - (int64_t)x * capacity;
            if (r >= start[x + 1] - start[x]) gidx[d] = -1;
        }
    }
    struct Pre { int64_t tag; uint32_t gate; };
    __device__ __forceinline__ Pre fetch(int64_t p) const {
        Pre pre{tags_in ? tags_in[p] : -1, 0u};
        if (gate_in) pre.gate = gate_bytes == 4 ? ((const uint32_t *)gate_in)[p * gate_pitch]
                                                : (uint32_t)((const uint16_t *)gate_in)[p * gate_pitch];
        return pre;
    }
    __device__ __forceinline__ int operator()(int64_t p, int key, int32_t dest, int64_t, Pre pre,
                                              const int32_t *start, int *) const {
        order32[dest] = (int32_t)p;
        if (order) order[dest] = p;
        if (gate_in) {
            if (gate_bytes == 4) ((uint32_t *)gate_out)[dest] = pre.gate;
            else ((uint16_t *)gate_out)[dest] = (uint16_t)pre.gate;
        }
        int64_t d = dest;
        bool keep = true;
        if (capacity >= 0) {
            const int64_t rank = dest - start[key];
            keep = rank < capacity;
            d = keep ? key * capacity + rank : -1;
        }
        if (dest_out) dest_out[p] = d;
        if (kept) kept[p] = keep ? 1 : 0;
        if (capacity >= 0 && gidx && keep) gidx[d] = (int32_t)p;
        if (place_by_tag && (uint64_t)pre.tag < (uint64_t)n_tags) place_by_tag[pre.tag] = d;
        return 0;
    }
};

template <int KMAX>
struct EmitPack {            // terrace/ta2a.py:246-253 + terrace/ta2a_fwd.py:236-248
    const int64_t *expert_idx;
    const void *gates;
    int gate_bytes, k, groups_m, quota, slots, n_experts;
    int64_t *mask, *u_src, *u_node, *inverse, *pair_table, *sort_order, *token_rows;
    void *gate_rows, *gate_sorted;
    int32_t *pos32;
    int64_t *pair_src;                   // [T*M*quota]: t*k + rank behind each Hop-A pair, -1 where none
    int64_t *combine_table;              // [T, k]: ranks that own no pair are set to -1 here
    int64_t mask_pitch, gate_pitch;      // row pitches of the mask / gate_rows planes, in their own elements
    int gate_pad;                        // gate elements to zero after a row's quota gates
    // status word 1 receives the number of occupied (token, node) pairs, word 2 the number of
    // those holding other than k/M experts: the two quantities terrace/ta2a.py:170-204 checks.
    static constexpr bool kTallies = true;
    static constexpr bool kFills = false;
    typedef NoPre Pre;
    __device__ __forceinline__ Pre fetch(int64_t) const { return Pre{}; }
    // rank m*quota + i of token t and cell i of its send row `row`: no pair, zero slot, zero gate
    __device__ __forceinline__ void put_defaults(int64_t t, int m, int32_t row, int i) const {
        const int64_t at = t * k + (int64_t)m * quota + i;
        if (pair_table) pair_table[at] = -1;
        if (sort_order) sort_order[at] = 0;
        if (combine_table) combine_table[at] = -1;
        if (pair_src) pair_src[(int64_t)row * quota + i] = -1;
        mask[(int64_t)row * mask_pitch + i] = 0;
        if (!gates) return;
        const int64_t gcell = (int64_t)row * gate_pitch + i;
        if (gate_bytes == 4) {
            ((uint32_t *)gate_rows)[gcell] = 0u;
            if (gate_sorted) ((uint32_t *)gate_sorted)[at] = 0u;
        } else {
            ((uint16_t *)gate_rows)[gcell] = (uint16_t)0;
            if (gate_sorted) ((uint16_t *)gate_sorted)[at] = (uint16_t)0;
        }
    }
    __device__ __forceinline__ int operator()(int64_t item, int node, int32_t row, int64_t, Pre, const int32_t *,
                                              int *tally) const {
        const int64_t t = item / groups_m;
        const int m = (int)(item - t * groups_m);
        RowIds<KMAX> ids;
        ids.load(expert_idx + t * k, k, slots);
        int fault = 0;
        if (m == 0) {
            int occupied = 0, off_quota = 0;
            auto census = [&](int j) {
                const int nj = ids.node(j);
                int same = 0, earlier = 0;
                auto cmp = [&](int i) {
                    const bool hit = ids.node(i) == nj;
                    same += hit ? 1 : 0;
                    earlier += (hit && i < j) ? 1 : 0;
                };
                if constexpr (KMAX > 0) {
#pragma unroll
                    for (int i = 0; i < KMAX; ++i)
                        if (i < k) cmp(i);
                } else {
                    for (int i = 0; i < k; ++i) cmp(i);
                }
                if (earlier == 0) {
                    occupied += 1;
                    off_quota += same != quota ? 1 : 0;
                }
            };
            if constexpr (KMAX > 0) {
#pragma unroll
                for (int j = 0; j < KMAX; ++j)
                    if (j < k) census(j);
            } else {
                for (int j = 0; j < k; ++j) census(j);
            }
            tally[0] += occupied;
            tally[1] += off_quota;
            if (occupied != groups_m) fault |= TERRACE_FAULT_FANOUT;
            if (off_quota) fault |= TERRACE_FAULT_QUOTA;
        }
        u_src[row] = t;
        if (u_node) u_node[row] = node;
        if (token_rows) token_rows[item] = row;
        pos32[item] = row;
        // A run owns ranks [m*quota, (m+1)*quota) of its token's per-rank planes and the quota cells of its
        // row.  With duplicate ids ranks collide and some of those are claimed by no element: they are given
        // the defaults below (no pair, zero cells), so every entry is defined whatever the routing.
        // the row's pad after its quota gates (wire containers).  One loop per element width: with the width test
        // inside a single loop this toolchain's backend fails to select an instruction at build time.
        if (gates && gate_bytes == 4)
            for (int z = 0; z < gate_pad; ++z) ((uint32_t *)gate_rows)[(int64_t)row * gate_pitch + quota + z] = 0u;
        if (gates && gate_bytes != 4)
            for (int z = 0; z < gate_pad; ++z) ((uint16_t *)gate_rows)[(int64_t)row * gate_pitch + quota + z] = (uint16_t)0;
        uint64_t claimed = 0;
        const bool wide = quota > 64;            // more ranks than the mask holds: defaults first, for all of them
        if (wide)
            for (int i = 0; i < quota; ++i) put_defaults(t, m, row, i);
        auto body = [&](int j) {
            const int e = ids.at(j);
            if (e < 0 || e >= n_experts) fault |= TERRACE_FAULT_ID_RANGE;
            const int r = rank_in_row(ids, j);
            if (r / quota != m) return;
            const int i = r - m * quota;
            if (!wide) claimed |= 1ull << i;
            const int64_t cell = (int64_t)row * quota + i;
            mask[(int64_t)row * mask_pitch + i] = e >= 0 ? e - ids.node(j) * slots : 0;
            if (gates) {
                const int64_t gcell = (int64_t)row * gate_pitch + i;
                if (gate_bytes == 4) {
                    const uint32_t gv = ((const uint32_t *)gates)[t * k + j];
                    ((uint32_t *)gate_rows)[gcell] = gv;
                    if (gate_sorted) ((uint32_t *)gate_sorted)[t * k + r] = gv;
                } else {
                    const uint16_t gv = ((const uint16_t *)gates)[t * k + j];
                    ((uint16_t *)gate_rows)[gcell] = gv;
                    if (gate_sorted) ((uint16_t *)gate_sorted)[t * k + r] = gv;
                }
            }
            if (inverse) inverse[t * k + j] = row;
            if (pair_table) pair_table[t * k + r] = cell;
            if (sort_order) sort_order[t * k + r] = j;
            if (pair_src) pair_src[cell] = t * k + r;
        };
        if constexpr (KMAX > 0) {
#pragma unroll
            for (int j = 0; j < KMAX; ++j)
                if (j < k) body(j);
        } else {
            for (int j = 0; j < k; ++j) body(j);
        }
        if (!wide) {
            const uint64_t all = quota == 64 ? ~0ull : (1ull << quota) - 1ull;
            uint64_t holes = ~claimed & all;
            while (holes) {
                put_defaults(t, m, row, __builtin_ctzll(holes));
                holes &= holes - 1;
            }
        }
        return fault;
    }
};

__global__ __launch_bounds__(kBlock) void fill_zero_kernel(uint8_t *__restrict__ p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) p[i] = 0;
}

__global__ __launch_bounds__(kBlock) void fill_minus_one_kernel(int64_t *__restrict__ p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) p[i] = -1;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void gather_elems_kernel(const T *__restrict__ src,
                                                              const int32_t *__restrict__ idx, int64_t n,
                                                              int64_t src_pitch, T *__restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int32_t a = idx[i];
    out[i] = a < 0 ? T(0) : src[(int64_t)a * src_pitch];
}

__global__ void empty_outputs_kernel(int64_t *hist, float *hist_f, int64_t *offsets, int n, int32_t *status) {
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        if (hist) hist[i] = 0;
        if (hist_f) hist_f[i] = 0.0f;
        if (offsets) offsets[i] = 0;
    }
    if (status && threadIdx.x < TERRACE_STATUS_WORDS) status[threadIdx.x] = 0;
}

// _pack_quota_wire for a caller-provided inverse: one lane per token.
template <int KMAX>
__global__ __launch_bounds__(kBlock) void pack_quota_wire_kernel(const int64_t *__restrict__ expert_idx,
                                                                 const void *__restrict__ gates,
                                                                 const int64_t *__restrict__ inverse, int64_t T, int k,
                                                                 int gate_bytes, int64_t n_rows, int slots, int quota,
                                                                 int64_t *__restrict__ slot_tab,
                                                                 void *__restrict__ gate_tab,
                                                                 int32_t *__restrict__ status) {
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= T) return;
    RowIds<KMAX> ids;
    ids.load(expert_idx + t * k, k, slots);
    bool bad = false;
    auto body = [&](int j) {
        const int e = ids.at(j);
        const int r = rank_in_row(ids, j);
        const int m = r / quota, i = r - m * quota;
        // the run's row is the one `inverse` names for its first (smallest) expert
        int64_t row = -1;
        auto find = [&](int jj) {
            if (rank_in_row(ids, jj) == m * quota) row = inverse[t * k + jj];
        };
        if constexpr (KMAX > 0) {
#pragma unroll
            for (int jj = 0; jj < KMAX; ++jj)
                if (jj < k) find(jj);
        } else {
            for (int jj = 0; jj < k; ++jj) find(jj);
        }
        if (row < 0 || row >= n_rows) {
            bad = true;
            return;
        }
        const int64_t cell = row * quota + i;
        slot_tab[cell] = ((e % slots) + slots) % slots;
        if (gates) {
            if (gate_bytes == 4) ((uint32_t *)gate_tab)[cell] = ((const uint32_t *)gates)[t * k + j];
            else ((uint16_t *)gate_tab)[cell] = ((const uint16_t *)gates)[t * k + j];
        }
    };
    if constexpr (KMAX > 0) {
#pragma unroll
        for (int j = 0; j < KMAX; ++j)
            if (j < k) body(j);
    } else {
        for (int j = 0; j < k; ++j) body(j);
    }
    if (bad && status) atomicOr(&status[0], TERRACE_FAULT_ID_RANGE);
}

// ---------------------------------------------------------------------------------------------
// host drivers
// ---------------------------------------------------------------------------------------------
static size_t lds_count(const Units &u) { return (size_t)u.wpb * u.n_buckets * sizeof(int32_t); }
static size_t lds_rank(const Units &u) {
    return ((size_t)u.wpb * u.n_buckets + (u.direct ? 3 * (size_t)u.n_buckets + 1 : 0)) * sizeof(int32_t);
}

template <typename KeyFn, typename EmitFn>
static int run_sort(const KeyFn &key, const EmitFn &emit, Units u, int32_t *table, const TableOut &out,
                    int32_t *status, bool do_rank, hipStream_t s) {
    if (!do_rank && u.direct) {          // the histogram alone: the scan launch writes it, so take that path
        u.direct = 0;                    // (the table region of a direct layout is large enough for it)
        u.solo = 0;
        u.wpb = 4;
        u.n_blocks = (u.n_units + u.wpb - 1) / u.wpb;
    }
    const int blocks = u.n_blocks, threads = u.wpb * kWave;
    const size_t lc = lds_count(u), lr = lds_rank(u);
    if (!u.solo) {
        if (u.chunks == 1) count_kernel<KeyFn, 1><<<blocks, threads, lc, s>>>(key, u, table, status);
        else if (u.chunks == 4) count_kernel<KeyFn, 4><<<blocks, threads, lc, s>>>(key, u, table, status);
        else count_kernel<KeyFn, 16><<<blocks, threads, lc, s>>>(key, u, table, status);
    }
    if (!u.direct) launch_scan(u, table, out, status, s);
    if (do_rank) {
        if (u.chunks == 1) rank_kernel<KeyFn, EmitFn, 1><<<blocks, threads, lr, s>>>(key, emit, u, table, out, status);
        else if (u.chunks == 4) rank_kernel<KeyFn, EmitFn, 4><<<blocks, threads, lr, s>>>(key, emit, u, table, out, status);
        else rank_kernel<KeyFn, EmitFn, 16><<<blocks, threads, lr, s>>>(key, emit, u, table, out, status);
    }
    return check_launch();
}

static int empty_outputs(int64_t *hist, float *hist_f, int64_t *offsets, int n, int32_t *status, hipStream_t s) {
    empty_outputs_kernel<<<1, 256, 0, s>>>(hist, hist_f, offsets, n, status);
    return check_launch();
}

// ---- histogram / argsort --------------------------------------------------------------------
size_t hist_workspace(int64_t n, int n_buckets) {
    if (n <= 0 || n_buckets <= 0 || n_buckets > kMaxBuckets) return 256;
    return units_table_bytes(make_units(n, n_buckets));
}

int run_hist(const int64_t *idx, int64_t n, int n_buckets, void *out, int as_float, int32_t *status, void *ws,
             size_t ws_bytes, hipStream_t s) {
    if (n_buckets <= 0 || n_buckets > kMaxBuckets || n < 0 || !out) return TERRACE_EINVAL;
    int64_t *h = as_float ? nullptr : (int64_t *)out;
    float *hf = as_float ? (float *)out : nullptr;
    if (n == 0) return empty_outputs(h, hf, nullptr, n_buckets, status, s);
    if (!idx || !ws) return TERRACE_EINVAL;
    const Units u = make_units(n, n_buckets);
    if (ws_bytes < units_table_bytes(u)) return TERRACE_ENOSPC;
    KeyAffine key{idx, 0, 1, n_buckets, 1, 1, true};
    // the rank pass runs only to report out-of-range ids
    TableOut planes;
    planes.hist_i64 = h;
    planes.hist_f32 = hf;
    return run_sort(key, EmitNothing{}, u, (int32_t *)ws, planes, status, status != nullptr, s);
}

int run_argsort_small(const int64_t *keyp, int64_t n, int n_buckets, int64_t *order, int64_t *hist, int32_t *status,
                      void *ws, size_t ws_bytes, hipStream_t s) {
    if (n_buckets <= 0 || n_buckets > kMaxBuckets || n < 0) return TERRACE_EINVAL;
    if (n == 0) return empty_outputs(hist, nullptr, nullptr, hist ? n_buckets : 0, status, s);
    if (!keyp || !order || !ws) return TERRACE_EINVAL;
    const Units u = make_units(n, n_buckets);
    if (ws_bytes < units_table_bytes(u)) return TERRACE_ENOSPC;
    KeyAffine key{keyp, 0, 1, n_buckets};
    TableOut out;
    out.hist_i64 = hist;
    return run_sort(key, EmitOrder{order}, u, (int32_t *)ws, out, status, true, s);
}

// ---- general plan beyond 64 nodes ----------------------------------------------------------------
size_t plan_wide_workspace(int64_t T, int k, int n_nodes) {
    if (T <= 0 || k <= 0 || n_nodes <= 0 || n_nodes > kMaxBuckets) return 256;
    return units_table_bytes(make_units(T * k, n_nodes));
}

int run_plan_wide(const int64_t *expert_idx, int64_t T, int k, int slots, int n_nodes, int n_experts, int64_t *u_src,
                  int64_t *u_node, int64_t *counts, int64_t *inverse, int32_t *status, void *ws, size_t ws_bytes,
                  hipStream_t s) {
    if (n_nodes > kMaxBuckets) return TERRACE_EINVAL;
    if (T == 0) return empty_outputs(counts, nullptr, nullptr, n_nodes, status, s);
    const Units u = make_units(T * k, n_nodes);
    if (!ws || ws_bytes < units_table_bytes(u)) return TERRACE_ENOSPC;
    KeyFirstOnNode key{expert_idx, k, slots, n_nodes, n_experts};
    EmitPlanWide emit{expert_idx, k, slots, n_experts, u_src, u_node, inverse};
    TableOut out;
    out.hist_i64 = counts;
    int rc = run_sort(key, emit, u, (int32_t *)ws, out, status, true, s);
    if (rc != TERRACE_OK) return rc;
    mark_bad_ids_kernel<<<(int)((T * k + kBlock - 1) / kBlock), kBlock, 0, s>>>(expert_idx, T * k, n_experts, inverse);
    return check_launch();
}

// ---- Hop-B arrival ----------------------------------------------------------------------------
size_t k1_workspace(int64_t R, int quota, int rpn) {
    const int64_t P = R * quota;
    if (P <= 0 || rpn <= 0 || rpn > kMaxBuckets) return 256;
    return units_table_bytes(make_units(P, rpn)) + align_up((size_t)P * sizeof(int32_t), 256);
}

int run_k1_arrival(const void *rx, const int64_t *rslot, const void *rgate, int64_t R, int64_t row_bytes,
                   int gate_bytes, int quota, int epr, int rpn, int my_local, void *send_buf, void *gate_pairs,
                   int64_t *r_idx, int64_t *slot_idx, int64_t *i_send, int64_t *pair_pos, int32_t *status, void *ws,
                   size_t ws_bytes, int64_t slot_pitch, int64_t gate_pitch, int64_t *meta, const int64_t *tags_in,
                   int64_t *tags_out, hipStream_t s) {
    if (R < 0 || quota <= 0 || epr <= 0 || rpn <= 0 || rpn > kMaxBuckets || my_local < 0 || my_local >= rpn ||
        !i_send || (gate_bytes != 2 && gate_bytes != 4) || row_bytes < 0 || slot_pitch < quota || gate_pitch < quota)
        return TERRACE_EINVAL;
    const int64_t P = R * quota;
    if (P >= (int64_t)1 << 31) return TERRACE_EINVAL;
    if (P == 0) return empty_outputs(i_send, nullptr, nullptr, rpn, status, s);
    if (!rslot || !r_idx || (!slot_idx && !meta) || !ws || (rx && !send_buf) || (rgate && !gate_pairs && !meta))
        return TERRACE_EINVAL;
    const Units u = make_units(P, rpn);
    const size_t table_bytes = units_table_bytes(u);
    if (ws_bytes < table_bytes + align_up((size_t)P * sizeof(int32_t), 256)) return TERRACE_ENOSPC;
    int32_t *table = (int32_t *)ws;
    int32_t *pos32 = (int32_t *)((char *)ws + table_bytes);
    KeyAffine key{rslot, 0, epr, rpn, quota, slot_pitch};
    EmitArrival emit{rslot, rgate, gate_bytes, quota, slot_pitch, gate_pitch, gate_pairs, r_idx, slot_idx, pair_pos,
                     pos32, meta, tags_out ? tags_in : nullptr, tags_in ? tags_out : nullptr};
    TableOut out;
    out.hist_i64 = i_send;
    int rc = run_sort(key, emit, u, table, out, status, true, s);
    if (rc != TERRACE_OK || !rx) return rc;
    return launch_scatter_rows<int32_t>(rx, send_buf, pos32, R, quota, row_bytes, P, s);
}

// ---- Hop-B arrival, general branch (pairs listed explicitly) -------------------------------------
size_t arrival_pairs_workspace(int64_t P, int rpn) {
    if (P <= 0 || rpn <= 0 || rpn > kMaxBuckets) return 256;
    return units_table_bytes(make_units(P, rpn)) + align_up((size_t)P * sizeof(int32_t), 256);
}

int run_arrival_pairs(const void *rx, const int64_t *r_in, const int64_t *slot_in, const void *rgate, int64_t R,
                      int64_t P, int64_t row_bytes, int gate_bytes, int gate_width, int epr, int rpn, void *send_buf,
                      void *gate_pairs, int64_t *r_idx, int64_t *slot_idx, int64_t *i_send, int64_t *ordo,
                      int32_t *status, void *ws, size_t ws_bytes, hipStream_t s) {
    if (R < 0 || P < 0 || epr <= 0 || rpn <= 0 || rpn > kMaxBuckets || !i_send || row_bytes < 0 ||
        (gate_bytes != 2 && gate_bytes != 4) || gate_width < 0 || P >= (int64_t)1 << 31 || R >= (int64_t)1 << 31)
        return TERRACE_EINVAL;
    if (P == 0) return empty_outputs(i_send, nullptr, nullptr, rpn, status, s);
    if (!r_in || !slot_in || !r_idx || !slot_idx || !ws || (rx && !send_buf) || (rgate && !gate_pairs))
        return TERRACE_EINVAL;
    const Units u = make_units(P, rpn);
    const size_t table_bytes = units_table_bytes(u);
    if (ws_bytes < table_bytes + align_up((size_t)P * sizeof(int32_t), 256)) return TERRACE_ENOSPC;
    int32_t *table = (int32_t *)ws;
    int32_t *src32 = (int32_t *)((char *)ws + table_bytes);
    KeyAffine key{slot_in, 0, epr, rpn};
    EmitPairs emit{r_in, slot_in, rgate, gate_bytes, gate_width, R, gate_pairs, r_idx, slot_idx, ordo, src32};
    TableOut out;
    out.hist_i64 = i_send;
    int rc = run_sort(key, emit, u, table, out, status, true, s);
    if (rc != TERRACE_OK || !rx) return rc;
    return launch_gather_rows<int32_t>(rx, send_buf, src32, P, row_bytes, R, s);
}

// ---- Hop-B local scatter in one pass ------------------------------------------------------------
// = run_k1_arrival followed by run_regroup over all n_local slots of the node, without the buffer between them:
// a stable sort by owner card and then by local expert is one stable sort by slot.
typedef uint32_t pad_u32x4 __attribute__((ext_vector_type(4)));

size_t hopb_workspace(int64_t R, int quota, int n_local) {
    const int64_t P = R * quota;
    if (P <= 0 || n_local <= 0 || n_local > kMaxBuckets) return 256;
    return units_table_bytes(make_units(P, n_local)) + align_up((size_t)P * sizeof(int32_t), 256);
}

static int launch_zero_pad(const int32_t *start, int epr, int64_t capacity, void *rows, int64_t row_bytes,
                           void *gate_plane, int gate_bytes, int64_t *pair_of_place, int64_t *kept_per_expert,
                           hipStream_t s) {
    if (epr <= 0) return TERRACE_OK;
    // places per workgroup: about 16 KB of rows (a shorter run of padding per workgroup measured faster -- the
    // one-pass Hop B of the 4 KB-row capacity workload went 0.673 -> 0.658 ms from 16 places to 4 -- until the
    // workgroups that find nothing to do, which still have to be launched, outweigh it), at most kPadRows; more
    // where that many workgroups would pass what one launch can hold (blocks * kBlock has to stay below 2^32)
    int pad_rows = kPadRows;
    const RowGeom geom = row_geom(row_bytes);
    if (!row_geom_ok(geom) || (geom.pitched() && ((uintptr_t)rows & 15))) return TERRACE_EINVAL;
    if (rows && geom.width > 0) {
        while (pad_rows > 1 && (int64_t)pad_rows * geom.width > 16384) pad_rows /= 2;
    }
    while ((int64_t)epr * ((capacity + pad_rows - 1) / pad_rows) > (int64_t)1 << 22) pad_rows *= 2;
    const int chunks = capacity > 0 ? (int)((capacity + pad_rows - 1) / pad_rows) : 1;
    const int64_t blocks = (int64_t)epr * chunks;
    if (!rows || geom.width == 0) {
        zero_pad_kernel<uint8_t><<<(unsigned)blocks, kBlock, 0, s>>>(start, epr, capacity, chunks, pad_rows, nullptr, 0, 0,
                                                                    gate_plane, gate_bytes, pair_of_place,
                                                                    kept_per_expert);
    } else if ((((uintptr_t)rows | (uintptr_t)geom.width | (uintptr_t)geom.pitch) & 15) == 0) {
        zero_pad_kernel<pad_u32x4><<<(unsigned)blocks, kBlock, 0, s>>>(start, epr, capacity, chunks, pad_rows,
                                                                      (pad_u32x4 *)rows, geom.pitch / 16, geom.width / 16,
                                                                      gate_plane, gate_bytes, pair_of_place,
                                                                      kept_per_expert);
    } else {
        zero_pad_kernel<uint8_t><<<(unsigned)blocks, kBlock, 0, s>>>(start, epr, capacity, chunks, pad_rows,
                                                                    (uint8_t *)rows, geom.pitch, geom.width, gate_plane,
                                                                    gate_bytes, pair_of_place, kept_per_expert);
    }
    return check_launch();
}

int run_hopb_scatter(const void *rx, const int64_t *rslot, const void *rgate, int64_t R, int64_t row_bytes,
                     int gate_bytes, int quota, int first_slot, int n_local, int64_t capacity, void *permuted,
                     void *permuted_gate, int64_t *place, uint8_t *kept, int64_t *pair_of_place,
                     int64_t *tokens_per_expert, int64_t *kept_per_expert, const int64_t *tags_in,
                     int64_t *place_by_tag, int64_t n_tags, int32_t *status, void *ws, size_t ws_bytes,
                     hipStream_t s) {
    if (R < 0 || quota <= 0 || n_local <= 0 || n_local > kMaxBuckets || first_slot < 0 || !tokens_per_expert ||
        (gate_bytes != 2 && gate_bytes != 4) || row_bytes < 0 ||
        (capacity >= 0 && (int64_t)n_local * capacity >= (int64_t)1 << 31))
        return TERRACE_EINVAL;
    if (R > (((int64_t)1 << 31) - 1) / quota) return TERRACE_EINVAL;
    const int64_t P = R * quota;
    const int64_t places = capacity >= 0 ? (int64_t)n_local * capacity : P;
    if (places > 0 && rx && !permuted) return TERRACE_EINVAL;
    if (P == 0) {
        int rc = empty_outputs(tokens_per_expert, nullptr, kept_per_expert, n_local, status, s);
        if (rc != TERRACE_OK || places == 0) return rc;
        if (permuted && row_bytes) fill_zero_kernel<<<1024, kBlock, 0, s>>>((uint8_t *)permuted, places * row_geom(row_bytes).pitch);
        if (permuted_gate) fill_zero_kernel<<<64, kBlock, 0, s>>>((uint8_t *)permuted_gate, places * gate_bytes);
        if (pair_of_place) fill_minus_one_kernel<<<64, kBlock, 0, s>>>(pair_of_place, places);
        return check_launch();
    }
    if (!rslot || !ws) return TERRACE_EINVAL;
    const Units u = make_units(P, n_local);
    const size_t table_bytes = units_table_bytes(u);
    if (ws_bytes < hopb_workspace(R, quota, n_local)) return TERRACE_ENOSPC;
    int32_t *table = (int32_t *)ws;
    int32_t *pos32 = (int32_t *)((char *)ws + table_bytes);
    KeyAffine key{rslot, (int64_t)first_slot, 1, n_local, quota, (int64_t)quota};
    const bool tagged = tags_in && place_by_tag && n_tags > 0;
    EmitHopB emit{rgate, gate_bytes, quota, (int64_t)quota, capacity, place, kept, pair_of_place,
                  rgate ? permuted_gate : nullptr, pos32, tagged ? tags_in : nullptr,
                  tagged ? place_by_tag : nullptr, n_tags};
    TableOut out;
    out.hist_i64 = tokens_per_expert;
    if (capacity < 0) out.kept_i64 = kept_per_expert;          // nothing is dropped: the sort's own publication
    int rc = run_sort(key, emit, u, table, out, status, true, s);
    if (rc != TERRACE_OK) return rc;
    const int32_t *start = table + units_start_at(u);
    if (capacity >= 0) {
        // padding planes now; the padding rows with the row mover (they may be moved later, by the _move call)
        rc = launch_zero_pad(start, n_local, capacity, rx ? permuted : nullptr, rx ? row_bytes : 0,
                             rgate ? permuted_gate : nullptr, gate_bytes, pair_of_place, kept_per_expert, s);
        if (rc != TERRACE_OK) return rc;
    }
    if (!rx) return rc;
    return launch_scatter_rows<int32_t>(rx, permuted, pos32, R, quota, row_bytes, places, s);
}

int run_hopb_scatter_move(const void *rx, int64_t R, int64_t row_bytes, int quota, int n_local, int64_t capacity,
                          void *permuted, const void *ws, size_t ws_bytes, hipStream_t s) {
    if (R < 0 || quota <= 0 || n_local <= 0 || n_local > kMaxBuckets || row_bytes < 0 ||
        (capacity >= 0 && (int64_t)n_local * capacity >= (int64_t)1 << 31))
        return TERRACE_EINVAL;
    if (R > (((int64_t)1 << 31) - 1) / quota) return TERRACE_EINVAL;
    const int64_t P = R * quota;
    const int64_t places = capacity >= 0 ? (int64_t)n_local * capacity : P;
    if (places == 0 || row_bytes == 0) return TERRACE_OK;
    if (!permuted) return TERRACE_EINVAL;
    if (P == 0) {       // all padding
        fill_zero_kernel<<<1024, kBlock, 0, s>>>((uint8_t *)permuted, places * row_geom(row_bytes).pitch);
        return check_launch();
    }
    if (!rx || !ws) return TERRACE_EINVAL;
    if (ws_bytes < hopb_workspace(R, quota, n_local)) return TERRACE_ENOSPC;
    const Units u = make_units(P, n_local);
    const int32_t *table = (const int32_t *)ws;
    const int32_t *pos32 = (const int32_t *)((const char *)ws + units_table_bytes(u));
    if (capacity >= 0) {
        int rc = launch_zero_pad(table + units_start_at(u), n_local, capacity, permuted, row_bytes, nullptr, 4, nullptr,
                                 nullptr, s);
        if (rc != TERRACE_OK) return rc;
    }
    return launch_scatter_rows<int32_t>(rx, permuted, pos32, R, quota, row_bytes, places, s);
}

// ---- expert-order regroup ---------------------------------------------------------------------
size_t regroup_workspace(int64_t P, int epr, int64_t capacity) {
    if (P <= 0 || epr <= 0 || epr > kMaxBuckets) return 256;
    size_t b = units_table_bytes(make_units(P, epr)) + align_up((size_t)P * sizeof(int32_t), 256);
    if (capacity >= 0) b += align_up((size_t)epr * (size_t)capacity * sizeof(int32_t), 256);
    return b;
}

int run_regroup(const void *node_rx, const int64_t *my_slot, const void *my_gate, int64_t P, int64_t row_bytes,
                int gate_bytes, int epr, int my_local, int64_t capacity, void *permuted, void *permuted_gate,
                int64_t *order, int64_t *dest, uint8_t *kept, int64_t *tokens_per_expert, int64_t *kept_per_expert,
                int32_t *status, void *ws, size_t ws_bytes, int64_t slot_pitch, int64_t gate_pitch,
                const int64_t *tags_in, int64_t *place_by_tag, int64_t n_tags, hipStream_t s) {
    if (P < 0 || epr <= 0 || epr > kMaxBuckets || my_local < 0 || !tokens_per_expert || row_bytes < 0 ||
        slot_pitch < 1 || gate_pitch < 1 ||
        (gate_bytes != 2 && gate_bytes != 4) || P >= (int64_t)1 << 31 ||
        (capacity >= 0 && (int64_t)epr * capacity >= (int64_t)1 << 31))
        return TERRACE_EINVAL;
    const int64_t places = capacity >= 0 ? (int64_t)epr * capacity : P;
    if (places > 0 && ((node_rx && !permuted) || (my_gate && !permuted_gate))) return TERRACE_EINVAL;
    if (P == 0) {
        int rc = empty_outputs(tokens_per_expert, nullptr, kept_per_expert, epr, status, s);
        if (rc != TERRACE_OK || places == 0) return rc;
        if (permuted && row_bytes) fill_zero_kernel<<<1024, kBlock, 0, s>>>((uint8_t *)permuted, places * row_geom(row_bytes).pitch);
        if (permuted_gate) fill_zero_kernel<<<64, kBlock, 0, s>>>((uint8_t *)permuted_gate, places * gate_bytes);
        return check_launch();
    }
    if (!my_slot || !ws) return TERRACE_EINVAL;
    const Units u = make_units(P, epr);
    const size_t table_bytes = units_table_bytes(u);
    if (ws_bytes < regroup_workspace(P, epr, capacity)) return TERRACE_ENOSPC;
    int32_t *table = (int32_t *)ws;
    int32_t *order32 = (int32_t *)((char *)ws + table_bytes);
    int32_t *gidx = (int32_t *)((char *)order32 + align_up((size_t)P * sizeof(int32_t), 256));
    KeyAffine key{my_slot, (int64_t)my_local * epr, 1, epr, 1, slot_pitch};
    const bool tagged = tags_in && place_by_tag && n_tags > 0;
    const bool gate_in_sort = my_gate && capacity < 0;
    EmitRegroup emit{capacity, order, dest, kept, order32, tagged ? tags_in : nullptr,
                     tagged ? place_by_tag : nullptr, n_tags, gate_in_sort ? my_gate : nullptr,
                     gate_in_sort ? permuted_gate : nullptr, gate_bytes, gate_pitch, capacity >= 0 ? gidx : nullptr,
                     epr};
    TableOut out;
    out.hist_i64 = tokens_per_expert;
    out.kept_i64 = kept_per_expert;                            // min(count, capacity): the sort's own publication
    if (capacity >= 0) out.capacity = capacity;
    int rc = run_sort(key, emit, u, table, out, status, true, s);
    if (rc != TERRACE_OK) return rc;
    const int32_t *src_of_place = capacity >= 0 ? gidx : order32;    // the rank kernel filled gidx, padding included
    if (my_gate && places > 0 && !gate_in_sort) {
        const int grid = (int)((places + kBlock - 1) / kBlock);
        if (gate_bytes == 4)
            gather_elems_kernel<uint32_t><<<grid, kBlock, 0, s>>>((const uint32_t *)my_gate, src_of_place, places, gate_pitch, (uint32_t *)permuted_gate);
        else
            gather_elems_kernel<uint16_t><<<grid, kBlock, 0, s>>>((const uint16_t *)my_gate, src_of_place, places, gate_pitch, (uint16_t *)permuted_gate);
    }
    rc = check_launch();
    if (rc != TERRACE_OK || !node_rx) return rc;
    return launch_gather_rows<int32_t>(node_rx, permuted, src_of_place, places, row_bytes, P, s);
}

int run_pack_quota_wire(const int64_t *expert_idx, const void *gates, const int64_t *inverse, int64_t T, int k,
                        int gate_bytes, int64_t n_rows, int slots, int quota, int64_t *slot_tab, void *gate_tab,
                        int32_t *status, hipStream_t s) {
    if (T < 0 || k <= 0 || quota <= 0 || k % quota || slots <= 0 || n_rows < 0 ||
        (gate_bytes != 2 && gate_bytes != 4))
        return TERRACE_EINVAL;
    empty_outputs_kernel<<<1, 64, 0, s>>>(nullptr, nullptr, nullptr, 0, status);
    if (T == 0) return check_launch();
    if (!expert_idx || !inverse || !slot_tab || (gates && !gate_tab)) return TERRACE_EINVAL;
    const int grid = (int)((T + kBlock - 1) / kBlock);
    if (k <= 8)
        pack_quota_wire_kernel<8><<<grid, kBlock, 0, s>>>(expert_idx, gates, inverse, T, k, gate_bytes, n_rows, slots, quota, slot_tab, gate_tab, status);
    else if (k <= 16)
        pack_quota_wire_kernel<16><<<grid, kBlock, 0, s>>>(expert_idx, gates, inverse, T, k, gate_bytes, n_rows, slots, quota, slot_tab, gate_tab, status);
    else
        pack_quota_wire_kernel<0><<<grid, kBlock, 0, s>>>(expert_idx, gates, inverse, T, k, gate_bytes, n_rows, slots, quota, slot_tab, gate_tab, status);
    return check_launch();
}

// ---- send side: plan + Hop-A pack ---------------------------------------------------------------
size_t k2_workspace(int64_t T, int k, int n_nodes, int groups_m) {
    const int64_t S = T * groups_m;
    if (S <= 0 || n_nodes <= 0 || n_nodes > kMaxBuckets) return 256;
    const size_t item_path = units_table_bytes(make_units(S, n_nodes)) + align_up((size_t)S * sizeof(int32_t), 256);
    const size_t token_path = k2_token_path_applies(T, k, n_nodes) ? k2_token_workspace(T, k, n_nodes, groups_m) : 0;
    return item_path > token_path ? item_path : token_path;
}

template <int KMAX>
static int run_k2_t(const void *hidden, const int64_t *expert_idx, const void *gates, int64_t T, int64_t row_bytes,
                    int gate_bytes, int k, int slots, int n_nodes, int n_experts, int groups_m, void *payload,
                    int64_t *mask, void *gate_rows, int64_t *u_src, int64_t *node_counts, int64_t *u_node,
                    int64_t *inverse, int64_t *node_offsets, int64_t *pair_table, int64_t *sort_order,
                    int64_t *token_rows, void *gate_sorted, int64_t *pair_src, int64_t *combine_table,
                    int32_t *status, const Units &u, int32_t *table, int32_t *pos32, int64_t mask_pitch,
                    int64_t gate_pitch, int gate_pad, hipStream_t s) {
    const int quota = k / groups_m;
    KeyRun<KMAX> key{expert_idx, k, groups_m, quota, slots, n_nodes};
    EmitPack<KMAX> emit{expert_idx, gates, gate_bytes, k, groups_m, quota, slots, n_experts,
                        mask, u_src, u_node, inverse, pair_table, sort_order, token_rows, gate_rows, gate_sorted,
                        pos32, pair_src, combine_table, mask_pitch, gate_pitch, gate_pad};
    TableOut out;
    out.hist_i64 = node_counts;
    out.offsets_i64 = node_offsets;
    int rc = run_sort(key, emit, u, table, out, status, true, s);
    if (rc != TERRACE_OK || !hidden) return rc;
    return launch_scatter_rows<int32_t>(hidden, payload, pos32, T, groups_m, row_bytes, T * groups_m, s);
}

int run_k2_pack(const void *hidden, const int64_t *expert_idx, const void *gates, int64_t T, int64_t row_bytes,
                int gate_bytes, int k, int world, int n_experts, int rpn, int groups_m, void *payload, int64_t *mask,
                void *gate_rows, int64_t *u_src, int64_t *node_counts, int64_t *u_node, int64_t *inverse,
                int64_t *node_offsets, int64_t *pair_table, int64_t *sort_order, int64_t *token_rows,
                void *gate_sorted, int64_t *pair_src, int64_t *combine_table, int32_t *status, void *ws,
                size_t ws_bytes, int64_t mask_pitch, int64_t gate_pitch, int gate_pad, hipStream_t s) {
    if (mask_pitch <= 0) mask_pitch = groups_m > 0 ? k / groups_m : 0;       // dense planes
    if (gate_pitch <= 0) gate_pitch = groups_m > 0 ? k / groups_m : 0;
    if (T < 0 || k <= 0 || world <= 0 || rpn <= 0 || n_experts <= 0 || groups_m <= 0 || world % rpn ||
        n_experts % world || k % groups_m || row_bytes < 0 || (gate_bytes != 2 && gate_bytes != 4) || !node_counts)
        return TERRACE_EINVAL;
    const int n_nodes = world / rpn;
    const int slots = (n_experts / world) * rpn;
    const int64_t S = T * groups_m;
    if (n_nodes > kMaxBuckets || T * k >= (int64_t)1 << 31 || S >= (int64_t)1 << 31) return TERRACE_EINVAL;
    if (S == 0) return empty_outputs(node_counts, nullptr, node_offsets, n_nodes, status, s);
    if (!expert_idx || !mask || !u_src || !ws || (hidden && !payload) || (gates && !gate_rows)) return TERRACE_EINVAL;
    if (ws_bytes < k2_workspace(T, k, n_nodes, groups_m)) return TERRACE_ENOSPC;
    if (k2_token_path_applies(T, k, n_nodes))
        return run_k2_token(hidden, expert_idx, gates, T, row_bytes, gate_bytes, k, slots, n_nodes, n_experts,
                            groups_m, payload, mask, gate_rows, u_src, node_counts, u_node, inverse, node_offsets,
                            pair_table, sort_order, token_rows, gate_sorted, pair_src, combine_table, status, ws,
                            mask_pitch, gate_pitch, gate_pad, s);
    const Units u = make_units(S, n_nodes);
    const size_t table_bytes = units_table_bytes(u);
    int32_t *table = (int32_t *)ws;
    int32_t *pos32 = (int32_t *)((char *)ws + table_bytes);
#define TERRACE_K2(KM)                                                                                        \
    run_k2_t<KM>(hidden, expert_idx, gates, T, row_bytes, gate_bytes, k, slots, n_nodes, n_experts, groups_m, \
                 payload, mask, gate_rows, u_src, node_counts, u_node, inverse, node_offsets, pair_table,     \
                 sort_order, token_rows, gate_sorted, pair_src, combine_table, status, u, table, pos32, mask_pitch,   \
                 gate_pitch, gate_pad, s)
    if (k <= 8) return TERRACE_K2(8);
    if (k <= 16) return TERRACE_K2(16);
    return TERRACE_K2(0);
#undef TERRACE_K2
}

// ---- second phase of the three stage operators ---------------------------------------------------
// A stage call with its row pointers NULL builds the index planes only and leaves the int32 position plane
// of its row mover in the workspace; these launch that mover later, possibly on another stream, so the
// index chain of the next stage can run beside the row traffic of this one.  The geometry arguments must
// repeat the first phase's: they locate the plane.
int run_k2_pack_move(const void *hidden, int64_t T, int64_t row_bytes, int k, int n_nodes, int groups_m,
                     void *payload, const void *ws, size_t ws_bytes, hipStream_t s) {
    if (T < 0 || k <= 0 || groups_m <= 0 || k % groups_m || n_nodes <= 0 || n_nodes > kMaxBuckets ||
        row_bytes < 0 || T * groups_m >= (int64_t)1 << 31)
        return TERRACE_EINVAL;
    const int64_t S = T * groups_m;
    if (S == 0 || row_bytes == 0) return TERRACE_OK;
    if (!hidden || !payload || !ws) return TERRACE_EINVAL;
    if (ws_bytes < k2_workspace(T, k, n_nodes, groups_m)) return TERRACE_ENOSPC;
    const int32_t *pos32 = k2_token_path_applies(T, k, n_nodes)
                               ? k2_token_positions(ws, T, k, n_nodes)
                               : (const int32_t *)((const char *)ws + units_table_bytes(make_units(S, n_nodes)));
    return launch_scatter_rows<int32_t>(hidden, payload, pos32, T, groups_m, row_bytes, T * groups_m, s);
}

int run_k1_arrival_move(const void *rx, int64_t R, int64_t row_bytes, int quota, int rpn, void *send_buf,
                        const void *ws, size_t ws_bytes, hipStream_t s) {
    if (R < 0 || quota <= 0 || rpn <= 0 || rpn > kMaxBuckets || row_bytes < 0 || R * quota >= (int64_t)1 << 31)
        return TERRACE_EINVAL;
    const int64_t P = R * quota;
    if (P == 0 || row_bytes == 0) return TERRACE_OK;
    if (!rx || !send_buf || !ws) return TERRACE_EINVAL;
    if (ws_bytes < k1_workspace(R, quota, rpn)) return TERRACE_ENOSPC;
    const int32_t *pos32 = (const int32_t *)((const char *)ws + units_table_bytes(make_units(P, rpn)));
    return launch_scatter_rows<int32_t>(rx, send_buf, pos32, R, quota, row_bytes, P, s);
}

int run_regroup_move(const void *node_rx, int64_t P, int64_t row_bytes, int epr, int64_t capacity, void *permuted,
                     const void *ws, size_t ws_bytes, hipStream_t s) {
    if (P < 0 || epr <= 0 || epr > kMaxBuckets || row_bytes < 0 || P >= (int64_t)1 << 31 ||
        (capacity >= 0 && (int64_t)epr * capacity >= (int64_t)1 << 31))
        return TERRACE_EINVAL;
    const int64_t places = capacity >= 0 ? (int64_t)epr * capacity : P;
    if (places == 0 || row_bytes == 0) return TERRACE_OK;
    if (!permuted) return TERRACE_EINVAL;
    if (P == 0) {       // all padding
        fill_zero_kernel<<<1024, kBlock, 0, s>>>((uint8_t *)permuted, places * row_geom(row_bytes).pitch);
        return check_launch();
    }
    if (!node_rx || !ws) return TERRACE_EINVAL;
    if (ws_bytes < regroup_workspace(P, epr, capacity)) return TERRACE_ENOSPC;
    const int32_t *order32 = (const int32_t *)((const char *)ws + units_table_bytes(make_units(P, epr)));
    const int32_t *gidx = (const int32_t *)((const char *)order32 + align_up((size_t)P * sizeof(int32_t), 256));
    return launch_gather_rows<int32_t>(node_rx, permuted, capacity >= 0 ? gidx : order32, places, row_bytes, P, s);
}

}  // namespace terrace
