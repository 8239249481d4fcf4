// Send side (dispatch index build + Hop-A wire planes) with one lane per token.
//
// Applies when a node set fits one 64-bit mask (n_nodes <= 64) and k <= 16, which covers every
// benchmark geometry.  A lane loads its token's k expert ids once, derives the set of nodes the
// token touches, and the wave ranks (token, node) pairs node by node with ballots:
//     row(n, t) = start[n] + (tokens of earlier units on n) + (lower lanes of this chunk on n)
// which is the (node ascending, token ascending) order of terrace/ta2a.py:131-137,228-230.
// The same lane then writes everything the token owns: its M rows' u_src / u_node, the
// ascending slot ids and co-indexed gates of each row (terrace/ta2a_fwd.py:232-248), `inverse`
// (terrace/ta2a.py:251-253) and the combine's per-token tables.
//
// Malformed routings are contained, never trusted: only a token's lowest M nodes get rows (so
// rows stay below T*M), a run's elements beyond the quota are skipped, missing cells and rows
// nobody claimed are zero-filled, and the exact fan-out / quota census goes to the status words.
#include "sort.hpp"

namespace terrace {

// 64 tokens per wave while that keeps the count table small, 256 beyond a quarter million tokens:
// the work per token is latency-bound, so more, shorter waves finish sooner.
static int token_chunks(int64_t T) { return T <= ((int64_t)1 << 18) ? 1 : 4; }

bool k2_token_path_applies(int k, int n_nodes) { return k <= 16 && n_nodes <= 64; }

static Units token_units(int64_t T, int n_nodes) {
    Units u;
    u.n_items = T;
    u.n_buckets = n_nodes;
    u.chunks = token_chunks(T);
    u.n_units = (int)((T + 64 * u.chunks - 1) / (64 * u.chunks));
    if (u.n_units < 1) u.n_units = 1;
    return u;
}

const int32_t *k2_token_positions(const void *ws, int64_t T, int n_nodes) {
    return (const int32_t *)((const char *)ws + units_table_bytes(token_units(T, n_nodes)));
}

size_t k2_token_workspace(int64_t T, int n_nodes, int groups_m) {
    return units_table_bytes(token_units(T, n_nodes)) + align_up((size_t)T * groups_m * sizeof(int32_t), 256);
}

template <int KMAX>
struct TokenRow {
    int e[KMAX];        // expert id, -1 when padding or out of range
    int nd[KMAX];       // its node, -1 likewise
    uint64_t all;       // every node the token touches
    uint64_t occ;       // the lowest M of them: the ones that get a send row
    int fault;
    __device__ __forceinline__ void load(const int64_t *row, int k, int slots, int n_experts, int M) {
        // the k ids first, as unconditional loads with nothing between them that waits on memory
        int64_t v[KMAX];
#pragma unroll
        for (int j = 0; j < KMAX; ++j) v[j] = row[j < k ? j : 0];
        fault = 0;
        all = 0;
#pragma unroll
        for (int j = 0; j < KMAX; ++j) {
            const bool ok = j < k && v[j] >= 0 && v[j] < n_experts;
            e[j] = ok ? (int)v[j] : -1;
            nd[j] = ok ? (int)v[j] / slots : -1;
            if (ok) all |= 1ull << nd[j];
            if (j < k && !ok) fault |= TERRACE_FAULT_ID_RANGE;
        }
        uint64_t rest = all;
        occ = 0;
        for (int m = 0; m < M && rest; ++m) {
            const uint64_t bit = rest & (~rest + 1);
            occ |= bit;
            rest ^= bit;
        }
    }
};

template <int KMAX, int kTokChunks>
__global__ __launch_bounds__(kBlock) void k2_count_kernel(const int64_t *__restrict__ expert_idx, int64_t T, int k,
                                                          int slots, int n_nodes, int n_experts, int M, int n_units,
                                                          int32_t *__restrict__ table) {
    const int lane = lane_id();
    const int unit = blockIdx.x * kWavesPerBlock + wave_in_block();
    if (unit >= n_units) return;
    uint64_t occ[kTokChunks];
#pragma unroll
    for (int c = 0; c < kTokChunks; ++c) {
        const int64_t t = ((int64_t)unit * kTokChunks + c) * kWave + lane;
        occ[c] = 0;
        if (t < T) {
            TokenRow<KMAX> row;
            row.load(expert_idx + t * k, k, slots, n_experts, M);
            occ[c] = row.occ;
        }
    }
    int mine = 0;                       // lane n counts node n
    for (int n = 0; n < n_nodes; ++n) {
        int cnt = 0;
#pragma unroll
        for (int c = 0; c < kTokChunks; ++c) cnt += __popcll(__ballot((occ[c] >> n) & 1ull));
        if (lane == n) mine = cnt;
    }
    if (lane < n_nodes) table[(int64_t)lane * n_units + unit] = mine;
}

template <typename G>
__device__ __forceinline__ void put_gate(void *plane, int64_t at, const void *gates, int64_t from) {
    ((G *)plane)[at] = ((const G *)gates)[from];
}

template <int KMAX, typename G, int kTokChunks>
__global__ __launch_bounds__(kBlock) void k2_place_kernel(
    const int64_t *__restrict__ expert_idx, const G *__restrict__ gates, int64_t T, int k, int slots, int n_nodes,
    int n_experts, int M, int quota, int n_units, const int32_t *__restrict__ table, int64_t *__restrict__ mask,
    G *__restrict__ gate_rows, int64_t *__restrict__ u_src, int64_t *__restrict__ u_node,
    int64_t *__restrict__ inverse, int64_t *__restrict__ pair_table, int64_t *__restrict__ sort_order,
    int64_t *__restrict__ token_rows, G *__restrict__ gate_sorted, int32_t *__restrict__ pos32,
    int32_t *__restrict__ status, int64_t mask_pitch, int64_t gate_pitch, int gate_pad) {
    __shared__ int census[kWavesPerBlock][3];
    const int lane = lane_id();
    const int unit = blockIdx.x * kWavesPerBlock + wave_in_block();
    const bool active = unit < n_units;             // an idle wave of the last workgroup still joins the census
    // mask / gate_rows may be [rows, quota] tables inside wider rows (a wire container): cell (r, i) of
    // each is at r*pitch + i, and the gate_pad elements after a row's gates are zeroed
    auto zero_row = [&](int64_t r) {
        for (int i = 0; i < quota; ++i) mask[r * mask_pitch + i] = 0;
        if (gates)
            for (int i = 0; i < quota + gate_pad; ++i) gate_rows[r * gate_pitch + i] = G(0);
    };
    int cur = (active && lane < n_nodes) ? table[(int64_t)lane * n_units + unit] : 0;      // lane n: cursor of node n
    int fault = 0, occupied = 0, off_quota = 0;
    for (int c = 0; c < (active ? kTokChunks : 0); ++c) {
        const int64_t t = ((int64_t)unit * kTokChunks + c) * kWave + lane;
        const bool live = t < T;
        TokenRow<KMAX> row;
        row.all = row.occ = 0;
        row.fault = 0;
        G gate_of[KMAX];                  // the token's k gates: their loads go out ahead of the id loads
#pragma unroll
        for (int j = 0; j < KMAX; ++j) gate_of[j] = (live && gates) ? gates[t * k + (j < k ? j : 0)] : G(0);
        if (live) row.load(expert_idx + t * k, k, slots, n_experts, M);
        // ---- rank this chunk's (token, node) pairs, node by node ----
        int rows[KMAX];
#pragma unroll
        for (int m = 0; m < KMAX; ++m) rows[m] = -1;
        for (int n = 0; n < n_nodes; ++n) {
            const bool has = (row.occ >> n) & 1ull;
            const uint64_t peers = __ballot(has);
            const int base = read_lane(cur, n);
            if (has) {
                const int r = base + __popcll(peers & lanes_below(lane));
                const int m = __popcll(row.occ & ((1ull << n) - 1ull));
#pragma unroll
                for (int mm = 0; mm < KMAX; ++mm)
                    if (mm == m) rows[mm] = r;
                u_src[r] = t;
                if (u_node) u_node[r] = n;
            }
            if (lane == n) cur += __popcll(peers);
        }
        if (!live) continue;
        // ---- census (terrace/ta2a.py:170-204): occupied pairs, pairs holding other than k/M ----
        const int n_all = __popcll(row.all);
        occupied += n_all;
        fault |= row.fault;
        int bad_pairs = 0;
#pragma unroll
        for (int j = 0; j < KMAX; ++j) {
            if (row.nd[j] < 0) continue;
            int same = 0, earlier = 0;
#pragma unroll
            for (int i = 0; i < KMAX; ++i) {
                const bool hit = row.nd[i] == row.nd[j];
                same += hit ? 1 : 0;
                earlier += (hit && i < j) ? 1 : 0;
            }
            if (earlier == 0 && same != quota) ++bad_pairs;
        }
        off_quota += bad_pairs;
        const bool clean = n_all == M && bad_pairs == 0 && row.fault == 0;
        if (n_all != M) fault |= TERRACE_FAULT_FANOUT;
        if (bad_pairs) fault |= TERRACE_FAULT_QUOTA;
        // ---- the token's rows ----
#pragma unroll
        for (int m = 0; m < KMAX; ++m) {
            if (m < M) {
                pos32[t * M + m] = rows[m];
                if (token_rows) token_rows[t * M + m] = rows[m];
            }
        }
        if (!clean) {                   // start from a defined state: no pair, zero cells
            for (int j = 0; j < k; ++j) {
                if (pair_table) pair_table[t * k + j] = -1;
                if (sort_order) sort_order[t * k + j] = 0;
                if (inverse) inverse[t * k + j] = -1;
                if (gate_sorted) gate_sorted[t * k + j] = G(0);
            }
#pragma unroll
            for (int m = 0; m < KMAX; ++m)
                if (m < M && rows[m] >= 0) zero_row(rows[m]);
        }
        // ---- the token's experts ----
#pragma unroll
        for (int j = 0; j < KMAX; ++j) {
            const int ej = row.e[j], nj = row.nd[j];
            if (nj < 0) continue;
            int rank = 0, within = 0;
#pragma unroll
            for (int i = 0; i < KMAX; ++i) {
                const bool lower = row.e[i] >= 0 && row.e[i] < ej;
                rank += lower ? 1 : 0;
                within += (lower && row.nd[i] == nj) ? 1 : 0;
            }
            if (!((row.occ >> nj) & 1ull) || within >= quota) continue;      // no row, or past the quota
            const int m = __popcll(row.occ & ((1ull << nj) - 1ull));
            int r = -1;
#pragma unroll
            for (int mm = 0; mm < KMAX; ++mm)
                if (mm == m) r = rows[mm];
            const int64_t cell = (int64_t)r * quota + within;
            mask[(int64_t)r * mask_pitch + within] = ej - nj * slots;
            if (gates) {
                gate_rows[(int64_t)r * gate_pitch + within] = gate_of[j];
                if (within == 0)
                    for (int z = 0; z < gate_pad; ++z) gate_rows[(int64_t)r * gate_pitch + quota + z] = G(0);
            }
            if (inverse) inverse[t * k + j] = r;
            if (pair_table) pair_table[t * k + rank] = cell;
            if (sort_order) sort_order[t * k + rank] = j;
            if (gates && gate_sorted) gate_sorted[t * k + rank] = gate_of[j];
        }
    }
    // rows nobody claimed (possible only under a fan-out fault): zero them
    if (active && unit == 0) {
        const int64_t n_cells = (int64_t)n_units * n_nodes;
        const int64_t used = table[n_cells + n_nodes], S = T * M;
        for (int64_t r = used + lane; r < S; r += kWave) {
            u_src[r] = 0;
            if (u_node) u_node[r] = 0;
            zero_row(r);
        }
    }
    // census: one atomic per workgroup and word.  Every wave of the grid adding to the same words one after
    // the other was a measurable part of this kernel (about 20 ns per wave, 1024 waves at 65536 tokens).
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        fault |= __shfl_xor(fault, d, kWave);
        occupied += __shfl_xor(occupied, d, kWave);
        off_quota += __shfl_xor(off_quota, d, kWave);
    }
    if (lane == 0) {
        census[wave_in_block()][0] = fault;
        census[wave_in_block()][1] = occupied;
        census[wave_in_block()][2] = off_quota;
    }
    __syncthreads();
    if (threadIdx.x == 0 && status) {
        int f = 0, o = 0, q = 0;
        for (int w = 0; w < kWavesPerBlock; ++w) {
            f |= census[w][0];
            o += census[w][1];
            q += census[w][2];
        }
        if (f) atomicOr(&status[0], f);
        if (o) atomicAdd(&status[1], o);
        if (q) atomicAdd(&status[2], q);
    }
}

template <int KMAX, typename G>
static void launch_place(const int64_t *expert_idx, const void *gates, int64_t T, int k, int slots, int n_nodes,
                         int n_experts, int M, const Units &u, const int32_t *table, int64_t *mask, void *gate_rows,
                         int64_t *u_src, int64_t *u_node, int64_t *inverse, int64_t *pair_table,
                         int64_t *sort_order, int64_t *token_rows, void *gate_sorted, int32_t *pos32,
                         int32_t *status, int64_t mask_pitch, int64_t gate_pitch, int gate_pad, hipStream_t s) {
    const int blocks = (u.n_units + kWavesPerBlock - 1) / kWavesPerBlock;
    if (u.chunks == 1)
        k2_place_kernel<KMAX, G, 1><<<blocks, kBlock, 0, s>>>(
            expert_idx, (const G *)gates, T, k, slots, n_nodes, n_experts, M, k / M, u.n_units, table, mask,
            (G *)gate_rows, u_src, u_node, inverse, pair_table, sort_order, token_rows, (G *)gate_sorted, pos32, status,
            mask_pitch, gate_pitch, gate_pad);
    else
        k2_place_kernel<KMAX, G, 4><<<blocks, kBlock, 0, s>>>(
            expert_idx, (const G *)gates, T, k, slots, n_nodes, n_experts, M, k / M, u.n_units, table, mask,
            (G *)gate_rows, u_src, u_node, inverse, pair_table, sort_order, token_rows, (G *)gate_sorted, pos32, status,
            mask_pitch, gate_pitch, gate_pad);
}

int run_k2_token(const void *hidden, const int64_t *expert_idx, const void *gates, int64_t T, int64_t row_bytes,
                 int gate_bytes, int k, int slots, int n_nodes, int n_experts, int groups_m, void *payload,
                 int64_t *mask, void *gate_rows, int64_t *u_src, int64_t *node_counts, int64_t *u_node,
                 int64_t *inverse, int64_t *node_offsets, int64_t *pair_table, int64_t *sort_order,
                 int64_t *token_rows, void *gate_sorted, int32_t *status, void *ws, int64_t mask_pitch,
                 int64_t gate_pitch, int gate_pad, hipStream_t s) {
    const Units u = token_units(T, n_nodes);
    int32_t *table = (int32_t *)ws;
    int32_t *pos32 = (int32_t *)((char *)ws + units_table_bytes(u));
    const int blocks = (u.n_units + kWavesPerBlock - 1) / kWavesPerBlock;
#define TERRACE_COUNT(KM, CH) \
    k2_count_kernel<KM, CH><<<blocks, kBlock, 0, s>>>(expert_idx, T, k, slots, n_nodes, n_experts, groups_m, u.n_units, table)
    if (k <= 8) {
        if (u.chunks == 1) TERRACE_COUNT(8, 1);
        else TERRACE_COUNT(8, 4);
    } else {
        if (u.chunks == 1) TERRACE_COUNT(16, 1);
        else TERRACE_COUNT(16, 4);
    }
#undef TERRACE_COUNT
    launch_scan(u, table, node_counts, nullptr, node_offsets, status, s);
#define TERRACE_PLACE(KM, G)                                                                                       \
    launch_place<KM, G>(expert_idx, gates, T, k, slots, n_nodes, n_experts, groups_m, u, table, mask, gate_rows,   \
                        u_src, u_node, inverse, pair_table, sort_order, token_rows, gate_sorted, pos32, status,      \
                        mask_pitch, gate_pitch, gate_pad, s)
    if (k <= 8) {
        if (gate_bytes == 4) TERRACE_PLACE(8, uint32_t);
        else TERRACE_PLACE(8, uint16_t);
    } else {
        if (gate_bytes == 4) TERRACE_PLACE(16, uint32_t);
        else TERRACE_PLACE(16, uint16_t);
    }
#undef TERRACE_PLACE
    int rc = check_launch();
    if (rc != TERRACE_OK || !hidden) return rc;
    return launch_scatter_rows<int32_t>(hidden, payload, pos32, T, groups_m, row_bytes, T * groups_m, s);
}

}  // namespace terrace
