// Send side (dispatch index build + Hop-A wire planes) when a token's node set fits one 64-bit word.
//
// Applies when n_nodes <= 64 and k <= 16, which covers every benchmark geometry.  Two launches (one, the place
// kernel counting for itself, when all tokens are one unit):
//
//   k2_count_kernel   one lane per token derives the set of nodes the token touches; a wave (64 tokens, one
//                     "unit") counts its tokens per node with ballots, the workgroup leaves each unit's prefix
//                     inside the workgroup and the workgroup's totals.
//   k2_place_kernel   one workgroup per unit with LPT lanes per token, lane (token, column j) holding expert
//                     j of the token: every [T, k] plane is then read and written with consecutive lanes on
//                     consecutive words.  The workgroup adds up the totals before it (no scan launch), ranks
//                     its (token, node) pairs
//                         row(n, t) = start[n] + (tokens of earlier units on n) + (earlier tokens of the unit on n)
//                     which is the (node ascending, token ascending) order of terrace/ta2a.py:131-137,228-230,
//                     lane (token, m) writes the token's m-th row (u_src / u_node / the mover's position) and lane
//                     (token, j) what expert j owns: its ascending slot id and gate in the row
//                     (terrace/ta2a_fwd.py:232-248), `inverse` (terrace/ta2a.py:251-253) and the combine's
//                     per-token tables.
//
// A token's experts are ranked by (id, column): equal ids keep their column order, so ranks are always a
// permutation and a routing with a repeated id fills every cell it owns.  Malformed routings are contained, never
// trusted: only a token's lowest M nodes get rows (so rows stay below T*M), a run's elements beyond the quota are
// skipped, the cells of such a token start from defaults (no pair, zero slot, zero gate), rows nobody claimed are
// zero-filled, and the exact fan-out / quota census goes to the status words.
#include "sort.hpp"

namespace terrace {

constexpr int kTokUnit = kWave;          // tokens per unit

// Lanes per token of the two kernels: the smallest of 4, 8, 16 that holds the token's k ids.
static int lanes_per_token(int k) { return k <= 4 ? 4 : (k <= 8 ? 8 : 16); }

// One count workgroup is kSortBlockMax lanes = 1024 / LPT tokens = 16 / LPT units.
static Units token_units(int64_t T, int k, int n_nodes) {
    Units u;
    u.n_items = T;
    u.n_buckets = n_nodes;
    u.chunks = 1;
    u.n_units = (int)((T + kTokUnit - 1) / kTokUnit);
    if (u.n_units < 1) u.n_units = 1;
    u.wpb = 16 / lanes_per_token(k);
    u.n_blocks = (u.n_units + u.wpb - 1) / u.wpb;
    u.direct = n_nodes <= kDirectMaxBuckets && (int64_t)n_nodes * u.n_blocks <= kDirectMaxWords;
    // up to 64 tokens are one place workgroup, which then counts for itself: no count launch (about 4.5 us of a
    // decode-sized step)
    u.solo = u.direct && u.n_units == 1 && n_nodes <= kWave;
    return u;
}

bool k2_token_path_applies(int64_t T, int k, int n_nodes) {
    return k <= 16 && n_nodes <= 64 && token_units(T, k, n_nodes).direct;
}

const int32_t *k2_token_positions(const void *ws, int64_t T, int k, int n_nodes) {
    return (const int32_t *)((const char *)ws + units_table_bytes(token_units(T, k, n_nodes)));
}

size_t k2_token_workspace(int64_t T, int k, int n_nodes, int groups_m) {
    return units_table_bytes(token_units(T, k, n_nodes)) + align_up((size_t)T * groups_m * sizeof(int32_t), 256);
}

// The lowest M set bits of a node set: the nodes that get a send row.
__device__ __forceinline__ uint64_t lowest_bits(uint64_t all, int M) {
    uint64_t rest = all, occ = 0;
    for (int m = 0; m < M && rest; ++m) {
        const uint64_t bit = rest & (~rest + 1);
        occ |= bit;
        rest ^= bit;
    }
    return occ;
}

__device__ __forceinline__ uint64_t read_lane64(uint64_t v, int src_lane) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, src_lane);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), src_lane);
    return ((uint64_t)hi << 32) | lo;
}

// What lane (token, column) knows once the token's ids are shared inside its group of LPT lanes.
template <int LPT>
struct TokenView {
    int e, nd;                  // the lane's expert and node, -1 when the column is padding or out of range
    bool ok;
    uint64_t all, occ;          // every node the token touches; the lowest M of them (identical in the group)
    int rank, within;           // of the lane's expert among the token's by (id, column); among those of its node
    bool first_of_node, bad_pair;
    __device__ __forceinline__ void build(int64_t v, bool has_col, int col, int tok_lane, int slots, int n_experts,
                                          int M, int quota) {
        ok = has_col && v >= 0 && v < n_experts;
        e = ok ? (int)v : -1;
        nd = ok ? e / slots : -1;
        int E[LPT], N[LPT];
#pragma unroll
        for (int i = 0; i < LPT; ++i) {
            E[i] = __shfl(e, tok_lane + i, kWave);
            N[i] = __shfl(nd, tok_lane + i, kWave);
        }
        all = 0;
#pragma unroll
        for (int i = 0; i < LPT; ++i)
            if (N[i] >= 0) all |= 1ull << N[i];
        occ = lowest_bits(all, M);
        rank = within = 0;
        int same = 0, earlier = 0;
#pragma unroll
        for (int i = 0; i < LPT; ++i) {
            const bool lower = E[i] >= 0 && (E[i] < e || (E[i] == e && i < col));
            const bool hit = N[i] == nd;
            rank += lower ? 1 : 0;
            within += (lower && hit) ? 1 : 0;
            same += hit ? 1 : 0;
            earlier += (hit && i < col) ? 1 : 0;
        }
        first_of_node = ok && earlier == 0;
        bad_pair = first_of_node && same != quota;
    }
};

// Count: 1024 lanes per workgroup, LPT lanes per token (lane = token * LPT + column, so the ids are read with
// consecutive lanes on consecutive words), 16 / LPT units per workgroup.  Also takes the census the guard of
// terrace/ta2a.py:170-204 reads -- occupied (token, node) pairs, pairs holding other than k/M experts, the fault
// bits -- and leaves it per workgroup beside the totals: the place kernel's first workgroup adds the few entries up
// and stores the status block, so no workgroup ever waits on an atomic to a word every other workgroup adds to.
template <int LPT>
__global__ __launch_bounds__(kSortBlockMax) void k2_count_kernel(const int64_t *__restrict__ expert_idx, int64_t T,
                                                                 int k, int slots, int n_experts, int M, int quota,
                                                                 Units u, int32_t *__restrict__ table) {
    constexpr int kTpw = kWave / LPT;               // tokens per wave
    constexpr int kWpu = LPT;                       // waves per unit
    __shared__ int32_t s_counts[16 / LPT * 64];     // [unit in block][node]
    __shared__ int32_t s_census[4];
    const int lane = lane_id(), w = wave_in_block();
    const int n_nodes = u.n_buckets;
    const int col = lane & (LPT - 1), tok_lane = lane & ~(LPT - 1);
    const int unit_in_block = w / kWpu;
    const int64_t t = ((int64_t)blockIdx.x * u.wpb + unit_in_block) * kTokUnit + (w % kWpu) * kTpw + lane / LPT;
    const bool live = t < T, has_col = live && col < k;
    const int64_t v = has_col ? expert_idx[t * k + col] : -1;
    for (int i = threadIdx.x; i < u.wpb * n_nodes; i += blockDim.x) s_counts[i] = 0;
    if (threadIdx.x < 4) s_census[threadIdx.x] = 0;
    __syncthreads();
    TokenView<LPT> tv;
    tv.build(v, has_col, col, tok_lane, slots, n_experts, M, quota);
    int wave_cnt = 0;                               // lane n: tokens of this wave on node n
#pragma unroll
    for (int i = 0; i < kTpw; ++i) wave_cnt += (int)((read_lane64(tv.occ, i * LPT) >> lane) & 1ull);
    if (lane < n_nodes && wave_cnt) atomicAdd(&s_counts[unit_in_block * n_nodes + lane], wave_cnt);
    int fault = (has_col && !tv.ok) ? TERRACE_FAULT_ID_RANGE : 0;
    if (live && col == 0 && __popcll(tv.all) != M) fault |= TERRACE_FAULT_FANOUT;
    if (tv.bad_pair) fault |= TERRACE_FAULT_QUOTA;
    const int occupied = __popcll(__ballot(tv.first_of_node)), off_quota = __popcll(__ballot(tv.bad_pair));
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) fault |= __shfl_xor(fault, d, kWave);
    if (lane == 0) {
        if (fault) atomicOr(&s_census[0], fault);
        if (occupied) atomicAdd(&s_census[1], occupied);
        if (off_quota) atomicAdd(&s_census[2], off_quota);
    }
    __syncthreads();
    direct_block_counts(u, table, (lds_i32 *)s_counts);
    if (threadIdx.x < 4) table[units_census_at(u) + 4 * (int64_t)blockIdx.x + threadIdx.x] = s_census[threadIdx.x];
}

// LPT lanes per token (k <= LPT), 64 tokens per workgroup: blockDim = 64 * LPT, thread = token_local * LPT + column.
template <int LPT, typename G>
__global__ __launch_bounds__(kWave *LPT) void k2_place_kernel(
    const int64_t *__restrict__ expert_idx, const G *__restrict__ gates, int64_t T, int k, int slots, int n_experts,
    int M, int quota, Units u, int32_t *__restrict__ table, int64_t *__restrict__ mask, G *__restrict__ gate_rows,
    int64_t *__restrict__ u_src, int64_t *__restrict__ u_node, int64_t *__restrict__ inverse,
    int64_t *__restrict__ pair_table, int64_t *__restrict__ sort_order, int64_t *__restrict__ token_rows,
    G *__restrict__ gate_sorted, int64_t *__restrict__ pair_src, int64_t *__restrict__ combine_table,
    int32_t *__restrict__ pos32, int64_t *__restrict__ node_counts, int64_t *__restrict__ node_offsets,
    int32_t *__restrict__ status, int64_t mask_pitch, int64_t gate_pitch, int gate_pad) {
    constexpr int kWaves = LPT;                     // waves per workgroup
    constexpr int kTpw = kWave / LPT;               // tokens per wave
    __shared__ int32_t s_tot[64], s_base[64], s_start[65], s_tab[64];
    __shared__ int32_t s_wcnt[kWaves][64];
    __shared__ int32_t s_dirty[kWaves];
    __shared__ int32_t s_census[kWaves][3];          // solo: each wave's fault bits, occupied pairs, pairs off the quota
    const int lane = lane_id(), w = wave_in_block();
    const int unit = blockIdx.x;
    const int n_nodes = u.n_buckets;
    const int col = lane & (LPT - 1);               // the lane's column j, and the row index m it owns
    const int tok_lane = lane & ~(LPT - 1);         // first lane of the token's group
    const int tw = lane / LPT;                      // token inside the wave
    const int64_t t = (int64_t)unit * kTokUnit + w * kTpw + tw;
    const bool live = t < T;
    const bool has_col = live && col < k;
    // ---- every global load of the kernel is issued here, before anything waits: the token's ids and gates (one
    // coalesced load each), this unit's prefixes inside its count workgroup, and (inside direct_block_base) the
    // workgroup totals ----
    const int64_t v = has_col ? expert_idx[t * k + col] : -1;
    G gate = G(0);
    if (has_col && gates) gate = gates[t * k + col];
    int tab = 0;
    if (!u.solo && threadIdx.x < n_nodes) tab = table[(int64_t)threadIdx.x * u.n_units + unit];
    // ---- cursors of this unit: start[n] + earlier workgroups (+ s_tab: earlier units of the count workgroup) ----
    const int me = unit / u.wpb;
    TableOut out;
    out.hist_i64 = node_counts;
    out.offsets_i64 = node_offsets;
    if (!u.solo) direct_block_base(u, table, me, unit == 0, (lds_i32 *)s_tot, (lds_i32 *)s_base, (lds_i32 *)s_start, out);
    // ---- the token's ids, shared inside the group; ranks by (id, column) ----
    TokenView<LPT> tv;
    tv.build(v, has_col, col, tok_lane, slots, n_experts, M, quota);
    const bool ok = tv.ok;
    const int e = tv.e, nd = tv.nd, rank = tv.rank, within = tv.within;
    const uint64_t occ = tv.occ;
    // a token is clean when it touches exactly M nodes, each with exactly `quota` in-range experts
    const uint64_t dirty_lanes = __ballot(tv.bad_pair || (has_col && !ok));
    const bool dirty_group = ((dirty_lanes >> tok_lane) & ((LPT == 64 ? 0 : (1ull << LPT)) - 1ull)) != 0;
    const bool clean = live && __popcll(tv.all) == M && !dirty_group;
    // a token that is not clean starts from a defined state: its per-column cells first, ordered before the
    // stores that fill cells by the barrier below
    if (has_col && !clean) {
        if (pair_table) pair_table[t * k + col] = -1;
        if (sort_order) sort_order[t * k + col] = 0;
        if (inverse) inverse[t * k + col] = -1;
        if (gates && gate_sorted) gate_sorted[t * k + col] = G(0);
        if (combine_table) combine_table[t * k + col] = -1;
    }
    // ---- tokens of this wave per node (lane n counts node n); the owner lanes count their earlier peers ----
    const bool owner = live && col < M;             // lane (token, m) owns the token's m-th send row
    int my_node = -1;
    {
        uint64_t rest = occ;
        for (int m = 0; m < col && rest; ++m) rest &= rest - 1;
        if (owner && rest) my_node = __builtin_ctzll(rest);
    }
    int wave_cnt = 0, peers_before = 0;
#pragma unroll
    for (int i = 0; i < kTpw; ++i) {
        const uint64_t occ_i = read_lane64(occ, i * LPT);
        wave_cnt += (int)((occ_i >> lane) & 1ull);
        if (my_node >= 0 && i < tw) peers_before += (int)((occ_i >> my_node) & 1ull);
    }
    if (lane < n_nodes) s_wcnt[w][lane] = wave_cnt;
    if (threadIdx.x < n_nodes) s_tab[threadIdx.x] = tab;
    // ---- does any token of the workgroup start from defaults?  (uniform across the workgroup after the barrier) ----
    const uint64_t any_dirty = __ballot(live && !clean);
    if (lane == 0) s_dirty[w] = any_dirty != 0;
    if (u.solo) {           // the census the count kernel takes otherwise (same definitions), one entry per wave
        int fault = (has_col && !ok) ? TERRACE_FAULT_ID_RANGE : 0;
        if (live && col == 0 && __popcll(tv.all) != M) fault |= TERRACE_FAULT_FANOUT;
        if (tv.bad_pair) fault |= TERRACE_FAULT_QUOTA;
        const int occupied = __popcll(__ballot(tv.first_of_node)), off_quota = __popcll(__ballot(tv.bad_pair));
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) fault |= __shfl_xor(fault, d, kWave);
        if (lane == 0) {
            s_census[w][0] = fault;
            s_census[w][1] = occupied;
            s_census[w][2] = off_quota;
        }
    }
    __syncthreads();
    if (u.solo) {
        // this workgroup holds every token: the per-node totals are its waves' counts, the cursors start at the
        // nodes' offsets, and wave 0 (lane n = node n) publishes what the count + base steps publish otherwise
        if (w == 0) {
            int tot = 0;
            if (lane < n_nodes)
                for (int x = 0; x < kWaves; ++x) tot += s_wcnt[x][lane];
            const int incl = wave_inclusive_scan(tot);
            if (lane < n_nodes) {
                s_start[lane] = incl - tot;
                s_base[lane] = incl - tot;
                table[units_start_at(u) + lane] = incl - tot;
                out.put(lane, tot, incl - tot);
            }
            if (lane == n_nodes - 1) {
                s_start[n_nodes] = incl;
                table[units_start_at(u) + n_nodes] = incl;
            }
        }
        __syncthreads();
    }
    bool dirty_block = false;
    for (int x = 0; x < kWaves; ++x) dirty_block = dirty_block || s_dirty[x];
    // ---- the status block: the count kernel's per-workgroup census, added up and stored by the first workgroup ----
    if (unit == 0 && w == 0 && status) {
        const int32_t *census = table + units_census_at(u);
        int f = 0, o = 0, q = 0;
        if (u.solo) {
            if (lane < kWaves) {
                f = s_census[lane][0];
                o = s_census[lane][1];
                q = s_census[lane][2];
            }
        } else {
            for (int b = lane; b < u.n_blocks; b += kWave) {
                f |= census[4 * b + 0];
                o += census[4 * b + 1];
                q += census[4 * b + 2];
            }
        }
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
            f |= __shfl_xor(f, d, kWave);
            o += __shfl_xor(o, d, kWave);
            q += __shfl_xor(q, d, kWave);
        }
        if (lane == 0) {
            status[0] = f;
            status[1] = o;
            status[2] = q;
            status[3] = 0;
        }
    }
    int r = -1;
    if (my_node >= 0) {
        r = s_base[my_node] + s_tab[my_node] + peers_before;
        for (int x = 0; x < w; ++x) r += s_wcnt[x][my_node];
        u_src[r] = t;
        if (u_node) u_node[r] = my_node;
        // the cells after the row's quota gates (wire containers), and for a token that is not clean all cells
        if (gates)
            for (int z = 0; z < gate_pad; ++z) gate_rows[(int64_t)r * gate_pitch + quota + z] = G(0);
        if (!clean)
            for (int i = 0; i < quota; ++i) {
                mask[(int64_t)r * mask_pitch + i] = 0;
                if (gates) gate_rows[(int64_t)r * gate_pitch + i] = G(0);
                if (pair_src) pair_src[(int64_t)r * quota + i] = -1;
            }
    }
    if (owner) {
        pos32[t * M + col] = r;
        if (token_rows) token_rows[t * M + col] = r;
    }
    // rows nobody claimed (possible only under a fan-out fault): zero them
    if (unit == 0) {
        const int64_t used = s_start[n_nodes], S = T * M;
        for (int64_t x = used + threadIdx.x; x < S; x += blockDim.x) {
            u_src[x] = 0;
            if (u_node) u_node[x] = 0;
            for (int i = 0; i < quota; ++i) {
                mask[x * mask_pitch + i] = 0;
                if (pair_src) pair_src[x * quota + i] = -1;
            }
            if (gates)
                for (int i = 0; i < quota + gate_pad; ++i) gate_rows[x * gate_pitch + i] = G(0);
        }
    }
    // the defaults above must be in memory before any cell is filled: a barrier (which waits for the stores), but
    // only in a workgroup that wrote defaults -- well-formed routings never pay for it
    if (dirty_block) __syncthreads();
    // ---- what the lane's expert owns ----
    const bool placed = ok && ((occ >> nd) & 1ull) && within < quota;
    const int m_of = ok ? __popcll(occ & ((1ull << nd) - 1ull)) : 0;
    const int row = __shfl(r, tok_lane + m_of, kWave);
    if (placed && row >= 0) {
        mask[(int64_t)row * mask_pitch + within] = e - nd * slots;
        if (gates) gate_rows[(int64_t)row * gate_pitch + within] = gate;
        if (inverse) inverse[t * k + col] = row;
        if (pair_table) pair_table[t * k + rank] = (int64_t)row * quota + within;
        if (pair_src) pair_src[(int64_t)row * quota + within] = t * k + rank;
        if (sort_order) sort_order[t * k + rank] = col;
        if (gates && gate_sorted) gate_sorted[t * k + rank] = gate;
    }
}

template <int LPT, typename G>
static void launch_place(const int64_t *expert_idx, const void *gates, int64_t T, int k, int slots, int n_experts,
                         int M, const Units &u, int32_t *table, int64_t *mask, void *gate_rows, int64_t *u_src,
                         int64_t *u_node, int64_t *inverse, int64_t *pair_table, int64_t *sort_order,
                         int64_t *token_rows, void *gate_sorted, int64_t *pair_src, int64_t *combine_table,
                         int32_t *pos32, int64_t *node_counts, int64_t *node_offsets, int32_t *status,
                         int64_t mask_pitch, int64_t gate_pitch, int gate_pad, hipStream_t s) {
    k2_place_kernel<LPT, G><<<u.n_units, kWave * LPT, 0, s>>>(
        expert_idx, (const G *)gates, T, k, slots, n_experts, M, k / M, u, table, mask, (G *)gate_rows, u_src, u_node,
        inverse, pair_table, sort_order, token_rows, (G *)gate_sorted, pair_src, combine_table, pos32, node_counts,
        node_offsets, status, mask_pitch, gate_pitch, gate_pad);
}

int run_k2_token(const void *hidden, const int64_t *expert_idx, const void *gates, int64_t T, int64_t row_bytes,
                 int gate_bytes, int k, int slots, int n_nodes, int n_experts, int groups_m, void *payload,
                 int64_t *mask, void *gate_rows, int64_t *u_src, int64_t *node_counts, int64_t *u_node,
                 int64_t *inverse, int64_t *node_offsets, int64_t *pair_table, int64_t *sort_order,
                 int64_t *token_rows, void *gate_sorted, int64_t *pair_src, int64_t *combine_table, int32_t *status,
                 void *ws, int64_t mask_pitch, int64_t gate_pitch, int gate_pad, hipStream_t s) {
    const Units u = token_units(T, k, n_nodes);
    int32_t *table = (int32_t *)ws;
    int32_t *pos32 = (int32_t *)((char *)ws + units_table_bytes(u));
#define TERRACE_COUNT(L)                                                                                          \
    k2_count_kernel<L><<<u.n_blocks, kSortBlockMax, 0, s>>>(expert_idx, T, k, slots, n_experts, groups_m, k / groups_m, \
                                                           u, table)
    if (!u.solo) {
        if (k <= 4) TERRACE_COUNT(4);
        else if (k <= 8) TERRACE_COUNT(8);
        else TERRACE_COUNT(16);
    }
#undef TERRACE_COUNT
#define TERRACE_PLACE(L, G)                                                                                        \
    launch_place<L, G>(expert_idx, gates, T, k, slots, n_experts, groups_m, u, table, mask, gate_rows, u_src, u_node, \
                       inverse, pair_table, sort_order, token_rows, gate_sorted, pair_src, combine_table, pos32,    \
                       node_counts, node_offsets, status, mask_pitch, gate_pitch, gate_pad, s)
    if (k <= 4) {
        if (gate_bytes == 4) TERRACE_PLACE(4, uint32_t);
        else TERRACE_PLACE(4, uint16_t);
    } else if (k <= 8) {
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
