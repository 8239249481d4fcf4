// The general (non-quota) branch of the dispatch index build, and the seam's entry helper.
//
//   plan_place_kernel       plan_ta2a with a data-dependent fan-out (terrace/ta2a.py:205-253):
//                           one send row per occupied (node, token) pair, whatever their number
//   build_mask_kernel       build_expansion (terrace/ta2a_fwd.py:348-442): bit j of row r is set iff
//                           node-local slot j wants the row
//   scatter_elems_kernel    the sparse gate plane gate_rows[inverse, slot] = gates (ta2a_fwd.py:499-500)
//   expand_quota_kernel     _expand_arrival with a quota (ta2a_fwd.py:120-174): a row's `quota` lowest
//                           set bits ascending, then (if it has fewer) its unset columns ascending
//   expand_count/fill       _expand_arrival without one: every set bit, row-major, columns ascending
//   map_count/map_topk      routing_map_to_topk (terrace/ta2a_dispatch.py:224-260): a dense boolean
//                           [T,E] map to ascending expert ids and their probabilities
// None of this is bandwidth-critical; the kernels are written for clarity.
#include "sort.hpp"

namespace terrace {

// ---- general plan --------------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void plan_count_kernel(const int64_t *__restrict__ expert_idx, int64_t T, int k,
                                                            int slots, int n_nodes, int n_experts, int n_units,
                                                            int32_t *__restrict__ table) {
    const int lane = lane_id();
    const int unit = blockIdx.x * kWavesPerBlock + wave_in_block();
    if (unit >= n_units) return;
    const int64_t t = (int64_t)unit * kWave + lane;
    uint64_t occ = 0;
    if (t < T) {
        for (int j = 0; j < k; ++j) {
            const int64_t e = expert_idx[t * k + j];
            if (e >= 0 && e < n_experts) occ |= 1ull << (int)(e / slots);
        }
    }
    int mine = 0;
    for (int n = 0; n < n_nodes; ++n) {
        const int cnt = __popcll(__ballot((occ >> n) & 1ull));
        if (lane == n) mine = cnt;
    }
    if (lane < n_nodes) table[(int64_t)lane * n_units + unit] = mine;
}

__global__ __launch_bounds__(kBlock) void plan_place_kernel(const int64_t *__restrict__ expert_idx, int64_t T, int k,
                                                            int slots, int n_nodes, int n_experts, int n_units,
                                                            const int32_t *__restrict__ table,
                                                            int64_t *__restrict__ u_src, int64_t *__restrict__ u_node,
                                                            int64_t *__restrict__ inverse,
                                                            int32_t *__restrict__ status) {
    const int lane = lane_id();
    const int unit = blockIdx.x * kWavesPerBlock + wave_in_block();
    if (unit >= n_units) return;
    int cur = lane < n_nodes ? table[(int64_t)lane * n_units + unit] : 0;
    const int64_t t = (int64_t)unit * kWave + lane;
    uint64_t occ = 0;
    bool bad = false;
    if (t < T) {
        for (int j = 0; j < k; ++j) {
            const int64_t e = expert_idx[t * k + j];
            if (e >= 0 && e < n_experts) occ |= 1ull << (int)(e / slots);
            else bad = true;
        }
    }
    for (int n = 0; n < n_nodes; ++n) {
        const bool has = (occ >> n) & 1ull;
        const uint64_t peers = __ballot(has);
        const int base = read_lane(cur, n);
        if (has) {
            const int r = base + __popcll(peers & lanes_below(lane));
            u_src[r] = t;
            u_node[r] = n;
            for (int j = 0; j < k; ++j) {
                const int64_t e = expert_idx[t * k + j];
                if (e >= 0 && e < n_experts && (int)(e / slots) == n) inverse[t * k + j] = r;
            }
        }
        if (lane == n) cur += __popcll(peers);
    }
    if (t < T && bad) {
        for (int j = 0; j < k; ++j) {
            const int64_t e = expert_idx[t * k + j];
            if (e < 0 || e >= n_experts) inverse[t * k + j] = -1;
        }
        if (status) atomicOr(&status[0], TERRACE_FAULT_ID_RANGE);
    }
}

size_t plan_wide_workspace(int64_t T, int k, int n_nodes);
int run_plan_wide(const int64_t *expert_idx, int64_t T, int k, int slots, int n_nodes, int n_experts, int64_t *u_src,
                  int64_t *u_node, int64_t *counts, int64_t *inverse, int32_t *status, void *ws, size_t ws_bytes,
                  hipStream_t s);

// Up to 64 nodes a token's node set is one mask word and a lane handles a token; beyond, the (token, column)
// item sort of sort.hip takes over.
size_t plan_general_workspace(int64_t T, int k, int n_nodes) {
    if (n_nodes > 64) return plan_wide_workspace(T, k, n_nodes);
    Units u{T, 1, (int)((T + 63) / 64 > 0 ? (T + 63) / 64 : 1), n_nodes};
    return units_table_bytes(u);
}

int run_plan_general(const int64_t *expert_idx, int64_t T, int k, int world, int n_experts, int rpn, int64_t *u_src,
                     int64_t *u_node, int64_t *counts, int64_t *inverse, int32_t *status, void *ws, size_t ws_bytes,
                     hipStream_t s) {
    if (T < 0 || k <= 0 || world <= 0 || rpn <= 0 || n_experts <= 0 || world % rpn || n_experts % world || !counts)
        return TERRACE_EINVAL;
    const int n_nodes = world / rpn, slots = (n_experts / world) * rpn;
    if (T * (int64_t)k >= (int64_t)1 << 31) return TERRACE_EINVAL;
    if (T > 0 && (!expert_idx || !u_src || !u_node || !inverse)) return TERRACE_EINVAL;
    if (n_nodes > 64)
        return run_plan_wide(expert_idx, T, k, slots, n_nodes, n_experts, u_src, u_node, counts, inverse, status, ws,
                             ws_bytes, s);
    Units u{T, 1, (int)((T + 63) / 64 > 0 ? (T + 63) / 64 : 1), n_nodes};
    if (!ws || ws_bytes < units_table_bytes(u)) return TERRACE_ENOSPC;
    int32_t *table = (int32_t *)ws;
    const int blocks = (u.n_units + kWavesPerBlock - 1) / kWavesPerBlock;
    if (T > 0 && (!expert_idx || !u_src || !u_node || !inverse)) return TERRACE_EINVAL;
    plan_count_kernel<<<blocks, kBlock, 0, s>>>(expert_idx, T, k, slots, n_nodes, n_experts, u.n_units, table);
    TableOut out;
    out.hist_i64 = counts;
    launch_scan(u, table, out, status, s);
    plan_place_kernel<<<blocks, kBlock, 0, s>>>(expert_idx, T, k, slots, n_nodes, n_experts, u.n_units, table, u_src,
                                                u_node, inverse, status);
    return check_launch();
}

// ---- bitmask planes -------------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void build_mask_kernel(const int64_t *__restrict__ expert_idx,
                                                            const int64_t *__restrict__ inverse, int64_t n, int slots,
                                                            int64_t n_rows, unsigned long long *__restrict__ mask,
                                                            int32_t *__restrict__ status) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int64_t r = inverse[i], e = expert_idx[i];
    if (r < 0 || r >= n_rows || e < 0) {
        if (status) atomicOr(&status[0], TERRACE_FAULT_ID_RANGE);
        return;
    }
    atomicOr(&mask[r], 1ull << (int)(e % slots));       // rows are unique per (token, node): no bit is set twice
}

template <typename G>
__global__ __launch_bounds__(kBlock) void scatter_elems_kernel(const G *__restrict__ vals,
                                                               const int64_t *__restrict__ rows,
                                                               const int64_t *__restrict__ cols, int col_mod,
                                                               int64_t n, int64_t n_rows, int width,
                                                               G *__restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int64_t r = rows[i];
    int64_t c = cols[i];
    if (col_mod > 0 && c >= 0) c %= col_mod;
    if (r < 0 || r >= n_rows || c < 0 || c >= width) return;
    out[r * width + c] = vals[i];
}

__global__ __launch_bounds__(kBlock) void expand_quota_kernel(const int64_t *__restrict__ rmask, int64_t R, int slots,
                                                              int quota, int64_t *__restrict__ r_idx,
                                                              int64_t *__restrict__ slot_idx) {
    const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (r >= R) return;
    const uint64_t all = slots >= 64 ? ~0ull : ((1ull << slots) - 1ull);
    uint64_t set = (uint64_t)rmask[r] & all, unset = ~(uint64_t)rmask[r] & all;
    for (int i = 0; i < quota; ++i) {
        uint64_t &pool = set ? set : unset;
        const int col = pool ? __builtin_ctzll(pool) : 0;
        pool &= pool - 1;
        r_idx[r * quota + i] = r;
        slot_idx[r * quota + i] = col;
    }
}

__global__ __launch_bounds__(kBlock) void expand_count_kernel(const int64_t *__restrict__ rmask, int64_t R, int slots,
                                                              int32_t *__restrict__ cnt) {
    const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (r >= R) return;
    const uint64_t all = slots >= 64 ? ~0ull : ((1ull << slots) - 1ull);
    cnt[r] = __popcll((uint64_t)rmask[r] & all);
}

__global__ __launch_bounds__(kBlock) void expand_fill_kernel(const int64_t *__restrict__ rmask, int64_t R, int slots,
                                                             const int32_t *__restrict__ offset,
                                                             int64_t *__restrict__ r_idx,
                                                             int64_t *__restrict__ slot_idx) {
    const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (r >= R) return;
    const uint64_t all = slots >= 64 ? ~0ull : ((1ull << slots) - 1ull);
    uint64_t set = (uint64_t)rmask[r] & all;
    int64_t at = offset[r];
    while (set) {
        r_idx[at] = r;
        slot_idx[at] = __builtin_ctzll(set);
        set &= set - 1;
        ++at;
    }
}

__global__ void set_i64_kernel(int64_t *p, int64_t v) { *p = v; }

int run_build_mask(const int64_t *expert_idx, const int64_t *inverse, int64_t n, int slots, int64_t n_rows,
                   int64_t *mask, int32_t *status, hipStream_t s) {
    if (n < 0 || slots <= 0 || slots > 63 || n_rows < 0) return TERRACE_EINVAL;
    if (n == 0) return TERRACE_OK;
    if (!expert_idx || !inverse || !mask) return TERRACE_EINVAL;
    build_mask_kernel<<<(unsigned)((n + kBlock - 1) / kBlock), kBlock, 0, s>>>(expert_idx, inverse, n, slots, n_rows,
                                                                             (unsigned long long *)mask, status);
    return check_launch();
}

int run_scatter_elems(const void *vals, int elem_bytes, const int64_t *rows, const int64_t *cols, int col_mod,
                      int64_t n, int64_t n_rows, int width, void *out, hipStream_t s) {
    if (n < 0 || n_rows < 0 || width <= 0 || (elem_bytes != 2 && elem_bytes != 4)) return TERRACE_EINVAL;
    if (n == 0) return TERRACE_OK;
    if (!vals || !rows || !cols || !out) return TERRACE_EINVAL;
    const unsigned grid = (unsigned)((n + kBlock - 1) / kBlock);
    if (elem_bytes == 4)
        scatter_elems_kernel<uint32_t><<<grid, kBlock, 0, s>>>((const uint32_t *)vals, rows, cols, col_mod, n, n_rows, width, (uint32_t *)out);
    else
        scatter_elems_kernel<uint16_t><<<grid, kBlock, 0, s>>>((const uint16_t *)vals, rows, cols, col_mod, n, n_rows, width, (uint16_t *)out);
    return check_launch();
}

int run_expand_quota(const int64_t *rmask, int64_t R, int slots, int quota, int64_t *r_idx, int64_t *slot_idx,
                     hipStream_t s) {
    if (R < 0 || slots <= 0 || slots > 64 || quota <= 0 || quota > slots) return TERRACE_EINVAL;
    if (R == 0) return TERRACE_OK;
    if (!rmask || !r_idx || !slot_idx) return TERRACE_EINVAL;
    expand_quota_kernel<<<(unsigned)((R + kBlock - 1) / kBlock), kBlock, 0, s>>>(rmask, R, slots, quota, r_idx, slot_idx);
    return check_launch();
}

size_t expand_workspace(int64_t R) {
    Units u{R, 1, (int)(R > 0 ? R : 1), 1};
    return units_table_bytes(u);
}

int run_expand_count(const int64_t *rmask, int64_t R, int slots, int64_t *n_pairs, void *ws, size_t ws_bytes,
                     hipStream_t s) {
    if (R < 0 || slots <= 0 || slots > 64 || !n_pairs || R >= (int64_t)1 << 31) return TERRACE_EINVAL;
    Units u{R, 1, (int)(R > 0 ? R : 1), 1};
    if (!ws || ws_bytes < units_table_bytes(u)) return TERRACE_ENOSPC;
    int32_t *cnt = (int32_t *)ws;
    if (R == 0) {
        set_i64_kernel<<<1, 1, 0, s>>>(n_pairs, 0);
        return check_launch();
    }
    if (!rmask) return TERRACE_EINVAL;
    expand_count_kernel<<<(unsigned)((R + kBlock - 1) / kBlock), kBlock, 0, s>>>(rmask, R, slots, cnt);
    TableOut pairs_out;
    pairs_out.hist_i64 = n_pairs;
    launch_scan(u, cnt, pairs_out, nullptr, s);
    return check_launch();
}

int run_expand_fill(const int64_t *rmask, int64_t R, int slots, int64_t *r_idx, int64_t *slot_idx, const void *ws,
                    hipStream_t s) {
    if (R < 0 || slots <= 0 || slots > 64) return TERRACE_EINVAL;
    if (R == 0) return TERRACE_OK;
    if (!rmask || !r_idx || !slot_idx || !ws) return TERRACE_EINVAL;
    expand_fill_kernel<<<(unsigned)((R + kBlock - 1) / kBlock), kBlock, 0, s>>>(rmask, R, slots, (const int32_t *)ws,
                                                                              r_idx, slot_idx);
    return check_launch();
}

// ---- segment table: the items of each segment, ascending, as a padded [n_seg, width] table ---------
// The read side of an index_add: out[s] = sum of src[i] over the items i with seg[i] == s becomes a
// fixed-fan gather-reduce over table[s, :].  Slots are claimed with an atomic cursor (any order) and
// each row is then sorted ascending, so the result does not depend on the claim order.
__global__ __launch_bounds__(kBlock) void segment_claim_kernel(const int64_t *__restrict__ seg, int64_t n,
                                                               int64_t n_seg, int width, int32_t *__restrict__ cursor,
                                                               int64_t *__restrict__ table,
                                                               int32_t *__restrict__ status) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int64_t sg = seg[i];
    if (sg < 0 || sg >= n_seg) {
        if (status) atomicOr(&status[0], TERRACE_FAULT_ID_RANGE);
        return;
    }
    const int c = atomicAdd(&cursor[sg], 1);
    if (c < width) table[sg * width + c] = i;
    else if (status) atomicOr(&status[0], TERRACE_FAULT_FANOUT);
}

__global__ __launch_bounds__(kBlock) void segment_sort_kernel(int64_t n_seg, int width,
                                                              const int32_t *__restrict__ cursor,
                                                              int64_t *__restrict__ table) {
    const int64_t sg = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (sg >= n_seg) return;
    int64_t *row = table + sg * width;
    int cnt = cursor[sg];
    if (cnt > width) cnt = width;
    for (int a = 1; a < cnt; ++a) {                       // insertion sort: cnt is a handful
        const int64_t v = row[a];
        int b = a - 1;
        while (b >= 0 && row[b] > v) {
            row[b + 1] = row[b];
            --b;
        }
        row[b + 1] = v;
    }
    for (int a = cnt; a < width; ++a) row[a] = -1;
}

__global__ __launch_bounds__(kBlock) void fill_i32_kernel(int32_t *__restrict__ p, int64_t n, int32_t v) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) p[i] = v;
}

// cursors cleared and the status block zeroed in one launch
__global__ __launch_bounds__(kBlock) void segment_init_kernel(int32_t *__restrict__ cursor, int64_t n_seg,
                                                              int32_t *__restrict__ status) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n_seg) cursor[i] = 0;
    if (status && blockIdx.x == 0 && threadIdx.x < TERRACE_STATUS_WORDS) status[threadIdx.x] = 0;
}

size_t segment_table_workspace(int64_t n_seg) { return align_up((size_t)(n_seg > 0 ? n_seg : 1) * sizeof(int32_t), 256); }

int run_segment_table(const int64_t *seg, int64_t n, int64_t n_seg, int width, int64_t *table, int32_t *status,
                      void *ws, size_t ws_bytes, hipStream_t s) {
    if (n < 0 || n_seg < 0 || width <= 0 || width > 64) return TERRACE_EINVAL;
    if (n_seg == 0) {
        if (status) fill_i32_kernel<<<1, kBlock, 0, s>>>(status, TERRACE_STATUS_WORDS, 0);
        return check_launch();
    }
    if (!table || !ws || (n > 0 && !seg)) return TERRACE_EINVAL;
    if (ws_bytes < segment_table_workspace(n_seg)) return TERRACE_ENOSPC;
    int32_t *cursor = (int32_t *)ws;
    segment_init_kernel<<<(unsigned)((n_seg + kBlock - 1) / kBlock), kBlock, 0, s>>>(cursor, n_seg, status);
    if (n > 0)
        segment_claim_kernel<<<(unsigned)((n + kBlock - 1) / kBlock), kBlock, 0, s>>>(seg, n, n_seg, width, cursor, table, status);
    segment_sort_kernel<<<(unsigned)((n_seg + kBlock - 1) / kBlock), kBlock, 0, s>>>(n_seg, width, cursor, table);
    return check_launch();
}

// ---- where each (token, expert) pair sits in the expert-order buffer --------------------------------
// One lane per place i of the buffer: the arrival row behind it is a = order[i], its send row
// r = r_idx[a], its token t = u_src[r] and its expert e = u_node[r]*slots + slot_idx[a]; the column j
// with expert_idx[t, j] == e gets where[t, j] = i.  These are the tables the adjoints of the two seam
// halves read (terrace/ta2a_dispatch.py:263-498): permuted[i] = hidden[token_of_place[i]] and
// y[t] = sum_j expert_out[where[t, j]].
__global__ __launch_bounds__(kBlock) void fill_i64_kernel(int64_t *__restrict__ p, int64_t n, int64_t v) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) p[i] = v;
}

// where = -1 everywhere and the status block cleared, in one launch ahead of the kernel that fills them
__global__ __launch_bounds__(kBlock) void pair_places_init_kernel(int64_t *__restrict__ where, int64_t n,
                                                                  int32_t *__restrict__ status) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) where[i] = -1;
    if (status && blockIdx.x == 0 && threadIdx.x < TERRACE_STATUS_WORDS) status[threadIdx.x] = 0;
}

__global__ __launch_bounds__(kBlock) void pair_places_kernel(
    const int64_t *__restrict__ order, const int64_t *__restrict__ r_idx, const int64_t *__restrict__ slot_idx,
    const int64_t *__restrict__ u_src, const int64_t *__restrict__ u_node, const int64_t *__restrict__ expert_idx,
    int64_t P, int64_t T, int k, int slots, int64_t n_rows, int64_t *__restrict__ where,
    int64_t *__restrict__ token_of_place, int32_t *__restrict__ status) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= P) return;
    bool ok = false;
    int64_t t = -1;
    const int64_t a = order[i];
    if (a >= 0 && a < P) {
        const int64_t r = r_idx[a];
        if (r >= 0 && r < n_rows) {
            t = u_src[r];
            if (t >= 0 && t < T) {
                const int64_t e = u_node[r] * slots + slot_idx[a];
                for (int j = 0; j < k; ++j) {
                    if (expert_idx[t * k + j] == e) {
                        where[t * k + j] = i;
                        ok = true;
                    }
                }
            }
        }
    }
    if (token_of_place) token_of_place[i] = ok ? t : -1;
    if (!ok && status) atomicOr(&status[0], TERRACE_FAULT_ID_RANGE);
}

int run_pair_places(const int64_t *order, const int64_t *r_idx, const int64_t *slot_idx, const int64_t *u_src,
                    const int64_t *u_node, const int64_t *expert_idx, int64_t P, int64_t T, int k, int slots,
                    int64_t n_rows, int64_t *where, int64_t *token_of_place, int32_t *status, hipStream_t s) {
    if (P < 0 || T < 0 || k <= 0 || slots <= 0 || n_rows < 0) return TERRACE_EINVAL;
    if (T > 0 && !where) return TERRACE_EINVAL;
    if (T > 0 || status) {
        const int64_t n = T > 0 ? T * k : 0;
        const int64_t blocks = n > 0 ? (n + kBlock - 1) / kBlock : 1;
        pair_places_init_kernel<<<(unsigned)blocks, kBlock, 0, s>>>(where, n, status);
    }
    if (P > 0) {
        if (!order || !r_idx || !slot_idx || !u_src || !u_node || !expert_idx || !where) return TERRACE_EINVAL;
        pair_places_kernel<<<(unsigned)((P + kBlock - 1) / kBlock), kBlock, 0, s>>>(
            order, r_idx, slot_idx, u_src, u_node, expert_idx, P, T, k, slots, n_rows, where, token_of_place, status);
    }
    return check_launch();
}

// ---- routing_map -> top-k ---------------------------------------------------------------------------
// one wave per token; row_stats = {min count, max count} over tokens (int32, pre-set by the first kernel's block 0
// is not possible without ordering, so the caller provides them initialised to {INT_MAX, 0}).
__global__ __launch_bounds__(kBlock) void map_count_kernel(const uint8_t *__restrict__ map, int64_t T, int E,
                                                           int32_t *__restrict__ row_stats) {
    // a resident grid: every wave walks its share of the tokens keeping a running min / max, the workgroup
    // folds its four waves, and only then two atomics go out (per-token atomics on the same two words
    // serialise at about 20 ns each)
    __shared__ int32_t lo_of[kWavesPerBlock], hi_of[kWavesPerBlock];
    const int lane = lane_id();
    const int w = wave_in_block();
    int lo = 0x7FFFFFFF, hi = 0;
    const int64_t stride = (int64_t)gridDim.x * kWavesPerBlock;
    for (int64_t t = (int64_t)blockIdx.x * kWavesPerBlock + w; t < T; t += stride) {
        int cnt = 0;
        for (int e0 = 0; e0 < E; e0 += kWave) {
            const int e = e0 + lane;
            cnt += __popcll(__ballot(e < E && map[t * E + e] != 0));
        }
        lo = cnt < lo ? cnt : lo;
        hi = cnt > hi ? cnt : hi;
    }
    if (lane == 0) {
        lo_of[w] = lo;
        hi_of[w] = hi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < kWavesPerBlock; ++i) {
            lo = lo_of[i] < lo ? lo_of[i] : lo;
            hi = hi_of[i] > hi ? hi_of[i] : hi;
        }
        if (lo != 0x7FFFFFFF) atomicMin(&row_stats[0], lo);
        if (hi != 0) atomicMax(&row_stats[1], hi);
    }
}

// The same census when a token's E map bytes are LPTOK = E/16 whole 16-byte vectors (E = 16, 32, ... 1024) on a
// 16-byte-aligned map: the map is one flat run of vectors, a wave takes 64 * UN of them with every load issued before
// any is counted, a lane counts the non-zero bytes of its vector and the LPTOK lanes of a token add up by butterflies.
// One memory round trip per 64 * UN * 16 bytes instead of one per 64 bytes (28 -> about 6 us at 16384 x 256).
typedef uint32_t map_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ int nonzero_bytes(uint32_t x) {
    return __popc((((x & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | x) & 0x80808080u);
}
template <int LPTOK, int UN>
__global__ __launch_bounds__(kBlock) void map_count_vec_kernel(const map_u32x4 *__restrict__ map, int64_t n_vec,
                                                               int32_t *__restrict__ row_stats) {
    __shared__ int32_t lo_of[kWavesPerBlock], hi_of[kWavesPerBlock];
    const int lane = lane_id();
    const int w = wave_in_block();
    int lo = 0x7FFFFFFF, hi = 0;
    const int64_t stride = (int64_t)gridDim.x * kWavesPerBlock * kWave * UN;
    for (int64_t base = ((int64_t)blockIdx.x * kWavesPerBlock + w) * kWave * UN; base < n_vec; base += stride) {
        map_u32x4 v[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int64_t i = base + (int64_t)u * kWave + lane;
            v[u] = i < n_vec ? map[i] : map_u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            int c = nonzero_bytes(v[u][0]) + nonzero_bytes(v[u][1]) + nonzero_bytes(v[u][2]) + nonzero_bytes(v[u][3]);
#pragma unroll
            for (int d = 1; d < LPTOK; d <<= 1) c += __shfl_xor(c, d, kWave);
            // a token's vectors are all inside or all outside the map: n_vec is a multiple of LPTOK
            if (base + (int64_t)u * kWave + lane < n_vec) {
                lo = c < lo ? c : lo;
                hi = c > hi ? c : hi;
            }
        }
    }
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int ol = __shfl_xor(lo, d, kWave), oh = __shfl_xor(hi, d, kWave);
        lo = ol < lo ? ol : lo;
        hi = oh > hi ? oh : hi;
    }
    if (lane == 0) {
        lo_of[w] = lo;
        hi_of[w] = hi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < kWavesPerBlock; ++i) {
            lo = lo_of[i] < lo ? lo_of[i] : lo;
            hi = hi_of[i] > hi ? hi_of[i] : hi;
        }
        if (lo != 0x7FFFFFFF) atomicMin(&row_stats[0], lo);
        if (hi != 0) atomicMax(&row_stats[1], hi);
    }
}

__global__ void map_stats_init_kernel(int32_t *row_stats) {
    row_stats[0] = 0x7FFFFFFF;
    row_stats[1] = 0;
}

template <typename G>
__global__ __launch_bounds__(kBlock) void map_topk_kernel(const uint8_t *__restrict__ map, const G *__restrict__ probs,
                                                          int64_t T, int E, int k, int64_t *__restrict__ expert_idx,
                                                          G *__restrict__ gates) {
    const int lane = lane_id();
    const int64_t t = (int64_t)blockIdx.x * kWavesPerBlock + wave_in_block();
    if (t >= T) return;
    int before = 0;
    for (int e0 = 0; e0 < E; e0 += kWave) {
        const int e = e0 + lane;
        const bool on = e < E && map[t * E + e] != 0;
        const uint64_t peers = __ballot(on);
        if (on) {
            const int at = before + __popcll(peers & lanes_below(lane));
            if (at < k) {
                expert_idx[t * k + at] = e;
                gates[t * k + at] = probs[t * E + e];
            }
        }
        before += __popcll(peers);
    }
}

int run_map_count(const void *map, int64_t T, int E, int32_t *row_stats, hipStream_t s) {
    if (T < 0 || E <= 0 || !row_stats) return TERRACE_EINVAL;
    map_stats_init_kernel<<<1, 1, 0, s>>>(row_stats);
    if (T > 0) {
        if (!map) return TERRACE_EINVAL;
        const int lptok = E / 16;
        if (E % 16 == 0 && lptok <= kWave && (lptok & (lptok - 1)) == 0 && (((uintptr_t)map) & 15) == 0) {
            constexpr int kUn = 4;
            const int64_t n_vec = T * lptok;
            int64_t blocks = (n_vec + (int64_t)kBlock * kUn - 1) / ((int64_t)kBlock * kUn);
            if (blocks > 2048) blocks = 2048;
#define TERRACE_MAPC(L) \
    map_count_vec_kernel<L, kUn><<<(unsigned)blocks, kBlock, 0, s>>>((const map_u32x4 *)map, n_vec, row_stats)
            switch (lptok) {
                case 1: TERRACE_MAPC(1); break;
                case 2: TERRACE_MAPC(2); break;
                case 4: TERRACE_MAPC(4); break;
                case 8: TERRACE_MAPC(8); break;
                case 16: TERRACE_MAPC(16); break;
                case 32: TERRACE_MAPC(32); break;
                default: TERRACE_MAPC(64); break;
            }
#undef TERRACE_MAPC
            return check_launch();
        }
        int64_t blocks = (T + kWavesPerBlock - 1) / kWavesPerBlock;
        if (blocks > 1024) blocks = 1024;
        map_count_kernel<<<(unsigned)blocks, kBlock, 0, s>>>((const uint8_t *)map, T, E, row_stats);
    }
    return check_launch();
}

int run_map_topk(const void *map, const void *probs, int elem_bytes, int64_t T, int E, int k, int64_t *expert_idx,
                 void *gates, hipStream_t s) {
    if (T < 0 || E <= 0 || k <= 0 || k > E || (elem_bytes != 2 && elem_bytes != 4)) return TERRACE_EINVAL;
    if (T == 0) return TERRACE_OK;
    if (!map || !probs || !expert_idx || !gates) return TERRACE_EINVAL;
    const unsigned grid = (unsigned)((T + kWavesPerBlock - 1) / kWavesPerBlock);
    if (elem_bytes == 4)
        map_topk_kernel<uint32_t><<<grid, kBlock, 0, s>>>((const uint8_t *)map, (const uint32_t *)probs, T, E, k, expert_idx, (uint32_t *)gates);
    else
        map_topk_kernel<uint16_t><<<grid, kBlock, 0, s>>>((const uint8_t *)map, (const uint16_t *)probs, T, E, k, expert_idx, (uint16_t *)gates);
    return check_launch();
}

}  // namespace terrace
