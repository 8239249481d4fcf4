// Shared pieces of the counting-sort index build (sort.hip, pack.hip).
#pragma once

#include "common.hpp"

namespace terrace {

constexpr int kMaxBuckets = 2048;
constexpr int kScanThreads = 1024;

// A "unit" is the contiguous run of items one wave owns: chunks * 64 of them.
struct Units {
    int64_t n_items;
    int chunks;       // 64-item chunks per unit: 1, 4 or 16, growing with the item count
    int n_units;
    int n_buckets;
};

Units make_units(int64_t n_items, int n_buckets);
size_t units_table_bytes(const Units &u);

// Exclusive prefix over the bucket-major count table table[b * n_units + unit], in place; also
// start[b] (n_buckets + 1 int32 right after the table), the optional histogram / offsets planes
// and a zeroed status block.
void launch_scan(const Units &u, int32_t *table, int64_t *hist_i64, float *hist_f32, int64_t *offsets_i64,
                 int32_t *status, hipStream_t s);

// n_dst / n_src bound the row ids the movers accept: an id outside [0, bound) is a dead entry.
template <typename I>
int launch_scatter_rows(const void *src, void *dst, const I *pos, int64_t n_src, int fan, int64_t row_bytes,
                        int64_t n_dst, hipStream_t s);
template <typename I>
int launch_gather_rows(const void *src, void *out, const I *idx, int64_t n_out, int64_t row_bytes, int64_t n_src,
                       hipStream_t s);

// Send side with one lane per token (n_nodes <= 64, k <= 16); returns false when the geometry
// is outside that and the caller must take the (token, run)-item path.
bool k2_token_path_applies(int k, int n_nodes);
size_t k2_token_workspace(int64_t T, int n_nodes, int groups_m);
// Where run_k2_token leaves the [T, groups_m] int32 send-row positions inside its workspace.
const int32_t *k2_token_positions(const void *ws, int64_t T, int n_nodes);
int run_k2_token(const void *hidden, const int64_t *expert_idx, const void *gates, int64_t T, int64_t row_bytes,
                 int gate_bytes, int k, int slots, int n_nodes, int n_experts, int groups_m, void *payload,
                 int64_t *mask, void *gate_rows, int64_t *u_src, int64_t *node_counts, int64_t *u_node,
                 int64_t *inverse, int64_t *node_offsets, int64_t *pair_table, int64_t *sort_order,
                 int64_t *token_rows, void *gate_sorted, int32_t *status, void *ws, int64_t mask_pitch,
                 int64_t gate_pitch, int gate_pad, hipStream_t s);

}  // namespace terrace
