// extern "C" surface of libterrace_hip.so: argument checks and dispatch to the launchers.
#include "common.hpp"

namespace terrace {
int launch_copy(const void *x, void *y, size_t nbytes, hipStream_t s);
int launch_stream_probe(int kind, const void *x, void *y, size_t nbytes, hipStream_t s);
int launch_combine2(const void *src, int64_t n_src, int src_dtype, const int64_t *inner, int64_t n_rows, int fan_inner,
                    const int64_t *outer, int64_t n_out, int fan_outer, int64_t hidden, void *out, int out_dtype,
                    hipStream_t s);
int launch_combine(const void *src, int64_t n_src, int src_dtype, const int64_t *idx, const void *w, int w_dtype,
                   int64_t n_out, int fan, int64_t hidden, void *out, int out_dtype, int64_t src_pitch,
                   hipStream_t s);
int launch_index_chain(const int64_t *table, int64_t n_table, const int64_t *idx, int64_t n, int64_t *out,
                       hipStream_t s);
int launch_index_chain2(const int64_t *outer, int64_t n_outer, const int64_t *inner, int64_t n_inner,
                        const int64_t *idx, int64_t n, int64_t *out, hipStream_t s);
int launch_pack_planes(const void *a, int64_t a_bytes, const void *b, int64_t b_bytes, const void *c, int64_t c_bytes,
                       int64_t n_rows, int64_t row_bytes, void *out, hipStream_t s);
int launch_unpack_planes(const void *packed, int64_t row_bytes, int64_t n_rows, void *a, int64_t a_bytes, void *b,
                         int64_t b_bytes, void *c, int64_t c_bytes, hipStream_t s);
int launch_send_splits(const int64_t *node_counts, int world, int rpn, int my_local, int64_t *send, hipStream_t s);
template <typename I>
int launch_scatter_rows(const void *src, void *dst, const I *pos, int64_t n_src, int fan, int64_t row_bytes,
                        int64_t n_dst, hipStream_t s);
template <typename I>
int launch_gather_rows(const void *src, void *out, const I *idx, int64_t n_out, int64_t row_bytes, int64_t n_src,
                       hipStream_t s);
int run_t_route(const float *affinity, const float *bias, const float *gate_affinity, int64_t T, int E, int n_groups,
                int k, int M, int pool, int mode, int64_t *expert_idx, void *gates, int gate_dtype,
                int64_t *group_idx, int force_generic, hipStream_t s);
size_t hist_workspace(int64_t n, int n_buckets);
int run_hist(const int64_t *idx, int64_t n, int n_buckets, void *out, int as_float, int32_t *status, void *ws,
             size_t ws_bytes, hipStream_t s);
int run_argsort_small(const int64_t *key, int64_t n, int n_buckets, int64_t *order, int64_t *hist, int32_t *status,
                      void *ws, size_t ws_bytes, hipStream_t s);
size_t k1_workspace(int64_t R, int quota, int rpn);
int run_k1_arrival(const void *rx, const int64_t *rslot, const void *rgate, int64_t R, int64_t row_bytes,
                   int gate_bytes, int quota, int epr, int rpn, int my_local, void *send_buf, void *gate_pairs,
                   int64_t *r_idx, int64_t *slot_idx, int64_t *i_send, int64_t *pair_pos, int32_t *status, void *ws,
                   size_t ws_bytes, int64_t slot_pitch, int64_t gate_pitch, int64_t *meta, const int64_t *tags_in,
                   int64_t *tags_out, hipStream_t s);
size_t regroup_workspace(int64_t P, int epr, int64_t capacity);
int run_regroup(const void *node_rx, const int64_t *my_slot, const void *my_gate, int64_t P, int64_t row_bytes,
                int gate_bytes, int epr, int my_local, int64_t capacity, void *permuted, void *permuted_gate,
                int64_t *order, int64_t *dest, uint8_t *kept, int64_t *tokens_per_expert, int64_t *kept_per_expert,
                int32_t *status, void *ws, size_t ws_bytes, int64_t slot_pitch, int64_t gate_pitch,
                const int64_t *tags_in, int64_t *place_by_tag, int64_t n_tags, hipStream_t s);
size_t hopb_workspace(int64_t R, int quota, int n_local);
int run_hopb_scatter(const void *rx, const int64_t *rslot, const void *rgate, int64_t R, int64_t row_bytes,
                     int gate_bytes, int quota, int first_slot, int n_local, int64_t capacity, void *permuted,
                     void *permuted_gate, int64_t *place, uint8_t *kept, int64_t *pair_of_place,
                     int64_t *tokens_per_expert, int64_t *kept_per_expert, const int64_t *tags_in,
                     int64_t *place_by_tag, int64_t n_tags, int32_t *status, void *ws, size_t ws_bytes,
                     hipStream_t s);
int run_hopb_scatter_move(const void *rx, int64_t R, int64_t row_bytes, int quota, int n_local, int64_t capacity,
                          void *permuted, const void *ws, size_t ws_bytes, hipStream_t s);
size_t k2_workspace(int64_t T, int k, int n_nodes, int groups_m);
int run_k2_pack(const void *hidden, const int64_t *expert_idx, const void *gates, int64_t T, int64_t row_bytes,
                int gate_bytes, int k, int world, int n_experts, int rpn, int groups_m, void *payload, int64_t *mask,
                void *gate_rows, int64_t *u_src, int64_t *node_counts, int64_t *u_node, int64_t *inverse,
                int64_t *node_offsets, int64_t *pair_table, int64_t *sort_order, int64_t *token_rows,
                void *gate_sorted, int64_t *pair_src, int64_t *combine_table, int32_t *status, void *ws,
                size_t ws_bytes, int64_t mask_pitch, int64_t gate_pitch, int gate_pad, hipStream_t s);
int run_pack_quota_wire(const int64_t *expert_idx, const void *gates, const int64_t *inverse, int64_t T, int k,
                        int gate_bytes, int64_t n_rows, int slots, int quota, int64_t *slot_tab, void *gate_tab,
                        int32_t *status, hipStream_t s);
size_t plan_general_workspace(int64_t T, int k, int n_nodes);
int run_plan_general(const int64_t *expert_idx, int64_t T, int k, int world, int n_experts, int rpn, int64_t *u_src,
                     int64_t *u_node, int64_t *counts, int64_t *inverse, int32_t *status, void *ws, size_t ws_bytes,
                     hipStream_t s);
int run_build_mask(const int64_t *expert_idx, const int64_t *inverse, int64_t n, int slots, int64_t n_rows,
                   int64_t *mask, int32_t *status, hipStream_t s);
int run_scatter_elems(const void *vals, int elem_bytes, const int64_t *rows, const int64_t *cols, int col_mod,
                      int64_t n, int64_t n_rows, int width, void *out, hipStream_t s);
int run_expand_quota(const int64_t *rmask, int64_t R, int slots, int quota, int64_t *r_idx, int64_t *slot_idx,
                     hipStream_t s);
size_t expand_workspace(int64_t R);
int run_expand_count(const int64_t *rmask, int64_t R, int slots, int64_t *n_pairs, void *ws, size_t ws_bytes,
                     hipStream_t s);
int run_expand_fill(const int64_t *rmask, int64_t R, int slots, int64_t *r_idx, int64_t *slot_idx, const void *ws,
                    hipStream_t s);
size_t arrival_pairs_workspace(int64_t P, int rpn);
int run_arrival_pairs(const void *rx, const int64_t *r_in, const int64_t *slot_in, const void *rgate, int64_t R,
                      int64_t P, int64_t row_bytes, int gate_bytes, int gate_width, int epr, int rpn, void *send_buf,
                      void *gate_pairs, int64_t *r_idx, int64_t *slot_idx, int64_t *i_send, int64_t *ordo,
                      int32_t *status, void *ws, size_t ws_bytes, hipStream_t s);
size_t segment_table_workspace(int64_t n_seg);
int run_segment_table(const int64_t *seg, int64_t n, int64_t n_seg, int width, int64_t *table, int32_t *status,
                      void *ws, size_t ws_bytes, hipStream_t s);
int run_pair_places(const int64_t *order, const int64_t *r_idx, const int64_t *slot_idx, const int64_t *u_src,
                    const int64_t *u_node, const int64_t *expert_idx, int64_t P, int64_t T, int k, int slots,
                    int64_t n_rows, int64_t *where, int64_t *token_of_place, int32_t *status, hipStream_t s);
int run_map_count(const void *map, int64_t T, int E, int32_t *row_stats, hipStream_t s);
int run_map_topk(const void *map, const void *probs, int elem_bytes, int64_t T, int E, int k, int64_t *expert_idx,
                 void *gates, hipStream_t s);
int run_k2_pack_move(const void *hidden, int64_t T, int64_t row_bytes, int k, int n_nodes, int groups_m,
                     void *payload, const void *ws, size_t ws_bytes, hipStream_t s);
int run_k1_arrival_move(const void *rx, int64_t R, int64_t row_bytes, int quota, int rpn, void *send_buf,
                        const void *ws, size_t ws_bytes, hipStream_t s);
int run_regroup_move(const void *node_rx, int64_t P, int64_t row_bytes, int epr, int64_t capacity, void *permuted,
                     const void *ws, size_t ws_bytes, hipStream_t s);
}  // namespace terrace

using namespace terrace;

static bool float_dtype(int d) { return d == TERRACE_F32 || d == TERRACE_BF16 || d == TERRACE_F16; }

extern "C" {

#ifndef TERRACE_SOURCE_HASH
#define TERRACE_SOURCE_HASH "unstamped"
#endif
// ends with the digest of the sources this library was built from (csrc/build.py stamps it)
const char *terrace_version(void) { return "terrace-hip 0.1 (gfx950) src:" TERRACE_SOURCE_HASH; }

const char *terrace_strerror(int status) {
    switch (status) {
        case TERRACE_OK: return "ok";
        case TERRACE_EINVAL: return "invalid argument (geometry, null pointer or unsupported size)";
        case TERRACE_ENOSPC: return "workspace too small";
        case TERRACE_ELAUNCH: return "HIP kernel launch failed";
        case TERRACE_E2BIG: return "input larger than the fixed scratch of the no-allocation entry point";
        default: return "unknown status";
    }
}

int terrace_passthrough(const void *x, void *y, size_t nbytes, terrace_stream_t stream) {
    if (nbytes && (!x || !y)) return TERRACE_EINVAL;
    return launch_copy(x, y, nbytes, (hipStream_t)stream);
}

int terrace_stream_probe(int kind, const void *x, void *y, size_t nbytes, terrace_stream_t stream) {
    return launch_stream_probe(kind, x, y, nbytes, (hipStream_t)stream);
}

int terrace_t_route(const float *affinity, const float *bias, const float *gate_affinity, int64_t T, int n_experts,
                    int n_groups, int top_k, int top_groups, int pool, int mode, int64_t *expert_idx, void *gates,
                    int64_t *group_idx, terrace_stream_t stream) {
    const int force = (mode & TERRACE_ROUTE_FORCE_GENERIC) ? 1 : 0;
    const int flags = TERRACE_ROUTE_FORCE_GENERIC | TERRACE_ROUTE_GATES_BF16 | TERRACE_ROUTE_GATES_F16;
    if ((mode & TERRACE_ROUTE_GATES_BF16) && (mode & TERRACE_ROUTE_GATES_F16)) return TERRACE_EINVAL;
    const int gate_dtype = (mode & TERRACE_ROUTE_GATES_BF16) ? TERRACE_BF16
                                                             : ((mode & TERRACE_ROUTE_GATES_F16) ? TERRACE_F16 : TERRACE_F32);
    return run_t_route(affinity, bias, gate_affinity, T, n_experts, n_groups, top_k, top_groups, pool, mode & ~flags,
                       expert_idx, gates, gate_dtype, group_idx, force, (hipStream_t)stream);
}

size_t terrace_hist_workspace(int64_t n, int n_buckets) { return hist_workspace(n, n_buckets); }

int terrace_hist(const int64_t *idx, int64_t n, int n_buckets, void *out, int as_float, int32_t *status,
                 void *workspace, size_t workspace_bytes, terrace_stream_t stream) {
    return run_hist(idx, n, n_buckets, out, as_float, status, workspace, workspace_bytes, (hipStream_t)stream);
}

size_t terrace_argsort_small_workspace(int64_t n, int n_buckets) { return hist_workspace(n, n_buckets); }

int terrace_argsort_small(const int64_t *key, int64_t n, int n_buckets, int64_t *order, int64_t *hist,
                          int32_t *status, void *workspace, size_t workspace_bytes, terrace_stream_t stream) {
    return run_argsort_small(key, n, n_buckets, order, hist, status, workspace, workspace_bytes, (hipStream_t)stream);
}

size_t terrace_k2_pack_workspace(int64_t T, int k, int n_nodes, int groups_m) {
    return k2_workspace(T, k, n_nodes, groups_m);
}

int terrace_k2_pack(const void *hidden, const int64_t *expert_idx, const void *gates, int64_t T, int64_t row_bytes,
                    int gate_bytes, int k, int world, int n_experts, int rpn, int groups_m, void *payload,
                    int64_t *mask, void *gate_rows, int64_t *u_src, int64_t *node_counts, int64_t *u_node,
                    int64_t *inverse, int64_t *node_offsets, int64_t *pair_table, int64_t *sort_order,
                    int64_t *token_rows, void *gate_sorted, int64_t *pair_src, int64_t *combine_table,
                    int32_t *status, void *workspace, size_t workspace_bytes, terrace_stream_t stream) {
    return run_k2_pack(hidden, expert_idx, gates, T, row_bytes, gate_bytes, k, world, n_experts, rpn, groups_m,
                       payload, mask, gate_rows, u_src, node_counts, u_node, inverse, node_offsets, pair_table,
                       sort_order, token_rows, gate_sorted, pair_src, combine_table, status, workspace,
                       workspace_bytes, 0, 0, 0, (hipStream_t)stream);
}

// Words of one Hop-A small container row holding `quota` slot ids and `quota` gates.
static int wire_words_needed(int quota, int gate_bytes) { return quota + (quota * gate_bytes + 7) / 8; }

int terrace_k2_pack_wire(const void *hidden, const int64_t *expert_idx, const void *gates, int64_t T, int64_t row_bytes,
                         int gate_bytes, int k, int world, int n_experts, int rpn, int groups_m, void *payload,
                         int64_t *wire, int wire_words, int64_t *u_src, int64_t *node_counts, int64_t *u_node,
                         int64_t *inverse, int64_t *node_offsets, int64_t *pair_table, int64_t *sort_order,
                         int64_t *token_rows, void *gate_sorted, int32_t *status, void *workspace,
                         size_t workspace_bytes, terrace_stream_t stream) {
    if (groups_m <= 0 || k <= 0 || k % groups_m || (gate_bytes != 2 && gate_bytes != 4)) return TERRACE_EINVAL;
    const int quota = k / groups_m;
    if (wire_words < wire_words_needed(quota, gate_bytes) || (T > 0 && (!wire || !gates))) return TERRACE_EINVAL;
    const int per_word = 8 / gate_bytes;
    void *gate_plane = (void *)(wire + quota);                 // the gates start on the word after the ids
    return run_k2_pack(hidden, expert_idx, gates, T, row_bytes, gate_bytes, k, world, n_experts, rpn, groups_m,
                       payload, wire, gate_plane, u_src, node_counts, u_node, inverse, node_offsets, pair_table,
                       sort_order, token_rows, gate_sorted, nullptr, nullptr, status, workspace, workspace_bytes,
                       wire_words,
                       (int64_t)wire_words * per_word, (wire_words - quota) * per_word - quota, (hipStream_t)stream);
}

int terrace_pack_quota_wire(const int64_t *expert_idx, const void *gates, const int64_t *inverse, int64_t T, int k,
                            int gate_bytes, int64_t n_rows, int slots, int quota, int64_t *slot_tab, void *gate_tab,
                            int32_t *status, terrace_stream_t stream) {
    return run_pack_quota_wire(expert_idx, gates, inverse, T, k, gate_bytes, n_rows, slots, quota, slot_tab,
                               gate_tab, status, (hipStream_t)stream);
}

size_t terrace_k1_arrival_workspace(int64_t R, int quota, int rpn) { return k1_workspace(R, quota, rpn); }

int terrace_k1_arrival(const void *rx, const int64_t *rslot, const void *rgate, int64_t R, int64_t row_bytes,
                       int gate_bytes, int quota, int epr, int rpn, int my_local, void *send_buf, void *gate_pairs,
                       int64_t *r_idx, int64_t *slot_idx, int64_t *i_send, int64_t *pair_pos, const int64_t *tags_in,
                       int64_t *tags_out, int32_t *status, void *workspace, size_t workspace_bytes,
                       terrace_stream_t stream) {
    return run_k1_arrival(rx, rslot, rgate, R, row_bytes, gate_bytes, quota, epr, rpn, my_local, send_buf,
                          gate_pairs, r_idx, slot_idx, i_send, pair_pos, status, workspace, workspace_bytes, quota,
                          quota, nullptr, tags_in, tags_out, (hipStream_t)stream);
}

int terrace_k1_arrival_wire(const void *rx, const int64_t *rwire, int wire_words, int64_t R, int64_t row_bytes,
                            int gate_bytes, int quota, int epr, int rpn, int my_local, void *send_buf, int64_t *meta,
                            int64_t *r_idx, int64_t *slot_idx, void *gate_pairs, int64_t *i_send, int64_t *pair_pos,
                            int32_t *status, void *workspace, size_t workspace_bytes, terrace_stream_t stream) {
    if (quota <= 0 || (gate_bytes != 2 && gate_bytes != 4) || wire_words < wire_words_needed(quota, gate_bytes))
        return TERRACE_EINVAL;
    if (R > 0 && (!rwire || !meta)) return TERRACE_EINVAL;
    const void *gate_plane = rwire ? (const void *)(rwire + quota) : nullptr;
    return run_k1_arrival(rx, rwire, gate_plane, R, row_bytes, gate_bytes, quota, epr, rpn, my_local, send_buf,
                          gate_pairs, r_idx, slot_idx, i_send, pair_pos, status, workspace, workspace_bytes,
                          wire_words, (int64_t)wire_words * (8 / gate_bytes), meta, nullptr, nullptr,
                          (hipStream_t)stream);
}

size_t terrace_regroup_workspace(int64_t P, int epr, int64_t capacity) { return regroup_workspace(P, epr, capacity); }

int terrace_regroup(const void *node_rx, const int64_t *my_slot, const void *my_gate, int64_t P, int64_t row_bytes,
                    int gate_bytes, int epr, int my_local, int64_t capacity, void *permuted, void *permuted_gate,
                    int64_t *order, int64_t *dest, uint8_t *kept, int64_t *tokens_per_expert,
                    int64_t *kept_per_expert, const int64_t *tags_in, int64_t *place_by_tag, int64_t n_tags,
                    int32_t *status, void *workspace, size_t workspace_bytes, terrace_stream_t stream) {
    return run_regroup(node_rx, my_slot, my_gate, P, row_bytes, gate_bytes, epr, my_local, capacity, permuted,
                       permuted_gate, order, dest, kept, tokens_per_expert, kept_per_expert, status, workspace,
                       workspace_bytes, 1, 1, tags_in, place_by_tag, n_tags, (hipStream_t)stream);
}

int terrace_regroup_wire(const void *node_rx, const int64_t *my_meta, int64_t P, int64_t row_bytes, int gate_bytes,
                         int epr, int my_local, int64_t capacity, void *permuted, void *permuted_gate, int64_t *order,
                         int64_t *dest, uint8_t *kept, int64_t *tokens_per_expert, int64_t *kept_per_expert,
                         int32_t *status, void *workspace, size_t workspace_bytes, terrace_stream_t stream) {
    if (gate_bytes != 2 && gate_bytes != 4) return TERRACE_EINVAL;
    if (P > 0 && !my_meta) return TERRACE_EINVAL;
    // word 0 of a pair's row is its slot id, word 1 starts with its gate
    const void *gate_plane = (permuted_gate && my_meta) ? (const void *)(my_meta + 1) : nullptr;
    return run_regroup(node_rx, my_meta, gate_plane, P, row_bytes, gate_bytes, epr, my_local, capacity, permuted,
                       permuted_gate, order, dest, kept, tokens_per_expert, kept_per_expert, status, workspace,
                       workspace_bytes, 2, 2 * (8 / gate_bytes), nullptr, nullptr, 0, (hipStream_t)stream);
}

size_t terrace_hopb_scatter_workspace(int64_t R, int quota, int n_local) { return hopb_workspace(R, quota, n_local); }

int terrace_hopb_scatter(const void *rx, const int64_t *rslot, const void *rgate, int64_t R, int64_t row_bytes,
                         int gate_bytes, int quota, int first_slot, int n_local, int64_t capacity, void *permuted,
                         void *permuted_gate, int64_t *place, uint8_t *kept, int64_t *pair_of_place,
                         int64_t *tokens_per_expert, int64_t *kept_per_expert, const int64_t *tags_in,
                         int64_t *place_by_tag, int64_t n_tags, int32_t *status, void *workspace,
                         size_t workspace_bytes, terrace_stream_t stream) {
    return run_hopb_scatter(rx, rslot, rgate, R, row_bytes, gate_bytes, quota, first_slot, n_local, capacity, permuted,
                            permuted_gate, place, kept, pair_of_place, tokens_per_expert, kept_per_expert, tags_in,
                            place_by_tag, n_tags, status, workspace, workspace_bytes, (hipStream_t)stream);
}

int terrace_hopb_scatter_move(const void *rx, int64_t R, int64_t row_bytes, int quota, int n_local, int64_t capacity,
                              void *permuted, const void *workspace, size_t workspace_bytes, terrace_stream_t stream) {
    return run_hopb_scatter_move(rx, R, row_bytes, quota, n_local, capacity, permuted, workspace, workspace_bytes,
                                 (hipStream_t)stream);
}

int terrace_k2_pack_move(const void *hidden, int64_t T, int64_t row_bytes, int k, int n_nodes, int groups_m,
                         void *payload, const void *workspace, size_t workspace_bytes, terrace_stream_t stream) {
    return run_k2_pack_move(hidden, T, row_bytes, k, n_nodes, groups_m, payload, workspace, workspace_bytes,
                            (hipStream_t)stream);
}

int terrace_k1_arrival_move(const void *rx, int64_t R, int64_t row_bytes, int quota, int rpn, void *send_buf,
                            const void *workspace, size_t workspace_bytes, terrace_stream_t stream) {
    return run_k1_arrival_move(rx, R, row_bytes, quota, rpn, send_buf, workspace, workspace_bytes,
                               (hipStream_t)stream);
}

int terrace_regroup_move(const void *node_rx, int64_t P, int64_t row_bytes, int epr, int64_t capacity,
                         void *permuted, const void *workspace, size_t workspace_bytes, terrace_stream_t stream) {
    return run_regroup_move(node_rx, P, row_bytes, epr, capacity, permuted, workspace, workspace_bytes,
                            (hipStream_t)stream);
}

int terrace_gather_rows(const void *src, int64_t n_src, const int64_t *idx, int64_t n_out, int64_t row_bytes,
                        void *out, terrace_stream_t stream) {
    if (n_out < 0 || row_bytes < 0 || n_src < 0) return TERRACE_EINVAL;
    if (n_out && row_bytes && ((!src && n_src) || !idx || !out)) return TERRACE_EINVAL;
    return launch_gather_rows<int64_t>(src, out, idx, n_out, row_bytes, n_src, (hipStream_t)stream);
}

int terrace_scatter_rows(const void *src, const int64_t *pos, int64_t n_src, int fan, int64_t row_bytes, void *dst,
                         int64_t n_dst, terrace_stream_t stream) {
    if (n_src < 0 || fan <= 0 || row_bytes < 0 || n_dst < 0) return TERRACE_EINVAL;
    if (n_src && row_bytes && (!src || !pos || (!dst && n_dst))) return TERRACE_EINVAL;
    return launch_scatter_rows<int64_t>(src, dst, pos, n_src, fan, row_bytes, n_dst, (hipStream_t)stream);
}

int terrace_index_chain(const int64_t *table, int64_t n_table, const int64_t *idx, int64_t n, int64_t *out,
                        terrace_stream_t stream) {
    if (n < 0 || n_table < 0 || (n && ((!table && n_table) || !idx || !out))) return TERRACE_EINVAL;
    return launch_index_chain(table, n_table, idx, n, out, (hipStream_t)stream);
}

int terrace_index_chain2(const int64_t *outer, int64_t n_outer, const int64_t *inner, int64_t n_inner,
                         const int64_t *idx, int64_t n, int64_t *out, terrace_stream_t stream) {
    if (n < 0 || n_outer < 0 || n_inner < 0) return TERRACE_EINVAL;
    if (n && ((!outer && n_outer) || (!inner && n_inner) || !idx || !out)) return TERRACE_EINVAL;
    return launch_index_chain2(outer, n_outer, inner, n_inner, idx, n, out, (hipStream_t)stream);
}

int terrace_combine_pitched(const void *src, int64_t n_src, int src_dtype, int64_t src_row_pitch, const int64_t *idx,
                            const void *weights, int w_dtype, int64_t n_out, int fan, int64_t hidden, void *out,
                            int out_dtype, terrace_stream_t stream) {
    if (n_out < 0 || fan <= 0 || hidden < 0 || n_src < 0 || src_row_pitch < 0) return TERRACE_EINVAL;
    if (src_dtype < TERRACE_F32 || src_dtype > TERRACE_FP8_E4M3_B128 || !float_dtype(out_dtype)) return TERRACE_EINVAL;
    if (weights && !float_dtype(w_dtype)) return TERRACE_EINVAL;
    if (src_dtype == TERRACE_FP8_E4M3_B128 && hidden % 128) return TERRACE_EINVAL;
    if (n_out && hidden && ((!src && n_src) || !idx || !out)) return TERRACE_EINVAL;
    return launch_combine(src, n_src, src_dtype, idx, weights, w_dtype, n_out, fan, hidden, out, out_dtype,
                          src_row_pitch, (hipStream_t)stream);
}

int terrace_combine(const void *src, int64_t n_src, int src_dtype, const int64_t *idx, const void *weights,
                    int w_dtype, int64_t n_out, int fan, int64_t hidden, void *out, int out_dtype,
                    terrace_stream_t stream) {
    return terrace_combine_pitched(src, n_src, src_dtype, 0, idx, weights, w_dtype, n_out, fan, hidden, out, out_dtype,
                                   stream);
}

int terrace_combine_two_level(const void *src, int64_t n_src, int src_dtype, const int64_t *inner, int64_t n_rows,
                              int fan_inner, const int64_t *outer, int64_t n_out, int fan_outer, int64_t hidden,
                              void *out, int out_dtype, terrace_stream_t stream) {
    return launch_combine2(src, n_src, src_dtype, inner, n_rows, fan_inner, outer, n_out, fan_outer, hidden, out,
                           out_dtype, (hipStream_t)stream);
}

int terrace_pack_planes(const void *a, int64_t a_bytes, const void *b, int64_t b_bytes, const void *c, int64_t c_bytes,
                        int64_t n_rows, int64_t row_bytes, void *out, terrace_stream_t stream) {
    if (n_rows < 0 || a_bytes < 0 || b_bytes < 0 || c_bytes < 0) return TERRACE_EINVAL;
    const int64_t used = (a ? a_bytes : 0) + (b ? b_bytes : 0) + (c ? c_bytes : 0);
    if (row_bytes < used || (n_rows && row_bytes && !out)) return TERRACE_EINVAL;
    // an absent plane must not leave a hole in front of a present one
    if ((!a && a_bytes && (b || c)) || (!b && b_bytes && c)) return TERRACE_EINVAL;
    return launch_pack_planes(a, a_bytes, b, b_bytes, c, c_bytes, n_rows, row_bytes, out, (hipStream_t)stream);
}

int terrace_unpack_planes(const void *packed, int64_t row_bytes, int64_t n_rows, void *a, int64_t a_bytes, void *b,
                          int64_t b_bytes, void *c, int64_t c_bytes, terrace_stream_t stream) {
    if (n_rows < 0 || a_bytes < 0 || b_bytes < 0 || c_bytes < 0 || row_bytes < a_bytes + b_bytes + c_bytes)
        return TERRACE_EINVAL;
    if (n_rows && row_bytes && !packed) return TERRACE_EINVAL;
    return launch_unpack_planes(packed, row_bytes, n_rows, a, a_bytes, b, b_bytes, c, c_bytes, (hipStream_t)stream);
}

size_t terrace_plan_general_workspace(int64_t T, int k, int n_nodes) {
    return plan_general_workspace(T, k, n_nodes);
}

int terrace_plan_general(const int64_t *expert_idx, int64_t T, int k, int world, int n_experts, int rpn,
                         int64_t *u_src, int64_t *u_node, int64_t *counts, int64_t *inverse, int32_t *status,
                         void *workspace, size_t workspace_bytes, terrace_stream_t stream) {
    return run_plan_general(expert_idx, T, k, world, n_experts, rpn, u_src, u_node, counts, inverse, status,
                            workspace, workspace_bytes, (hipStream_t)stream);
}

int terrace_build_mask(const int64_t *expert_idx, const int64_t *inverse, int64_t n, int slots, int64_t n_rows,
                       int64_t *mask, int32_t *status, terrace_stream_t stream) {
    return run_build_mask(expert_idx, inverse, n, slots, n_rows, mask, status, (hipStream_t)stream);
}

int terrace_scatter_elems(const void *vals, int elem_bytes, const int64_t *rows, const int64_t *cols, int col_mod,
                          int64_t n, int64_t n_rows, int width, void *out, terrace_stream_t stream) {
    return run_scatter_elems(vals, elem_bytes, rows, cols, col_mod, n, n_rows, width, out, (hipStream_t)stream);
}

int terrace_expand_mask_quota(const int64_t *rmask, int64_t R, int slots, int quota, int64_t *r_idx,
                              int64_t *slot_idx, terrace_stream_t stream) {
    return run_expand_quota(rmask, R, slots, quota, r_idx, slot_idx, (hipStream_t)stream);
}

size_t terrace_expand_mask_workspace(int64_t R) { return expand_workspace(R); }

int terrace_expand_mask_count(const int64_t *rmask, int64_t R, int slots, int64_t *n_pairs, void *workspace,
                              size_t workspace_bytes, terrace_stream_t stream) {
    return run_expand_count(rmask, R, slots, n_pairs, workspace, workspace_bytes, (hipStream_t)stream);
}

int terrace_expand_mask_fill(const int64_t *rmask, int64_t R, int slots, int64_t *r_idx, int64_t *slot_idx,
                             const void *workspace, terrace_stream_t stream) {
    return run_expand_fill(rmask, R, slots, r_idx, slot_idx, workspace, (hipStream_t)stream);
}

size_t terrace_arrival_pairs_workspace(int64_t P, int rpn) { return arrival_pairs_workspace(P, rpn); }

int terrace_arrival_pairs(const void *rx, const int64_t *r_in, const int64_t *slot_in, const void *rgate, int64_t R,
                          int64_t P, int64_t row_bytes, int gate_bytes, int gate_width, int epr, int rpn,
                          void *send_buf, void *gate_pairs, int64_t *r_idx, int64_t *slot_idx, int64_t *i_send,
                          int64_t *ordo, int32_t *status, void *workspace, size_t workspace_bytes,
                          terrace_stream_t stream) {
    return run_arrival_pairs(rx, r_in, slot_in, rgate, R, P, row_bytes, gate_bytes, gate_width, epr, rpn, send_buf,
                             gate_pairs, r_idx, slot_idx, i_send, ordo, status, workspace, workspace_bytes,
                             (hipStream_t)stream);
}

size_t terrace_segment_table_workspace(int64_t n_seg) { return segment_table_workspace(n_seg); }

int terrace_segment_table(const int64_t *seg, int64_t n, int64_t n_seg, int width, int64_t *table, int32_t *status,
                          void *workspace, size_t workspace_bytes, terrace_stream_t stream) {
    return run_segment_table(seg, n, n_seg, width, table, status, workspace, workspace_bytes, (hipStream_t)stream);
}

int terrace_pair_places(const int64_t *order, const int64_t *r_idx, const int64_t *slot_idx, const int64_t *u_src,
                        const int64_t *u_node, const int64_t *expert_idx, int64_t P, int64_t T, int k, int slots,
                        int64_t n_rows, int64_t *where, int64_t *token_of_place, int32_t *status,
                        terrace_stream_t stream) {
    return run_pair_places(order, r_idx, slot_idx, u_src, u_node, expert_idx, P, T, k, slots, n_rows, where,
                           token_of_place, status, (hipStream_t)stream);
}

int terrace_routing_map_count(const void *routing_map, int64_t T, int n_experts, int32_t *row_stats,
                              terrace_stream_t stream) {
    return run_map_count(routing_map, T, n_experts, row_stats, (hipStream_t)stream);
}

int terrace_routing_map_topk(const void *routing_map, const void *probs, int elem_bytes, int64_t T, int n_experts,
                             int k, int64_t *expert_idx, void *gates, terrace_stream_t stream) {
    return run_map_topk(routing_map, probs, elem_bytes, T, n_experts, k, expert_idx, gates, (hipStream_t)stream);
}

// ---- the whole dispatch in one call ----
namespace {
struct DispatchGeometry {
    int64_t S, P;
    int n_nodes, epr, slots, quota;
    size_t ws_k2, ws_a, ws_r, ws_b, carried;
};

bool dispatch_geometry(int64_t T, int k, int world, int n_experts, int rpn, int groups_m, int64_t capacity,
                       DispatchGeometry *g) {
    if (T < 0 || k <= 0 || world <= 0 || rpn <= 0 || groups_m <= 0 || n_experts <= 0 || world % rpn ||
        n_experts % world || k % groups_m)
        return false;
    if (T > (((int64_t)1 << 31) - 1) / k) return false;
    g->S = T * groups_m;
    g->P = T * k;
    g->n_nodes = world / rpn;
    g->epr = n_experts / world;
    g->slots = g->epr * rpn;
    g->quota = k / groups_m;
    g->ws_k2 = align_up(k2_workspace(T, k, g->n_nodes, groups_m), 256);
    g->ws_a = align_up(k1_workspace(g->S, g->quota, rpn), 256);
    g->ws_r = align_up(regroup_workspace(g->P, g->slots, capacity), 256);
    g->ws_b = align_up(hopb_workspace(g->S, g->quota, g->slots), 256);
    g->carried = align_up((size_t)g->P * sizeof(int64_t), 256);
    return true;
}
}  // namespace

size_t terrace_dispatch_workspace(int64_t T, int k, int world, int n_experts, int rpn, int groups_m, int64_t capacity,
                                  int onepass) {
    DispatchGeometry g;
    if (!dispatch_geometry(T, k, world, n_experts, rpn, groups_m, capacity, &g)) return 256;
    return onepass ? g.ws_k2 + g.ws_b : g.ws_k2 + g.ws_a + g.ws_r + g.carried;
}

int terrace_dispatch(const void *x, const int64_t *expert_idx, const void *gates, int64_t T, int64_t row_bytes,
                     int gate_bytes, int k, int world, int n_experts, int rpn, int groups_m, int64_t capacity,
                     int onepass, void *payload, void *send_buf, void *permuted, void *planes,
                     const int64_t *plane_offsets, void *workspace, size_t workspace_bytes, terrace_stream_t stream) {
    DispatchGeometry g;
    if (!dispatch_geometry(T, k, world, n_experts, rpn, groups_m, capacity, &g) || !plane_offsets) return TERRACE_EINVAL;
    if (workspace_bytes < terrace_dispatch_workspace(T, k, world, n_experts, rpn, groups_m, capacity, onepass))
        return TERRACE_ENOSPC;
    if (!workspace || !planes) return TERRACE_EINVAL;
    auto at = [&](int which) -> void * {
        const int64_t off = plane_offsets[which];
        return off < 0 ? nullptr : (void *)((char *)planes + off);
    };
    int32_t *status = (int32_t *)at(TERRACE_DP_STATUS), *status_b = (int32_t *)at(TERRACE_DP_STATUS_HOPB);
    int32_t *status_r = (int32_t *)at(TERRACE_DP_STATUS_REGROUP);
    int64_t *pair_src = (int64_t *)at(TERRACE_DP_PAIR_SRC), *where = (int64_t *)at(TERRACE_DP_WHERE);
    if (!status || !status_b || (!onepass && !status_r) || !at(TERRACE_DP_PLACE) || !at(TERRACE_DP_TOKENS_PER_EXPERT) || (where && !pair_src))
        return TERRACE_EINVAL;
    if (!onepass && (!at(TERRACE_DP_GATE_PAIRS) || !at(TERRACE_DP_R_IDX) || !at(TERRACE_DP_SLOT_IDX) ||
                     !at(TERRACE_DP_I_SEND)))
        return TERRACE_EINVAL;
    char *ws = (char *)workspace;
    hipStream_t s = (hipStream_t)stream;
    int rc = run_k2_pack(x, expert_idx, gates, T, row_bytes, gate_bytes, k, world, n_experts, rpn, groups_m, payload,
                         (int64_t *)at(TERRACE_DP_MASK), at(TERRACE_DP_GATE_ROWS), (int64_t *)at(TERRACE_DP_U_SRC),
                         (int64_t *)at(TERRACE_DP_NODE_COUNTS), (int64_t *)at(TERRACE_DP_U_NODE),
                         (int64_t *)at(TERRACE_DP_INVERSE), (int64_t *)at(TERRACE_DP_NODE_OFFSETS),
                         (int64_t *)at(TERRACE_DP_PAIR_TABLE), (int64_t *)at(TERRACE_DP_SORT_ORDER),
                         (int64_t *)at(TERRACE_DP_TOKEN_ROWS), at(TERRACE_DP_GATE_SORTED), pair_src, where, status,
                         ws, g.ws_k2, 0, 0, 0, s);
    if (rc != TERRACE_OK) return rc;
    const int64_t n_tags = where ? g.P : 0;
    if (onepass)
        return run_hopb_scatter(payload, (const int64_t *)at(TERRACE_DP_MASK), nullptr, g.S, row_bytes, gate_bytes,
                                g.quota, 0, g.slots, capacity, permuted, nullptr, (int64_t *)at(TERRACE_DP_PLACE),
                                (uint8_t *)at(TERRACE_DP_KEPT), nullptr, (int64_t *)at(TERRACE_DP_TOKENS_PER_EXPERT),
                                (int64_t *)at(TERRACE_DP_KEPT_PER_EXPERT), where ? pair_src : nullptr, where, n_tags,
                                status_b, ws + g.ws_k2, g.ws_b, s);
    int64_t *carried = where ? (int64_t *)(ws + g.ws_k2 + g.ws_a + g.ws_r) : nullptr;
    rc = run_k1_arrival(payload, (const int64_t *)at(TERRACE_DP_MASK), at(TERRACE_DP_GATE_ROWS), g.S, row_bytes,
                        gate_bytes, g.quota, g.epr, rpn, 0, send_buf, at(TERRACE_DP_GATE_PAIRS),
                        (int64_t *)at(TERRACE_DP_R_IDX), (int64_t *)at(TERRACE_DP_SLOT_IDX),
                        (int64_t *)at(TERRACE_DP_I_SEND), (int64_t *)at(TERRACE_DP_PAIR_POS),
                        status_b, ws + g.ws_k2, g.ws_a, g.quota, g.quota, nullptr,
                        where ? pair_src : nullptr, carried, s);
    if (rc != TERRACE_OK) return rc;
    return run_regroup(send_buf, (const int64_t *)at(TERRACE_DP_SLOT_IDX), nullptr, g.P, row_bytes, gate_bytes,
                       g.slots, 0, capacity, permuted, nullptr, (int64_t *)at(TERRACE_DP_ORDER),
                       (int64_t *)at(TERRACE_DP_PLACE), (uint8_t *)at(TERRACE_DP_KEPT),
                       (int64_t *)at(TERRACE_DP_TOKENS_PER_EXPERT), (int64_t *)at(TERRACE_DP_KEPT_PER_EXPERT),
                       status_r, ws + g.ws_k2 + g.ws_a, g.ws_r, 1, 1, carried, where, n_tags, s);
}

int terrace_hopa_send_splits(const int64_t *node_counts, int world, int rpn, int my_local, int64_t *send,
                             terrace_stream_t stream) {
    if (world <= 0 || rpn <= 0 || world % rpn || my_local < 0 || my_local >= rpn || !node_counts || !send)
        return TERRACE_EINVAL;
    return launch_send_splits(node_counts, world, rpn, my_local, send, (hipStream_t)stream);
}

}  // extern "C"
