/*
 * terrace_hip.h -- C ABI of libterrace_hip.so: one rank's TerraceMoE dispatch/combine data
 * path as hand-written gfx950 (MI355X) HIP kernels.
 *
 * Every entry point
 *   - takes plain device pointers and sizes (no torch types), a caller-provided workspace
 *     where one is needed, and the HIP stream to launch on (a hipStream_t passed as void*);
 *   - only enqueues work: it never allocates, frees, synchronises or keeps a pointer, and
 *     keeps no mutable global state, so it may be called from any host thread on any stream;
 *   - returns TERRACE_OK or a negative terrace_status and never throws.
 * Outputs are allocated by the caller (the Python binding uses torch's caching allocator,
 * as the reference binding uses at::empty: terrace/ops/csrc/terrace_ops.cpp:147-160).
 *
 * Index planes are int64 and gate planes travel in the payload's storage type, exactly as
 * the reference operators return them.  Payload rows are moved as opaque bytes: `row_bytes`
 * is hidden*itemsize (or the fp8-with-scales row width); any value is accepted, rows whose
 * width and base pointers are multiples of 16 bytes take the 16-byte-per-lane path.
 *
 * `status` arguments point to TERRACE_STATUS_WORDS int32 in device memory that the call
 * overwrites: word 0 is a bit set of terrace_fault values (0 = inputs were well formed).
 * Kernels cannot raise, so malformed input is contained (ids clamped, results unspecified
 * but in range) and reported there; the caller decides when to pay the read-back, as the
 * reference's plan does on its first and every 256th call (terrace/ta2a.py:161-204).
 */
#ifndef TERRACE_HIP_H
#define TERRACE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *terrace_stream_t; /* hipStream_t */

#if defined(__GNUC__)
#define TERRACE_API __attribute__((visibility("default")))
#else
#define TERRACE_API
#endif

enum terrace_status {
    TERRACE_OK = 0,
    TERRACE_EINVAL = -22,  /* bad geometry / null pointer / unsupported size */
    TERRACE_ENOSPC = -28,  /* workspace smaller than the matching *_workspace() answer */
    TERRACE_ELAUNCH = -5,  /* the HIP runtime refused a launch (hipGetLastError != 0) */
    TERRACE_E2BIG = -7     /* input larger than the fixed scratch of terrace_k1_arrival_static */
};

enum terrace_dtype {
    TERRACE_F32 = 0,
    TERRACE_BF16 = 1,
    TERRACE_F16 = 2,
    TERRACE_FP8_E4M3_B128 = 3 /* row = hidden e4m3 codes, then hidden/128 fp32 block scales */
};

enum terrace_route_mode { /* terrace/routing.py:66 _MODES, same order */
    TERRACE_ROUTE_FULL = 0,
    TERRACE_ROUTE_GROUP_LIMITED = 1,
    TERRACE_ROUTE_QUOTA_ONLY = 2,
    TERRACE_ROUTE_GLOBAL_TOPK = 3,
    /* or-ed into `mode`: use the LDS-staged kernel even where the register-resident one
     * applies (both give identical results; this exists so tests can compare them) */
    TERRACE_ROUTE_FORCE_GENERIC = 0x100,
    /* or-ed into `mode`: `gates` is a bf16 / f16 plane and each gate is rounded to nearest-even on the way
     * out -- the cast to the payload dtype that the gate plane needs anyway (terrace/ta2a_dispatch.py:550-564),
     * without a launch of its own */
    TERRACE_ROUTE_GATES_BF16 = 0x200,
    TERRACE_ROUTE_GATES_F16 = 0x400
};

enum terrace_fault {
    TERRACE_FAULT_ID_RANGE = 1, /* an expert / slot id outside its range was clamped */
    TERRACE_FAULT_QUOTA = 2,    /* a token's run on a node does not hold exactly k/M experts */
    TERRACE_FAULT_FANOUT = 4    /* a token does not touch exactly M distinct nodes */
};

#define TERRACE_STATUS_WORDS 4

/* Rows on a pitch.  Wherever an entry point takes `row_bytes` for the payload rows it moves, the rows may sit
 * `pitch` bytes apart instead of back to back: pass TERRACE_ROW_PITCHED(width, pitch).  Every row buffer of that
 * call (source and destination alike) is then [n_rows, pitch] bytes with `width` bytes of data at the start of
 * each row; the bytes between width and pitch are never read and never written.  Requirements: width a multiple
 * of 16, pitch a multiple of 1024 and >= width, every row buffer aligned to 16 bytes (to 1024 for full speed), width
 * and pitch below 2^31; anything else is TERRACE_EINVAL.  A plain width (no pitch) means rows back to back, as in the reference.
 * Why it exists: a wave of the row movers copies one aligned kilobyte of both buffers.  Rows that are not whole
 * kilobytes (the 7392-byte fp8 row with its block scales) otherwise start at ever-shifting offsets inside a
 * kilobyte, and every copy needs a re-loaded, shifted window; on an 8192-byte pitch the same rows move like
 * kilobyte rows, at the cost of address space, not of traffic.  No counterpart in the reference. */
#define TERRACE_ROW_PITCHED(width, pitch) ((int64_t)(width) | ((int64_t)(pitch) << 32))

TERRACE_API const char *terrace_version(void);
TERRACE_API const char *terrace_strerror(int status);

/* Identity copy of nbytes; the streaming-copy roofline probe.
 * Replaces terrace::passthrough (terrace/ops/csrc/terrace_ops.cpp:230, kernel
 * terrace/ops/ascendc/op_kernel/terrace_passthrough.cpp:119). */
TERRACE_API int terrace_passthrough(const void *x, void *y, size_t nbytes, terrace_stream_t stream);

/* Stream probes beside terrace_passthrough: what the part sustains for the traffic mixes the row movers are made
 * of, in the movers' own launch shape (one-wave workgroups, 16 bytes per lane, streaming loads and stores).  The
 * benchmark times them in the run that times the movers, so every "this mover sits at its bytes' stream rate"
 * statement can be checked from one record.  No counterpart in the reference beyond its passthrough toolchain
 * probe (terrace/ops/ascendc/op_kernel/terrace_passthrough.cpp:119).
 *   TERRACE_PROBE_READ   reads nbytes from x, writes nothing (y is only named by a store that never happens when x
 *                        holds zeros)
 *   TERRACE_PROBE_WRITE  writes nbytes to y
 *   TERRACE_PROBE_SUM8   y = the fp32-accumulated sum of eight contiguous bf16 streams of nbytes each starting at x
 *                        (reads 8 * nbytes): the combine's read:write mix and arithmetic with no row ids
 *   TERRACE_PROBE_COPY   y = x, one wave per kilobyte
 * nbytes must be a multiple of 8192 and both pointers 16-byte aligned, else TERRACE_EINVAL. */
enum terrace_probe { TERRACE_PROBE_READ = 0, TERRACE_PROBE_WRITE = 1, TERRACE_PROBE_SUM8 = 2, TERRACE_PROBE_COPY = 3 };
TERRACE_API int terrace_stream_probe(int kind, const void *x, void *y, size_t nbytes, terrace_stream_t stream);

/* T-Route (terrace/routing.py:45-96).  affinity [T,E] f32, bias [E] f32, gate_affinity
 * [T,E] f32 or NULL (= affinity).  Writes expert_idx [T,k] i64, gates [T,k] f32 (bf16 / f16 with the mode flags),
 * group_idx [T,G] i64 with G = top_groups (full, group_limited), n_groups (quota_only) or
 * top_k (global_topk).  Ties go to the lowest index; gates are raw/sum(raw) with the sum
 * taken left to right in fp32.  pool = TRouteConfig.group_score_pool (>= 1): a group's score is the mean of its
 * top-min(pool, g) scores, added from the largest down in fp32 and divided once (pool 2: an exact halving). */
TERRACE_API int terrace_t_route(const float *affinity, const float *bias, const float *gate_affinity, int64_t T,
                    int n_experts, int n_groups, int top_k, int top_groups, int pool, int mode,
                    int64_t *expert_idx, void *gates, int64_t *group_idx, terrace_stream_t stream);

/* expert_load (terrace/routing.py:112-113) and fixed_hist (terrace/ta2a_fwd.py:299-321):
 * out[b] = #{i : idx[i] == b}; out is int64 [n_buckets] or, with as_float != 0, float32.  An index outside
 * [0, n_buckets) is counted nowhere and sets TERRACE_FAULT_ID_RANGE in the status block (the reference's bincount
 * would grow its result and its scatter_add_ would fail on the spot; a kernel can do neither). */
TERRACE_API size_t terrace_hist_workspace(int64_t n, int n_buckets);
TERRACE_API int terrace_hist(const int64_t *idx, int64_t n, int n_buckets, void *out, int as_float, int32_t *status,
                 void *workspace, size_t workspace_bytes, terrace_stream_t stream);

/* _stable_argsort_small (terrace/ta2a_fwd.py:324-345): order [n] i64 = stable ascending
 * argsort of key (values in [0, n_buckets)); hist [n_buckets] i64 may be NULL. */
TERRACE_API size_t terrace_argsort_small_workspace(int64_t n, int n_buckets);
TERRACE_API int terrace_argsort_small(const int64_t *key, int64_t n, int n_buckets, int64_t *order, int64_t *hist,
                          int32_t *status, void *workspace, size_t workspace_bytes,
                          terrace_stream_t stream);

/* Send side: dispatch index build + Hop-A deduplicated pack under equal quota.
 * Replaces terrace::k2_pack (terrace/ops/csrc/terrace_k2_pack.cpp:209-211; spec
 * terrace/ops/k2_ref.py:70-134) = plan_ta2a(groups_m=M) (terrace/ta2a.py:70-275)
 * + hidden[u_src] (terrace/ta2a_fwd.py:473) + _pack_quota_wire (terrace/ta2a_fwd.py:177-249).
 *   hidden [T,row_bytes] (NULL: index build only, payload ignored), expert_idx [T,k] i64,
 *   gates [T,k] elements of gate_bytes (2 or 4) bytes (NULL: gate_rows ignored).
 * Writes payload [T*M,row_bytes], mask [T*M,q] i64 ascending node-local slot ids, gate_rows
 * [T*M,q], u_src [T*M] i64, node_counts [n_nodes] i64; each of the optional planes may be
 * NULL: u_node [T*M] i64, inverse [T*k] i64 (row carrying slot (t,j)), node_offsets
 * [n_nodes] i64 (exclusive prefix of node_counts), pair_table [T,k] i64 (flat Hop-A pair id
 * row*q+i of the token's s-th smallest expert), sort_order [T,k] i64 (its column j),
 * token_rows [T,M] i64 (the token's send rows, node ascending) and gate_sorted [T,k] (the
 * token's gates in ascending expert order, gate_bytes-wide elements).
 * Rows come out in (node ascending, token ascending) order.
 * status word 1 = number of occupied (token, node) pairs, word 2 = how many of them hold other
 * than k/M experts (the two quantities the guard of terrace/ta2a.py:170-204 tests). */
TERRACE_API size_t terrace_k2_pack_workspace(int64_t T, int k, int n_nodes, int groups_m);
TERRACE_API int terrace_k2_pack(const void *hidden, const int64_t *expert_idx, const void *gates, int64_t T,
                    int64_t row_bytes, int gate_bytes, int k, int world, int n_experts, int rpn,
                    int groups_m, void *payload, int64_t *mask, void *gate_rows, int64_t *u_src,
                    int64_t *node_counts, int64_t *u_node, int64_t *inverse, int64_t *node_offsets,
                    int64_t *pair_table, int64_t *sort_order, int64_t *token_rows, void *gate_sorted,
                    int64_t *pair_src, int64_t *combine_table, int32_t *status, void *workspace,
                    size_t workspace_bytes, terrace_stream_t stream);

/* _pack_quota_wire (terrace/ta2a_fwd.py:177-249) for a caller that already holds `inverse`:
 * for the token's s-th smallest expert (column j), run m = s/q, i = s%q:
 *   slot_tab[inverse[t,j0(m)]][i] = expert % slots, gate_tab[same] = gates[t,j]
 * where j0(m) is the column of the run's first expert.  slot_tab [n_rows,q] i64 and gate_tab
 * [n_rows,q] must be zero-filled by the caller (rows never named keep slot 0 / gate 0);
 * rows outside [0, n_rows) are skipped and reported as TERRACE_FAULT_ID_RANGE. */
TERRACE_API int terrace_pack_quota_wire(const int64_t *expert_idx, const void *gates, const int64_t *inverse,
                                        int64_t T, int k, int gate_bytes, int64_t n_rows, int slots, int quota,
                                        int64_t *slot_tab, void *gate_tab, int32_t *status,
                                        terrace_stream_t stream);

/* Hop-B arrival chain.  Replaces terrace::k1_arrival (terrace/ops/csrc/terrace_ops.cpp:231-232;
 * spec terrace/ops/__init__.py:255-300; kernel terrace/ops/ascendc/op_kernel/terrace_k1_arrival.cpp).
 *   rx [R,row_bytes] (NULL: index planes only), rslot [R,quota] i64, rgate [R,quota] of
 *   gate_bytes-wide elements (NULL: gate_pairs ignored).
 * Pairs p = r*quota+i are placed in stable ascending order of rslot[p]/epr.  Writes send_buf
 * [P,row_bytes], gate_pairs [P], r_idx [P] i64, slot_idx [P] i64, i_send [rpn] i64 and, when
 * not NULL, pair_pos [P] i64 (the place pair p landed at: the inverse permutation).
 * Tags: with tags_in [P] i64 and tags_out [P] i64 both given, a caller's tag rides with each pair:
 * tags_out[place of p] = tags_in[p] (no counterpart in the reference; it lets a later stage name what it
 * placed in the caller's own terms without a look-up launch). */
TERRACE_API size_t terrace_k1_arrival_workspace(int64_t R, int quota, int rpn);
TERRACE_API int terrace_k1_arrival(const void *rx, const int64_t *rslot, const void *rgate, int64_t R,
                       int64_t row_bytes, int gate_bytes, int quota, int epr, int rpn, int my_local,
                       void *send_buf, void *gate_pairs, int64_t *r_idx, int64_t *slot_idx,
                       int64_t *i_send, int64_t *pair_pos, const int64_t *tags_in, int64_t *tags_out,
                       int32_t *status, void *workspace, size_t workspace_bytes, terrace_stream_t stream);

/* Expert-order regroup on the expert card (terrace/ta2a_fwd.py:641-646), optionally with a
 * per-expert capacity (no counterpart in the reference, which is drop-less:
 * terrace/ta2a_dispatch.py:248-250).  exp_j = my_slot - my_local*epr in [0, epr).
 *   capacity < 0: permuted [P,row_bytes] = node_rx[order], order [P] i64 stable by exp_j.
 *   capacity >= 0: permuted [epr*capacity,row_bytes], expert x keeps its first `capacity`
 *     rows in stable order at x*capacity+rank, unused rows are zero; dest [P] i64 is that
 *     place or -1 for a dropped row; kept [P] u8.
 * tokens_per_expert [epr] i64 counts before the cut; kept_per_expert [epr] i64 (may be NULL).
 * node_rx NULL: index planes only.  gate planes ride along when my_gate != NULL:
 * permuted_gate has one gate_bytes-wide element per permuted row.
 * Tags: with tags_in [P] i64 and place_by_tag [n_tags] i64 given, place_by_tag[tags_in[p]] = place of row p
 * (-1 when dropped; tags outside [0, n_tags) are skipped).  Fed with the tags terrace_k1_arrival carried from
 * terrace_k2_pack's pair_src, place_by_tag is the combine's [T,k] table (terrace_combine's idx), with no
 * look-up launch between dispatch and combine. */
TERRACE_API size_t terrace_regroup_workspace(int64_t P, int epr, int64_t capacity);
TERRACE_API int terrace_regroup(const void *node_rx, const int64_t *my_slot, const void *my_gate, int64_t P,
                    int64_t row_bytes, int gate_bytes, int epr, int my_local, int64_t capacity,
                    void *permuted, void *permuted_gate, int64_t *order, int64_t *dest, uint8_t *kept,
                    int64_t *tokens_per_expert, int64_t *kept_per_expert, const int64_t *tags_in,
                    int64_t *place_by_tag, int64_t n_tags, int32_t *status, void *workspace,
                    size_t workspace_bytes, terrace_stream_t stream);

/* Hop-B local scatter in one pass (north-star stage 4; the arrival-side chain of terrace/ta2a_fwd.py:605-646 when
 * every expert slot the arriving rows name is local to this GPU -- one GPU per node, or the one-GPU loop-back).
 * Equals terrace_k1_arrival followed by terrace_regroup(epr = n_local, my_local = 0) without the [P, row_bytes]
 * buffer between them: a stable sort by owner card and then by local expert is one stable sort by slot, so each
 * arrived row is read once and written straight to the expert-order place of each of its `quota` pairs.
 *   rx [R,row_bytes] (NULL: index planes only), rslot [R,quota] i64 with first_slot <= id < first_slot + n_local,
 *   rgate [R,quota] of gate_bytes-wide elements or NULL.
 * Pair p = r*quota+i goes to expert x = rslot[p] - first_slot; pairs of one expert keep their order in p.
 *   capacity < 0: permuted [P,row_bytes]; place[p] = position in that order.
 *   capacity >= 0: permuted [n_local*capacity,row_bytes]; expert x keeps its first `capacity` pairs at
 *     x*capacity+rank, later ones are dropped (place[p] = -1, kept[p] = 0), unused places are zero rows.
 * place [P] i64, kept [P] u8, pair_of_place [places] i64 (-1 on a padding place), permuted_gate [places] (0 on
 * padding; written when rgate != NULL) may each be NULL.  tokens_per_expert [n_local] i64 counts before the cut;
 * kept_per_expert [n_local] i64 may be NULL.  tags_in [P] / place_by_tag [n_tags] as in terrace_regroup:
 * place_by_tag[tags_in[p]] = place[p].  With rx == NULL, terrace_hopb_scatter_move moves the rows later
 * (same geometry, same untouched workspace), like the *_move calls of the other stages. */
TERRACE_API size_t terrace_hopb_scatter_workspace(int64_t R, int quota, int n_local);
TERRACE_API int terrace_hopb_scatter(const void *rx, const int64_t *rslot, const void *rgate, int64_t R,
                                     int64_t row_bytes, int gate_bytes, int quota, int first_slot, int n_local,
                                     int64_t capacity, void *permuted, void *permuted_gate, int64_t *place,
                                     uint8_t *kept, int64_t *pair_of_place, int64_t *tokens_per_expert,
                                     int64_t *kept_per_expert, const int64_t *tags_in, int64_t *place_by_tag,
                                     int64_t n_tags, int32_t *status, void *workspace, size_t workspace_bytes,
                                     terrace_stream_t stream);
TERRACE_API int terrace_hopb_scatter_move(const void *rx, int64_t R, int64_t row_bytes, int quota, int n_local,
                                          int64_t capacity, void *permuted, const void *workspace,
                                          size_t workspace_bytes, terrace_stream_t stream);

/* Row ids a caller passes to the four entry points below are never turned into an address unchecked: an id
 * outside [0, n_src) (resp. [0, n_dst), the table length) is a dead entry -- a zero row, a copy not made,
 * no contribution, -1 -- exactly like a negative one.  (The reference's x[u_src] / index_add would raise.) */

/* out[i] = src[idx[i]] for i < n_out (row gather over the n_src rows of src; a dead idx writes a zero row). */
TERRACE_API int terrace_gather_rows(const void *src, int64_t n_src, const int64_t *idx, int64_t n_out,
                                    int64_t row_bytes, void *out, terrace_stream_t stream);

/* dst[pos[r*fan + f]] = src[r] for r < n_src, f < fan (a dead pos skips that copy; dst has n_dst rows): a
 * source row is read once and written fan times.  The mover behind terrace_k2_pack (pos = token_rows)
 * and terrace_k1_arrival (pos = pair_pos); exposed so it can be driven and timed on its own. */
TERRACE_API int terrace_scatter_rows(const void *src, const int64_t *pos, int64_t n_src, int fan,
                                     int64_t row_bytes, void *dst, int64_t n_dst, terrace_stream_t stream);

/* out[i] = table[idx[i]] over int64 planes (table has n_table entries); a dead idx gives -1. */
TERRACE_API int terrace_index_chain(const int64_t *table, int64_t n_table, const int64_t *idx, int64_t n,
                                    int64_t *out, terrace_stream_t stream);

/* out[i] = outer[inner[idx[i]]], -1 propagating at either level (one launch for the two
 * look-ups that turn a token's Hop-A pair ids into places of the expert-order buffer). */
TERRACE_API int terrace_index_chain2(const int64_t *outer, int64_t n_outer, const int64_t *inner, int64_t n_inner,
                                     const int64_t *idx, int64_t n, int64_t *out, terrace_stream_t stream);

/* Gate-weighted combine (terrace/ta2a_fwd.py:658-670; one level: terrace/ep_dist.py:121-122):
 *   out[i,:] = sum_{j<fan} w[i,j] * decode(src[idx[i,j],:])      (idx outside [0, n_src) contributes nothing)
 * accumulated in fp32 as acc = fl(acc + fl(w*x)) for j = 0..fan-1, rounded once to out_dtype.
 * src rows are src_dtype (F32, BF16, F16 or FP8_E4M3_B128 with `hidden` elements per row),
 * weights [n_out,fan] are w_dtype (F32, BF16, F16) or NULL (all ones), idx is [n_out,fan] i64,
 * out is [n_out,hidden] of out_dtype (F32, BF16 or F16).  The weights plane must be 4-byte aligned; a 16-bit
 * weight is read as the aligned 32-bit word that holds it, so when n_out*fan is odd the last read covers the two
 * bytes after the plane (the same aligned word: never another page, never used). */
/* terrace_combine with the source rows `src_row_pitch` bytes apart (0: back to back, which is terrace_combine). */
TERRACE_API int terrace_combine_pitched(const void *src, int64_t n_src, int src_dtype, int64_t src_row_pitch,
                                        const int64_t *idx, const void *weights, int w_dtype, int64_t n_out, int fan,
                                        int64_t hidden, void *out, int out_dtype, terrace_stream_t stream);
TERRACE_API int terrace_combine(const void *src, int64_t n_src, int src_dtype, const int64_t *idx, const void *weights,
                    int w_dtype, int64_t n_out, int fan, int64_t hidden, void *out, int out_dtype,
                    terrace_stream_t stream);

/* The reference's TWO combine levels in one pass (terrace/ta2a_dispatch.py:483-494: a send row sums the expert outputs
 * of its pairs, a token sums its send rows, each level an fp32 index_add rounded once to the tensor dtype), for a
 * caller whose two levels run on the same GPU with no exchange between them (loop-back):
 *   out[t] = round_out( sum_m f32( round_src( sum_i f32(src[inner[outer[t, m], i]]) ) ) )
 * inner [n_rows, fan_inner] i64 names source rows (fan_inner = 1, 2, 4 or 8), outer [n_out, fan_outer] i64 names rows
 * of inner; entries outside their range are skipped.  Bit for bit terrace_combine(src, inner) into the source dtype
 * followed by terrace_combine(that, outer), without the [n_rows, hidden] plane between them.  src f32 / bf16 / f16,
 * rows 16-byte multiples on 16-byte-aligned buffers; anything else returns TERRACE_EINVAL (run the two levels). */
TERRACE_API int terrace_combine_two_level(const void *src, int64_t n_src, int src_dtype, const int64_t *inner,
                                          int64_t n_rows, int fan_inner, const int64_t *outer, int64_t n_out,
                                          int fan_outer, int64_t hidden, void *out, int out_dtype,
                                          terrace_stream_t stream);

/* Wire containers (terrace/ta2a_pack.py:319-336 hopa_pack, :398-414 hopa_pack_small, :474-497
 * hopb_pack_meta): each out row of row_bytes is plane a's row, then b's, then c's, then zeros.
 * A NULL plane is absent (its width counts as 0).  Pure byte moves.
 *   Hop-A full:  a = ids [n, id_w] i64, b = payload [n, H], c = gates [n, gw]; row = W*8 bytes
 *   Hop-A small: a = ids, b = gates;  Hop-B meta: a = slot ids [P] i64, b = gates [P]; row = 16 */
TERRACE_API int terrace_pack_planes(const void *a, int64_t a_bytes, const void *b, int64_t b_bytes, const void *c,
                                    int64_t c_bytes, int64_t n_rows, int64_t row_bytes, void *out,
                                    terrace_stream_t stream);

/* The inverse (hopa_unpack :339-356, hopa_unpack_small :417-423, hopb_unpack_meta :500-503): row
 * bytes [0, a_bytes) go to a, the next b_bytes to b, the next c_bytes to c; each destination is a
 * dense plane of its own (never a view of the container); a NULL destination is skipped. */
TERRACE_API int terrace_unpack_planes(const void *packed, int64_t row_bytes, int64_t n_rows, void *a,
                                      int64_t a_bytes, void *b, int64_t b_bytes, void *c, int64_t c_bytes,
                                      terrace_stream_t stream);

/* ---- the stage operators in two phases: index planes first, rows later ----
 * The reference ships counts and metadata ahead of the payload so that the receiving side's index work
 * overlaps the row traffic (terrace/ta2a_dispatch.py:78-100 and :399-412, the "async counts" path).  Here:
 * terrace_k2_pack with hidden == NULL and payload == NULL, terrace_k1_arrival[_wire] with rx == NULL and
 * send_buf == NULL, and terrace_regroup[_wire] with node_rx == NULL and permuted == NULL write every index
 * plane and leave the row mover's int32 position plane in the workspace.  The *_move call below then moves
 * the rows -- on any stream that is ordered after the first phase -- reading that plane; its geometry
 * arguments must repeat the first phase's and the workspace must be the same untouched buffer.
 * n_nodes = world / rpn.  terrace_regroup_move also writes the zero padding rows of a capacity layout. */
TERRACE_API int terrace_k2_pack_move(const void *hidden, int64_t T, int64_t row_bytes, int k, int n_nodes,
                                     int groups_m, void *payload, const void *workspace, size_t workspace_bytes,
                                     terrace_stream_t stream);
TERRACE_API int terrace_k1_arrival_move(const void *rx, int64_t R, int64_t row_bytes, int quota, int rpn,
                                        void *send_buf, const void *workspace, size_t workspace_bytes,
                                        terrace_stream_t stream);
TERRACE_API int terrace_regroup_move(const void *node_rx, int64_t P, int64_t row_bytes, int epr, int64_t capacity,
                                     void *permuted, const void *workspace, size_t workspace_bytes,
                                     terrace_stream_t stream);

/* ---- zero-copy wire containers: the three stage kernels write / read the containers themselves ----
 * (the follow-up terrace/ta2a_pack.py:462-466 asks for; layouts as terrace_pack_planes above)
 *
 * terrace_k2_pack_wire = terrace_k2_pack, but the slot-id and gate planes are written straight into the
 * Hop-A small container wire [T*M, wire_words] i64: words [0,q) of a row are its ascending slot ids, the
 * gates follow from word q, the rest of the row is zeroed (wire_words >= q + ceil(q*gate_bytes/8)).
 * terrace_k1_arrival_wire = terrace_k1_arrival reading that container as it arrived (rwire) and writing the
 * Hop-B container meta [P, 2] i64 (word 0 slot id, word 1 the gate then zeros); slot_idx / gate_pairs are
 * optional extra outputs.  terrace_regroup_wire = terrace_regroup reading my_slot / my_gate out of an
 * arrived Hop-B container my_meta [P, 2] (the gate plane is gathered only when permuted_gate != NULL). */
TERRACE_API int terrace_k2_pack_wire(const void *hidden, const int64_t *expert_idx, const void *gates, int64_t T,
                                     int64_t row_bytes, int gate_bytes, int k, int world, int n_experts, int rpn,
                                     int groups_m, void *payload, int64_t *wire, int wire_words, int64_t *u_src,
                                     int64_t *node_counts, int64_t *u_node, int64_t *inverse, int64_t *node_offsets,
                                     int64_t *pair_table, int64_t *sort_order, int64_t *token_rows, void *gate_sorted,
                                     int32_t *status, void *workspace, size_t workspace_bytes, terrace_stream_t stream);
TERRACE_API int terrace_k1_arrival_wire(const void *rx, const int64_t *rwire, int wire_words, int64_t R,
                                        int64_t row_bytes, int gate_bytes, int quota, int epr, int rpn, int my_local,
                                        void *send_buf, int64_t *meta, int64_t *r_idx, int64_t *slot_idx,
                                        void *gate_pairs, int64_t *i_send, int64_t *pair_pos, int32_t *status,
                                        void *workspace, size_t workspace_bytes, terrace_stream_t stream);
TERRACE_API int terrace_regroup_wire(const void *node_rx, const int64_t *my_meta, int64_t P, int64_t row_bytes,
                                     int gate_bytes, int epr, int my_local, int64_t capacity, void *permuted,
                                     void *permuted_gate, int64_t *order, int64_t *dest, uint8_t *kept,
                                     int64_t *tokens_per_expert, int64_t *kept_per_expert, int32_t *status,
                                     void *workspace, size_t workspace_bytes, terrace_stream_t stream);

/* ---- the general (data-dependent fan-out) branch and the seam's entry helper ---- */

/* plan_ta2a without groups_m (terrace/ta2a.py:70-275, general branch): one send row per occupied
 * (node, token) pair in (node asc, token asc) order, for any n_nodes up to 2048.  u_src / u_node must hold
 * T*min(k, n_nodes) entries; the number actually written is sum(counts), which the caller reads
 * back (the reference pays the same synchronisation at terrace/ta2a.py:148). */
TERRACE_API size_t terrace_plan_general_workspace(int64_t T, int k, int n_nodes);
TERRACE_API int terrace_plan_general(const int64_t *expert_idx, int64_t T, int k, int world, int n_experts, int rpn,
                                     int64_t *u_src, int64_t *u_node, int64_t *counts, int64_t *inverse,
                                     int32_t *status, void *workspace, size_t workspace_bytes,
                                     terrace_stream_t stream);

/* build_expansion (terrace/ta2a_fwd.py:348-442): mask[inverse[i]] |= 1 << (expert_idx[i] % slots) for
 * i < n = T*k.  mask [n_rows] i64 must be zero-filled by the caller; slots <= 63. */
TERRACE_API int terrace_build_mask(const int64_t *expert_idx, const int64_t *inverse, int64_t n, int slots,
                                   int64_t n_rows, int64_t *mask, int32_t *status, terrace_stream_t stream);

/* out[rows[i]*width + c] = vals[i] (elements of elem_bytes = 2 or 4) with c = cols[i], or cols[i] % col_mod
 * when col_mod > 0: the sparse gate plane gate_rows[inverse, expert % slots] = gates of
 * terrace/ta2a_fwd.py:498-500.  out is pre-filled by the caller; cells outside it are skipped. */
TERRACE_API int terrace_scatter_elems(const void *vals, int elem_bytes, const int64_t *rows, const int64_t *cols,
                                      int col_mod, int64_t n, int64_t n_rows, int width, void *out,
                                      terrace_stream_t stream);

/* _expand_arrival (terrace/ta2a_fwd.py:120-174).  With a quota: per row its `quota` lowest set bits
 * ascending, then, if it has fewer, its unset columns ascending; r_idx / slot_idx hold R*quota.
 * Without: every set bit, row-major with columns ascending; _count leaves the exclusive offsets in
 * the workspace and the pair total in n_pairs (device int64, read back by the caller), _fill then
 * writes the n_pairs entries. */
TERRACE_API int terrace_expand_mask_quota(const int64_t *rmask, int64_t R, int slots, int quota, int64_t *r_idx,
                                          int64_t *slot_idx, terrace_stream_t stream);
TERRACE_API size_t terrace_expand_mask_workspace(int64_t R);
TERRACE_API int terrace_expand_mask_count(const int64_t *rmask, int64_t R, int slots, int64_t *n_pairs,
                                          void *workspace, size_t workspace_bytes, terrace_stream_t stream);
TERRACE_API int terrace_expand_mask_fill(const int64_t *rmask, int64_t R, int slots, int64_t *r_idx,
                                         int64_t *slot_idx, const void *workspace, terrace_stream_t stream);

/* The arrival chain of the general branch (terrace/ta2a_fwd.py:605-628): the P pairs (r_in[p], slot_in[p])
 * that terrace_expand_mask_* listed are placed in stable ascending order of slot/epr.  Writes r_idx [P],
 * slot_idx [P], i_send [rpn], ordo [P] (the source pair of each place; may be NULL), send_buf [P,row_bytes]
 * = rx[r_idx] (rx NULL: index planes only) and gate_pairs [P] = rgate[r_idx, slot_idx] looked up in the
 * sparse plane rgate [R, gate_width] (NULL: skipped). */
TERRACE_API size_t terrace_arrival_pairs_workspace(int64_t P, int rpn);
TERRACE_API int terrace_arrival_pairs(const void *rx, const int64_t *r_in, const int64_t *slot_in, const void *rgate,
                                      int64_t R, int64_t P, int64_t row_bytes, int gate_bytes, int gate_width, int epr,
                                      int rpn, void *send_buf, void *gate_pairs, int64_t *r_idx, int64_t *slot_idx,
                                      int64_t *i_send, int64_t *ordo, int32_t *status, void *workspace,
                                      size_t workspace_bytes, terrace_stream_t stream);

/* The read side of an index_add (red.index_add_(0, r_idx, ret) and y.index_add(0, u_src, back),
 * terrace/ta2a_dispatch.py:483-494) when the number of contributions per target varies: table
 * [n_seg, width] i64 lists, for each target s, the items i < n with seg[i] == s in ascending i, padded
 * with -1 (width <= 64).  terrace_combine over that table is then the reduction, adding in the same
 * ascending order.  A target with more than `width` items raises TERRACE_FAULT_FANOUT in status word 0. */
TERRACE_API size_t terrace_segment_table_workspace(int64_t n_seg);
TERRACE_API int terrace_segment_table(const int64_t *seg, int64_t n, int64_t n_seg, int width, int64_t *table,
                                      int32_t *status, void *workspace, size_t workspace_bytes,
                                      terrace_stream_t stream);

/* The tables the adjoints of ta2a_permute / ta2a_unpermute read (terrace/ta2a_dispatch.py:263-498): for every
 * place i < P of the expert-order buffer, behind it arrival row a = order[i], send row r = r_idx[a], token
 * t = u_src[r] and expert e = u_node[r]*slots + slot_idx[a]:  token_of_place[i] = t (may be NULL) and
 * where[t, j] = i for the column j with expert_idx[t, j] == e.  where [T,k] is first filled with -1. */
TERRACE_API int terrace_pair_places(const int64_t *order, const int64_t *r_idx, const int64_t *slot_idx,
                                    const int64_t *u_src, const int64_t *u_node, const int64_t *expert_idx, int64_t P,
                                    int64_t T, int k, int slots, int64_t n_rows, int64_t *where,
                                    int64_t *token_of_place, int32_t *status, terrace_stream_t stream);

/* routing_map_to_topk (terrace/ta2a_dispatch.py:224-260): routing_map [T,E] bytes (non-zero = chosen).
 * _count writes row_stats = {min, max} of the per-token counts (int32[2]); after the caller has
 * checked min == max == k, _topk writes the k chosen expert ids ascending and their probs
 * (elem_bytes-wide elements of probs [T,E]). */
TERRACE_API int terrace_routing_map_count(const void *routing_map, int64_t T, int n_experts, int32_t *row_stats,
                                          terrace_stream_t stream);
TERRACE_API int terrace_routing_map_topk(const void *routing_map, const void *probs, int elem_bytes, int64_t T,
                                         int n_experts, int k, int64_t *expert_idx, void *gates,
                                         terrace_stream_t stream);

/* Hop-A counts exchange buffer (terrace/ta2a_dispatch.py:197-211): send [world] i64 is zero
 * except send[n*rpn + my_local] = node_counts[n]. */
TERRACE_API int terrace_hopa_send_splits(const int64_t *node_counts, int world, int rpn, int my_local,
                             int64_t *send, terrace_stream_t stream);

/* ---- the whole dispatch in one call ----
 * terrace_k2_pack, then terrace_k1_arrival and terrace_regroup on the rank's own send buffers (the exchanges of
 * terrace/ta2a_fwd.py:471-646 looped back: every slot of the node counts as local, my_local = 0), or -- `onepass`
 * -- terrace_hopb_scatter in place of those two.  Same kernels, same planes bit for bit; what it saves is host
 * time: one call, one workspace, and the small planes addressed as offsets into ONE caller buffer, so a binding
 * computes the table of offsets once per geometry and passes two pointers per step.
 *   plane_offsets[TERRACE_DP_PLANES]: byte offset of each plane from `planes`, or -1 for a plane the caller does
 *   not want.  Required: MASK, U_SRC, NODE_COUNTS, PLACE, TOKENS_PER_EXPERT, STATUS, STATUS_HOPB, GATE_ROWS when
 *   gates is given, and in the two-step form GATE_PAIRS, R_IDX, SLOT_IDX, I_SEND, STATUS_REGROUP.  WHERE (the
 *   combine's [T, k] place table, filled through the pairs' tags) needs PAIR_SRC.  Shapes and dtypes are those of
 *   the same-named arguments of the three stage entry points; the three STATUS planes are 4 int32 each (pack;
 *   arrival or one-pass Hop B; regroup).
 *   capacity < 0: drop-less.  send_buf is not used with `onepass`.
 *   workspace: terrace_dispatch_workspace(...) bytes (it also holds the tags carried between the two sorts). */
enum terrace_dispatch_plane {
    TERRACE_DP_MASK = 0,
    TERRACE_DP_GATE_ROWS,
    TERRACE_DP_U_SRC,
    TERRACE_DP_NODE_COUNTS,
    TERRACE_DP_U_NODE,
    TERRACE_DP_INVERSE,
    TERRACE_DP_NODE_OFFSETS,
    TERRACE_DP_PAIR_TABLE,
    TERRACE_DP_SORT_ORDER,
    TERRACE_DP_TOKEN_ROWS,
    TERRACE_DP_GATE_SORTED,
    TERRACE_DP_PAIR_SRC,
    TERRACE_DP_WHERE,
    TERRACE_DP_STATUS,
    TERRACE_DP_GATE_PAIRS,
    TERRACE_DP_R_IDX,
    TERRACE_DP_SLOT_IDX,
    TERRACE_DP_I_SEND,
    TERRACE_DP_PAIR_POS,
    TERRACE_DP_STATUS_HOPB,
    TERRACE_DP_ORDER,
    TERRACE_DP_PLACE,
    TERRACE_DP_KEPT,
    TERRACE_DP_TOKENS_PER_EXPERT,
    TERRACE_DP_KEPT_PER_EXPERT,
    TERRACE_DP_STATUS_REGROUP,
    TERRACE_DP_PLANES
};
TERRACE_API size_t terrace_dispatch_workspace(int64_t T, int k, int world, int n_experts, int rpn, int groups_m,
                                              int64_t capacity, int onepass);
TERRACE_API int terrace_dispatch(const void *x, const int64_t *expert_idx, const void *gates, int64_t T,
                                 int64_t row_bytes, int gate_bytes, int k, int world, int n_experts, int rpn,
                                 int groups_m, int64_t capacity, int onepass, void *payload, void *send_buf,
                                 void *permuted, void *planes, const int64_t *plane_offsets, void *workspace,
                                 size_t workspace_bytes, terrace_stream_t stream);

/* ---- the entry point that brings its own scratch memory ----
 * No counterpart in the reference.  It is for callers that cannot allocate device memory at all -- code under
 * HIP graph capture, serving loops that must stay off the allocator, harnesses that forbid hipMalloc -- and so
 * cannot provide the workspace terrace_k1_arrival asks for.  terrace_k1_arrival_static is terrace_k1_arrival
 * (its arguments without the tags and the workspace, same outputs, same kernels) with the workspace taken from a device array of
 * TERRACE_STATIC_SCRATCH_BYTES that is part of the library image: every GPU the library runs on holds that
 * array until the process ends.  Inputs whose workspace would not fit (terrace_k1_arrival_workspace(R, quota,
 * rpn) > terrace_static_scratch_bytes(); about 900 thousand pairs) are refused with TERRACE_E2BIG.  The call
 * allocates and frees nothing.  Unlike the rest of the library it is not reentrant: all calls on one GPU use
 * that GPU's one array, so two of them must not overlap (same stream, or ordered by events).  The device the
 * stream belongs to must be current.
 *
 * The first call on a device looks the array's device address up (hipGetSymbolAddress, a runtime call that takes
 * a lock and may load the code object).  That must not happen under stream capture: call terrace_static_init()
 * once per device beforehand, with that device current (it does only the look-up, launches nothing and is
 * idempotent), or make one eager call first.  Every later call on that device is kernel launches only. */
#define TERRACE_STATIC_SCRATCH_BYTES (4u << 20)
TERRACE_API size_t terrace_static_scratch_bytes(void);
TERRACE_API int terrace_static_init(void);
TERRACE_API int terrace_k1_arrival_static(const void *rx, const int64_t *rslot, const void *rgate, int64_t R,
                                          int64_t row_bytes, int gate_bytes, int quota, int epr, int rpn,
                                          int my_local, void *send_buf, void *gate_pairs, int64_t *r_idx,
                                          int64_t *slot_idx, int64_t *i_send, int64_t *pair_pos, int32_t *status,
                                          terrace_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TERRACE_HIP_H */
