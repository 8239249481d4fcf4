/*
 * C restatement of the dispatch/combine path, threaded with OpenMP.
 *
 * TEST INFRASTRUCTURE, NOT PRODUCT: it is the multi-core CPU baseline that bench.py times next
 * to the GPU figures, and a second checker.  It is pinned by tests/test_oracle_c.py, which
 * requires bit-equality with the numpy oracle (oracle/terrace_oracle.py) -- itself pinned
 * against the reference's literals, library routines and brute force -- on every function.
 * Nothing in the shipped package links or loads it.
 *
 * Conventions (same as the numpy oracle): top-k ties go to the lowest index; the gate
 * normaliser is summed left to right in fp32; the combine accumulates fl(acc + fl(w*x)) in
 * fp32 in table order and rounds once.  Citations name the reference source each function
 * follows (paths relative to the reference tree).
 *
 * Build: gcc -O3 -march=native -fopenmp -ffp-contract=off -shared -fPIC (see oracle/build_c.py).
 */
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define API __attribute__((visibility("default")))

/* ---- terrace/routing.py:86-95, mode "full" -------------------------------------------- */
static int ahead(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

API void orc_route_full(const float *aff, const float *bias, const float *gate_aff, int64_t T, int E, int n_groups,
                        int k, int M, int pool, int64_t *expert_idx, float *gates, int64_t *group_idx) {
    const int g = E / n_groups, q = k / M;
#pragma omp parallel
    {
        float *s = (float *)malloc(sizeof(float) * (size_t)E);
        float *score = (float *)malloc(sizeof(float) * (size_t)n_groups);
        char *gtaken = (char *)malloc((size_t)n_groups);
        char *etaken = (char *)malloc((size_t)g);
#pragma omp for schedule(static)
        for (int64_t t = 0; t < T; ++t) {
            const float *row = aff + t * E;
            for (int e = 0; e < E; ++e) s[e] = row[e] + bias[e];
            for (int G = 0; G < n_groups; ++G) {
                float a1 = -INFINITY, a2 = -INFINITY;
                for (int x = 0; x < g; ++x) {
                    const float v = s[G * g + x];
                    if (v > a1) { a2 = a1; a1 = v; } else if (v > a2) { a2 = v; }
                }
                score[G] = (pool >= 2 && g >= 2) ? (a1 + a2) * 0.5f : a1;
                gtaken[G] = 0;
            }
            for (int m = 0; m < M; ++m) {
                int best = -1;
                for (int G = 0; G < n_groups; ++G)
                    if (!gtaken[G] && (best < 0 || ahead(score[G], G, score[best], best))) best = G;
                gtaken[best] = 1;
                group_idx[t * M + m] = best;
                memset(etaken, 0, (size_t)g);
                for (int i = 0; i < q; ++i) {
                    int bx = -1;
                    for (int x = 0; x < g; ++x)
                        if (!etaken[x] && (bx < 0 || ahead(s[best * g + x], x, s[best * g + bx], bx))) bx = x;
                    etaken[bx] = 1;
                    expert_idx[t * k + m * q + i] = (int64_t)best * g + bx;
                }
            }
            const float *grow = (gate_aff ? gate_aff : aff) + t * E;
            float den = 0.0f;
            for (int j = 0; j < k; ++j) den = j == 0 ? grow[expert_idx[t * k]] : den + grow[expert_idx[t * k + j]];
            for (int j = 0; j < k; ++j) gates[t * k + j] = grow[expert_idx[t * k + j]] / den;
        }
        free(s); free(score); free(gtaken); free(etaken);
    }
}

/* ---- terrace/ta2a.py:70-275 + terrace/ta2a_fwd.py:177-249,473 (= terrace/ops/k2_ref.py:70-134) ----
 * Equal-quota send side.  Returns 0, or 1 when the routing is not M nodes x k/M experts. */
API int orc_k2_pack(const uint8_t *hidden, const int64_t *expert_idx, const uint8_t *gates, int64_t T,
                    int64_t row_bytes, int gate_bytes, int k, int world, int n_experts, int rpn, int M,
                    uint8_t *payload, int64_t *mask, uint8_t *gate_rows, int64_t *u_src, int64_t *counts,
                    int64_t *u_node, int64_t *inverse, int64_t *pair_table, int64_t *sort_order) {
    const int slots = (n_experts / world) * rpn, n_nodes = world / rpn, q = k / M;
    int64_t *cursor = (int64_t *)calloc((size_t)n_nodes + 1, sizeof(int64_t));
    int64_t *row_of = (int64_t *)malloc(sizeof(int64_t) * (size_t)T * (size_t)M);    /* [T, M] rows, node ascending */
    int bad = 0;
    for (int n = 0; n < n_nodes; ++n) counts[n] = 0;
    /* pass 1: occupancy counts per node */
    for (int64_t t = 0; t < T && !bad; ++t) {
        int seen_nodes = 0;
        for (int j = 0; j < k; ++j) {
            const int64_t e = expert_idx[t * k + j];
            if (e < 0 || e >= n_experts) { bad = 1; break; }
            const int n = (int)(e / slots);
            int first = 1, same = 0;
            for (int i = 0; i < k; ++i) {
                if (expert_idx[t * k + i] / slots == n) { same++; if (i < j) first = 0; }
            }
            if (first) { counts[n]++; seen_nodes++; if (same != q) bad = 1; }
        }
        if (seen_nodes != M) bad = 1;
    }
    if (bad) { free(cursor); free(row_of); return 1; }
    for (int n = 0; n < n_nodes; ++n) cursor[n + 1] = cursor[n] + counts[n];
    /* pass 2: rows in (node, token) order; per token its rows in ascending node order */
    for (int64_t t = 0; t < T; ++t) {
        int order[64];
        for (int j = 0; j < k; ++j) {            /* ascending rank of each id inside the row */
            int r = 0;
            for (int i = 0; i < k; ++i) r += expert_idx[t * k + i] < expert_idx[t * k + j];
            order[r] = j;
        }
        for (int m = 0; m < M; ++m) {
            const int n = (int)(expert_idx[t * k + order[m * q]] / slots);
            const int64_t r = cursor[n]++;
            row_of[t * M + m] = r;
            u_src[r] = t;
            if (u_node) u_node[r] = n;
            for (int i = 0; i < q; ++i) {
                const int j = order[m * q + i];
                mask[r * q + i] = expert_idx[t * k + j] % slots;
                memcpy(gate_rows + (r * q + i) * gate_bytes, gates + (t * k + j) * gate_bytes, (size_t)gate_bytes);
                if (inverse) inverse[t * k + j] = r;
                if (pair_table) pair_table[t * k + m * q + i] = r * q + i;
                if (sort_order) sort_order[t * k + m * q + i] = j;
            }
        }
    }
    if (hidden) {
#pragma omp parallel for schedule(static)
        for (int64_t t = 0; t < T; ++t)
            for (int m = 0; m < M; ++m)
                memcpy(payload + row_of[t * M + m] * row_bytes, hidden + t * row_bytes, (size_t)row_bytes);
    }
    free(cursor); free(row_of);
    return 0;
}

/* ---- terrace/ops/__init__.py:255-300 ----------------------------------------------------- */
API void orc_k1_arrival(const uint8_t *rx, const int64_t *rslot, const uint8_t *rgate, int64_t R, int64_t row_bytes,
                        int gate_bytes, int quota, int epr, int rpn, uint8_t *send_buf, uint8_t *gate_pairs,
                        int64_t *r_idx, int64_t *slot_idx, int64_t *i_send, int64_t *pair_pos) {
    const int64_t P = R * quota;
    int64_t *cursor = (int64_t *)calloc((size_t)rpn + 1, sizeof(int64_t));
    for (int b = 0; b < rpn; ++b) i_send[b] = 0;
    for (int64_t p = 0; p < P; ++p) i_send[rslot[p] / epr]++;
    for (int b = 0; b < rpn; ++b) cursor[b + 1] = cursor[b] + i_send[b];
    for (int64_t p = 0; p < P; ++p) {
        const int64_t d = cursor[rslot[p] / epr]++;
        r_idx[d] = p / quota;
        slot_idx[d] = rslot[p];
        memcpy(gate_pairs + d * gate_bytes, rgate + p * gate_bytes, (size_t)gate_bytes);
        pair_pos[p] = d;
    }
    if (rx) {
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < R; ++r)
            for (int i = 0; i < quota; ++i)
                memcpy(send_buf + pair_pos[r * quota + i] * row_bytes, rx + r * row_bytes, (size_t)row_bytes);
    }
    free(cursor);
}

/* ---- terrace/ta2a_fwd.py:641-646, plus the capacity cut (own definition) ------------------ */
API void orc_regroup(const uint8_t *node_rx, const int64_t *my_slot, int64_t P, int64_t row_bytes, int epr,
                     int my_local, int64_t capacity, uint8_t *permuted, int64_t *place, uint8_t *kept,
                     int64_t *tokens_per_expert) {
    int64_t *cursor = (int64_t *)calloc((size_t)epr + 1, sizeof(int64_t));
    for (int x = 0; x < epr; ++x) tokens_per_expert[x] = 0;
    for (int64_t p = 0; p < P; ++p) tokens_per_expert[my_slot[p] - (int64_t)my_local * epr]++;
    for (int x = 0; x < epr; ++x) cursor[x + 1] = cursor[x] + tokens_per_expert[x];
    int64_t *rank_start = (int64_t *)malloc(sizeof(int64_t) * ((size_t)epr + 1));
    memcpy(rank_start, cursor, sizeof(int64_t) * ((size_t)epr + 1));
    for (int64_t p = 0; p < P; ++p) {
        const int64_t x = my_slot[p] - (int64_t)my_local * epr;
        const int64_t d = cursor[x]++;
        if (capacity < 0) {
            place[p] = d;
            if (kept) kept[p] = 1;
        } else {
            const int64_t rank = d - rank_start[x];
            const int keep = rank < capacity;
            place[p] = keep ? x * capacity + rank : -1;
            if (kept) kept[p] = (uint8_t)keep;
        }
    }
    if (node_rx) {
        if (capacity >= 0) memset(permuted, 0, (size_t)epr * (size_t)capacity * (size_t)row_bytes);
#pragma omp parallel for schedule(static)
        for (int64_t p = 0; p < P; ++p)
            if (place[p] >= 0) memcpy(permuted + place[p] * row_bytes, node_rx + p * row_bytes, (size_t)row_bytes);
    }
    free(cursor); free(rank_start);
}

/* ---- terrace/ta2a_fwd.py:658-670 (fused; one level: terrace/ep_dist.py:121-122) ------------ */
static float bf16_to_f32(uint16_t b) { uint32_t u = (uint32_t)b << 16; float f; memcpy(&f, &u, 4); return f; }
static uint16_t f32_to_bf16(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
static float e4m3_to_f32(uint8_t c) {
    const int e = (c >> 3) & 0xF, m = c & 7;
    float v;
    if (e == 0xF && m == 7) v = NAN;
    else if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return (c & 0x80) ? -v : v;
}

/* src_fmt / out_fmt: 0 f32, 1 bf16, 3 fp8 rows (hidden e4m3 codes + hidden/128 fp32 scales) */
API void orc_combine(const uint8_t *src, int src_fmt, const int64_t *idx, const float *w, int64_t n_out, int fan,
                     int64_t hidden, uint8_t *out, int out_fmt) {
    const int64_t srow = src_fmt == 0 ? hidden * 4 : (src_fmt == 1 ? hidden * 2 : hidden + 4 * (hidden / 128));
    float lut[256];
    for (int c = 0; c < 256; ++c) lut[c] = e4m3_to_f32((uint8_t)c);
#pragma omp parallel
    {
        float *acc = (float *)malloc(sizeof(float) * (size_t)hidden);
#pragma omp for schedule(static)
        for (int64_t t = 0; t < n_out; ++t) {
            for (int64_t h = 0; h < hidden; ++h) acc[h] = 0.0f;
            for (int j = 0; j < fan; ++j) {
                const int64_t from = idx[t * fan + j];
                if (from < 0) continue;
                const float wj = w ? w[t * fan + j] : 1.0f;
                const uint8_t *row = src + from * srow;
                if (src_fmt == 0) {
                    const float *r = (const float *)row;
                    for (int64_t h = 0; h < hidden; ++h) acc[h] = acc[h] + (w ? r[h] * wj : r[h]);
                } else if (src_fmt == 1) {
                    const uint16_t *r = (const uint16_t *)row;
                    for (int64_t h = 0; h < hidden; ++h) {
                        const float x = bf16_to_f32(r[h]);
                        acc[h] = acc[h] + (w ? x * wj : x);
                    }
                } else {
                    const float *scale = (const float *)(row + hidden);
                    for (int64_t h = 0; h < hidden; ++h) {
                        const float x = lut[row[h]] * scale[h / 128];
                        acc[h] = acc[h] + (w ? x * wj : x);
                    }
                }
            }
            if (out_fmt == 0) memcpy(out + t * hidden * 4, acc, (size_t)hidden * 4);
            else {
                uint16_t *o = (uint16_t *)(out + t * hidden * 2);
                for (int64_t h = 0; h < hidden; ++h) o[h] = f32_to_bf16(acc[h]);
            }
        }
        free(acc);
    }
}

API int orc_threads(void) {
    int n = 1;
#pragma omp parallel
    {
#pragma omp master
        n = omp_get_num_threads();
    }
    return n;
}
