// T-Route: group-limited top-k with equal per-group quota, a token's scores spread over the lanes of
// a wavefront.
//
// Selection order everywhere is the strict total order (value descending, index ascending):
// "the next pick" is the largest candidate strictly after the previous pick in that order, so
// no taken-flags are needed and ties always go to the lowest index.
//
//   route_wave_kernel     mode "full" when a token's E (padded) scores map onto 8..64 lanes as VPL
//                         consecutive values per lane and every group covers a power-of-two number
//                         of whole lanes; up to 8 tokens share a wave.  Scores never leave
//                         registers: group top-2 by a DPP butterfly inside the group's lanes, top-M
//                         groups by rank counting (or a butterfly across groups), then all M
//                         selected groups pick their q experts at once.
//   route_generic_kernel  every mode and every geometry; scores staged in wave-private LDS.
//
// Both write expert_idx / group_idx as int64 and gates = raw / (raw_0 + raw_1 + ... ) with the
// sum taken left to right in fp32 (terrace/routing.py:94-95).
#include "common.hpp"

#include <math.h>

namespace terrace {

constexpr float kNegInf = -INFINITY;
constexpr float kPosInf = INFINITY;

// (v, i) strictly after (pv, pi) in (value desc, index asc) order
__device__ __forceinline__ bool after(float v, int i, float pv, int pi) { return v < pv || (v == pv && i > pi); }
// (v, i) ahead of (bv, bi)
__device__ __forceinline__ bool ahead(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

// One butterfly step of a symmetric wave reduction at distance D.  Distances 4 and 8 use the
// DPP half-row / row mirrors, which pair a lane with one whose lower bits differ as well; that
// is the same reduction because every caller reduces at distances D/2, D/4, ... first (or the
// lanes below D already agree), so all lanes of the mirrored sub-row hold one value.
template <int D>
__device__ __forceinline__ int bfly_i(int v) {
    if constexpr (D == 1) return __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xF, 0xF, false);
    else if constexpr (D == 2) return __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xF, 0xF, false);
    else if constexpr (D == 4) return __builtin_amdgcn_update_dpp(v, v, 0x141, 0xF, 0xF, false);
    else if constexpr (D == 8) return __builtin_amdgcn_update_dpp(v, v, 0x140, 0xF, 0xF, false);
    else if constexpr (D == 16) return __builtin_amdgcn_ds_swizzle(v, 0x401F);
    else return __shfl_xor(v, 32, kWave);
}
template <int D>
__device__ __forceinline__ float bfly_f(float v) { return __int_as_float(bfly_i<D>(__float_as_int(v))); }

template <int D>
__device__ __forceinline__ void top2_step(float &a1, float &a2) {
    const float b1 = bfly_f<D>(a1), b2 = bfly_f<D>(a2);
    const float hi = fmaxf(a1, b1), lo = fminf(a1, b1);
    a2 = fmaxf(lo, fmaxf(a2, b2));
    a1 = hi;
}

template <int D>
__device__ __forceinline__ void best_step(float &v, int &i) {
    const float ov = bfly_f<D>(v);
    const int oi = bfly_i<D>(i);
    if (ahead(ov, oi, v, i)) {
        v = ov;
        i = oi;
    }
}

// Reduce over lane distances [FROM, TO): powers of two, known at compile time.
template <int FROM, int TO>
__device__ __forceinline__ void top2_range(float &a1, float &a2) {
    if constexpr (FROM <= 1 && TO > 1) top2_step<1>(a1, a2);
    if constexpr (FROM <= 2 && TO > 2) top2_step<2>(a1, a2);
    if constexpr (FROM <= 4 && TO > 4) top2_step<4>(a1, a2);
    if constexpr (FROM <= 8 && TO > 8) top2_step<8>(a1, a2);
    if constexpr (FROM <= 16 && TO > 16) top2_step<16>(a1, a2);
    if constexpr (FROM <= 32 && TO > 32) top2_step<32>(a1, a2);
}
template <int FROM, int TO>
__device__ __forceinline__ void best_range(float &v, int &i) {
    if constexpr (FROM <= 1 && TO > 1) best_step<1>(v, i);
    if constexpr (FROM <= 2 && TO > 2) best_step<2>(v, i);
    if constexpr (FROM <= 4 && TO > 4) best_step<4>(v, i);
    if constexpr (FROM <= 8 && TO > 8) best_step<8>(v, i);
    if constexpr (FROM <= 16 && TO > 16) best_step<16>(v, i);
    if constexpr (FROM <= 32 && TO > 32) best_step<32>(v, i);
}

// Shared epilogue of the generic kernel: sel[0..k) holds the chosen expert ids (wave-private LDS).
// An id outside [0, E) can only come from NaN scores (never ranked); it is clamped to 0.
// A gate goes out as fp32, or rounded to nearest-even to the 16-bit type the payload is in (what the caller's
// `gates.to(payload dtype)` would do in a launch of its own).
__device__ __forceinline__ void store_gate(void *gates, int gate_dtype, int64_t at, float v) {
    if (gate_dtype == TERRACE_F32) ((float *)gates)[at] = v;
    else if (gate_dtype == TERRACE_BF16) ((uint16_t *)gates)[at] = (uint16_t)f32_to_bf16_bits(v);
    else ((uint16_t *)gates)[at] = __half_as_ushort(__float2half_rn(v));
}

__device__ __forceinline__ void write_token(int *sel, float *raw, const float *gate_row, int k, int E, int64_t t,
                                            int64_t *expert_idx, void *gates, int gate_dtype) {
    const int lane = lane_id();
    for (int j = lane; j < k; j += kWave) {
        if ((unsigned)sel[j] >= (unsigned)E) sel[j] = 0;
        raw[j] = gate_row[sel[j]];
    }
    __builtin_amdgcn_wave_barrier();
    float den = 0.0f;
    for (int j = 0; j < k; ++j) den = j == 0 ? ((volatile float *)raw)[0] : __fadd_rn(den, ((volatile float *)raw)[j]);
    for (int j = lane; j < k; j += kWave) {
        expert_idx[t * k + j] = sel[j];
        store_gate(gates, gate_dtype, t * k + j, __fdiv_rn(((volatile float *)raw)[j], den));
    }
}

// ---------------------------------------------------------------------------------------------
// register-resident kernel, mode "full"
// ---------------------------------------------------------------------------------------------
// A wave holds TPW tokens side by side: LPT = 64/TPW lanes per token, VPL consecutive scores per lane,
// LPG lanes per group (g = VPL*LPG), LPT/LPG group positions per token, so short rows (E = 64, 128)
// fill the wave with 4 or 2 tokens instead of leaving lanes idle.  The kernel is bound by its vector
// instruction count (about 330 per token at E = 256, k = 8), not by the row it reads.  The token's row of gate values sits in registers beside its scores, so
// the lane that owns a chosen expert hands over the raw gate itself and nothing is re-read from memory
// after the selection.
template <int VPL, int LPG, int TPW>
__global__ __launch_bounds__(kBlock) void route_wave_kernel(const float *__restrict__ affinity,
                                                            const float *__restrict__ bias,
                                                            const float *__restrict__ gate_affinity, int64_t T, int E,
                                                            int k, int M, int pool,
                                                            int64_t *__restrict__ expert_idx,
                                                            void *__restrict__ gates, int gate_dtype,
                                                            int64_t *__restrict__ group_idx) {
    extern __shared__ int32_t lds[];
    constexpr int LPT = kWave / TPW;
    constexpr int g = VPL * LPG;
    constexpr int kGroupSlots = LPT / LPG;
    static_assert(LPG <= LPT, "a group cannot span more lanes than a token has");
    const int lane = lane_id();
    const int w = wave_in_block();
    const int tl = lane & (LPT - 1);             // lane within the token
    const int slot = lane / LPT;                 // which of the wave's tokens
    const int lane0 = lane - tl;                 // the token's first lane
    lds_i32 *sel = (lds_i32 *)lds + (w * TPW + slot) * 2 * k;   // per token: k chosen ids, then their k raw gates
    lds_f32 *raw = (lds_f32 *)(sel + k);
    const int q = k / M;
    const int my_group = tl / LPG;
    float b[VPL];
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int e = tl * VPL + i;
        b[i] = e < E ? bias[e] : 0.0f;
    }
    auto load_row = [&](const float *row, float *v) {
        if (E == LPT * VPL) {
            if constexpr (VPL == 1) {
                v[0] = row[tl];
            } else if constexpr (VPL <= 4) {
                typedef float fvec __attribute__((ext_vector_type(VPL)));
                const fvec x = *(const fvec *)(row + tl * VPL);
#pragma unroll
                for (int i = 0; i < VPL; ++i) v[i] = x[i];
            } else {
                typedef float f4 __attribute__((ext_vector_type(4)));
#pragma unroll
                for (int c = 0; c < VPL / 4; ++c) {
                    const f4 x = *(const f4 *)(row + tl * VPL + 4 * c);
#pragma unroll
                    for (int i = 0; i < 4; ++i) v[4 * c + i] = x[i];
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                const int e = tl * VPL + i;
                v[i] = e < E ? row[e] : 0.0f;
            }
        }
    };
    // value held by lane `src` of this token's lanes
    auto from_lane_f = [&](float v, int src) {
        if constexpr (TPW == 1) return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
        else return __shfl(v, lane0 + src, kWave);
    };
    auto from_lane_i = [&](int v, int src) {
        if constexpr (TPW == 1) return __builtin_amdgcn_readlane(v, src);
        else return __shfl(v, lane0 + src, kWave);
    };
    const int64_t stride = (int64_t)gridDim.x * kWavesPerBlock * TPW;
    for (int64_t t0 = ((int64_t)blockIdx.x * kWavesPerBlock + w) * TPW; t0 < T; t0 += stride) {
        const int64_t t = t0 + slot;
        const bool live = t < T;
        const int64_t tt = live ? t : T - 1;     // a dead slot recomputes the last token and stores nothing
        float a[VPL], ga[VPL], s[VPL];
        load_row(affinity + tt * E, a);
        if (gate_affinity) load_row(gate_affinity + tt * E, ga);
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const int e = tl * VPL + i;
            s[i] = e < E ? __fadd_rn(a[i], b[i]) : kNegInf;
            if (!gate_affinity) ga[i] = a[i];
        }
        if (tl < k) sel[tl] = -1;
        __builtin_amdgcn_wave_barrier();
        // group score: mean of the top two (or the top one) of the group's g values
        float a1 = kNegInf, a2 = kNegInf;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const float v = s[i];
            a2 = fmaxf(fminf(a1, v), a2);
            a1 = fmaxf(a1, v);
        }
        top2_range<1, LPG>(a1, a2);
        const bool real_group = my_group * g < E;
        float score = (pool >= 2 && g >= 2) ? __fmul_rn(__fadd_rn(a1, a2), 0.5f) : a1;
        if (!real_group) score = kNegInf;
        const int gid = real_group ? my_group : 0x7FFFFFFF;
        // top-M groups
        int my_rank = -1;
        if constexpr (kGroupSlots <= 16) {
            // few groups: every lane reads each group's score from that group's first lane and counts
            // the groups ahead of its own; a NaN score is ahead of nothing and behind nothing
            int ahead_of_me = 0;
#pragma unroll
            for (int G = 0; G < kGroupSlots; ++G) {
                const float sg = from_lane_f(score, G * LPG);
                const int ig = from_lane_i(gid, G * LPG);
                ahead_of_me += ahead(sg, ig, score, gid) ? 1 : 0;
            }
            if (real_group && ahead_of_me < M && score == score) my_rank = ahead_of_me;
            const bool files = (tl & (LPG - 1)) == 0 && my_rank >= 0;
            if (files && live) group_idx[t * M + my_rank] = gid;
            uint64_t filed = __ballot(files) >> lane0;
            if constexpr (LPT < kWave) filed &= (1ull << LPT) - 1ull;
            const int n_filed = __popcll(filed);
            if (n_filed < M && tl >= n_filed && tl < M && live) group_idx[t * M + tl] = 0x7FFFFFFF;   // NaN scores only
        } else {
            float pv = kPosInf;
            int pi = -1;
            for (int m = 0; m < M; ++m) {
                float cv = kNegInf;
                int ci = 0x7FFFFFFF;
                if (real_group && after(score, gid, pv, pi)) {
                    cv = score;
                    ci = gid;
                }
                best_range<LPG, LPT>(cv, ci);
                if (real_group && ci == gid) my_rank = m;
                pv = cv;
                pi = ci;
                if (tl == 0 && live) group_idx[t * M + m] = ci;
            }
        }
        // every selected group picks its q experts, all groups at once; the owner lane of a pick
        // files the id and its raw gate under the group's rank
        float ev = kPosInf;
        int ei = -1;
        for (int i = 0; i < q; ++i) {
            float cv = kNegInf;
            int ci = 0x7FFFFFFF;
#pragma unroll
            for (int x = 0; x < VPL; ++x) {
                const int e = tl * VPL + x;
                if (e < E && after(s[x], e, ev, ei) && ahead(s[x], e, cv, ci)) {
                    cv = s[x];
                    ci = e;
                }
            }
            best_range<1, LPG>(cv, ci);
            ev = cv;
            ei = ci;
            if (my_rank >= 0 && (unsigned)(ci - tl * VPL) < (unsigned)VPL) {
                float mine = ga[0];
#pragma unroll
                for (int x = 1; x < VPL; ++x)
                    if (ci - tl * VPL == x) mine = ga[x];
                sel[my_rank * q + i] = ci;
                raw[my_rank * q + i] = mine;
            }
        }
        __builtin_amdgcn_wave_barrier();
        // slots nobody filed (NaN scores are never picked): expert 0 and its gate
        if (tl < k && sel[tl] < 0) {
            sel[tl] = 0;
            raw[tl] = (gate_affinity ? gate_affinity : affinity)[tt * E];
        }
        __builtin_amdgcn_wave_barrier();
        // lane j of the token takes pick j into registers (one LDS round trip); the left-to-right sum of the
        // raw gates then reads lane after lane instead of walking LDS k times, one dependent load after the other
        const int my_pick = tl < k ? sel[tl] : 0;
        const float my_raw = tl < k ? raw[tl] : 0.0f;
        float den = from_lane_f(my_raw, 0);
        for (int j = 1; j < k; ++j) den = __fadd_rn(den, from_lane_f(my_raw, j));
        if (tl < k && live) {
            expert_idx[t * k + tl] = my_pick;
            store_gate(gates, gate_dtype, t * k + tl, __fdiv_rn(my_raw, den));
        }
        __builtin_amdgcn_wave_barrier();
    }
}

// ---------------------------------------------------------------------------------------------
// generic kernel: all modes, scores in wave-private LDS
// ---------------------------------------------------------------------------------------------
// Wave-wide best of per-lane candidates.
__device__ __forceinline__ void wave_best(float &v, int &i) {
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const float ov = __shfl_xor(v, d, kWave);
        const int oi = __shfl_xor(i, d, kWave);
        if (ahead(ov, oi, v, i)) {
            v = ov;
            i = oi;
        }
    }
}

__global__ __launch_bounds__(kBlock) void route_generic_kernel(const float *__restrict__ affinity,
                                                               const float *__restrict__ bias,
                                                               const float *__restrict__ gate_affinity, int64_t T,
                                                               int E, int n_groups, int k, int M, int pool, int mode,
                                                               int n_group_out, int64_t *__restrict__ expert_idx,
                                                               void *__restrict__ gates, int gate_dtype,
                                                               int64_t *__restrict__ group_idx) {
    extern __shared__ int32_t lds[];
    const int lane = lane_id();
    const int w = wave_in_block();
    const int g = E / n_groups;
    const int per_wave = E + n_groups + 2 * k + n_groups;
    volatile float *s = (volatile float *)(lds + w * per_wave);
    volatile float *gsc = s + E;
    int *sel = (int *)(gsc + n_groups);
    float *raw = (float *)(sel + k);
    volatile int *selg = (volatile int *)(raw + k);
    for (int64_t t = (int64_t)blockIdx.x * kWavesPerBlock + w; t < T; t += (int64_t)gridDim.x * kWavesPerBlock) {
        const float *row = affinity + t * E;
        for (int e = lane; e < E; e += kWave) s[e] = __fadd_rn(row[e], bias[e]);
        __builtin_amdgcn_wave_barrier();
        int n_sel_groups = 0, per_group = 0;
        if (mode == TERRACE_ROUTE_FULL || mode == TERRACE_ROUTE_GROUP_LIMITED) {
            for (int G = lane; G < n_groups; G += kWave) {
                const int p = pool < g ? pool : g;                     // mean of the top-min(pool, g)
                if (p <= 2) {
                    float a1 = kNegInf, a2 = kNegInf;
                    for (int x = 0; x < g; ++x) {
                        const float v = s[G * g + x];
                        a2 = fmaxf(fminf(a1, v), a2);
                        a1 = fmaxf(a1, v);
                    }
                    gsc[G] = p == 2 ? __fmul_rn(__fadd_rn(a1, a2), 0.5f) : a1;
                } else {
                    // the p largest, one after the other in (value desc, index asc) order, added from the
                    // largest down and divided once: fl(fl(..fl(v1 + v2).. + vp) / p)
                    float acc = 0.0f, pv = kPosInf;
                    int pi = -1;
                    for (int i = 0; i < p; ++i) {
                        float cv = kNegInf;
                        int ci = 0x7FFFFFFF;
                        for (int x = 0; x < g; ++x) {
                            const float v = s[G * g + x];
                            if (after(v, x, pv, pi) && ahead(v, x, cv, ci)) {
                                cv = v;
                                ci = x;
                            }
                        }
                        acc = i == 0 ? cv : __fadd_rn(acc, cv);
                        pv = cv;
                        pi = ci;
                    }
                    gsc[G] = __fdiv_rn(acc, (float)p);
                }
            }
            __builtin_amdgcn_wave_barrier();
            float pv = kPosInf;
            int pi = -1;
            for (int m = 0; m < M; ++m) {
                float cv = kNegInf;
                int ci = 0x7FFFFFFF;
                for (int G = lane; G < n_groups; G += kWave) {
                    const float v = gsc[G];
                    if (after(v, G, pv, pi) && ahead(v, G, cv, ci)) {
                        cv = v;
                        ci = G;
                    }
                }
                wave_best(cv, ci);
                pv = cv;
                pi = ci;
                if (lane == 0) selg[m] = ci;
            }
            n_sel_groups = M;
            per_group = k / M;
        } else if (mode == TERRACE_ROUTE_QUOTA_ONLY) {
            for (int G = lane; G < n_groups; G += kWave) selg[G] = G;
            n_sel_groups = n_groups;
            per_group = k / n_groups;
        }
        __builtin_amdgcn_wave_barrier();
        if (mode == TERRACE_ROUTE_FULL || mode == TERRACE_ROUTE_QUOTA_ONLY) {
            for (int m = 0; m < n_sel_groups; ++m) {
                const int G = selg[m];
                if ((unsigned)G >= (unsigned)n_groups) {      // a rank no group took (NaN group scores): no scores to
                    for (int i = lane; i < per_group; i += kWave) sel[m * per_group + i] = 0x7FFFFFFF;   // read
                    continue;
                }
                float pv = kPosInf;
                int pi = -1;
                for (int i = 0; i < per_group; ++i) {
                    float cv = kNegInf;
                    int ci = 0x7FFFFFFF;
                    for (int x = lane; x < g; x += kWave) {
                        const float v = s[G * g + x];
                        if (after(v, x, pv, pi) && ahead(v, x, cv, ci)) {
                            cv = v;
                            ci = x;
                        }
                    }
                    wave_best(cv, ci);
                    pv = cv;
                    pi = ci;
                    if (lane == 0) sel[m * per_group + i] = ci == 0x7FFFFFFF ? 0x7FFFFFFF : G * g + ci;
                }
            }
            for (int m = lane; m < n_sel_groups; m += kWave) group_idx[t * n_group_out + m] = selg[m];
        } else if (mode == TERRACE_ROUTE_GROUP_LIMITED) {
            // free top-k over the M*g candidates; ties by candidate position (group rank first)
            float pv = kPosInf;
            int pi = -1;
            for (int j = 0; j < k; ++j) {
                float cv = kNegInf;
                int ci = 0x7FFFFFFF;
                for (int c = lane; c < M * g; c += kWave) {
                    const int G = selg[c / g];
                    if ((unsigned)G >= (unsigned)n_groups) continue;     // a rank no group took (NaN group scores)
                    const float v = s[G * g + c % g];
                    if (after(v, c, pv, pi) && ahead(v, c, cv, ci)) {
                        cv = v;
                        ci = c;
                    }
                }
                wave_best(cv, ci);
                pv = cv;
                pi = ci;
                // no candidate left (NaN scores are never ranked): an id no expert has, which the epilogue turns
                // into expert 0 as in the other modes -- and no read of selg[] at a position that does not exist
                if (lane == 0) sel[j] = ci == 0x7FFFFFFF ? 0x7FFFFFFF : selg[ci / g] * g + ci % g;
            }
            for (int m = lane; m < M; m += kWave) group_idx[t * n_group_out + m] = selg[m];
        } else {
            float pv = kPosInf;
            int pi = -1;
            for (int j = 0; j < k; ++j) {
                float cv = kNegInf;
                int ci = 0x7FFFFFFF;
                for (int e = lane; e < E; e += kWave) {
                    const float v = s[e];
                    if (after(v, e, pv, pi) && ahead(v, e, cv, ci)) {
                        cv = v;
                        ci = e;
                    }
                }
                wave_best(cv, ci);
                pv = cv;
                pi = ci;
                if (lane == 0) {
                    sel[j] = ci;
                    group_idx[t * n_group_out + j] = ci == 0x7FFFFFFF ? 0x7FFFFFFF : ci / g;   // nothing ranked: no group
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
        write_token(sel, raw, (gate_affinity ? gate_affinity : affinity) + t * E, k, E, t, expert_idx, gates, gate_dtype);
        __builtin_amdgcn_wave_barrier();
    }
}

// ---------------------------------------------------------------------------------------------
static bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

int run_t_route(const float *affinity, const float *bias, const float *gate_affinity, int64_t T, int E, int n_groups,
                int k, int M, int pool, int mode, int64_t *expert_idx, void *gates, int gate_dtype,
                int64_t *group_idx, int force_generic, hipStream_t s) {
    if (T < 0 || E <= 0 || n_groups <= 0 || k <= 0 || M <= 0 || pool < 1 || mode < 0 || mode > 3 ||
        (gate_dtype != TERRACE_F32 && gate_dtype != TERRACE_BF16 && gate_dtype != TERRACE_F16))
        return TERRACE_EINVAL;
    if (E % n_groups || k % M || k > E || E > 2048 || M > n_groups) return TERRACE_EINVAL;
    const int g = E / n_groups;
    if ((mode == TERRACE_ROUTE_FULL && k / M > g) || (mode == TERRACE_ROUTE_GROUP_LIMITED && k > M * g) ||
        (mode == TERRACE_ROUTE_QUOTA_ONLY && (k % n_groups || k / n_groups > g)))
        return TERRACE_EINVAL;
    if (T == 0) return TERRACE_OK;
    if (!affinity || !bias || !expert_idx || !gates || !group_idx) return TERRACE_EINVAL;
    // Register-resident form.  VPL = 4 (one 16-byte load per lane) measured best wherever it fits
    // (E = 256: 14.2 us for 16384 tokens against 16.0 at VPL 8 and 16.6 at VPL 16); smaller VPL serve
    // groups of fewer than 4 experts, larger ones rows too long for 64 lanes of 4.  VPL must divide g
    // into a power-of-two number of lanes and leave the token k lanes for its outputs.
    const bool aligned = (((uintptr_t)affinity) & 15) == 0 && (!gate_affinity || (((uintptr_t)gate_affinity) & 15) == 0);
    // the register-resident form keeps a group's top two only; a wider pool takes the LDS-staged kernel
    if (!force_generic && mode == TERRACE_ROUTE_FULL && (pool <= 2 || g <= 2)) {
        static const int kVplOrder[] = {4, 2, 1, 8, 16};
        for (int vpl : kVplOrder) {
            if (g % vpl || !is_pow2(g / vpl)) continue;
            const int lpg = g / vpl;
            int lpt = 8;                                     // at most 8 tokens share a wave
            while (lpt < lpg || lpt * vpl < E || lpt < k) lpt *= 2;
            if (lpt > kWave) continue;
            if (E == lpt * vpl && vpl > 1 && !aligned) continue;     // vector loads need 16-byte rows
            const int tpw = kWave / lpt;
            const int64_t waves = (T + tpw - 1) / tpw;
            int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
            if (blocks > ((int64_t)1 << 24)) blocks = (int64_t)1 << 24;
            const size_t lds = (size_t)kWavesPerBlock * tpw * 2 * k * sizeof(int32_t);
#define TERRACE_ROUTE(V, L, W)                                                                                  \
    route_wave_kernel<V, L, W><<<(int)blocks, kBlock, lds, s>>>(affinity, bias, gate_affinity, T, E, k, M, pool, \
                                                                expert_idx, gates, gate_dtype, group_idx)
#define TERRACE_ROUTE_W(V, L)                                \
    switch (tpw) {                                           \
        case 1: TERRACE_ROUTE(V, L, 1); break;               \
        case 2: if constexpr (L <= 32) TERRACE_ROUTE(V, L, 2); break; \
        case 4: if constexpr (L <= 16) TERRACE_ROUTE(V, L, 4); break; \
        default: if constexpr (L <= 8) TERRACE_ROUTE(V, L, 8); break; \
    }
#define TERRACE_ROUTE_L(V)                              \
    switch (lpg) {                                      \
        case 1: TERRACE_ROUTE_W(V, 1); break;           \
        case 2: TERRACE_ROUTE_W(V, 2); break;           \
        case 4: TERRACE_ROUTE_W(V, 4); break;           \
        case 8: TERRACE_ROUTE_W(V, 8); break;           \
        case 16: TERRACE_ROUTE_W(V, 16); break;         \
        case 32: TERRACE_ROUTE_W(V, 32); break;         \
        default: TERRACE_ROUTE_W(V, 64); break;         \
    }
            switch (vpl) {
                case 16: TERRACE_ROUTE_L(16); break;
                case 8: TERRACE_ROUTE_L(8); break;
                case 4: TERRACE_ROUTE_L(4); break;
                case 2: TERRACE_ROUTE_L(2); break;
                default: TERRACE_ROUTE_L(1); break;
            }
#undef TERRACE_ROUTE_L
#undef TERRACE_ROUTE_W
#undef TERRACE_ROUTE
            return check_launch();
        }
    }
    int64_t blocks = (T + kWavesPerBlock - 1) / kWavesPerBlock;      // generic form: one token per wave
    if (blocks > ((int64_t)1 << 24)) blocks = (int64_t)1 << 24;
    const int n_group_out = mode == TERRACE_ROUTE_QUOTA_ONLY ? n_groups : (mode == TERRACE_ROUTE_GLOBAL_TOPK ? k : M);
    const size_t lds = (size_t)kWavesPerBlock * (E + 2 * n_groups + 2 * k) * sizeof(int32_t);
    route_generic_kernel<<<(int)blocks, kBlock, lds, s>>>(affinity, bias, gate_affinity, T, E, n_groups, k, M, pool,
                                                          mode, n_group_out, expert_idx, gates, gate_dtype, group_idx);
    return check_launch();
}

}  // namespace terrace
