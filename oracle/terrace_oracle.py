"""CPU oracle for one rank's TerraceMoE dispatch/combine path (numpy only).

TEST INFRASTRUCTURE, NOT PRODUCT.  Only the test-suite, the smoke check and the
benchmark's ``cpu_baseline`` leg may import this module, and only as the checker.
The shipped path (the ``terrace`` package) never touches it and raises when the HIP
library is missing.

Every function restates, from its closed form, what the reference computes; the
citation after each name is the reference source (relative to the reference tree)
the restatement follows.  Nothing here imports or executes the reference.

Conventions fixed by this build where the reference leaves a library behaviour open
("parity unpinned" against the reference for exactly these points, pinned against
mathematics instead):

  * top-k ties: the lowest index wins (``torch.topk`` leaves tie order unspecified,
    terrace/ta2a_fwd.py:137-153 warns about it);
  * ``gates.sum(-1)`` (terrace/routing.py:95): fp32, left to right over the k columns;
  * combine: fp32 accumulate, ``acc = fl(acc + fl(w*x))`` in the order the index table
    lists the rows, one rounding to the output dtype at the end (the reference rounds
    to the payload dtype after every ``index_add``, terrace/ta2a_fwd.py:661-670);
  * capacity padding and the fp8-with-scales row are not in the reference at all
    (terrace/ta2a_dispatch.py:248-250 is drop-less); their specification is the
    docstring of ``regroup`` / ``fp8_*`` below.

Payload rows are opaque to every dispatch stage (pure byte moves), so 16-bit and 8-bit
formats travel as ``uint16`` / ``uint8`` arrays; only ``combine`` decodes them.
"""
from __future__ import annotations

import math

import numpy as np

MODES = ("full", "group_limited", "quota_only", "global_topk")

# --------------------------------------------------------------------------------------
# number formats
# --------------------------------------------------------------------------------------


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    """bfloat16 bit patterns (uint16) -> float32 (exact: bf16 is the top half of fp32)."""
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns, round to nearest even (NaN kept quiet)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    rounded = ((u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)).astype(np.uint16)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    return np.where(nan, ((u >> np.uint32(16)) | np.uint32(0x0040)).astype(np.uint16), rounded)


def f16_to_f32(bits: np.ndarray) -> np.ndarray:
    return bits.view(np.float16).astype(np.float32)


def f32_to_f16(x: np.ndarray) -> np.ndarray:
    return np.asarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def _e4m3_table() -> np.ndarray:
    """All 256 values of fp8 e4m3 'fn' (bias 7, no infinities, 0x7f/0xff = NaN)."""
    t = np.zeros(256, dtype=np.float32)
    for b in range(256):
        s = -1.0 if b & 0x80 else 1.0
        e = (b >> 3) & 0xF
        m = b & 0x7
        if e == 0xF and m == 0x7:
            v = float("nan")
        elif e == 0:
            v = s * (m / 8.0) * 2.0 ** (-6)
        else:
            v = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
        t[b] = v
    return t


E4M3 = _e4m3_table()
E4M3_MAX = 448.0
FP8_BLOCK = 128


def f32_to_e4m3(x: np.ndarray) -> np.ndarray:
    """float32 -> e4m3fn codes, round to nearest even, saturating at +-448."""
    x = np.asarray(x, dtype=np.float32)
    pos = E4M3[:0x7F].astype(np.float64)            # 127 non-negative finite values, ascending
    a = np.minimum(np.abs(x).astype(np.float64), E4M3_MAX)
    hi = np.searchsorted(pos, a, side="left").clip(0, 126)
    lo = np.maximum(hi - 1, 0)
    dlo, dhi = a - pos[lo], pos[hi] - a
    pick_hi = (dhi < dlo) | ((dhi == dlo) & ((hi & 1) == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    return np.where(np.signbit(x), code | np.uint8(0x80), code).astype(np.uint8)


def fp8_row_bytes(hidden: int) -> int:
    return hidden + 4 * (hidden // FP8_BLOCK)


def fp8_quantise_rows(x: np.ndarray) -> np.ndarray:
    """[n, H] float32 -> [n, H + 4*H/128] uint8 rows: H e4m3 codes, then H/128 fp32 scales.

    Own specification (no counterpart in the reference): per 128-element block
    ``scale = max|x| / 448`` (1.0 for an all-zero block), ``code = e4m3(x / scale)``.
    """
    n, hidden = x.shape
    assert hidden % FP8_BLOCK == 0
    xb = np.asarray(x, dtype=np.float32).reshape(n, hidden // FP8_BLOCK, FP8_BLOCK)
    amax = np.abs(xb).max(-1)
    scale = np.where(amax > 0, amax / np.float32(E4M3_MAX), np.float32(1.0)).astype(np.float32)
    codes = f32_to_e4m3((xb / scale[..., None]).astype(np.float32)).reshape(n, hidden)
    out = np.empty((n, fp8_row_bytes(hidden)), dtype=np.uint8)
    out[:, :hidden] = codes
    out[:, hidden:] = scale.view(np.uint8).reshape(n, -1)
    return out


def fp8_dequantise_rows(rows: np.ndarray, hidden: int) -> np.ndarray:
    """Inverse view of ``fp8_quantise_rows``: value = fl32(E4M3[code] * scale[block])."""
    n = rows.shape[0]
    vals = E4M3[rows[:, :hidden]].reshape(n, hidden // FP8_BLOCK, FP8_BLOCK)
    scale = np.ascontiguousarray(rows[:, hidden:]).view(np.float32).reshape(n, -1)
    return (vals * scale[..., None]).astype(np.float32).reshape(n, hidden)


def decode_rows(rows: np.ndarray, fmt: str, hidden: int | None = None) -> np.ndarray:
    """Payload rows -> float32 for the combine.  fmt: f32 | bf16 | f16 | fp8."""
    if fmt == "f32":
        return np.asarray(rows, dtype=np.float32)
    if fmt == "bf16":
        return bf16_to_f32(rows)
    if fmt == "f16":
        return f16_to_f32(rows)
    if fmt == "fp8":
        return fp8_dequantise_rows(rows, hidden)
    raise ValueError(f"unknown row format {fmt!r}")


def encode_rows(x: np.ndarray, fmt: str) -> np.ndarray:
    if fmt == "f32":
        return np.asarray(x, dtype=np.float32)
    if fmt == "bf16":
        return f32_to_bf16(x)
    if fmt == "f16":
        return f32_to_f16(x)
    raise ValueError(f"unknown output format {fmt!r}")


# --------------------------------------------------------------------------------------
# (1) T-Route -- terrace/routing.py:20-96
# --------------------------------------------------------------------------------------


def check_route_config(n_experts: int, n_groups: int, top_k: int, top_groups: int) -> None:
    """TRouteConfig.__post_init__ (terrace/routing.py:28-34)."""
    if n_experts % n_groups:
        raise ValueError("n_experts must divide evenly into n_groups")
    if top_k % top_groups:
        raise ValueError("top_k must divide evenly into top_groups")
    if top_k // top_groups > n_experts // n_groups:
        raise ValueError("per-group quota exceeds group size")


def _topk_desc(x: np.ndarray, n: int) -> np.ndarray:
    """Indices of the n largest along the last axis, descending, lowest index first on ties."""
    return np.argsort(-x, axis=-1, kind="stable")[..., :n]


def _group_scores(sg: np.ndarray, pool: int) -> np.ndarray:
    """Mean of the top-``min(pool, g)`` entries of each group (terrace/routing.py:88).

    For pool 2 the value is fl((a+b)/2): one fp32 add and an exact halving, independent of
    any tie order.  For pool > 2 the top values are added from the largest down.
    """
    p = min(pool, sg.shape[-1])
    top = -np.sort(-sg, axis=-1)[..., :p]
    acc = top[..., 0].astype(np.float32)
    for i in range(1, p):
        acc = (acc + top[..., i]).astype(np.float32)
    return (acc / np.float32(p)).astype(np.float32)


def t_route(affinity, bias, n_experts, n_groups, top_k, top_groups, pool=2, mode="full",
            gate_affinity=None):
    """(expert_idx [T,k] i64, gates [T,k] f32, group_idx [T,M or N_g or k] i64).

    terrace/routing.py:45-96.  ``gate_affinity`` (extension, default = ``affinity``) is the
    table the gate values are read from, so a harness can select on logits and weigh by a
    softmax numerator; selection never looks at it.
    """
    if mode not in MODES:
        raise ValueError(f"unknown routing mode {mode!r}; expected one of {MODES}")
    check_route_config(n_experts, n_groups, top_k, top_groups)
    aff = np.asarray(affinity, dtype=np.float32)
    T = aff.shape[0]
    g = n_experts // n_groups
    s = (aff + np.asarray(bias, dtype=np.float32)).astype(np.float32)       # :70
    sg = s.reshape(T, n_groups, g)
    if mode == "global_topk":                                                # :72-74
        expert_idx = _topk_desc(s, top_k)
        group_idx = expert_idx // g
    elif mode == "quota_only":                                               # :75-76, :99-109
        per = top_k // n_groups
        if per < 1:
            raise ValueError(f"quota_only needs top_k ({top_k}) divisible by n_groups "
                             f"({n_groups}); got {per} experts/group")
        local = _topk_desc(sg, per)
        expert_idx = (np.arange(n_groups)[None, :, None] * g + local).reshape(T, -1)
        group_idx = np.broadcast_to(np.arange(n_groups)[None], (T, n_groups)).copy()
    elif mode == "group_limited":                                            # :77-85
        group_idx = _topk_desc(_group_scores(sg, pool), top_groups)
        cand = np.take_along_axis(sg, group_idx[..., None], axis=1).reshape(T, -1)
        local = _topk_desc(cand, top_k)
        expert_idx = np.take_along_axis(group_idx, local // g, axis=1) * g + local % g
    else:                                                                    # :86-92
        q = top_k // top_groups
        group_idx = _topk_desc(_group_scores(sg, pool), top_groups)
        picked = np.take_along_axis(sg, group_idx[..., None], axis=1)        # [T, M, g]
        local = _topk_desc(picked, q)
        expert_idx = (group_idx[..., None] * g + local).reshape(T, top_k)
    expert_idx = expert_idx.astype(np.int64)
    src = aff if gate_affinity is None else np.asarray(gate_affinity, dtype=np.float32)
    raw = np.take_along_axis(src, expert_idx, axis=1)                        # :94
    den = raw[:, 0].astype(np.float32)
    for j in range(1, raw.shape[1]):
        den = (den + raw[:, j]).astype(np.float32)
    gates = (raw / den[:, None]).astype(np.float32)                          # :95
    return expert_idx, gates, group_idx.astype(np.int64)


def expert_load(expert_idx, n_experts):
    """terrace/routing.py:112-113 -- per-expert pick counts as float32."""
    return np.bincount(np.asarray(expert_idx).reshape(-1), minlength=n_experts).astype(np.float32)


def update_bias(bias, load, gamma):
    """terrace/routing.py:116-121 -- bias += gamma * sign(mean(load) - load), fp32."""
    load = np.asarray(load, dtype=np.float32)
    err = (load.mean(dtype=np.float32) - load).astype(np.float32)
    return (np.asarray(bias, np.float32) + np.float32(gamma) * np.sign(err)).astype(np.float32)


# --------------------------------------------------------------------------------------
# (2) index build -- terrace/ta2a.py:70-275, terrace/ta2a_fwd.py:299-345
# --------------------------------------------------------------------------------------


def fixed_hist(idx, n_buckets):
    """terrace/ta2a_fwd.py:299-321 -- fixed-length int64 histogram; out-of-range raises."""
    idx = np.asarray(idx, dtype=np.int64).reshape(-1)
    if idx.size and (idx.min() < 0 or idx.max() >= n_buckets):
        raise IndexError("fixed_hist: index out of range")
    return np.bincount(idx, minlength=n_buckets).astype(np.int64)


def stable_argsort_small(key, n_buckets):
    """terrace/ta2a_fwd.py:324-345 -- stable ascending argsort of a small-range key."""
    return np.argsort(np.asarray(key, dtype=np.int64).reshape(-1), kind="stable").astype(np.int64)


def plan_ta2a(expert_idx, world, n_experts, rpn=8, groups_m=None):
    """(u_src [S], u_node [S], counts [n_nodes], inverse [T*k]), all int64.

    terrace/ta2a.py:70-275.  Send rows are the occupied (node, token) pairs in
    (node ascending, token ascending) order (:136-137, :228-230); ``inverse`` names, for
    each (token, expert) slot, the row that carries it (:251-253).  With ``groups_m`` the
    fan-out / divisibility / equal-quota guard of :161-204 is applied on every call (the
    reference applies it on the first and every 256th).
    """
    e = np.asarray(expert_idx, dtype=np.int64)
    T, k = e.shape
    epr = n_experts // world
    n_nodes = world // rpn
    if n_nodes * T >= (1 << 24):                                             # :106
        raise ValueError(f"plan_ta2a float32 key range exceeded: n_nodes*T = {n_nodes * T} >= 2^24")
    dest = e // (epr * rpn)                                                  # :116
    occ = np.zeros((T, n_nodes), dtype=bool)
    occ[np.arange(T)[:, None], dest] = True                                  # :127-128
    if groups_m is not None:
        actual = int(occ.sum())
        if actual != T * groups_m:                                           # :171-177
            raise ValueError(f"groups_m={groups_m} implies {T * groups_m} dispatch rows for T={T}, "
                             f"but the routing actually produces {actual} (fan-out "
                             f"{actual / max(T, 1):.4f} != {groups_m})")
        if k % groups_m:                                                     # :188-192
            raise ValueError(f"groups_m={groups_m} does not divide k={k}")
        per = np.zeros((T, n_nodes), dtype=np.int64)
        np.add.at(per, (np.arange(T)[:, None], dest), 1)
        bad = int((per[per > 0] != k // groups_m).sum())                     # :193-204
        if bad:
            raise ValueError(f"groups_m={groups_m} requires every touched node to hold exactly "
                             f"k/M={k // groups_m} of a token's experts, but {bad} (token, node) "
                             f"pairs violate the quota")
    node_first = occ.T                                                       # [n_nodes, T], :131
    sel = np.flatnonzero(node_first.reshape(-1))                             # ascending set bits
    u_node = (sel // T).astype(np.int64)                                     # :246
    u_src = (sel % T).astype(np.int64)                                       # :247
    counts = occ.sum(0).astype(np.int64)                                     # :250
    row_pos = np.cumsum(node_first.reshape(-1).astype(np.int64)) - 1         # :138-139
    flat = dest * T + np.arange(T)[:, None]                                  # :252
    inverse = row_pos[flat.reshape(-1)].astype(np.int64)                     # :253
    return u_src, u_node, counts, inverse


def send_offsets(counts):
    """Exclusive prefix of the per-node row counts: where each node's rows start."""
    c = np.asarray(counts, dtype=np.int64)
    return np.concatenate([[0], np.cumsum(c)[:-1]]).astype(np.int64)


def dispatch_stats(expert_idx, world, n_experts, rpn=8):
    """terrace/ta2a.py:278-298."""
    T, k = np.asarray(expert_idx).shape
    _, _, counts, _ = plan_ta2a(expert_idx, world, n_experts, rpn)
    rows = int(counts.sum())
    return {"rows_baseline": T * k, "rows_ta2a": rows, "dedup_x": (T * k) / max(rows, 1),
            "msgs_baseline": world, "msgs_ta2a": world // rpn, "msg_growth_x": rpn}


# --------------------------------------------------------------------------------------
# (3) Hop-A pack -- terrace/ta2a_fwd.py:177-249, :473 ; terrace/ops/k2_ref.py:70-134
# --------------------------------------------------------------------------------------


def pack_quota_wire(expert_idx, gates, inverse, n_rows, slots, quota):
    """(slot_tab [n_rows,q] i64, gate_tab [n_rows,q] gates.dtype), zero-initialised.

    terrace/ta2a_fwd.py:177-249 (``sorted_rows=False`` branch, which the sorted branch
    equals when rows already ascend).  ``gates`` must already be in the payload's storage
    dtype; values are moved, never computed.
    """
    e = np.asarray(expert_idx, dtype=np.int64)
    T, k = e.shape
    gates = np.asarray(gates)
    order = np.argsort(e, axis=1, kind="stable")                             # :232-235
    slot_vals = (np.take_along_axis(e, order, 1) % slots).reshape(-1, quota)
    gate_vals = np.take_along_axis(gates, order, 1).reshape(-1, quota)
    rof = np.take_along_axis(np.asarray(inverse).reshape(T, k), order[:, ::quota], 1).reshape(-1)
    slot_tab = np.zeros((n_rows, quota), dtype=np.int64)                     # :245
    gate_tab = np.zeros((n_rows, quota), dtype=gates.dtype)                  # :247
    slot_tab[rof] = slot_vals
    gate_tab[rof] = gate_vals
    return slot_tab, gate_tab


def check_k2_geometry(T, k, world, n_experts, rpn, groups_m):
    """Scalar checks of terrace/ops/k2_ref.py:95-108 (same exception classes)."""
    if world <= 0 or rpn <= 0 or groups_m <= 0 or n_experts <= 0:
        raise ValueError("k2_pack: bad geometry scalars")
    if world % rpn or n_experts % world or k % groups_m:
        raise ValueError(f"k2_pack: world={world} rpn={rpn} n_experts={n_experts} k={k} "
                         f"groups_m={groups_m} not divisible")
    slots = (n_experts // world) * rpn
    if slots > 63:
        raise ValueError(f"{slots} expert slots per node exceeds the chain bound")


def k2_pack(hidden, expert_idx, gates, world, n_experts, rpn, groups_m):
    """(payload [T*M,H], mask [T*M,q] i64, gate_rows [T*M,q], u_src [T*M] i64, node_counts).

    The fused send side: plan + dedup gather + wire planes, composed exactly as
    terrace/ta2a_fwd.py:471-489; terrace/ops/k2_ref.py:70-134 is the same object.
    """
    e = np.asarray(expert_idx, dtype=np.int64)
    if e.ndim != 2 or hidden.ndim != 2 or np.asarray(gates).ndim != 2:
        raise ValueError("k2_pack: hidden/expert_idx/gates must be 2-D")
    T, k = e.shape
    if hidden.shape[0] != T or np.asarray(gates).shape != e.shape:
        raise ValueError("k2_pack: geometry mismatch")
    check_k2_geometry(T, k, world, n_experts, rpn, groups_m)
    if T and (e.min() < 0 or e.max() >= n_experts):
        raise ValueError("k2_pack: expert id out of range")
    slots = (n_experts // world) * rpn
    u_src, _, counts, inverse = plan_ta2a(e, world, n_experts, rpn, groups_m)
    payload = hidden[u_src]                                                  # ta2a_fwd.py:473
    mask, gate_rows = pack_quota_wire(e, gates, inverse, T * groups_m, slots, k // groups_m)
    return payload, mask, gate_rows, u_src, counts


# --------------------------------------------------------------------------------------
# (4) Hop-B arrival chain and expert-order regroup
#     terrace/ops/__init__.py:255-300 ; terrace/ta2a_fwd.py:252-266, :605-628, :641-646
# --------------------------------------------------------------------------------------


def k1_arrival(rx, rslot, rgate, quota, epr, rpn, my_local=0):
    """(send_buf [P,H], gate_pairs [P], r_idx [P] i64, slot_idx [P] i64, i_send [rpn] i64).

    Pairs p = r*quota + i are put in stable ascending order of their owner card
    ``rslot[p] // epr`` (terrace/ops/__init__.py:287-299).
    """
    rslot = np.asarray(rslot, dtype=np.int64)
    R, q = rslot.shape
    assert q == quota
    flat = rslot.reshape(-1)
    owner = flat // epr
    ordo = stable_argsort_small(owner, rpn)
    r_idx = (ordo // quota).astype(np.int64)
    slot_idx = flat[ordo]
    i_send = fixed_hist(owner, rpn)
    send_buf = rx[r_idx]
    gate_pairs = np.asarray(rgate).reshape(-1)[ordo]
    return send_buf, gate_pairs, r_idx, slot_idx, i_send


def regroup(node_rx, my_slot, epr, my_local=0, capacity=None):
    """Expert-contiguous layout of the rows one expert card received.

    Drop-less form (terrace/ta2a_fwd.py:641-646): ``exp_j = my_slot - my_local*epr``;
    ``order`` = stable ascending sort by ``exp_j``; ``tokens_per_expert = hist(exp_j, epr)``;
    ``permuted = node_rx[order]``.  Returns (permuted, order, tokens_per_expert).

    Capacity form (own specification; the reference is drop-less): expert ``x`` keeps the
    first ``capacity`` of its rows in that same stable order and drops the rest.  Returns
    (padded [epr*capacity, H] with unused rows zero, dest [P] i64 = ``x*capacity + rank`` or
    -1 when dropped, kept [P] bool, tokens_per_expert [epr] i64 (before the cut),
    kept_per_expert [epr] i64 = min(count, capacity)).
    """
    exp_j = np.asarray(my_slot, dtype=np.int64).reshape(-1) - my_local * epr
    counts = fixed_hist(exp_j, epr)
    order = stable_argsort_small(exp_j, epr)
    if capacity is None:
        return node_rx[order], order, counts
    start = send_offsets(counts)
    rank = np.empty(exp_j.size, dtype=np.int64)
    rank[order] = np.arange(exp_j.size) - start[exp_j[order]]
    kept = rank < capacity
    dest = np.where(kept, exp_j * capacity + rank, -1).astype(np.int64)
    padded = np.zeros((epr * capacity,) + node_rx.shape[1:], dtype=node_rx.dtype)
    padded[dest[kept]] = node_rx[kept]
    return padded, dest, kept, counts, np.minimum(counts, capacity)


def hopb_local_scatter(rx, rslot, rgate, quota, n_local, first_slot=0, capacity=None):
    """The arrival chain and the expert-order regroup of a rank whose node's slots are all local, as the
    reference composes them (terrace/ta2a_fwd.py:605-646): ``k1_arrival`` with ``epr*rpn = n_local``, then
    ``regroup`` over all ``n_local`` slots of what arrived.  Returned per PAIR ``p = r*quota + i`` (the
    enumeration before the arrival reorder), which is what a one-pass kernel can know:

    (permuted, place [P] i64 (-1 dropped), kept [P] bool, tokens_per_expert, kept_per_expert,
     permuted_gate [places], pair_of_place [places] i64 (-1 on padding)).

    The owner-card split is immaterial to the result (a stable sort by ``slot // epr`` then by ``slot`` is a
    stable sort by ``slot``); it is taken with ``rpn = n_local`` cards of one expert each.
    """
    rslot = np.asarray(rslot, dtype=np.int64)
    R, q = rslot.shape
    P = R * q
    local = rslot - first_slot
    send_buf, gate_pairs, r_idx, slot_idx, _ = k1_arrival(rx, local, rgate, quota, 1, n_local)
    pos = arrival_positions(local, 1, n_local)                 # pair p -> arrival position
    ordo = np.empty_like(pos)
    ordo[pos] = np.arange(P)                                   # arrival position -> pair
    if capacity is None:
        permuted, order, counts = regroup(send_buf, slot_idx, n_local)
        place_arr = np.empty(P, dtype=np.int64)
        place_arr[order] = np.arange(P)
        kept_arr = np.ones(P, dtype=bool)
        kept_per = counts.copy()
        n_places = P
    else:
        permuted, place_arr, kept_arr, counts, kept_per = regroup(send_buf, slot_idx, n_local, capacity=capacity)
        n_places = n_local * capacity
    place = place_arr[pos]
    kept = kept_arr[pos]
    pair_of_place = np.full(n_places, -1, dtype=np.int64)
    pair_of_place[place_arr[kept_arr]] = ordo[kept_arr]
    g = np.asarray(rgate)
    permuted_gate = np.zeros(n_places, dtype=g.dtype)
    permuted_gate[place_arr[kept_arr]] = gate_pairs[kept_arr]
    return permuted, place, kept, counts, kept_per, permuted_gate, pair_of_place


# --------------------------------------------------------------------------------------
# (5) combine -- terrace/ta2a_fwd.py:658-670 ; one level: terrace/ep_dist.py:121-122
# --------------------------------------------------------------------------------------


def gather_reduce(src_f32, idx, weights=None):
    """out[i] = sum_j w[i,j] * src[idx[i,j]] in fp32, j ascending; idx < 0 contributes 0.

    ``acc = fl(acc + fl(w*x))`` starting from +0 -- multiply and add rounded separately.
    """
    idx = np.asarray(idx, dtype=np.int64)
    n, fan = idx.shape
    acc = np.zeros((n, src_f32.shape[1]), dtype=np.float32)
    for j in range(fan):
        ok = idx[:, j] >= 0
        rows = src_f32[np.where(ok, idx[:, j], 0)]
        if weights is not None:
            rows = (rows * np.asarray(weights, np.float32)[:, j:j + 1]).astype(np.float32)
        rows = np.where(ok[:, None], rows, np.float32(0))
        acc = (acc + rows).astype(np.float32)
    return acc


def combine(src_rows, idx, weights, in_fmt="f32", out_fmt="f32", hidden=None):
    """Decode, ``gather_reduce`` in fp32, round once to ``out_fmt``."""
    return encode_rows(gather_reduce(decode_rows(src_rows, in_fmt, hidden), idx, weights), out_fmt)


def combine_reference_order(ret_f32, gate_pairs_f32, r_idx, u_src, R, T):
    """Two-level combine exactly as written in terrace/ta2a_fwd.py:661-670, kept in fp32:
    ``red.index_add_(0, r_idx, ret*gate)`` then ``y.index_add(0, u_src, red)``, each adding
    in ascending enumeration order.  Used to show the fused one-level order is the same sum.
    """
    red = np.zeros((R, ret_f32.shape[1]), dtype=np.float32)
    contrib = (ret_f32 * gate_pairs_f32[:, None]).astype(np.float32)
    for j in range(len(r_idx)):
        red[r_idx[j]] = (red[r_idx[j]] + contrib[j]).astype(np.float32)
    y = np.zeros((T, ret_f32.shape[1]), dtype=np.float32)
    for r in range(R):
        y[u_src[r]] = (y[u_src[r]] + red[r]).astype(np.float32)
    return y


def arrival_positions(rslot, epr, rpn):
    """pos[p] = where pair p lands in the arrival order (inverse permutation of ``ordo``)."""
    flat = np.asarray(rslot, dtype=np.int64).reshape(-1)
    ordo = stable_argsort_small(flat // epr, rpn)
    pos = np.empty_like(ordo)
    pos[ordo] = np.arange(ordo.size)
    return pos


def token_pair_table(expert_idx, inverse, quota):
    """[T,k] table: for each token, the flat Hop-A pair ids ``row*quota + i`` of its k
    experts, listed in ascending expert id -- the order both reference ``index_add`` levels
    add in (ascending slot within a row, ascending node across rows)."""
    e = np.asarray(expert_idx, dtype=np.int64)
    T, k = e.shape
    order = np.argsort(e, axis=1, kind="stable")
    rows = np.take_along_axis(np.asarray(inverse).reshape(T, k), order, 1)
    return rows * quota + (np.arange(k)[None, :] % quota), order


# --------------------------------------------------------------------------------------
# general (data-dependent fan-out) branch -- terrace/ta2a_fwd.py:120-174, :348-442, :496-500
# and the seam's entry helper -- terrace/ta2a_dispatch.py:224-260
# --------------------------------------------------------------------------------------


def build_expansion(expert_idx, inverse, n_rows, world, n_experts, rpn=8):
    """mask [n_rows] i64: bit j of row r is set iff node-local slot j wants the row.

    terrace/ta2a_fwd.py:348-442.  The reference sums distinct powers of two per row (:440-441,
    and the structured path :425-438 sums the same set); for distinct experts per token that
    is the bitwise OR restated here.  ``slots > 63`` raises as at :372-373.
    """
    e = np.asarray(expert_idx, dtype=np.int64)
    slots = (n_experts // world) * rpn
    if slots > 63:
        raise ValueError(f"{slots} expert slots per node exceeds the int64 mask")
    mask = np.zeros(n_rows, dtype=np.int64)
    np.bitwise_or.at(mask, np.asarray(inverse, dtype=np.int64).reshape(-1),
                     np.int64(1) << (e.reshape(-1) % slots))
    return mask


def sparse_gate_plane(expert_idx, gates, inverse, n_rows, slots):
    """gate_rows [n_rows, slots], zero except [inverse[t,j], expert % slots] = gates[t,j]
    (terrace/ta2a_fwd.py:498-500)."""
    e = np.asarray(expert_idx, dtype=np.int64).reshape(-1)
    g = np.asarray(gates)
    out = np.zeros((n_rows, slots), dtype=g.dtype)
    out[np.asarray(inverse, dtype=np.int64).reshape(-1), e % slots] = g.reshape(-1)
    return out


def expand_arrival(rmask, slots, quota=None):
    """(r_idx, slot_idx) demand pairs of the arrived bitmasks (terrace/ta2a_fwd.py:120-174).

    ``quota`` None: every set bit, rows ascending and columns ascending inside a row
    (``nonzero`` order, :174).  With a quota: exactly ``quota`` columns per row, chosen by the
    distinct key ``bit*slots + (slots-1-col)`` descending (:165-169), i.e. the set columns
    ascending first, then -- for a row with fewer -- its unset columns ascending.
    """
    rmask = np.asarray(rmask, dtype=np.int64)
    R = rmask.shape[0]
    bits = (rmask[:, None] >> np.arange(slots, dtype=np.int64)[None, :]) & 1     # [R, slots]
    if quota is None:
        r, c = np.nonzero(bits)
        return r.astype(np.int64), c.astype(np.int64)
    key = bits * slots + (slots - 1 - np.arange(slots, dtype=np.int64))[None, :]
    cols = np.argsort(-key, axis=1, kind="stable")[:, :quota]
    r_idx = np.repeat(np.arange(R, dtype=np.int64), quota)
    return r_idx, cols.reshape(-1).astype(np.int64)


def arrival_pairs(rx, r_idx, slot_idx, rgate, epr, rpn):
    """The arrival chain of the general branch (terrace/ta2a_fwd.py:605-628): pairs in stable
    ascending owner-card order; the gate of a pair is looked up in the sparse plane
    ``rgate[r, slot]`` after the reorder (:626-627).
    Returns (send_buf, gate_pairs, r_idx, slot_idx, i_send, ordo)."""
    r_idx = np.asarray(r_idx, dtype=np.int64)
    slot_idx = np.asarray(slot_idx, dtype=np.int64)
    owner = slot_idx // epr
    ordo = stable_argsort_small(owner, rpn)
    r2, s2 = r_idx[ordo], slot_idx[ordo]
    i_send = fixed_hist(owner, rpn)
    return rx[r2], np.asarray(rgate)[r2, s2], r2, s2, i_send, ordo


def routing_map_to_topk(routing_map, probs):
    """(expert_idx [T,k] i64 ascending per row, gates [T,k] = probs at those columns).

    terrace/ta2a_dispatch.py:224-260: every row must hold the same non-zero number k of set
    entries, else RuntimeError.
    """
    rm = np.asarray(routing_map) != 0
    counts = rm.sum(1)
    if counts.size and counts.min() != counts.max():
        raise RuntimeError("T-A2A requires exactly k experts per token (drop-less); observed per-row "
                           "expert counts differ")
    k = int(counts[0]) if counts.size else 0
    if k == 0:
        raise RuntimeError("T-A2A got an all-empty routing_map (k=0); impossible under drop-less routing")
    expert_idx = np.nonzero(rm)[1].reshape(rm.shape[0], k).astype(np.int64)
    return expert_idx, np.take_along_axis(np.asarray(probs), expert_idx, 1)


def pair_places(order, r_idx, slot_idx, u_src, u_node, expert_idx, slots):
    """(where [T,k], token_of_place [P]) for the seam halves (terrace/ta2a_dispatch.py:263-498).

    Place i of the expert-order buffer holds arrival row ``a = order[i]``, a copy of send row
    ``r = r_idx[a]``, i.e. of token ``t = u_src[r]`` for expert ``u_node[r]*slots + slot_idx[a]``;
    ``where[t, j] = i`` for the column j holding that expert.  So ``permuted[i] =
    hidden[token_of_place[i]]`` and ``ta2a_unpermute`` computes ``y[t] = sum_j expert_out[where[t, j]]``;
    the adjoints of both halves read these two tables.
    """
    e = np.asarray(expert_idx, dtype=np.int64)
    T, k = e.shape
    a = np.asarray(order, dtype=np.int64)
    r = np.asarray(r_idx, dtype=np.int64)[a]
    tok = np.asarray(u_src, dtype=np.int64)[r]
    exp = np.asarray(u_node, dtype=np.int64)[r] * slots + np.asarray(slot_idx, dtype=np.int64)[a]
    where = np.full((T, k), -1, dtype=np.int64)
    hit = e[tok] == exp[:, None]                                  # [P, k]
    rows, cols = np.nonzero(hit)
    where[tok[rows], cols] = rows
    return where, tok


# --------------------------------------------------------------------------------------
# wire containers -- terrace/ta2a_pack.py:276-506
# --------------------------------------------------------------------------------------


def container_words(id_w, hidden, gate_w, itemsize):
    """Row width in int64 words: the id plane, then just enough words for hidden+gate_w
    elements (terrace/ta2a_pack.py:287-288; hidden = 0 gives the small layout, :380-381)."""
    per_word = 8 // itemsize
    return id_w + -(-(hidden + gate_w) // per_word)


def pack_planes(planes, n_rows, row_bytes):
    """Byte-level container: each row is the planes' rows back to back, then zeros.
    hopa_pack (:319-336) = (ids, payload, gates); hopa_pack_small (:398-414) = (ids, gates);
    hopb_pack_meta (:474-497) = (slot ids, gates) with row_bytes = 16."""
    out = np.zeros((n_rows, row_bytes), dtype=np.uint8)
    at = 0
    for p in planes:
        b = np.ascontiguousarray(p).reshape(n_rows, -1).view(np.uint8) if n_rows else np.zeros((0, 0), np.uint8)
        if n_rows:
            out[:, at:at + b.shape[1]] = b
            at += b.shape[1]
    return out.view(np.int64) if row_bytes % 8 == 0 else out


def unpack_planes(buf, specs):
    """Inverse: specs = [(dtype, elements per row), ...] consecutive from the row head
    (hopa_unpack :339-356, hopa_unpack_small :417-423, hopb_unpack_meta :500-503)."""
    raw = np.ascontiguousarray(buf).view(np.uint8).reshape(buf.shape[0], -1)
    out, at = [], 0
    for dtype, width in specs:
        nbytes = np.dtype(dtype).itemsize * width
        out.append(np.ascontiguousarray(raw[:, at:at + nbytes]).view(dtype).reshape(buf.shape[0], width))
        at += nbytes
    return out


def hopa_send_splits(node_counts, world, rpn, my_local):
    """terrace/ta2a_dispatch.py:197-211 -- length-`world` send counts, node n's rows go to its
    designated peer n*rpn + my_local, every other entry is zero."""
    send = np.zeros(world, dtype=np.int64)
    send[np.arange(world // rpn) * rpn + my_local] = np.asarray(node_counts, dtype=np.int64)
    return send
