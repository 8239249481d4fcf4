"""Formula-made inputs (no random generator of any library involved) and the digest of every plane the path
produces for them.  ``tests/golden/make_oracle_digests.py`` writes the oracle's digests to
``tests/golden/oracle_digests.json``; the CPU suite checks the oracle against that file, the GPU suite the kernels."""
from __future__ import annotations

import hashlib

import numpy as np

# name: (T, E, n_groups, k, M, rpn, H, fmt, capacity or None)
CASES = {
    "reference_shape": (192, 64, 8, 4, 2, 8, 64, "f32", None),
    "v3_shape": (160, 256, 8, 8, 4, 8, 256, "bf16", None),
    "high_dedup": (224, 128, 16, 8, 2, 8, 128, "bf16", None),
    "capacity": (256, 256, 8, 8, 4, 8, 64, "bf16", 36),
    "fp8_rows": (96, 256, 8, 8, 4, 8, 384, "fp8", None),
    "ragged_tail": (65, 32, 4, 4, 2, 4, 24, "f32", 3),
}


def _mixed(rows, cols, seed):
    """float32 values in [-0.5, 0.5) from an integer hash of (row, column, seed): 32-bit multiply-xorshift
    rounds done in uint64 with explicit masks, so every platform computes the same bits."""
    r = np.arange(rows, dtype=np.uint64)[:, None]
    c = np.arange(cols, dtype=np.uint64)[None, :]
    m32 = np.uint64(0xFFFFFFFF)
    h = (r * np.uint64(0x9E3779B1) + c * np.uint64(0x85EBCA77) + np.uint64(seed)) & m32
    for mul, shift in ((0x2C1B3C6D, 15), (0x297A2D39, 12), (0x85EBCA6B, 16)):
        h ^= h >> np.uint64(shift)
        h = (h * np.uint64(mul)) & m32
    h ^= h >> np.uint64(15)
    return ((h >> np.uint64(8)).astype(np.float32) / np.float32(1 << 24) - np.float32(0.5)).astype(np.float32)


def inputs(name):
    T, E, n_groups, k, M, rpn, H, fmt, cap = CASES[name]
    logits = _mixed(T, E, 1)
    bias = (_mixed(1, E, 2)[0] * np.float32(0.2)).astype(np.float32)
    x = _mixed(T, H, 3) * np.float32(4.0)
    return dict(T=T, E=E, n_groups=n_groups, k=k, M=M, rpn=rpn, H=H, fmt=fmt, capacity=cap, world=n_groups * rpn,
                logits=logits, bias=bias, x=x.astype(np.float32))


def digest(a) -> str:
    a = np.ascontiguousarray(a)
    return hashlib.sha256(str(a.dtype).encode() + str(a.shape).encode() + a.tobytes()).hexdigest()[:24]


def oracle_planes(name) -> dict:
    """Every plane of the path for one case, from the CPU oracle."""
    from oracle import terrace_oracle as orc
    c = inputs(name)
    E, k, M, rpn, world = c["E"], c["k"], c["M"], c["rpn"], c["world"]
    epr, q = E // world, k // M
    slots = epr * rpn
    e, gates, grp = orc.t_route(c["logits"], c["bias"], E, c["n_groups"], k, M)
    if c["fmt"] == "f32":
        rows, g_pay = c["x"], gates
    elif c["fmt"] == "bf16":
        rows, g_pay = orc.f32_to_bf16(c["x"]), orc.f32_to_bf16(gates)
    else:
        rows, g_pay = orc.fp8_quantise_rows(c["x"]), orc.f32_to_bf16(gates)
    payload, mask, gate_rows, u_src, counts = orc.k2_pack(rows, e, g_pay, world, E, rpn, M)
    send, gp, r_idx, s_idx, i_send = orc.k1_arrival(payload, mask, gate_rows, q, epr, rpn)
    out = dict(expert_idx=e, gates=gates, group_idx=grp, payload=payload, mask=mask, gate_rows=gate_rows, u_src=u_src,
               node_counts=counts, send_buf=send, gate_pairs=gp, r_idx=r_idx, slot_idx=s_idx, i_send=i_send)
    if c["capacity"] is None:
        perm, order, tpe = orc.regroup(send, s_idx, slots)
        place = np.empty_like(order)
        place[order] = np.arange(order.size)
    else:
        perm, place, kept, tpe, _ = orc.regroup(send, s_idx, slots, capacity=c["capacity"])
        out["kept"] = kept
    out.update(permuted=perm, place=place, tokens_per_expert=tpe)
    _, _, _, inverse = orc.plan_ta2a(e, world, E, rpn, M)
    pair_tab, sort_order = orc.token_pair_table(e, inverse, q)
    pos = orc.arrival_positions(mask, epr, rpn)
    where = np.where(pos[pair_tab] >= 0, place[pos[pair_tab]], -1)
    w_sorted = np.take_along_axis(g_pay, sort_order, 1)
    wf = orc.decode_rows(w_sorted, "f32" if c["fmt"] == "f32" else "bf16")
    out["y"] = orc.combine(perm, where, wf, c["fmt"], "f32" if c["fmt"] == "f32" else "bf16", hidden=c["H"])
    # the tables the stages hand on: each pair's arrival position, the [T, k] entry behind each Hop-A pair, the
    # combine's place table, and the one-pass Hop B's place of each pair in arrival order
    pair_src = np.full(pair_tab.size, -1, dtype=np.int64)
    live = pair_tab.reshape(-1) >= 0
    pair_src[pair_tab.reshape(-1)[live]] = np.nonzero(live)[0]
    one = orc.hopb_local_scatter(payload, mask, gate_rows, q, slots, 0, c["capacity"])
    assert np.array_equal(one[0], perm)
    out.update(pair_pos=pos, pair_src=pair_src, where=where.astype(np.int64), onepass_place=one[1],
               kept_per_expert=one[4])
    return out
