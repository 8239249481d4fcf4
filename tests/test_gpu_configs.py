"""The five benchmark geometries end to end on the device.

At a reduced token count every plane of every stage is compared bit for bit with the CPU
oracle.  At the full size the index / count / offset planes are still compared with the oracle
(they are small), while the moved rows are checked through size-independent properties: every
row of a stage's output equals the input row its index plane names, and with identity experts
the combine returns each token scaled by the sum of its kept gates (dispatch -> combine round
trip) within the stated tolerance.
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import terrace_oracle as orc
from test_gpu_parity import DEV, announce, same, to_np

pytestmark = pytest.mark.gpu

TOL = {"f32": 1e-5, "bf16": 1e-2, "fp8": 1e-2}


def _route(cfg, inp):
    import terrace
    rcfg = terrace.TRouteConfig(cfg.n_experts, cfg.n_groups, cfg.top_k, cfg.top_groups)
    ga = None if inp["gate_affinity"] is None else inp["gate_affinity"].to(DEV)
    e, g, grp = terrace.t_route(inp["logits"].to(DEV), inp["bias"].to(DEV), rcfg, gate_affinity=ga)
    oga = None if inp["gate_affinity"] is None else inp["gate_affinity"].numpy()
    oe, og, ogrp = orc.t_route(inp["logits"].numpy(), inp["bias"].numpy(), cfg.n_experts, cfg.n_groups, cfg.top_k,
                               cfg.top_groups, gate_affinity=oga)
    same(e, oe, "expert_idx"), same(g, og, "gates"), same(grp, ogrp, "group_idx")
    return e, g, oe, og


def _np_rows(x):
    return to_np(x)


def _expert_scale(cfg, u_node, r_idx, slot_idx, places, n_places):
    """(global expert id + 1) / E for the row sitting at each place of the expert-order buffer."""
    e = u_node[r_idx] * cfg.slots + slot_idx
    scale = np.zeros(n_places, dtype=np.float32)
    ok = places >= 0
    scale[places[ok]] = ((e[ok] + 1).astype(np.float32) / np.float32(cfg.n_experts))
    return scale


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4", "c5"])
def test_reduced_size_every_plane_matches_oracle(name):
    from terrace import configs
    cfg = configs.CONFIGS[name].scaled(1536)
    announce("reduced", cfg.name, cfg.T)
    _check_every_plane(cfg)


def _random_geometries(n, seed):
    """Seeded geometries off the benchmark grid: group counts 1..32, group sizes that are not powers
    of two, k up to 24, widths that miss the 16-byte and kilobyte paths, tiny and ragged T."""
    from terrace import configs
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        n_groups = int(rng.choice([1, 2, 4, 8, 16, 32]))
        rpn = int(rng.choice([1, 2, 4, 8]))
        g = rpn * int(rng.integers(1, 9))                     # experts per group, a multiple of rpn
        E = n_groups * g
        M = int(rng.integers(1, min(n_groups, 6) + 1))
        q = int(rng.integers(1, min(g, 6) + 1))
        if E > 2048 or M * q > 24:
            continue
        fmt = str(rng.choice(["f32", "bf16", "fp8"]))
        if fmt == "fp8":
            hidden = 128 * int(rng.integers(1, 9))
        else:
            hidden = int(rng.choice([8, 24, 40, 64, 200, 512, 520, 1024, 1000, 6, 13]))
        out.append(configs.PathConfig(
            f"random{len(out)}", int(rng.choice([1, 2, 63, 64, 65, 300, 700])), E, n_groups, M * q, M, rpn, hidden, fmt,
            bias=str(rng.choice(["none", "normal", "zipf"])), softmax_gates=bool(rng.integers(0, 2)),
            capacity_factor=[None, 0.5, 1.25][int(rng.integers(0, 3))], seed=int(rng.integers(1, 1 << 30))))
    return out


@pytest.mark.parametrize("index", range(32))
def test_random_geometries_every_plane_matches_oracle(index):
    cfg = _random_geometries(32, 20261125)[index]
    announce("random", cfg)
    _check_every_plane(cfg)


def _large_geometries(n, seed):
    """Seeded geometries with many tokens and narrow rows: every choice the sorts make of their unit size and of
    the way a workgroup finds its base (table re-derived per workgroup, or a scan launch) is met, at sizes the
    oracle still finishes in a second."""
    from terrace import configs
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        n_groups = int(rng.choice([1, 2, 4, 8, 16, 32, 64]))
        rpn = int(rng.choice([1, 2, 4, 8]))
        g = rpn * int(rng.integers(1, 9))
        E = n_groups * g
        M = int(rng.integers(1, min(n_groups, 6) + 1))
        q = int(rng.integers(1, min(g, 6) + 1))
        if E > 2048 or M * q > 24 or g > 63:
            continue
        fmt = str(rng.choice(["f32", "bf16", "fp8"]))
        hidden = 128 * int(rng.integers(1, 3)) if fmt == "fp8" else int(rng.choice([8, 24, 64, 200, 128]))
        T = int(rng.choice([1023, 1025, 4097, 9000, 16384, 30000, 65537, 100000]))
        if T * M * q * hidden > 2e9:
            continue
        out.append(configs.PathConfig(
            f"large{len(out)}", T, E, n_groups, M * q, M, rpn, hidden, fmt,
            bias=str(rng.choice(["none", "normal", "zipf"])), softmax_gates=bool(rng.integers(0, 2)),
            capacity_factor=[None, 0.5, 1.25][int(rng.integers(0, 3))], seed=int(rng.integers(1, 1 << 30))))
    return out


@pytest.mark.parametrize("index", range(10))
def test_large_random_geometries_every_plane_matches_oracle(index):
    cfg = _large_geometries(10, 20261126)[index]
    announce("large random", cfg)
    _check_every_plane(cfg)


# Up to 64 tokens the send side is one place workgroup that counts for itself, and up to 1024 items a sort is one
# rank workgroup that does; one more token or item and the count launch is back.  Token counts on both sides of each
# limit, at k = 8 (pairs = 8 T: 1024 at T = 128) and at k = 2, M = 1 (pairs = 2 T: 1024 at T = 512), with and
# without a capacity.
@pytest.mark.parametrize("capacity_factor", [None, 0.5])
@pytest.mark.parametrize("T,k,M", [(63, 8, 4), (64, 8, 4), (65, 8, 4), (127, 8, 4), (128, 8, 4), (129, 8, 4),
                                   (511, 2, 1), (512, 2, 1), (513, 2, 1), (1, 8, 4)])
def test_one_workgroup_limits_every_plane_matches_oracle(T, k, M, capacity_factor):
    from terrace import configs
    cfg = configs.PathConfig(f"limits_T{T}_k{k}", T, 64, 8, k, M, 4, 64, "bf16", bias="normal", softmax_gates=True,
                             capacity_factor=capacity_factor, seed=4000 + T)
    announce("one-workgroup limits", cfg)
    _check_every_plane(cfg)


def _check_every_plane(cfg):
    from terrace.ta2a_fwd import loopback_combine, loopback_dispatch, twolevel_combine
    from terrace import configs
    inp = configs.make_inputs(cfg)
    e, g32, oe, og = _route(cfg, inp)
    gates = g32.to(cfg.gate_dtype)
    ogates = to_np(gates)
    x = configs.rows_to(inp["x"], DEV)
    ox = _np_rows(inp["x"])
    cap = cfg.capacity(cfg.slots)
    st = loopback_dispatch(x, e, gates, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups, cap)
    # ---- send side
    payload, mask, gate_rows, u_src, counts = orc.k2_pack(ox, oe, ogates, cfg.world, cfg.n_experts, cfg.rpn,
                                                          cfg.top_groups)
    same(st.payload, payload, "payload"), same(st.mask, mask, "mask"), same(st.gate_rows, gate_rows, "gate_rows")
    same(st.u_src, u_src, "u_src"), same(st.node_counts, counts, "node_counts")
    _, u_node, _, inverse = orc.plan_ta2a(oe, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups)
    same(st.extras["u_node"], u_node, "u_node"), same(st.extras["inverse"], inverse, "inverse")
    same(st.extras["node_offsets"], orc.send_offsets(counts), "node_offsets")
    assert st.extras["status"].tolist() == [0, cfg.send_rows, 0, 0]
    # ---- arrival
    send, gp, r_idx, s_idx, i_send = orc.k1_arrival(payload, mask, gate_rows, cfg.quota, cfg.epr, cfg.rpn)
    same(st.send_buf, send, "send_buf"), same(st.gate_pairs, gp, "gate_pairs"), same(st.r_idx, r_idx, "r_idx")
    same(st.slot_idx, s_idx, "slot_idx"), same(st.i_send, i_send, "i_send")
    pos = orc.arrival_positions(mask, cfg.epr, cfg.rpn)
    same(st.pair_pos, pos, "pair_pos")
    # ---- regroup (+ capacity)
    if cap is None:
        perm, order, tpe = orc.regroup(send, s_idx, cfg.slots)
        place = np.empty_like(order)
        place[order] = np.arange(order.size)
    else:
        perm, place, kept, tpe, kpe = orc.regroup(send, s_idx, cfg.slots, capacity=cap)
        same(st.kept, kept, "kept")
        if cfg.name.startswith("c4"):
            assert 0 < kept.sum() < kept.size, "the skewed workload must overflow some expert but not all"
    same(st.permuted, perm, "permuted"), same(st.place, place, "place"), same(st.tokens_per_expert, tpe, "tokens_per_expert")
    # ---- the same Hop B as one pass: identical expert-order buffer, places named by pair
    import terrace.ops as tops
    from terrace.ta2a_fwd import loopback_dispatch_onepass
    hb = tops.hopb_scatter(st.payload, st.mask, st.gate_rows, cfg.quota, cfg.slots, 0, cap, want_pairs=True)
    o_perm, o_place, o_kept, o_tpe, o_kpe, o_pgate, o_pairs = orc.hopb_local_scatter(
        payload, mask, gate_rows, cfg.quota, cfg.slots, 0, cap)
    assert np.array_equal(o_perm, perm) and np.array_equal(o_place, place[pos])
    same(hb["permuted"], perm, "one-pass permuted"), same(hb["place"], o_place, "one-pass place")
    same(hb["tokens_per_expert"], tpe, "one-pass tokens_per_expert"), same(hb["pair_of_place"], o_pairs, "pair_of_place")
    same(hb["permuted_gate"], o_pgate, "one-pass permuted_gate"), same(hb["kept_per_expert"], o_kpe, "kept_per_expert")
    if cap is not None:
        same(hb["kept"], o_kept, "one-pass kept")
    st1 = loopback_dispatch_onepass(x, e, gates, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups, cap)
    assert torch.equal(st1.permuted, st.permuted) and torch.equal(st1.place, st.place[st.pair_pos])
    # ---- the combine's place table, filled on the way through the pairs' tags (no look-up launch)
    o_pair_tab, _ = orc.token_pair_table(oe, inverse, cfg.quota)
    o_where = place[pos[o_pair_tab]]
    o_pair_src = np.empty(cfg.pairs, dtype=np.int64)
    o_pair_src[o_pair_tab.reshape(-1)] = np.arange(cfg.T * cfg.top_k)
    same(st.extras["pair_src"], o_pair_src, "pair_src")
    same(st.extras["where"], o_where, "where (two-step dispatch)"), same(st1.extras["where"], o_where, "where (one pass)")
    assert torch.equal(st.extras["where"], tops.index_chain2(st.place, st.pair_pos, st.extras["pair_table"]))
    # ---- experts: row * (expert id + 1) / E, or fresh fp8 rows for the fp8 workload
    n_places = perm.shape[0]
    if cfg.fmt == "fp8":
        gq = torch.Generator().manual_seed(7)
        ye_rows = orc.fp8_quantise_rows(torch.randn(n_places, cfg.hidden, generator=gq).numpy())
        ye = torch.from_numpy(ye_rows).to(DEV)
        fmt_in, hid = "fp8", cfg.hidden
    else:
        scale = _expert_scale(cfg, u_node, r_idx, s_idx, place, n_places)
        dec = orc.decode_rows(perm, cfg.fmt)
        ye_rows = orc.encode_rows((dec * scale[:, None]).astype(np.float32), cfg.fmt)
        ye = (st.permuted.float() * torch.from_numpy(scale).to(DEV)[:, None]).to(st.permuted.dtype)
        same(ye, ye_rows, "expert output")
        fmt_in, hid = cfg.fmt, None
    # ---- combine, fused
    out_fmt = "f32" if cfg.fmt == "f32" else "bf16"
    pair_tab, sort_order = orc.token_pair_table(oe, inverse, cfg.quota)
    where = np.where(pos[pair_tab] >= 0, place[pos[pair_tab]], -1)
    w_sorted = np.take_along_axis(ogates, sort_order, 1)
    wf = orc.decode_rows(w_sorted, "f32" if cfg.fmt == "f32" else "bf16")
    want = orc.combine(ye_rows, where, wf, fmt_in, out_fmt, hidden=cfg.hidden)
    got = loopback_combine(ye, st, out_dtype=cfg.out_dtype, fp8_hidden=cfg.hidden if cfg.fmt == "fp8" else None)
    same(got, want, "combine")
    same(loopback_combine(ye, st1, out_dtype=cfg.out_dtype, fp8_hidden=cfg.hidden if cfg.fmt == "fp8" else None), want,
         "combine after the one-pass dispatch")
    # ---- the stated tolerance against float64
    src64 = orc.decode_rows(ye_rows, fmt_in, cfg.hidden).astype(np.float64)
    ref = np.zeros((cfg.T, cfg.hidden))
    mag = np.zeros((cfg.T, cfg.hidden))
    for j in range(cfg.top_k):
        ok = where[:, j] >= 0
        term = np.where(ok[:, None], src64[np.where(ok, where[:, j], 0)] * wf[:, j:j + 1].astype(np.float64), 0.0)
        ref += term
        mag += np.abs(term)
    got64 = orc.decode_rows(to_np(got), out_fmt).astype(np.float64)
    err = np.abs(got64 - ref).max() / (np.abs(ref).max() + 1e-30)
    assert err <= TOL[cfg.fmt], err
    # element by element: within the tolerance of the magnitudes that element adds up, plus one rounding of the
    # output dtype (2^-24 of |ref| for fp32, 2^-9 for bf16)
    ulp_out = 2.0 ** -24 if out_fmt == "f32" else 2.0 ** -9
    excess = np.abs(got64 - ref) - (TOL[cfg.fmt] * mag + ulp_out * np.abs(ref))
    assert excess.max() <= 0.0, ("element-wise", float(excess.max()), np.unravel_index(excess.argmax(), excess.shape))
    # ---- the reference's two-level shape agrees with the fused one to the same tolerance
    if cfg.fmt != "fp8":
        two = twolevel_combine(ye, st, out_dtype=cfg.out_dtype)
        # that shape rounds every partial sum to the payload dtype, so its error follows the magnitudes added, not
        # their sum: raw-affinity gates can be negative and cancel
        # (the workloads that feed raw logits as affinity: c1, c3, c4); with non-negative gates nothing cancels and the
        # bound is against the result itself
        den = mag.max() if (wf < 0).any() else np.abs(ref).max()
        err2 = np.abs(orc.decode_rows(to_np(two), out_fmt) - ref).max() / (den + 1e-30)
        assert err2 <= 2 * TOL[cfg.fmt], err2


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4", "c5"])
def test_full_size_index_planes_and_round_trip(name):
    from terrace import configs
    _full_size_check(configs.CONFIGS[name])


@pytest.mark.parametrize("fmt,tokens", [("bf16", 49152), ("fp8", 81920)])
def test_buffers_beyond_four_gigabytes(fmt, tokens):
    """Three (five, for the one-byte rows) times the tokens of the DeepSeek-V3-shaped slice: the arrival and
    expert-order buffers are 5.6 GB (4.8 GB) each, so every row offset past the first 4 GB needs more than 32 bits,
    in every mover -- the kilobyte-sliced ones and the ones for other widths -- and in the combine."""
    from terrace import configs
    cfg = configs.PathConfig("beyond_4gb_" + fmt, tokens, 256, 8, 8, 4, 8, 7168, fmt, bias="normal", softmax_gates=True,
                             seed=20261127)
    assert cfg.pairs * cfg.row_bytes > 4.5 * (1 << 30)
    _full_size_check(cfg)
    torch.cuda.empty_cache()


def _full_size_check(cfg):
    from terrace import configs
    from terrace.ta2a_fwd import loopback_combine, loopback_dispatch, loopback_dispatch_onepass
    announce("full", cfg.name, cfg.T)
    inp = configs.make_inputs(cfg)
    e, g32, oe, og = _route(cfg, inp)
    gates = g32.to(cfg.gate_dtype)
    x = configs.rows_to(inp["x"], DEV)
    cap = cfg.capacity(cfg.slots)
    st = loopback_dispatch(x, e, gates, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups, cap)
    u_src, u_node, counts, inverse = orc.plan_ta2a(oe, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups)
    mask, gate_rows = orc.pack_quota_wire(oe, to_np(gates), inverse, cfg.send_rows, cfg.slots, cfg.quota)
    same(st.u_src, u_src, "u_src"), same(st.node_counts, counts, "node_counts"), same(st.mask, mask, "mask")
    same(st.gate_rows, gate_rows, "gate_rows"), same(st.extras["inverse"], inverse, "inverse")
    assert int(counts.sum()) == cfg.send_rows and st.extras["status"].tolist() == [0, cfg.send_rows, 0, 0]
    assert torch.equal(st.payload, x[st.u_src]), "payload rows are not the rows u_src names"
    flat = mask.reshape(-1)
    ordo = orc.stable_argsort_small(flat // cfg.epr, cfg.rpn)
    same(st.r_idx, ordo // cfg.quota, "r_idx"), same(st.slot_idx, flat[ordo], "slot_idx")
    same(st.i_send, orc.fixed_hist(flat // cfg.epr, cfg.rpn), "i_send")
    same(st.gate_pairs, gate_rows.reshape(-1)[ordo], "gate_pairs")
    assert torch.equal(st.send_buf, st.payload[st.r_idx]), "send_buf rows are not the rows r_idx names"
    s_idx = flat[ordo]
    tpe = orc.fixed_hist(s_idx, cfg.slots)
    same(st.tokens_per_expert, tpe, "tokens_per_expert")
    order = orc.stable_argsort_small(s_idx, cfg.slots)
    if cap is None:
        place = np.empty_like(order)
        place[order] = np.arange(order.size)
        same(st.place, place, "place")
        assert torch.equal(st.permuted, st.send_buf[torch.from_numpy(order).to(DEV)])
        kept_gate_sum = None
    else:
        start = orc.send_offsets(tpe)
        rank = np.empty_like(order)
        rank[order] = np.arange(order.size) - start[s_idx[order]]
        kept = rank < cap
        place = np.where(kept, s_idx * cap + rank, -1)
        same(st.place, place, "place"), same(st.kept, kept, "kept")
        dropped = int((~kept).sum())
        assert 0 < dropped < kept.size
        pk = torch.from_numpy(place[kept]).to(DEV)
        assert torch.equal(st.permuted[pk], st.send_buf[torch.from_numpy(np.flatnonzero(kept)).to(DEV)])
        used = torch.zeros(st.permuted.shape[0], dtype=torch.bool, device=DEV)
        used[pk] = True
        assert not st.permuted[~used].any(), "capacity padding rows must be zero"
    # ---- Hop B as one pass gives the same buffer and the same places
    st1 = loopback_dispatch_onepass(x, e, gates, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups, cap)
    assert torch.equal(st1.permuted, st.permuted), "one-pass expert-order buffer differs"
    assert torch.equal(st1.place, st.place[st.pair_pos]) and torch.equal(st1.tokens_per_expert, st.tokens_per_expert)
    if cap is not None:
        assert torch.equal(st1.kept, st.kept[st.pair_pos])
    import terrace.ops as tops
    looked_up = tops.index_chain2(st.place, st.pair_pos, st.extras["pair_table"])
    assert torch.equal(st.extras["where"], looked_up) and torch.equal(st1.extras["where"], looked_up)
    del st1, looked_up
    # ---- round trip with identity experts: y[t] = x[t] * (sum of the token's kept gates)
    got = loopback_combine(st.permuted, st, out_dtype=cfg.out_dtype,
                           fp8_hidden=cfg.hidden if cfg.fmt == "fp8" else None).float()
    pos = np.empty_like(ordo)
    pos[ordo] = np.arange(ordo.size)
    pair_tab, sort_order = orc.token_pair_table(oe, inverse, cfg.quota)
    live = torch.from_numpy(place[pos[pair_tab]] >= 0).to(DEV)
    gsum = (st.extras["gate_sorted"].float() * live).sum(-1, keepdim=True)
    if cfg.fmt == "fp8":
        xf = torch.from_numpy(orc.fp8_dequantise_rows(inp["x"][:4096].numpy(), cfg.hidden)).to(DEV)
        got, gsum = got[:4096], gsum[:4096]
    else:
        xf = x.float()
    err = ((got - xf * gsum).abs().max() / xf.abs().max()).item()
    assert err <= 2 * TOL[cfg.fmt], err


def _state_planes(st):
    planes = {k: getattr(st, k) for k in ("payload", "mask", "gate_rows", "u_src", "node_counts", "send_buf",
                                           "gate_pairs", "r_idx", "slot_idx", "i_send", "pair_pos", "permuted",
                                           "tokens_per_expert", "place", "kept")}
    for k in ("u_node", "inverse", "node_offsets", "pair_table", "sort_order", "token_rows", "gate_sorted"):
        planes["extras." + k] = st.extras[k]
    return planes


@pytest.mark.parametrize("name", ["c1", "c2", "c4", "c5"])
def test_two_phase_operators_and_overlapped_dispatch_equal_the_single_calls(name):
    """Index-only first phases + the *_move second phases, run by loopback_dispatch(overlap=True) with the
    index chain on a second stream, must give bit for bit what the one-call operators give -- twice in a
    row, so that memory handed back by the first pass is reused while both streams are busy."""
    from terrace import configs
    from terrace.ta2a_fwd import loopback_combine, loopback_dispatch
    cfg = configs.CONFIGS[name].scaled(3000)
    announce("two-phase", cfg.name, cfg.T)
    inp = configs.make_inputs(cfg)
    e, g, _, _ = _route(cfg, inp)
    x = configs.rows_to(inp["x"], DEV)
    gates = g.to(cfg.gate_dtype)
    cap = cfg.capacity(cfg.slots)
    args = (x, e, gates, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups, cap)
    plain = loopback_dispatch(*args, overlap=False)
    ye = plain.permuted.clone() if cfg.fmt != "fp8" else configs.quantise_fp8_rows(
        torch.randn(plain.permuted.shape[0], cfg.hidden, device=DEV))
    fp8_hidden = cfg.hidden if cfg.fmt == "fp8" else None
    y_plain = loopback_combine(ye, plain, out_dtype=cfg.out_dtype, fp8_hidden=fp8_hidden)
    for _ in range(2):
        both = loopback_dispatch(*args, overlap=True)
        y_both = loopback_combine(ye, both, out_dtype=cfg.out_dtype, fp8_hidden=fp8_hidden)
        torch.cuda.synchronize()
        want, got = _state_planes(plain), _state_planes(both)
        for k, w in want.items():
            if w is None:
                assert got[k] is None, k
            else:
                assert torch.equal(got[k], w), f"{k} differs between the one-call and the two-phase dispatch"
        assert torch.equal(y_both, y_plain)


def test_move_phases_refuse_bad_arguments():
    from terrace import _hip
    import terrace.ops as tops
    tops.status()
    ws = torch.zeros(4096, dtype=torch.uint8, device=DEV)
    x = torch.zeros((64, 64), dtype=torch.float32, device=DEV)
    out = torch.zeros((128, 64), dtype=torch.float32, device=DEV)
    s = _hip.stream(DEV)
    lib = _hip.load()
    # a workspace smaller than the first phase's is refused, not read out of bounds
    assert lib.terrace_k2_pack_move(_hip.ptr(x), 1 << 20, 256, 8, 8, 4, _hip.ptr(out), _hip.ptr(ws), 4096, s) == _hip.ENOSPC
    assert lib.terrace_k1_arrival_move(_hip.ptr(x), 1 << 20, 256, 2, 8, _hip.ptr(out), _hip.ptr(ws), 4096, s) == _hip.ENOSPC
    assert lib.terrace_regroup_move(_hip.ptr(x), 1 << 20, 256, 32, -1, _hip.ptr(out), _hip.ptr(ws), 4096, s) == _hip.ENOSPC
    # geometry and null pointers
    assert lib.terrace_k2_pack_move(_hip.ptr(x), 64, 256, 8, 8, 3, _hip.ptr(out), _hip.ptr(ws), 4096, s) == _hip.EINVAL
    assert lib.terrace_k2_pack_move(None, 64, 256, 8, 8, 4, _hip.ptr(out), _hip.ptr(ws), 4096, s) == _hip.EINVAL
    assert lib.terrace_k1_arrival_move(_hip.ptr(x), 64, 256, 0, 8, _hip.ptr(out), _hip.ptr(ws), 4096, s) == _hip.EINVAL
    assert lib.terrace_regroup_move(_hip.ptr(x), 64, 256, 0, -1, _hip.ptr(out), _hip.ptr(ws), 4096, s) == _hip.EINVAL
    # nothing to move is fine without any pointer
    assert lib.terrace_k2_pack_move(None, 0, 256, 8, 8, 4, None, None, 0, s) == _hip.OK
    assert lib.terrace_k1_arrival_move(None, 0, 256, 2, 8, None, None, 0, s) == _hip.OK
    assert lib.terrace_regroup_move(None, 0, 256, 32, -1, None, None, 0, s) == _hip.OK
    torch.cuda.synchronize()


def test_two_host_threads_on_two_streams_do_not_disturb_each_other():
    """The library keeps no state between calls: two host threads, each on a stream of its own, running the
    whole path on different inputs at the same time get bit for bit what they get one after the other."""
    import threading
    from terrace import configs
    from terrace.ta2a_fwd import loopback_combine, loopback_dispatch
    announce("two threads, two streams")
    jobs = []
    for name, T in (("c1", 3000), ("c4", 2500)):
        cfg = configs.CONFIGS[name].scaled(T)
        inp = configs.make_inputs(cfg)
        e, g, _, _ = _route(cfg, inp)
        jobs.append((cfg, configs.rows_to(inp["x"], DEV), e, g.to(cfg.gate_dtype)))

    def run(job):
        cfg, x, e, gates = job
        st = loopback_dispatch(x, e, gates, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups, cfg.capacity(cfg.slots))
        y = loopback_combine(st.permuted, st, out_dtype=cfg.out_dtype)
        return st.permuted, st.place, st.tokens_per_expert, y

    serial = [run(j) for j in jobs]
    torch.cuda.synchronize()
    results, errors = [None, None], []

    def worker(i):
        try:
            with torch.cuda.stream(torch.cuda.Stream()):
                for _ in range(5):
                    out = run(jobs[i])
                torch.cuda.current_stream().synchronize()
                results[i] = out
        except Exception as exc:               # surfaced below: an exception in a thread is otherwise lost
            errors.append(exc)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    torch.cuda.synchronize()
    for want, got in zip(serial, results):
        assert got is not None
        for w, g_ in zip(want, got):
            assert torch.equal(w, g_)


@pytest.mark.parametrize("name,tokens,onepass", [("c2", 2048, False), ("c4", 2048, False), ("c5", 2048, False),
                                                 ("c2", 48, False), ("c2", 48, True), ("c4", 100, True)])
def test_the_whole_step_replays_as_one_hip_graph(name, tokens, onepass):
    """Route, dispatch and combine launch kernels only (no allocation of their own, no memset, no host
    synchronisation), so a step records into a HIP graph; every replay, with eager work and synchronisations
    in between, must reproduce the eager result bit for bit.  The decode-sized cases run the index kernels that
    count for themselves (one workgroup, no count launch, the status block cleared inside the kernel)."""
    import terrace
    from terrace import configs
    from terrace.ta2a_fwd import loopback_combine, loopback_dispatch_onepass
    from terrace.ta2a_fwd import loopback_dispatch as two_step
    loopback_dispatch = loopback_dispatch_onepass if onepass else two_step
    cfg = configs.CONFIGS[name].scaled(tokens)
    announce("graph replay", cfg.name, tokens, onepass)
    inp = configs.make_inputs(cfg)
    logits, bias, x = inp["logits"].to(DEV), inp["bias"].to(DEV), configs.rows_to(inp["x"], DEV)
    ga = None if inp["gate_affinity"] is None else inp["gate_affinity"].to(DEV)
    rcfg = terrace.TRouteConfig(cfg.n_experts, cfg.n_groups, cfg.top_k, cfg.top_groups)
    cap = cfg.capacity(cfg.slots)
    fp8_hidden = cfg.hidden if cfg.fmt == "fp8" else None
    first = loopback_dispatch(x, *terrace.t_route(logits, bias, rcfg, gate_affinity=ga, gates_dtype=cfg.gate_dtype)[:2],
                              cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups, cap)
    ye = first.permuted.clone() if cfg.fmt != "fp8" else configs.quantise_fp8_rows(
        torch.randn(first.permuted.shape[0], cfg.hidden, device=DEV))

    def step():
        e, g, _ = terrace.t_route(logits, bias, rcfg, gate_affinity=ga, gates_dtype=cfg.gate_dtype)
        st = loopback_dispatch(x, e, g, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups, cap)
        return loopback_combine(ye, st, out_dtype=cfg.out_dtype, fp8_hidden=fp8_hidden), st.permuted

    y_eager, p_eager = step()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_graph, p_graph = step()
    for _ in range(3):
        y_graph.zero_(), p_graph.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_graph, y_eager) and torch.equal(p_graph, p_eager)
        y_again, _ = step()
        torch.cuda.synchronize()
        assert torch.equal(y_again, y_eager)


@pytest.mark.parametrize("name", ["reference_shape", "v3_shape", "high_dedup", "capacity", "fp8_rows", "ragged_tail"])
def test_kernels_reproduce_the_committed_fixture(name):
    """The device path against tests/golden/oracle_digests.json directly (no oracle run in between): every plane
    of six formula-made cases, bit for bit."""
    import json
    import os
    import golden_cases as gc
    import terrace
    from terrace.ta2a_fwd import loopback_combine, loopback_dispatch
    announce("fixture", name)
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "oracle_digests.json")) as f:
        want = json.load(f)[name]
    c = gc.inputs(name)
    rcfg = terrace.TRouteConfig(c["E"], c["n_groups"], c["k"], c["M"])
    e, gates, grp = terrace.t_route(torch.from_numpy(c["logits"]).to(DEV), torch.from_numpy(c["bias"]).to(DEV), rcfg)
    x32 = torch.from_numpy(c["x"])
    if c["fmt"] == "f32":
        x, g_pay, out_dtype, fp8_hidden = x32, gates, torch.float32, None
    elif c["fmt"] == "bf16":
        x, g_pay, out_dtype, fp8_hidden = x32.to(torch.bfloat16), gates.to(torch.bfloat16), torch.bfloat16, None
    else:
        x, g_pay, out_dtype, fp8_hidden = torch.from_numpy(orc.fp8_quantise_rows(c["x"])), gates.to(torch.bfloat16), \
            torch.bfloat16, c["H"]
    st = loopback_dispatch(x.to(DEV), e, g_pay.to(DEV), c["world"], c["E"], c["rpn"], c["M"], c["capacity"])
    y = loopback_combine(st.permuted, st, out_dtype=out_dtype, fp8_hidden=fp8_hidden)
    got = dict(expert_idx=e, gates=gates, group_idx=grp, payload=st.payload, mask=st.mask, gate_rows=st.gate_rows,
               u_src=st.u_src, node_counts=st.node_counts, send_buf=st.send_buf, gate_pairs=st.gate_pairs,
               r_idx=st.r_idx, slot_idx=st.slot_idx, i_send=st.i_send, permuted=st.permuted, place=st.place,
               tokens_per_expert=st.tokens_per_expert, y=y)
    if c["capacity"] is not None:
        got["kept"] = st.kept
    from terrace.ta2a_fwd import loopback_dispatch_onepass
    one = loopback_dispatch_onepass(x.to(DEV), e, g_pay.to(DEV), c["world"], c["E"], c["rpn"], c["M"], c["capacity"])
    assert torch.equal(one.permuted, st.permuted)
    got.update(pair_pos=st.pair_pos, pair_src=st.extras["pair_src"], where=st.extras["where"], onepass_place=one.place,
               kept_per_expert=one.extras["kept_per_expert"])
    assert torch.equal(st.extras["kept_per_expert"], one.extras["kept_per_expert"])
    assert sorted(got) == sorted(want)
    wrong = [k for k, v in got.items() if gc.digest(to_np(v)) != want[k]]
    assert not wrong, f"{name}: {wrong} differ from the committed fixture"
