"""HIP path vs the CPU oracle for the general (data-dependent fan-out) branch and the two seam
halves -- through the C ABI only.  Index planes and moved rows bit-exact; the two-level combine
bit-exact against the oracle's fp32 definition and within tolerance of float64."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import equal_quota_routing
from oracle import terrace_oracle as orc
from test_gpu_parity import DEV, DT, announce, same, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _ops_loaded():
    import terrace.ops as tops
    tops.reset()
    assert tops.status().loaded, tops.status().reason
    yield


def _free_routing(T, k, E, seed):
    rng = np.random.default_rng(seed)
    return np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int64)


GEOMS = [(4, 2, 8, 9, 3), (32, 8, 64, 40, 4), (16, 8, 32, 17, 5), (64, 8, 128, 333, 6), (8, 4, 8, 1, 2),
         (64, 8, 256, 3000, 8), (512, 8, 512, 700, 12),
         # more than 64 destination nodes (the reference's general plan has no node bound, terrace/ta2a.py:205-253):
         # 80, 128 and 300 nodes, several experts of a token on one node, a single token, many units
         (640, 8, 1280, 500, 8), (1024, 8, 1024, 257, 12), (600, 2, 2400, 90, 16), (160, 2, 160, 1, 4),
         (1040, 8, 4160, 20000, 6),
         # the widest table the sorts take: 2048 nodes
         (2048, 1, 2048, 700, 8)]


@pytest.mark.parametrize("world,rpn,E,T,k", GEOMS)
@pytest.mark.parametrize("fmt", ["f32", "bf16"])
def test_general_send_side_planes(world, rpn, E, T, k, fmt):
    from terrace import ta2a
    from terrace.ta2a_fwd import build_expansion, general_hopa_planes
    announce("general send", (world, rpn, E, T, k), fmt)
    e = _free_routing(T, k, E, 21)
    slots = (E // world) * rpn
    g = torch.Generator().manual_seed(T)
    x = torch.randn(T, 24, generator=g).to(DT[fmt])
    gates = torch.rand(T, k, generator=g).to(DT[fmt])
    ed = torch.from_numpy(e).to(DEV)
    got = ta2a.plan_ta2a(ed, world, E, rpn)
    want = orc.plan_ta2a(e, world, E, rpn)
    for name, a, b in zip(("u_src", "u_node", "counts", "inverse"), got, want):
        same(a, b, name)
    payload, mask, gate_rows, u_src, counts, inverse, _u_node = general_hopa_planes(x.to(DEV), ed, gates.to(DEV), world, E, rpn)
    same(payload, to_np(x)[want[0]], "payload")
    same(mask, orc.build_expansion(e, want[3], want[0].size, world, E, rpn), "mask")
    same(gate_rows, orc.sparse_gate_plane(e, to_np(gates), want[3], want[0].size, slots), "gate_rows")
    same(u_src, want[0], "u_src"), same(counts, want[2], "counts"), same(inverse, want[3], "inverse")
    # the reference's cheaper formulations give the same bits
    m2 = build_expansion(ed, got[3], got[0].numel(), world, E, rpn, groups_m=None, sorted_rows=True,
                         slot_flat=ed.reshape(-1) % slots)
    assert torch.equal(m2, mask)
    stats = ta2a.dispatch_stats(ed, world, E, rpn)
    assert stats == orc.dispatch_stats(e, world, E, rpn)


def test_general_plan_errors_and_empty():
    from terrace import ta2a
    from terrace.ta2a_fwd import build_expansion
    announce("general plan errors")
    bad = torch.tensor([[0, 2, 99]] * 5, device=DEV)
    with pytest.raises(ValueError, match="out of range"):
        ta2a.plan_ta2a(bad, 4, 8, 2)
    with pytest.raises(ValueError, match="2\\^24"):
        ta2a.plan_ta2a(torch.zeros((1 << 21, 1), dtype=torch.int64, device=DEV), 64, 64, 8)
    with pytest.raises(ValueError, match="exceeds the int64 mask"):
        build_expansion(torch.zeros((2, 2), dtype=torch.int64, device=DEV), torch.zeros(4, dtype=torch.int64, device=DEV),
                        2, 2, 128, 2)
    u_src, u_node, counts, inverse = ta2a.plan_ta2a(torch.zeros((0, 4), dtype=torch.int64, device=DEV), 4, 8, 2)
    assert u_src.numel() == 0 and inverse.numel() == 0 and counts.tolist() == [0, 0]
    # the same on the wide-node form
    with pytest.raises(ValueError, match="out of range"):
        ta2a.plan_ta2a(torch.tensor([[0, 2, 999]] * 5, device=DEV), 400, 800, 4)
    u_src, u_node, counts, inverse = ta2a.plan_ta2a(torch.zeros((0, 4), dtype=torch.int64, device=DEV), 400, 800, 4)
    assert u_src.numel() == 0 and inverse.numel() == 0 and counts.tolist() == [0] * 100


@pytest.mark.parametrize("slots", [1, 5, 16, 24, 25, 40, 63])
def test_expand_arrival_both_forms(slots):
    from terrace.ta2a_fwd import _expand_arrival
    announce("expand", slots)
    rng = np.random.default_rng(slots)
    for R in (0, 1, 70, 5000):
        rmask = rng.integers(0, 1 << slots, size=R, dtype=np.int64)
        if R > 3:
            rmask[3] = 0
        md = torch.from_numpy(rmask).to(DEV)
        r, c = _expand_arrival(md, slots, None)
        wr, wc = orc.expand_arrival(rmask, slots, None)
        same(r, wr, "r_idx"), same(c, wc, "slot_idx")
        for quota in {1, min(2, slots), min(4, slots), slots}:
            r, c = _expand_arrival(md, slots, quota)
            wr, wc = orc.expand_arrival(rmask, slots, quota)
            same(r, wr, f"r_idx q={quota}"), same(c, wc, f"slot_idx q={quota}")


@pytest.mark.parametrize("R,slots,epr,rpn,H,fmt", [(30, 12, 3, 4, 5, "f32"), (700, 32, 4, 8, 64, "bf16"),
                                                    (1, 8, 1, 8, 16, "f16"), (4096, 16, 2, 8, 512, "bf16"),
                                                    # whole-kilobyte rows of other widths
                                                    (257, 8, 1, 8, 256, "f32"), (300, 32, 4, 8, 1536, "bf16")])
def test_arrival_pairs_general(R, slots, epr, rpn, H, fmt):
    import terrace.ops as tops
    announce("arrival_pairs", R, slots, epr, rpn, H, fmt)
    rng = np.random.default_rng(R + slots)
    rmask = rng.integers(0, 1 << slots, size=R, dtype=np.int64)
    r, c = orc.expand_arrival(rmask, slots, None)
    g = torch.Generator().manual_seed(R)
    rx = torch.randn(R, H, generator=g).to(DT[fmt])
    rgate = torch.randn(R, slots, generator=g).to(DT[fmt])
    got = tops.arrival_pairs(rx.to(DEV), torch.from_numpy(r).to(DEV), torch.from_numpy(c).to(DEV), rgate.to(DEV),
                             epr, rpn)
    want = orc.arrival_pairs(to_np(rx), r, c, to_np(rgate), epr, rpn)
    for name, a, b in zip(("send_buf", "gate_pairs", "r_idx", "slot_idx", "i_send", "ordo"), got, want):
        same(a, b, name)
    # no pairs at all
    z = torch.zeros(0, dtype=torch.int64, device=DEV)
    out = tops.arrival_pairs(rx.to(DEV), z, z, rgate.to(DEV), epr, rpn)
    assert out[0].shape == (0, H) and out[4].tolist() == [0] * rpn


@pytest.mark.parametrize("H", [256, 24])
def test_arrival_pairs_row_ids_out_of_range_give_zero_rows(H):
    """A pair naming a row that did not arrive: its place holds a zero row, whichever gather kernel the row width
    takes (whole kilobytes at H = 256 floats, 96-byte rows at H = 24)."""
    import terrace.ops as tops
    from terrace import _hip
    announce("arrival_pairs bad rows", H)
    R, epr, rpn = 50, 2, 4
    rng = np.random.default_rng(H)
    r = np.sort(rng.integers(0, R, size=180)).astype(np.int64)
    c = rng.integers(0, epr * rpn, size=180).astype(np.int64)
    bad = rng.random(180) < 0.1
    r[bad] = np.where(rng.random(bad.sum()) < 0.5, -1, R + 7)
    rx = torch.randn(R, H, generator=torch.Generator().manual_seed(1))
    send, _gp, r_idx, slot_idx, i_send, ordo = tops.arrival_pairs(rx.to(DEV), torch.from_numpy(r).to(DEV),
                                                                  torch.from_numpy(c).to(DEV), None, epr, rpn)
    order = np.argsort(c // epr, kind="stable")
    same(ordo, order.astype(np.int64), "ordo"), same(r_idx, r[order], "r_idx"), same(slot_idx, c[order], "slot_idx")
    want = np.zeros((180, H), dtype=np.float32)
    ok = (r[order] >= 0) & (r[order] < R)
    want[ok] = rx.numpy()[r[order][ok]]
    same(send, want, "send_buf")
    assert int(i_send.sum()) == 180


def test_segment_table_lists_items_in_ascending_order():
    import terrace.ops as tops
    announce("segment_table")
    rng = np.random.default_rng(8)
    for n, n_seg, width in [(0, 5, 3), (40, 7, 40), (5000, 300, 64), (9, 9, 1)]:
        seg = np.sort(rng.integers(0, n_seg, size=n)) if width == 1 and n else rng.integers(0, n_seg, size=n)
        if width == 1:
            seg = rng.permutation(n_seg)[:n]
        table, st = tops.segment_table(torch.from_numpy(seg.astype(np.int64)).to(DEV), n_seg, width)
        want = np.full((n_seg, width), -1, dtype=np.int64)
        for s in range(n_seg):
            items = np.flatnonzero(seg == s)
            want[s, :items.size] = items
        same(table, want, f"table {n},{n_seg},{width}")
        assert st.tolist()[0] == 0
    # overflow and range faults are reported, never written out of bounds
    from terrace import _hip
    seg = torch.tensor([0, 0, 0, 5, -1], device=DEV)
    table, st = tops.segment_table(seg, 2, 2)
    assert st.tolist()[0] == (_hip.FAULT_ID_RANGE | _hip.FAULT_FANOUT)
    assert table.tolist()[1] == [-1, -1] and sorted(table.tolist()[0])[0] >= 0


def test_routing_map_to_topk_and_refusals():
    from terrace.ta2a_dispatch import routing_map_to_topk
    announce("routing_map_to_topk")
    rng = np.random.default_rng(2)
    # E = 24 and 300 take the byte-per-lane census, the others the 16-byte one at every lanes-per-token it has
    # (E/16 = 1 .. 64), with token counts that leave the last wave ragged
    for T, E, k, dt in [(19, 24, 5, torch.float32), (1000, 256, 8, torch.bfloat16), (64, 64, 64, torch.float16),
                        (3, 300, 2, torch.float32), (130, 16, 3, torch.float32), (77, 32, 5, torch.bfloat16),
                        (1031, 128, 8, torch.float32), (65, 512, 9, torch.float16), (33, 1024, 4, torch.float32),
                        (4099, 64, 4, torch.float32)]:
        e = np.sort(np.stack([rng.permutation(E)[:k] for _ in range(T)]), 1)
        rm = np.zeros((T, E), dtype=bool)
        rm[np.arange(T)[:, None], e] = True
        probs = torch.from_numpy(rng.random((T, E)).astype(np.float32)).to(dt)
        ge, gg = routing_map_to_topk(torch.from_numpy(rm).to(DEV), probs.to(DEV))
        we, wg = orc.routing_map_to_topk(rm, to_np(probs))
        same(ge, we, "expert_idx"), same(gg, wg, "gates")
        # a byte map: any non-zero byte means chosen (0x80 and 0xFF included)
        rm8 = rm.astype(np.uint8) * rng.choice(np.array([1, 2, 0x7F, 0x80, 0xFF], dtype=np.uint8), size=rm.shape)
        ge, gg = routing_map_to_topk(torch.from_numpy(rm8).to(DEV), probs.to(DEV))
        same(ge, we, "expert_idx (byte map)"), same(gg, wg, "gates (byte map)")
        if T > 1 and k > 1:          # one token short of an expert, somewhere in the middle
            bad = rm.copy()
            bad[T // 2, e[T // 2, 0]] = False
            with pytest.raises(RuntimeError, match="exactly k experts"):
                routing_map_to_topk(torch.from_numpy(bad).to(DEV), probs.to(DEV))
    bad = rm.copy()
    bad[1, e[1, 0]] = False
    with pytest.raises(RuntimeError, match="exactly k experts"):
        routing_map_to_topk(torch.from_numpy(bad).to(DEV), probs.to(DEV))
    with pytest.raises(RuntimeError, match="all-empty"):
        routing_map_to_topk(torch.zeros(4, 8, dtype=torch.bool, device=DEV), torch.zeros(4, 8, device=DEV))


def _seam_oracle(x_rows, e, gate_bits, world, E, rpn, M, fmt):
    """Dispatch half by the oracle, loop-back: every slot of the node is a local expert."""
    epr, slots = E // world, (E // world) * rpn
    T, k = e.shape
    if M:
        payload, mask, gate_rows, u_src, counts = orc.k2_pack(x_rows, e, gate_bits, world, E, rpn, M)
        send, gp, r_idx, slot_idx, i_send = orc.k1_arrival(payload, mask, gate_rows, k // M, epr, rpn)
    else:
        u_src, _, counts, inverse = orc.plan_ta2a(e, world, E, rpn)
        payload = x_rows[u_src]
        mask = orc.build_expansion(e, inverse, u_src.size, world, E, rpn)
        plane = orc.sparse_gate_plane(e, gate_bits, inverse, u_src.size, slots)
        r_in, s_in = orc.expand_arrival(mask, slots, None)
        send, gp, r_idx, slot_idx, i_send, _ = orc.arrival_pairs(payload, r_in, s_in, plane, epr, rpn)
    permuted, order, tpe = orc.regroup(send, slot_idx, slots)
    return dict(permuted=permuted, tpe=tpe, pprobs=gp[order], u_src=u_src, r_idx=r_idx, order=order,
                R=payload.shape[0])


def _unpermute_oracle(out_rows, o, T, fmt, out_fmt):
    """Two index_add levels as terrace/ta2a_dispatch.py:483-494 writes them, each level in fp32
    with one rounding: a row sums its pairs in arrival order, a token its rows ascending."""
    P = o["order"].size
    place = np.empty(P, dtype=np.int64)
    place[o["order"]] = np.arange(P)
    R = o["R"]
    fan1 = max(int(np.bincount(o["r_idx"], minlength=R).max()), 1) if P else 1
    t1 = np.full((R, fan1), -1, dtype=np.int64)
    fill = np.zeros(R, dtype=np.int64)
    for j in range(P):
        r = o["r_idx"][j]
        t1[r, fill[r]] = place[j]
        fill[r] += 1
    red = orc.combine(out_rows, t1, None, fmt, fmt)
    fan2 = max(int(np.bincount(o["u_src"], minlength=T).max()), 1)
    t2 = np.full((T, fan2), -1, dtype=np.int64)
    fill = np.zeros(T, dtype=np.int64)
    for r in range(R):
        t = o["u_src"][r]
        t2[t, fill[t]] = r
        fill[t] += 1
    return orc.combine(red, t2, None, fmt, out_fmt), t1, t2


SEAM = [(4, 2, 8, 8, 4, 2, 6), (32, 8, 64, 48, 4, 2, 32), (32, 8, 96, 32, 8, 4, 16), (16, 4, 16, 12, 4, 1, 24),
        (64, 8, 256, 1500, 8, 4, 128), (64, 8, 128, 33, 6, 3, 8)]


# every geometry in the default container mode; the other two modes on the small geometries
SEAM_CASES = [(geom, mode) for geom in SEAM for mode in ("small", "full", "off") if mode == "small" or geom[3] <= 100]


@pytest.mark.parametrize("geom,mode", SEAM_CASES)
@pytest.mark.parametrize("fmt", ["f32", "bf16"])
@pytest.mark.parametrize("branch", ["quota", "general"])
def test_seam_halves_loopback(geom, fmt, branch, mode, monkeypatch):
    from terrace import ta2a, ta2a_pack
    from terrace.ta2a_dispatch import ta2a_permute, ta2a_unpermute
    world, rpn, E, T, k, M, H = geom
    assert (E // world) * rpn <= 63, "every seam geometry fits the bitmask branch"
    announce("seam", (world, rpn, E, T, k, M, H), fmt, branch, mode)
    monkeypatch.setenv("TERRACE_TA2A_PACK", mode)
    ta2a_pack.reset()
    ta2a._VERIFIED.clear(), ta2a._VERIFY_COUNT.clear()
    e = equal_quota_routing(T, k, E, world // rpn, M, 31, sort_rows=True)
    g = torch.Generator().manual_seed(T + H)
    x = torch.randn(T, H, generator=g).to(DT[fmt])
    probs = torch.rand(T, E, generator=g).to(DT[fmt])
    rm = torch.zeros(T, E, dtype=torch.bool)
    rm[torch.arange(T)[:, None], torch.from_numpy(e)] = True
    try:
        permuted, tpe, pprobs, st = ta2a_permute(x.to(DEV), probs.to(DEV), rm.to(DEV), world=world, rank=1, rpn=rpn,
                                                 n_experts=E, groups_m=M if branch == "quota" else None)
    finally:
        ta2a_pack.reset()
    gate_bits = np.take_along_axis(to_np(probs), e, 1)
    o = _seam_oracle(to_np(x), e, gate_bits, world, E, rpn, M if branch == "quota" else None, fmt)
    same(permuted, o["permuted"], "permuted"), same(tpe, o["tpe"], "tokens_per_expert")
    same(pprobs, o["pprobs"], "permuted_probs")
    same(st.u_src, o["u_src"], "u_src"), same(st.r_idx, o["r_idx"], "r_idx"), same(st.order, o["order"], "order")
    assert (st.R, st.T, st.hidden, st.dtype) == (o["R"], T, H, DT[fmt])
    # tokens_per_expert is forced by the routing alone: node-local slot histogram
    assert np.array_equal(o["tpe"], np.bincount(e.reshape(-1) % ((E // world) * rpn), minlength=(E // world) * rpn))
    # the vendor's expert layer: a per-row scale by the gate, then the combine half
    slots = (E // world) * rpn
    slot_sorted = torch.repeat_interleave(torch.arange(slots, device=DEV), tpe)
    expert_out = (permuted.float() * ((slot_sorted + 1).float() / slots)[:, None] * pprobs.float()[:, None]).to(DT[fmt])
    y = ta2a_unpermute(expert_out, st, x.to(DEV))
    want, t1, t2 = _unpermute_oracle(to_np(expert_out), o, T, fmt, fmt)
    same(y, want, "y")
    e64 = orc.decode_rows(to_np(expert_out), fmt).astype(np.float64)
    red64 = np.where((t1 >= 0)[:, :, None], e64[np.maximum(t1, 0)], 0.0).sum(1)
    y64 = np.where((t2 >= 0)[:, :, None], red64[np.maximum(t2, 0)], 0.0).sum(1)
    tol = 1e-5 if fmt == "f32" else 1e-2
    assert np.abs(orc.decode_rows(to_np(y), fmt) - y64).max() <= tol * (np.abs(y64).max() + 1e-30)
    # ... which is the one-level definition y[t] = sum_j gate[t,j] * f(x[t], e[t,j])
    x64 = orc.decode_rows(to_np(x), fmt).astype(np.float64)
    direct = np.zeros((T, H))
    for j in range(k):
        direct += x64 * ((e[:, j] % slots + 1) / slots)[:, None] * orc.decode_rows(gate_bits, fmt).astype(np.float64)[:, j:j + 1]
    assert np.abs(y64 - direct).max() <= (2e-6 if fmt == "f32" else 2e-2) * (np.abs(direct).max() + 1e-30)


@pytest.mark.parametrize("world,rpn,E,T,k,M,H", [(4, 2, 8, 8, 4, 2, 6), (32, 8, 64, 48, 4, 2, 32),
                                                   (64, 8, 256, 700, 8, 4, 64), (16, 4, 16, 12, 4, 1, 24)])
@pytest.mark.parametrize("branch", ["quota", "general"])
def test_seam_backward_is_the_adjoint(world, rpn, E, T, k, M, H, branch):
    """Gradients of both halves against torch autograd (float64, CPU) over the same map written
    with index ops: permuted = x[token_of_place], probs gathered at (token, expert) of each place,
    y = index_add by token.  The tables themselves are checked bit-exact against the oracle."""
    from terrace import ta2a
    from terrace.ta2a_dispatch import ta2a_permute, ta2a_unpermute
    if (E // world) * rpn > 63 and branch == "general":
        pytest.skip("bitmask branch needs <= 63 slots per node")
    announce("seam backward", (world, rpn, E, T, k, M, H), branch)
    ta2a._VERIFIED.clear(), ta2a._VERIFY_COUNT.clear()
    slots = (E // world) * rpn
    e = equal_quota_routing(T, k, E, world // rpn, M, 77, sort_rows=True)
    g = torch.Generator().manual_seed(T * H)
    x = torch.randn(T, H, generator=g)
    probs = torch.rand(T, E, generator=g)
    G = torch.randn(T, H, generator=g)
    rm = torch.zeros(T, E, dtype=torch.bool)
    rm[torch.arange(T)[:, None], torch.from_numpy(e)] = True
    xd, pd = x.to(DEV).requires_grad_(), probs.to(DEV).requires_grad_()
    permuted, tpe, pprobs, st = ta2a_permute(xd, pd, rm.to(DEV), world=world, rank=0, rpn=rpn, n_experts=E,
                                             groups_m=M if branch == "quota" else None)
    o = _seam_oracle(x.numpy(), e, np.take_along_axis(probs.numpy(), e, 1), world, E, rpn,
                     M if branch == "quota" else None, "f32")
    _, u_node, _, _ = orc.plan_ta2a(e, world, E, rpn)
    slot_sorted_np = np.repeat(np.arange(slots), o["tpe"])
    # slot id of each arrival row, recovered from the expert-order histogram
    slot_of_arrival = np.empty(o["order"].size, dtype=np.int64)
    slot_of_arrival[o["order"]] = slot_sorted_np
    where, tok = orc.pair_places(o["order"], o["r_idx"], slot_of_arrival, o["u_src"], u_node, e, slots)
    same(st.where, where, "where"), same(st.token_of_place, tok, "token_of_place")
    scale = ((torch.repeat_interleave(torch.arange(slots, device=DEV), tpe) + 1).float() / slots)[:, None]
    expert_out = permuted * scale * pprobs[:, None]
    assert expert_out.requires_grad
    y = ta2a_unpermute(expert_out, st, xd)
    (y * G.to(DEV)).sum().backward()
    # reference: the same map with index ops, float64 autograd on the CPU
    x64, p64 = x.double().requires_grad_(), probs.double().requires_grad_()
    tok_t = torch.from_numpy(tok)
    exp_of_place = torch.from_numpy(e)[tok_t][torch.from_numpy(where)[tok_t] == torch.arange(tok.size)[:, None]]
    perm64 = x64[tok_t]
    pp64 = p64[tok_t, exp_of_place]
    eo64 = perm64 * scale.cpu().double() * pp64[:, None]
    y64 = torch.zeros(T, H, dtype=torch.float64).index_add(0, tok_t, eo64)
    (y64 * G.double()).sum().backward()
    assert np.abs(y.detach().cpu().double().numpy() - y64.detach().numpy()).max() <= 1e-5 * float(y64.detach().abs().max())
    for name, got, want in (("x.grad", xd.grad, x64.grad), ("probs.grad", pd.grad, p64.grad)):
        assert got is not None, f"{name} is missing: the edge is not attached"
        err = (got.cpu().double() - want).abs().max().item()
        assert err <= 1e-5 * max(want.abs().max().item(), 1.0), f"{name} differs by {err}"
    # probs.grad is zero exactly where the routing map is
    assert torch.equal(pd.grad.cpu() != 0, rm) or (pd.grad.cpu()[~rm] == 0).all()
    # without grad mode nothing is attached
    with torch.no_grad():
        p2, _, g2, st2 = ta2a_permute(xd, pd, rm.to(DEV), world=world, rank=0, rpn=rpn, n_experts=E,
                                      groups_m=M if branch == "quota" else None)
    assert not p2.requires_grad and not g2.requires_grad and torch.equal(p2, permuted.detach())


@pytest.mark.parametrize("fmt", ["f32", "bf16", "f16"])
def test_stage_kernels_write_and_read_the_wire_containers_themselves(literals, fmt):
    """The zero-copy forms against the two-step forms (planes, then pack / unpack kernels): the same
    container bits, padding included, and the same downstream planes."""
    import terrace.ops as tops
    from terrace import ta2a_pack
    for world, rpn, E, T, k, M in literals["k2_geometries"]["rows"] + [[64, 8, 256, 3000, 8, 4], [64, 8, 256, 700, 24, 2], [1024, 8, 1024, 300, 4, 2]]:
        announce("wire", (world, rpn, E, T, k, M), fmt)
        q, epr, slots = k // M, E // world, (E // world) * rpn
        e = equal_quota_routing(T, k, E, world // rpn, M, 13)
        g = torch.Generator().manual_seed(T)
        x = torch.randn(T, 32, generator=g).to(DT[fmt]).to(DEV)
        gates = torch.rand(T, k, generator=g).to(DT[fmt]).to(DEV)
        ed = torch.from_numpy(e).to(DEV)
        plain, pex = tops.k2_pack_raw(x, ed, gates, world, E, rpn, M, extras=True)
        fused, fex = tops.k2_pack_wire(x, ed, gates, world, E, rpn, M)
        want_wire, lay = ta2a_pack.hopa_pack_small(plain[2], plain[1])
        assert fex["wire"].shape == want_wire.shape == (T * M, lay.words)
        assert torch.equal(fex["wire"], want_wire)
        for a, b in zip(fused, plain):
            assert torch.equal(a, b)
        for name in ("u_node", "inverse", "node_offsets", "pair_table", "sort_order", "token_rows", "gate_sorted"):
            assert torch.equal(fex[name], pex[name]), name
        assert fex["status"].tolist() == pex["status"].tolist()
        # arrival: reads the container, writes the Hop-B container
        send, gp, r_idx, slot_idx, i_send, pair_pos = tops.k1_arrival_raw(plain[0], plain[1], plain[2], q, epr, rpn, 0,
                                                                          want_pair_pos=True)
        send2, meta, r_idx2, i_send2, pair_pos2 = tops.k1_arrival_wire(fused[0], fex["wire"], DT[fmt], q, epr, rpn, 0)
        assert torch.equal(meta, ta2a_pack.hopb_pack_meta(slot_idx, gp))
        for a, b in ((send2, send), (r_idx2, r_idx), (i_send2, i_send), (pair_pos2, pair_pos)):
            assert torch.equal(a, b)
        # expert card: reads the Hop-B container
        perm, order, tpe, pgate = tops.regroup(send, slot_idx, slots, 0, None, my_gate=gp)
        perm2, order2, tpe2, place2, pgate2 = tops.regroup_wire(send2, meta, DT[fmt], slots, 0)
        for a, b in ((perm2, perm), (order2, order), (tpe2, tpe), (pgate2, pgate)):
            assert torch.equal(a, b)
        assert torch.equal(place2[order2], torch.arange(order2.numel(), device=DEV))
    with pytest.raises(RuntimeError, match="cannot hold"):
        tops.k1_arrival_wire(torch.zeros(4, 8, device=DEV), torch.zeros(4, 2, dtype=torch.int64, device=DEV),
                             torch.float32, 2, 1, 4, 0)
    empty = tops.k1_arrival_wire(torch.zeros(0, 8, device=DEV), torch.zeros(0, 3, dtype=torch.int64, device=DEV),
                                 torch.float32, 2, 1, 4, 0)
    assert empty[1].shape == (0, 2) and empty[3].tolist() == [0, 0, 0, 0]


def test_seam_refuses_process_groups_and_mismatched_probs():
    from terrace.ta2a_dispatch import ta2a_permute
    announce("seam refusals")
    x = torch.randn(4, 8, device=DEV)
    rm = torch.zeros(4, 8, dtype=torch.bool, device=DEV)
    rm[:, [0, 2, 4, 6]] = True
    with pytest.raises(NotImplementedError, match="loop-back"):
        ta2a_permute(x, torch.rand(4, 8, device=DEV), rm, world=4, rank=0, rpn=2, n_experts=8, intra_group=object(),
                     groups_m=2)
    with pytest.raises(RuntimeError, match="dtypes match"):
        ta2a_permute(x.bfloat16(), torch.rand(4, 8, device=DEV), rm, world=4, rank=0, rpn=2, n_experts=8, groups_m=2)


# ------------------------------------------------------------------------------- the overlap seam

@pytest.mark.parametrize("world,rpn,E,T,k,M,H", [(4, 2, 8, 8, 4, 2, 6), (32, 8, 64, 48, 4, 2, 32), (64, 8, 256, 300, 8, 4, 64)])
@pytest.mark.parametrize("branch", ["quota", "general"])
@pytest.mark.parametrize("pack_mode", ["small", "off"])
def test_overlap_seam_seats_and_hand_replayed_backward(world, rpn, E, T, k, M, H, branch, pack_mode, monkeypatch):
    """The overlap halves append 7 + 3 save_tensors entries at the positions the vendor layer's hand-written
    backward unpacks (terrace/ta2a_dispatch.py:519-535 of the reference), give the forward values of the plain
    halves, and -- replayed segment by segment the way that backward does it -- the plain halves' gradients."""
    from terrace import ta2a, ta2a_pack
    from terrace.ta2a_dispatch import (ta2a_permute, ta2a_permute_overlap, ta2a_unpermute, ta2a_unpermute_overlap)
    if (E // world) * rpn > 63 and branch == "general":
        pytest.skip("bitmask branch needs <= 63 slots per node")
    announce("overlap seam", (world, rpn, E, T, k, M, H), branch, pack_mode)
    monkeypatch.setenv("TERRACE_TA2A_PACK", pack_mode)
    ta2a_pack.reset()
    ta2a._VERIFIED.clear(), ta2a._VERIFY_COUNT.clear()
    slots = (E // world) * rpn
    gm = M if branch == "quota" else None
    e = equal_quota_routing(T, k, E, world // rpn, M, 91, sort_rows=True)
    g = torch.Generator().manual_seed(T + H)
    x, probs, G = torch.randn(T, H, generator=g), torch.rand(T, E, generator=g), torch.randn(T, H, generator=g)
    rm = torch.zeros(T, E, dtype=torch.bool)
    rm[torch.arange(T)[:, None], torch.from_numpy(e)] = True
    geom = dict(world=world, rank=0, rpn=rpn, n_experts=E, groups_m=gm)
    # ---- the plain halves: values and gradients to match
    xp, pp = x.to(DEV).requires_grad_(), probs.to(DEV).requires_grad_()
    permuted0, tpe0, pprobs0, st0 = ta2a_permute(xp, pp, rm.to(DEV), **geom)
    scale = ((torch.repeat_interleave(torch.arange(slots, device=DEV), tpe0) + 1).float() / slots)[:, None]
    y0 = ta2a_unpermute(permuted0 * scale * pprobs0[:, None], st0, xp)
    (y0 * G.to(DEV)).sum().backward()
    # ---- the overlap halves
    xd, pd = x.to(DEV).requires_grad_(), probs.to(DEV).requires_grad_()
    save, calls = [], []
    permuted, tpe, pprobs, shared, st = ta2a_permute_overlap(
        xd, pd, rm.to(DEV), save_tensors=save, run_shared_experts=lambda: calls.append(len(save)) or "shared", **geom)
    assert shared == "shared" and calls == [2], "the shared-expert callback runs once, after Hop A is launched"
    assert len(save) == 7 and save[2] is None
    assert save[4] is permuted and save[6] is pprobs
    assert save[3].is_leaf and save[3].requires_grad and save[5].is_leaf and save[5].requires_grad
    assert save[0].requires_grad and save[1].requires_grad and not save[0].is_leaf and not save[1].is_leaf
    assert save[0].shape == save[3].shape and save[1].shape == save[5].shape
    assert torch.equal(permuted.detach(), permuted0.detach()) and torch.equal(pprobs.detach(), pprobs0.detach())
    assert torch.equal(tpe, tpe0) and torch.equal(save[3].detach(), save[0].detach())
    # the expert layer is a segment of its own, on detached leaves
    p_in, pp_in = permuted.detach().requires_grad_(), pprobs.detach().requires_grad_()
    eo = p_in * scale * pp_in[:, None]
    y = ta2a_unpermute_overlap(eo.detach(), st, save, out_shape=(T, H))
    assert len(save) == 10 and save[7].is_leaf and save[9].is_leaf and not save[8].is_leaf
    assert torch.equal(y.detach(), y0.detach())
    # ---- the backward, replayed by fixed position
    y.backward(G.to(DEV))
    save[8].backward(save[9].grad)                 # Hop A's reverse is loop-back: the leaf's gradient is the row's
    eo.backward(save[7].grad)
    save[4].backward(p_in.grad)
    save[6].backward(pp_in.grad)
    save[0].backward(save[3].grad)
    save[1].backward(save[5].grad)
    for name, got, want in (("hidden.grad", xd.grad, xp.grad), ("probs.grad", pd.grad, pp.grad)):
        assert got is not None, f"{name} is missing"
        err = (got - want).abs().max().item()
        assert err <= 1e-5 * max(want.abs().max().item(), 1.0), f"{name} differs by {err}"
    ta2a_pack.reset()


def test_overlap_seam_switches(monkeypatch):
    from terrace import ta2a_dispatch as td
    monkeypatch.delenv("TERRACE_TA2A", raising=False)
    assert not td.ta2a_enabled(128, 8)
    monkeypatch.setenv("TERRACE_TA2A", "1")
    assert td.ta2a_enabled(128, 8) and td.ta2a_enabled(16, 8) and not td.ta2a_enabled(8, 8)
    td.reset_shared_overlap()
    monkeypatch.setenv("TERRACE_SHARED_OVERLAP", "0")
    assert not td.shared_overlap_enabled()
    td.reset_shared_overlap()
    monkeypatch.delenv("TERRACE_SHARED_OVERLAP")
    assert td.shared_overlap_enabled()
    # with the switch off the callback runs after every dispatch exchange: all seven seats are filled by then
    from terrace import ta2a
    ta2a._VERIFIED.clear(), ta2a._VERIFY_COUNT.clear()
    monkeypatch.setenv("TERRACE_SHARED_OVERLAP", "0")
    td.reset_shared_overlap()
    e = equal_quota_routing(8, 4, 8, 2, 2, 5, sort_rows=True)
    rm = torch.zeros(8, 8, dtype=torch.bool)
    rm[torch.arange(8)[:, None], torch.from_numpy(e)] = True
    save, calls = [], []
    td.ta2a_permute_overlap(torch.randn(8, 6, device=DEV), torch.rand(8, 8, device=DEV), rm.to(DEV), world=4, rank=0,
                            rpn=2, n_experts=8, groups_m=2, save_tensors=save,
                            run_shared_experts=lambda: calls.append(len(save)))
    assert calls == [7]
    td.reset_shared_overlap()


# ---------------------------------------------------------------------------------------------
# the two combine levels in one pass (terrace_combine_two_level)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("fmt,out_fmt", [("f32", "f32"), ("bf16", "bf16"), ("f16", "f16"), ("bf16", "f32"),
                                         ("f32", "bf16")])
@pytest.mark.parametrize("q,M,H", [(1, 3, 64), (2, 4, 512), (4, 2, 1024), (8, 1, 72), (2, 5, 8), (4, 9, 520)])
def test_two_level_combine_in_one_pass(fmt, out_fmt, q, M, H):
    """Against the oracle's two fp32 levels (round to the source format between them) and against the two launches,
    bit for bit: tables with dead entries at both levels (negative and past-the-end ids), outer fans that do not fill
    the last batch of rows, widths on the one-wave and the 256-lane shape."""
    import terrace.ops as tops
    announce("two-level combine", fmt, out_fmt, (q, M, H))
    rng = np.random.default_rng(q * 100 + M)
    n_src, R, T = 301, 97, 53
    src = torch.from_numpy(rng.standard_normal((n_src, H)).astype(np.float32)).to(DT[fmt])
    inner = rng.integers(0, n_src, size=(R, q)).astype(np.int64)
    inner[rng.random((R, q)) < 0.15] = -1
    inner[3, 0] = n_src + 5                     # past the end: dead
    outer = rng.integers(0, R, size=(T, M)).astype(np.int64)
    outer[rng.random((T, M)) < 0.2] = -1
    outer[7, 0] = R                             # past the end: dead
    outer[11, :] = -1                           # a token with no rows at all: a zero row
    want_red = orc.combine(to_np(src), np.where((inner >= 0) & (inner < n_src), inner, -1), None, fmt, fmt)
    want = orc.combine(want_red, np.where((outer >= 0) & (outer < R), outer, -1), None, fmt, out_fmt)
    sd, ind, outd = src.to(DEV), torch.from_numpy(inner).to(DEV), torch.from_numpy(outer).to(DEV)
    got = tops.combine_two_level(sd, ind, outd, out_dtype=DT[out_fmt])
    same(got, want, "one pass vs the oracle's two levels")
    two = tops.combine(tops.combine(sd, ind, None, out_dtype=sd.dtype), outd, None, out_dtype=DT[out_fmt])
    assert torch.equal(got.view(torch.uint8), two.view(torch.uint8)), "one pass differs from the two launches"


def test_two_level_combine_shapes_outside_the_one_pass_form():
    """An inner table three ids wide, and rows that are not 16-byte multiples: the operator runs the two levels one
    after the other and gives the same definition."""
    import terrace.ops as tops
    announce("two-level combine, fallback shapes")
    rng = np.random.default_rng(5)
    for q, H in [(3, 64), (2, 7)]:
        src = torch.from_numpy(rng.standard_normal((40, H)).astype(np.float32))
        inner = rng.integers(-1, 40, size=(19, q)).astype(np.int64)
        outer = rng.integers(-1, 19, size=(11, 2)).astype(np.int64)
        want = orc.combine(orc.combine(to_np(src), inner, None, "f32", "f32"), outer, None, "f32", "f32")
        got = tops.combine_two_level(src.to(DEV), torch.from_numpy(inner).to(DEV), torch.from_numpy(outer).to(DEV))
        same(got, want, f"fallback q={q} H={H}")
