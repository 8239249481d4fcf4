"""HIP path vs the CPU oracle on identical seeded inputs -- through the C ABI (ctypes) only.

Bit-exact for every index / count / offset plane and every moved row; the combine is
bit-exact against the oracle's fp32 left-to-right definition and within the stated
tolerance (1e-5 fp32, 1e-2 bf16) of a float64 evaluation of the same sum.
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import arrival_plane, equal_quota_routing
from oracle import terrace_oracle as orc

pytestmark = pytest.mark.gpu

DEV = "cuda"
DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def announce(*what):
    print("[case]", *what, flush=True)


def to_np(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.bool:
        return t.numpy()
    return t.numpy()


def rows_of(x_f32: torch.Tensor, fmt: str) -> torch.Tensor:
    return x_f32.to(DT[fmt])


def same(a: torch.Tensor, b: np.ndarray, what: str):
    got = to_np(a)
    assert got.shape == tuple(b.shape), f"{what}: shape {got.shape} != {b.shape}"
    assert got.dtype == b.dtype, f"{what}: dtype {got.dtype} != {b.dtype}"
    assert np.array_equal(got, b), f"{what}: values differ"


@pytest.fixture(scope="module", autouse=True)
def _ops_loaded():
    import terrace.ops as tops
    tops.reset()
    assert tops.status().loaded, tops.status().reason
    yield


# ------------------------------------------------------------------------------- passthrough

@pytest.mark.parametrize("shape,dtype", [((0,), torch.float32), ((1,), torch.uint8), ((17,), torch.uint8),
                                          ((33, 7), torch.bfloat16), ((4096, 1024), torch.float32),
                                          ((1000, 7168), torch.bfloat16)])
def test_passthrough_is_a_bitwise_copy(shape, dtype):
    import terrace.ops as tops
    announce("passthrough", shape, dtype)
    g = torch.Generator().manual_seed(1)
    x = torch.randint(0, 255, shape, generator=g, dtype=torch.uint8) if dtype == torch.uint8 else \
        torch.randn(shape, generator=g).to(dtype)
    xd = x.to(DEV)
    y = tops.passthrough(xd)
    assert y.data_ptr() != xd.data_ptr() or xd.numel() == 0
    assert y.dtype == x.dtype and y.shape == x.shape and torch.equal(y.cpu(), x)
    assert torch.equal(torch.ops.terrace.passthrough(xd).cpu(), x)


def test_stream_probes_do_what_they_are_priced_for():
    """The benchmark prices the probes by the bytes they are said to move: the copy must copy, the 8:1 sum must be
    the fp32 sum of eight bf16 streams scaled by 1/8 and rounded once, the write probe must write every vector and
    the read probe must leave its destination alone."""
    import terrace.ops as tops
    announce("stream probes")
    n = 1 << 20                                            # bytes written
    g = torch.Generator().manual_seed(3)
    src = torch.randn(8 * n // 2, generator=g).to(torch.bfloat16).to(DEV)
    out = torch.full((n // 2,), 7.0, dtype=torch.bfloat16, device=DEV)
    tops.stream_probe("copy", src, out)
    assert torch.equal(out.view(torch.int16), src[: n // 2].view(torch.int16))
    tops.stream_probe("sum8", src, out)
    parts = src.view(8, n // 2).float()
    acc = torch.zeros(n // 2, device=DEV)
    for j in range(8):
        acc = acc + parts[j] * 0.125
    assert torch.equal(out.view(torch.int16), acc.to(torch.bfloat16).view(torch.int16))
    out.fill_(7.0)
    tops.stream_probe("read", torch.zeros(n, dtype=torch.uint8, device=DEV), out.view(torch.uint8))
    assert bool((out == 7.0).all())
    tops.stream_probe("write", None, out)
    words = out.view(torch.int32).view(-1, 4).cpu()
    assert torch.equal(words[:, 0], torch.arange(n // 16, dtype=torch.int32)) and bool((words[:, 1:] == torch.tensor([1, 2, 3])).all())
    with pytest.raises(RuntimeError):
        tops.stream_probe("copy", src, out[:1000])          # not a multiple of 8192 bytes


# ------------------------------------------------------------------------------- routing

ROUTE_GEOMS = [  # (T, E, N_g, k, M)
    (512, 64, 8, 8, 4), (4096, 64, 8, 4, 2), (2048, 256, 8, 8, 4), (1024, 128, 16, 8, 2),
    (257, 16, 4, 4, 2), (33, 24, 3, 6, 3), (64, 8, 8, 2, 2), (100, 32, 1, 4, 1), (65, 96, 4, 8, 4),
    (31, 512, 8, 8, 4), (9, 1024, 8, 16, 4), (40, 40, 5, 4, 2),
]


@pytest.mark.parametrize("geom", ROUTE_GEOMS, ids=lambda g: "T%dE%dG%dk%dM%d" % g)
@pytest.mark.parametrize("generic", [False, True])
def test_route_full_bit_exact(geom, generic):
    import terrace
    T, E, Ng, k, M = geom
    announce("route", geom, "generic" if generic else "auto")
    g = torch.Generator().manual_seed(T + E)
    logits = torch.randn(T, E, generator=g)
    bias = torch.randn(E, generator=g) * 0.1
    cfg = terrace.TRouteConfig(E, Ng, k, M)
    e, gt, grp = terrace.t_route(logits.to(DEV), bias.to(DEV), cfg, _force_generic=generic)
    oe, og, ogrp = orc.t_route(logits.numpy(), bias.numpy(), E, Ng, k, M)
    same(e, oe, "expert_idx"), same(grp, ogrp, "group_idx"), same(gt, og, "gates")
    # sigmoid affinities with a separate gate table
    aff = torch.sigmoid(logits)
    gate_tab = torch.exp(logits - logits.max(-1, keepdim=True).values)
    e, gt, grp = terrace.t_route(aff.to(DEV), bias.to(DEV), cfg, gate_affinity=gate_tab.to(DEV),
                                 _force_generic=generic)
    oe, og, ogrp = orc.t_route(aff.numpy(), bias.numpy(), E, Ng, k, M, gate_affinity=gate_tab.numpy())
    same(e, oe, "expert_idx"), same(grp, ogrp, "group_idx"), same(gt, og, "gates")


@pytest.mark.parametrize("generic", [False, True])
def test_route_ties_and_pool(generic):
    import terrace
    announce("route ties", generic)
    aff = torch.full((5, 64), 0.5)
    aff[1, 10] = 0.75
    aff[2, 63] = 0.25
    aff[3] = torch.arange(64).float().div(64).roll(7)
    aff[4, ::2] = 0.125
    zero = torch.zeros(64)
    for pool in (1, 2):
        cfg = terrace.TRouteConfig(64, 8, 8, 4, group_score_pool=pool)
        e, gt, grp = terrace.t_route(aff.to(DEV), zero.to(DEV), cfg, _force_generic=generic)
        oe, og, ogrp = orc.t_route(aff.numpy(), zero.numpy(), 64, 8, 8, 4, pool=pool)
        same(e, oe, "expert_idx"), same(grp, ogrp, "group_idx"), same(gt, og, "gates")
    assert to_np(e)[0].tolist() == [0, 1, 8, 9, 16, 17, 24, 25]


@pytest.mark.parametrize("mode", ["full", "group_limited"])
@pytest.mark.parametrize("pool", [3, 4, 5, 8, 100])
def test_route_group_score_pool_beyond_two(mode, pool):
    """mean of the top-min(pool, g) scores of a group (terrace/routing.py:24,88), any pool: bit-exact against the
    oracle's largest-first fp32 sum, ties and all-equal tokens included."""
    import terrace
    announce("route pool", mode, pool)
    g = torch.Generator().manual_seed(pool)
    for (T, E, Ng, k, M) in [(300, 64, 8, 8, 4), (130, 256, 8, 8, 4), (65, 24, 3, 6, 3), (40, 16, 8, 2, 2),
                             (50, 96, 4, 8, 2)]:
        aff = torch.rand(T, E, generator=g)
        aff[1] = 0.5
        aff[2, ::3] = 0.25
        bias = torch.randn(E, generator=g) * 0.05
        cfg = terrace.TRouteConfig(E, Ng, k, M, group_score_pool=pool)
        e, gt, grp = terrace.t_route(aff.to(DEV), bias.to(DEV), cfg, mode=mode)
        oe, og, ogrp = orc.t_route(aff.numpy(), bias.numpy(), E, Ng, k, M, pool=pool, mode=mode)
        same(e, oe, "expert_idx"), same(grp, ogrp, "group_idx"), same(gt, og, "gates")


@pytest.mark.parametrize("mode", ["group_limited", "quota_only", "global_topk"])
def test_route_other_modes(mode):
    import terrace
    announce("route mode", mode)
    g = torch.Generator().manual_seed(11)
    for (T, E, Ng, k, M) in [(300, 64, 8, 8, 4), (77, 32, 4, 8, 2), (50, 256, 8, 8, 4)]:
        aff = torch.rand(T, E, generator=g)
        bias = torch.randn(E, generator=g) * 0.05
        cfg = terrace.TRouteConfig(E, Ng, k, M)
        e, gt, grp = terrace.t_route(aff.to(DEV), bias.to(DEV), cfg, mode=mode)
        oe, og, ogrp = orc.t_route(aff.numpy(), bias.numpy(), E, Ng, k, M, mode=mode)
        same(e, oe, "expert_idx"), same(grp, ogrp, "group_idx"), same(gt, og, "gates")


@pytest.mark.parametrize("generic", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_route_gates_in_the_payload_dtype(generic, dtype):
    """gates_dtype: the kernel's 16-bit gates are the fp32 gates rounded to nearest-even -- the bits of torch's
    own cast (and of the oracle's) -- and nothing else of the result moves."""
    import terrace
    announce("route gates dtype", generic, dtype)
    g = torch.Generator().manual_seed(3)
    for (T, E, Ng, k, M) in [(2048, 256, 8, 8, 4), (700, 64, 8, 4, 2), (65, 96, 4, 8, 4), (300, 128, 16, 8, 2)]:
        logits = torch.randn(T, E, generator=g)
        bias = torch.randn(E, generator=g) * 0.1
        gate_tab = torch.exp(logits - logits.max(-1, keepdim=True).values)
        cfg = terrace.TRouteConfig(E, Ng, k, M)
        args = (logits.to(DEV), bias.to(DEV), cfg)
        e32, g32, grp32 = terrace.t_route(*args, gate_affinity=gate_tab.to(DEV), _force_generic=generic)
        e16, g16, grp16 = terrace.t_route(*args, gate_affinity=gate_tab.to(DEV), gates_dtype=dtype,
                                          _force_generic=generic)
        assert g16.dtype == dtype and torch.equal(e16, e32) and torch.equal(grp16, grp32)
        assert torch.equal(g16, g32.to(dtype))
        _, og, _ = orc.t_route(logits.numpy(), bias.numpy(), E, Ng, k, M, gate_affinity=gate_tab.numpy())
        assert torch.equal(g16.cpu(), torch.from_numpy(og).to(dtype))
    for mode in ("group_limited", "quota_only", "global_topk"):
        cfg = terrace.TRouteConfig(64, 8, 8, 4)
        aff = torch.rand(200, 64, generator=g).to(DEV)
        zero = torch.zeros(64, device=DEV)
        _, g32, _ = terrace.t_route(aff, zero, cfg, mode=mode)
        _, g16, _ = terrace.t_route(aff, zero, cfg, mode=mode, gates_dtype=dtype)
        assert torch.equal(g16, g32.to(dtype))
    with pytest.raises(ValueError):
        terrace.t_route(aff, zero, cfg, gates_dtype=torch.float64)


@pytest.mark.parametrize("generic", [False, True])
def test_route_with_masked_experts(generic):
    """A bias of -inf is how a caller switches an expert off.  With at least two live experts left in every
    group nothing but the order (value descending, index ascending, -inf last) is involved: bit-exact against
    the oracle, and no masked expert is ever picked while its group has q live ones."""
    import terrace
    announce("route masked", generic)
    g = torch.Generator().manual_seed(21)
    for (T, E, Ng, k, M) in [(1500, 256, 8, 8, 4), (700, 64, 8, 4, 2), (300, 128, 16, 8, 2)]:
        gs, q = E // Ng, k // M
        logits = torch.randn(T, E, generator=g)
        bias = torch.randn(E, generator=g) * 0.1
        dead = torch.zeros(E, dtype=torch.bool)
        for grp in range(Ng):                                      # switch off all but q+1 .. gs experts of each group
            n_dead = int(torch.randint(0, gs - q, (1,), generator=g))
            dead[grp * gs + torch.randperm(gs, generator=g)[:n_dead]] = True
        bias[dead] = -float("inf")
        cfg = terrace.TRouteConfig(E, Ng, k, M)
        e, gt, grp_idx = terrace.t_route(logits.to(DEV), bias.to(DEV), cfg, _force_generic=generic)
        oe, og, ogrp = orc.t_route(logits.numpy(), bias.numpy(), E, Ng, k, M)
        same(e, oe, "expert_idx"), same(grp_idx, ogrp, "group_idx"), same(gt, og, "gates")
        assert not bool(dead.to(DEV)[e].any())


@pytest.mark.parametrize("generic", [False, True])
def test_route_contains_nan_scores(generic):
    """NaN affinities mean a broken model, not a defined routing; what is promised is containment: every id
    written is a valid expert (or, for group_idx, the no-group sentinel), clean tokens of the same batch are
    routed as if the bad ones were not there, and nothing hangs."""
    import terrace
    announce("route nan", generic)
    T, E, Ng, k, M = 512, 256, 8, 8, 4
    g = torch.Generator().manual_seed(22)
    logits = torch.randn(T, E, generator=g)
    bad = torch.zeros(T, dtype=torch.bool)
    bad[::7] = True
    poisoned = logits.clone()
    poisoned[bad, ::3] = float("nan")
    poisoned[5 * 7] = float("nan")                                   # one token with nothing but NaN
    zero = torch.zeros(E)
    cfg = terrace.TRouteConfig(E, Ng, k, M)
    e, gt, grp = terrace.t_route(poisoned.to(DEV), zero.to(DEV), cfg, _force_generic=generic)
    torch.cuda.synchronize()
    assert bool(((e >= 0) & (e < E)).all())
    assert bool(((grp >= 0) & (grp < Ng) | (grp == 0x7FFFFFFF)).all())
    oe, og, ogrp = orc.t_route(logits.numpy(), zero.numpy(), E, Ng, k, M)
    ok = ~bad
    assert np.array_equal(to_np(e)[ok.numpy()], oe[ok.numpy()]) and np.array_equal(to_np(gt)[ok.numpy()], og[ok.numpy()])
    assert np.array_equal(to_np(grp)[ok.numpy()], ogrp[ok.numpy()])


@pytest.mark.parametrize("mode", ["full", "group_limited", "quota_only", "global_topk"])
@pytest.mark.parametrize("E,Ng,k,M", [(8, 8, 8, 8), (64, 8, 8, 4), (48, 6, 6, 3)])
def test_route_nan_rows_are_contained_and_repeatable_in_every_mode(mode, E, Ng, k, M):
    """A token whose scores are all NaN ranks nothing: in every mode its ids must be valid experts, the same on every
    run (what is written must not depend on what a workgroup's LDS held), and the tokens beside it untouched."""
    import terrace
    announce("route nan, every mode", mode, (E, Ng, k, M))
    T = 300
    g = torch.Generator().manual_seed(E + k)
    logits = torch.randn(T, E, generator=g)
    poisoned = logits.clone()
    poisoned[3] = float("nan")
    poisoned[77, ::2] = float("nan")
    zero = torch.zeros(E)
    cfg = terrace.TRouteConfig(E, Ng, k, M)
    runs = [terrace.t_route(poisoned.to(DEV), zero.to(DEV), cfg, mode) for _ in range(3)]
    torch.cuda.synchronize()
    e, gt, grp = runs[0]
    assert bool(((e >= 0) & (e < E)).all())
    assert bool(((grp >= 0) & (grp < Ng) | (grp == 0x7FFFFFFF)).all())      # a group, or the no-group sentinel
    for e2, gt2, grp2 in runs[1:]:
        assert torch.equal(e, e2) and torch.equal(grp, grp2)
        assert torch.equal(gt.view(torch.int32), gt2.view(torch.int32))
    oe, og, _ = orc.t_route(logits.numpy(), zero.numpy(), E, Ng, k, M, mode=mode)
    ok = np.ones(T, dtype=bool)
    ok[[3, 77]] = False
    assert np.array_equal(to_np(e)[ok], oe[ok]) and np.array_equal(to_np(gt)[ok], og[ok])


def test_expert_load_and_hist_and_argsort():
    import terrace
    from terrace.ta2a_fwd import _stable_argsort_small, fixed_hist
    announce("hist/argsort")
    rng = np.random.default_rng(3)
    for n, nb in [(0, 8), (1, 8), (100, 8), (24576, 8), (300000, 32), (5000, 256), (70000, 1)]:
        key = rng.integers(0, nb, n).astype(np.int64)
        kd = torch.from_numpy(key).to(DEV)
        same(fixed_hist(kd, nb), orc.fixed_hist(key, nb), "fixed_hist")
        same(_stable_argsort_small(kd, nb), orc.stable_argsort_small(key, nb), "argsort")
    e = rng.integers(0, 64, (4096, 8)).astype(np.int64)
    same(terrace.expert_load(torch.from_numpy(e).to(DEV), 64), orc.expert_load(e, 64), "expert_load")
    # an index outside the range is counted nowhere and reported, in the direct and in the scan-launch form
    import terrace.ops as tops
    from terrace import _hip
    for n, nb in [(5000, 16), (40000, 1500)]:
        key = rng.integers(0, nb, n).astype(np.int64)
        bad = key.copy()
        bad[[3, n // 2, n - 1]] = [-1, nb, 1 << 40]
        out, st = tops.hist(torch.from_numpy(bad).to(DEV), nb)
        want = np.bincount(np.delete(key, [3, n // 2, n - 1]), minlength=nb)
        same(out, want.astype(np.int64), "hist with bad ids")
        assert st.tolist()[0] & _hip.FAULT_ID_RANGE
        _, st = tops.hist(torch.from_numpy(key).to(DEV), nb)
        assert st.tolist()[0] == 0


# ------------------------------------------------------------------------------- plan + pack

def _k2_case(world, rpn, E, T, k, M, fmt, sort_rows, seed, H=16):
    n_nodes = world // rpn
    e = equal_quota_routing(T, k, E, n_nodes, M, seed, sort_rows)
    g = torch.Generator().manual_seed(seed)
    hidden = rows_of(torch.randn(T, H, generator=g), fmt)
    gates = rows_of(torch.rand(T, k, generator=g), fmt)
    return e, hidden, gates


# beyond the reference's list: k in 9..16 (wider register row), more than 64 nodes and k > 16
# (the (token, run)-item kernels), several units per launch, a single token per wave tail
EXTRA_K2_GEOMS = [(8, 2, 64, 37, 12, 3), (80, 1, 160, 50, 4, 2), (8, 2, 64, 21, 24, 4), (64, 8, 256, 3000, 8, 4),
                  (128, 8, 128, 1025, 8, 2), (64, 8, 64, 257, 4, 2)]


@pytest.mark.parametrize("fmt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("sort_rows", [True, False])
def test_k2_pack_reference_geometries(literals, fmt, sort_rows):
    import terrace.ops as tops
    for world, rpn, E, T, k, M in literals["k2_geometries"]["rows"] + EXTRA_K2_GEOMS:
        for seed in (500, 501):
            announce("k2", (world, rpn, E, T, k, M), fmt, sort_rows, seed)
            e, hidden, gates = _k2_case(world, rpn, E, T, k, M, fmt, sort_rows, seed)
            want = orc.k2_pack(to_np(hidden), e, to_np(gates), world, E, rpn, M)
            ed = torch.from_numpy(e).to(DEV)
            got, ex = tops.k2_pack_raw(hidden.to(DEV), ed, gates.to(DEV), world, E, rpn, M, extras=True)
            for name, a, b in zip(("payload", "mask", "gate_rows", "u_src", "node_counts"), got, want):
                same(a, b, name)
            assert got[0].dtype == hidden.dtype and got[2].dtype == gates.dtype
            u_src, u_node, counts, inverse = orc.plan_ta2a(e, world, E, rpn, M)
            same(ex["u_node"], u_node, "u_node"), same(ex["inverse"], inverse, "inverse")
            same(ex["node_offsets"], orc.send_offsets(counts), "node_offsets")
            pair_tab, order = orc.token_pair_table(e, inverse, k // M)
            same(ex["pair_table"], pair_tab, "pair_table"), same(ex["sort_order"], order, "sort_order")
            same(ex["token_rows"], pair_tab[:, ::k // M] // (k // M), "token_rows")
            same(ex["gate_sorted"], np.take_along_axis(to_np(gates), order, 1), "gate_sorted")
            assert ex["status"].tolist() == [0, T * M, 0, 0]
            # the registered torch op is the same call
            for a, b in zip(torch.ops.terrace.k2_pack(hidden.to(DEV), ed, gates.to(DEV), world, E, rpn, M), got):
                assert torch.equal(a, b)


@pytest.mark.parametrize("geom", [(8, 8, 64, 500, 4, 1), (16, 8, 192, 333, 8, 2), (16, 8, 1024, 700, 8, 2),
                                  (64, 8, 1024, 2100, 8, 4)], ids=lambda g: "w%dr%dE%dT%dk%dM%d" % g)
def test_nodes_wider_than_the_reference_mask_bound(geom):
    """The reference stops at 63 expert slots per node because its general branch ships them as one int64 bitmask
    (terrace/ops/k2_ref.py:95-108, csrc/terrace_ops.cpp:123-144).  The quota wire format has no such limit and
    this build lifts it there: the send side, the arrival chain and the regroup on nodes of 64 to 512 slots,
    against the oracle's pieces (plan + row gather + quota wire planes), which carry no bound of their own."""
    import terrace.ops as tops
    world, rpn, E, T, k, M = geom
    epr, n_nodes, q = E // world, world // rpn, k // M
    slots = epr * rpn
    assert slots > 63
    announce("wide nodes", geom, slots)
    e = equal_quota_routing(T, k, E, n_nodes, M, 77, False)
    g = torch.Generator().manual_seed(78)
    hidden = rows_of(torch.randn(T, 96, generator=g), "bf16")
    gates = rows_of(torch.rand(T, k, generator=g), "bf16")
    with pytest.raises(ValueError, match="slots"):
        orc.k2_pack(to_np(hidden), e, to_np(gates), world, E, rpn, M)        # the oracle keeps the reference's refusal
    u_src, u_node, counts, inverse = orc.plan_ta2a(e, world, E, rpn, M)
    payload = to_np(hidden)[u_src]
    mask, gate_rows = orc.pack_quota_wire(e, to_np(gates), inverse, T * M, slots, q)
    got, ex = tops.k2_pack_raw(hidden.to(DEV), torch.from_numpy(e).to(DEV), gates.to(DEV), world, E, rpn, M, extras=True)
    for name, a, b in zip(("payload", "mask", "gate_rows", "u_src", "node_counts"), got, (payload, mask, gate_rows, u_src, counts)):
        same(a, b, name)
    same(ex["u_node"], u_node, "u_node"), same(ex["inverse"], inverse, "inverse")
    assert ex["status"].tolist() == [0, T * M, 0, 0] and int(to_np(got[1]).max()) >= 63
    send, gp, r_idx, s_idx, i_send = orc.k1_arrival(payload, mask, gate_rows, q, epr, rpn)
    arr = tops.k1_arrival_raw(got[0], got[1], got[2], q, epr, rpn, 0)
    for name, a, b in zip(("send_buf", "gate_pairs", "r_idx", "slot_idx", "i_send"), arr, (send, gp, r_idx, s_idx, i_send)):
        same(a, b, name)
    perm, order, tpe = orc.regroup(send, s_idx, slots)
    rg = tops.regroup(arr[0], arr[3], slots)
    same(rg[0], perm, "permuted"), same(rg[1], order, "order"), same(rg[2], tpe, "tokens_per_expert")


def test_plan_and_wire_functions_match_oracle(literals):
    from terrace import ta2a
    from terrace.ta2a_fwd import _pack_quota_wire
    for world, rpn, E, T, k, M in literals["k2_geometries"]["rows"]:
        announce("plan", (world, rpn, E, T, k, M))
        ta2a._VERIFIED.clear(), ta2a._VERIFY_COUNT.clear()
        e, hidden, gates = _k2_case(world, rpn, E, T, k, M, "bf16", False, 900)
        ed = torch.from_numpy(e).to(DEV)
        got = ta2a.plan_ta2a(ed, world, E, rpn, groups_m=M)
        want = orc.plan_ta2a(e, world, E, rpn, M)
        for name, a, b in zip(("u_src", "u_node", "counts", "inverse"), got, want):
            same(a, b, name)
        slots = (E // world) * rpn
        payload = hidden.to(DEV)[got[0]]
        st, gt = _pack_quota_wire(ed, gates.to(DEV), got[3], payload, T * M, slots, k // M, E)
        ws, wg = orc.pack_quota_wire(e, to_np(gates), want[3], T * M, slots, k // M)
        same(st, ws, "slot_tab"), same(gt, wg, "gate_tab")
        with pytest.raises(RuntimeError, match="dtype"):
            _pack_quota_wire(ed, gates.float().to(DEV), got[3], payload, T * M, slots, k // M, E)
        stats = ta2a.dispatch_stats(ed, world, E, rpn, groups_m=M)
        assert stats["rows_ta2a"] == T * M and stats["rows_baseline"] == T * k


def test_plan_guard_literal_cases(literals):
    from terrace import ta2a
    lit = literals["plan_quota_guard"]
    geo = lit["geometry"]
    for case in lit["cases"]:
        announce("guard", case["name"])
        ta2a._VERIFIED.clear(), ta2a._VERIFY_COUNT.clear()
        idx = torch.tensor([case["expert_idx_row"]] * case["repeat"], device=DEV)
        if case["raises"]:
            with pytest.raises(ValueError, match=case["raises"]):
                ta2a.plan_ta2a(idx, geo["world"], geo["n_experts"], geo["rpn"], groups_m=case["groups_m"])
        else:
            u_src, _, counts, _ = ta2a.plan_ta2a(idx, geo["world"], geo["n_experts"], geo["rpn"],
                                                 groups_m=case["groups_m"])
            assert u_src.numel() == case["n_rows"] and int(counts.sum()) == case["counts_sum"]
    # group_limited routing has exact fan-out without quota: refused, not corrupted
    import terrace
    ta2a._VERIFIED.clear(), ta2a._VERIFY_COUNT.clear()
    g = torch.Generator().manual_seed(5)
    aff = torch.rand(256, 8, generator=g).to(DEV)
    cfg = terrace.TRouteConfig(8, 2, 4, 2)
    e, _, _ = terrace.t_route(aff, torch.zeros(8, device=DEV), cfg, mode="group_limited")
    with pytest.raises(ValueError):
        ta2a.plan_ta2a(e, 4, 8, 2, groups_m=2)
    # and the guard sleeps between its periodic checks, as documented
    ta2a._VERIFIED.clear(), ta2a._VERIFY_COUNT.clear()
    good = torch.tensor([[0, 2, 4, 6]] * 4, device=DEV)
    ta2a.plan_ta2a(good, 4, 8, 2, groups_m=2)
    bad = torch.tensor([[0, 2, 3, 5]] * 4, device=DEV)
    ta2a.plan_ta2a(bad, 4, 8, 2, groups_m=2)              # call 2 of this shape: unchecked
    ta2a._VERIFY_COUNT[(4, 4, 2, 2)] = 256
    with pytest.raises(ValueError, match="quota"):
        ta2a.plan_ta2a(bad, 4, 8, 2, groups_m=2)


def test_malformed_routing_is_contained_and_counted():
    """Unchecked calls on a routing that breaks the invariants must stay in range and report the
    census the guard reads: occupied (token, node) pairs and pairs off the quota."""
    import terrace.ops as tops
    from terrace import _hip
    announce("k2 malformed")
    # 6 tokens are one place workgroup that takes the census itself; 70 go through the count launch
    for n in (6, 70):
        cases = {
            "three_one": ([[0, 2, 3, 5]] * n, 2 * n, 2 * n),        # 2 nodes each, both off the 2/2 quota
            "fanout_one": ([[0, 1, 2, 3]] * n, n, n),               # one node holding 4
            "id_range": ([[0, 2, 4, 99]] * n, 2 * n, n),            # one id outside [0, 8)
        }
        for name, (rows, occupied, off_quota) in cases.items():
            e = torch.tensor(rows, device=DEV)
            x = torch.randn(n, 16, device=DEV)
            gts = torch.rand(n, 4, device=DEV)
            (payload, mask, gate_rows, u_src, counts), ex = tops.k2_pack_raw(x, e, gts, 4, 8, 2, 2, extras=True,
                                                                             combine_table=True)
            assert ((ex["pair_src"] >= -1) & (ex["pair_src"] < 4 * n)).all()
            assert (ex["where"] == -1).all(), "the pre-set combine table of a malformed token must read -1"
            fault, occ, offq, _ = ex["status"].tolist()
            assert fault != 0 and occ == occupied and offq == off_quota, (name, n, fault, occ, offq)
            assert int(counts.sum()) <= 2 * n and (counts >= 0).all()
            assert ((u_src >= 0) & (u_src < n)).all() and ((mask >= 0) & (mask < 4)).all()
            assert ((ex["pair_table"] >= -1) & (ex["pair_table"] < 4 * n)).all()
            assert ((ex["token_rows"] >= -1) & (ex["token_rows"] < 2 * n)).all()
            assert torch.isfinite(gate_rows).all()
            if name == "id_range":
                assert fault & _hip.FAULT_ID_RANGE
    # the (token, run)-item kernels (k > 16, or more than 64 nodes) contain the same breakage: every address they
    # form comes from an item's sorted position or from a rank below k, never from an id
    g = torch.Generator().manual_seed(9)
    for world, rpn, E, T, k, M in [(8, 2, 64, 40, 24, 4), (160, 2, 160, 50, 4, 2)]:
        n_nodes, slots, q = world // rpn, (E // world) * rpn, k // M
        e = torch.from_numpy(equal_quota_routing(T, k, E, n_nodes, M, 5, False)).clone()
        e[1, 0] = E + 7                          # outside [0, E)
        e[2, 1] = -3
        e[3, :] = e[3, 0]                        # one expert k times: one node, ranks collide
        e[4, : k // 2] = e[4, k // 2:][: k // 2] if k % 2 == 0 else e[4, : k // 2]     # duplicates
        e[5] = torch.randint(0, E, (k,), generator=g)                                  # no quota structure at all
        x = torch.randn(T, 24, device=DEV)
        gts = torch.rand(T, k, device=DEV)
        (payload, mask, gate_rows, u_src, counts), ex = tops.k2_pack_raw(x, e.to(DEV), gts, world, E, rpn, M, extras=True)
        torch.cuda.synchronize()
        fault = ex["status"].tolist()[0]
        assert fault & _hip.FAULT_ID_RANGE and fault & (_hip.FAULT_FANOUT | _hip.FAULT_QUOTA), fault
        assert int(counts.sum()) == T * M and bool((counts >= 0).all())
        assert bool(((u_src >= 0) & (u_src < T)).all())
        assert bool(((ex["token_rows"] >= 0) & (ex["token_rows"] < T * M)).all())
        assert bool(((ex["pair_table"] >= -1) & (ex["pair_table"] < T * M * q)).all())
        assert bool(((mask >= 0) & (mask < slots)).all()) and bool(torch.isfinite(gate_rows).all())
        assert bool(((ex["sort_order"] >= 0) & (ex["sort_order"] < k)).all())
        # the clean tokens still get their rows right
        clean = torch.ones(T, dtype=torch.bool)
        clean[1:6] = False
        rows_of_clean = ex["token_rows"].cpu()[clean]
        assert torch.equal(payload.cpu()[rows_of_clean.reshape(-1)], x.cpu()[clean].repeat_interleave(M, 0))


@pytest.mark.parametrize("onepass", [False, True])
def test_one_call_dispatch_equals_the_stage_calls(onepass):
    """terrace_dispatch against terrace_k2_pack + terrace_k1_arrival + terrace_regroup (or terrace_hopb_scatter) called
    one after the other: every plane and every row buffer bit for bit, with and without a capacity, on the
    lane-per-token send side and on the item kernels, and on an empty batch."""
    from terrace import ta2a_fwd
    announce("dispatch one call", onepass)
    cases = [(64, 8, 256, 1000, 8, 4, 48, torch.bfloat16, None), (64, 8, 256, 1000, 8, 4, 48, torch.bfloat16, 30),
             (64, 8, 64, 777, 4, 2, 33, torch.float32, None), (8, 2, 64, 90, 24, 4, 16, torch.float16, 20),
             (160, 2, 160, 50, 4, 2, 8, torch.float32, None), (64, 8, 256, 0, 8, 4, 48, torch.bfloat16, None)]
    for world, rpn, E, T, k, M, H, dtype, cap in cases:
        n_nodes = world // rpn
        g = torch.Generator().manual_seed(T + k)
        e = torch.from_numpy(equal_quota_routing(T, k, E, n_nodes, M, 3, False)).reshape(T, k).to(DEV)
        x = torch.randn(T, H, generator=g).to(dtype).to(DEV)
        gts = torch.rand(T, k, generator=g).to(dtype).to(DEV)
        a = ta2a_fwd._dispatch_one_slab(x, e, gts, world, E, rpn, M, cap, onepass)
        b = ta2a_fwd._dispatch_one_slab(x, e, gts, world, E, rpn, M, cap, onepass, stagewise=True)
        torch.cuda.synchronize()
        names = [n for n in a._slab.layout.at if not n.startswith("_")]
        assert names and set(names) == {n for n in b._slab.layout.at if not n.startswith("_")}
        for n in names:
            ta, tb = a._slab.tensor(n), b._slab.tensor(n)
            if n in ("x.status",):
                assert ta.tolist()[:3] == tb.tolist()[:3], n
                continue
            assert torch.equal(ta.view(torch.uint8) if ta.is_floating_point() else ta,
                               tb.view(torch.uint8) if tb.is_floating_point() else tb), (n, T, k, cap)
        for n in ("payload", "permuted") + (() if onepass else ("send_buf",)):
            assert torch.equal(getattr(a, n).view(torch.uint8), getattr(b, n).view(torch.uint8)), n


def _poison_next_allocation(nbytes):
    """Leaves a freed block of ``nbytes`` full of 0x5A bytes at the head of torch's cache, so that the next
    allocation of that size starts from garbage that reads as huge positive ids."""
    junk = torch.full((nbytes,), 0x5A, dtype=torch.uint8, device=DEV)
    torch.cuda.synchronize()
    del junk


@pytest.mark.parametrize("onepass", [False, True])
def test_malformed_routing_through_the_whole_dispatch(onepass):
    """The loop-back dispatch on a slab that arrives full of garbage, with tokens that break every invariant: the
    combine's place table, filled through the tag chain, must name a valid place or -1 for every entry, pair_src
    must stay inside [-1, T*k), and the combine over it must be finite -- on the lane-per-token send side (k <= 16,
    <= 64 nodes) and on the item kernels (k = 24; 80 nodes)."""
    from terrace import ta2a_fwd
    announce("dispatch malformed", onepass)
    for world, rpn, E, T, k, M in [(4, 2, 8, 70, 4, 2), (64, 8, 256, 300, 8, 4), (8, 2, 64, 40, 24, 4),
                                   (160, 2, 160, 50, 4, 2)]:
        n_nodes, slots, q = world // rpn, (E // world) * rpn, k // M
        g = torch.Generator().manual_seed(T)
        e = torch.from_numpy(equal_quota_routing(T, k, E, n_nodes, M, 5, False)).clone()
        e[1, 0] = E + 7                          # outside [0, E)
        e[2, 1] = -3
        e[3, :] = e[3, 0]                        # one expert k times
        e[5] = torch.randint(0, E, (k,), generator=g)     # no quota structure at all
        e[7, :q + 1] = e[7, 0] // slots * slots + torch.arange(q + 1) % slots   # q + 1 experts on one node
        x = torch.randn(T, 32, generator=g).to(DEV)
        gts = torch.rand(T, k, generator=g).to(DEV)
        lay = ta2a_fwd._dispatch_layout(T, k, world, E, rpn, M, None, gts.dtype, onepass)
        dispatch = ta2a_fwd.loopback_dispatch_onepass if onepass else ta2a_fwd.loopback_dispatch
        # the first dispatch of a shape reads the guard's census back and raises on such a routing; later ones
        # (up to the 256th) run unchecked, which is the case that has to be contained
        from terrace import ta2a
        ta2a._VERIFIED.discard((T, k, n_nodes, M)), ta2a._VERIFY_COUNT.pop((T, k, n_nodes, M), None)
        with pytest.raises(ValueError):
            dispatch(x, e.to(DEV), gts, world, E, rpn, M)
        ta2a._VERIFIED.add((T, k, n_nodes, M))
        _poison_next_allocation(max(lay.total, 256))
        st = dispatch(x, e.to(DEV), gts, world, E, rpn, M)
        torch.cuda.synchronize()
        P = T * k
        pair_src, where = st.extras["pair_src"], st.extras["where"]
        assert bool(((pair_src >= -1) & (pair_src < P)).all()), "pair_src out of range"
        assert bool(((where >= -1) & (where < st.permuted.shape[0])).all()), "combine table out of range"
        assert st.extras["status"].tolist()[0] != 0
        # a live entry names the place of the very pair that answers it
        live = where.reshape(-1) >= 0
        assert int(live.sum()) >= (T - 6) * k
        y = ta2a_fwd.loopback_combine(st.permuted, st)
        assert bool(torch.isfinite(y).all())
        # the clean tokens combine to what the oracle's table gives on the clean part alone
        clean = torch.ones(T, dtype=torch.bool)
        clean[[1, 2, 3, 5, 7]] = False
        assert bool((where.cpu()[clean] >= 0).all())
        rows = st.permuted[where[clean.to(DEV)].reshape(-1)].view(-1, k, 32)
        assert torch.equal(rows, x[clean.to(DEV)][:, None, :].expand(-1, k, -1)), "a clean token's places hold other rows"


def test_hopa_send_splits_literal(literals):
    import terrace.ops as tops
    lit = literals["hopa_counts"]
    send = tops.hopa_send_splits(torch.tensor(lit["node_counts"], device=DEV), lit["world"], lit["rpn"],
                                 lit["my_local"])
    assert send.dtype == torch.int64 and send.tolist() == lit["send"]


# ------------------------------------------------------------------------------- arrival

@pytest.mark.parametrize("fmt", ["f32", "bf16", "f16"])
def test_k1_arrival_reference_geometries(literals, fmt):
    import terrace.ops as tops
    for R, q, epr, rpn, H in literals["k1_geometries"]["rows"]:
        for seed in (100, 101):
            announce("k1", (R, q, epr, rpn, H), fmt, seed)
            rslot = arrival_plane(R, q, epr, rpn, seed)
            g = torch.Generator().manual_seed(seed)
            rx = rows_of(torch.randn(R, H, generator=g), fmt)
            rgate = rows_of(torch.rand(R, q, generator=g), fmt)
            want = orc.k1_arrival(to_np(rx), rslot, to_np(rgate), q, epr, rpn)
            got = tops.k1_arrival_raw(rx.to(DEV), torch.from_numpy(rslot).to(DEV), rgate.to(DEV), q, epr, rpn, 0,
                                      want_pair_pos=True)
            for name, a, b in zip(("send_buf", "gate_pairs", "r_idx", "slot_idx", "i_send"), got, want):
                same(a, b, name)
            same(got[5], orc.arrival_positions(rslot, epr, rpn), "pair_pos")
            for a, b in zip(torch.ops.terrace.k1_arrival(rx.to(DEV), torch.from_numpy(rslot).to(DEV),
                                                         rgate.to(DEV), q, epr, rpn, 0), got):
                assert torch.equal(a, b)


def test_k1_arrival_degenerate_empty_and_large(literals):
    import terrace.ops as tops
    d = literals["k1_degenerate"]["all_zero_slot_rows"]
    announce("k1 degenerate")
    rslot = arrival_plane(d["R"], d["quota"], d["epr"], d["rpn"], 5, degenerate=True)
    g = torch.Generator().manual_seed(5)
    rx, rgate = torch.randn(d["R"], d["H"], generator=g), torch.rand(d["R"], d["quota"], generator=g)
    want = orc.k1_arrival(rx.numpy(), rslot, rgate.numpy(), d["quota"], d["epr"], d["rpn"])
    got = tops.k1_arrival(rx.to(DEV), torch.from_numpy(rslot).to(DEV), rgate.to(DEV), d["quota"], d["epr"], d["rpn"])
    for name, a, b in zip(("send_buf", "gate_pairs", "r_idx", "slot_idx", "i_send"), got, want):
        same(a, b, name)
    z = literals["k1_degenerate"]["empty_arrival"]
    announce("k1 empty")
    got = tops.k1_arrival(torch.zeros(0, z["H"], device=DEV), torch.zeros(0, z["quota"], dtype=torch.int64, device=DEV),
                          torch.zeros(0, z["quota"], device=DEV), z["quota"], z["epr"], z["rpn"])
    assert got[0].shape == (0, z["H"]) and got[4].shape == (z["rpn"],) and int(got[4].sum()) == z["i_send_sum"]
    announce("k1 large, many units")
    R, q, epr, rpn, H = 150001, 2, 4, 8, 64
    rslot = arrival_plane(R, q, epr, rpn, 9)
    rx = torch.randn(R, H, generator=g).bfloat16()
    rgate = torch.rand(R, q, generator=g).bfloat16()
    want = orc.k1_arrival(to_np(rx), rslot, to_np(rgate), q, epr, rpn)
    got = tops.k1_arrival(rx.to(DEV), torch.from_numpy(rslot).to(DEV), rgate.to(DEV), q, epr, rpn)
    for name, a, b in zip(("send_buf", "gate_pairs", "r_idx", "slot_idx", "i_send"), got, want):
        same(a, b, name)


def test_k1_out_of_range_slot_is_contained_and_reported():
    import terrace.ops as tops
    from terrace import _hip
    announce("k1 bad slot")
    rslot = torch.tensor([[0, 3], [1, 99], [2, 5]], device=DEV)
    st = _hip.new_status(DEV)
    out = tops.k1_arrival_raw(torch.randn(3, 8, device=DEV), rslot, torch.rand(3, 2, device=DEV), 2, 2, 4, 0,
                              status_out=st)
    assert st.tolist()[0] & _hip.FAULT_ID_RANGE
    assert int(out[4].sum()) == 6 and sorted(out[2].tolist()) == [0, 0, 1, 1, 2, 2]


def test_k1_backward_is_the_gather_adjoint():
    import terrace.ops as tops
    announce("k1 backward")
    R, q, epr, rpn, H = 12, 2, 2, 4, 8
    rslot = arrival_plane(R, q, epr, rpn, 9)
    g = torch.Generator().manual_seed(1)
    rx0, rg0 = torch.randn(R, H, generator=g), torch.rand(R, q, generator=g)
    gs, gg = torch.randn(R * q, H, generator=g), torch.randn(R * q, generator=g)
    _, _, r_idx, _, _ = orc.k1_arrival(rx0.numpy(), rslot, rg0.numpy(), q, epr, rpn)
    pos = orc.arrival_positions(rslot, epr, rpn)
    want_rx = orc.gather_reduce(gs.numpy(), pos.reshape(R, q), None)
    want_rg = gg.numpy()[pos].reshape(R, q)
    for fn in (tops.k1_arrival, tops.k1_arrival_segment):
        rx, rg = rx0.to(DEV).requires_grad_(True), rg0.to(DEV).requires_grad_(True)
        s, p, *_ = fn(rx, torch.from_numpy(rslot).to(DEV), rg, q, epr, rpn)
        ((s * gs.to(DEV)).sum() + (p * gg.to(DEV)).sum()).backward()
        same(rx.grad, want_rx, "grad_rx"), same(rg.grad, want_rg, "grad_rgate")


# ------------------------------------------------------------------------------- regroup

@pytest.mark.parametrize("P,epr,my_local,H,fmt", [(7, 4, 1, 3, "f32"), (1000, 4, 0, 16, "bf16"), (30000, 32, 0, 64, "bf16"),
                                                  (513, 1, 5, 8, "f16"), (4097, 63, 2, 24, "f32")])
def test_regroup_dropless_and_capacity(P, epr, my_local, H, fmt):
    import terrace.ops as tops
    announce("regroup", P, epr, my_local, H, fmt)
    rng = np.random.default_rng(P)
    my_slot = (rng.integers(0, epr, P) + my_local * epr).astype(np.int64)
    if P == 7:
        my_slot = np.array([5, 4, 5, 5, 4, 7, 5], dtype=np.int64)
    g = torch.Generator().manual_seed(P)
    rows = rows_of(torch.randn(P, H, generator=g), fmt)
    gate = rows_of(torch.rand(P, generator=g), fmt)
    sd = torch.from_numpy(my_slot).to(DEV)
    permuted, order, tpe, pgate = tops.regroup(rows.to(DEV), sd, epr, my_local, my_gate=gate.to(DEV))
    wp, wo, wt = orc.regroup(to_np(rows), my_slot, epr, my_local)
    same(permuted, wp, "permuted"), same(order, wo, "order"), same(tpe, wt, "tokens_per_expert")
    same(pgate, to_np(gate)[wo], "permuted_gate")
    mean = max(P // epr, 1)
    for cap in (0, 1, mean, int(mean * 1.25) + 1, P + 3):
        padded, dest, kept, tpe, kpe, pg = tops.regroup(rows.to(DEV), sd, epr, my_local, capacity=cap,
                                                        my_gate=gate.to(DEV))
        wpad, wdest, wkept, wt, wk = orc.regroup(to_np(rows), my_slot, epr, my_local, capacity=cap)
        same(padded, wpad, f"padded cap={cap}"), same(dest, wdest, "dest"), same(kept, wkept, "kept")
        same(tpe, wt, "tokens_per_expert"), same(kpe, wk, "kept_per_expert")
        wg = np.zeros(epr * cap, dtype=to_np(gate).dtype)
        wg[wdest[wkept]] = to_np(gate)[wkept]
        same(pg, wg, "padded_gate")


def test_regroup_empty():
    import terrace.ops as tops
    announce("regroup empty")
    permuted, order, tpe = tops.regroup(torch.zeros(0, 8, device=DEV), torch.zeros(0, dtype=torch.int64, device=DEV), 4)
    assert permuted.shape == (0, 8) and order.numel() == 0 and tpe.tolist() == [0, 0, 0, 0]
    padded, dest, kept, tpe, kpe = tops.regroup(torch.zeros(0, 8, device=DEV),
                                                torch.zeros(0, dtype=torch.int64, device=DEV), 4, capacity=3)
    assert padded.shape == (12, 8) and not padded.any() and kpe.tolist() == [0, 0, 0, 0]


# ------------------------------------------------------------------------------- combine

@pytest.mark.parametrize("src_fmt,out_fmt,H", [("f32", "f32", 1024), ("bf16", "bf16", 7168), ("bf16", "f32", 512),
                                               ("f16", "f16", 256), ("f32", "bf16", 64), ("bf16", "bf16", 24),
                                               ("f32", "f32", 6), ("f16", "f32", 13)])
@pytest.mark.parametrize("fan", [1, 2, 3, 4, 8, 11])
def test_combine_bit_exact_and_within_tolerance(src_fmt, out_fmt, H, fan):
    import terrace.ops as tops
    announce("combine", src_fmt, out_fmt, H, fan)
    n_src, n_out = 300, 97
    g = torch.Generator().manual_seed(H + fan)
    src = rows_of(torch.randn(n_src, H, generator=g), src_fmt)
    idx = torch.randint(0, n_src, (n_out, fan), generator=g)
    idx[5, 0] = -1
    idx[6, :] = -1
    idx[8, fan - 1] = n_src                                          # past the end of src: dead, like a negative id
    idx[9, 0] = 1 << 41
    dead_too = idx.clone()
    idx[idx >= n_src] = -1                                           # what the oracle is given instead
    got_oob = tops.combine(src.to(DEV), dead_too.to(DEV), None, out_dtype=DT[out_fmt])
    assert torch.equal(got_oob, tops.combine(src.to(DEV), idx.to(DEV), None, out_dtype=DT[out_fmt]))
    for wfmt in (None, "f32", src_fmt):
        w = None if wfmt is None else rows_of(torch.rand(n_out, fan, generator=g), wfmt)
        got = tops.combine(src.to(DEV), idx.to(DEV), None if w is None else w.to(DEV), out_dtype=DT[out_fmt])
        wf = None if w is None else orc.decode_rows(to_np(w), wfmt)
        want = orc.combine(to_np(src), idx.numpy(), wf, src_fmt, out_fmt)
        same(got, want, f"combine w={wfmt}")
        # the stated tolerance, against float64
        ok = idx.numpy() >= 0
        s64 = orc.decode_rows(to_np(src), src_fmt).astype(np.float64)
        w64 = np.ones((n_out, fan)) if wf is None else wf.astype(np.float64)
        ref = sum(np.where(ok[:, j:j + 1], s64[np.where(ok[:, j], idx.numpy()[:, j], 0)] * w64[:, j:j + 1], 0.0)
                  for j in range(fan))
        tol = 1e-5 if out_fmt == "f32" else 1e-2
        scale = np.abs(ref).max() + 1e-30
        assert np.abs(orc.decode_rows(to_np(got), out_fmt) - ref).max() <= tol * scale * (2 if out_fmt == "f16" else 1)


def test_combine_fp8_rows():
    import terrace.ops as tops
    announce("combine fp8")
    for H in (512, 7168, 384):
        g = torch.Generator().manual_seed(H)
        x = torch.randn(64, H, generator=g) * 3
        rows = orc.fp8_quantise_rows(x.numpy())
        idx = torch.randint(0, 64, (33, 8), generator=g)
        w = torch.rand(33, 8, generator=g)
        for out_fmt in ("bf16", "f32"):
            got = tops.combine(torch.from_numpy(rows).to(DEV), idx.to(DEV), w.to(DEV), out_dtype=DT[out_fmt],
                               fp8_hidden=H)
            want = orc.combine(rows, idx.numpy(), w.numpy(), "fp8", out_fmt, hidden=H)
            same(got, want, f"fp8 H={H} {out_fmt}")
    # every e4m3 code decodes as the table says
    codes = np.arange(256, dtype=np.uint8)
    codes = codes[~np.isnan(orc.E4M3)]
    row = np.zeros((1, 256 + 8), dtype=np.uint8)
    row[0, :codes.size] = codes
    row[0, 256:] = np.array([1.0, 1.0], dtype=np.float32).view(np.uint8)
    got = tops.combine(torch.from_numpy(row).to(DEV), torch.zeros(1, 1, dtype=torch.int64, device=DEV), None,
                       out_dtype=torch.float32, fp8_hidden=256)
    assert np.array_equal(to_np(got)[0, :codes.size], orc.E4M3[codes])


def test_gather_rows_and_index_chain():
    import terrace.ops as tops
    announce("gather/index_chain")
    g = torch.Generator().manual_seed(4)
    for H, dt in [(7168, torch.bfloat16), (1024, torch.float32), (7392, torch.uint8), (5, torch.float16), (3, torch.uint8)]:
        src = torch.randint(0, 255, (50, H), generator=g, dtype=torch.uint8) if dt == torch.uint8 else \
            torch.randn(50, H, generator=g).to(dt)
        idx = torch.randint(0, 50, (200,), generator=g)
        idx[3] = -1
        out = tops.gather_rows(src.to(DEV), idx.to(DEV)).cpu()
        want = src[idx.clamp(min=0)]
        want[3] = 0
        assert torch.equal(out, want)
    table = torch.randint(-1, 100, (100,), generator=g)
    idx = torch.randint(-1, 100, (4, 7), generator=g)
    want = torch.where(idx < 0, torch.full_like(idx, -1), table[idx.clamp(min=0)])
    assert torch.equal(tops.index_chain(table.to(DEV), idx.to(DEV)).cpu(), want)
    # ids past the end of a table are dead at either level of the two-step form, and never read
    inner = torch.randint(-1, 130, (60,), generator=g)               # values 100..129 miss the outer table
    idx2 = torch.randint(-1, 75, (9, 5), generator=g)                # values 60..74 miss the inner table
    mid = torch.where((idx2 >= 0) & (idx2 < 60), inner[idx2.clamp(0, 59)], torch.full_like(idx2, -1))
    want2 = torch.where((mid >= 0) & (mid < 100), table[mid.clamp(0, 99)], torch.full_like(idx2, -1))
    assert torch.equal(tops.index_chain2(table.to(DEV), inner.to(DEV), idx2.to(DEV)).cpu(), want2)
    assert torch.equal(tops.index_chain(table.to(DEV), (idx + 101).to(DEV)).cpu(), torch.full_like(idx, -1))
    empty = torch.zeros(0, dtype=torch.int64, device=DEV)
    assert bool((tops.index_chain(empty, idx.clamp(min=0).to(DEV)) == -1).all())
    rows = torch.randn(0, 64, device=DEV)
    assert not tops.gather_rows(rows, torch.zeros(5, dtype=torch.int64, device=DEV)).any()
    assert not tops.combine(rows, torch.zeros(5, 3, dtype=torch.int64, device=DEV)).any()


# ------------------------------------------------------------------------------- wire containers

HOPA_GEOMS = [(5, 6, 2, 2), (5, 6, 4, 1), (1, 7, 3, 3), (17, 2048, 3, 3), (4, 5, 1, 1), (3, 24, 24, 1),
              (9, 2048, 24, 1), (0, 16, 2, 2), (1000, 7168, 2, 2)]


@pytest.mark.parametrize("geom", HOPA_GEOMS, ids=lambda g: "n%dh%dg%di%d" % g)
@pytest.mark.parametrize("fmt", ["f32", "bf16"])
def test_hopa_containers_round_trip_bitwise(geom, fmt):
    from terrace import ta2a_pack as pk
    n, hidden, gate_w, id_w = geom
    announce("hopa container", geom, fmt)
    g = torch.Generator().manual_seed(1000 + n * 31 + hidden + id_w)
    payload = rows_of(torch.randn(n, hidden, generator=g), fmt)
    gate = rows_of(torch.rand(n, gate_w, generator=g), fmt)
    ids = torch.randint(0, 1 << 40, (n,), generator=g) if id_w == 1 else torch.randint(0, 24, (n, id_w), generator=g)
    es = payload.element_size()
    buf, lay = pk.hopa_pack(payload.to(DEV), gate.to(DEV), ids.to(DEV))
    assert buf.shape == (n, lay.words) and buf.dtype == torch.int64 and buf.is_contiguous()
    assert lay.id_w == id_w and lay.id_1d is (ids.dim() == 1) and lay.words == orc.container_words(id_w, hidden, gate_w, es)
    want = orc.pack_planes([ids.numpy().reshape(n, id_w), to_np(payload), to_np(gate)], n, lay.words * 8)
    same(buf, want.reshape(n, lay.words), "hopa container")
    p2, g2, i2 = pk.hopa_unpack(buf, lay)
    assert torch.equal(p2.cpu(), payload) and torch.equal(g2.cpu(), gate) and torch.equal(i2.cpu(), ids)
    assert p2.is_contiguous() and g2.is_contiguous() and i2.is_contiguous() and i2.shape == ids.shape
    pk.assert_not_aliased(buf, p2, g2, i2)
    sbuf, slay = pk.hopa_pack_small(gate.to(DEV), ids.to(DEV))
    assert slay.words == orc.container_words(id_w, 0, gate_w, es)
    same(sbuf, orc.pack_planes([ids.numpy().reshape(n, id_w), to_np(gate)], n, slay.words * 8).reshape(n, slay.words),
         "hopa small container")
    g3, i3 = pk.hopa_unpack_small(sbuf, slay)
    assert torch.equal(g3.cpu(), gate) and torch.equal(i3.cpu(), ids)


def test_hopb_meta_and_container_errors():
    from terrace import ta2a_pack as pk
    announce("hopb meta")
    g = torch.Generator().manual_seed(3)
    for P in (0, 1, 7, 24576):
        for fmt in ("f32", "bf16"):
            slot = torch.randint(0, 63, (P,), generator=g)
            gate = rows_of(torch.rand(P, generator=g), fmt)
            buf = pk.hopb_pack_meta(slot.to(DEV), gate.to(DEV))
            assert buf.shape == (P, 2) and buf.dtype == torch.int64 and pk.hopb_meta_words() == 2
            same(buf, orc.pack_planes([slot.numpy(), to_np(gate)], P, 16).reshape(P, 2), "hopb meta")
            s2, g2 = pk.hopb_unpack_meta(buf, gate.dtype)
            assert torch.equal(s2.cpu(), slot) and torch.equal(g2.cpu(), gate)
    ids = torch.tensor([0, 1, (1 << 62) + 12345, -1, (1 << 63) - 1], device=DEV)
    buf, lay = pk.hopa_pack(torch.randn(5, 6, device=DEV).bfloat16(), torch.rand(5, 3, device=DEV).bfloat16(), ids)
    assert torch.equal(pk.hopa_unpack(buf, lay)[2], ids)
    with pytest.raises(RuntimeError, match="dtype"):
        pk.hopa_pack(torch.zeros(2, 4, device=DEV), torch.zeros(2, 2, device=DEV).bfloat16(), ids[:2])
    with pytest.raises(RuntimeError, match="int64"):
        pk.hopa_pack_small(torch.zeros(2, 2, device=DEV), ids[:2].int())
    with pytest.raises(RuntimeError, match="shape"):
        pk.hopb_pack_meta(ids[:2], torch.zeros(3, device=DEV))


@pytest.mark.parametrize("rows", [0, 1, 2, 3, 17])
def test_unpacked_planes_own_their_memory(rows):
    """What the reference guards with ``_own`` (terrace/ta2a_pack.py:182-205 there, exercised by its
    tests/test_ta2a_pack_alias.py): no unpacked plane may live in the container's storage, at one row
    least of all, so the planes must read back right after the container's memory is handed back."""
    from terrace import ta2a_pack as pk
    announce("container ownership", rows)
    H, q, slots = 2048, 3, 24
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        payload = (torch.arange(rows * H, dtype=torch.float32).reshape(rows, H) % 251).to(dtype).to(DEV)
        gate = torch.full((rows, q), 0.5, dtype=dtype, device=DEV)
        ids = torch.arange(rows * q, dtype=torch.int64, device=DEV).reshape(rows, q)
        buf, lay = pk.hopa_pack(payload, gate, ids)
        rx, rgate, rmask = pk.hopa_unpack(buf, lay)
        pk.assert_not_aliased(buf, rx, rgate, rmask)
        for plane in (rx, rgate, rmask):
            assert plane.numel() == 0 or plane.untyped_storage().data_ptr() != buf.untyped_storage().data_ptr()
        torch.cuda.synchronize()
        buf.untyped_storage().resize_(0)
        assert torch.equal(rx, payload) and torch.equal(rgate, gate) and torch.equal(rmask, ids)
        assert torch.equal(rmask // 3, ids // 3)
    # the bitmask format (1-D id plane) and the Hop-B container
    payload = torch.zeros(rows, H, dtype=torch.bfloat16, device=DEV)
    buf, lay = pk.hopa_pack(payload, torch.zeros(rows, slots, dtype=torch.bfloat16, device=DEV),
                            torch.arange(rows, dtype=torch.int64, device=DEV))
    assert lay.id_1d
    pk.assert_not_aliased(buf, *pk.hopa_unpack(buf, lay))
    slot = torch.arange(rows, dtype=torch.int64, device=DEV)
    meta = pk.hopb_pack_meta(slot, torch.ones(rows, dtype=torch.bfloat16, device=DEV))
    s2, g2 = pk.hopb_unpack_meta(meta, torch.bfloat16)
    pk.assert_not_aliased(meta, s2, g2)
    torch.cuda.synchronize()
    meta.untyped_storage().resize_(0)
    assert torch.equal(s2, slot) and bool((g2 == 1).all())


def test_alias_tripwire_fires_on_a_view():
    from terrace import ta2a_pack as pk
    buf = torch.zeros(4, 8, dtype=torch.int64, device=DEV)
    view = buf[:, :2]
    with pytest.raises(RuntimeError, match="shares storage"):
        pk.assert_not_aliased(buf, view)
    pk.assert_not_aliased(buf, view.clone())
    pk.assert_not_aliased(buf, torch.zeros(0, dtype=torch.int64, device=DEV), None)


@pytest.mark.parametrize("row_bytes", [16, 48, 1024, 1040, 7392, 14336, 40, 6, 3])
def test_row_movers_at_every_base_alignment(row_bytes):
    """Straight through the C ABI with source and destination bases at 16-byte-granular (and, for
    narrow rows, odd) offsets: the kilobyte-aligned chunking must neither skip nor overrun a byte."""
    from ctypes import c_void_p
    from terrace import _hip
    announce("mover alignment", row_bytes)
    lib = _hip.load()
    g = torch.Generator().manual_seed(row_bytes)
    n_src, n_out, fan = 37, 53, 3
    step = 16 if row_bytes % 16 == 0 else (8 if row_bytes % 8 == 0 else 1)
    stream = _hip.stream(torch.device(DEV))
    for off_src, off_dst in [(0, 0), (step, 0), (0, step), (3 * step, 5 * step), (63 * step, 62 * step)]:
        pad = 4096
        src_buf = torch.randint(0, 256, (pad + n_src * row_bytes,), dtype=torch.uint8, generator=g).to(DEV)
        src = src_buf[off_src:off_src + n_src * row_bytes].view(n_src, row_bytes)
        idx = torch.randint(0, n_src, (n_out,), generator=g)
        idx[7] = -1
        idx[9], idx[11] = n_src, 1 << 40                         # past the end of src: dead entries, never addresses
        out_buf = torch.full((pad + n_out * row_bytes + pad,), 0xAB, dtype=torch.uint8, device=DEV)
        rc = lib.terrace_gather_rows(c_void_p(src.data_ptr()), n_src, _hip.ptr(idx.to(DEV)), n_out, row_bytes,
                                     c_void_p(out_buf.data_ptr() + off_dst), stream)
        assert rc == 0
        got = out_buf[off_dst:off_dst + n_out * row_bytes].view(n_out, row_bytes).cpu()
        dead = (idx < 0) | (idx >= n_src)
        want = src.cpu()[idx.clamp(0, n_src - 1)]
        want[dead] = 0
        assert torch.equal(got, want), (off_src, off_dst)
        assert bool((out_buf[:off_dst] == 0xAB).all()) and bool((out_buf[off_dst + n_out * row_bytes:] == 0xAB).all())
        # scatter: every destination row named at most once, a few left unnamed
        n_dst = n_src * fan + 5
        pos = torch.randperm(n_dst, generator=g)[:n_src * fan].view(n_src, fan).clone()
        pos[3, 1] = -1
        pos[5, 0], pos[6, 2] = n_dst, 1 << 40                    # past the end of dst: copies not made
        dst_buf = torch.full((pad + n_dst * row_bytes + pad,), 0xCD, dtype=torch.uint8, device=DEV)
        rc = lib.terrace_scatter_rows(c_void_p(src.data_ptr()), _hip.ptr(pos.to(DEV)), n_src, fan, row_bytes,
                                      c_void_p(dst_buf.data_ptr() + off_dst), n_dst, stream)
        assert rc == 0
        got = dst_buf[off_dst:off_dst + n_dst * row_bytes].view(n_dst, row_bytes).cpu()
        want = torch.full((n_dst, row_bytes), 0xCD, dtype=torch.uint8)
        for r in range(n_src):
            for f in range(fan):
                if 0 <= pos[r, f] < n_dst:
                    want[pos[r, f]] = src.cpu()[r]
        assert torch.equal(got, want), (off_src, off_dst)
        assert bool((dst_buf[:off_dst] == 0xCD).all()) and bool((dst_buf[off_dst + n_dst * row_bytes:] == 0xCD).all())


# ------------------------------------------------------------------------------- K2 gradients, reference names

@pytest.mark.parametrize("entry", ["functional", "torch_ops", "k2_pack_ref"])
def test_k2_pack_backward_is_the_adjoint(literals, entry):
    """payload = hidden[u_src] and gate_rows (a permutation gather of gates) carry gradients
    (terrace/ops/k2_ref.py:77-81): both against float64 autograd over the oracle's index planes."""
    import terrace.ops as tops
    from terrace import ta2a
    from terrace.ops.k2_ref import k2_pack_ref
    for world, rpn, E, T, k, M in literals["k2_geometries"]["rows"] + [[64, 8, 256, 700, 8, 4]]:
        announce("k2 backward", entry, (world, rpn, E, T, k, M))
        ta2a._VERIFIED.clear(), ta2a._VERIFY_COUNT.clear()
        q = k // M
        e = equal_quota_routing(T, k, E, world // rpn, M, 31)
        g = torch.Generator().manual_seed(T + k)
        x, gates = torch.randn(T, 12, generator=g), torch.rand(T, k, generator=g)
        Gp, Gg = torch.randn(T * M, 12, generator=g), torch.randn(T * M, q, generator=g)
        xd, gd = x.to(DEV).requires_grad_(), gates.to(DEV).requires_grad_()
        fn = {"functional": tops.k2_pack, "torch_ops": torch.ops.terrace.k2_pack, "k2_pack_ref": k2_pack_ref}[entry]
        payload, mask, gate_rows, u_src, counts = fn(xd, torch.from_numpy(e).to(DEV), gd, world, E, rpn, M)
        assert payload.requires_grad and gate_rows.requires_grad and not mask.requires_grad
        o_payload, o_mask, o_gate_rows, o_src, o_counts = orc.k2_pack(x.numpy(), e, gates.numpy(), world, E, rpn, M)
        same(payload, o_payload, "payload"), same(mask, o_mask, "mask"), same(gate_rows, o_gate_rows, "gate_rows")
        same(u_src, o_src, "u_src"), same(counts, o_counts, "node_counts")
        ((payload * Gp.to(DEV)).sum() + (gate_rows * Gg.to(DEV)).sum()).backward()
        _, _, _, inverse = orc.plan_ta2a(e, world, E, rpn, M)
        pair_tab, sort_order = orc.token_pair_table(e, inverse, q)
        x64, g64 = x.double().requires_grad_(), gates.double().requires_grad_()
        pay64 = x64[torch.from_numpy(o_src)]
        # cell (row, i) of gate_rows holds gates[t, sort_order[t, s]] for the (t, s) whose pair id is row*q + i
        flat = torch.zeros(T * k, dtype=torch.float64)
        flat = flat.index_add(0, torch.from_numpy(pair_tab.reshape(-1)),
                              g64.gather(1, torch.from_numpy(sort_order)).reshape(-1))
        ((pay64 * Gp.double()).sum() + (flat.view(T * M, q) * Gg.double()).sum()).backward()
        for name, got, want in (("hidden.grad", xd.grad, x64.grad), ("gates.grad", gd.grad, g64.grad)):
            assert got is not None, f"{name} missing"
            err = (got.cpu().double() - want).abs().max().item()
            assert err <= 1e-5 * max(want.abs().max().item(), 1.0), f"{name} differs by {err}"


def test_public_k2_pack_raises_on_a_malformed_routing_and_ref_names_resolve():
    import terrace.ops as tops
    from terrace import ta2a
    from terrace.ops.k2_ref import k2_pack_ref
    announce("k2 guard, reference names")
    x = torch.randn(6, 16, device=DEV)
    gts = torch.rand(6, 4, device=DEV)
    ta2a._VERIFIED.clear(), ta2a._VERIFY_COUNT.clear()
    with pytest.raises(ValueError, match="out of range"):
        tops.k2_pack(x, torch.tensor([[0, 2, 4, 99]] * 6, device=DEV), gts, 4, 8, 2, 2)
    ta2a._VERIFIED.clear(), ta2a._VERIFY_COUNT.clear()
    with pytest.raises(ValueError, match="quota"):
        tops.k2_pack(x, torch.tensor([[0, 2, 3, 5]] * 6, device=DEV), gts, 4, 8, 2, 2)
    with pytest.raises(ValueError, match="out of range"):          # the reference function checks ids on every call
        k2_pack_ref(x, torch.tensor([[0, 2, 4, 99]] * 6, device=DEV), gts, 4, 8, 2, 2)
    with pytest.raises(ValueError, match="chain bound"):
        k2_pack_ref(torch.randn(4, 8, device=DEV), torch.zeros(4, 2, dtype=torch.int64, device=DEV),
                    torch.rand(4, 2, device=DEV), 8, 1024, 8, 1)
    with pytest.raises(RuntimeError, match="dtype"):
        k2_pack_ref(x.to(torch.bfloat16), torch.tensor([[0, 1, 4, 5]] * 6, device=DEV), gts, 4, 8, 2, 2)
    # a repeated id inside a well-formed count pattern: every plane is defined and in range
    ta2a._VERIFIED.clear(), ta2a._VERIFY_COUNT.clear()
    e = torch.tensor([[0, 0, 4, 6], [1, 3, 5, 7]], device=DEV)
    (payload, mask, gate_rows, u_src, counts), ex = tops.k2_pack_raw(x[:2], e, gts[:2], 4, 8, 2, 2, extras=True)
    assert ex["status"].tolist()[0] == 0                     # two per node on two nodes: the census cannot see it
    assert sorted(ex["pair_table"][0].tolist()) == [0, 1, 4, 5] and ex["sort_order"][0].tolist() == [0, 1, 2, 3]
    assert mask.tolist() == [[0, 0], [1, 3], [0, 2], [1, 3]] and ex["gate_sorted"][0].tolist() == gts[0].tolist()
    assert gate_rows[0].tolist() == gts[0, :2].tolist() and gate_rows[2].tolist() == gts[0, 2:].tolist()
    # k1_arrival_ref is the arrival operator under the reference's name
    rslot = torch.from_numpy(arrival_plane(40, 2, 2, 8, 3)).to(DEV)
    rx, rg = torch.randn(40, 8, device=DEV), torch.rand(40, 2, device=DEV)
    for a, b in zip(tops.k1_arrival_ref(rx, rslot, rg, 2, 2, 8), tops.k1_arrival(rx, rslot, rg, 2, 2, 8)):
        assert torch.equal(a, b)
    with pytest.raises(AssertionError):
        tops.k1_arrival_ref(rx, rslot, rg, 3, 2, 8)
