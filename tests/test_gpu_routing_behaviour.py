"""What the router guarantees and what it only tends to, checked on the device path.

The same behaviours the reference's own tests hold its router to (tests/test_routing.py and
tests/test_mode_distinctness.py there), asked of the HIP kernels: structure that must hold for every
token under any affinity, statistics that hold only for benign ones, and the four modes being four
different selections.
"""
from __future__ import annotations

import pytest
import torch

from test_gpu_parity import DEV, announce

pytestmark = pytest.mark.gpu


def _groups_per_token(expert_idx, group_size):
    g = (expert_idx // group_size).sort(dim=1).values
    return 1 + (g[:, 1:] != g[:, :-1]).sum(dim=1)


def _group_load(expert_idx, n_groups, group_size):
    return torch.bincount((expert_idx // group_size).reshape(-1), minlength=n_groups).float()


def _cv(x):
    return float(x.std(unbiased=False) / x.mean())


def test_every_token_gets_k_distinct_experts_m_groups_and_the_quota():
    import terrace
    announce("route structure")
    cfg = terrace.TRouteConfig(n_experts=64, n_groups=8, top_k=8, top_groups=4)
    g = torch.Generator().manual_seed(0)
    aff = torch.sigmoid(torch.randn(512, 64, generator=g)).to(DEV)
    e, gates, grp = terrace.t_route(aff, torch.zeros(64, device=DEV), cfg)
    assert e.shape == (512, 8) and grp.shape == (512, 4) and e.dtype == grp.dtype == torch.int64
    se = e.sort(dim=1).values
    assert bool((se[:, 1:] != se[:, :-1]).all())                                   # k distinct experts
    sg = grp.sort(dim=1).values
    assert bool((sg[:, 1:] != sg[:, :-1]).all())                                   # M distinct groups
    counts = torch.zeros(512, 8, dtype=torch.int64, device=DEV).scatter_add_(1, e // 8, torch.ones_like(e))
    assert bool((counts.gather(1, grp) == cfg.per_group_k).all())                  # k/M in each chosen group
    assert bool((counts.sum(1) == 8).all()) and bool(((counts > 0).sum(1) == 4).all())   # and nowhere else
    assert torch.allclose(gates.sum(-1), torch.ones(512, device=DEV), atol=1e-5) and bool((gates > 0).all())


def test_bias_update_evens_out_a_skewed_router():
    import terrace
    announce("bias balancing")
    cfg = terrace.TRouteConfig(n_experts=64, n_groups=8, top_k=8, top_groups=4)
    torch.manual_seed(0)
    router = terrace.Router(hidden_size=64, cfg=cfg).to(DEV)
    with torch.no_grad():
        router.weight[: cfg.group_size] += 0.5              # the first group is favoured
    g = torch.Generator(device=DEV).manual_seed(1)

    def run(steps, use_bias):
        loads = torch.zeros(64, device=DEV)
        for _ in range(steps):
            x = torch.randn(2048, 64, generator=g, device=DEV)
            with torch.no_grad():
                e, _, _ = router(x)
            load = terrace.expert_load(e, 64)
            if use_bias:
                terrace.update_bias_(router.bias, load, gamma=5e-3)
            loads += load
        return loads

    router.bias.zero_()
    base = run(50, False)
    router.bias.zero_()
    run(400, True)
    settled = run(50, True)
    cv, base_cv = float(settled.std() / settled.mean()), float(base.std() / base.mean())
    assert cv < 0.25 and cv < base_cv, (cv, base_cv)


def test_group_balance_is_statistical_but_fan_out_and_quota_are_not():
    import terrace
    announce("adversarial affinity")
    T, E, n_g, M = 2048, 128, 8, 4
    gs = E // n_g
    g = torch.Generator().manual_seed(2)
    aff = torch.rand(T, E, generator=g) * 0.01
    aff[:, : 4 * gs] += 1.0                                  # every token prefers the first four groups
    aff = aff.to(DEV)
    zero = torch.zeros(E, device=DEV)
    cfg = terrace.TRouteConfig(n_experts=E, n_groups=n_g, top_k=8, top_groups=M)
    e, _, grp = terrace.t_route(aff, zero, cfg, mode="full")
    load = _group_load(e, n_g, gs)
    assert _cv(load) == pytest.approx(1.0, abs=1e-6)         # all load on half the groups
    assert bool((load[4:] == 0).all()) and bool((load[:4] > 0).all())
    assert bool((_groups_per_token(e, gs) == M).all())       # yet exactly M groups per token
    counts = torch.zeros(T, n_g, dtype=torch.int64, device=DEV).scatter_add_(1, e // gs, torch.ones_like(e))
    assert bool(((counts == 0) | (counts == cfg.top_k // M)).all())
    # M == N_g is the one case that is balanced by construction
    every = terrace.TRouteConfig(n_experts=E, n_groups=n_g, top_k=8, top_groups=n_g)
    for a in (torch.rand(T, E, generator=g).to(DEV), aff):
        e, _, _ = terrace.t_route(a, zero, every, mode="quota_only")
        load = _group_load(e, n_g, gs)
        assert bool((load == T * 8 / n_g).all())


def test_the_four_modes_are_four_selections():
    import terrace
    announce("mode distinctness")
    E, n_g, K, M, T = 128, 8, 8, 4, 2048
    cfg = terrace.TRouteConfig(n_experts=E, n_groups=n_g, top_k=K, top_groups=M)
    g = torch.Generator().manual_seed(0)
    aff = (torch.rand(T, E, generator=g) * 0.998 + 1e-3).to(DEV)
    zero = torch.zeros(E, device=DEV)
    picked = {m: terrace.t_route(aff, zero, cfg, mode=m)[0] for m in ("full", "group_limited", "quota_only", "global_topk")}
    span = {m: _groups_per_token(v, E // n_g) for m, v in picked.items()}
    assert bool((span["full"] == M).all())
    assert bool((span["quota_only"] == n_g).all())
    assert bool((span["group_limited"] <= M).all())
    assert int(span["global_topk"].max()) > M                # the unconstrained baseline really is unconstrained
    modes = list(picked)
    for i, a in enumerate(modes):
        for b in modes[i + 1:]:
            differ = (picked[a].sort(dim=1).values != picked[b].sort(dim=1).values).any(dim=1).float().mean()
            assert float(differ) > 0.5, (a, b, float(differ))
    for bad in ("Full", "quota", "", "toplevel"):
        with pytest.raises(ValueError, match="unknown routing mode"):
            terrace.t_route(aff[:4], zero, cfg, mode=bad)
