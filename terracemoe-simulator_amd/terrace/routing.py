"""T-Route: terraced group-quota routing on MI355X.

Same interface as the reference module (terrace/routing.py there): ``TRouteConfig``,
``t_route``, ``expert_load``, ``update_bias_``, ``Router``.  Selection uses bias-corrected
affinities, gate values use raw affinities; per token exactly ``top_k`` distinct experts
spanning exactly ``top_groups`` groups with ``top_k // top_groups`` in each.

Where torch leaves a choice open this build fixes it: top-k ties go to the lowest index and
the gate normaliser is summed left to right in fp32.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import _hip
from . import ops as _ops

_MODES = ("full", "group_limited", "quota_only", "global_topk")


@dataclass(frozen=True)
class TRouteConfig:
    n_experts: int      # E
    n_groups: int       # N_g
    top_k: int          # k
    top_groups: int     # M
    group_score_pool: int = 2   # group score = mean of the top-`pool` affinities in the group

    def __post_init__(self):
        if self.n_experts % self.n_groups:
            raise ValueError("n_experts must divide evenly into n_groups")
        if self.top_k % self.top_groups:
            raise ValueError("top_k must divide evenly into top_groups")
        if self.per_group_k > self.group_size:
            raise ValueError("per-group quota exceeds group size")

    @property
    def group_size(self) -> int:
        return self.n_experts // self.n_groups

    @property
    def per_group_k(self) -> int:
        return self.top_k // self.top_groups


def t_route(affinity: torch.Tensor, bias: torch.Tensor, cfg: TRouteConfig, mode: str = "full", *,
            gate_affinity: torch.Tensor | None = None, gates_dtype: torch.dtype = torch.float32,
            _force_generic: bool = False):
    """Returns (expert_idx [T, k] int64, gates [T, k] float32, group_idx [T, M] int64).

    Two additions to the reference signature: ``gate_affinity`` is the [T, E] table the gate values
    are read from (default ``affinity``; selection never looks at it), and ``gates_dtype``
    (float32, bfloat16 or float16) has the kernel write ``gates.to(gates_dtype)`` directly -- the
    payload-dtype gate plane the dispatch needs, without the extra cast launch.
    """
    if gates_dtype not in _hip.GATES_FLAG:
        raise ValueError(f"gates_dtype must be float32, bfloat16 or float16, got {gates_dtype}")
    if mode not in _MODES:
        raise ValueError(f"unknown routing mode {mode!r}; expected one of {_MODES}")
    if mode == "quota_only" and cfg.top_k // cfg.n_groups < 1:
        raise ValueError(f"quota_only needs top_k ({cfg.top_k}) divisible by n_groups ({cfg.n_groups}); "
                         f"got {cfg.top_k // cfg.n_groups} experts/group")
    if mode == "quota_only" and cfg.top_k % cfg.n_groups:
        raise ValueError(f"quota_only needs top_k ({cfg.top_k}) divisible by n_groups ({cfg.n_groups})")
    if cfg.group_score_pool < 1:
        raise ValueError(f"group_score_pool must be at least 1, got {cfg.group_score_pool}")
    _ops._require()
    _hip.need_device(affinity, bias, gate_affinity)
    if affinity.dim() != 2 or affinity.shape[1] != cfg.n_experts or bias.numel() != cfg.n_experts:
        raise ValueError(f"affinity {tuple(affinity.shape)} / bias {tuple(bias.shape)} do not match "
                         f"n_experts={cfg.n_experts}")
    aff = affinity.to(torch.float32).contiguous()
    b = bias.to(torch.float32).contiguous()
    ga = None
    if gate_affinity is not None:
        if gate_affinity.shape != affinity.shape:
            raise ValueError("gate_affinity must have affinity's shape")
        ga = gate_affinity.to(torch.float32).contiguous()
    T = aff.shape[0]
    dev = aff.device
    n_g_out = {"full": cfg.top_groups, "group_limited": cfg.top_groups, "quota_only": cfg.n_groups,
               "global_topk": cfg.top_k}[mode]
    expert_idx = torch.empty((T, cfg.top_k), dtype=torch.int64, device=dev)
    gates = torch.empty((T, cfg.top_k), dtype=gates_dtype, device=dev)
    group_idx = torch.empty((T, n_g_out), dtype=torch.int64, device=dev)
    code = _hip.MODE_CODES[mode] | (_hip.FORCE_GENERIC if _force_generic else 0) | _hip.GATES_FLAG[gates_dtype]
    _hip.call("terrace_t_route", _hip.ptr(aff), _hip.ptr(b), _hip.ptr(ga), T, cfg.n_experts, cfg.n_groups,
              cfg.top_k, cfg.top_groups, cfg.group_score_pool, code, _hip.ptr(expert_idx), _hip.ptr(gates),
              _hip.ptr(group_idx), _hip.stream(dev))
    return expert_idx, gates, group_idx


def expert_load(expert_idx: torch.Tensor, n_experts: int) -> torch.Tensor:
    """Per-expert pick counts as float32 (``bincount(...).float()`` in the reference).  An id outside
    ``[0, n_experts)`` is counted nowhere; the status words that report it are not read back here (no host sync on
    this path): use ``terrace.ops.hist`` to get them."""
    out, _ = _ops.hist(expert_idx, n_experts, as_float=True)
    return out


@torch.no_grad()
def update_bias_(bias: torch.Tensor, load: torch.Tensor, gamma: float) -> torch.Tensor:
    """Aux-loss-free balancing step: nudge bias toward under-loaded experts (E elements)."""
    err = load.mean() - load
    bias.add_(gamma * torch.sign(err))
    return bias


class Router(torch.nn.Module):
    def __init__(self, hidden_size: int, cfg: TRouteConfig):
        super().__init__()
        self.cfg = cfg
        self.weight = torch.nn.Parameter(torch.empty(cfg.n_experts, hidden_size))
        torch.nn.init.normal_(self.weight, std=hidden_size ** -0.5)
        self.register_buffer("bias", torch.zeros(cfg.n_experts))

    def forward(self, hidden: torch.Tensor, mode: str = "full"):
        affinity = torch.sigmoid(hidden @ self.weight.t())        # dense GEMM: library call
        return t_route(affinity, self.bias, self.cfg, mode)
