"""TerraceMoE dispatch/combine data path, MI355X build.

Same import surface as the reference ``terrace`` package for the routing and two-hop
dispatch path (``terrace.routing``, ``terrace.ta2a``, ``terrace.ta2a_fwd``, ``terrace.ops``);
every function runs hand-written gfx950 kernels from libterrace_hip.so on ROCm tensors.
"""
from .routing import Router, TRouteConfig, expert_load, t_route, update_bias_

__all__ = ["Router", "TRouteConfig", "expert_load", "t_route", "update_bias_"]
