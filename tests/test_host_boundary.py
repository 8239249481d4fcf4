"""CPU-side checks of the drop-in boundary: the C-ABI library loads and exports every symbol
the header declares, the ctypes table covers them all, the loader switch behaves as
documented, and host-side validation raises what the reference raises -- no kernel runs."""
from __future__ import annotations

import ctypes
import logging
import os
import re

import pytest
import torch

from conftest import ROOT

HEADER = os.path.join(ROOT, "include", "terrace_hip.h")


def _declared():
    text = open(HEADER).read()
    return sorted(set(re.findall(r"TERRACE_API[^;(]*?\b(terrace_\w+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = _declared()
    for must in ("terrace_passthrough", "terrace_t_route", "terrace_k2_pack", "terrace_k1_arrival",
                 "terrace_regroup", "terrace_combine", "terrace_hist", "terrace_argsort_small",
                 "terrace_pack_quota_wire", "terrace_gather_rows", "terrace_index_chain"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from terrace import _hip
    lib = ctypes.CDLL(_hip.find_library())
    for name in _declared():
        assert hasattr(lib, name), f"{name} declared in terrace_hip.h but not exported"
    assert lib.terrace_version is not None
    lib.terrace_version.restype = ctypes.c_char_p
    assert b"gfx950" in lib.terrace_version()
    lib.terrace_strerror.restype = ctypes.c_char_p
    assert lib.terrace_strerror(0) == b"ok" and b"workspace" in lib.terrace_strerror(-28)


def test_ctypes_table_matches_header():
    from terrace import _hip
    assert sorted(_hip.SIGNATURES) == _declared()
    text = open(HEADER).read()
    for name, (_res, args) in _hip.SIGNATURES.items():
        decl = re.search(r"TERRACE_API[^;]*?\b%s\s*\(([^;]*?)\)\s*;" % name, text, re.S).group(1)
        n_params = 0 if decl.strip() == "void" else decl.count(",") + 1
        assert n_params == len(args), f"{name}: header has {n_params} parameters, ctypes table {len(args)}"


def test_workspace_queries_need_no_device():
    from terrace import _hip
    assert _hip.query("terrace_k1_arrival_workspace", 65536, 2, 8) >= 131072 * 4
    assert _hip.query("terrace_k2_pack_workspace", 16384, 8, 8, 4) >= 65536 * 4
    assert _hip.query("terrace_regroup_workspace", 1000, 4, 10) > _hip.query("terrace_regroup_workspace", 1000, 4, -1)
    assert _hip.query("terrace_hist_workspace", 0, 8) > 0


@pytest.fixture()
def clean_ops(monkeypatch):
    import terrace.ops as tops
    monkeypatch.delenv("TERRACE_CUSTOM_OPS", raising=False)
    monkeypatch.delenv("TERRACE_OPS_LIB", raising=False)
    tops.reset()
    yield monkeypatch
    tops.reset()


def test_loader_default_loads_and_registers_schemas(clean_ops):
    import terrace.ops as tops
    st = tops.status()
    assert st.loaded and st.reason == "ok" and st.lib.endswith(".so") and st.requested == "1"
    assert tops.custom_ops_enabled() is True
    for op in ("passthrough", "k1_arrival", "k2_pack"):
        assert hasattr(torch.ops.terrace, op)
    assert tops.status() is st                      # cached verdict


def test_loader_off_switch_is_loud_not_silent(clean_ops):
    import terrace.ops as tops
    clean_ops.setenv("TERRACE_CUSTOM_OPS", "0")
    tops.reset()
    st = tops.status()
    assert not st.loaded and st.requested == "0" and "explicitly off" in st.reason
    with pytest.raises(tops.OpsLoadError):
        tops.k1_arrival(torch.zeros(2, 4), torch.zeros(2, 1, dtype=torch.int64), torch.zeros(2, 1), 1, 1, 1)
    with pytest.raises(tops.OpsLoadError):
        tops.passthrough(torch.zeros(4))


def test_loader_missing_library_warns_once_or_raises(clean_ops, caplog):
    import terrace.ops as tops
    clean_ops.setenv("TERRACE_OPS_LIB", "/nonexistent/libterrace_hip.so")
    clean_ops.setenv("TERRACE_CUSTOM_OPS", "1")
    tops.reset()
    with caplog.at_level(logging.WARNING, logger="terrace.ops"):
        assert tops.custom_ops_enabled() is False
        assert tops.custom_ops_enabled() is False
    assert len([r for r in caplog.records if r.levelno == logging.WARNING]) == 1
    clean_ops.setenv("TERRACE_CUSTOM_OPS", "require")
    tops.reset()
    with pytest.raises(RuntimeError, match="requires the kernel library"):
        tops.status()


def test_meta_kernels_give_reference_shapes(clean_ops):
    import terrace.ops as tops
    tops.status()
    rx = torch.empty(6, 32, device="meta", dtype=torch.bfloat16)
    rslot = torch.empty(6, 2, device="meta", dtype=torch.int64)
    rgate = torch.empty(6, 2, device="meta", dtype=torch.bfloat16)
    out = torch.ops.terrace.k1_arrival(rx, rslot, rgate, 2, 2, 8, 0)
    assert [tuple(o.shape) for o in out] == [(12, 32), (12,), (12,), (12,), (8,)]
    assert out[0].dtype == torch.bfloat16 and out[2].dtype == torch.int64
    hid = torch.empty(8, 16, device="meta")
    e = torch.empty(8, 4, device="meta", dtype=torch.int64)
    g = torch.empty(8, 4, device="meta")
    out = torch.ops.terrace.k2_pack(hid, e, g, 4, 8, 2, 2)
    assert [tuple(o.shape) for o in out] == [(16, 16), (16, 2), (16, 2), (16,), (2,)]


def test_cpu_tensors_are_refused_not_computed(clean_ops):
    import terrace
    import terrace.ops as tops
    from terrace.ta2a import plan_ta2a
    cfg = terrace.TRouteConfig(8, 2, 2, 1)
    with pytest.raises(RuntimeError, match="ROCm device"):
        terrace.t_route(torch.rand(4, 8), torch.zeros(8), cfg)
    with pytest.raises(RuntimeError, match="ROCm device"):
        plan_ta2a(torch.zeros(4, 2, dtype=torch.int64), 4, 8, 2, groups_m=1)
    with pytest.raises(RuntimeError, match="ROCm device"):
        tops.k1_arrival(torch.zeros(2, 4), torch.zeros(2, 1, dtype=torch.int64), torch.zeros(2, 1), 1, 1, 1)


def test_route_config_and_mode_errors_match_reference():
    import terrace
    for bad in [(30, 4, 4, 2), (32, 4, 6, 4), (32, 16, 8, 2)]:
        with pytest.raises(ValueError):
            terrace.TRouteConfig(*bad)
    cfg = terrace.TRouteConfig(n_experts=64, n_groups=8, top_k=8, top_groups=4)
    assert cfg.group_size == 8 and cfg.per_group_k == 2 and cfg.group_score_pool == 2
    for mode in ("Full", "quota", "", None):
        with pytest.raises(ValueError, match="unknown routing mode"):
            terrace.t_route(torch.rand(2, 64), torch.zeros(64), cfg, mode=mode)
    with pytest.raises(ValueError, match="quota_only"):
        terrace.t_route(torch.rand(2, 64), torch.zeros(64), terrace.TRouteConfig(64, 8, 4, 2), mode="quota_only")


def test_k1_and_k2_argument_refusals(clean_ops):
    import terrace.ops as tops
    tops.status()
    rx, rslot, rgate = torch.zeros(4, 8), torch.zeros(4, 2, dtype=torch.int64), torch.zeros(4, 2)
    with pytest.raises(RuntimeError, match="int64"):
        tops._check_k1(rx, rslot.int(), rgate, 2, 2, 4, 0)
    with pytest.raises(RuntimeError, match="dtype"):
        tops._check_k1(rx, rslot, rgate.bfloat16(), 2, 2, 4, 0)
    with pytest.raises(RuntimeError, match="geometry"):
        tops._check_k1(rx, rslot, rgate, 3, 2, 4, 0)
    with pytest.raises(RuntimeError, match="scalars"):
        tops._check_k1(rx, rslot, rgate, 2, 2, 4, 4)
    hid, e, g = torch.zeros(4, 8), torch.zeros(4, 4, dtype=torch.int64), torch.zeros(4, 4)
    with pytest.raises(RuntimeError, match="dtype"):
        tops._check_k2(hid, e, g.bfloat16(), 4, 8, 2, 2)
    with pytest.raises(ValueError, match="divisible"):
        tops._check_k2(hid, e, g, 4, 8, 3, 2)
    with pytest.raises(ValueError, match="geometry"):
        tops._check_k2(hid, e, g[:, :3], 4, 8, 2, 2)
    with pytest.raises(ValueError, match="2-D"):
        tops._check_k2(hid, e.reshape(-1), g, 4, 8, 2, 2)


def test_plan_guard_messages_from_status_words():
    from terrace import ta2a
    st = torch.tensor([4, 4, 0, 0], dtype=torch.int32)       # 4 occupied pairs where 8 were promised
    with pytest.raises(ValueError, match="fan-out"):
        ta2a._raise_from_status(st, 4, 4, 2)
    st = torch.tensor([2, 8, 8, 0], dtype=torch.int32)       # right fan-out, 8 pairs off quota
    with pytest.raises(ValueError, match="quota"):
        ta2a._raise_from_status(st, 4, 4, 2)
    st = torch.tensor([1, 8, 0, 0], dtype=torch.int32)
    with pytest.raises(ValueError, match="out of range"):
        ta2a._raise_from_status(st, 4, 4, 2)
    ta2a._raise_from_status(torch.tensor([0, 8, 0, 0], dtype=torch.int32), 4, 4, 2)


def test_pack_mode_switch(monkeypatch):
    from terrace import ta2a_pack as pk
    monkeypatch.delenv("TERRACE_TA2A_PACK", raising=False)
    pk.reset()
    assert pk.pack_mode() == "small" and pk.pack_enabled()
    for raw, mode in [("0", "off"), ("1", "small"), ("full", "full"), ("2", "full"), ("meta", "small")]:
        monkeypatch.setenv("TERRACE_TA2A_PACK", raw)
        pk.reset()
        assert pk.pack_mode() == mode
    monkeypatch.setenv("TERRACE_TA2A_PACK", "ful")
    pk.reset()
    with pytest.raises(RuntimeError, match="not a valid mode"):
        pk.pack_mode()
    monkeypatch.delenv("TERRACE_TA2A_PACK")
    pk.reset()
    monkeypatch.setattr(pk, "pack_enabled", lambda: False)
    assert pk.pack_mode() == "off"
    lay = pk.HopALayout(2048, 3, 3, False, torch.bfloat16)
    assert lay.words == 516 and pk.HopASmallLayout(3, 3, False, torch.bfloat16).words == 4


def test_traffic_file_is_what_bench_reads():
    """profiles/traffic.json: a source digest and positive byte counts keyed "<config>:<kernel>"; bench.py hands
    the roofline's `traffic` out of it only when the digest is the loaded library's, and None otherwise."""
    import json
    import bench
    with open(bench.TRAFFIC_FILE) as f:
        rec = json.load(f)
    assert isinstance(rec["source_digest"], str) and len(rec["source_digest"]) == 16
    per_launch = rec["bytes_per_launch"]
    assert "c2:gather_rows_sliced_kernel(regroup)" in per_launch
    for key, nbytes in per_launch.items():
        config, kernel = key.split(":", 1)
        assert config in ("c1", "c2", "c3", "c4", "c5") and kernel and isinstance(nbytes, int) and nbytes > 0
    key = "c2:gather_rows_sliced_kernel(regroup)"
    assert bench.measured_traffic("c2", "gather_rows_sliced_kernel(regroup)", rec["source_digest"]) == per_launch[key]
    assert bench.measured_traffic("c2", "gather_rows_sliced_kernel(regroup)", "0" * 16) is None
    assert bench.measured_traffic("c2", "no_such_kernel", rec["source_digest"]) is None
