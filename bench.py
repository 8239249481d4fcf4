"""Benchmark of one rank's dispatch/combine path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2] [--no-cpu-baseline] [--graph]

A step is one pass of the hot path over one batch of synthetic input that is already resident
in HBM: T-Route -> dispatch index build + Hop-A deduplicated pack -> Hop-B arrival chain ->
expert-order regroup (with capacity padding where the workload has a capacity factor) ->
gate-weighted fp32-accumulating combine.  The expert FFN between regroup and combine is not
part of the path; its output is a fixed synthetic tensor prepared before the timed region.
The all-to-all exchanges are not executed (one GPU): the rank's Hop-A send buffer is looped
back as its arrival buffer.

Prints ONE JSON line: whole-step algorithmic GB/s as `value` (each payload row counted once on the
read side and once on the write side of every stage) and, beside it, the same step priced on the
bytes that must cross HBM (`min_traffic`); per-stage ms / GB/s / fraction of the 8 TB/s HBM peak
and the arrival chain's us/row in `stages`, the roofline record of
the slowest row-moving kernel (timed alone with HIP events on the launch stream), and the CPU
oracle timed on the host cores over a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "terracemoe-simulator_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of a workload's dominant kernel, measured with rocprofv3 --pmc FETCH_SIZE
# and WRITE_SIZE and scaled by the same counters' reading for the copy kernel (fetch x2.00,
# write x1.00).  Only workloads that have been measured are listed; others report null.
MEASURED_TRAFFIC_BYTES = {("c2", "gather_rows_sliced_kernel(regroup)"): 3.767e9}
REFERENCE_TARGET_US_PER_ROW = 0.012     # the reference's fused-chain design target


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="c2")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--graph", action="store_true",
                    help="also capture the step into a HIP graph and time its replays (reported beside the eager "
                         "figure, which stays `value`)")
    ap.add_argument("--cpu-sample-tokens", type=int, default=1 << 20,
                    help="tokens of the workload the CPU baseline runs on (default: all of them)")
    return ap.parse_args()


def event_ms(fn, reps, torch):
    """Average milliseconds of fn() over reps launches, HIP events on the current stream."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    fn()
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / reps


def cpu_baseline(cfg, sample_tokens):
    """The CPU oracle timed on the host cores over `sample_tokens` tokens of the same geometry:
    the OpenMP C restatement (oracle/terrace_oracle.c) when its library is built, else the numpy
    one.  Passes are repeated for about eight seconds (3 to 40 of them: the hosts are shared and noisy) and
    each stage's best time counts; algorithmic GB/s over the same stage set as the GPU figure."""
    import numpy as np
    import torch
    from oracle import c_oracle as corc
    from oracle import terrace_oracle as orc
    from terrace import configs
    use_c = corc.available()
    small = cfg.scaled(min(sample_tokens if use_c else min(sample_tokens, 1024), cfg.T))
    inp = configs.make_inputs(small)
    logits, bias = inp["logits"].numpy(), inp["bias"].numpy()
    ga = None if inp["gate_affinity"] is None else inp["gate_affinity"].numpy()
    if small.fmt == "f32":
        x, gcast, fmt = inp["x"].numpy(), (lambda g: g), "f32"
    elif small.fmt == "bf16":
        x, gcast, fmt = inp["x"].view(torch.int16).numpy().view(np.uint16), orc.f32_to_bf16, "bf16"
    else:
        x, gcast, fmt = inp["x"].numpy(), orc.f32_to_bf16, "fp8"
    impl = corc if use_c else orc
    best, totals, began = None, [], time.perf_counter()
    while len(totals) < 3 or (len(totals) < 40 and time.perf_counter() - began < 8.0):
        t = _oracle_pass(impl, orc, np, small, logits, bias, ga, x, gcast, fmt, use_c)
        totals.append(sum(t.values()))
        best = t if best is None else {k: min(best[k], t[k]) for k in t}
    t = best
    nbytes = sum(configs.algorithmic_bytes(small).values())
    total = sum(t.values())
    cores = corc.threads() if use_c else 1
    what = f"OpenMP C oracle ({cores} threads)" if use_c else "numpy oracle (1 thread)"
    return {"value": round(nbytes / total / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"{what}, whole path on {small.T} of {cfg.T} tokens of {cfg.name}, each stage's best of "
                      f"{len(totals)} passes ({total:.3f} s: " + ", ".join(f"{k} {v:.3f}" for k, v in t.items()) +
                      f"; whole passes took {min(totals):.3f} to {max(totals):.3f} s, median "
                      f"{sorted(totals)[len(totals) // 2]:.3f})",
            "arrival_us_per_row": round(t["arrival"] * 1e6 / small.pairs, 4)}


def _oracle_pass(impl, orc, np, small, logits, bias, ga, x, gcast, fmt, use_c):
    t = {}
    t0 = time.perf_counter()
    if use_c:
        e, gates, _ = impl.t_route(logits, bias, small.n_experts, small.n_groups, small.top_k, small.top_groups,
                                   2, ga)
    else:
        e, gates, _ = impl.t_route(logits, bias, small.n_experts, small.n_groups, small.top_k, small.top_groups,
                                   gate_affinity=ga)
    t["route"] = time.perf_counter() - t0
    gq = gcast(gates)
    t0 = time.perf_counter()
    packed = impl.k2_pack(x, e, gq, small.world, small.n_experts, small.rpn, small.top_groups)
    payload, mask, gate_rows = packed[0], packed[1], packed[2]
    t["pack"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    arrived = impl.k1_arrival(payload, mask, gate_rows, small.quota, small.epr, small.rpn)
    send, s_idx = arrived[0], arrived[3]
    t["arrival"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    cap = small.capacity(small.slots)
    if use_c:
        perm, place, _kept, _tpe = impl.regroup(send, s_idx, small.slots, 0, cap)
    elif cap is None:
        perm, order, _tpe = impl.regroup(send, s_idx, small.slots)
        place = np.empty_like(order)
        place[order] = np.arange(order.size)
    else:
        perm, place, _kept, _tpe, _kpe = impl.regroup(send, s_idx, small.slots, capacity=cap)
    t["regroup"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    if use_c:
        pair_tab, sort_order, pos = packed[5]["pair_table"], packed[5]["sort_order"], arrived[5]
    else:
        _, _, _, inverse = orc.plan_ta2a(e, small.world, small.n_experts, small.rpn, small.top_groups)
        pair_tab, sort_order = orc.token_pair_table(e, inverse, small.quota)
        pos = orc.arrival_positions(mask, small.epr, small.rpn)
    where = place[pos[pair_tab]]
    w_sorted = np.take_along_axis(gates, sort_order, 1)
    impl.combine(perm, where, w_sorted, fmt, "f32" if fmt == "f32" else "bf16", hidden=small.hidden)
    t["combine"] = time.perf_counter() - t0
    return t


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU's share of the path; the all-to-all exchanges "
              "between ranks are not part of it, so --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    import torch

    import terrace
    import terrace.ops as tops
    from terrace import _hip, configs
    from terrace.ta2a_fwd import loopback_combine, loopback_dispatch

    if not torch.cuda.is_available():
        print("bench.py: no ROCm device", file=sys.stderr)
        sys.exit(3)
    st = tops.status()
    if not st.loaded:
        print(f"bench.py: kernel library not loaded: {st.reason}", file=sys.stderr)
        sys.exit(3)
    cfg = configs.CONFIGS[args.config]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    inp = configs.make_inputs(cfg)
    logits, bias, x = inp["logits"].to(dev), inp["bias"].to(dev), inp["x"].to(dev)
    gate_aff = None if inp["gate_affinity"] is None else inp["gate_affinity"].to(dev)
    rcfg = terrace.TRouteConfig(cfg.n_experts, cfg.n_groups, cfg.top_k, cfg.top_groups)
    cap = cfg.capacity(cfg.slots)
    fp8_hidden = cfg.hidden if cfg.fmt == "fp8" else None

    def route():            # the gates leave the kernel in the payload dtype: no cast launch between the stages
        return terrace.t_route(logits, bias, rcfg, gate_affinity=gate_aff, gates_dtype=cfg.gate_dtype)

    e, gates, _ = route()
    state = loopback_dispatch(x, e, gates, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups, cap)
    # fixed synthetic expert output, one row per place of the expert-order buffer
    if cfg.fmt == "fp8":
        g = torch.Generator(device=dev).manual_seed(cfg.seed)
        ye = configs.quantise_fp8_rows(torch.randn(state.permuted.shape[0], cfg.hidden, generator=g, device=dev))
    else:
        ye = state.permuted.clone()
    torch.cuda.synchronize()

    def step():
        e_, g_, _ = route()
        s_ = loopback_dispatch(x, e_, g_, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups, cap)
        return loopback_combine(ye, s_, out_dtype=cfg.out_dtype, fp8_hidden=fp8_hidden)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # ---- optional: the same step as one HIP graph (launch overhead off the critical path) ----
    graph_rec = None
    if args.graph:
        y_eager = step()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y_graph = step()
        same = True
        for _ in range(3):                 # replays interleaved with eager work must all reproduce the eager result
            graph.replay()
            torch.cuda.synchronize()
            same = same and bool(torch.equal(y_graph, y_eager))
            step()
            torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_rec = {"ms_per_step": round((time.perf_counter() - t0) * 1e3 / args.steps, 4),
                     "replays_match_eager": same}

    # ---- per-stage timings (each stage alone, HIP events on the launch stream) ----
    nbytes = configs.algorithmic_bytes(cfg)
    reps = max(args.steps, 5)
    quota = cfg.quota

    def pack():
        return tops.k2_pack_raw(x, e, gates, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups, extras=True)

    def arrival():
        return tops.k1_arrival_raw(state.payload, state.mask, state.gate_rows, quota, cfg.epr, cfg.rpn, 0,
                                   want_pair_pos=True)

    def regroup():
        return tops.regroup(state.send_buf, state.slot_idx, cfg.slots, 0, cap)

    def combine():
        return loopback_combine(ye, state, out_dtype=cfg.out_dtype, fp8_hidden=fp8_hidden)

    stage_ms = {"route": event_ms(route, reps, torch), "pack": event_ms(pack, reps, torch),
                "arrival": event_ms(arrival, reps, torch), "regroup": event_ms(regroup, reps, torch),
                "combine": event_ms(combine, reps, torch)}
    kept_pairs = int((state.place >= 0).sum()) if cap is not None else None
    min_bytes = configs.minimum_traffic_bytes(cfg, kept_pairs, None if cap is None else cfg.slots * cap)
    stages = {}
    # rows a stage writes: send rows, (row, slot) pairs, places of the expert-order buffer, tokens
    rows_out = {"route": cfg.T, "pack": cfg.send_rows, "arrival": cfg.pairs,
                "regroup": cfg.pairs if cap is None else cfg.slots * cap, "combine": cfg.T}
    for name, ms in stage_ms.items():
        gbps = nbytes[name] / ms / 1e6
        min_gbps = min_bytes[name] / ms / 1e6
        # "GBps" follows the convention that counts a payload row once on the read and once on the write side of
        # a stage (a scatter that reads a row once for all its copies can thus exceed the peak); "min_traffic"
        # prices the bytes that must cross HBM
        stages[name] = {"ms": round(ms, 4), "GBps": round(gbps, 1), "frac_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4),
                        "min_traffic_GBps": round(min_gbps, 1),
                        "min_traffic_frac_hbm_peak": round(min_gbps / HBM_PEAK_GBPS, 4),
                        "us_per_row": round(ms * 1e3 / max(rows_out[name], 1), 6)}
    stages["arrival"]["reference_target_us_per_row"] = REFERENCE_TARGET_US_PER_ROW
    pc_bytes = nbytes["pack"] + nbytes["combine"]
    pc_ms = stage_ms["pack"] + stage_ms["combine"]

    # ---- the row-moving kernels alone ----
    row = cfg.row_bytes
    where = tops.index_chain2(state.place, state.pair_pos, state.extras["pair_table"])
    w_sorted = state.extras["gate_sorted"]
    token_rows, pair_pos2 = state.extras["token_rows"], state.pair_pos.view(cfg.send_rows, quota)
    if cap is None:
        _, order, _ = tops.regroup(state.send_buf, state.slot_idx, cfg.slots, 0, None)
        gather_idx = order
    else:
        gather_idx = torch.full((cfg.slots * cap,), -1, dtype=torch.int64, device=dev)
        ok = state.place >= 0
        gather_idx[state.place[ok]] = torch.arange(cfg.pairs, device=dev)[ok]
    out_row = cfg.hidden * (4 if cfg.fmt == "f32" else 2)
    # names of the kernels the library picks for this row width (whole kilobytes or not)
    kb_rows = row % 1024 == 0
    k_scatter = "scatter_rows_sliced_kernel" if kb_rows else "scatter_rows_aligned_kernel"
    k_gather = "gather_rows_sliced_kernel" if kb_rows else "gather_rows_flat_kernel"
    kernels = {
        f"{k_scatter}(pack)": (lambda: tops.scatter_rows(x, token_rows, cfg.send_rows), 2 * cfg.send_rows * row),
        f"{k_scatter}(arrival)": (lambda: tops.scatter_rows(state.payload, pair_pos2, cfg.pairs),
                                  2 * cfg.pairs * row),
        f"{k_gather}(regroup)": (lambda: tops.gather_rows(state.send_buf, gather_idx),
                                 2 * gather_idx.numel() * row),
        "combine_kernel": (lambda: tops.combine(ye, where, w_sorted, out_dtype=cfg.out_dtype, fp8_hidden=fp8_hidden),
                           cfg.pairs * row + cfg.pairs * 12 + cfg.T * out_row),
        "copy_kernel(passthrough)": (lambda: tops.passthrough(state.send_buf), 2 * state.send_buf.numel()
                                     * state.send_buf.element_size()),
    }
    kern = {}
    for name, (fn, nb) in kernels.items():
        ms = event_ms(fn, reps, torch)
        kern[name] = {"ms": round(ms, 4), "algorithmic_bytes": nb, "GBps": round(nb / ms / 1e6, 1)}
    dominant = max((k for k in kern if not k.startswith("copy")), key=lambda k: kern[k]["ms"])
    achieved = kern[dominant]["GBps"]
    roofline = {"bound": "hbm", "kernel": dominant, "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBPS, 4),
                "traffic": MEASURED_TRAFFIC_BYTES.get((args.config, dominant)),
                "avg_launch_ms": kern[dominant]["ms"], "algorithmic_bytes_per_launch": kern[dominant]["algorithmic_bytes"]}

    total_bytes = sum(nbytes.values())
    value = total_bytes / ms_per_step / 1e6
    out = {
        "metric": "dispatch_combine_algorithmic_GBps",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"f32": "f32", "bf16": "bf16", "fp8": "fp8_e4m3+f32 scales"}[cfg.fmt] + " rows, fp32 accumulate",
        "data": "synthetic",
        "config": {"workload": cfg.name, "T": cfg.T, "E": cfg.n_experts, "n_groups": cfg.n_groups, "k": cfg.top_k,
                   "M": cfg.top_groups, "cards_per_group": cfg.rpn, "hidden": cfg.hidden, "row_bytes": row,
                   "send_rows": cfg.send_rows, "pairs": cfg.pairs, "capacity": cap,
                   "exchange": "loop-back (no all-to-all on one GPU)",
                   "expert_outputs": "fixed synthetic tensor prepared before the timed region"},
        "frac_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "min_traffic": {"GBps": round(sum(min_bytes.values()) / ms_per_step / 1e6, 1),
                        "frac_hbm_peak": round(sum(min_bytes.values()) / ms_per_step / 1e6 / HBM_PEAK_GBPS, 4),
                        "note": "bytes that must cross HBM: a scatter reads each source row once however many "
                                "copies it writes, a capacity layout reads only the rows it keeps"},
        "pack_plus_combine": {"GBps": round(pc_bytes / pc_ms / 1e6, 1),
                              "frac_hbm_peak": round(pc_bytes / pc_ms / 1e6 / HBM_PEAK_GBPS, 4),
                              "min_traffic_GBps": round((min_bytes["pack"] + min_bytes["combine"]) / pc_ms / 1e6, 1),
                              "min_traffic_frac_hbm_peak": round((min_bytes["pack"] + min_bytes["combine"]) / pc_ms
                                                                 / 1e6 / HBM_PEAK_GBPS, 4)},
        "arrival_chain_us_per_row": stages["arrival"]["us_per_row"],
        "stages": stages, "kernels": kern, "roofline": roofline,
        "library": os.path.relpath(st.lib, ROOT),
    }
    if graph_rec is not None:
        out["hip_graph"] = graph_rec
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, args.cpu_sample_tokens)
        out["cpu_baseline"]["host_cores_available"] = os.cpu_count()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
