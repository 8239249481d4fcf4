"""Benchmark of one rank's dispatch/combine path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2] [--no-cpu-baseline] [--no-other-configs]
                    [--no-seam] [--no-in-order] [--tokens N] [--graph]

A step is one pass of the hot path over one batch of synthetic input that is already resident
in HBM: T-Route -> dispatch index build + Hop-A deduplicated pack -> Hop-B arrival chain ->
expert-order regroup (with capacity padding where the workload has a capacity factor) ->
gate-weighted fp32-accumulating combine.  The expert FFN between regroup and combine is not
part of the path; its output is a fixed synthetic tensor prepared before the timed region.
The all-to-all exchanges are not executed (one GPU): the rank's Hop-A send buffer is looped
back as its arrival buffer.

Prints ONE JSON line.  `value` is the whole step priced on the bytes that must cross HBM (a scatter
reads each source row once however many copies it writes; a capacity layout reads only the rows it
keeps) over the step time; no figure in the line named `frac_hbm_peak` uses any other convention.
The convention that counts a payload row once on the read and once on the write side of every stage
is reported beside it as `rows_counted_twice_GBps` only.  Also in the line: per-stage ms / GB/s /
fraction of the 8 TB/s HBM peak and the arrival chain's us/row (`stages`), the same step with Hop B
as one pass (`onepass`), every stage timed between events inside whole steps (`in_step`), the row movers alone
with their floor at the run's own stream rates and their time over tables that list the rows in order (`kernels`:
`ms_rows_in_order`), those stream rates -- read-only, write-only, 8:1 sum,
copy -- from the library's probe kernels (`ceilings`), the seam halves ta2a_permute + ta2a_unpermute on the quota
branch, the general branch and the overlap seam with their launches named (`seam`), the other four workloads
(`other_configs`), the roofline record of the
slowest row-moving kernel (timed alone with HIP events on the launch stream; `traffic` from
profiles/traffic.json when that file was measured on the sources the loaded library was built
from), and the CPU baseline: the fastest CPU implementation measured in the run (the OpenMP C restatement of
the oracle over the whole workload), with the path as a chain of torch CPU operators beside it.
"""
from __future__ import annotations

import argparse
import gc
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "terracemoe-simulator_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")
REFERENCE_TARGET_US_PER_ROW = 0.012     # the reference's fused-chain design target


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="c2")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true")
    ap.add_argument("--no-seam", action="store_true", help="skip the ta2a_permute / ta2a_unpermute timings")
    ap.add_argument("--no-in-order", action="store_true",
                    help="skip the movers' launches over renumbered tables (a kernel trace then holds only launches "
                         "over the workload's own tables)")
    ap.add_argument("--row-pitch", type=int, default=None,
                    help="bytes between payload rows in every row buffer of --config (0: rows back to back; default: "
                         "what the workload names)")
    ap.add_argument("--tokens", type=int, default=None,
                    help="run --config with this many tokens instead of its own (e.g. a decode-sized batch; the "
                         "measured-traffic record of profiles/ then does not apply and `traffic` is null)")
    ap.add_argument("--graph", action="store_true",
                    help="also capture the step into a HIP graph and time its replays (reported beside the eager "
                         "figure, which stays `value`)")
    ap.add_argument("--cpu-sample-tokens", type=int, default=1024,
                    help="tokens of the workload the torch-CPU chain runs on")
    return ap.parse_args()


EVENT_BATCHES = 5


def event_ms(fn, reps, torch, batches=EVENT_BATCHES):
    """Milliseconds per launch of fn(): the median over `batches` batches of the average over `reps` back-to-back
    launches, each batch between two HIP events on the current stream (a median so that one disturbed batch
    does not move the figure)."""
    fn()
    torch.cuda.synchronize()
    per_batch = []
    for _ in range(batches):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            fn()
        stop.record()
        stop.synchronize()
        per_batch.append(start.elapsed_time(stop) / reps)
    return statistics.median(per_batch)


def wall_ms(fn, steps, warmup, torch):
    """W untimed steps, then exactly K timed ones between two device synchronisations.  The interpreter's cyclic
    garbage collector is held off for the timed region, as ``timeit`` does: a full collection pass stalls the host
    for tens of milliseconds, which is this process's bookkeeping and not a cost of the path."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    was_enabled = gc.isenabled()
    gc.disable()
    try:
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps
    finally:
        if was_enabled:
            gc.enable()


def measured_traffic(workload, kernel, digest):
    """HBM bytes per launch of `kernel` on `workload` from profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE and
    WRITE_SIZE, scaled by the copy kernel's reading), or None when the file was measured on other sources."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None
    if rec.get("source_digest") != digest:
        return None
    return rec.get("bytes_per_launch", {}).get(f"{workload}:{kernel}")


# ------------------------------------------------------------------------------------------------------------------
# CPU baseline
# ------------------------------------------------------------------------------------------------------------------

def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _torch_chain_pass(tch, torch, cfg, inp, x, ye_of):
    """One pass of the operator chain; per-stage seconds."""
    t = {}
    t0 = time.perf_counter()
    e, gates, _ = tch.t_route(inp["logits"], inp["bias"], cfg.n_experts, cfg.n_groups, cfg.top_k, cfg.top_groups,
                              inp["gate_affinity"])
    t["route"] = time.perf_counter() - t0
    gq = gates.to(cfg.gate_dtype)
    t0 = time.perf_counter()
    payload, mask, gate_rows, u_src, _counts, _inv = tch.k2_pack(x, e, gq, cfg.world, cfg.n_experts, cfg.rpn,
                                                                 cfg.top_groups)
    t["pack"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    send, gp, r_idx, s_idx, _i_send, _ordo = tch.k1_arrival(payload, mask, gate_rows, cfg.quota, cfg.epr, cfg.rpn)
    t["arrival"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    perm, place, _tpe = tch.regroup(send, s_idx, cfg.slots, cfg.capacity(cfg.slots))
    t["regroup"] = time.perf_counter() - t0
    ye = ye_of(perm)
    t0 = time.perf_counter()
    tch.combine_two_level(ye, place, r_idx, gp, u_src, u_src.numel(), cfg.T)
    t["combine"] = time.perf_counter() - t0
    return t


def torch_chain_baseline(cfg, sample_tokens, threads):
    """Median-of-10 per stage (3 warm-up passes) of the torch-CPU operator chain on `sample_tokens` tokens of the
    workload, at `threads` intra-op threads."""
    import torch
    from oracle import torch_chain as tch
    from terrace import configs
    small = cfg.scaled(min(sample_tokens, cfg.T))
    inp = configs.make_inputs(small)
    x = inp["x"].contiguous()           # the CPU chain moves packed rows
    if small.fmt == "fp8":          # the rows travel as bytes; the expert output is dequantised where the combine reads it
        h = small.hidden

        def ye_of(perm):
            codes = perm[:, :h].contiguous().view(torch.float8_e4m3fn).float()
            scales = perm[:, h:].contiguous().view(torch.float32).repeat_interleave(configs.FP8_BLOCK, dim=1)
            return (codes * scales).to(torch.bfloat16)
    else:
        def ye_of(perm):
            return perm
    before = torch.get_num_threads()
    torch.set_num_threads(threads)
    try:
        for _ in range(3):
            _torch_chain_pass(tch, torch, small, inp, x, ye_of)
        passes = [_torch_chain_pass(tch, torch, small, inp, x, ye_of) for _ in range(10)]
    finally:
        torch.set_num_threads(before)
    med = {k: statistics.median(p[k] for p in passes) for k in passes[0]}
    total = sum(med.values())
    kept = None
    nbytes = sum(configs.minimum_traffic_bytes(small, kept, None if small.capacity(small.slots) is None
                                               else small.slots * small.capacity(small.slots)).values())
    return {"threads": threads, "tokens": small.T, "GBps": round(nbytes / total / 1e9, 3),
            "ms_per_pass": round(total * 1e3, 2), "stage_ms": {k: round(v * 1e3, 3) for k, v in med.items()},
            "arrival_us_per_row": round(med["arrival"] * 1e6 / small.pairs, 4),
            "repetitions": len(passes), "statistic": "median per stage"}


def openmp_port_baseline(cfg):
    """The OpenMP C restatement (oracle/terrace_oracle.c) over the whole workload; None when it is not built."""
    import numpy as np
    import torch
    from oracle import c_oracle as corc
    from oracle import terrace_oracle as orc
    from terrace import configs
    if not corc.available():
        return None
    inp = configs.make_inputs(cfg)
    logits, bias = inp["logits"].numpy(), inp["bias"].numpy()
    ga = None if inp["gate_affinity"] is None else inp["gate_affinity"].numpy()
    if cfg.fmt == "f32":
        x, gcast, fmt = inp["x"].numpy(), (lambda g: g), "f32"
    elif cfg.fmt == "bf16":
        x, gcast, fmt = inp["x"].view(torch.int16).numpy().view(np.uint16), orc.f32_to_bf16, "bf16"
    else:
        x, gcast, fmt = inp["x"].contiguous().numpy(), orc.f32_to_bf16, "fp8"
    passes, began = [], time.perf_counter()
    while len(passes) < 3 or (len(passes) < 12 and time.perf_counter() - began < 6.0):
        passes.append(_openmp_pass(corc, np, cfg, logits, bias, ga, x, gcast, fmt))
    med = {k: statistics.median(p[k] for p in passes) for k in passes[0]}
    total = sum(med.values())
    cap = cfg.capacity(cfg.slots)
    nbytes = sum(configs.minimum_traffic_bytes(cfg, None, None if cap is None else cfg.slots * cap).values())
    return {"threads": corc.threads(), "tokens": cfg.T, "GBps": round(nbytes / total / 1e9, 3),
            "ms_per_pass": round(total * 1e3, 2), "stage_ms": {k: round(v * 1e3, 3) for k, v in med.items()},
            "arrival_us_per_row": round(med["arrival"] * 1e6 / cfg.pairs, 4), "repetitions": len(passes),
            "statistic": "median per stage"}


def _openmp_pass(impl, np, cfg, logits, bias, ga, x, gcast, fmt):
    t = {}
    t0 = time.perf_counter()
    e, gates, _ = impl.t_route(logits, bias, cfg.n_experts, cfg.n_groups, cfg.top_k, cfg.top_groups, 2, ga)
    t["route"] = time.perf_counter() - t0
    gq = gcast(gates)
    t0 = time.perf_counter()
    packed = impl.k2_pack(x, e, gq, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups)
    t["pack"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    arrived = impl.k1_arrival(packed[0], packed[1], packed[2], cfg.quota, cfg.epr, cfg.rpn)
    t["arrival"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    perm, place, _kept, _tpe = impl.regroup(arrived[0], arrived[3], cfg.slots, 0, cfg.capacity(cfg.slots))
    t["regroup"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    where = place[arrived[5][packed[5]["pair_table"]]]
    w_sorted = np.take_along_axis(gates, packed[5]["sort_order"], 1)
    impl.combine(perm, where, w_sorted, fmt, "f32" if fmt == "f32" else "bf16", hidden=cfg.hidden)
    t["combine"] = time.perf_counter() - t0
    return t


def cpu_baseline(cfg, sample_tokens):
    """`value` is the fastest CPU implementation measured in this run: the OpenMP C restatement of the oracle over
    the whole workload when it is built, else the torch operator chain at all threads.  The torch chain -- the
    reference's own op composition -- is always reported beside it, at one thread and at all."""
    cores = os.cpu_count() or 1
    one = torch_chain_baseline(cfg, sample_tokens, 1)
    many = torch_chain_baseline(cfg, sample_tokens, cores) if cores > 1 else one
    port = openmp_port_baseline(cfg)
    chain_sample = (f"the path as a chain of torch CPU operators (oracle/torch_chain.py: topk/gather, "
                    f"scatter_+cumsum+searchsorted, row gathers, composite-key argsort+scatter_add_, index_add_) on "
                    f"{many['tokens']} of {cfg.T} tokens of {cfg.name}, 3 warm-up passes then the median of 10 per stage")
    if port is not None and port["GBps"] >= many["GBps"]:
        value, threads = port["GBps"], port["threads"]
        sample = (f"oracle/terrace_oracle.c (OpenMP restatement of the path) over all {cfg.T} tokens of {cfg.name}, "
                  f"median per stage of {port['repetitions']} passes at {port['threads']} threads; same "
                  f"bytes-that-must-cross-memory pricing as `value`")
    else:
        value, threads = many["GBps"], many["threads"]
        sample = chain_sample + f", at {many['threads']} threads; same bytes-that-must-cross-memory pricing as `value`"
    return {"value": value, "unit": "GB/s", "cores": threads, "kind": "port", "sample": sample,
            "cpu_model": _cpu_model(), "host_cores_available": cores,
            "torch_chain_GBps": many["GBps"], "torch_chain_1_thread_GBps": one["GBps"],
            "openmp_c_port_GBps": None if port is None else port["GBps"],
            "torch_chain_sample": chain_sample,
            "torch_chain_1_thread": one, "torch_chain_all_threads": many, "openmp_c_port_whole_workload": port}


# ------------------------------------------------------------------------------------------------------------------
# stream ceilings, the seam halves, a step inside a HIP graph
# ------------------------------------------------------------------------------------------------------------------

def stream_ceilings(torch, reps):
    """What the part sustains, in this run, for the traffic mixes the row movers are made of: the library's own
    stream probes (terrace_stream_probe) at the c2 sizes -- a 1.88 GB read-only stream, a 0.94 GB write-only one,
    the 8:1 streaming sum (1.88 GB read, 0.23 GB written) and a 1.88 + 1.88 GB copy in one-wave workgroups --
    beside terrace_passthrough's 256-lane copy."""
    import terrace.ops as tops
    dev = torch.device("cuda:0")
    big = 1879048192                       # bytes of c2's arrival buffer
    src = torch.zeros(big, dtype=torch.uint8, device=dev)
    dst = torch.empty(big, dtype=torch.uint8, device=dev)
    out = {}
    cases = {"read_only": ("read", src, dst, big), "write_only": ("write", None, dst[: big // 2], big // 2),
             "sum_8_to_1": ("sum8", src, dst[: big // 8], big + big // 8), "copy_one_wave": ("copy", src, dst, 2 * big)}
    for name, (kind, x, y, nbytes) in cases.items():
        ms = event_ms(lambda: tops.stream_probe(kind, x, y), reps, torch)
        out[name] = {"ms": round(ms, 4), "bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1),
                     "frac_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    ms = event_ms(lambda: tops.passthrough(src), reps, torch)
    out["copy_passthrough"] = {"ms": round(ms, 4), "bytes": 2 * big, "GBps": round(2 * big / ms / 1e6, 1),
                               "frac_hbm_peak": round(2 * big / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    out["note"] = ("terrace_stream_probe kernels timed like the movers (HIP events, median of batches); a mover's "
                   "floor on this part is its read bytes at the read_only rate plus its written bytes at the "
                   "write_only rate")
    return out


def predicted_floor_ms(ceil, read_bytes, written_bytes):
    """Milliseconds a kernel's bytes cost at the run's own read-only and write-only stream rates."""
    return read_bytes / (ceil["read_only"]["GBps"] * 1e6) + written_bytes / (ceil["write_only"]["GBps"] * 1e6)


def count_launches(fn, torch, names=None):
    """Kernel launches one call of fn() makes, from torch's profiler (None when it is unavailable, e.g. under
    another profiler).  `names`, a dict, receives kernel name -> [launches, microseconds on the device]."""
    try:
        from torch.profiler import ProfilerActivity, profile
        fn()
        torch.cuda.synchronize()
        with profile(activities=[ProfilerActivity.CUDA]) as prof:
            fn()
            torch.cuda.synchronize()
        n = 0
        for ev in prof.events():
            if ev.device_type is not None and "cuda" in str(ev.device_type).lower() and "memcpy" not in ev.name.lower() \
                    and "memset" not in ev.name.lower():
                n += 1
                if names is not None:
                    short = ev.name.split("(")[0].split("<")[0].split("::")[-1].strip() or ev.name[:40]
                    rec = names.setdefault(short, [0, 0.0])
                    rec[0] += 1
                    rec[1] = round(rec[1] + float(getattr(ev, "device_time_total", 0.0) or 0.0), 1)
        return n or None
    except Exception:
        return None


def seam_block(cfg, args, torch, raw_step_ms, e, gates, x):
    """The Megatron-shaped surface (terrace/ta2a_dispatch.py of the reference: ta2a_permute -> experts ->
    ta2a_unpermute) at this workload's shape: ms per permute + unpermute pair, launches and host synchronisations
    per pair, and the ratio to the raw loop-back step (route excluded there as here)."""
    import terrace.ta2a_dispatch as seam
    from terrace import ta2a_pack
    dev = x.device
    T, E = cfg.T, cfg.n_experts
    routing_map = torch.zeros((T, E), dtype=torch.bool, device=dev)
    routing_map.scatter_(1, e, True)
    probs = torch.zeros((T, E), dtype=x.dtype, device=dev)
    probs.scatter_(1, e, gates.to(x.dtype))
    kw = dict(world=cfg.world, rank=0, rpn=cfg.rpn, n_experts=E)
    ta2a_pack.reset()

    def plain(groups_m):
        def run():
            permuted, _tpe, _pp, st = seam.ta2a_permute(x, probs, routing_map, groups_m=groups_m, **kw)
            return seam.ta2a_unpermute(permuted, st, x)
        return run

    def overlap():
        saved = []
        permuted, _tpe, _pp, _sh, st = seam.ta2a_permute_overlap(x, probs, routing_map, groups_m=cfg.top_groups,
                                                                save_tensors=saved, **kw)
        return seam.ta2a_unpermute_overlap(permuted.detach(), st, saved)

    legs = {"quota_branch_small_containers": (plain(cfg.top_groups), 1),
            "general_branch": (plain(None), 2),
            "overlap_seam_quota_branch": (overlap, 1)}
    out = {"container_mode": ta2a_pack.pack_mode(), "raw_dispatch_plus_combine_ms": round(raw_step_ms, 4),
           "note": "wall time per ta2a_permute + ta2a_unpermute pair (expert output = the permuted rows), host "
                   "synchronisations included; the raw figure is loopback_dispatch + the fused combine on the same "
                   "rows.  The seam's combine is the reference's two levels (a send row sums its pairs, a token its "
                   "rows): it writes and re-reads the [T*M, H] plane the fused combine never forms"}
    with torch.no_grad():
        for name, (fn, syncs) in legs.items():
            ms = wall_ms(fn, max(args.steps // 2, 5), 2, torch)
            names = {}
            out[name] = {"ms_per_call": round(ms, 4), "ratio_to_raw": round(ms / raw_step_ms, 3),
                         "kernel_launches": count_launches(fn, torch, names), "host_syncs": syncs,
                         "kernels_launches_us": names}
    return out


def graph_replay_ms(step, args, torch):
    """The step captured once into a HIP graph: ms per replay, and whether replays interleaved with eager steps
    reproduce the eager result every time."""
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
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        same = same and bool(torch.equal(y_graph, y_eager))
        step()
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        graph.replay()
    torch.cuda.synchronize()
    return {"ms_per_step": round((time.perf_counter() - t0) * 1e3 / args.steps, 4), "replays_match_eager": same}


# ------------------------------------------------------------------------------------------------------------------
# one workload on the GPU
# ------------------------------------------------------------------------------------------------------------------

def run_workload(cfg, args, torch, detail):
    """Times the step (two-step Hop B: the drop-in operators), the same step with Hop B as one pass, and --
    with `detail` -- every stage and every row mover alone.  Returns a dict of figures."""
    import terrace
    import terrace.ops as tops
    from terrace import configs
    from terrace.ta2a_fwd import loopback_combine, loopback_dispatch, loopback_dispatch_onepass

    dev = torch.device("cuda:0")
    inp = configs.make_inputs(cfg)
    logits, bias, x = inp["logits"].to(dev), inp["bias"].to(dev), configs.rows_to(inp["x"], dev)
    gate_aff = None if inp["gate_affinity"] is None else inp["gate_affinity"].to(dev)
    rcfg = terrace.TRouteConfig(cfg.n_experts, cfg.n_groups, cfg.top_k, cfg.top_groups)
    cap = cfg.capacity(cfg.slots)
    fp8_hidden = cfg.hidden if cfg.fmt == "fp8" else None
    geom = (cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups, cap)

    def route():            # the gates leave the kernel in the payload dtype: no cast launch between the stages
        return terrace.t_route(logits, bias, rcfg, gate_affinity=gate_aff, gates_dtype=cfg.gate_dtype)

    e, gates, _ = route()
    state = loopback_dispatch(x, e, gates, *geom)
    # fixed synthetic expert output, one row per place of the expert-order buffer
    if cfg.fmt == "fp8":
        g = torch.Generator(device=dev).manual_seed(cfg.seed)
        ye = configs.quantise_fp8_rows(torch.randn(state.permuted.shape[0], cfg.hidden, generator=g, device=dev),
                                       cfg.row_pitch)
    else:
        ye = state.permuted.clone()
    torch.cuda.synchronize()

    def step():
        e_, g_, _ = route()
        s_ = loopback_dispatch(x, e_, g_, *geom)
        return loopback_combine(ye, s_, out_dtype=cfg.out_dtype, fp8_hidden=fp8_hidden)

    def step_onepass():
        e_, g_, _ = route()
        s_ = loopback_dispatch_onepass(x, e_, g_, *geom)
        return loopback_combine(ye, s_, out_dtype=cfg.out_dtype, fp8_hidden=fp8_hidden)

    y_two = step()
    same_y = bool(torch.equal(y_two, step_onepass()))
    del y_two
    ms_per_step = wall_ms(step, args.steps, args.warmup, torch)
    ms_onepass = wall_ms(step_onepass, args.steps, args.warmup, torch)

    kept_pairs = int((state.place >= 0).sum()) if cap is not None else None
    places = None if cap is None else cfg.slots * cap
    phys = configs.minimum_traffic_bytes(cfg, kept_pairs, places)
    conv = configs.algorithmic_bytes(cfg)
    hopb_bytes = configs.onepass_traffic_bytes(cfg, places)
    onepass_bytes = phys["route"] + phys["pack"] + hopb_bytes + phys["combine"]
    reps = max(args.steps, 5)
    quota = cfg.quota

    def arrival():
        return tops.k1_arrival_raw(state.payload, state.mask, state.gate_rows, quota, cfg.epr, cfg.rpn, 0,
                                   want_pair_pos=True)

    def pack():
        return tops.k2_pack_raw(x, e, gates, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups, extras=True)

    def combine():
        return loopback_combine(ye, state, out_dtype=cfg.out_dtype, fp8_hidden=fp8_hidden)

    def hopb():
        return tops.hopb_scatter(state.payload, state.mask, None, quota, cfg.slots, 0, cap)

    gbps = lambda nbytes, ms: nbytes / ms / 1e6
    out = {
        "ms_per_step": ms_per_step,
        "GBps": gbps(sum(phys.values()), ms_per_step),
        "rows_counted_twice_GBps": gbps(sum(conv.values()), ms_per_step),
        "onepass": {"ms_per_step": round(ms_onepass, 4), "GBps": round(gbps(onepass_bytes, ms_onepass), 1),
                    "frac_hbm_peak": round(gbps(onepass_bytes, ms_onepass) / HBM_PEAK_GBPS, 4),
                    "same_output_as_two_step": same_y,
                    "note": "Hop B as one scatter from the arrived rows to their expert-order places "
                            "(terrace_hopb_scatter) instead of arrival chain + regroup; priced on its own bytes"},
        "kept_pairs": kept_pairs, "places": places, "phys": phys, "conv": conv, "hopb_bytes": hopb_bytes,
    }
    def measure_in_step():
        # ---- each stage timed INSIDE the step: events between the stage calls of K whole steps, so that no stage sees
        # inputs a previous launch of itself left in a cache (alone, back to back, the pack re-reads the same 235 MB)
        names = ("route", "pack", "arrival", "regroup", "combine")
        marks = []
        for it in range(reps + 2):
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(6)]
            ev[0].record()
            e_, g_, _ = route()
            ev[1].record()
            (pl_, mk_, gr_, _us, _nc), ex_ = tops.k2_pack_raw(x, e_, g_, cfg.world, cfg.n_experts, cfg.rpn, cfg.top_groups,
                                                              extras=True, combine_table=True)
            ev[2].record()
            tg_ = []
            sb_, _gp, _ri, si_, _is, _pp = tops.k1_arrival_raw(pl_, mk_, gr_, quota, cfg.epr, cfg.rpn, 0, want_pair_pos=True,
                                                               tags=ex_["pair_src"], tags_out=tg_)
            ev[3].record()
            tops.regroup(sb_, si_, cfg.slots, 0, cap, tags=tg_[0], table=ex_["where"])
            ev[4].record()
            tops.combine(ye, ex_["where"], ex_["gate_sorted"], out_dtype=cfg.out_dtype, fp8_hidden=fp8_hidden)
            ev[5].record()
            if it >= 2:
                marks.append(ev)
        torch.cuda.synchronize()
        in_step = {n: statistics.median(m[i].elapsed_time(m[i + 1]) for m in marks) for i, n in enumerate(names)}
        pc_in = in_step["pack"] + in_step["combine"]
        return {"stage_ms": {n: round(v, 4) for n, v in in_step.items()},
                          "stage_frac_hbm_peak": {n: round(gbps(phys[n], v) / HBM_PEAK_GBPS, 4) for n, v in in_step.items()},
                          "pack_plus_combine_ms": round(pc_in, 4),
                          "pack_plus_combine_frac_hbm_peak": round(gbps(phys["pack"] + phys["combine"], pc_in) / HBM_PEAK_GBPS, 4),
                          "note": "median over the timed steps of the time between HIP events recorded around each stage "
                                  "call inside whole steps (stage operators called one by one, same kernels)"}

    out["in_step"] = measure_in_step()
    if not detail:
        ms_arr, ms_pack, ms_comb = event_ms(arrival, reps, torch), event_ms(pack, reps, torch), event_ms(combine, reps, torch)
        out["arrival_us_per_row"] = ms_arr * 1e3 / cfg.pairs
        out["pack_plus_combine_frac_hbm_peak"] = gbps(phys["pack"] + phys["combine"], ms_pack + ms_comb) / HBM_PEAK_GBPS
        # a step this short is bound by the host's launches: its HIP-graph replay says what the kernels alone take
        out["graph"] = graph_replay_ms(step, args, torch) if (args.graph or ms_per_step < 0.3) else None
        return out

    # ---- per-stage timings (each stage alone, HIP events on the launch stream) ----
    def regroup():
        return tops.regroup(state.send_buf, state.slot_idx, cfg.slots, 0, cap)

    stage_ms = {"route": event_ms(route, reps, torch), "pack": event_ms(pack, reps, torch),
                "arrival": event_ms(arrival, reps, torch), "regroup": event_ms(regroup, reps, torch),
                "combine": event_ms(combine, reps, torch)}
    ms_hopb = event_ms(hopb, reps, torch)
    # rows a stage writes: send rows, (row, slot) pairs, places of the expert-order buffer, tokens
    rows_out = {"route": cfg.T, "pack": cfg.send_rows, "arrival": cfg.pairs,
                "regroup": cfg.pairs if cap is None else places, "combine": cfg.T}
    stages = {}
    for name, ms in stage_ms.items():
        stages[name] = {"ms": round(ms, 4), "GBps": round(gbps(phys[name], ms), 1),
                        "frac_hbm_peak": round(gbps(phys[name], ms) / HBM_PEAK_GBPS, 4),
                        "rows_counted_twice_GBps": round(gbps(conv[name], ms), 1),
                        "us_per_row": round(ms * 1e3 / max(rows_out[name], 1), 6)}
    stages["arrival"]["reference_target_us_per_row"] = REFERENCE_TARGET_US_PER_ROW
    stages["hopb_onepass"] = {"ms": round(ms_hopb, 4), "GBps": round(gbps(hopb_bytes, ms_hopb), 1),
                              "frac_hbm_peak": round(gbps(hopb_bytes, ms_hopb) / HBM_PEAK_GBPS, 4),
                              "us_per_row": round(ms_hopb * 1e3 / cfg.pairs, 6),
                              "replaces": "arrival + regroup",
                              "two_step_ms": round(stage_ms["arrival"] + stage_ms["regroup"], 4)}
    pc_ms = stage_ms["pack"] + stage_ms["combine"]
    out["stages"] = stages
    out["pack_plus_combine"] = {
        "ms": round(pc_ms, 4), "GBps": round(gbps(phys["pack"] + phys["combine"], pc_ms), 1),
        "frac_hbm_peak": round(gbps(phys["pack"] + phys["combine"], pc_ms) / HBM_PEAK_GBPS, 4),
        "rows_counted_twice_GBps": round(gbps(conv["pack"] + conv["combine"], pc_ms), 1), "target_frac_hbm_peak": 0.70}

    # ---- the row-moving kernels alone ----
    row = cfg.row_bytes
    where, w_sorted = state.extras["where"], state.extras["gate_sorted"]
    token_rows, pair_pos2 = state.extras["token_rows"], state.pair_pos.view(cfg.send_rows, quota)
    if cap is None:
        _, order, _ = tops.regroup(state.send_buf, state.slot_idx, cfg.slots, 0, None)
        gather_idx = order
    else:
        gather_idx = torch.full((places,), -1, dtype=torch.int64, device=dev)
        ok = state.place >= 0
        gather_idx[state.place[ok]] = torch.arange(cfg.pairs, device=dev)[ok]
    place_of_pair = state.place[state.pair_pos].view(cfg.send_rows, quota).contiguous()
    n_places = cfg.pairs if cap is None else places
    kept = cfg.pairs if kept_pairs is None else kept_pairs
    out_row = cfg.hidden * (4 if cfg.fmt == "f32" else 2)
    # names of the kernels the library picks for this row width (whole kilobytes or not)
    kb_rows = row % 1024 == 0 or cfg.row_pitch is not None
    def k_scatter(fan):     # two copies have a kernel of their own
        return ("scatter_rows_sliced_fan2_kernel" if fan == 2 else "scatter_rows_sliced_kernel") if kb_rows \
            else "scatter_rows_aligned_kernel"
    k_gather = "gather_rows_sliced_kernel" if kb_rows else "gather_rows_flat_kernel"
    flat = torch.empty(cfg.pairs * row, dtype=torch.uint8, device=dev)      # as many bytes as the arrival buffer holds
    kernels = {     # name: (launch, bytes that must cross HBM per launch)
        f"{k_scatter(cfg.top_groups)}(pack)": (lambda: tops.scatter_rows(x, token_rows, cfg.send_rows), (cfg.T + cfg.send_rows) * row),
        f"{k_scatter(quota)}(arrival)": (lambda: tops.scatter_rows(state.payload, pair_pos2, cfg.pairs),
                                  (cfg.send_rows + cfg.pairs) * row),
        f"{k_scatter(quota)}(hopb_onepass)": (lambda: tops.scatter_rows(state.payload, place_of_pair, n_places),
                                       (cfg.send_rows + kept) * row),
        f"{k_gather}(regroup)": (lambda: tops.gather_rows(state.send_buf, gather_idx), (kept + n_places) * row),
        "combine_kernel": (lambda: tops.combine(ye, where, w_sorted, out_dtype=cfg.out_dtype, fp8_hidden=fp8_hidden),
                           kept * row + cfg.pairs * 12 + cfg.T * out_row),
        "copy_kernel(passthrough)": (lambda: tops.passthrough(flat), 2 * flat.numel()),
    }
    kern = {}
    for name, (fn, nb) in kernels.items():
        ms = event_ms(fn, reps, torch)
        kern[name] = {"ms": round(ms, 4), "bytes_per_launch": nb, "GBps": round(nb / ms / 1e6, 1),
                      "frac_hbm_peak": round(nb / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    if detail and not args.no_in_order:
        # The same launches over the same tables with their live entries renumbered in order of appearance (entry i of
        # the table names row i; dead entries stay where they are): every read and every write becomes one
        # contiguous stream.  Same kernels, same bytes: what remains of a mover's distance to the stream rates here
        # is the kernel's own, the rest is what the placement of the rows costs.
        def in_order(t):
            live = (t >= 0).reshape(-1)
            r = torch.cumsum(live.to(torch.int64), 0) - 1
            return torch.where(live, r, torch.full_like(r, -1)).view_as(t).contiguous()
        ordered = {
            f"{k_scatter(cfg.top_groups)}(pack)": lambda t=in_order(token_rows): tops.scatter_rows(x, t, cfg.send_rows),
            f"{k_scatter(quota)}(arrival)": lambda t=in_order(pair_pos2): tops.scatter_rows(state.payload, t, cfg.pairs),
            f"{k_scatter(quota)}(hopb_onepass)": lambda t=in_order(place_of_pair): tops.scatter_rows(state.payload, t, n_places),
            f"{k_gather}(regroup)": lambda t=in_order(gather_idx): tops.gather_rows(state.send_buf, t),
            "combine_kernel": lambda t=in_order(where): tops.combine(
                ye, t, w_sorted, out_dtype=cfg.out_dtype, fp8_hidden=fp8_hidden),
        }
        for name, fn in ordered.items():
            kern[name]["ms_rows_in_order"] = round(event_ms(fn, reps, torch), 4)
    out["kernels"] = kern
    out["graph"] = graph_replay_ms(step, args, torch) if args.graph else None
    out["raw_dispatch_plus_combine_ms"] = sum(v for n, v in out["in_step"]["stage_ms"].items() if n != "route")
    out["tensors"] = (e, gates, x)
    return out


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU's share of the path; the all-to-all exchanges "
              "between ranks are not part of it, so --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    import torch

    import terrace.ops as tops
    from terrace import _hip, configs

    if not torch.cuda.is_available():
        print("bench.py: no ROCm device", file=sys.stderr)
        sys.exit(3)
    st = tops.status()
    if not st.loaded:
        print(f"bench.py: kernel library not loaded: {st.reason}", file=sys.stderr)
        sys.exit(3)
    digest = _hip.load().terrace_version().decode().rsplit("src:", 1)[-1]
    cfg = configs.CONFIGS[args.config]
    if args.row_pitch is not None:
        import dataclasses
        cfg = dataclasses.replace(cfg, row_pitch=args.row_pitch or None)
    if args.tokens is not None:
        import dataclasses
        if args.tokens < 1:
            print("bench.py: --tokens must be positive", file=sys.stderr)
            sys.exit(2)
        cfg = dataclasses.replace(cfg, T=args.tokens, name=f"{cfg.name}_T{args.tokens}")
    torch.cuda.set_device(0)

    r = run_workload(cfg, args, torch, detail=True)
    kern, stages = r["kernels"], r["stages"]
    seam = None
    if not args.no_seam and cfg.fmt != "fp8":          # the seam's probs plane has the payload's float dtype
        seam = seam_block(cfg, args, torch, r["raw_dispatch_plus_combine_ms"], *r["tensors"])
    del r["tensors"]
    torch.cuda.empty_cache()
    ceilings = stream_ceilings(torch, max(args.steps, 5))
    torch.cuda.empty_cache()
    # every mover beside what its bytes cost at this run's own read-only and write-only stream rates
    row, S, P, T = cfg.row_bytes, cfg.send_rows, cfg.pairs, cfg.T
    kept = P if r["kept_pairs"] is None else r["kept_pairs"]
    n_places = P if r["places"] is None else r["places"]
    out_row = cfg.hidden * (4 if cfg.fmt == "f32" else 2)
    rw = {"(pack)": (T * row, S * row), "(arrival)": (S * row, P * row), "(hopb_onepass)": (S * row, kept * row),
          "(regroup)": (kept * row, n_places * row), "combine_kernel": (kept * row + P * 12, T * out_row)}
    for name, v in kern.items():
        for tag, (rd, wr) in rw.items():
            if name.endswith(tag):
                floor = predicted_floor_ms(ceilings, rd, wr)
                v["floor_ms_at_stream_rates"] = round(floor, 4)
                v["ms_over_floor"] = round(v["ms"] / floor, 3)
                if "ms_rows_in_order" in v:
                    v["rows_in_order_over_floor"] = round(v["ms_rows_in_order"] / floor, 3)
    dominant = max((k for k in kern if not k.startswith("copy") and "onepass" not in k), key=lambda k: kern[k]["ms"])
    # algorithmic bytes of the dominant kernel per launch: every row it moves, read once and written once
    roofline = {"bound": "hbm", "kernel": dominant, "achieved": kern[dominant]["GBps"], "peak": HBM_PEAK_GBPS,
                "unit": "GB/s", "frac": kern[dominant]["frac_hbm_peak"],
                "traffic": None if args.tokens is not None else measured_traffic(args.config, dominant, digest),
                "traffic_source": "profiles/traffic.json (null when measured on other sources than the loaded library's)",
                "avg_launch_ms": kern[dominant]["ms"], "algorithmic_bytes_per_launch": kern[dominant]["bytes_per_launch"]}

    cap = cfg.capacity(cfg.slots)
    value = r["GBps"]
    out = {
        "metric": "dispatch_combine_GBps_on_bytes_that_cross_HBM",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(r["ms_per_step"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"f32": "f32", "bf16": "bf16", "fp8": "fp8_e4m3+f32 scales"}[cfg.fmt] + " rows, fp32 accumulate",
        "data": "synthetic",
        "config": {"workload": cfg.name, "T": cfg.T, "E": cfg.n_experts, "n_groups": cfg.n_groups, "k": cfg.top_k,
                   "M": cfg.top_groups, "cards_per_group": cfg.rpn, "hidden": cfg.hidden, "row_bytes": cfg.row_bytes,
                   "row_pitch": cfg.row_pitch, "send_rows": cfg.send_rows, "pairs": cfg.pairs, "capacity": cap,
                   "exchange": "loop-back (no all-to-all on one GPU)",
                   "expert_outputs": "fixed synthetic tensor prepared before the timed region"},
        "frac_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "bytes_per_step": sum(r["phys"].values()),
        "rows_counted_twice_GBps": round(r["rows_counted_twice_GBps"], 1),
        "pricing": "value, every GBps and every frac_hbm_peak: bytes that must cross HBM (a scatter reads each source "
                   "row once however many copies it writes; a capacity layout reads only the rows it keeps). "
                   "rows_counted_twice_GBps: a payload row counted once on the read and once on the write side of "
                   "every stage (can exceed the peak for a scatter; never used for a fraction)",
        "pack_plus_combine": r["pack_plus_combine"],
        "arrival_chain_us_per_row": stages["arrival"]["us_per_row"],
        "onepass": r["onepass"],
        "stages": stages, "in_step": r["in_step"], "kernels": kern, "ceilings": ceilings, "seam": seam,
        "roofline": roofline,
        "stage_and_kernel_timing": f"each alone on the launch stream between HIP events: median of {EVENT_BATCHES} "
                                   f"batches of {max(args.steps, 5)} back-to-back launches",
        "library": os.path.relpath(st.lib, ROOT), "source_digest": digest,
    }
    if r["graph"] is not None:
        out["hip_graph"] = r["graph"]
    del r
    torch.cuda.empty_cache()
    if not args.no_other_configs:
        others = {}
        for name, c in configs.CONFIGS.items():
            if name == args.config:
                continue
            o = run_workload(c, args, torch, detail=False)
            others[name] = {"workload": c.name, "ms_per_step": round(o["ms_per_step"], 4), "GBps": round(o["GBps"], 1),
                            "frac_hbm_peak": round(o["GBps"] / HBM_PEAK_GBPS, 4),
                            "arrival_us_per_row": round(o["arrival_us_per_row"], 6),
                            "pack_plus_combine_frac_hbm_peak": round(o["pack_plus_combine_frac_hbm_peak"], 4),
                            "pack_plus_combine_in_step_frac_hbm_peak": o["in_step"]["pack_plus_combine_frac_hbm_peak"],
                            "onepass_ms_per_step": o["onepass"]["ms_per_step"],
                            "onepass_frac_hbm_peak": o["onepass"]["frac_hbm_peak"],
                            "onepass_same_output": o["onepass"]["same_output_as_two_step"]}
            if o.get("graph") is not None:
                others[name]["hip_graph"] = o["graph"]
            del o
            torch.cuda.empty_cache()
        out["other_configs"] = others
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, args.cpu_sample_tokens)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
