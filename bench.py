#!/usr/bin/env python3
"""Benchmark of the MoE dispatch -> expert stub -> combine path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload dsv3_rank]

A step is one pass of the path over one resident batch, in the configuration `custom_kernel`
runs: routing + dispatch in one launch, then the combine with the expert stand-in folded in (two
launches at the default workload), replayed from a hipGraph.  Inputs are in HBM before the timed
region starts.  Prints ONE JSON line:

  value        achieved GB/s of dispatch+combine: algorithmic bytes (read x once, write R
               rows; read R rows, write T rows) / summed GPU durations of the routing,
               dispatch and combine kernels of a step.  Kernel durations come from HIP
               events bound to each launch, on the stream the kernels run on.
  ms_per_step  wall time of a whole step: events around K steps launched back to back from a C loop
               behind an already filled queue (graph_ms_per_step: the same K steps as hipGraph replays,
               which pay about 9 us per graph launch on top).
  roofline     the slower of the dispatch / combine kernels against the 8 TB/s HBM peak; `traffic`
               from profiles/traffic.json when that record was taken on the present kernel sources.
  cpu_baseline the CPU oracle (a port of the reference's torch path) timed on the host
               cores for the same workload, and used to check the GPU result.
Beside the headline: the same path with the stub as a launch of its own, and with the
f32-accumulating combine.  `--graph-only` runs the graph replays and nothing else (for rocprofv3).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
GRAPH_STEPS = 40  # steps captured into one hipGraph

# HBM bytes per launch, measured: profiles/traffic.json holds rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# readings (KiB per dispatch, each scaled by what the same counter reads for a plain 256 MiB device
# copy) together with the kernel's name and a hash of the kernel sources they were taken from.
# `python bench.py --record-traffic DIR` writes that file from the CSVs of such runs.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")
KERNEL_SOURCES = ("kernel_amd/csrc/moe_a2a.hip", "kernel_amd/csrc/route_kernels.inc", "kernel_amd/csrc/row_kernels.inc")


def kernel_source_hash():
    """sha256 over the sources of the dispatch / combine kernels: a traffic record counts only for
    the code it was measured on."""
    import hashlib

    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload, kernel, path=TRAFFIC_FILE, source_hash=None):
    """(bytes per launch or None, where the figure comes from / why there is none)."""
    try:
        with open(path) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None, "no traffic record (profiles/traffic.json missing or unreadable)"
    source_hash = source_hash or kernel_source_hash()
    for e in rec.get("entries", []):
        if e.get("workload") == workload and e.get("kernel") == kernel:
            if e.get("source_hash") != source_hash:
                return None, (f"record of {kernel} at {workload} was measured on other kernel sources "
                              f"({e.get('source_hash')}, now {source_hash}): not reported")
            return int(e["bytes"]), (f"profiles/traffic.json: rocprofv3 --pmc, {e['fetch_kib']} KiB FETCH_SIZE x "
                                     f"{rec['factor']['FETCH_SIZE']} + {e['write_kib']} KiB WRITE_SIZE x "
                                     f"{rec['factor']['WRITE_SIZE']}, kernel {e.get('symbol', kernel)}, "
                                     f"sources {e['source_hash']}, commit {e.get('commit', '?')}")
    return None, f"no record of {kernel} at {workload}"


METRIC = "dispatch+combine µs and achieved HBM GB/s (% of peak), 256E/top8/h7168 bf16"


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--workload", default="dsv3_rank")
    p.add_argument("--combine", choices=["strict", "f32"], default=None,
                   help="default: what the workload's configuration names -- f32 accumulation for fp8_dispatch, the "
                        "reference's rounding after every step (bit-identical) for the others")
    p.add_argument("--no-graph", action="store_true", help="launch eagerly from Python instead of a hipGraph")
    p.add_argument("--no-fuse-route", action="store_true", help="separate routing kernel even for small worlds")
    p.add_argument("--no-fuse-stub", action="store_true",
                   help="expert stub as a launch of its own (the default folds it into the combine, as custom_kernel does)")
    p.add_argument("--graph-only", action="store_true",
                   help="wall-clock legs of the default configuration only (hipGraph replays, then plain launches from "
                        "the C loop): no launch carries events -- the form to run under rocprofv3")
    p.add_argument("--single", action="store_true", help="skip the legs reported beside the headline (other stub form, f32 combine)")
    p.add_argument("--timer-event-flags", default="", metavar="FLAGS",
                   help="hipEventCreateWithFlags value for the launch timer's events (measurement aid)")
    p.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                   help="library option switch (moe_a2a_set_option), e.g. COMBINE_LANES=128 (measurement aid)")
    p.add_argument("--record-traffic", metavar="DIR",
                   help="no measurement: fold rocprofv3 --pmc CSVs under DIR into profiles/traffic.json")
    p.add_argument("--bf16-dispatch", action="store_true", help="fp8 workload with a 16-bit dispatch")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    p.add_argument("--cold", action="store_true",
                   help="kept for older command lines: the cold-cache leg is part of every full run now")
    p.add_argument("--no-workloads", action="store_true",
                   help="skip the other named workloads and the expert-layer leg reported beside the headline")
    p.add_argument("--cpu-seconds", type=float, default=12.0)
    p.add_argument("--fp8-weights", action="store_true",
                   help="with --expert-gemm: weights as e4m3fn bytes with one f32 scale per 128 x 128 block")
    p.add_argument("--fp8-rows", action="store_true", help="with --expert-gemm: fp8 dispatch on a 16-bit workload")
    p.add_argument("--pow2-scales", action="store_true",
                   help="with --expert-gemm --fp8-weights on an fp8 workload: power-of-two scales for rows and weights, "
                        "multiplied with the scales as the matrix instruction's block exponents")
    p.add_argument("--gemm-rs", default="", metavar="M,N,K[,bias]",
                   help="measure the GEMM + reduce-scatter of the reference's other problem instead (8 emulated ranks "
                        "as K shards of one buffer), e.g. 8192,8192,29568 or 512,4096,12288,bias; `all` runs the six "
                        "benchmark shapes of gemm_rs/task.yml, one JSON line each")
    p.add_argument("--equal-segments", action="store_true",
                   help="with --expert-gemm: a routing table that gives every expert the same number of rows "
                        "(entry i goes to expert i %% E) instead of the workload's")
    p.add_argument("--expert-gemm", type=int, default=0, metavar="N",
                   help="measure the grouped expert GEMM (N output columns per expert) on the workload's "
                        "dispatched rows instead of the dispatch/combine path")
    p.add_argument("--dump-times", metavar="FILE", help="write every timed launch's duration (us, in launch order) as JSON")
    p.add_argument("--calibrate-copy", action="store_true",
                   help="end with three plain 256 MiB device copies (a known-size reference for rocprof counters)")
    return p.parse_args()


def kernel_times(lib, run_n, steps, torch, before_each=None, lead=0, launches_per_step=0, wall=None):
    """Per-kernel GPU durations (µs) of `steps` passes launched back to back from C, from the
    library's launch timer (HIP events bound to each launch).  `lead` passes go first in the same
    loop WITHOUT events: a launch that carries events costs the host about 13 µs, a plain one
    2.5 µs, a small kernel runs 7 µs -- the plain passes put the host ahead, so that the timed ones
    find the queue full and run back to back as in a hipGraph replay.  `wall = (stream, list)`
    appends the wall clock per step of the timed passes themselves (an upper bound for the sum of
    their kernels)."""
    cap = steps * 8
    rc = lib.moe_a2a_timer_begin(cap)
    if rc != 0:
        raise RuntimeError(f"moe_a2a_timer_begin: {lib.moe_a2a_strerror(rc).decode()}")
    if before_each is None:
        if lead:
            lib.moe_a2a_timer_skip(lead * launches_per_step)
            run_n(lead)
        if wall is not None:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(wall[0])
        run_n(steps)
        if wall is not None:
            e1.record(wall[0])
            torch.cuda.synchronize()
            wall[1].append(e0.elapsed_time(e1) * 1e3 / steps)
    else:
        for _ in range(steps):
            before_each()
            run_n(1)
    torch.cuda.synchronize()
    ids = (ctypes.c_int * cap)()
    us = (ctypes.c_float * cap)()
    n = lib.moe_a2a_timer_end(ids, us, cap)
    per = {}
    for i in range(n):
        per.setdefault(lib.moe_a2a_kernel_name(ids[i]).decode(), []).append(float(us[i]))
    return per


def lead_passes(lib, run_n, steps, gpu_step_us, torch, floor):
    """How many plain passes must go first so that the queue outlasts `steps` timed passes: measures
    what a plain and a timed pass cost the host (µs) and how many launches a pass holds."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run_n(20)
    plain = (time.perf_counter() - t0) / 20 * 1e6
    torch.cuda.synchronize()
    lib.moe_a2a_timer_begin(20 * 8)
    t0 = time.perf_counter()
    run_n(20)
    timed = (time.perf_counter() - t0) / 20 * 1e6
    torch.cuda.synchronize()
    ids, us = (ctypes.c_int * 160)(), (ctypes.c_float * 160)()
    launches = lib.moe_a2a_timer_end(ids, us, 160) // 20
    deficit = max(0.0, timed - gpu_step_us) * steps
    gain = max(gpu_step_us - plain, 0.1 * gpu_step_us)
    lead = int(1.3 * deficit / gain) + 1
    return max(floor, min(lead, 2000)), launches, plain, timed


def c_loop(step):
    """run(n): n back-to-back steps launched from C with the planned step's own arguments."""
    from kernel_amd import build as _build

    loop = ctypes.CDLL(_build.BENCH_LIB_PATH)
    loop.moe_a2a_bench_steps.restype = ctypes.c_int
    from kernel_amd._lib import ForwardArgs

    loop.moe_a2a_bench_steps.argtypes = [ctypes.c_int, ctypes.POINTER(ForwardArgs), ctypes.POINTER(ForwardArgs)]
    sets = [ForwardArgs(*a) for a in step.args]

    def run(n):
        rc = loop.moe_a2a_bench_steps(n, ctypes.byref(sets[0]), ctypes.byref(sets[1]))
        if rc:
            raise RuntimeError(f"moe_a2a_forward failed with code {rc}")

    return run


def summarise(per):
    return {k: dict(mean_us=round(statistics.fmean(v), 3), std_us=round(statistics.pstdev(v), 3),
                    err_us=round(statistics.pstdev(v) / max(1, len(v)) ** 0.5, 4), min_us=round(min(v), 3),
                    max_us=round(max(v), 3), median_us=round(statistics.median(v), 3), launches=len(v))
            for k, v in per.items()}


ROUTE_KERNELS = ("route_tiles", "route_hist", "route_scan", "route_rank")
DISPATCH_KERNELS = ("dispatch_rows", "route_dispatch", "route_dispatch_tile", "dispatch_fp8", "route_dispatch_fp8")
COMBINE_KERNELS = ("combine_rows", "stub_combine")
FORWARD_KERNELS = ("forward_token", "forward_tile", "dispatch_fold")  # dispatch and combine of a token in one launch
STUB_KERNELS = ("stub_rows", "stub_fp8")


def per_step(per, names, steps):
    return sum(sum(per.get(n, [])) for n in names) / steps


class Leg:
    """One configuration of the path (host object, planned step, hipGraphs) and its measurements."""

    def __init__(self, torch, lib, wl, tensors, main, mode, fp8, fuse_route, fuse_stub):
        from kernel_amd.all2all import HipAllToAll

        self.torch, self.lib, self.main = torch, lib, main
        x, idx, w, rs = tensors
        self.ata = HipAllToAll(wl.cfg, 0, wl.world_size, stub_kind=wl.stub_kind, combine_mode=mode, fp8_dispatch=fp8,
                               fuse_route=fuse_route, fuse_stub=fuse_stub)
        with torch.cuda.stream(main):
            self.step = self.ata.plan(x, idx, w, rs, stream=main)  # pre-marshalled: one foreign call per step
            self.step()
            self.y = self.step()  # both buffer sets exist now
            main.synchronize()
        self.run_n = None

    def graph_wall(self, steps, warmup, use_graph=True):
        """Wall time per step (ms) of exactly `steps` steps replayed from hipGraphs of up to
        GRAPH_STEPS steps each (an even number: the host class alternates between two buffer sets; what
        is left over ends in a shorter graph).  Inside a graph the launches follow each other with
        nothing but the GPU's own launch overhead between them, and a graph launch (a few us of
        host-visible latency) is spread over its steps, so for a configuration whose steps are all
        dispatch/combine kernels this IS the mean launch-to-launch period of those kernels -- the
        duration a profiler's kernel trace reports for back-to-back launches."""
        torch, main, step = self.torch, self.main, self.step

        def capture(n):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=main):
                for _ in range(n):
                    self.y = step()
            return g

        with torch.cuda.stream(main):
            if use_graph:
                chunk = min(GRAPH_STEPS, steps - steps % 2) or 1
                full, rem = capture(chunk), steps % chunk
                tail = capture(rem) if rem else None
                n_full = steps // chunk
                run = full.replay
            else:
                chunk, tail, n_full, run = 1, None, steps, step
            # spin-up: the first milliseconds of GPU work after an idle period run below the
            # sustained clocks; 0.3 s of untimed steps come before the W warm-up steps
            t_spin = time.perf_counter()
            while time.perf_counter() - t_spin < 0.3:
                for _ in range(max(1, 100 // chunk)):
                    run()
                main.synchronize()
            for _ in range(max(1, warmup // chunk)):
                run()
            main.synchronize()
            # two more untimed replays go out right in front of the timed region: the GPU works on
            # them while the host enqueues the start event and the timed launches (submitting a graph
            # of 40 launches takes the host longer than a step takes the GPU), so the K timed steps
            # start back to back instead of behind an idle queue
            for _ in range(2):
                run()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(main)
            for _ in range(n_full):
                run()
            if tail is not None:
                tail.replay()
            e1.record(main)
            main.synchronize()
        return e0.elapsed_time(e1) / steps

    def loop_wall(self, steps, warmup):
        """Wall time per step (ms) of exactly `steps` steps launched one by one from a C loop (plain
        launches, no graph): the host issues a launch in a fraction of the time a step takes the GPU,
        so with a few steps already queued the timed ones run back to back, and there is no graph
        boundary (about 9 us per hipGraphLaunch here) inside the timed region."""
        torch, main = self.torch, self.main
        with torch.cuda.stream(main):
            if self.run_n is None:
                self.run_n = c_loop(self.step)
                self.run_n(4)
                main.synchronize()
            t_spin = time.perf_counter()
            while time.perf_counter() - t_spin < 0.3:  # sustained clocks, as in graph_wall
                self.run_n(100)
                main.synchronize()
            self.run_n(max(1, warmup))
            main.synchronize()
            self.run_n(16)  # the queue the timed steps start behind
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(main)
            self.run_n(steps)
            e1.record(main)
            main.synchronize()
        return e0.elapsed_time(e1) / steps

    def kernels(self, steps, warmup, gpu_step_us, want_wall=False):
        """Per-kernel durations (us) of `steps` steps launched back to back from C, every launch with
        its own pair of HIP events; returns (per-kernel lists, details)."""
        torch, lib, main = self.torch, self.lib, self.main
        with torch.cuda.stream(main):
            if self.run_n is None:
                self.run_n = c_loop(self.step)
                self.run_n(4)
                main.synchronize()
            run_n = self.run_n
            lead, n_launch, host_plain_us, host_timed_us = lead_passes(lib, run_n, steps, gpu_step_us, torch, warmup)
            # the first pass only populates the runtime's pool of events and completion signals
            # (creating them costs driver calls that land in the middle of the launch sequence)
            kernel_times(lib, run_n, steps, torch, lead=lead, launches_per_step=n_launch)
            pass_wall = []
            per = kernel_times(lib, run_n, steps, torch, lead=lead, launches_per_step=n_launch,
                               wall=(main, pass_wall) if want_wall else None)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(main)
            run_n(steps)
            e1.record(main)
            main.synchronize()
        details = dict(plain_lead_passes=lead, host_us_per_plain_pass=round(host_plain_us, 2),
                       host_us_per_timed_pass=round(host_timed_us, 2), launches_per_step=n_launch,
                       eager_ms_per_step=e0.elapsed_time(e1) / steps)
        if want_wall:
            details["wall_us_per_step"] = round(pass_wall[0], 3)
        return per, details


def spin_up(main, fn, seconds=0.3):
    """Untimed calls of fn for `seconds`: the first milliseconds of GPU work after an idle period run
    below the sustained clocks (memory-bound kernels as well), and a leg that starts measuring right
    after its set-up measures those."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(4):
            fn()
        main.synchronize()


def phase_times(per, steps, wall_us):
    """Per-step times of the phases.  `*_kernel` figures are the kernels' own durations (HIP events
    bound to each launch).  The figures without the suffix add to every launch its share of the
    launch overhead, (wall clock of a step in the hipGraph - sum of the kernel durations) / launches:
    the launch-to-launch PERIOD, which is what a profiler's kernel trace reports as the duration of
    back-to-back launches (it stamps a kernel's start when the one before it ends) and what a caller
    pays.  `dc` = routing + dispatch + combine; when those are all the launches of a step it equals
    the wall clock of the step."""
    names = dict(route=ROUTE_KERNELS, dispatch=DISPATCH_KERNELS, combine=COMBINE_KERNELS, stub=STUB_KERNELS,
                 forward=FORWARD_KERNELS)
    t = {}
    launches = {k: sum(len(per.get(n, [])) for n in v) / steps for k, v in names.items()}
    kernel = {k: per_step(per, v, steps) for k, v in names.items()}
    n_all = sum(launches.values())
    gap = max(0.0, wall_us - sum(kernel.values())) / n_all if n_all else 0.0
    for k in names:
        t[k + "_kernel"] = kernel[k]
        t[k] = kernel[k] + gap * launches[k]
    t["gap"] = gap
    t["dc"] = t["route"] + t["dispatch"] + t["combine"] + t["forward"]
    t["dc_kernel"] = kernel["route"] + kernel["dispatch"] + kernel["combine"] + kernel["forward"]
    return t


def main():
    args = parse_args()
    if args.record_traffic:
        return record_traffic(args.record_traffic)
    if args.gpus != 1:
        print(f"bench.py measures one GPU: the emulated destination ranks are partitions of one HBM buffer and "
              f"there is no cross-GPU path in this build (got --gpus {args.gpus}).", file=sys.stderr)
        sys.exit(2)
    if args.steps < 1:
        raise SystemExit("--steps must be at least 1")
    import torch

    from kernel_amd import _lib, contract
    from kernel_amd.all2all import concat_world

    lib = _lib.load()
    if not torch.cuda.is_available():
        raise RuntimeError("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.timer_event_flags:
        lib.moe_a2a_set_option(_lib.OPT_TIMER_EVENT_FLAGS, int(args.timer_event_flags, 0))
    for item in args.option:
        name, _, val = item.partition("=")
        if lib.moe_a2a_set_option(getattr(_lib, "OPT_" + name), int(val, 0)) < 0:
            raise SystemExit(f"unknown option {name}")

    if args.gemm_rs:
        return gemm_rs_leg(args, lib, torch, dev)
    wl = contract.generate_workload(args.workload)
    cfg, W = wl.cfg, wl.world_size
    T, K, H, E = wl.total_tokens, cfg.experts_per_token, cfg.hidden_dim, cfg.num_experts
    fp8 = wl.fp8_dispatch and not args.bf16_dispatch
    if args.combine is None:
        args.combine = "f32" if fp8 else "strict"
    mode = contract.COMBINE_STRICT if args.combine == "strict" else contract.COMBINE_F32
    fuse_route, fuse_stub = not args.no_fuse_route, not args.no_fuse_stub
    tensors = concat_world(wl.world, dev)
    if args.expert_gemm:
        return expert_gemm_leg(args, lib, torch, wl, tensors[0], tensors[1], tensors[3], dev)

    # Everything runs on one non-blocking stream of its own: launches on the legacy default
    # stream carry implicit waits on every other stream of the process.
    main = torch.cuda.Stream()
    main.wait_stream(torch.cuda.current_stream())
    # with the stub folded in, the combine reads the dispatched rows themselves (fp8 bytes and scales
    # after an fp8 dispatch, not 16-bit expert rows)
    ab = contract.algorithmic_bytes(T, K, H, 2, 2, fp8, stub_folded=fuse_stub)
    b_dc = ab["dispatch"] + ab["combine"]
    use_graph = not args.no_graph
    dtype = "fp8-e4m3 dispatch, bf16 combine" if fp8 else {"bfloat16": "bf16", "float16": "f16"}[
        str(cfg.in_dtype).replace("torch.", "")]
    config = dict(workload=args.workload, tokens=T, experts=E, top_k=K, hidden=H, emulated_ranks=W, routed_rows=T * K,
                  combine=args.combine,
                  launch="plain launches, back to back from a C loop (ms_per_step); hipGraph replays of up to "
                         f"{GRAPH_STEPS} steps per graph beside it (graph_ms_per_step)",
                  fused_route=bool(fuse_route and not fp8 and lib.moe_a2a_fused_ok(T, K, H)),
                  fused_stub=bool(fuse_stub),
                  launches_per_step=int(lib.moe_a2a_forward_launches(
                      T, K, H, 0, _lib.BF16, _lib.BF16, 2 if fp8 == "pow2" else int(bool(fp8)), int(fuse_route),
                      int(fuse_stub))),
                  entry_point="what custom_kernel runs (moe_a2a_forward with the expert stub folded in)" if fuse_stub
                  else "routing+dispatch, stub kernel, combine")

    # the configuration custom_kernel runs (kernel_amd/submission.py): the expert stand-in folded
    # in: one launch per step at the default workload
    leg = Leg(torch, lib, wl, tensors, main, mode, fp8, fuse_route, fuse_stub)
    graph_ms_per_step = leg.graph_wall(args.steps, args.warmup, use_graph)
    # the headline wall clock: the same K steps as plain launches from a C loop (no graph boundary in
    # the timed region; measured 13.67 against 13.96 us per step at K = 20, 13.53 / 13.65 at K = 200)
    ms_per_step = leg.loop_wall(args.steps, args.warmup)

    if args.graph_only:
        # Nothing but the two wall-clock measurements above: no event-carrying launch, no second
        # configuration.  This is the form to put under `rocprofv3 --kernel-trace --stats`, whose
        # per-kernel averages then describe exactly these launches.  `value` is the wall-clock figure,
        # which includes the launch overhead between kernels: a lower bound of the kernels' own rate.
        wall_us = ms_per_step * 1e3
        out = dict(metric=METRIC, value=round(b_dc / wall_us / 1e3, 1), unit="GB/s", n_gpus=1, steps=args.steps,
                   warmup=args.warmup, ms_per_step=round(ms_per_step, 6), graph_ms_per_step=round(graph_ms_per_step, 6),
                   higher_is_better=True, scaling="weak", vs_baseline=None, dtype=dtype, data="synthetic",
                   config=dict(config, launch="hipGraph replays, then the same steps as plain launches from a C loop; "
                                              "no launch carries events; value from the wall clock of whole steps"),
                   bytes=dict(dispatch=ab["dispatch"], combine=ab["combine"], stub=ab["stub"]),
                   roofline=None, cpu_baseline=None)
        if args.calibrate_copy:
            calibrate_copy(torch, main, dev)
        print(json.dumps(out, ensure_ascii=False), flush=True)
        return

    per, det = leg.kernels(args.steps, args.warmup, ms_per_step * 1e3, want_wall=True)
    if args.dump_times:
        with open(args.dump_times, "w") as f:
            json.dump({**per, "_wall_us_per_step_of_the_timed_passes": [det["wall_us_per_step"]]}, f)
    wall_us = ms_per_step * 1e3
    t = phase_times(per, args.steps, wall_us)
    value = b_dc / t["dc"] / 1e3  # bytes/us -> GB/s

    # dominant kernel for the roofline entry
    if any(n in per for n in FORWARD_KERNELS):  # one launch moves the bytes of both phases
        cand = [(next(n for n in FORWARD_KERNELS if n in per), b_dc)]
    else:
        disp_name = next(n for n in DISPATCH_KERNELS if n in per)
        comb_name = next(n for n in COMBINE_KERNELS if n in per)
        cand = [(disp_name, ab["dispatch"]), (comb_name, ab["combine"])]
    dom_name, dom_bytes = max(cand, key=lambda c: statistics.fmean(per[c[0]]))
    dom_kernel_us = statistics.fmean(per[dom_name])
    dom_us = dom_kernel_us + t["gap"]
    traffic, traffic_source = measured_traffic(args.workload, dom_name)
    roofline = dict(bound="hbm", kernel=dom_name, achieved=round(dom_bytes / dom_us / 1e3, 1), peak=HBM_PEAK_GBPS,
                    unit="GB/s", frac=round(dom_bytes / dom_us / 1e3 / HBM_PEAK_GBPS, 4),
                    bytes_per_launch=dom_bytes, avg_us=round(dom_us, 3),
                    avg_us_is="launch-to-launch period of back-to-back launches: the kernel's own duration from its HIP "
                              "events plus its share of the launch overhead (what a profiler's kernel trace "
                              "reports for back-to-back launches)",
                    kernel_only_us=round(dom_kernel_us, 3), traffic=traffic, traffic_source=traffic_source)

    out = dict(
        metric=METRIC, value=round(value, 1), unit="GB/s", n_gpus=1, steps=args.steps, warmup=args.warmup,
        ms_per_step=round(ms_per_step, 6), higher_is_better=True, scaling="weak", vs_baseline=None, dtype=dtype,
        data="synthetic", config=config,
        dispatch_combine_us=round(t["dc"], 3), route_us=round(t["route"], 3), dispatch_us=round(t["dispatch"], 3),
        stub_us=round(t["stub"], 3), combine_us=round(t["combine"], 3), one_launch_us=round(t["forward"], 3),
        launch_overhead_us_per_launch=round(t["gap"], 3),
        pct_of_hbm_peak=round(100.0 * value / HBM_PEAK_GBPS, 2),
        kernel_only=dict(dispatch_combine_us=round(t["dc_kernel"], 3),
                         pct_of_hbm_peak=round(100.0 * b_dc / t["dc_kernel"] / 1e3 / HBM_PEAK_GBPS, 2),
                         what="sum of the kernels' own durations (HIP events), launch overhead left out"),
        tokens_per_s=round(T / (t["dc"] * 1e-6), 1),
        tokens_per_s_wall=round(T / (ms_per_step * 1e-3), 1),
        graph_ms_per_step=round(graph_ms_per_step, 6),
        timed_passes={k: v for k, v in det.items() if k != "eager_ms_per_step"},
        bytes=dict(dispatch=ab["dispatch"], combine=ab["combine"], stub=ab["stub"]),
        kernels=summarise(per),
        roofline=roofline,
    )

    if not args.single:
        # The same path with the expert stand-in as a launch of its own (three launches per step; the
        # stub's time is then outside dispatch+combine) ...
        # Beside the headline: the same path with the expert stand-in as a launch of its own; when the
        # headline ran in one launch, its two-launch form (routing+dispatch, then the combine with the
        # stub folded in); and the f32-accumulating combine (one rounding at the end: within the
        # rtol = atol = 1e-2 bar instead of bit-identical to the reference's per-step rounding).
        legs = [("stub_as_its_own_launch" if fuse_stub else "stub_folded_into_combine", mode, not fuse_stub)]
        if fuse_stub and t["forward"] > 0:
            legs.insert(0, ("two_launches", mode, True))
        if mode == contract.COMBINE_STRICT:
            legs.append(("f32_combine", contract.COMBINE_F32, fuse_stub))
        else:
            legs.append(("strict_combine", contract.COMBINE_STRICT, fuse_stub))
        for name, leg_mode, leg_fuse in legs:
            lib.moe_a2a_set_option(_lib.OPT_TWO_LAUNCHES, 0 if name in ("f32_combine", "strict_combine") else 1)
            other = Leg(torch, lib, wl, tensors, main, leg_mode, fp8, fuse_route, leg_fuse)
            o_ms = other.loop_wall(args.steps, args.warmup)
            o_per, _ = other.kernels(args.steps, args.warmup, o_ms * 1e3)
            ot = phase_times(o_per, args.steps, o_ms * 1e3)
            o_ab = contract.algorithmic_bytes(T, K, H, 2, 2, fp8, stub_folded=leg_fuse)
            o_bytes = o_ab["dispatch"] + o_ab["combine"]
            out[name] = dict(
                dispatch_combine_us=round(ot["dc"], 3), dispatch_us=round(ot["dispatch"] + ot["route"], 3),
                stub_us=round(ot["stub"], 3), combine_us=round(ot["combine"], 3),
                one_launch_us=round(ot["forward"], 3), ms_per_step=round(o_ms, 6),
                bytes=o_bytes, value=round(o_bytes / ot["dc"] / 1e3, 1),
                pct_of_hbm_peak=round(100.0 * o_bytes / ot["dc"] / 1e3 / HBM_PEAK_GBPS, 2),
                kernel_only_dispatch_combine_us=round(ot["dc_kernel"], 3))
            del other
        lib.moe_a2a_set_option(_lib.OPT_TWO_LAUNCHES, 0)

    # a profiler's interception slows the host's launches; wall clocks taken with one attached are
    # not those of the path (its kernel trace is the thing to read then)
    out["profiler_attached"] = any(k.startswith(("ROCPROF", "ROCP_", "ROCTRACER")) for k in os.environ) or \
        "rocprofiler" in os.environ.get("LD_PRELOAD", "")
    # Cold caches, as the reference's benchmark protocol has them (utils.py:169-176 flushes before
    # every timed call; eval.py:349): 1 GiB (4x the 256 MB memory-side cache) is overwritten before
    # every step; at most 30 steps; the kernels' own durations from their events.
    out["cold"] = cold_leg(torch, lib, leg, main, dev, min(args.steps, 30), b_dc)

    if not args.single and not args.no_workloads:
        # every named workload in the same process (the reference ranks by the geometric mean over its
        # benchmark specs, all2all/task.yml:71-79): wall clock per step, dispatch+combine period,
        # roofline fraction of the dominant kernel, and one pass of the CPU oracle as the checker
        this = dict(ms_per_step=round(ms_per_step, 6), dispatch_combine_us=round(t["dc"], 3), value=round(value, 1),
                    pct_of_hbm_peak=round(100.0 * value / HBM_PEAK_GBPS, 2), kernel=dom_name,
                    roofline_frac=roofline["frac"], kernel_avg_us=roofline["avg_us"],
                    launches_per_step=config["launches_per_step"], combine=args.combine, bytes=b_dc,
                    two_launches_pct_of_hbm_peak=out.get("two_launches", {}).get("pct_of_hbm_peak"))
        out["workloads"] = {}
        for name in contract.WORKLOAD_NAMES:
            if name == args.workload:
                out["workloads"][name] = this
            else:
                out["workloads"][name] = workload_leg(torch, lib, contract, name, main, dev, args)
        dcs = [w_["dispatch_combine_us"] for w_ in out["workloads"].values()]
        pcts = [w_["pct_of_hbm_peak"] for w_ in out["workloads"].values()]
        out["workloads_geomean"] = dict(dispatch_combine_us=round(statistics.geometric_mean(dcs), 3),
                                        pct_of_hbm_peak=round(statistics.geometric_mean(pcts), 2),
                                        over=list(out["workloads"]))
        # the path around a real expert: dispatch -> grouped expert GEMM (H -> H) -> combine
        out["moe_layer"] = moe_layer_leg(torch, lib, contract, wl, tensors, main, dev, mode, args)

    if args.calibrate_copy:
        calibrate_copy(torch, main, dev)

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(wl, mode, fp8, leg.y, b_dc, args.cpu_seconds)
    print(json.dumps(out, ensure_ascii=False), flush=True)


def cold_leg(torch, lib, leg, main, dev, n_cold, b_dc):
    flush = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    with torch.cuda.stream(main):
        if leg.run_n is None:
            leg.run_n = c_loop(leg.step)
        flush.fill_(1)
        leg.run_n(2)
        perc = kernel_times(lib, leg.run_n, n_cold, torch, before_each=lambda: flush.fill_(1))
    tc = per_step(perc, ROUTE_KERNELS + DISPATCH_KERNELS + COMBINE_KERNELS + FORWARD_KERNELS, n_cold)
    del flush
    return dict(dispatch_combine_us=round(tc, 3), GBps=round(b_dc / tc / 1e3, 1),
                pct_of_hbm_peak=round(100.0 * b_dc / tc / 1e3 / HBM_PEAK_GBPS, 2), steps=n_cold,
                flush="1 GiB overwritten before every step",
                kernels={k: v["mean_us"] for k, v in summarise(perc).items()})


def workload_leg(torch, lib, contract, name, main, dev, args):
    """One of the named workloads in the configuration `custom_kernel` runs (stub folded in, the
    combine mode its configuration names), measured as the headline is: wall clock of plain launches
    from the C loop, per-kernel events, and the GPU output compared bit for bit with one pass of the
    vectorised CPU oracle."""
    from kernel_amd import _lib
    from kernel_amd.all2all import concat_world
    from oracle import all2all_vec as V  # checker only

    wl = contract.generate_workload(name)
    cfg = wl.cfg
    T, K, H = wl.total_tokens, cfg.experts_per_token, cfg.hidden_dim
    fp8 = wl.fp8_dispatch
    mode = contract.COMBINE_F32 if fp8 else contract.COMBINE_STRICT
    tensors = concat_world(wl.world, dev)
    leg = Leg(torch, lib, wl, tensors, main, mode, fp8, True, True)
    steps = args.steps
    ms = leg.loop_wall(steps, args.warmup)
    per, _ = leg.kernels(steps, args.warmup, ms * 1e3)
    t = phase_times(per, steps, ms * 1e3)
    ab = contract.algorithmic_bytes(T, K, H, 2, 2, fp8, stub_folded=True)
    b_dc = ab["dispatch"] + ab["combine"]
    if any(n in per for n in FORWARD_KERNELS):
        cand = [(next(n for n in FORWARD_KERNELS if n in per), b_dc)]
    else:
        cand = [(next(n for n in DISPATCH_KERNELS if n in per), ab["dispatch"]),
                (next(n for n in COMBINE_KERNELS if n in per), ab["combine"])]
    dom, dom_bytes = max(cand, key=lambda c: statistics.fmean(per[c[0]]))
    dom_us = statistics.fmean(per[dom]) + t["gap"]
    want = V.run_world(cfg, wl.world, stub_kind=wl.stub_kind, fp8=bool(fp8), combine_mode=mode)["y"]
    same = bool(torch.equal(leg.y.cpu().view(torch.int16), want.view(torch.int16)))
    value = b_dc / t["dc"] / 1e3
    return dict(ms_per_step=round(ms, 6), dispatch_combine_us=round(t["dc"], 3), value=round(value, 1),
                pct_of_hbm_peak=round(100.0 * value / HBM_PEAK_GBPS, 2), kernel=dom,
                roofline_frac=round(dom_bytes / dom_us / 1e3 / HBM_PEAK_GBPS, 4), kernel_avg_us=round(dom_us, 3),
                launches_per_step=int(lib.moe_a2a_forward_launches(T, K, H, 0, _lib.BF16, _lib.BF16, int(bool(fp8)), 1, 1)),
                combine="f32" if mode else "strict", bytes=b_dc,
                kernels_us={k: round(statistics.fmean(v), 3) for k, v in per.items()},
                gpu_output_bit_identical=same)


def moe_layer_leg(torch, lib, contract, wl, tensors, main, dev, mode, args):
    """dispatch -> grouped expert GEMM (hidden -> hidden, random weights) -> combine: the path as it
    runs around a real expert layer (all2all/reference.py:261-270 with the stub replaced by a linear
    layer per expert).  Per-kernel durations from the launch timer, wall clock of whole steps, and
    a check of each stage: the expert rows of a sample of experts against the oracle's f32 product,
    the combine output bit for bit against the oracle's combine of the GPU's expert rows."""
    from kernel_amd.all2all import HipAllToAll
    from oracle import all2all_vec as V  # checker only

    cfg = wl.cfg
    x, idx, w, rs = tensors
    E, H, K, T = cfg.num_experts, cfg.hidden_dim, cfg.experts_per_token, x.shape[0]
    weight_bytes = E * H * H * 2
    free = torch.cuda.mem_get_info(dev)[0]
    if weight_bytes > 0.6 * free:
        return dict(skipped=f"{weight_bytes / 1e9:.1f} GB of expert weights do not fit beside the rest")
    g = torch.Generator(device=dev).manual_seed(4321)
    weights = torch.empty(E, H, H, dtype=cfg.in_dtype, device=dev)
    for e in range(E):  # in place, expert by expert: no f32 copy of the whole tensor
        weights[e] = (torch.randn(H, H, generator=g, device=dev) * (H ** -0.5)).to(cfg.in_dtype)
    ata = HipAllToAll(cfg, 0, wl.world_size, stub_kind=wl.stub_kind, combine_mode=mode)
    steps = max(5, min(args.steps, 50))

    def step():
        d = ata.dispatch(x, idx, rs)
        ey = ata.expert_gemm(d, weights, out=step.ey)
        return d, ey, ata.combine(None, w, d, ey)

    with torch.cuda.stream(main):
        step.ey = torch.empty(T * K, H, dtype=cfg.out_dtype, device=dev)
        d, ey, y = step()
        spin_up(main, step)
        per = kernel_times(lib, lambda n: [step() for _ in range(n)], steps, torch)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(main)
        for _ in range(steps):
            d, ey, y = step()
        e1.record(main)
        main.synchronize()
    wall_us = e0.elapsed_time(e1) * 1e3 / steps
    per.pop("route_empty", None)
    mean = {k: statistics.fmean(v) for k, v in per.items()}
    gemm_name = next(k for k in mean if k.startswith("expert_gemm"))
    dc_us = sum(v for k, v in mean.items() if k != gemm_name and not k.startswith("fill"))
    # the fill that clears the status word is torch's kernel, not the library's: it is not in `per`
    ab = contract.algorithmic_bytes(T, K, H, 2, 2, False, stub_folded=False)
    b_dc = ab["dispatch"] + ab["combine"]
    flops = 2.0 * T * K * H * H
    live = int((d.counts > 0).sum())
    gemm_bytes = T * K * H * 2 * 2 + live * H * H * 2
    # checks
    off = d.offsets.cpu()
    sample = [e for e in range(E) if int(off[e + 1]) > int(off[e])][:6]
    worst = 0.0
    for e in sample:
        lo, hi = int(off[e]), int(off[e + 1])
        ref = V.expert_gemm(d.disp_x[lo:hi].cpu(), torch.tensor([0, hi - lo], dtype=torch.int32), weights[e:e + 1].cpu(),
                            cfg.out_dtype).float()
        got = ey[lo:hi].cpu().float()
        tol = 1e-2 * ref.abs() + 1e-2 * ref.pow(2).mean(dim=1, keepdim=True).sqrt()
        worst = max(worst, float(((got - ref).abs() / tol).max()))
    comb = V.combine_strict if mode == 0 else V.combine_f32
    y_ref = comb(ey.cpu(), w.cpu(), d.slot_of_entry.cpu(), cfg.out_dtype)
    out = dict(what="dispatch -> moe_a2a_expert_gemm (hidden -> hidden, 16-bit weights) -> combine, three launches",
               wall_us_per_step=round(wall_us, 2), steps=steps,
               kernels_us={k: round(v, 3) for k, v in mean.items()},
               dispatch_combine_kernel_us=round(dc_us, 3),
               dispatch_combine_pct_of_hbm_peak=round(100.0 * b_dc / dc_us / 1e3 / HBM_PEAK_GBPS, 2),
               expert_gemm=dict(kernel=gemm_name, us=round(mean[gemm_name], 2),
                                tflops=round(flops / mean[gemm_name] / 1e6, 1),
                                weight_stream_GBps=round(gemm_bytes / mean[gemm_name] / 1e3, 1),
                                bound="hbm (weights read once)" if gemm_bytes / (HBM_PEAK_GBPS * 1e3) >
                                flops / (MFMA_PEAK_TFLOPS * 1e6) else "mfma",
                                frac_of_hbm_peak=round(gemm_bytes / mean[gemm_name] / 1e3 / HBM_PEAK_GBPS, 4)),
               expert_rows_worst_error_of_tolerance=round(worst, 3), experts_checked=len(sample),
               combine_bit_identical_to_oracle_on_gpu_expert_rows=bool(
                   torch.equal(y.cpu().view(torch.int16), y_ref.view(torch.int16))))
    if worst > 1.0:
        raise RuntimeError(f"expert rows outside the tolerance of the f32 reference: {worst:.2f}x")
    del weights
    return out


def calibrate_copy(torch, main, dev):
    """Three plain 256 MiB device copies: the known-size reference for the profiler's byte counters."""
    with torch.cuda.stream(main):
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(3)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
    torch.cuda.synchronize()


KERNEL_OF_SYMBOL = (("route_dispatch_fp8_tile_kernel", "route_dispatch_fp8"),
                    ("route_dispatch_tile_kernel", "route_dispatch_tile"), ("route_dispatch_kernel", "route_dispatch"),
                    ("forward_token_kernel", "forward_token"), ("forward_tile_kernel", "forward_tile"),
                    ("dispatch_fold_kernel", "dispatch_fold"),
                    ("stub_combine_rows_kernel", "stub_combine"), ("stub_combine_fp8_kernel", "stub_combine"),
                    ("combine_rows_kernel", "combine_rows"), ("dispatch_rows_kernel", "dispatch_rows"),
                    ("dispatch_fp8_kernel", "dispatch_fp8"), ("stub_rows_kernel", "stub_rows"),
                    ("stub_fp8_kernel", "stub_fp8"))


def record_traffic(directory):
    """Fold the counter CSVs of `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` runs of
    `bench.py --graph-only --calibrate-copy --workload W` into profiles/traffic.json.

    `directory` holds one sub-directory per run named <workload>_<COUNTER> with rocprofv3's
    *_counter_collection.csv inside.  The scale of each counter is what it reads for the 256 MiB
    copies at the end of every run.  Each entry records the kernel's symbol, the hash of the kernel
    sources and the commit the tree was at."""
    import csv
    import glob
    import subprocess

    COPY_BYTES = 256 << 20
    runs = {}
    for path in sorted(glob.glob(os.path.join(directory, "*", "**", "*counter_collection.csv"), recursive=True)):
        run = os.path.relpath(path, directory).split(os.sep)[0]
        workload, counter = run.rsplit("_", 2)[0], "_".join(run.rsplit("_", 2)[1:])
        per_kernel = {}
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] != counter:
                    continue
                per_kernel.setdefault(row["Kernel_Name"], []).append(float(row["Counter_Value"]))
        runs[(workload, counter)] = per_kernel
    if not runs:
        raise SystemExit(f"no *_counter_collection.csv under {directory}/<workload>_<COUNTER>/")
    try:
        commit = subprocess.run(["git", "rev-parse", "--short=12", "HEAD"], capture_output=True, text=True,
                                cwd=ROOT).stdout.strip() or "?"
    except OSError:
        commit = "?"
    factor, entries, src = {}, [], kernel_source_hash()
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        reads = [statistics.median(v) for (wl_, c), ks in runs.items() if c == counter
                 for k, v in ks.items() if "copyBuffer" in k]
        if not reads:
            raise SystemExit(f"no calibration copy in the {counter} runs (run bench.py with --calibrate-copy)")
        factor[counter] = round(COPY_BYTES / (statistics.median(reads) * 1024.0), 3)
    for workload in sorted({wl_ for wl_, _ in runs}):
        fetch, write = runs.get((workload, "FETCH_SIZE"), {}), runs.get((workload, "WRITE_SIZE"), {})
        for symbol in sorted(set(fetch) & set(write)):
            name = next((n for pat, n in KERNEL_OF_SYMBOL if pat in symbol), None)
            if name is None:
                continue
            f_kib, w_kib = statistics.median(fetch[symbol]), statistics.median(write[symbol])
            entries.append(dict(workload=workload, kernel=name,
                                symbol=symbol.replace("void ", "").replace("(anonymous namespace)::", "")[:100],
                                fetch_kib=round(f_kib, 1), write_kib=round(w_kib, 1),
                                bytes=int((f_kib * factor["FETCH_SIZE"] + w_kib * factor["WRITE_SIZE"]) * 1024),
                                launches=len(fetch[symbol]), source_hash=src, commit=commit))
    rec = dict(what="HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch, L2 <-> fabric), "
                    "median over the launches of `bench.py --graph-only --calibrate-copy --workload W`",
               factor=factor, factor_from="the same counters' medians for the three 256 MiB device copies that end each run",
               entries=entries)
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    print(f"wrote {TRAFFIC_FILE}: {len(entries)} entries, factors {factor}, sources {src}, commit {commit}")


MFMA_PEAK_TFLOPS = 2500.0  # dense bf16 / fp16
FP8_MFMA_PEAK_TFLOPS = 5000.0  # dense fp8


def expert_gemm_leg(args, lib, torch, wl, x, idx, rs, dev):
    """Grouped expert GEMM y[seg e] = x[seg e] @ W_e^T on the workload's 16-bit dispatched rows.
    One JSON line: TFLOP/s against the dense 16-bit MFMA peak, kernel time from the launch timer,
    and a CPU leg (the oracle's per-expert f32 matmul on a bounded number of experts) that also
    checks the GPU rows it covers."""
    from kernel_amd.all2all import HipAllToAll

    cfg = wl.cfg
    E, H, N = cfg.num_experts, cfg.hidden_dim, args.expert_gemm
    fp8 = (wl.fp8_dispatch or args.fp8_rows) and not args.bf16_dispatch
    pow2 = bool(args.pow2_scales)
    if pow2 and not (fp8 and args.fp8_weights):
        raise SystemExit("--pow2-scales needs an fp8 workload (fp8 rows) and --fp8-weights")
    ata = HipAllToAll(cfg, 0, wl.world_size, stub_kind=wl.stub_kind, fp8_dispatch="pow2" if pow2 else fp8)
    gen = torch.Generator(device="cpu").manual_seed(1234)
    weights = (torch.randn(E, N, H, generator=gen) / H ** 0.5).to(cfg.in_dtype).to(dev)
    w_scale = None
    if args.fp8_weights:  # block quantisation of the synthetic weights (input preparation, not timed)
        wf = weights.float().view(E, N // 128, 128, H // 128, 128)
        amax = wf.abs().amax(dim=(2, 4))
        w_scale = torch.where(amax == 0, torch.ones_like(amax), amax / 448.0).contiguous()
        if pow2:  # the next power of two at or above (exponent field + 1 when the mantissa is not zero)
            u = w_scale.view(torch.int32)
            w_scale = (((u >> 23) + ((u & 0x7FFFFF) != 0).to(torch.int32)).clamp(1, 254) << 23).view(torch.float32)
        weights = (wf / w_scale[:, :, None, :, None]).to(torch.float8_e4m3fn).view(E, N, H).contiguous()
    main = torch.cuda.Stream()
    main.wait_stream(torch.cuda.current_stream())
    if args.equal_segments:
        idx = (torch.arange(idx.numel(), device=dev, dtype=torch.int32) % E).view_as(idx).contiguous()
    with torch.cuda.stream(main):
        d = ata.dispatch(x, idx, rs)
        R = d.num_rows
        y = torch.empty(R, N, dtype=cfg.in_dtype, device=dev)
        spin_up(main, lambda: ata.expert_gemm(d, weights, out=y, w_scale=w_scale, scales_pow2=pow2))
        for _ in range(args.warmup):
            ata.expert_gemm(d, weights, out=y, w_scale=w_scale, scales_pow2=pow2)
        main.synchronize()
        per = kernel_times(lib, lambda n: [ata.expert_gemm(d, weights, out=y, w_scale=w_scale, scales_pow2=pow2) for _ in range(n)], args.steps, torch)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(main)
        for _ in range(args.steps):
            ata.expert_gemm(d, weights, out=y, w_scale=w_scale, scales_pow2=pow2)
        e1.record(main)
        main.synchronize()
    ms_step = e0.elapsed_time(e1) / args.steps
    kernel = next(k for k in ("expert_gemm_mx", "expert_gemm_f8", "expert_gemm_wide", "expert_gemm_skinny", "expert_gemm") if k in per)
    t_us = statistics.fmean(per[kernel])
    flops = 2.0 * R * H * N
    tflops = flops / t_us / 1e6
    out = dict(metric=f"grouped expert GEMM TFLOP/s, {E}E h{H} n{N}", value=round(tflops, 1), unit="TFLOP/s",
               n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=round(ms_step, 5), higher_is_better=True,
               scaling="weak", vs_baseline=None, dtype="bf16" if cfg.in_dtype == torch.bfloat16 else "f16",
               data="synthetic",
               config=dict(workload=wl.name + "+expert_gemm", rows=R, experts=E, hidden=H, out_columns=N, kernel=kernel,
                           segments="equal" if args.equal_segments else "the workload's routing",
                           rows_dtype="fp8 e4m3fn + f32 scale per 128 columns" if fp8 else "16-bit",
                           weights_dtype="fp8 e4m3fn + f32 scale per 128 x 128 block" if args.fp8_weights else "16-bit"),
               kernels_us=summarise(per),
               )
    # which roof: the operands must cross HBM once (rows, the weights of every expert that has rows,
    # the output); if that takes longer at 8 TB/s than the flops at the MFMA peak, the launch is HBM-bound
    live = int((d.counts > 0).sum())
    # the kernel with both operands fp8 multiplies on the fp8 matrix instruction (dense peak 5.0 PFLOP/s)
    mfma_peak = FP8_MFMA_PEAK_TFLOPS if kernel in ("expert_gemm_f8", "expert_gemm_mx") else MFMA_PEAK_TFLOPS
    if kernel in ("expert_gemm_f8", "expert_gemm_mx") or (fp8 and args.fp8_weights):
        out["dtype"] = "fp8"
    gemm_bytes = R * H * (1 + 4 / 128 if fp8 else 2) + live * N * H * (1 if args.fp8_weights else 2) + R * N * 2
    if gemm_bytes / (HBM_PEAK_GBPS * 1e3) > flops / (mfma_peak * 1e6):
        gbps = gemm_bytes / t_us / 1e3
        out["roofline"] = dict(bound="hbm", achieved=round(gbps, 1), peak=HBM_PEAK_GBPS, unit="GB/s",
                               frac=round(gbps / HBM_PEAK_GBPS, 4), traffic=None)
    else:
        out["roofline"] = dict(bound="mfma", achieved=round(tflops, 1), peak=mfma_peak, unit="TFLOP/s",
                               frac=round(tflops / mfma_peak, 4), traffic=None)
    if not args.no_cpu:
        from oracle import all2all_vec as O

        off = d.offsets.cpu()
        dx, wc, yg = d.disp_x.cpu(), weights.cpu(), y.cpu()
        dsc = d.disp_scale.cpu() if fp8 else None
        t0, done, rows_done, worst = time.perf_counter(), 0, 0, 0.0
        for e in range(E):
            lo, hi = int(off[e]), int(off[e + 1])
            if hi > lo:
                seg = torch.tensor([0, hi - lo], dtype=torch.int32)
                if args.fp8_weights:
                    ref = O.expert_gemm_q8(dx[lo:hi], dsc[lo:hi] if fp8 else None, wc[e:e + 1].view(torch.uint8),
                                           w_scale[e:e + 1].cpu(), seg, cfg.in_dtype)
                elif fp8:
                    ref = O.expert_gemm_fp8(dx[lo:hi], dsc[lo:hi], seg, wc[e:e + 1], cfg.in_dtype)
                else:
                    ref = O.expert_gemm(dx[lo:hi], seg, wc[e:e + 1], cfg.in_dtype)
                want, got = ref.float(), yg[lo:hi].float()
                # summation order (and, for quantised weights on long segments, one rounding of the
                # dequantised weight) differs from the CPU's: 1 % of the value + 1 % of the row's rms
                tol = 1e-2 * want.abs() + 1e-2 * want.pow(2).mean(dim=1, keepdim=True).sqrt()
                worst = max(worst, float(((got - want).abs() / tol).max()))
                rows_done += hi - lo
            done += 1
            if time.perf_counter() - t0 > args.cpu_seconds:
                break
        dt = time.perf_counter() - t0
        if worst > 1.0:
            raise RuntimeError(f"expert GEMM outside the tolerance of the f32 reference: {worst:.2f}x")
        out["cpu_baseline"] = dict(value=round(2.0 * rows_done * H * N / dt / 1e12, 4), unit="TFLOP/s",
                                   cores=torch.get_num_threads(), kind="port",
                                   sample=f"first {done} of {E} experts ({rows_done} rows), f32 matmul; "
                                          f"worst error {worst:.2f} of the tolerance")
    print(json.dumps(out))


def gemm_rs_leg(args, lib, torch, dev):
    """GEMM + reduce-scatter of gemm_rs/reference.py:36-60 for a world of 8 ranks held as K shards of
    one buffer.  One JSON line per shape: TFLOP/s of the whole world's product (2 M N K) against the
    dense 16-bit MFMA peak, or GB/s when moving the operands once takes longer than the flops; the
    reference's speed-of-light figure for the shape (task.yml:49-54: per GPU of an 8-GPU node, so one
    GPU doing all eight shares has eight times the flops to do); a CPU leg on sampled rows."""
    from kernel_amd import gemm_rs as G

    sol_us = {(64, 7168, 18432): 6.46, (512, 4096, 12288): 8.19, (2048, 2880, 2880): 23.04,
              (4096, 4096, 4096): 65.54, (8192, 4096, 14336): 131.07, (8192, 8192, 29568): 379.43}
    if args.gemm_rs == "all":
        specs = G.BENCHMARK_SPECS
    else:
        parts = args.gemm_rs.split(",")
        specs = [dict(world_size=8, m=int(parts[0]), n=int(parts[1]), k=int(parts[2]),
                      has_bias=len(parts) > 3 and parts[3] == "bias", seed=1234)]
    main = torch.cuda.Stream()
    main.wait_stream(torch.cuda.current_stream())
    for spec in specs:
        W, m, n, k = spec["world_size"], spec["m"], spec["n"], spec["k"]
        datas = [G.generate_input(r, **spec) for r in range(W)]
        x, w, bias = G.pack_world(datas, dev)
        op = G.HipGemmReduceScatter(W)
        out = torch.empty((m, n), dtype=x.dtype, device=dev)
        with torch.cuda.stream(main):
            spin_up(main, lambda: op.forward(x, w, bias, out=out))
            for _ in range(max(args.warmup, 2)):
                op.forward(x, w, bias, out=out)
            main.synchronize()
            per = kernel_times(lib, lambda cnt: [op.forward(x, w, bias, out=out) for _ in range(cnt)], args.steps, torch)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(main)
            for _ in range(args.steps):
                op.forward(x, w, bias, out=out)
            e1.record(main)
            main.synchronize()
        ms_step = e0.elapsed_time(e1) / args.steps
        t_us = sum(statistics.fmean(v) for v in per.values())  # one or two kernels per call
        kernel = max(per, key=lambda kk: statistics.fmean(per[kk]))
        flops = 2.0 * m * n * k
        tflops = flops / t_us / 1e6
        ws = int(lib.gemm_rs_workspace_bytes(m, n, k, W))
        line = dict(metric=f"GEMM + reduce-scatter TFLOP/s, 8 K-shards on one GPU, m{m} n{n} k{k}", value=round(tflops, 1),
                    unit="TFLOP/s", n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=round(ms_step, 5),
                    higher_is_better=True, scaling="weak", vs_baseline=None, dtype="bf16", data="synthetic",
                    config=dict(workload="gemm_rs", m=m, n=n, k=k, emulated_ranks=W, has_bias=spec["has_bias"],
                                kernel=kernel, workspace_bytes=ws),
                    kernels_us=summarise(per), kernel_us=round(t_us, 2),
                    reference_speed_of_light_us_per_gpu_of_8=sol_us.get((m, n, k)))
        # algorithmic bytes: operands in and the result out, once (what a split form writes and reads again
        # as partial products, or a padded copy, is the implementation's own traffic and earns nothing)
        gemm_bytes = (m + n) * k * 2 + m * n * 2
        if gemm_bytes / (HBM_PEAK_GBPS * 1e3) > flops / (MFMA_PEAK_TFLOPS * 1e6):
            gbps = gemm_bytes / t_us / 1e3
            line["roofline"] = dict(bound="hbm", achieved=round(gbps, 1), peak=HBM_PEAK_GBPS, unit="GB/s",
                                    frac=round(gbps / HBM_PEAK_GBPS, 4), traffic=None)
        else:
            line["roofline"] = dict(bound="mfma", achieved=round(tflops, 1), peak=MFMA_PEAK_TFLOPS, unit="TFLOP/s",
                                    frac=round(tflops / MFMA_PEAK_TFLOPS, 4), traffic=None)
        if not args.no_cpu:
            from oracle import gemm_rs as O  # checker and baseline only

            rows = min(m, 64)
            sample = [(d[0][:rows], d[1], d[2]) for d in datas]
            t0, reps = time.perf_counter(), 0
            while True:
                want = O.ref_world(sample)
                reps += 1
                if time.perf_counter() - t0 > min(args.cpu_seconds, 10.0) or reps >= 20:
                    break
            dt = (time.perf_counter() - t0) / reps
            ok, msg = O.check_implementation(want, out[:rows].cpu())
            if not ok:
                raise RuntimeError("GEMM + reduce-scatter outside the reference's tolerance on the sampled rows")
            line["cpu_baseline"] = dict(value=round(2.0 * rows * n * k / dt / 1e12, 4), unit="TFLOP/s",
                                        cores=torch.get_num_threads(), kind="port",
                                        sample=f"first {rows} of {m} rows, every rank's bf16 matmul + bias and the sum "
                                               f"over the ranks; the GPU rows are within the reference's tolerance")
        print(json.dumps(line), flush=True)
        del x, w, bias, out, datas


def cpu_baseline(wl, mode, fp8, y_gpu, b_dc, budget_s):
    """The CPU oracle on the host cores: same workload, same bytes; also checks the GPU output."""
    import torch

    from oracle import all2all_vec as V  # checker and baseline only

    cfg = wl.cfg
    K = cfg.experts_per_token
    x, idx, w, starts = V.concat_world(wl.world)
    comb = V.combine_strict if mode == 0 else V.combine_f32
    times = []
    t_begin = time.perf_counter()
    y_cpu = None
    while True:
        t0 = time.perf_counter_ns()
        r = V.route(idx, starts, cfg.num_experts)
        if fp8:
            dx, sc = V.dispatch_fp8(x, r["src_of_slot"], K)
        else:
            dx, sc = V.dispatch(x, r["src_of_slot"], K), None
        t1 = time.perf_counter_ns()
        ey = V.stub(dx, r["meta"], wl.stub_kind, cfg.num_experts, wl.world_size, cfg.out_dtype, scale=sc)
        t2 = time.perf_counter_ns()
        y_cpu = comb(ey, w, r["slot_of_entry"], cfg.out_dtype)
        t3 = time.perf_counter_ns()
        times.append(((t1 - t0) + (t3 - t2)) / 1e3)
        if len(times) >= 3 and (time.perf_counter() - t_begin > budget_s or len(times) >= 50):
            break
    us = statistics.median(times[1:])
    same = bool(torch.equal(y_gpu.cpu().view(torch.int16), y_cpu.view(torch.int16)))
    out = dict(value=round(b_dc / us / 1e3, 3), unit="GB/s", cores=torch.get_num_threads(), kind="port",
               dispatch_combine_us=round(us, 1),
               sample=f"full workload {wl.name}: {len(times) - 1} timed passes of route+dispatch+combine "
                      f"(vectorised torch-CPU oracle), median",
               gpu_output_bit_identical=same)
    # the row-by-row form of the reference's loops (all2all/reference.py:123-146, 227-232), where it
    # finishes in a second: three passes, median; fp8 has no row-loop form
    if not fp8 and mode == 0 and x.shape[0] * K <= 8192:
        from oracle import all2all_literal as Lit

        lit = []
        for _ in range(3):
            t0 = time.perf_counter_ns()
            disp = Lit.dispatch_world(cfg, wl.world)
            t1 = time.perf_counter_ns()
            ey = Lit.stub_world(cfg, disp, wl.stub_kind)
            t2 = time.perf_counter_ns()
            Lit.combine_world(cfg, wl.world, disp, ey)
            t3 = time.perf_counter_ns()
            lit.append(((t1 - t0) + (t3 - t2)) / 1e3)
        out["row_loop_dispatch_combine_us"] = round(statistics.median(lit), 1)
    return out


if __name__ == "__main__":
    main()
