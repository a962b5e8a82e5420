#!/usr/bin/env python3
"""Benchmark of the dispatch / combine hot path on one MI355X.

A step is one cached-handle dispatch followed by one combine of the DeepSeek-V3-shaped batch
(4096 tokens x 7168 bf16, 256 experts, top-8, 10% of choices masked, expanded layout with
zero_padding) through the public API, with every input already resident in HBM.  The script prints
ONE JSON line: whole-step achieved HBM bandwidth (algorithmic bytes / wall time), the per-kernel
microseconds measured with HIP events on the stream the kernels run on, the roofline of the
dominant kernel and a CPU baseline (the torch-CPU oracle timed on this host's cores).

Timing protocol, the same whatever --steps / --warmup say: at least 20 untimed warm-up launches,
then REGIONS timed regions of REGION_LAUNCHES back-to-back launches each, every region bracketed by
a device synchronisation and two HIP events on the kernels' stream; the figure reported for a kernel
is the MEDIAN of the regions' per-launch times, with the fastest region beside it (`*_min`).  The
region of exactly --steps steps after --warmup warm-up steps is timed as well and reported as
`cli_region`.  The other benchmark shapes follow under `roofline_by_workload` (same protocol, shorter
CPU samples; `--workload deepseek-v3` leaves them out).
"""

from __future__ import annotations

import argparse
import json
import os
import re
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E peak
WARMUP_MIN = 20        # untimed launches ahead of every series of timed regions
REGIONS = 7            # timed regions per figure
REGION_LAUNCHES = 100  # back-to-back launches per region
HEADLINE = "deepseek-v3"


def log(*parts):
    print(*parts, file=sys.stderr, flush=True)


def parse_args():
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=200)
    parser.add_argument("--warmup", type=int, default=50)
    parser.add_argument("--workload", default="all",
                        help="`all` (default): the headline shape, then the other benchmark shapes under roofline_by_workload; "
                             "or the name of one shape")
    parser.add_argument("--cpu-seconds", type=float, default=15.0, help="CPU baseline budget per workload; 0 skips it")
    parser.add_argument("--no-scalar-oracle", dest="scalar_oracle", action="store_false",
                        help="skip timing the scalar-loop oracle (it runs once on the readme-toy and mixtral shapes only: "
                             "it is a specification, not a performance path)")
    parser.add_argument("--regions", type=int, default=REGIONS)
    parser.add_argument("--region-launches", type=int, default=REGION_LAUNCHES)
    parser.add_argument("--calibration-copy-mib", type=int, default=0,
                        help="also launch the plain copy kernel on this many MiB (known-size reference for profiler byte counters)")
    return parser.parse_args()


def measured_traffic(kernel: str, workload: str):
    """(HBM bytes per launch, where that number comes from) out of the committed profiler summary.

    The counters are not collected by this run: they come from two `rocprofv3 --pmc` runs of this
    script whose summary is kept under profiles/, and `source` names that file and the commit the
    library was built from when it was taken, so that a stale summary shows."""
    path = ROOT / "profiles" / f"{kernel}_{workload}_pmc.txt"
    if not path.exists():
        return None, None
    text = path.read_text()
    match = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", text, flags=re.M)
    commit = re.search(r"^source_commit:\s*(\S+)", text, flags=re.M)
    source = {"file": str(path.relative_to(ROOT)), "commit": commit.group(1) if commit else "not recorded",
              "collected_by": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (separate runs), not by this run"}
    return (float(match.group(1)) if match else None), source


def layout_gpu_us(workload, idx, iterations=100):
    """GPU time of the routing-layout launches alone (no host wait), through the C ABI."""
    import ctypes

    import torch

    library = ctypes.CDLL(str(ROOT / "nanoep_amd" / "libnanoep_hip.so"))
    p, i64 = ctypes.c_void_p, ctypes.c_int64
    library.nanoep_layout_workspace_bytes.restype = ctypes.c_size_t
    library.nanoep_layout_workspace_bytes.argtypes = [i64, ctypes.c_int, i64]
    library.nanoep_slot_order_entries.restype = i64
    library.nanoep_slot_order_entries.argtypes = [i64, ctypes.c_int, i64]
    library.nanoep_layout.argtypes = [p, i64, ctypes.c_int, i64, i64, ctypes.c_int, ctypes.c_int, p, p, p, p, p, p, p, p, p, p, ctypes.c_size_t, p, p]
    tokens, topk, experts = workload.tokens, workload.topk, workload.experts
    device = idx.device
    nbytes = library.nanoep_layout_workspace_bytes(tokens, topk, experts)
    workspace = torch.empty(nbytes, dtype=torch.uint8, device=device)
    metadata = torch.empty((tokens, topk + 2), dtype=torch.int32, device=device)
    table = torch.empty((tokens, topk), dtype=torch.int32, device=device)
    order = torch.empty(max(1, library.nanoep_slot_order_entries(tokens, topk, experts)), dtype=torch.int64, device=device)
    snapshot = torch.empty_like(idx)
    dst_slots = torch.empty((tokens, 1), dtype=torch.int64, device=device)
    counts = torch.empty(experts, dtype=torch.int64, device=device)
    offsets = torch.empty(experts + 1, dtype=torch.int64, device=device)
    sent = torch.empty(1, dtype=torch.int64, device=device)
    prefix = torch.empty(1, dtype=torch.int64, device=device)
    mailbox = torch.empty(4, dtype=torch.int64, pin_memory=True)
    stream = torch.cuda.current_stream()

    def launch():
        status = library.nanoep_layout(idx.data_ptr(), tokens, topk, experts, workload.alignment, int(workload.expand),
                                       workload.hidden, metadata.data_ptr(), counts.data_ptr(), offsets.data_ptr(), dst_slots.data_ptr(),
                                       sent.data_ptr(), snapshot.data_ptr(), prefix.data_ptr(),
                                       table.data_ptr() if workload.expand else None,
                                       order.data_ptr() if workload.expand else None, workspace.data_ptr(), nbytes,
                                       mailbox.data_ptr(), stream.cuda_stream)
        if status != 0:
            raise RuntimeError(f"nanoep_layout failed with status {status}")

    for _ in range(WARMUP_MIN):
        launch()
    samples = []
    for _ in range(5):
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        begin.record(stream)
        for _ in range(iterations):
            launch()
        end.record(stream)
        torch.cuda.synchronize()
        samples.append(begin.elapsed_time(end) * 1e3 / iterations)
    return statistics.median(samples)


def host_description():
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as info:
            model = next((line.split(":", 1)[1].strip() for line in info if line.startswith("model name")), model)
    except OSError:
        pass
    return model, os.cpu_count() or 1


def cpu_baseline(workload, x, idx, weights, budget_seconds, gpu_dispatched=None, gpu_combined=None, scalar=False):
    """The vectorised torch-CPU oracle on the same batch: dispatch + combine, bounded in time.

    When the GPU results of the same batch are given, they are compared bit for bit with the
    oracle's (NaN-free synthetic data, so plain bit equality is the bar) and the verdict is returned.
    """
    import torch

    from nanoep_amd import workloads
    from oracle import nanoep_oracle as oracle

    cpu_model, host_cpus = host_description()
    # the GPU box gives one GPU's share of its host: 16 cores, whatever the machine has
    cores = min(16, host_cpus)
    torch.set_num_threads(cores)
    layout = oracle.layout(idx, workload.experts, workload.alignment)
    received, capacity = layout.recv_count, layout.expanded_capacity
    assignments = int(layout.expert_counts.sum())
    nbytes = (workloads.dispatch_bytes(workload, received, assignments, capacity)
              + workloads.combine_bytes(workload, received, assignments, weighted=workload.combine_weights))
    metadata = layout.recv_metadata(workload.expand)

    def step():
        out_x, _, out_w, _ = oracle.dispatch(x, idx, workload.experts, weights, do_expand=workload.expand,
                                             alignment=workload.alignment, lay=layout)
        oracle.combine(out_x, metadata, layout.dst_slots, do_expand=workload.expand,
                       weights=out_w if workload.combine_weights else None)

    parity = None
    if gpu_dispatched is not None:
        want_x, _, want_w, _ = oracle.dispatch(x, idx, workload.experts, weights, do_expand=workload.expand,
                                               alignment=workload.alignment, lay=layout)
        want_combined, _ = oracle.combine(want_x, metadata, layout.dst_slots, do_expand=workload.expand)
        parity = bool(torch.equal(gpu_dispatched.view(torch.int16), want_x.view(torch.int16))
                      and torch.equal(gpu_combined.view(torch.int16), want_combined.view(torch.int16)))
        del want_x, want_combined

    def sample(limit_seconds, limit_steps):
        step()  # warm caches and the allocator
        times = []
        started = time.perf_counter()
        while True:
            t0 = time.perf_counter()
            step()
            times.append(time.perf_counter() - t0)
            if time.perf_counter() - started > limit_seconds or len(times) >= limit_steps:
                break
        return statistics.median(times), len(times)

    seconds, count = sample(budget_seconds, 20)
    torch.set_num_threads(1)
    single_seconds, single_count = sample(budget_seconds / 2, 5)
    torch.set_num_threads(cores)
    baseline = {
        "value": round(nbytes / seconds / 1e9, 3),
        "unit": "GB/s",
        "cores": cores,
        "host_cpu_count": host_cpus,
        "cpu_model": cpu_model,
        "kind": "port",
        "us_per_step": round(seconds * 1e6, 1),
        "value_1_thread": round(nbytes / single_seconds / 1e9, 3),
        "sample": f"{count} timed steps (cached-layout dispatch + combine) of the full {workload.name} batch "
                  f"with the vectorised torch-CPU oracle, {cores} threads; {single_count} steps with 1 thread",
    }
    if scalar and workload.tokens * workload.topk <= 4096 * 2:
        # the scalar-loop restatement of the reference's oracle, once, for the record
        t0 = time.perf_counter()
        out_x, _, _, scalar_layout = oracle.dispatch_scalar(x, idx, workload.experts, weights, do_expand=workload.expand,
                                                            alignment=workload.alignment)
        oracle.combine_scalar(out_x, scalar_layout.recv_metadata(workload.expand), scalar_layout.dst_slots, do_expand=workload.expand)
        elapsed = time.perf_counter() - t0
        baseline["scalar_oracle_us_per_step"] = round(elapsed * 1e6, 1)
        baseline["scalar_oracle_GBps"] = round(nbytes / elapsed / 1e9, 4)
    return baseline, parity


def summarize(samples_seconds, launches):
    """(median, min) microseconds per launch over timed regions of `launches` launches each."""
    per_launch = [s / launches * 1e6 for s in samples_seconds]
    return statistics.median(per_launch), min(per_launch)


def roofline_entry(kernel, workload_name, nbytes, median_us, min_us):
    traffic, source = measured_traffic(kernel, workload_name)
    return {
        "kernel": kernel,
        "bound": "hbm",
        "achieved": round(nbytes / median_us / 1e3, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(nbytes / median_us / 1e3 / HBM_PEAK_GBS, 4),
        "frac_fastest_region": round(nbytes / min_us / 1e3 / HBM_PEAK_GBS, 4),
        "traffic": traffic,
        "traffic_source": source,
        "algorithmic_bytes": nbytes,
        "avg_us": round(median_us, 2),
        "min_us": round(min_us, 2),
    }


def measure(workload, args, device, detailed):
    """All figures of one workload.  `detailed` adds the fresh-dispatch, cache-resident and layout
    figures and the --steps region (the headline workload)."""
    import torch

    from nanoep_amd import Buffer, EPConfig, workloads

    # Rotating source copies: at least 8, and at least three times the 256 MiB last-level cache in
    # total, so that no launch finds its source cache resident (14 x 58.7 MB at the headline batch,
    # 24 copies of a 33.5 MB source).  Copy 0 is the batch that is checked against the oracle.
    x_cpu, idx_cpu, w_cpu = workloads.make_inputs(workload, seed=0)
    source_bytes = max(1, x_cpu.numel() * x_cpu.element_size())
    rotation = min(32, max(8, -(-3 * (256 << 20) // source_bytes)))
    generator = torch.Generator(device=device).manual_seed(1)
    xs = [x_cpu.to(device)] + [
        torch.randn(x_cpu.shape, device=device, generator=generator, dtype=torch.float32).to(torch.bfloat16)
        for _ in range(rotation - 1)
    ]
    idx = idx_cpu.to(device)
    weights = w_cpu.to(device)
    regions, launches = max(1, args.regions), max(1, args.region_launches)

    buffer = Buffer(None, EPConfig(workload.experts, workload.topk, workload.hidden, workload.tokens))
    stream = buffer.comm_stream  # run the loop on the stream the kernels are launched on
    result = {}
    with torch.cuda.stream(stream):
        # fresh dispatch: layout kernels + host wait for N/C + permute, as seen by the caller
        # (two series: wall clock around call + synchronisation with nothing else in between, then the
        # same calls between two HIP events, whose recording costs the host a few microseconds)
        fresh_times, fresh_gpu_times = [], []
        fresh_calls = WARMUP_MIN + (4 * rotation if detailed else 20)
        for with_events in (False, True):
            for call in range(fresh_calls, -1, -1):  # rotating sources like the timed steps; the last call takes xs[0]
                begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                if with_events:
                    begin.record(stream)
                received = buffer.dispatch(xs[call % rotation], topk_idx=idx, weights=weights, do_expand=workload.expand,
                                           alignment=workload.alignment, zero_padding=workload.zero_padding)
                if with_events:
                    end.record(stream)
                torch.cuda.synchronize()
                if call < fresh_calls - WARMUP_MIN:
                    if with_events:
                        fresh_gpu_times.append(begin.elapsed_time(end) * 1e-3)
                    else:
                        fresh_times.append(time.perf_counter() - t0)
        handle = received.handle
        check_combined = buffer.combine(received.x, handle).x
        torch.cuda.synchronize()
        gpu_dispatched, gpu_combined = received.x.cpu(), check_combined.cpu()
        held_bytes = received.x.untyped_storage().nbytes()
        del check_combined
        n_recv, capacity = handle.layout.recv_count, handle.layout.expanded_capacity
        assignments = int(handle.layout.expert_counts.sum().item())
        d_bytes = workloads.dispatch_bytes(workload, n_recv, assignments, capacity)
        c_bytes = workloads.combine_bytes(workload, n_recv, assignments, weighted=workload.combine_weights)

        ring = [received.x, received.x.clone(), received.x.clone()]  # combine reads a two-steps-old dispatch output

        asynchronous = workload.async_op
        ring_weights = received.topk_weights if workload.combine_weights else None

        def do_dispatch(i):
            out = buffer.dispatch(xs[i % rotation], weights=weights, handle=handle, zero_padding=workload.zero_padding,
                                  async_op=asynchronous)
            if asynchronous:
                out.event.current_stream_wait()
            ring[i % 3] = out.x

        def do_combine(i):
            out = buffer.combine(ring[(i + 1) % 3], handle, weights=ring_weights, async_op=asynchronous)
            if asynchronous:
                out.event.current_stream_wait()
            return out

        def step(i):
            do_dispatch(i)
            return do_combine(i)

        def do_dispatch_hot(i):
            # the same dispatch when its source is still cache resident (one source copy, as when the
            # producer of x ran just before): reported beside the cold figure, never as `value`
            out = buffer.dispatch(xs[0], weights=weights, handle=handle, zero_padding=workload.zero_padding)
            ring[i % 3] = out.x

        def timed(fn, count, first=0):
            """(wall seconds, GPU seconds between two HIP events on the kernels' stream) of `count` calls."""
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            begin.record(stream)
            for i in range(first, first + count):
                fn(i)
            end.record(stream)
            torch.cuda.synchronize()
            return time.perf_counter() - t0, begin.elapsed_time(end) * 1e-3

        def series(fn):
            """WARMUP_MIN untimed launches, then the timed regions: lists of wall and GPU seconds."""
            timed(fn, WARMUP_MIN)
            samples = [timed(fn, launches, first=r * launches) for r in range(regions)]
            return [s[0] for s in samples], [s[1] for s in samples]

        cli = None
        if detailed:
            # the region the command line asks for: --warmup untimed steps, then exactly --steps timed
            timed(step, max(args.warmup, 0))
            cli_wall, cli_gpu = timed(step, max(1, args.steps))
            cli = {"steps": args.steps, "warmup": args.warmup,
                   "ms_per_step": round(cli_wall / max(1, args.steps) * 1e3, 5),
                   "gpu_us_per_step": round(cli_gpu / max(1, args.steps) * 1e6, 2)}
        step_wall, step_gpu = series(step)
        _, dispatch_gpu = series(do_dispatch)
        _, combine_gpu = series(do_combine)
        hot_gpu = series(do_dispatch_hot)[1] if detailed else None
        layout_us = layout_gpu_us(workload, idx) if detailed else None

    wall_us, wall_us_min = summarize(step_wall, launches)
    gpu_step_us, gpu_step_us_min = summarize(step_gpu, launches)
    d_us, d_us_min = summarize(dispatch_gpu, launches)
    c_us, c_us_min = summarize(combine_gpu, launches)
    value = (d_bytes + c_bytes) / wall_us / 1e3
    # the kernels the library routes this workload to (names as a kernel trace shows them)
    dispatch_kernel = "dispatch_ordered_kernel" if workload.expand else "dispatch_compact_kernel"
    if not workload.expand:
        combine_kernel = "combine_compact_kernel"
    else:
        combine_kernel = "combine_few_rows_kernel" if workload.topk <= 4 else "combine_rows_kernel"
    result.update(
        {
            "value": round(value, 1),
            "unit": "GB/s",
            "ms_per_step": round(wall_us * 1e-3, 5),
            "ms_per_step_min": round(wall_us_min * 1e-3, 5),
            "config": {
                "workload": workload.name,
                "description": workload.description,
                "tokens": workload.tokens,
                "hidden": workload.hidden,
                "experts": workload.experts,
                "topk": workload.topk,
                "layout": "expanded" if workload.expand else "compact",
                "alignment": workload.alignment,
                "zero_padding": workload.zero_padding,
                "received_rows": n_recv,
                "assignments": assignments,
                "expanded_capacity": capacity,
                "step": "cached-handle dispatch + combine through Buffer.dispatch / Buffer.combine"
                        + (", async_op=True with the consumer stream waiting on each completion event" if workload.async_op else "")
                        + (", combine returning the weights" if workload.combine_weights else ""),
                "rotating_source_copies": rotation,
            },
            "timing": {"warmup_launches": WARMUP_MIN, "regions": regions, "launches_per_region": launches,
                       "reported": "median over regions of the per-launch time; *_min is the fastest region"},
            "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
            "gpu_us_per_step": round(gpu_step_us, 2),
            "gpu_us_per_step_min": round(gpu_step_us_min, 2),
            "dispatch_us": round(d_us, 2),
            "dispatch_us_min": round(d_us_min, 2),
            "dispatch_GBps": round(d_bytes / d_us / 1e3, 1),
            "combine_us": round(c_us, 2),
            "combine_us_min": round(c_us_min, 2),
            "combine_GBps": round(c_bytes / c_us / 1e3, 1),
            "fresh_dispatch_us_host": round(statistics.median(fresh_times) * 1e6, 1),
            "fresh_dispatch_us_gpu": round(statistics.median(fresh_gpu_times) * 1e6, 1),
            "fresh_dispatch_held_bytes_over_used": round(held_bytes / max(1, gpu_dispatched.numel() * 2), 3),
            "dispatch_bytes": d_bytes,
            "combine_bytes": c_bytes,
            "roofline": roofline_entry(dispatch_kernel, workload.name, d_bytes, d_us, d_us_min),
            "roofline_combine": roofline_entry(combine_kernel, workload.name, c_bytes, c_us, c_us_min),
        }
    )
    if detailed:
        hot_us, hot_us_min = summarize(hot_gpu, launches)
        result["cli_region"] = cli
        result["dispatch_us_cache_resident_source"] = round(hot_us, 2)
        result["dispatch_us_cache_resident_source_min"] = round(hot_us_min, 2)
        result["fresh_dispatch_us_host_min"] = round(min(fresh_times) * 1e6, 1)
        result["layout_us_gpu_no_host_wait"] = round(layout_us, 2)
    buffer.close()
    del xs, ring, received, handle
    torch.cuda.empty_cache()
    if args.cpu_seconds > 0:
        result["cpu_baseline"], result["bit_exact_vs_oracle"] = cpu_baseline(
            workload, x_cpu, idx_cpu, w_cpu, args.cpu_seconds if detailed else min(args.cpu_seconds, 6.0),
            gpu_dispatched, gpu_combined, scalar=args.scalar_oracle)
    return result


def main():
    args = parse_args()
    if args.gpus != 1:
        log("bench.py measures one rank on ONE GPU; --gpus", args.gpus, "is not supported (no collectives are part of this path)")
        return 2

    import torch

    from nanoep_amd import workloads

    names = [HEADLINE, "mixtral", "qwen3-moe", "ep8-share", "deepseek-v3-a128", "readme-toy"] if args.workload == "all" else [args.workload]
    if any(name not in workloads.WORKLOADS for name in names):
        log("unknown workload", args.workload, "choose from", sorted(workloads.WORKLOADS), "or all")
        return 2
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)

    workload = workloads.WORKLOADS[names[0]]
    measured = measure(workload, args, device, detailed=True)
    result = {
        "metric": "dispatch+combine achieved HBM bandwidth (algorithmic bytes / wall time), "
                  f"{workload.tokens}x{workload.hidden} bf16, {workload.experts} experts top-{workload.topk}",
        "value": measured.pop("value"),
        "unit": measured.pop("unit"),
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": measured.pop("ms_per_step"),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "payload_dtype": "bf16",
        "data": "synthetic",
    }
    result.update(measured)
    failed = result.get("bit_exact_vs_oracle") is False
    if len(names) > 1:
        others = {}
        for name in names[1:]:
            log("workload", name)
            entry = measure(workloads.WORKLOADS[name], args, device, detailed=False)
            failed = failed or entry.get("bit_exact_vs_oracle") is False
            others[name] = {key: entry[key] for key in (
                "value", "unit", "ms_per_step", "dispatch_us", "dispatch_us_min", "combine_us", "combine_us_min",
                "fresh_dispatch_us_host", "roofline", "roofline_combine", "cpu_baseline", "bit_exact_vs_oracle") if key in entry}
            others[name]["config"] = {key: entry["config"][key] for key in (
                "tokens", "hidden", "experts", "topk", "layout", "alignment", "zero_padding", "rotating_source_copies")}
        result["roofline_by_workload"] = others
    if args.calibration_copy_mib > 0:
        import ctypes

        library = ctypes.CDLL(str(ROOT / "nanoep_amd" / "libnanoep_hip.so"))
        library.nanoep_copy_bytes.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        nbytes = args.calibration_copy_mib << 20
        source = torch.full((nbytes,), 3, dtype=torch.uint8, device=device)
        target = torch.empty_like(source)
        torch.cuda.synchronize()
        for _ in range(3):
            status = library.nanoep_copy_bytes(source.data_ptr(), target.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream)
            assert status == 0, status
        torch.cuda.synchronize()
        assert torch.equal(source[:4096], target[:4096])
        result["calibration_copy_bytes"] = nbytes
        del source, target
    if failed:
        log("ERROR: GPU results of a timed configuration differ from the oracle")
    print(json.dumps(result), flush=True)
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main())
