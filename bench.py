#!/usr/bin/env python3
"""Benchmark of the paged KV-cache attention path on one MI355X.

A step is one decode layer-step over one batch of synthetic input resident in HBM:
KV append (one token per sequence) -> split-KV grouped-query decode map -> log-sum-exp combine; the
append rides in the map launch unless --separate-append is given.
Default workload: batch 32, contexts uniform in [1024, 8192], 24 Q / 4 KV heads, head_dim 256,
bf16 K/V in 16-token pages from a shuffled pool, 512-token partitions.

Prints ONE JSON line.  `value` is the achieved HBM bandwidth of the whole layer-step (algorithmic
bytes / wall time); `us_per_layer_step` is the time itself.  `roofline` prices the dominant kernel
(the split-KV map) against the 8 TB/s HBM3E peak from HIP events on the launch stream around a run of
back-to-back launches (the figure with one event pair per launch is reported next to it); `cpu_baseline`
times the scalar CPU oracle on a bounded sample of the same workload on this box's host cores.
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--batch", type=int, default=32)
    p.add_argument("--ctx-lo", type=int, default=1024)
    p.add_argument("--ctx-hi", type=int, default=8192)
    p.add_argument("--partition", type=int, default=None,
                   help="split-KV partition length in tokens (default 512; the whole context for the prefill workload)")
    p.add_argument("--arenas", type=int, default=2, help="independent page arenas rotated between steps")
    p.add_argument("--q-heads", type=int, default=24, help="decode workload: query heads (24; 16 for the long-context shape)")
    p.add_argument("--kv-heads", type=int, default=4, help="decode workload: KV heads (4; 2 for the long-context shape)")
    p.add_argument("--dtype", choices=["bf16", "f16"], default="bf16", help="K/V/Q element type (f16 for the 1 x 512 shape)")
    p.add_argument("--seed", type=int, default=2)
    p.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline sample")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--identity-pages", action="store_true", help="unshuffled page pool (diagnostic)")
    p.add_argument("--plan-order", action="store_true",
                   help="dispatch the split rows in plan order instead of longest first")
    p.add_argument("--separate-append", action="store_true",
                   help="decode workload: launch the append as its own kernel instead of folding it into the map")
    p.add_argument("--workers", type=int, default=0,
                   help="balanced plan: workers per KV head (0 = one workgroup per compute unit over all KV heads)")
    p.add_argument("--row-per-workgroup", action="store_true",
                   help="decode workload: one workgroup per partition row instead of the balanced worker plan")
    p.add_argument("--kernel-only", action="store_true", help="time only the map kernel (for profiling runs)")
    p.add_argument("--graph", action="store_true",
                   help="replay a captured HIP graph per step instead of launching its three kernels one by one "
                        "(measured slower on this stack: 133 vs 126 us per step)")
    p.add_argument("--workload", choices=["decode", "verify", "prefill"], default="decode",
                   help="decode: one new token per sequence (the headline workload); verify: --q-len tokens per "
                        "sequence through the multi-query kernels (batch 64, contexts 2048-16384 unless overridden)")
    p.add_argument("--q-len", type=int, default=2)
    p.add_argument("--prefix", type=int, default=4096, help="prefill workload: cached tokens before the chunk")
    p.add_argument("--chunk", type=int, default=2048, help="prefill workload: new tokens of the one sequence")
    p.add_argument("--no-row-groups", action="store_true",
                   help="prefill workload: one workgroup per (row, KV head) instead of the row-group map")
    p.add_argument("--calibrate-copy", action="store_true",
                   help="run only the plain copy / read probes of known size (counter calibration, practical ceiling)")
    p.add_argument("--probe-mib", type=int, default=1024)
    return p.parse_args()


def read_profile_traffic(workload_key):
    """HBM bytes per launch of the dominant kernel measured with rocprofv3 --pmc (FETCH_SIZE +
    WRITE_SIZE, scaled by the copy calibration), if a committed summary covers this workload."""
    folder = os.path.join(ROOT, "profiles")
    try:
        names = sorted(os.listdir(folder))
    except OSError:
        return None
    for name in names:
        if not name.endswith(".txt"):
            continue
        with open(os.path.join(folder, name)) as f:
            text = f.read()
        if f"workload={workload_key}" not in text:
            continue
        for line in text.splitlines():
            if line.startswith("traffic_bytes_per_launch="):
                return float(line.split("=", 1)[1])
    return None


def cpu_baseline(psi, wl, w, dw, budget_s):
    """Scalar oracle (a C restatement of the reference's sequential f32 oracle) on the first
    requests of the batch, one thread, on this box's host cores."""
    import numpy as np

    from oracle import binding as oracle

    dt = {0: oracle.F32, 1: oracle.BF16, 2: oracle.F16}[int(w.dtype)]
    pages = dw.pages_host()
    layout = (w.layout.num_req_slots, w.layout.num_gqa_layers, w.layout.num_blocks, w.layout.num_page_ids_per_block)
    es = w.dtype.item_size()

    def run(n_reqs, threads):
        cu = w.cu_tokens[: n_reqs + 1]
        t0 = time.perf_counter()
        oracle.paged_gqa(w.num_q_heads, w.num_kv_heads, w.head_dim, w.scale, w.page_bytes, dt, layout, w.layer,
                         w.req_slots[:n_reqs], w.token_indices[:n_reqs], cu, w.q[: int(cu[-1])], pages, w.page_ids,
                         num_threads=threads)
        dt_s = time.perf_counter() - t0
        ctx = int(w.context_lens[:n_reqs].astype(np.int64).sum())
        nbytes = ctx * 2 * w.num_kv_heads * w.head_dim * es + 2 * int(cu[-1]) * w.num_q_heads * w.head_dim * es
        return dt_s, nbytes

    t1, b1 = run(1, 1)
    n = int(max(1, min(len(w.req_slots), budget_s / max(t1, 1e-3))))
    t, b = (t1, b1) if n == 1 else run(n, 1)
    cores = os.cpu_count() or 1
    threads = min(cores, 16)
    tp, bp = run(n, threads)
    return {
        "value": b / t / 1e9,
        "unit": "GB/s",
        "cores": 1,
        "kind": "port",
        "sample": f"attention of the first {n} of {len(w.req_slots)} requests of the same batch "
                  f"({b / 1e6:.1f} MB algorithmic), scalar f32 oracle, {t:.2f} s",
        "us_per_layer_step_extrapolated": t * 1e6 * (w.algorithmic_bytes() / b),
        "openmp": {"value": bp / tp / 1e9, "unit": "GB/s", "cores": threads, "seconds": tp},
    }


def calibrate_copy(device, args):
    """Copies (and separately just reads) a buffer of known size with the probe kernels of
    psi-dec_amd/lib/libpsi_hip_probe.so.  Under `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` the counter value of
    these launches against the known byte count gives the scale factor applied to the attention kernels'
    counter readings."""
    import ctypes

    import torch

    probe = ctypes.CDLL(os.path.join(ROOT, "psi-dec_amd", "lib", "libpsi_hip_probe.so"))
    probe.psi_probe_copy.restype = ctypes.c_int
    probe.psi_probe_copy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int]
    nbytes = args.probe_mib << 20
    src = torch.empty(nbytes, dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    stream = ctypes.c_void_p(device.stream.cuda_stream)
    out = {"probe_bytes": nbytes, "launches": args.steps}

    def launch(read_only):
        rc = probe.psi_probe_copy(stream, dst.data_ptr(), src.data_ptr(), nbytes, int(read_only))
        if rc != 0:
            raise RuntimeError(f"psi_probe_copy failed: {rc}")

    for name, read_only in (("copy_probe", False), ("read_probe", True)):
        for _ in range(args.warmup):
            launch(read_only)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(device.stream)
        for _ in range(args.steps):
            launch(read_only)
        stop.record(device.stream)
        stop.synchronize()
        us = start.elapsed_time(stop) * 1e3 / args.steps
        moved = nbytes if read_only else 2 * nbytes
        out[name] = {"avg_launch_us": us, "bytes_moved_per_launch": moved, "GB/s": moved / (us / 1e6) / 1e9}
    print(json.dumps(out))


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {args.gpus}); the path does not shard in this build",
              file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch

    psi = importlib.import_module("psi-dec_amd")
    wl = importlib.import_module("psi-dec_amd.workloads")
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    device = psi.Device(0)
    if args.calibrate_copy:
        calibrate_copy(device, args)
        return

    verify = args.workload in ("verify", "prefill")
    prefill = args.workload == "prefill"
    if args.partition is None:
        # prefill: one kv_split row per query tile (no split of the context) measures best for a single chunk
        args.partition = max(2048, 1 << (args.prefix + args.chunk - 1).bit_length()) if prefill else 512
    if prefill:
        args.batch, args.q_len = 1, args.chunk
    if verify and args.batch == 32 and args.ctx_lo == 1024 and args.ctx_hi == 8192:
        args.batch, args.ctx_lo, args.ctx_hi = 64, 2048, 16384
    map_kernel = "tiled_q_map" if verify else "split_kv_map"
    elem = psi.Dtype.Bfloat16 if args.dtype == "bf16" else psi.Dtype.Float16
    arenas = []
    for i in range(max(1, args.arenas)):
        if verify:
            ctx = ([args.prefix + args.chunk] if prefill else
                   wl.config_c2_context_lens(args.seed, args.batch, args.ctx_lo, args.ctx_hi) + args.q_len)
            w = wl.make_workload(args.seed, ctx, 24, 4, 256, elem, 16, q_lens=args.q_len,
                                 host_pages=False, shuffle_pages=not args.identity_pages)
        else:
            ctx = wl.config_c2_context_lens(args.seed, args.batch, args.ctx_lo, args.ctx_hi) + 1
            w = wl.make_workload(args.seed, ctx, args.q_heads, args.kv_heads, 256, elem, 16,
                                 host_pages=False, shuffle_pages=not args.identity_pages)
        w.seed = args.seed + 1000 * i  # same geometry, different page contents
        arenas.append(wl.DeviceWorkload(device, w, partition_tokens=args.partition, balanced=not args.row_per_workgroup,
                                        longest_first=not args.plan_order,
                                        grouped=prefill and not args.no_row_groups,
                                        fused_append=not args.separate_append, num_workers=args.workers or None))
    w = arenas[0].w
    shape = arenas[0].shape
    step_bytes = w.algorithmic_bytes()
    map_bytes = w.map_algorithmic_bytes()

    def run_steps(n, first=0):
        for i in range(first, first + n):
            arenas[i % len(arenas)].step()

    run_steps_direct = run_steps

    def run_maps(n, first=0):
        for i in range(first, first + n):
            arenas[i % len(arenas)].map()

    # Optional: one HIP graph per arena holds the step's three launches (append, map, combine).
    graphs = []
    if args.graph and not args.kernel_only:
        main_stream = device.stream
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        try:
            with torch.cuda.stream(side):
                device.use_stream(side)
                for a in arenas:
                    a.step()
                side.synchronize()
                for a in arenas:
                    g = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(g, stream=side):
                        a.step()
                    graphs.append(g)
        finally:
            device.use_stream(main_stream)
        torch.cuda.synchronize()

        def run_steps(n, first=0):  # noqa: F811
            for i in range(first, first + n):
                graphs[i % len(graphs)].replay()

    body = run_maps if args.kernel_only else run_steps
    body(args.warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    body(args.steps)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps

    # Spread of the step time: an event on the launch stream after every step of a further run, differences between
    # neighbours (the queue stays full, so a difference is one step's device time plus its share of launch gaps).
    n_spread = min(args.steps, 100)
    body(4)
    ticks = [torch.cuda.Event(enable_timing=True) for _ in range(n_spread + 1)]
    ticks[0].record(device.stream)
    for i in range(n_spread):
        body(1, first=i)
        ticks[i + 1].record(device.stream)
    ticks[-1].synchronize()
    step_us = sorted(ticks[i].elapsed_time(ticks[i + 1]) * 1e3 for i in range(n_spread))

    def percentile(fraction):
        return step_us[min(len(step_us) - 1, int(fraction * len(step_us)))]

    # Dominant kernel, timed by HIP events on the launch stream around every map launch.
    device.set_timing(True)
    device.reset_timing()
    run_maps(min(args.steps, 100))
    map_ms, map_launches = device.kernel_time_ms(map_kernel)
    device.set_timing(False)
    map_avg_s = map_ms / max(map_launches, 1) / 1e3
    # The same launches back to back, an event on the launch stream after every 40 of them: the
    # per-launch pairs above add the record latency of two events to every launch, a group adds the gap between two
    # launches instead.  The median group is reported, so that a host-side hiccup inside one group (a profiler
    # flushing its buffers, say) does not pass for kernel time.
    group_launches = 40
    n_groups = 5 if args.steps >= 100 else 1
    run_maps(4)  # the queue is full when the first event is recorded
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(n_groups + 1)]
    marks[0].record(device.stream)
    for g in range(n_groups):
        run_maps(group_launches)
        marks[g + 1].record(device.stream)
    marks[-1].synchronize()
    group_us = [marks[g].elapsed_time(marks[g + 1]) * 1e3 / group_launches for g in range(n_groups)]
    map_back_to_back_us = sorted(group_us)[len(group_us) // 2]
    n_back_to_back = n_groups * group_launches
    map_pair_us = map_avg_s * 1e6
    # Both figures bound the kernel's own duration from above (one adds launch gaps, the other event latency); the
    # roofline uses the smaller one.  Unprofiled that is the back-to-back average, which the profiler's kernel
    # trace reproduces (End - Start per launch); under a profiler, which instruments every dispatch, the per-launch
    # pairs are the tighter bound.
    map_avg_s = min(map_back_to_back_us, map_pair_us) / 1e6
    # the other two kernels of the step, for the record
    device.set_timing(True)
    device.reset_timing()
    run_steps_direct(min(args.steps, 50))
    kernels_us = {}
    for name in ("kv_page_write", map_kernel, "tiled_q_reduce" if verify else "split_kv_reduce"):
        ms, n = device.kernel_time_ms(name)
        kernels_us[name] = ms / max(n, 1) * 1e3
    device.set_timing(False)
    achieved = map_bytes / map_avg_s / 1e9

    workload_key = (f"{'verify_q%d' % args.q_len if verify else 'decode'}_b{args.batch}_ctx{args.ctx_lo}-{args.ctx_hi}"
                    f"_{w.num_q_heads}q{w.num_kv_heads}kv_d256_{args.dtype}_p16_part{args.partition}_seed{args.seed}")
    result = {
        "metric": "decode attn achieved HBM GB/s per layer-step (B=32, ctx 1k-8k); us/layer-step alongside",
        "value": (map_bytes if args.kernel_only else step_bytes) / (ms_per_step / 1e3) / 1e9,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "us_per_layer_step": ms_per_step * 1e3,
        "us_per_layer_step_p10_median_p90": [percentile(0.1), percentile(0.5), percentile(0.9)],
        "hbm_frac_of_peak": (map_bytes if args.kernel_only else step_bytes) / (ms_per_step / 1e3) / 1e9 / HBM_PEAK_GBPS,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic",
        "config": {
            "workload": workload_key,
            "step": "map kernel only" if args.kernel_only else "kv append -> split-KV map -> LSE combine",
            "launch": "hip graph replay" if graphs else "direct launches",
            "batch": args.batch,
            "context_tokens_total": int(w.context_lens.astype(np.int64).sum()),
            "kv_splits": shape.num_sdpa_map_task_templates,
            "algorithmic_bytes_per_step": step_bytes,
            "arenas_rotated": len(arenas),
            "kernel_us_in_step": kernels_us,
            "dispatch": ("one workgroup per compute unit and KV head over equal shares of the tiles of the "
                         "512-token plan" if arenas[0].balanced else
                         "one workgroup per plan row, " + ("plan order" if args.plan_order else "longest first")),
            "append": "folded into the map launch" if arenas[0].fused_append else "separate kernel",
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "split_kv_tiled_map" if verify else "split_kv_decode_map",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "traffic": read_profile_traffic(workload_key),
            "algorithmic_bytes_per_launch": map_bytes,
            "avg_launch_us": map_avg_s * 1e6,
            "launches_timed": int(n_back_to_back if map_back_to_back_us <= map_pair_us else map_launches),
            "timing": "HIP events on the launch stream; the smaller of the two figures below",
            "back_to_back_launch_us": map_back_to_back_us,
            "event_pair_per_launch_us": map_pair_us,
        },
    }
    if prefill:
        # multi-query chunk: priced against the matrix cores as well (4 * Hq * D flops per visible (query, key) pair)
        pairs = sum(args.prefix + i + 1 for i in range(args.chunk))
        flops = 4 * w.num_q_heads * w.head_dim * pairs
        result["config"]["workload"] = f"prefill_chunk{args.chunk}_on_prefix{args.prefix}_24q4kv_d256_{args.dtype}_p16_part{args.partition}"
        result["config"]["row_groups"] = arenas[0].meta.num_row_groups
        # the chunk map is bound by the matrix cores: that is its roofline; the HBM view stays alongside
        hbm_view = result["roofline"]
        result["roofline"] = {"bound": "mfma", "kernel": "split_kv_chunk_map" if arenas[0].grouped else "split_kv_tiled_map",
                              "achieved": flops / map_avg_s / 1e12, "peak": 2500.0, "unit": "TFLOP/s",
                              "frac": flops / map_avg_s / 1e12 / 2500.0, "traffic": None, "flops_per_launch": flops,
                              "avg_launch_us": hbm_view["avg_launch_us"], "launches_timed": hbm_view["launches_timed"],
                              "timing": hbm_view["timing"], "back_to_back_launch_us": hbm_view["back_to_back_launch_us"],
                              "event_pair_per_launch_us": hbm_view["event_pair_per_launch_us"]}
        result["hbm"] = {k: hbm_view[k] for k in ("achieved", "peak", "unit", "frac", "algorithmic_bytes_per_launch")}
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(psi, wl, w, arenas[0], args.cpu_seconds)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
