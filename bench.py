#!/usr/bin/env python3
"""Benchmark of the paged KV-cache attention path on one MI355X.

A step is one attention layer-step over one batch of synthetic input resident in HBM, issued through the layer
entry (`GQA.record`): KV append -> split-KV map -> log-sum-exp combine (decode: the append rides in the map
launch).  Headline workload (`C2`): batch 32, contexts uniform in [1024, 8192], 24 Q / 4 KV heads, head_dim
256, bf16 K/V in 16-token pages from a shuffled pool, 512-token partitions re-cut into equal worker shares.

Prints ONE JSON line.  Top level = the headline workload: `value` is the achieved HBM bandwidth of the whole
layer-step (algorithmic bytes / wall time), `us_per_layer_step` the time itself; `roofline` prices the dominant
kernel (the split-KV map) against the 8 TB/s HBM3E peak from HIP events on the launch stream; `cpu_baseline` times
the scalar CPU oracle on a bounded sample of the same workload on this box's host cores (`cpu_baseline_openmp`: the
same sample on all of them).  `configs` carries the same figures for the other benchmark configurations (C1, the
headline batch with one workgroup per 512-token partition row, the headline's shape at batch 4 / 8 / 16, C3, C4 with
one, three and seven drafts, C5's decode side, its prefill chunk, and the mixed step) and for the shapes the
reference itself times (`REF_*`), each timed in this run with the same step and warm-up counts.  Every workload
also carries a `cold` figure (the first steps after set-up), every HBM roofline the read bandwidth of a bare
page stream measured in the same run, in launches of 1 GiB and in launches of the map's own size
(`measured_stream_GBps`, `frac_of_measured_stream`, `measured_stream_same_size_GBps`,
`frac_of_measured_stream_same_size`), and the matrix-core
roofline of the prefill chunk the rate of a bare matrix-instruction loop and the LDS read rates of its two operand
reads, measured in the same run (`measured_mfma_TFLOPs`, `frac_of_measured_mfma`, `measured_lds_read_GBps_per_cu`).

Clocks.  `ms_per_step` / `us_per_layer_step`: host wall clock around K queued steps, device synchronised on both
sides -- steps run back to back, as the layers of a decoder do.  `us_per_layer_step_p10_median_p90`: a HIP event
after every single step of a further run; the event between two steps keeps the next step's first kernel from
starting under the previous step's tail, so these read a few microseconds higher than the back-to-back figure.
`host_plan_us`: what the host does per step before it can launch -- metadata update, worker plan, upload -- and is
not part of the step time (the launches of step n overlap the planning of step n + 1 only if the caller
pipelines them).  Before the W warm-up steps every workload runs untimed for about 100 ms (`settle_steps_before_warmup`):
set-up, so that the clocks have settled after the arena was generated.
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
MFMA_BF16_PEAK_TFLOPS = 2500.0
CONFIG_NAMES = ["C1", "C2_rows512", "C2_b4", "C2_b8", "C2_b16", "C3", "C4_q2", "C4_q4", "C4_q8", "C4_q8_g8", "C5_decode", "C5_prefill", "PREFILL_d128",
                "PREFILL_p16k", "PREFILL_c512", "C5_mixed", "GENERIC_f32_b8"]
# The shapes the reference itself times (the only figures it publishes for these kernels, on an Apple M3 Max):
#   REF_tiled      "SplitKV TiledQ only", 40 Q / 8 KV heads, head_dim 128, 8-token pages, one request with 8 new tokens
#                  on 128 cached ones: 0.319 ms median, map + reduce (docs/qwen3_dspark_design_draft.md:1453-1458, the
#                  command at :1470-1477)
#   REF_criterion  its Criterion bench of the decode kernels, map + reduce per iteration, no recorded result: 32 / 8
#                  heads, head_dim 128, 16-token pages, contexts 128 / 1024 / 2048 / 4096 and the ragged batch
#                  7 x 128 + 1 x 4096 (crates/inference-backend-metal/benches/gqa/split_kv.rs:19-27,44)
REF_NAMES = ["REF_tiled", "REF_criterion_ctx128", "REF_criterion_ctx1024", "REF_criterion_ctx2048",
             "REF_criterion_ctx4096", "REF_criterion_ragged"]


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--only", default=None,
                   help="time one workload only: C2 (the headline), " + ", ".join(CONFIG_NAMES + REF_NAMES) +
                        ", or `custom`")
    p.add_argument("--no-configs", action="store_true", help="headline workload only")
    p.add_argument("--kernel-only", action="store_true", help="time only the map kernel (for profiling runs)")
    p.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline sample")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--seed", type=int, default=2)
    # the `custom` decode workload (and overrides of the headline's launch mode, for comparisons)
    p.add_argument("--batch", type=int, default=32)
    p.add_argument("--ctx-lo", type=int, default=1024)
    p.add_argument("--ctx-hi", type=int, default=8192)
    p.add_argument("--q-heads", type=int, default=24)
    p.add_argument("--kv-heads", type=int, default=4)
    p.add_argument("--q-len", type=int, default=1, help="custom workload: new tokens per sequence")
    p.add_argument("--head-dim", type=int, default=256, help="custom workload: head_dim")
    p.add_argument("--page-tokens", type=int, default=16, help="custom workload: tokens per page")
    p.add_argument("--dtype", choices=["bf16", "f16", "f32"], default="bf16",
                   help="custom workload: element type (f32 runs the shape-generic kernels)")
    p.add_argument("--partition", type=int, default=512)
    p.add_argument("--prefill-partition", type=int, default=0,
                   help="C5_prefill, PREFILL_d128: tokens per KV partition (0, the default: what the library's partition "
                        "planner picks - 4096 and 3072)")
    p.add_argument("--arenas", type=int, default=0, help="page arenas rotated between steps (0 = per workload)")
    p.add_argument("--identity-pages", action="store_true", help="unshuffled page pool (diagnostic)")
    p.add_argument("--plan-order", action="store_true", help="row-per-workgroup launch in plan order, not longest first")
    p.add_argument("--separate-append", action="store_true", help="decode: launch the append as its own kernel")
    p.add_argument("--workers", type=int, default=0, help="balanced plan: workers per KV head (0 = one workgroup per CU)")
    p.add_argument("--grouped", action="store_true", help="custom multi-query workload: row-group (prefill-chunk) map")
    p.add_argument("--row-per-workgroup", action="store_true", help="one workgroup per partition row, no worker plan")
    p.add_argument("--graph", action="store_true",
                   help="submit every step through the per-bucket program cache (HIP graph replay) instead of launching")
    p.add_argument("--graph-cache-counts", action="store_true",
                   help="with --graph: the cache sets the active counts with a launch of its own ahead of each program "
                        "(default: they travel with the metadata upload)")
    p.add_argument("--calibrate-copy", action="store_true",
                   help="run only the plain copy / read probes of known size (counter calibration, practical ceiling)")
    p.add_argument("--probe-mib", type=int, default=1024)
    return p.parse_args()


def read_profile_traffic(workload_key):
    """HBM bytes per launch of the dominant kernel measured with rocprofv3 --pmc (FETCH_SIZE + WRITE_SIZE, scaled by
    the copy calibration), if a committed summary under profiles/ covers this workload."""
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
        blocks = text.split("workload=")
        for block in blocks[1:]:
            if block.split()[0] != workload_key:
                continue
            for line in block.splitlines():
                if line.startswith("traffic_bytes_per_launch="):
                    return float(line.split("=", 1)[1])
    return None


class Case:
    """One workload: page arenas rotated between steps, how a step and its dominant launch are issued."""

    def __init__(self, name, key, arenas, kind, map_kernel, roof_kernel, description):
        self.name, self.key, self.arenas, self.kind = name, key, arenas, kind
        self.map_kernel, self.roof_kernel, self.description = map_kernel, roof_kernel, description
        self.flops = None  # per map launch, for MFMA-priced workloads
        self.submit_and_wait = False  # also time every step with a synchronisation after it


def build_case(psi, wl, device, name, args):
    import numpy as np

    bf16 = psi.Dtype.Bfloat16
    decode_how = dict(balanced=not args.row_per_workgroup, longest_first=not args.plan_order,
                      fused_append=not args.separate_append, num_workers=args.workers or None)
    verify_how = dict(balanced=not args.row_per_workgroup, longest_first=not args.plan_order,
                      num_workers=args.workers or None)

    def decode_case(key, ctxs, hq, hkv, dtype, partition, arenas, seed, kernel="split_kv_decode_map", d=256, p=16,
                    how=None, **kw):
        out = []
        for i in range(arenas):
            w = wl.make_workload(seed, ctxs, hq, hkv, d, dtype, p, host_pages=False,
                                 shuffle_pages=not args.identity_pages, **kw)
            w.seed = seed + 1000 * i  # same geometry, different page contents
            out.append(wl.DeviceWorkload(device, w, partition_tokens=partition, **(how or decode_how)))
        return Case(name, key, out, "decode", "split_kv_map", kernel, "kv append + split-KV map (one launch) -> LSE combine")

    def verify_case(key, ctxs, q_len, partition, arenas, seed, hq=24, hkv=4, d=256, p=16, dtype=bf16, variant=None):
        out = []
        for i in range(arenas):
            w = wl.make_workload(seed, ctxs, hq, hkv, d, dtype, p, q_lens=q_len, host_pages=False,
                                 shuffle_pages=not args.identity_pages)
            w.seed = seed + 1000 * i
            out.append(wl.DeviceWorkload(device, w, partition_tokens=partition, variant=variant, **verify_how))
        # (tiles of more than 48 query columns go to the row-group kernel, a row per group)
        wide = min(hq // hkv, 8) * min(int(np.max(q_len)), 8) > 48
        return Case(name, key, out, "verify", "tiled_q_map", "split_kv_chunk_map" if wide else "split_kv_tiled_paired_map",
                    "kv append -> multi-query split-KV map -> LSE combine")

    def map_and_reduce_only(case):
        """The reference's own benches time the map and the reduce of an attention whose K/V are already in the
        pages: the step of such a case is those two launches."""
        for dw in case.arenas:
            dw.append()  # once, so that the pages hold the new tokens' K/V
            dw.step = (lambda d: lambda: (d.map(), d.reduce()))(dw)
        case.description = "split-KV map -> LSE combine (the new tokens' K/V already in their pages)"
        case.submit_and_wait = True
        return case

    if name == "C2":
        ctx = wl.config_c2_context_lens(args.seed, 32, 1024, 8192) + 1
        key = f"decode_b32_ctx1024-8192_24q4kv_d256_bf16_p16_part{args.partition}_seed{args.seed}"
        return decode_case(key, ctx, 24, 4, bf16, args.partition, args.arenas or 2, args.seed)
    if name == "custom":
        elem = {"bf16": bf16, "f16": psi.Dtype.Float16, "f32": psi.Dtype.Float32}[args.dtype]
        d, p = args.head_dim, args.page_tokens
        ctx = wl.config_c2_context_lens(args.seed, args.batch, args.ctx_lo, args.ctx_hi) + args.q_len
        key = (f"{'decode' if args.q_len == 1 else 'verify_q%d' % args.q_len}_b{args.batch}_ctx{args.ctx_lo}-{args.ctx_hi}"
               f"_{args.q_heads}q{args.kv_heads}kv_d{d}_{args.dtype}_p{p}_part{args.partition}_seed{args.seed}")
        fast = elem != psi.Dtype.Float32 and d in (128, 256) and p >= 8 and p & (p - 1) == 0 and \
            args.q_heads // args.kv_heads <= 8
        if args.q_len == 1:
            return decode_case(key, ctx, args.q_heads, args.kv_heads, elem, args.partition, args.arenas or 2, args.seed,
                               kernel="split_kv_decode_map" if fast else "split_kv_map_generic", d=d, p=p)
        group = min(args.q_heads // args.kv_heads, 8)
        if args.grouped:
            w = wl.make_workload(args.seed, ctx, args.q_heads, args.kv_heads, d, elem, p, q_lens=args.q_len,
                                 host_pages=False)
            dw = wl.DeviceWorkload(device, w, partition_tokens=args.partition or "auto", grouped=True,
                                   variant=psi.GQASplitKVVariant.TiledQ(8, 16, group))
            key = key.replace(f"_part{args.partition}_", f"_part{dw.partition_tokens}_")
            return Case(name, key + "_grouped", [dw], "verify", "tiled_q_map", "split_kv_chunk_map",
                        "kv append -> row-group (prefill-chunk) map -> LSE combine")
        return verify_case(key, ctx, args.q_len, args.partition, args.arenas or 1, args.seed, hq=args.q_heads,
                           hkv=args.kv_heads, d=d, p=p, dtype=elem, variant=psi.GQASplitKVVariant.TiledQ(8, 16, group))
    if name == "C2_rows512":
        # the headline batch with its 512-token partitions launched as they are: one workgroup per partition row
        ctx = wl.config_c2_context_lens(args.seed, 32, 1024, 8192) + 1
        key = f"decode_b32_ctx1024-8192_24q4kv_d256_bf16_p16_part512_seed{args.seed}_row_per_workgroup"
        return decode_case(key, ctx, 24, 4, bf16, 512, args.arenas or 2, args.seed,
                           how=dict(balanced=False, longest_first=True, fused_append=not args.separate_append))
    if name in ("C2_b4", "C2_b8", "C2_b16"):
        # the headline's shape at the batch sizes of a lightly loaded server
        b = int(name[4:])
        ctx = wl.config_c2_context_lens(args.seed, b, 1024, 8192) + 1
        return decode_case(f"decode_b{b}_ctx1024-8192_24q4kv_d256_bf16_p16_part512_seed{args.seed}", ctx, 24, 4, bf16, 512,
                           args.arenas or max(2, 64 // b), args.seed)
    if name == "GENERIC_f32_b8":
        # what the shape-generic kernels cost (f32 storage, and every geometry outside the fast kernels' domain):
        # the headline's shape at batch 8 with f32 K/V
        ctx = wl.config_c2_context_lens(args.seed, 8, 1024, 8192) + 1
        return decode_case(f"decode_b8_ctx1024-8192_24q4kv_d256_f32_p16_part512_seed{args.seed}", ctx, 24, 4,
                           psi.Dtype.Float32, 512, args.arenas or 2, args.seed, kernel="split_kv_map_generic")
    if name == "REF_tiled":
        case = verify_case("ref_tiled_q8_b1_ctx128_40q8kv_d128_bf16_p8_seed7", [128 + 8], 8, 512, args.arenas or 64, 7,
                           hq=40, hkv=8, d=128, p=8, variant=psi.GQASplitKVVariant.TiledQ(8, 16, 5))
        return map_and_reduce_only(case)
    if name.startswith("REF_criterion_"):
        which = name[len("REF_criterion_"):]
        ctxs = [128] * 7 + [4096] if which == "ragged" else [int(which[3:])]
        case = decode_case(f"ref_criterion_{which}_32q8kv_d128_bf16_p16_part512_seed8", ctxs, 32, 8, bf16, 512,
                           args.arenas or 64, 8, d=128, p=16,
                           how=dict(balanced=True, longest_first=True, fused_append=False))
        return map_and_reduce_only(case)
    if name == "C1":
        # 1 MB per arena: enough arenas that a page comes back only after 300 MB of other pages went through the
        # 256 MB last-level cache
        key = "decode_b1_ctx512_16q2kv_d256_f16_p16_part512_seed1"
        return decode_case(key, [512], 16, 2, psi.Dtype.Float16, 512, args.arenas or 300, 1, input_scale=1.0 / 16.0,
                           spare_pages=0, shuffle_slots=False)
    if name == "C3":
        key = "decode_b4_ctx131072_16q2kv_d256_bf16_p16_part512_outliers1e-4_seed33"
        return decode_case(key, [131072] * 4, 16, 2, bf16, 512, args.arenas or 1, 33, outlier_rate=1e-4, outlier_sigma=8.0)
    if name in ("C4_q2", "C4_q4", "C4_q8"):
        q_len = int(name[-1])  # one draft, three drafts, or the reference's full eight-token query tile
        ctx = wl.config_c2_context_lens(4, 64, 2048, 16384) + q_len
        return verify_case(f"verify_q{q_len}_b64_ctx2048-16384_24q4kv_d256_bf16_p16_part512_seed4", ctx, q_len, 512,
                           args.arenas or 1, 4)
    if name == "C4_q8_g8":
        # the same batch with 8 heads per KV head (32 Q / 4 KV): 64 query columns per tile, more than the multi-query
        # map's pipeline holds, so the step goes through the row-group map - short chunks whose tokens times all the
        # heads fit one workgroup, walked once per KV head, with the partition the planner picks
        ctx = wl.config_c2_context_lens(4, 64, 2048, 16384) + 8
        w = wl.make_workload(4, ctx, 32, 4, 256, bf16, 16, q_lens=8, host_pages=False,
                             shuffle_pages=not args.identity_pages)
        dw = wl.DeviceWorkload(device, w, partition_tokens="auto", grouped=True,
                               variant=psi.GQASplitKVVariant.TiledQ(8, 16, 8))
        return Case(name, f"verify_q8_b64_ctx2048-16384_32q4kv_d256_bf16_p16_part{dw.partition_tokens}_planned_seed4_grouped",
                    [dw], "verify", "tiled_q_map", "split_kv_chunk_map",
                    "kv append -> row-group map (all heads of a KV head per work item) -> LSE combine")
    if name == "C5_decode":
        ctx = wl.config_c2_context_lens(5, 128, 512, 32768) + 1
        return decode_case("decode_b128_ctx512-32768_24q4kv_d256_bf16_p16_part512_seed5", ctx, 24, 4, bf16, 512,
                           args.arenas or 1, 5)
    if name == "C5_prefill":
        w = wl.make_workload(5, [4096 + 2048], 24, 4, 256, bf16, 16, q_lens=2048, host_pages=False)
        # the planner's 4096-token partitions: two rows per query tile, 192 work items of 128 KV tiles and 192 of
        # 4 to 64 that fill the end of the launch
        dw = wl.DeviceWorkload(device, w, partition_tokens=args.prefill_partition or "auto", grouped=True,
                               variant=psi.GQASplitKVVariant.TiledQ(8, 16, 6))
        case = Case(name, f"prefill_chunk2048_on_prefix4096_24q4kv_d256_bf16_p16_part{dw.partition_tokens}_seed5", [dw], "prefill",
                    "tiled_q_map", "split_kv_chunk_map", "kv append -> row-group (prefill-chunk) map -> LSE combine")
        case.flops = 4 * 24 * 256 * sum(4096 + i + 1 for i in range(2048))
        return case
    if name == "PREFILL_d128":
        # the same chunk on the geometry of the reference's published figures (Qwen3-14B: 40 Q / 8 KV heads of 128,
        # 8-token pages; gqa_split_kv_tiled_q.rs:66-76 profile (128, 8))
        w = wl.make_workload(5, [4096 + 2048], 40, 8, 128, bf16, 8, q_lens=2048, host_pages=False)
        dw = wl.DeviceWorkload(device, w, partition_tokens=args.prefill_partition or "auto", grouped=True,
                               variant=psi.GQASplitKVVariant.TiledQ(8, 16, 5))
        case = Case(name, f"prefill_chunk2048_on_prefix4096_40q8kv_d128_bf16_p8_part{dw.partition_tokens}_seed5", [dw], "prefill",
                    "tiled_q_map", "split_kv_chunk_map", "kv append -> row-group (prefill-chunk) map -> LSE combine")
        case.flops = 4 * 40 * 128 * sum(4096 + i + 1 for i in range(2048))
        return case
    if name in ("PREFILL_p16k", "PREFILL_c512"):
        # other shapes of the same model, with the partition that psi_hip_split_kv_chunk_partition_tokens picks:
        # a chunk of 2048 tokens on a 16384-token prefix, and one of 512 tokens on a 4096-token prefix
        prefix, chunk = (16384, 2048) if name == "PREFILL_p16k" else (4096, 512)
        w = wl.make_workload(5, [prefix + chunk], 24, 4, 256, bf16, 16, q_lens=chunk, host_pages=False)
        dw = wl.DeviceWorkload(device, w, partition_tokens="auto", grouped=True,
                               variant=psi.GQASplitKVVariant.TiledQ(8, 16, 6))
        case = Case(name, f"prefill_chunk{chunk}_on_prefix{prefix}_24q4kv_d256_bf16_p16_part{dw.partition_tokens}_planned_seed5",
                    [dw], "prefill", "tiled_q_map", "split_kv_chunk_map",
                    "kv append -> row-group (prefill-chunk) map -> LSE combine")
        case.flops = 4 * 24 * 256 * sum(prefix + i + 1 for i in range(chunk))
        return case
    if name == "C5_mixed":
        step = wl.MixedStep(device, wl.config_c5())
        case = Case(name, "mixed_chunk2048_on_prefix4096_plus_decode_b128_ctx512-32768_24q4kv_d256_bf16_p16_seed5",
                    [step], "mixed", None, None,
                    "chunk: kv append -> row-group map -> combine; decode: append + map (one launch) -> combine; "
                    "one arena, one page table, one stream")
        return case
    raise SystemExit(f"unknown workload {name}")


def algorithmic_bytes(case):
    a = case.arenas[0]
    return a.w.algorithmic_bytes()


def host_plan_us(psi, wl, case, repeats=15):
    """Median host time of one step's planning for the workload: metadata update (+ worker plan / dispatch order /
    row groups) and the upload of the arrays to their fixed device buffers, as the Python mirror issues it."""
    dw = case.arenas[0]
    times = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        dw.plan()
        times.append((time.perf_counter() - t0) * 1e6)
    dw.device.sync()
    return sorted(times)[len(times) // 2]


def time_case(psi, wl, device, case, args, with_spread=True):
    import torch

    arenas = case.arenas
    step_bytes = algorithmic_bytes(case)
    graph_cache = None
    if args.graph and case.kind != "mixed":
        graph_cache = psi.GQAReplayCache(device, arenas[0].gqa, max_programs=2 * len(arenas) + 2)

    def run_steps(n, first=0):
        for i in range(first, first + n):
            a = arenas[i % len(arenas)]
            if graph_cache is not None:
                inp = a.layer_input()
                inp.counts_uploaded = not args.graph_cache_counts
                graph_cache.submit(inp)
            else:
                a.step()

    def run_maps(n, first=0):
        for i in range(first, first + n):
            arenas[i % len(arenas)].map()

    kernel_only = args.kernel_only and case.kind != "mixed"
    body = run_maps if kernel_only else run_steps
    # Cold: the very first step after the arenas were set up (code objects loaded on first use, clocks wherever the
    # set-up left them), then the mean of the next K steps, before anything has settled.
    device.sync()
    t0 = time.perf_counter()
    body(1)
    device.sync()
    first_step_us = (time.perf_counter() - t0) * 1e6
    t0 = time.perf_counter()
    body(args.steps, first=1)
    device.sync()
    cold_us = (time.perf_counter() - t0) * 1e6 / args.steps
    # Set-up, not measurement: generating a workload's arena leaves the GPU's clocks unsettled for some 20 ms of
    # attention work (step times drift by 5-10 % over the first 40 steps), and an arena's first step pays for the
    # first touch of its buffers; steps of a millisecond keep speeding up for longer (C5's decode side: 1313 us per
    # step after 30 ms against 1262 us later).  Every arena is run once and the workload for at least 100 ms before
    # the W warm-up steps and the K timed ones.
    settle_steps, t_settle = 0, time.perf_counter()
    while settle_steps < len(arenas) or (time.perf_counter() - t_settle < 0.1 and settle_steps < 4000):
        body(1, first=settle_steps)
        settle_steps += 1
        if settle_steps % 8 == 0:
            device.sync()
    device.sync()
    body(args.warmup)
    device.sync()
    t0 = time.perf_counter()
    body(args.steps)
    device.sync()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    out = {"workload": case.key, "step": "map kernel only" if kernel_only else case.description,
           "us_per_layer_step": ms_per_step * 1e3, "settle_steps_before_warmup": settle_steps,
           "cold": {"first_step_us": first_step_us, "us_per_layer_step_first_k_steps": cold_us,
                    "note": "wall clock, before the settle run: the first step alone, then the mean of the next K"},
           "algorithmic_bytes_per_step": step_bytes,
           "step_GBps": step_bytes / (ms_per_step / 1e3) / 1e9,
           "step_frac_of_hbm_peak": step_bytes / (ms_per_step / 1e3) / 1e9 / HBM_PEAK_GBPS}
    if with_spread:
        n_spread = min(args.steps, 100)
        body(4)
        ticks = [torch.cuda.Event(enable_timing=True) for _ in range(n_spread + 1)]
        ticks[0].record(device.stream)
        for i in range(n_spread):
            body(1, first=i)
            ticks[i + 1].record(device.stream)
        ticks[-1].synchronize()
        step_us = sorted(ticks[i].elapsed_time(ticks[i + 1]) * 1e3 for i in range(n_spread))
        out["us_per_layer_step_p10_median_p90"] = [step_us[int(f * (len(step_us) - 1))] for f in (0.1, 0.5, 0.9)]
    if case.submit_and_wait:
        # what a bench that waits for every submission sees (the reference's Criterion bench and its `--iters`
        # diagnostics do): launch latency and the host's wake-up included
        n = min(args.steps, 100)
        device.sync()
        t0 = time.perf_counter()
        for i in range(n):
            body(1, first=i)
            device.sync()
        out["us_per_step_submit_and_wait"] = (time.perf_counter() - t0) * 1e6 / n
    if case.kind == "mixed":
        m = arenas[0]
        device.set_timing(True)
        device.reset_timing()
        run_steps(min(args.steps, 20))
        kernels = {}
        for k in ("kv_page_write", "tiled_q_map", "tiled_q_reduce", "split_kv_map", "split_kv_reduce"):
            ms, n = device.kernel_time_ms(k)
            kernels[k] = ms / max(n, 1) * 1e3
        device.set_timing(False)
        out["kernel_us_in_step"] = kernels
        # Two dominant kernels with two bounds, issued in turn: each priced against its own peak with its time
        # inside the step, and the step against the time the two peaks would allow one after the other.
        chunk_us, decode_us = kernels["tiled_q_map"], kernels["split_kv_map"]
        flops, dbytes = m.chunk_flops(), m.decode_map_bytes()
        tflops = flops / (chunk_us / 1e6) / 1e12
        gbps = dbytes / (decode_us / 1e6) / 1e9
        ideal_us = flops / (MFMA_BF16_PEAK_TFLOPS * 1e12) * 1e6 + dbytes / (HBM_PEAK_GBPS * 1e9) * 1e6
        out["roofline"] = {
            "bound": "hbm", "kernel": "split_kv_decode_map", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": gbps / HBM_PEAK_GBPS, "traffic": None, "algorithmic_bytes_per_launch": dbytes,
            "avg_launch_us": decode_us, "timing": "HIP event pairs around every launch inside the step",
            "second_kernel": {"bound": "mfma", "kernel": "split_kv_chunk_map", "achieved": tflops,
                              "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tflops / MFMA_BF16_PEAK_TFLOPS,
                              "flops_per_launch": flops, "avg_launch_us": chunk_us},
            "step_frac_of_both_peaks_in_turn": ideal_us / (ms_per_step * 1e3)}
        out["chunk_rows"] = m.chunk_meta.replay_shape().num_sdpa_map_task_templates
        out["decode_rows"] = m.decode_meta.replay_shape().num_sdpa_map_task_templates
        out["step"] = "one planning call and one layer call for the whole batch: " + case.description
        return out

    # Dominant kernel: HIP events on the launch stream around every map launch ...
    device.set_timing(True)
    device.reset_timing()
    run_maps(min(args.steps, 100))
    map_ms, map_launches = device.kernel_time_ms(case.map_kernel)
    device.set_timing(False)
    map_pair_us = map_ms / max(map_launches, 1) * 1e3
    # ... and the same launches back to back with an event after every group: a pair of events per launch adds the
    # events' own record latency to every launch, a group adds the gap between two launches instead.  The median
    # group is taken, so that a host-side hiccup inside one group does not pass for kernel time.
    est = max(map_pair_us, 1.0)
    group_launches = int(min(40, max(4, 4000.0 / est)))
    n_groups = 5 if args.steps >= 100 else (3 if args.steps >= 20 else 1)
    run_maps(4)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(n_groups + 1)]
    marks[0].record(device.stream)
    for g in range(n_groups):
        run_maps(group_launches)
        marks[g + 1].record(device.stream)
    marks[-1].synchronize()
    group_us = sorted(marks[g].elapsed_time(marks[g + 1]) * 1e3 / group_launches for g in range(n_groups))
    map_b2b_us = group_us[len(group_us) // 2]
    # Both bound the kernel's own duration from above; the roofline takes the smaller.  Unprofiled that is the
    # back-to-back average, which a profiler's kernel trace reproduces (End - Start per launch).
    map_us = min(map_b2b_us, map_pair_us)
    a0 = arenas[0]
    map_bytes = a0.w.map_algorithmic_bytes()
    device.set_timing(True)
    device.reset_timing()
    run_steps(min(args.steps, 50))
    kernels = {}
    names = ("kv_page_write", case.map_kernel, "tiled_q_reduce" if case.kind != "decode" else "split_kv_reduce")
    for k in names:
        ms, n = device.kernel_time_ms(k)
        kernels[k] = ms / max(n, 1) * 1e3
    device.set_timing(False)
    timing = {"avg_launch_us": map_us, "back_to_back_launch_us": map_b2b_us, "event_pair_per_launch_us": map_pair_us,
              "launches_timed": int(n_groups * group_launches if map_b2b_us <= map_pair_us else map_launches),
              "timing": "HIP events on the launch stream; the smaller of the back-to-back and per-launch figures"}
    achieved = map_bytes / (map_us / 1e6) / 1e9
    stream_gbps = measured_stream_gbps(device)
    # ... and in a launch that reads as many bytes as this map does (a short launch's start and end weigh more)
    same_size = (map_bytes // (16 << 20)) * (16 << 20)
    stream_same_gbps = measured_stream_gbps(device, same_size) if 0 < same_size <= 9 << 30 else None
    hbm = {"bound": "hbm", "kernel": case.roof_kernel, "achieved": achieved,
           "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
           "traffic": read_profile_traffic(case.key), "algorithmic_bytes_per_launch": map_bytes,
           "measured_stream_GBps": stream_gbps,
           "frac_of_measured_stream": achieved / stream_gbps if stream_gbps else None,
           "measured_stream_same_size_GBps": stream_same_gbps,
           "frac_of_measured_stream_same_size": achieved / stream_same_gbps if stream_same_gbps else None, **timing}
    if case.flops:
        tflops = case.flops / (map_us / 1e6) / 1e12
        rates = measured_matrix_rates(device)
        out["roofline"] = {"bound": "mfma", "kernel": case.roof_kernel, "achieved": tflops, "peak": MFMA_BF16_PEAK_TFLOPS,
                           "unit": "TFLOP/s", "frac": tflops / MFMA_BF16_PEAK_TFLOPS,
                           "traffic": read_profile_traffic(case.key), "flops_per_launch": case.flops,
                           "measured_mfma_TFLOPs": rates.get("mfma_tflops"),
                           "frac_of_measured_mfma": tflops / rates["mfma_tflops"] if rates.get("mfma_tflops") else None,
                           "measured_lds_read_GBps_per_cu": {"b128": rates.get("lds_b128"),
                                                             "b64_transposing": rates.get("lds_b64_tr")},
                           **timing}
        out["hbm_view"] = {k: hbm[k] for k in ("achieved", "peak", "unit", "frac", "algorithmic_bytes_per_launch")}
    else:
        out["roofline"] = hbm
    out["kernel_us_in_step"] = kernels
    out["kv_split_rows"] = a0.shape.num_sdpa_map_task_templates
    out["context_tokens_total"] = int(a0.w.context_lens.astype("int64").sum())
    out["dispatch"] = (("row groups of the prefill-chunk map" if a0.grouped else
                        "one workgroup per compute unit and KV head over equal shares of the plan's tiles")
                       if (a0.balanced or a0.grouped) else
                       "one workgroup per plan row, " + ("plan order" if args.plan_order else "longest first"))
    out["launch"] = "per-bucket program cache (HIP graph replay)" if graph_cache is not None else "direct launches"
    if graph_cache is not None:
        out["replay_cache_programs_recordings_replays"] = list(graph_cache.stats())
        graph_cache.close()
    return out


def cpu_baseline(psi, wl, w, dw, budget_s):
    """Scalar oracle (a C restatement of the reference's sequential f32 oracle) on the first requests of the
    batch, one thread, on this box's host cores."""
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


_STREAM_PROBE = {}


def measured_stream_gbps(device, nbytes=1 << 30):
    """Read bandwidth of a bare stream in the attention's access pattern, measured in this run: the page-stream
    probe of psi-dec_amd/lib/libpsi_hip_probe.so over `nbytes` (1 GiB unless a launch of a workload's own size is asked
    for; a multiple of 16 MiB) of scattered 64 KiB pages, 1 KiB per load through LDS, eight loads in flight per wave.
    What the HBM-bound maps could reach at best on this box, in a launch of that size."""
    import ctypes

    import torch

    key = "gbps" if nbytes == 1 << 30 else f"gbps_{nbytes}"
    if key in _STREAM_PROBE:
        return _STREAM_PROBE[key]
    try:
        probe = ctypes.CDLL(os.path.join(ROOT, "psi-dec_amd", "lib", "libpsi_hip_probe.so"))
        probe.psi_probe_page_stream.restype = ctypes.c_int
        probe.psi_probe_page_stream.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int]
        # successive launches read successive slices of at least 1 GiB in all, so that none finds its bytes in the
        # 256 MiB last-level cache (the workloads rotate their arenas for the same reason)
        copies = max(1, -(-(1 << 30) // nbytes))
        src = torch.empty(nbytes * copies, dtype=torch.uint8, device="cuda").random_(0, 255)
        stream = ctypes.c_void_p(device.stream.cuda_stream)
        best = 0.0
        for _ in range(2):
            for i in range(5):
                if probe.psi_probe_page_stream(stream, src.data_ptr() + (i % copies) * nbytes, nbytes, 8) != 0:
                    raise RuntimeError("psi_probe_page_stream failed")
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record(device.stream)
            for i in range(20):
                probe.psi_probe_page_stream(stream, src.data_ptr() + (i % copies) * nbytes, nbytes, 8)
            stop.record(device.stream)
            stop.synchronize()
            best = max(best, nbytes / (start.elapsed_time(stop) * 1e-3 / 20) / 1e9)
        del src
        torch.cuda.empty_cache()
        _STREAM_PROBE[key] = best
    except (OSError, RuntimeError) as e:  # the probe library is a measurement aid: a figure less, not a failure
        print(f"bench.py: stream probe unavailable ({e})", file=sys.stderr)
        _STREAM_PROBE[key] = None
    return _STREAM_PROBE[key]


_MATRIX_PROBE = {}


def measured_matrix_rates(device):
    """What bounds the prefill-chunk map, measured in this run with the probes of psi-dec_amd/lib/libpsi_hip_probe.so:
    the rate of back-to-back v_mfma_f32_16x16x32_bf16 from eight waves per compute unit (at the clock the chip keeps
    under that load), and the LDS read rates per compute unit of the map's two operand reads (128-bit reads of a K
    tile, transposing 64-bit reads of a V tile)."""
    import ctypes

    import torch

    if _MATRIX_PROBE:
        return _MATRIX_PROBE
    try:
        probe = ctypes.CDLL(os.path.join(ROOT, "psi-dec_amd", "lib", "libpsi_hip_probe.so"))
        probe.psi_probe_mfma_rate.restype = ctypes.c_int
        probe.psi_probe_mfma_rate.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32]
        probe.psi_probe_lds_read_rate.restype = ctypes.c_int
        probe.psi_probe_lds_read_rate.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_uint32]
        sink = torch.zeros(512, dtype=torch.float32, device="cuda")
        stream = ctypes.c_void_p(device.stream.cuda_stream)

        def timed(launch, launches=10):
            for _ in range(3):
                if launch() != 0:
                    raise RuntimeError("probe launch failed")
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record(device.stream)
            for _ in range(launches):
                launch()
            stop.record(device.stream)
            stop.synchronize()
            return start.elapsed_time(stop) * 1e-3 / launches

        iters = 2000  # about 250 us per launch, the length of the chunk map's own launches
        seconds = timed(lambda: probe.psi_probe_mfma_rate(stream, sink.data_ptr(), iters))
        _MATRIX_PROBE["mfma_tflops"] = 256 * 8 * 8 * iters * 16384 / seconds / 1e12
        for name, pattern in (("lds_b128", 0), ("lds_b64_tr", 1)):
            seconds = timed(lambda: probe.psi_probe_lds_read_rate(stream, sink.data_ptr(), pattern, 4000))
            _MATRIX_PROBE[name] = 8 * 16384 * 4000 / seconds / 1e9
    except (OSError, AttributeError, RuntimeError) as e:  # a measurement aid: a figure less, not a failure
        print(f"bench.py: matrix probes unavailable ({e})", file=sys.stderr)
        _MATRIX_PROBE["mfma_tflops"] = None
    return _MATRIX_PROBE


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
    # the ceiling of the attention kernels' access pattern: scattered 64 KiB pages, 1 KiB per load, through LDS
    probe.psi_probe_page_stream.restype = ctypes.c_int
    probe.psi_probe_page_stream.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int]
    stream_bytes = nbytes - nbytes % (1024 * 16384)
    out["page_stream_probe"] = {"bytes_read_per_launch": stream_bytes, "GB/s_by_loads_in_flight_per_wave": {}}
    for outstanding in (1, 2, 4, 8, 32):
        def launch_stream():
            rc = probe.psi_probe_page_stream(stream, src.data_ptr(), stream_bytes, outstanding)
            if rc != 0:
                raise RuntimeError(f"psi_probe_page_stream failed: {rc}")
        for _ in range(args.warmup):
            launch_stream()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(device.stream)
        for _ in range(args.steps):
            launch_stream()
        stop.record(device.stream)
        stop.synchronize()
        us = start.elapsed_time(stop) * 1e3 / args.steps
        out["page_stream_probe"]["GB/s_by_loads_in_flight_per_wave"][str(outstanding)] = stream_bytes / (us / 1e6) / 1e9
    print(json.dumps(out))


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {args.gpus}); the path does not shard in this build",
              file=sys.stderr)
        sys.exit(2)
    import torch

    psi = importlib.import_module("psi-dec_amd")
    wl = importlib.import_module("psi-dec_amd.workloads")
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    # a created stream: the program cache records by stream capture, which the null stream does not allow
    stream = torch.cuda.Stream()
    torch.cuda.set_stream(stream)
    device = psi.Device(0, stream)
    if args.calibrate_copy:
        calibrate_copy(device, args)
        return

    headline_name = args.only if args.only else "C2"
    case = build_case(psi, wl, device, headline_name, args)
    head = time_case(psi, wl, device, case, args)
    head["host_plan_us"] = host_plan_us(psi, wl, case)
    result = {
        "metric": ("decode attn achieved HBM GB/s per layer-step (B=32, ctx 1k-8k); us/layer-step alongside"
                   if headline_name == "C2" else f"attention layer-step of workload {headline_name}: achieved HBM GB/s; "
                   "us/layer-step alongside"),
        "value": head["step_GBps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["us_per_layer_step"] / 1e3,
        "us_per_layer_step": head["us_per_layer_step"],
        "us_per_layer_step_p10_median_p90": head.get("us_per_layer_step_p10_median_p90"),
        "hbm_frac_of_peak": head["step_frac_of_hbm_peak"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("f16" if headline_name == "C1" else args.dtype if headline_name == "custom" else "bf16"),
        "data": "synthetic",
        "config": {k: v for k, v in head.items() if k not in ("roofline", "step_GBps", "step_frac_of_hbm_peak",
                                                              "us_per_layer_step", "us_per_layer_step_p10_median_p90",
                                                              "hbm_view")},
        "roofline": head["roofline"],
    }
    result["config"]["arenas_rotated"] = len(case.arenas)
    result["config"]["clocks"] = {
        "ms_per_step": "host wall clock over the K queued steps, device synchronised before and after",
        "us_per_layer_step_p10_median_p90": "one HIP event after every step of a further run (adds an event per step)",
        "roofline.avg_launch_us": "HIP events on the launch stream around runs of map launches",
        "host_plan_us": "host time to plan and upload one step's metadata; not inside ms_per_step"}
    if "hbm_view" in head:
        result["hbm"] = head["hbm_view"]
    if not args.no_cpu_baseline and case.kind != "mixed":
        result["cpu_baseline"] = cpu_baseline(psi, wl, case.arenas[0].w, case.arenas[0], args.cpu_seconds)
        result["cpu_baseline_openmp"] = dict(result["cpu_baseline"]["openmp"], kind="port",
                                             sample=result["cpu_baseline"]["sample"].split(", scalar")[0] +
                                             ", the same oracle with OpenMP over (token, head) rows")
    del case, head
    torch.cuda.empty_cache()
    if not args.only and not args.no_configs and not args.kernel_only:
        configs = {}
        for name in CONFIG_NAMES + REF_NAMES:
            c = build_case(psi, wl, device, name, args)
            r = time_case(psi, wl, device, c, args)
            r["host_plan_us"] = host_plan_us(psi, wl, c)
            r["arenas_rotated"] = len(c.arenas)
            configs[name] = r
            del c
            torch.cuda.empty_cache()
        result["configs"] = configs
    print(json.dumps(result))


if __name__ == "__main__":
    main()
