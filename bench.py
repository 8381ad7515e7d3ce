#!/usr/bin/env python3
"""Benchmark of the routed-expert hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload exl3_decode]

Workload `exl3_decode` (the configuration the metric is quoted on): the routed MoE layer of a decode step of 8
tokens: hidden 4096, 256 SwiGLU experts of intermediate 2048, sigmoid router choosing 8 experts a token, EXL3 expert
weights with one width K in {2, 3, 4} drawn per tensor (about 2.9 bits a weight), seeded synthetic tensors, bf16
activations N(0, 1). A step is one pass of the path over the batch: router projection, select (top-k, weights, job
table) and the five launches of the fused EXL3 experts, with every input already resident in HBM.

Prints ONE JSON line: tokens/s of the whole job, the roofline of the dominant kernel (the gate/up products: achieved
HBM bytes/s of its algorithmic bytes against the published 8 TB/s) and the CPU oracle timed on this box's host cores
on the same step. The oracle is used here as checker and baseline only; the measured path is the HIP library."""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
# HBM bytes of the roofline kernel's launch as rocprofv3 counted them (FETCH_SIZE + WRITE_SIZE, each scaled by what the
# same counter reads for a 1 GiB copy), for the workloads at the sizes profiled: constants of those runs (the summaries
# under profiles/ hold the commands and the counts), reported as roofline.traffic when a run has the same sizes
MEASURED_TRAFFIC_BYTES = {
    ("exl3_decode", 8): 375.1e6 + 4.2e6,
    ("exl3_linear", 1): 8.495e6 + 0.016e6,
    ("fp4_decode", 32): 1434.7e6 + 1.0e6,
    ("fp8_decode", 32): 2746.8e6 + 1.0e6,
    ("fp4_prefill", 8192): 4777.9e6 + 447.0e6,
    ("fp8_prefill", 2048): 5626.5e6 + 117.6e6,
    ("expert_join", 8192): 877.7e6 + 402.7e6,
    ("fp8_decode_block128", 64): 3713.0e6 + 2.1e6,
    ("fp8_prefill_block128", 2048): 5386.8e6 + 67.2e6,
    ("fp4_prefill_native", 8192): 5500.8e6 + 421.1e6,
    ("exl3_prefill", 4096): 2858.6e6 + 538.5e6,
    ("fp8_prefill_native", 2048): 4711.8e6 + 113.5e6,
    ("fp8_prefill_block128_native", 2048): 4693.9e6 + 67.1e6,
    ("fp4_decode_native", 32): 1434.2e6 + 1.0e6,
    ("fp8_decode_native", 32): 2746.7e6 + 1.0e6,
}
TRAFFIC_SOURCE = {
    "exl3_linear": "profiles/exl3_down_k4_thin_single_linear.md",
    "exl3_decode": "profiles/exl3_tc_products_decode8.md", "exl3_prefill": "profiles/exl3_tcp_gemm_prefill4096.md", "fp4_decode": "profiles/expert_gate_up_fp4_fp8_decode32.md",
    "fp8_decode": "profiles/expert_gate_up_fp4_fp8_decode32.md", "fp4_prefill": "profiles/wide_expert_fp4_fp8_prefill.md",
    "fp8_prefill": "profiles/wide_expert_fp4_fp8_prefill.md",
    "fp8_decode_block128": "profiles/expert_b128_fp8_block128_decode64_prefill2048.md",
    "fp8_prefill_block128": "profiles/expert_b128_fp8_block128_decode64_prefill2048.md",
    "fp4_prefill_native": "profiles/native_expert_fp4_fp8_gfx950_lane_order.md", "fp8_prefill_native": "profiles/native_expert_fp4_fp8_gfx950_lane_order.md",
    "fp8_prefill_block128_native": "profiles/native_expert_b128_gfx950_prefill2048.md",
    "fp4_decode_native": "profiles/native_expert_fp4_fp8_gfx950_lane_order.md", "fp8_decode_native": "profiles/native_expert_fp4_fp8_gfx950_lane_order.md",
}
HIDDEN, INNER, EXPERTS, PICKS, ROWS = 4096, 2048, 256, 8, 8
CONFIG = 1


def cpu_oracle_step(orc_module, x, router, matrices, widths, threads):
    """The same step on the host cores by the CPU oracle: routing (one C call), then the experts (one C call). Returns
    (seconds, output, experts)."""
    import ctypes as C
    o = orc_module
    orc, ptr = o.orc, o.ptr
    experts = np.zeros((ROWS, PICKS), dtype=np.uint32)
    weights = np.zeros((ROWS, PICKS), dtype=np.float32)
    bias = np.zeros(EXPERTS, dtype=np.float32)
    pointers = (C.c_void_p * (EXPERTS * 3))(*[m.ctypes.data for trio in matrices for m in trio])
    out = np.zeros((ROWS, HIDDEN), dtype=np.float32)
    widths8 = np.ascontiguousarray(widths.astype(np.uint8))
    start = time.perf_counter()
    orc.orc_router_route(ptr(x, o.u16p), ptr(router, o.u16p), ptr(bias, o.f32p), ROWS, HIDDEN, EXPERTS, PICKS, 1, 0, 1.5, None,
                         ptr(experts, o.u32p), ptr(weights, o.f32p))
    orc.orc_exl3_moe_layer(ptr(x, o.u16p), ROWS, HIDDEN, INNER, PICKS, ptr(experts, o.u32p), ptr(weights, o.f32p), EXPERTS,
                           pointers, ptr(widths8, o.u8p), 10.0, ptr(out, o.f32p), None, None, threads)
    return time.perf_counter() - start, out, experts


def median_seconds(run, warmup, count):
    """`run()` returns seconds: `warmup` calls unrecorded, then the median of `count`."""
    for _ in range(warmup):
        run()
    return float(np.median([run() for _ in range(count)]))


def queue_steps(card, step, count, graph):
    """`count` steps queued without waiting: launch by launch, or (graph) as replays of the step captured once with
    the backend's graph_capture, as the reference's model runs its steps."""
    if graph is None:
        for _ in range(count):
            card.run(step, wait=False)
    else:
        for _ in range(count):
            card.run_graph(graph, wait=False)


def calibrate(amd):
    """A copy of 1 GiB inside the arena (1 GiB read, 1 GiB written), five launches."""
    import ctypes as C
    amd.probe_library()
    size = 1 << 30
    card = amd.Card(3 << 30)
    source, destination = card.reserve(size), card.reserve(size)
    record = (C.c_uint64 * 3)(source, destination, size)
    launch = amd.launches_of(1)
    launch[0].kernel = card.kernel("kernel_calibrate", "arena_copy", 24)
    launch[0].grid[0], launch[0].grid[1], launch[0].grid[2] = 256 * 16, 1, 1
    launch[0].block[0], launch[0].block[1], launch[0].block[2] = 256, 1, 1
    launch[0].argument_byte_count = 24
    C.memmove(launch[0].argument, record, 24)
    times = [card.run_timed(launch)[0] for _ in range(5)]
    # the vector unit's issue rate: one wavefront a block, `waves` wavefronts a SIMD (1,024 SIMDs), eight chains a lane
    rates = {}
    kinds = ["v_mul_lo_u32", "v_sad_u8", "v_bfe_u32", "v_and_b32", "v_pk_fma_f16", "v_alignbit_b32", "v_lshrrev_b32", "v_perm_b32",
             "4 mfma_16x16x32_f16 a trip", "4 x (v_mul_lo_u32, v_sad_u8) a trip", "4 mfma with 2 of the 8 vector instructions behind each, a trip",
             "v_mfma_f32_16x16x1_4b_f32", "v_mfma_f32_32x32x16_f16 alone", "v_mfma_f32_32x32x16_f16 with 7 vector instructions behind it",
             "v_mfma_f32_32x32x16_f16 with 14 vector instructions behind it", "v_mfma_f32_32x32x16_f16 with 30 vector instructions behind it"]
    iterations, out = 20000, card.reserve(64 << 20)
    probe = amd.launches_of(1)
    probe[0].kernel = card.kernel("kernel_calibrate", "issue_rate", 16)
    probe[0].block[0], probe[0].block[1], probe[0].block[2] = 64, 1, 1
    probe[0].argument_byte_count = 16
    for waves in (2, 4, 8):
        probe[0].grid[0], probe[0].grid[1], probe[0].grid[2] = 1024 * waves, 1, 1
        for kind, name in enumerate(kinds):
            C.memmove(probe[0].argument, (C.c_uint64 * 1)(out), 8)
            trips = iterations if kind < 12 else iterations // 4
            C.memmove(C.byref(probe[0], type(probe[0]).argument.offset + 8), (C.c_uint32 * 2)(kind, trips), 8)
            card.run_timed(probe)
            microseconds = min(card.run_timed(probe)[0] for _ in range(2))
            per = 8.0 if kind < 8 or kind == 11 else 10.0 if kind >= 12 else 1.0  # instructions (or trips) a loop body
            rates["%d waves a SIMD: %s" % (waves, name)] = round(microseconds * 1e-6 * 2.4e9 / (trips * per * waves), 2)
    card.close()
    print(json.dumps({"calibrate": "arena_copy", "bytes_read": size, "bytes_written": size, "launch_us": times,
                      "GBps_read_plus_write": 2 * size / (min(times) * 1e-6) / 1e9,
                      "cycles_at_2.4GHz_a_SIMD_per_instruction_or_trip": rates}))


def fp4_decode(amd, workloads, arguments, fp8=False, prefill=False):
    """Secondary workloads (with `prefill`, the wide form: --rows defaults to 8192 tokens of FP4 weights, 2048 of FP8;
    the wide select's tiles, wide gate/up with the quantization fused, wide down, row sum; the roofline is the MFMA's): the same layer shape with the original FP4 weights (E2M1 codes, one E8M0 scale per 32
    inputs) or FP8 weights (E4M3 codes, one E8M0 scale per 32 x 32), a decode step of `--rows` tokens (32 by default):
    quantizer, router, and the four launches of the routed experts. A few distinct seeded experts are generated and laid
    at 256 distinct places of the arena."""
    import ctypes as C
    rows = arguments.rows if not prefill or arguments.rows != 32 else 2048 if fp8 else 8192
    distinct_generated = 4 if fp8 else 16
    base = workloads.SEED + ((3 if fp8 else 4) << 20)
    block128 = fp8 and arguments.block128  # float32 scales of 128 x 128 blocks and of 128 values (the usual FP8 block scaling)
    native = getattr(arguments, "native", False)  # the weights in gfx950's own lane order (a load-time re-lay-out of the same bytes)
    matrix = workloads.fp8_block128_matrix if block128 else workloads.fp8_matrix if fp8 else workloads.fp4_matrix
    trios = [[matrix(base + 16 + 3 * e + 0, INNER, HIDDEN), matrix(base + 16 + 3 * e + 1, INNER, HIDDEN),
              matrix(base + 16 + 3 * e + 2, HIDDEN, INNER)] for e in range(distinct_generated)]
    matrices = [trios[e % distinct_generated] for e in range(EXPERTS)]
    router = workloads.to_bf16(workloads.normals(base + 2, EXPERTS * HIDDEN) * 0.02).reshape(EXPERTS, HIDDEN)
    x = workloads.activations(4, rows, HIDDEN)
    card = amd.Card(((9 if fp8 else 5) << 30) + rows * (1 << 18))
    layer = amd.Fp4Layer(card, HIDDEN, INNER, EXPERTS, PICKS, rows, matrices, router_weights_bf16=router,
                         gate_up_slices=arguments.gate_up_slices, down_slices=arguments.down_slices,
                         weight_format=(amd.WEIGHT_FORMAT_E4M3_BLOCK128_GFX950 if block128 else amd.WEIGHT_FORMAT_E4M3_GFX950 if fp8 else amd.WEIGHT_FORMAT_E2M1_GFX950) if native else
                         amd.WEIGHT_FORMAT_E4M3_BLOCK128 if block128 else amd.WEIGHT_FORMAT_E4M3_SCALED if fp8 else amd.WEIGHT_FORMAT_E2M1_SCALED)
    layer.set_rows(x, rows)
    wide = layer.wide_router() if rows > 8 or prefill else None  # more than eight rows: the wide select sorts the pairs by expert
    small = wide is not None and rows <= amd.ROUTER_SORT_ROWS and not prefill  # count, place and jobs in one block
    routing = [layer.select_launch(0)[0]] if wide is None else list(wide.launches(small=small))
    routing_names = ["router_select_entry"] if wide is None else ["router_wide_select", "router_wide_small"] if small else \
        ["router_wide_select", "router_wide_count", "router_wide_place", "router_wide_jobs"]
    if prefill:
        routing, routing_names = routing[:3], routing_names[:3]  # the tiles are the place's; no job table
        experts = layer.wide_expert_launches(wide)
        parts = [layer.projection_launch()[0]] + routing + [layer.quantize_launch()[0]] + [experts[i] for i in range(len(experts))]
        names = ["router_projection"] + routing_names + ["activation_quantize", "expert_gate_up"] + \
            (["activation_quantize(hidden)"] if block128 else []) + ["expert_down", "expert_row_sum_entry"]
    else:
        experts = layer.expert_launches(wide)
        parts = [layer.projection_launch()[0]] + routing + [layer.quantize_launch()[0]] + [experts[i] for i in range(4)]
        names = ["router_projection"] + routing_names + ["activation_quantize", "expert_gate_up", "activation_quantize(hidden)",
                                                         "expert_down", "expert_row_sum_entry"]
    shared = front = None
    if arguments.site and block128:
        raise SystemExit("--site takes the reference's scaling: the shared expert's kernels read E8M0 scales of 32 values")
    if arguments.site:
        # the whole FFN site: the shared expert (three E4M3 matrices applied to every row) and the join in place of the
        # row sum (a row's routed sum, which it also stores, the shared output added, the post of the four streams)
        shared_matrices = [workloads.fp8_matrix(base + 900, INNER, HIDDEN), workloads.fp8_matrix(base + 901, INNER, HIDDEN),
                           workloads.fp8_matrix(base + 902, HIDDEN, INNER)]
        many = rows > 64
        shared = amd.SharedExpert(layer, shared_matrices, gate_up_slices=1 if many else 4, down_slices=1 if many else 2,
                                  wide_form=amd.LINEAR_INTERLEAVED_CHUNK_BLOCKS if many else amd.LINEAR_WIDE_GROUP_BLOCKS)
        site_streams = workloads.to_bf16(workloads.normals(base + 903, rows * 4 * HIDDEN)).reshape(rows, 4, HIDDEN)
        site_post, site_comb = np.ones((rows, 4), dtype=np.float32), np.full((rows, 4, 4), 0.25, dtype=np.float32)
        shared.set_site(site_streams, site_post, site_comb)
        four = shared.launches()
        if rows <= amd.LINEAR_MAXIMUM_ROWS:  # a thin step: the shared expert's down and the join in one launch
            parts = parts[:-1] + [four[i] for i in range(3)] + [shared.shared_join_launch()[0]]
            names = names[:-1] + ["trunk_gate_up", "trunk_hidden", "activation_quantize(shared)", "expert_shared_join"]
        else:
            parts = parts[:-1] + [four[i] for i in range(4)] + [shared.join_launch()[0]]
            names = names[:-1] + ["trunk_gate_up", "trunk_hidden", "activation_quantize(shared)", "trunk_down", "expert_join"]
        # and the step ahead of the router: the site's mix project and mix finish, whose hidden rows (the collapse of the
        # streams with the carried pre, normed) are the rows the router and the quantizer then read
        front = amd.SiteFront(card, rows, HIDDEN, (workloads.normals(base + 910, 24 * 4 * HIDDEN) * 0.02).reshape(24, 4 * HIDDEN),
                              [1.0, 1.0, 1.0], workloads.normals(base + 911, 24) * 0.5, workloads.to_bf16(np.ones(HIDDEN)),
                              hidden_range=amd.Range(layer.x_offset, rows * HIDDEN * 2))
        for name in ("streams", "post", "comb"):  # the join reads the post and comb the finish writes
            front.ranges[name] = shared.ranges[name]
        card.upload(front.ranges["carried_pre"].byte_offset, np.full((rows, 4), 0.25, dtype=np.float32))
        parts = [front.mix_project_launch()[0], front.site_launches()[0]] + parts
        names = ["dense_linear(mix project)", "hyper_mix_finish"] + names
    step = amd.launches_of(len(parts))
    for i, launch in enumerate(parts):
        step[i] = launch
    graph = None
    if arguments.graph:
        # the rows' quantizer reads the rows alone: a side run beside the router's launches, joined by the gate/up launch
        at = names.index("activation_quantize")
        order = [parts[at]] + parts[:at] + parts[at + 1:]
        branched = amd.launches_of(len(order))
        for i, launch in enumerate(order):
            branched[i] = launch
        branched[0].branch, branched[1].branch, branched[at + 1].branch = amd.LAUNCH_SIDE, amd.LAUNCH_RESUME, amd.LAUNCH_JOIN
        graph = card.capture(branched)
    queue_steps(card, step, arguments.warmup, graph)
    card.wait()
    device_us = card.measure(lambda: queue_steps(card, step, arguments.steps, graph))
    seconds = device_us * 1e-6
    per_launch = np.zeros(len(names))
    for _ in range(arguments.steps):
        per_launch += np.array(card.run_timed(step))
    per_launch /= arguments.steps
    if prefill:
        picks = wide.read("picks", np.dtype([("expert", "<u4"), ("route_weight", "<f4")])).reshape(rows, PICKS)
        tiles = wide.read("tiles", amd.WIDE_TILE_DTYPE)
        live = tiles[tiles["pair_count"] > 0]
        distinct = np.unique(picks["expert"])
    else:
        jobs = layer.jobs() if wide is None else wide.read("jobs", amd.JOB_DTYPE)
        live = jobs[jobs["row_count"] > 0]
        distinct = np.unique(live["expert"])
    matrix_bytes = HIDDEN * INNER + HIDDEN * INNER // 16384 * 4 if block128 else HIDDEN * INNER + HIDDEN * INNER // 1024 if fp8 else \
        HIDDEN * INNER // 2 + HIDDEN * INNER // 32
    gate_up_bytes = 2 * matrix_bytes * len(distinct)
    gate_up_us = float(per_launch[names.index("expert_gate_up")])
    down_us = float(per_launch[names.index("expert_down")])
    result = {
        "metric": "MoE layer tok/s; decode HBM GB/s & prefill MFMA % of peak, 1 GPU",
        "value": rows * arguments.steps / seconds, "unit": "tok/s", "n_gpus": 1, "steps": arguments.steps,
        "warmup": arguments.warmup, "ms_per_step": 1000.0 * seconds / arguments.steps, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "fp8 x fp8 -> f32" if fp8 else "fp4 x fp8 -> f32", "data": "synthetic",
        "config": {"workload": "%s_moe_decode: %d tokens, H 4096, 256 experts x I 2048, top-8, %s"
                               % ("fp8" if fp8 else "fp4", rows, "E4M3, f32 scales per 128x128 / per 128" if block128 else
                                  "E4M3, E8M0 scales per 32x32" if fp8 else "E2M1, E8M0 scales per 32") + (", gfx950 lane order" if native else ""),
                   "distinct_experts": int(len(distinct)), "jobs": int(len(live)),
                   "launch_us": {name: round(float(us), 2) for name, us in zip(names, per_launch)},
                   "down_GBps": matrix_bytes * len(distinct) / (down_us * 1e-6) / 1e9},
        "roofline": {"bound": "hbm", "kernel": "expert_gate_up_%s%s%d" % ("b128_" if block128 else "e4m3_" if fp8 else "", "gfx950_" if native else "", arguments.gate_up_slices),
                     "achieved": gate_up_bytes / (gate_up_us * 1e-6) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": gate_up_bytes / (gate_up_us * 1e-6) / 1e9 / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes_per_launch": int(gate_up_bytes), "launch_us": gate_up_us},
    }
    if shared is not None:
        # the join moves (pairs_per_row + 1 + 4) bf16 values in and 4 bf16 values and a float32 sum out, a value
        join_name = "expert_shared_join" if rows <= amd.LINEAR_MAXIMUM_ROWS else "expert_join"
        join_us = float(per_launch[names.index(join_name)])
        join_bytes = rows * HIDDEN * ((PICKS + 1 + 4) * 2 + 4 * 2 + 4)
        trunk_us = float(per_launch[names.index("trunk_gate_up")])
        shared_matrix_bytes = HIDDEN * INNER + HIDDEN * INNER // 1024
        result["config"]["site"] = {
            "launches": "the shared expert (E4M3 weights) and the join in place of the row sum",
            "join_us": join_us, "join_algorithmic_bytes": int(join_bytes),
            "join_GBps": None if join_name == "expert_shared_join" else join_bytes / (join_us * 1e-6) / 1e9,
            "join_frac_of_hbm_peak": None if join_name == "expert_shared_join" else join_bytes / (join_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
            "join_traffic": MEASURED_TRAFFIC_BYTES.get(("expert_join", rows)),
            "trunk_gate_up_us": trunk_us, "trunk_gate_up_GBps": 2 * shared_matrix_bytes / (trunk_us * 1e-6) / 1e9,
            "trunk_gate_up_TFLOPs": 2.0 * rows * 2 * HIDDEN * INNER / (trunk_us * 1e-6) / 1e12}
        if front is not None:
            result["config"]["site"]["launches"] = "the site's mix project and mix finish ahead of the router, the shared expert (E4M3 weights) and the join"
            result["config"]["site"]["front_us"] = float(per_launch[0] + per_launch[1])
            result["config"]["site"]["mix_project_GBps"] = 24 * 4 * HIDDEN * 4 / (float(per_launch[0]) * 1e-6) / 1e9
    key = ("%s_%s" % ("fp8" if fp8 else "fp4", "prefill" if prefill else "decode"), rows)
    if block128:
        key = (key[0] + "_block128", rows)
    if native:
        key = (key[0] + "_native", rows)
    if key in MEASURED_TRAFFIC_BYTES and (prefill or (arguments.gate_up_slices, arguments.down_slices) == (4, 2)):
        result["roofline"]["traffic"] = MEASURED_TRAFFIC_BYTES[key]
        result["roofline"]["traffic_source"] = TRAFFIC_SOURCE[key[0]] + " (counter bytes of the profiled run, not of this one)"
    if prefill:
        pairs = rows * PICKS
        gate_up_flops, down_flops = 2.0 * pairs * 2 * HIDDEN * INNER, 2.0 * pairs * HIDDEN * INNER
        achieved = gate_up_flops / (gate_up_us * 1e-6) / 1e12
        result["config"]["workload"] = result["config"]["workload"].replace("_moe_decode", "_moe_prefill")
        result["config"]["tiles"] = result["config"].pop("jobs")
        result["config"].pop("down_GBps")
        result["config"]["down_TFLOPs"] = down_flops / (down_us * 1e-6) / 1e12
        result["config"]["step_TFLOPs"] = (gate_up_flops + down_flops) / (seconds / arguments.steps) / 1e12
        # the products are MFMAs of FP8 activations (with FP4 or FP8 weights): the FP8 rate is the instruction's peak.
        # What bounds the launch is read off its arithmetic intensity against the card's balance of the two peaks.
        kernel = ("native_expert_gate_up_%s1" if native else "wide_expert_gate_up_%s1") % ("b128_" if block128 else "e4m3_" if fp8 else "")
        if gate_up_flops / gate_up_bytes >= MFMA_F8_PEAK_TFLOPS * 1e12 / (HBM_PEAK_GBS * 1e9):
            result["roofline"] = {"bound": "mfma", "kernel": kernel, "achieved": achieved, "peak": MFMA_F8_PEAK_TFLOPS, "unit": "TFLOP/s",
                                  "frac": achieved / MFMA_F8_PEAK_TFLOPS, "traffic": result["roofline"]["traffic"],
                                  "algorithmic_flops_per_launch": gate_up_flops,
                                  "launch_us": gate_up_us, **({"traffic_source": result["roofline"]["traffic_source"]}
                                                              if "traffic_source" in result["roofline"] else {})}
        else:
            result["roofline"]["kernel"] = kernel  # the matrices' bytes of the distinct experts against the memory's peak
            result["roofline"]["TFLOPs"] = achieved
            result["roofline"]["flop_per_byte"] = gate_up_flops / gate_up_bytes
    if not arguments.no_cpu:
        import _oracle as o
        threads = min(os.cpu_count() or 1, 16)
        sample = min(rows, 4)
        if front is not None:
            # one step from the site's first state: the rows are then the front's (the collapse of the streams, normed),
            # post and comb its Sinkhorn's, and the job table that step's
            shared.set_site(site_streams, site_post, site_comb)
            card.upload(front.ranges["carried_pre"].byte_offset, np.full((rows, 4), 0.25, dtype=np.float32))
            card.run(step)
            if prefill:
                picks = wide.read("picks", np.dtype([("expert", "<u4"), ("route_weight", "<f4")])).reshape(rows, PICKS)
            else:
                live = layer.jobs() if wide is None else wide.read("jobs", amd.JOB_DTYPE)
                live = live[live["row_count"] > 0]
            checked = rows if rows <= 64 else sample  # the rows the oracle's front computes
            flat = np.ascontiguousarray(site_streams[:checked].reshape(checked, -1))
            mixes = np.zeros((checked, 24), dtype=np.float32)
            assert o.orc.orc_dense_linear(1, front.constants["mix_weights"].ctypes.data_as(C.c_void_p), 24, 4 * HIDDEN, 1, 1e-20, 1.0, 1,
                                          o.ptr(flat, o.u16p), checked, mixes.ctypes.data_as(C.c_void_p)) == 0
            x, site_post, site_comb = np.zeros((rows, HIDDEN), dtype=np.uint16), np.zeros((rows, 4), dtype=np.float32), np.zeros((rows, 4, 4), dtype=np.float32)
            for r in range(checked):
                pre = np.full(4, 0.25, dtype=np.float32)
                row_hidden, row_post, row_comb = np.zeros(HIDDEN, dtype=np.uint16), np.zeros(4, dtype=np.float32), np.zeros(16, dtype=np.float32)
                o.orc.orc_hyper_mix_finish(o.ptr(np.ascontiguousarray(site_streams[r]), o.u16p), o.ptr(pre, o.f32p), o.ptr(np.ascontiguousarray(mixes[r]), o.f32p),
                                           o.ptr(front.constants["scale"], o.f32p), o.ptr(front.constants["base"], o.f32p),
                                           o.ptr(front.constants["norm_weight"], o.u16p), HIDDEN, o.ptr(row_post, o.f32p), o.ptr(row_comb, o.f32p),
                                           o.ptr(row_hidden, o.u16p))
                x[r], site_post[r], site_comb[r] = row_hidden, row_post, row_comb.reshape(4, 4)
            assert np.array_equal(card.download(layer.x_offset, rows * HIDDEN * 2, np.uint16).reshape(rows, HIDDEN)[:checked], x[:checked]), \
                "the front's rows are the oracle's bits"
        experts_of = np.zeros((rows, PICKS), dtype=np.uint32)
        weights_of = np.zeros((rows, PICKS), dtype=np.float32)
        if prefill:
            experts_of[:], weights_of[:] = picks["expert"], picks["route_weight"]
        for job in ([] if prefill else live):
            for c in range(job["row_count"]):
                experts_of.reshape(-1)[job["pair_index"][c]] = job["expert"]
                weights_of.reshape(-1)[job["pair_index"][c]] = job["route_weight"][c]
        pointers = (C.c_void_p * (EXPERTS * 3))(*[m.ctypes.data for trio in matrices for m in trio])
        want = np.zeros((sample, HIDDEN), dtype=np.float32)
        want_pairs = np.zeros((sample * PICKS, HIDDEN), dtype=np.uint16)
        start = time.perf_counter()
        # the oracle reads the reference's bytes, from which the card's native lay-out was made
        o.orc.orc_linear_moe_layer(6 if block128 else 5 if fp8 else 3, o.ptr(np.ascontiguousarray(x[:sample]), o.u16p), sample, HIDDEN, INNER, PICKS,
                                   o.ptr(np.ascontiguousarray(experts_of[:sample]), o.u32p),
                                   o.ptr(np.ascontiguousarray(weights_of[:sample]), o.f32p), EXPERTS, pointers, 10.0,
                                   o.ptr(want, o.f32p), None, o.ptr(want_pairs, o.u16p), threads)
        if shared is not None:  # the shared expert of the same sample, and the join of the two
            shared_pointers = (C.c_void_p * 3)(*[m.ctypes.data for m in shared_matrices])
            zero, one = np.zeros((sample, 1), dtype=np.uint32), np.ones((sample, 1), dtype=np.float32)
            unused, shared_want = np.zeros((sample, HIDDEN), dtype=np.float32), np.zeros((sample, HIDDEN), dtype=np.uint16)
            o.orc.orc_linear_moe_layer(5, o.ptr(np.ascontiguousarray(x[:sample]), o.u16p), sample, HIDDEN, INNER, 1, o.ptr(zero, o.u32p),
                                       o.ptr(one, o.f32p), 1, shared_pointers, 10.0, o.ptr(unused, o.f32p), None, o.ptr(shared_want, o.u16p),
                                       threads)
            want_streams = site_streams[:sample].copy()  # joined in place
            o.orc.orc_expert_join(o.ptr(want_pairs, o.u16p), o.ptr(shared_want, o.u16p), o.ptr(want_streams, o.u16p),
                                  o.ptr(site_post, o.f32p), o.ptr(site_comb, o.f32p), None, sample, PICKS, HIDDEN)
        cpu_seconds = time.perf_counter() - start
        if shared is None:
            got = layer.read("row_output", np.float32).reshape(rows, HIDDEN)[:sample]
        else:  # one step from the streams' first values
            if front is None:
                shared.set_site(site_streams, site_post, site_comb)
                card.run(step)
            got = shared.read("row_sums", np.float32).reshape(rows, HIDDEN)[:sample]
            got_streams = o.bf16_to_f32(shared.read("streams", np.uint16).reshape(rows, 4, HIDDEN)[:sample].reshape(-1)).astype(np.float64)
            wanted = o.bf16_to_f32(want_streams.reshape(-1)).astype(np.float64)
            stream_error = float(np.sqrt(np.mean((got_streams - wanted) ** 2) / np.mean(wanted ** 2)))
            assert stream_error < 2e-2, "the streams differ from the oracle's: rms %g" % stream_error
            result["config"]["site"]["streams_vs_oracle_rms_err"] = stream_error
        error = float(np.sqrt(np.mean((got - want) ** 2) / np.mean(want.astype(np.float64) ** 2)))
        assert error < 2e-2, "GPU output differs from the oracle's: rms %g" % error
        result["cpu_baseline"] = {"value": sample / cpu_seconds, "unit": "tok/s", "cores": threads, "kind": "port",
                                  "sample": "the first %d tokens of the same step by the CPU oracle" % sample,
                                  "seconds": cpu_seconds, "gpu_vs_oracle_rms_err": error}
    card.close()
    return result


MFMA_F16_PEAK_TFLOPS = 2500.0
MFMA_F8_PEAK_TFLOPS = 5000.0


def zipf_capped_load(rows, picks, experts, s):
    """Pairs an expert of rank 0, 1, ... takes when the picks of `rows` tokens follow Zipf(s) over the experts and no
    token picks an expert twice: rows . picks . pmf, the experts above `rows` held at `rows` and the rest scaled up."""
    pmf = (1.0 + np.arange(experts)) ** -s
    pmf /= pmf.sum()
    load, capped = np.zeros(experts), np.zeros(experts, dtype=bool)
    for _ in range(experts):
        free = rows * picks - rows * capped.sum()
        load = np.where(capped, rows, free * pmf / pmf[~capped].sum())
        over = (load > rows) & ~capped
        if not over.any():
            break
        capped |= over
    return load


def zipf_fitted_bias(workloads, x, router, ranks, target):
    """The router's bias under which the sigmoid router's top-k loads follow `target` (by rank): ln(target share) to begin
    with, then each expert's bias moved by the logarithm of target over realised load until the loads agree (computed
    here on the host from float32 scores: the bias is an input of the step, the loads the card realises are reported
    beside the target)."""
    scores = workloads.bf16_to_f32(x).astype(np.float32) @ workloads.bf16_to_f32(router).astype(np.float32).T
    affinities = 1.0 / (1.0 + np.exp(-scores))
    wanted = np.zeros(EXPERTS)
    wanted[ranks] = target
    bias = 0.05 * np.log(wanted / wanted.max())
    for _ in range(200):
        top = np.argpartition(-(affinities + bias[None, :]), PICKS - 1, axis=1)[:, :PICKS]
        realised = np.bincount(top.reshape(-1), minlength=EXPERTS).astype(np.float64)
        if np.abs(realised - wanted).sum() / wanted.sum() < 0.02:
            break
        bias += 0.02 * np.log(wanted / np.maximum(realised, 0.5))
    return (bias - bias.max()).astype(np.float32)


def exl3_prefill(amd, workloads, arguments):
    """Secondary workload: the EXL3 layer of the main workload for a prefill of `--rows` tokens (4096 by default), the
    router biased so that the experts' load is Zipf-skewed (s = 1.1 over a seeded permutation of the experts; the bias
    is zipf_strength x ln(pmf), scaled to the spread of the sigmoid affinities so that load, not only rank, is skewed):
    router projection, the picks of every row, and the seven launches of the prefill form (sort by expert, operands,
    gate/up GEMM with the trellis decode fused into the tile loads, activation, down GEMM, combine)."""
    rows = arguments.rows if arguments.rows != 32 else 4096
    widths, matrices, router = workloads.exl3_moe_layer(CONFIG, HIDDEN, INNER, EXPERTS)
    x = workloads.activations(2, rows, HIDDEN)
    ranks = np.argsort(workloads.uniform01(workloads.SEED + (2 << 20) + 7, EXPERTS))
    target = zipf_capped_load(rows, PICKS, EXPERTS, 1.1)  # pairs of the expert of each rank
    if arguments.zipf_strength > 0.0:
        bias = np.zeros(EXPERTS, dtype=np.float32)
        pmf = (1.0 + np.arange(EXPERTS)) ** -1.1
        bias[ranks] = (arguments.zipf_strength * np.log(pmf / pmf.max())).astype(np.float32)
    else:
        bias = zipf_fitted_bias(workloads, x, router, ranks, target)
    card = amd.Card(10 << 30)
    layer = amd.Exl3Layer(card, HIDDEN, INNER, EXPERTS, PICKS, rows, matrices, widths, router_weights_bf16=router, bias=bias,
                          affinity_kind=amd.AFFINITY_SIGMOID, route_scale=1.5, limit=10.0)
    layer.set_rows(x, rows)
    wide = layer.wide_router()
    parts = [layer.projection_launch()[0], wide.launches()[0]] + list(layer.tcp_launches(wide.ranges["picks"].byte_offset))
    step = amd.launches_of(len(parts))
    for i, launch in enumerate(parts):
        step[i] = launch
    names = ["router_projection", "router_wide_select", "exl3_tcp_count", "exl3_tcp_place", "exl3_tcp_operands", "exl3_tcp_gemm(gate/up)",
             "exl3_tcp_activate", "exl3_tcp_gemm(down)", "exl3_tcp_combine"]
    graph = card.capture(step) if arguments.graph else None
    queue_steps(card, step, arguments.warmup, graph)
    card.wait()
    device_us = card.measure(lambda: queue_steps(card, step, arguments.steps, graph))
    seconds = device_us * 1e-6
    per_launch = np.zeros(len(names))
    for _ in range(arguments.steps):
        per_launch += np.array(card.run_timed(step))
    per_launch /= arguments.steps
    pairs = rows * PICKS
    gate_up_flops, down_flops = 2.0 * pairs * 2 * HIDDEN * INNER, 2.0 * pairs * HIDDEN * INNER
    gate_up_us, down_us = float(per_launch[5]), float(per_launch[7])
    picks = wide.read("picks", np.dtype([("expert", "<u4"), ("route_weight", "<f4")])).reshape(rows, PICKS)
    counts = np.bincount(picks["expert"].reshape(-1), minlength=EXPERTS)
    achieved = gate_up_flops / (gate_up_us * 1e-6) / 1e12
    chunk = amd.EXL3_TCP_CHUNK_PAIRS
    result = {
        "metric": "MoE layer tok/s; decode HBM GB/s & prefill MFMA % of peak, 1 GPU",
        "value": rows * arguments.steps / seconds, "unit": "tok/s", "n_gpus": 1, "steps": arguments.steps,
        "warmup": arguments.warmup, "ms_per_step": 1000.0 * seconds / arguments.steps, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "exl3_moe_prefill: %d tokens, H 4096, 256 experts x I 2048, top-8, Zipf(1.1) loads (%s), %.2f bpw"
                               % (rows, "fitted bias" if arguments.zipf_strength <= 0.0 else
                                  "bias %.2f ln pmf" % arguments.zipf_strength, float(np.mean(widths))),
                   "pairs_of_the_busiest_expert": int(counts.max()), "experts_without_a_pair": int((counts == 0).sum()),
                   "zipf_target_pairs_by_rank": [int(round(v)) for v in target[[0, 1, 3, 15, 63, 255]]],
                   "realised_pairs_at_those_ranks": [int(counts[ranks[r]]) for r in (0, 1, 3, 15, 63, 255)],
                   "load_fit_total_variation": float(np.abs(counts[ranks] - target).sum() / (2.0 * target.sum())),
                   "chunks": int(((counts + chunk - 1) // chunk).sum()),
                   "launch_us": {name: round(float(us), 2) for name, us in zip(names, per_launch)},
                   "down_TFLOPs": down_flops / (down_us * 1e-6) / 1e12,
                   "step_TFLOPs": (gate_up_flops + down_flops) / (seconds / arguments.steps) / 1e12},
        "roofline": {"bound": "mfma", "kernel": "exl3_tcp_gemm (gate/up pass)", "achieved": achieved, "peak": MFMA_F16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / MFMA_F16_PEAK_TFLOPS, "traffic": None,
                     "algorithmic_flops_per_launch": gate_up_flops, "launch_us": gate_up_us},
    }
    if ("exl3_prefill", rows) in MEASURED_TRAFFIC_BYTES and arguments.zipf_strength <= 0.0:
        result["roofline"]["traffic"] = MEASURED_TRAFFIC_BYTES[("exl3_prefill", rows)]
        result["roofline"]["traffic_source"] = TRAFFIC_SOURCE["exl3_prefill"] + " (counter bytes of the profiled run, not of this one)"
    if not arguments.no_cpu:
        import ctypes as C
        import _oracle as o
        threads = min(os.cpu_count() or 1, 16)
        sample = min(rows, 8)
        experts_of = np.ascontiguousarray(picks["expert"][:sample])
        weights_of = np.ascontiguousarray(picks["route_weight"][:sample])
        pointers = (C.c_void_p * (EXPERTS * 3))(*[m.ctypes.data for trio in matrices for m in trio])
        want = np.zeros((sample, HIDDEN), dtype=np.float32)
        widths8 = np.ascontiguousarray(widths.astype(np.uint8))
        start = time.perf_counter()
        o.orc.orc_exl3_moe_layer(o.ptr(np.ascontiguousarray(x[:sample]), o.u16p), sample, HIDDEN, INNER, PICKS, o.ptr(experts_of, o.u32p),
                                 o.ptr(weights_of, o.f32p), EXPERTS, pointers, o.ptr(widths8, o.u8p), 10.0, o.ptr(want, o.f32p), None, None,
                                 threads)
        cpu_seconds = time.perf_counter() - start
        got = layer.output()[:sample]
        rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
        error = float(np.max(np.abs(got - want))) / rms
        assert error <= 4e-3, "GPU output differs from the oracle's: %g of rms" % error
        result["cpu_baseline"] = {"value": sample / cpu_seconds, "unit": "tok/s", "cores": threads, "kind": "port",
                                  "sample": "the first %d tokens of the same call by the CPU oracle, double-precision sums" % sample,
                                  "seconds": cpu_seconds, "gpu_vs_oracle_max_err_over_rms": error}
    card.close()
    return result


def exl3_decode(amd, workloads, arguments):
    """The workload the metric is quoted on (see the head of this file)."""
    widths, matrices, router = workloads.exl3_moe_layer(CONFIG, HIDDEN, INNER, EXPERTS)
    x = workloads.activations(CONFIG, ROWS, HIDDEN)
    card = amd.Card(4 << 30)
    layer = amd.Exl3Layer(card, HIDDEN, INNER, EXPERTS, PICKS, ROWS, matrices, widths, router_weights_bf16=router,
                          affinity_kind=amd.AFFINITY_SIGMOID, route_scale=1.5, limit=10.0)
    layer.set_rows(x, ROWS)
    step = amd.launches_of(2 + amd.EXL3_TC_LAUNCHES)
    step[0] = layer.projection_launch()[0]
    step[1] = layer.select_launch(0)[0]
    fused = layer.tc_launches()
    for i in range(amd.EXL3_TC_LAUNCHES):
        step[2 + i] = fused[i]
    names = ["router_projection", "router_select_entry", "exl3_tc_operands", "exl3_tc_products(gate/up)",
             "exl3_tc_activate", "exl3_tc_products(down)", "exl3_tc_combine"]

    graph = card.capture(step) if arguments.graph else None
    queue_steps(card, step, arguments.warmup, graph)
    card.wait()
    # the timed region: exactly K steps between two waits, on the card's own clock and on the host's
    host_start = time.perf_counter()
    device_us = card.measure(lambda: queue_steps(card, step, arguments.steps, graph))
    host_seconds = time.perf_counter() - host_start
    seconds = max(device_us * 1e-6, 1e-12)
    ms_per_step = 1000.0 * seconds / arguments.steps

    # per-launch durations with a device timestamp between launches, over the same K steps
    per_launch = np.zeros(len(names))
    for _ in range(arguments.steps):
        per_launch += np.array(card.run_timed(step))
    per_launch /= arguments.steps

    # what one gate/up launch reads by the algorithm: the gate and up matrices of the distinct routed experts
    jobs = layer.jobs()
    distinct = jobs[jobs["row_count"] > 0]["expert"]
    gate_up_bytes = sum(workloads.exl3_matrix_bytes(HIDDEN, INNER, int(widths[e, 0])) +
                        workloads.exl3_matrix_bytes(HIDDEN, INNER, int(widths[e, 1])) for e in distinct)
    down_bytes = sum(workloads.exl3_matrix_bytes(INNER, HIDDEN, int(widths[e, 2])) for e in distinct)
    step_bytes = gate_up_bytes + down_bytes + ROWS * HIDDEN * 2 + ROWS * HIDDEN * 4
    gate_up_us = float(per_launch[names.index("exl3_tc_products(gate/up)")])
    down_us = float(per_launch[names.index("exl3_tc_products(down)")])
    achieved = gate_up_bytes / (gate_up_us * 1e-6) / 1e9

    result = {
        "metric": "MoE layer tok/s; decode HBM GB/s & prefill MFMA % of peak, 1 GPU",
        "value": ROWS * arguments.steps / seconds,
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": arguments.steps,
        "warmup": arguments.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "exl3_moe_decode: 8 tokens, H 4096, 256 experts x I 2048, top-8 sigmoid router, EXL3 K in {2,3,4} (%.2f bpw)"
                               % float(np.mean(widths)),
                   "distinct_experts": int(len(distinct)), "step_algorithmic_bytes": int(step_bytes),
                   "step_GBps": step_bytes / seconds * arguments.steps / 1e9,
                   "host_clock_ms_per_step": 1000.0 * host_seconds / arguments.steps,
                   "launch_us": {name: round(float(us), 2) for name, us in zip(names, per_launch)},
                   "down_pass": {"launch_us": down_us, "algorithmic_bytes": int(down_bytes),
                                 "frac_of_hbm_peak": down_bytes / (down_us * 1e-6) / 1e9 / HBM_PEAK_GBS}},
        "roofline": {"bound": "hbm", "kernel": "exl3_tc_products (gate/up pass)", "achieved": achieved,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": MEASURED_TRAFFIC_BYTES[("exl3_decode", ROWS)],
                     "traffic_source": TRAFFIC_SOURCE["exl3_decode"] + " (counter bytes of the profiled run, not of this one)",
                     "algorithmic_bytes_per_launch": int(gate_up_bytes), "launch_us": gate_up_us},
    }

    got = layer.output()
    if arguments.cached_what_if:
        # how much of a products pass is memory: the five launches of the fused decode alone, with the job table as the
        # select wrote it and with every job's matrices taken from the first expert of the same width (9 matrices, which
        # the caches hold), in turns
        table = jobs.copy()
        first = {}
        for j in range(len(table)):
            if table[j]["row_count"] > 0:
                for m, name in enumerate(("gate_offset", "up_offset", "down_offset")):
                    table[j][name] = first.setdefault((m, int(widths[int(table[j]["expert"]), m])), int(table[j][name]))
        turns = {"as_routed": [], "one_expert_a_width": []}
        for _ in range(4):
            for name, which in (("as_routed", jobs), ("one_expert_a_width", table)):
                card.upload(layer.jobs_offset, which.view(np.uint8))
                for _ in range(5):
                    card.run_timed(fused)
                spent = np.zeros(amd.EXL3_TC_LAUNCHES)
                for _ in range(arguments.steps):
                    spent += np.array(card.run_timed(fused))
                turns[name].append([round(float(us), 2) for us in (spent / arguments.steps)[[1, 3]]])
        card.upload(layer.jobs_offset, jobs.view(np.uint8))
        result["config"]["cached_what_if"] = {"launch_us_gate_up_and_down_a_turn": turns, "distinct_matrices": len(first)}
    if not arguments.no_cpu:
        import _oracle
        threads = min(os.cpu_count() or 1, 16)
        outputs = []

        def one_step():
            cpu_seconds, want, experts = cpu_oracle_step(_oracle, x, router, matrices, widths, threads)
            outputs[:] = [want, experts]
            return cpu_seconds
        cpu_seconds = median_seconds(one_step, 4, 20)  # every step reads the experts' 0.55 GB anew: cold to the host's caches
        want, experts = outputs
        rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
        error = float(np.max(np.abs(got - want))) / rms
        assert sorted(set(experts.reshape(-1).tolist())) == sorted(distinct.tolist()), "expert ids differ from the oracle's"
        assert error <= 4e-3, "GPU output differs from the oracle's: %g of rms" % error
        result["cpu_baseline"] = {"value": ROWS / cpu_seconds, "unit": "tok/s", "cores": threads, "kind": "port",
                                  "sample": "the same step (8 tokens, %d experts) by the CPU oracle (routing and experts, two C calls; "
                                            "double-precision sums): 4 warm-ups, median of 20" % len(distinct),
                                  "seconds": cpu_seconds, "gpu_vs_oracle_max_err_over_rms": error}
    card.close()
    return result


def exl3_linear(amd, workloads, arguments):
    """BASELINE's configuration 0: one EXL3 linear y = (((x.suh)Hb)T)Hb.svh at 4096 x 4096, K = 4, batch 1, as the chain's
    input, product and finish launches on one job, beside the CPU oracle's same product on one host core. Algorithmic
    bytes: the stored matrix (codes, suh, svh), the bfloat16 input and the float32 output: 8,429,568."""
    import ctypes as C
    n, width = 4096, 4
    matrix = workloads.exl3_matrix(workloads.SEED, n, n, width)
    x = workloads.to_bf16(workloads.normals(workloads.SEED + 1, n))
    card = amd.Card(1 << 30)
    at = card.place(matrix, 256)
    jobs = np.zeros(1, dtype=amd.JOB_DTYPE)
    jobs[0]["gate_offset"] = jobs[0]["up_offset"] = jobs[0]["down_offset"] = at
    jobs[0]["row_count"], jobs[0]["route_weight"][0] = 1, 1.0
    record = amd.Exl3ExpertRecord()
    record.jobs_offset = card.place(jobs.view(np.uint8))
    record.input_offset = card.place(x)
    record.operands_offset = card.reserve(n * 4)
    record.products_offset = record.output_offset = card.reserve(n * 8)
    record.hidden_offset = card.reserve(n * 2)
    record.input_size = record.inner_size = n
    record.pair_count = record.pairs_per_row = record.job_count = 1
    record.bits_per_weight, record.activation_limit = width, 10.0
    launches = amd.launches_of(5)
    amd.check(card.lib.exl3_experts_prepare(C.byref(record), card.arena_bytes, amd.backend_table(), card.handle, 950, launches), "exl3_experts_prepare")
    step = amd.launches_of(3)
    step[0], step[1], step[2] = launches[0], launches[3], launches[4]  # input, the product of one matrix, finish
    step[0].grid[2] = 1
    names = ["exl3_input", "exl3_down_k4_thin", "exl3_finish"]  # one job: the product kernel of one output tile a block
    queue_steps(card, step, arguments.warmup, None)
    card.wait()
    device_us = card.measure(lambda: queue_steps(card, step, arguments.steps, None))
    per_launch = np.zeros(3)
    for _ in range(arguments.steps):
        per_launch += np.array(card.run_timed(step))
    per_launch /= arguments.steps
    seconds = device_us * 1e-6
    algorithmic = workloads.exl3_matrix_bytes(n, n, width) + n * 2 + n * 4
    product_us = float(per_launch[1])
    achieved = algorithmic / (product_us * 1e-6) / 1e9
    result = {
        "metric": "MoE layer tok/s; decode HBM GB/s & prefill MFMA % of peak, 1 GPU", "value": arguments.steps / seconds, "unit": "tok/s",
        "n_gpus": 1, "steps": arguments.steps, "warmup": arguments.warmup, "ms_per_step": 1000.0 * seconds / arguments.steps,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "exl3_linear: one matrix 4096 x 4096, K 4, batch 1 (BASELINE configuration 0)",
                   "launch_us": {name: round(float(us), 2) for name, us in zip(names, per_launch)},
                   "step_GBps": algorithmic / (seconds / arguments.steps) / 1e9},
        "roofline": {"bound": "hbm", "kernel": "exl3_down_k4_thin (the product launch)", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC_BYTES[("exl3_linear", 1)],
                     "traffic_source": TRAFFIC_SOURCE["exl3_linear"] + " (counter bytes of the profiled run, not of this one)",
                     "algorithmic_bytes_per_launch": int(algorithmic), "launch_us": product_us},
    }
    got = card.download(record.output_offset, n * 4, np.float32)
    card.close()
    if not arguments.no_cpu:
        import _oracle as o
        xs = o.bf16_to_f32(x).astype(np.float64)
        want = np.zeros(n)

        def once():
            start = time.perf_counter()
            o.orc.orc_exl3_linear_f64(o.ptr(matrix, o.u8p), n, n, width, o.ptr(xs, o.f64p), o.ptr(want, o.f64p))
            return time.perf_counter() - start
        cpu_seconds = median_seconds(once, 4, 20)
        rms = float(np.sqrt(np.mean(want ** 2)))
        error = float(np.max(np.abs(got - want))) / rms
        assert error <= 2e-3, "GPU output differs from the oracle's: %g of rms" % error
        result["cpu_baseline"] = {"value": 1.0 / cpu_seconds, "unit": "tok/s", "cores": 1, "kind": "port",
                                  "sample": "the same product by the CPU oracle (orc_exl3_linear_f64, one thread, double-precision sums): "
                                            "4 warm-ups, median of 20", "seconds": cpu_seconds, "GBps": algorithmic / cpu_seconds / 1e9,
                                  "gpu_vs_oracle_max_err_over_rms": error}
    return result


def summary(result):
    """What the default line keeps of a secondary workload."""
    roofline, config = result["roofline"], result["config"]
    keep = {"workload": config["workload"], "ms_per_step": result["ms_per_step"], "tok_s": result["value"], "steps": result["steps"],
            "kernel": roofline["kernel"], "launch_us": roofline["launch_us"], "bound": roofline["bound"], "achieved": roofline["achieved"],
            "peak": roofline["peak"], "unit": roofline["unit"], "frac": roofline["frac"]}
    for name in ("algorithmic_bytes_per_launch", "algorithmic_flops_per_launch", "TFLOPs", "flop_per_byte", "traffic", "traffic_source"):
        if name in roofline:
            keep[name] = roofline[name]
    for name in ("pairs_of_the_busiest_expert", "load_fit_total_variation", "chunks", "distinct_experts", "down_TFLOPs", "down_GBps"):
        if name in config:
            keep[name] = config[name]
    baseline = result.get("cpu_baseline", {})
    for name in ("gpu_vs_oracle_max_err_over_rms", "gpu_vs_oracle_rms_err"):
        if name in baseline:
            keep[name] = baseline[name]
    if config["workload"].startswith("exl3_linear"):
        keep["launch_us_all"] = config["launch_us"]
        keep["cpu_baseline"] = baseline
    return keep


# the workloads of the other configurations the metric names, as the default run's config.also: (workload, rows, block128, gfx950 lane order)
ALSO = [("exl3_linear", 1, False, False), ("exl3_prefill", 4096, False, False), ("fp8_decode", 1, True, False), ("fp8_decode", 64, True, False),
        ("fp8_prefill", 2048, True, False), ("fp8_prefill", 2048, True, True), ("fp8_prefill", 2048, False, False), ("fp8_prefill", 2048, False, True),
        ("fp4_prefill", 8192, False, False), ("fp4_prefill", 8192, False, True), ("fp4_decode", 32, False, False), ("fp4_decode", 32, False, True),
        # configuration 4 is reported against the FP8 run of configuration 3 on the same inputs: that scaling at its sizes
        ("fp8_prefill", 8192, True, True), ("fp8_decode", 32, True, False)]
# the other configurations' headline fractions as scalars of config (beside config.also, which holds the whole lines)
HEADLINES = {("exl3_linear", False, False): "exl3_linear_hbm_frac", ("exl3_prefill", False, False): "exl3_prefill_mfma_frac",
             ("fp8_prefill", True, False): "fp8_block128_prefill_hbm_frac", ("fp8_prefill", True, True): "fp8_block128_gfx950_prefill_hbm_frac",
             ("fp8_prefill", False, False): "fp8_prefill_hbm_frac",
             ("fp8_prefill", False, True): "fp8_gfx950_prefill_hbm_frac", ("fp4_prefill", False, False): "fp4_prefill_mfma_frac",
             ("fp4_prefill", False, True): "fp4_gfx950_prefill_mfma_frac", ("fp4_decode", False, False): "fp4_decode32_hbm_frac",
             ("fp4_decode", False, True): "fp4_gfx950_decode32_hbm_frac"}


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=200)
    parser.add_argument("--warmup", type=int, default=20)
    parser.add_argument("--workload", default="all",
                        help="all (default): exl3_decode as the line, the other configurations' workloads in config.also; or one of "
                             "exl3_decode, exl3_linear, exl3_prefill, fp4_decode, fp8_decode, fp4_prefill, fp8_prefill")
    parser.add_argument("--zipf-strength", type=float, default=0.0,
                        help="exl3_prefill: 0 (default): the router's bias is fitted so that the experts' loads follow Zipf (s = 1.1), an "
                             "expert at most one pair a token; above 0: the bias is this times ln(Zipf pmf)")
    parser.add_argument("--rows", type=int, default=32, help="tokens of a step (fp4_decode)")
    parser.add_argument("--gate-up-slices", type=int, default=4)
    parser.add_argument("--down-slices", type=int, default=2)
    parser.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    parser.add_argument("--block128", action="store_true",
                        help="fp8 workloads: float32 scales of 128 x 128 weight blocks and of 128 activation values in place of the reference's E8M0 scales")
    parser.add_argument("--native", action="store_true",
                        help="fp4 and fp8 workloads: the experts' weights in gfx950's own lane order (WEIGHT_FORMAT_E2M1_GFX950 / _E4M3_GFX950, "
                             "made from the same bytes by the library's load-time re-lay-out)")
    parser.add_argument("--cached-what-if", action="store_true",
                        help="exl3_decode: also time the fused decode's launches with every job's matrices taken from one expert of "
                             "the same width (the bytes come from the caches): what of a products pass is memory")
    parser.add_argument("--site", action="store_true",
                        help="fp4/fp8 workloads: the whole FFN site: the mix project and mix finish ahead of the router, the shared expert and the join "
                             "in place of the row sum")
    parser.add_argument("--graph", action="store_true", help="time replays of the step captured as one graph (graph_capture / graph_run)")
    parser.add_argument("--calibrate", action="store_true",
                        help="run only a 1 GiB arena copy, five times: the yardstick of the traffic counters")
    arguments = parser.parse_args()
    if arguments.gpus != 1:
        print("bench.py measures one GPU: this build holds no multi-GPU code (--gpus %d refused)" % arguments.gpus, file=sys.stderr)
        sys.exit(2)
    if arguments.workload not in ("all", "exl3_decode", "exl3_linear", "fp4_decode", "fp8_decode", "exl3_prefill", "fp4_prefill", "fp8_prefill"):
        print("unknown workload %s" % arguments.workload, file=sys.stderr)
        sys.exit(2)

    import anemone_amd as amd
    from anemone_amd import workloads

    if arguments.calibrate:
        calibrate(amd)
        return

    def run(workload, options):
        if workload == "exl3_decode":
            return exl3_decode(amd, workloads, options)
        if workload == "exl3_prefill":
            return exl3_prefill(amd, workloads, options)
        if workload == "exl3_linear":
            return exl3_linear(amd, workloads, options)
        return fp4_decode(amd, workloads, options, fp8=workload.startswith("fp8"), prefill=workload.endswith("prefill"))

    if arguments.workload != "all":
        print(json.dumps(run(arguments.workload, arguments)))
        return
    result = run("exl3_decode", arguments)
    also = []
    for workload, rows, block128, native in ALSO:
        options = argparse.Namespace(**vars(arguments))
        options.rows, options.block128, options.native, options.site, options.graph = rows, block128, native, False, False
        prefill = workload.endswith("prefill")
        options.steps, options.warmup = (min(arguments.steps, 5), min(arguments.warmup, 2)) if prefill else (min(arguments.steps, 20), min(arguments.warmup, 5))
        start = time.perf_counter()
        entry = summary(run(workload, options))
        entry["bench_seconds"] = time.perf_counter() - start
        also.append(entry)
        if (workload, block128, native) in HEADLINES and not (workload == "fp8_prefill" and rows != 2048):
            result["config"][HEADLINES[(workload, block128, native)]] = entry["frac"]
        if workload == "fp8_decode":
            result["config"]["fp8_block128_decode%d_hbm_frac" % rows] = entry["frac"]
    # the FP4 layer's steps against the FP8 layer's (float32 block scales) on the same rows: tokens a second, FP4 over FP8
    rate = {(w, r, b, n): e["tok_s"] for (w, r, b, n), e in zip(ALSO, also)}
    result["config"]["fp4_over_fp8_prefill8192_tok_s"] = rate[("fp4_prefill", 8192, False, True)] / rate[("fp8_prefill", 8192, True, True)]
    result["config"]["fp4_over_fp8_decode32_tok_s"] = rate[("fp4_decode", 32, False, True)] / rate[("fp8_decode", 32, True, False)]
    result["config"]["also"] = also
    print(json.dumps(result))


if __name__ == "__main__":
    main()
