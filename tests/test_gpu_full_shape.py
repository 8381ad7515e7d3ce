"""GPU parity at the full shape of the benchmark's configurations (hidden 4096, intermediate 2048, 256 experts, 8 picks a
token), through the C ABI, against the CPU oracle on a sample of rows: the fused EXL3 decode at 8 rows, the EXL3 prefill
at 4096 rows (every sorted place, the first and last rows' outputs), the wide FP4 experts at 8192 rows and the wide FP8
experts at 2048 rows in both scalings. The smaller shapes of the other test files cover the edge cases; these cover the
indexing of the sizes that are measured."""
import ctypes as C
import sys

import numpy as np
import pytest

import _oracle as o

pytestmark = pytest.mark.gpu

HIDDEN, INNER, EXPERTS, PICKS = 4096, 2048, 256, 8


def say(*words):
    print(*words, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def amd():
    import anemone_amd
    return anemone_amd


@pytest.fixture(scope="module")
def workloads():
    from anemone_amd import workloads
    return workloads


@pytest.fixture(scope="module")
def exl3_layer_tensors(workloads):
    return workloads.exl3_moe_layer(1, HIDDEN, INNER, EXPERTS)


def exl3_oracle_rows(x_rows, experts, weights, matrices, widths, limit=10.0, threads=16):
    rows = x_rows.shape[0]
    pointers = (C.c_void_p * (EXPERTS * 3))(*[m.ctypes.data for trio in matrices for m in trio])
    out = np.zeros((rows, HIDDEN), dtype=np.float32)
    widths8 = np.ascontiguousarray(widths.astype(np.uint8))
    o.orc.orc_exl3_moe_layer(o.ptr(np.ascontiguousarray(x_rows), o.u16p), rows, HIDDEN, INNER, PICKS,
                             o.ptr(np.ascontiguousarray(experts), o.u32p), o.ptr(np.ascontiguousarray(weights), o.f32p), EXPERTS,
                             pointers, o.ptr(widths8, o.u8p), limit, o.ptr(out, o.f32p), None, None, threads)
    return out


def test_fused_decode_of_eight_rows(amd, workloads, exl3_layer_tensors):
    say("full shape: fused EXL3 decode, 8 rows")
    widths, matrices, router = exl3_layer_tensors
    rows = 8
    x = workloads.activations(1, rows, HIDDEN)
    card = amd.Card(4 << 30)
    try:
        layer = amd.Exl3Layer(card, HIDDEN, INNER, EXPERTS, PICKS, rows, matrices, widths, router_weights_bf16=router,
                              affinity_kind=amd.AFFINITY_SIGMOID, route_scale=1.5, limit=10.0)
        layer.set_rows(x, rows)
        card.run(layer.projection_launch())
        card.run(layer.select_launch(0))
        card.run(layer.tc_launches())
        got, jobs = layer.output(), layer.jobs()
    finally:
        card.close()
    experts, weights = np.zeros((rows, PICKS), np.uint32), np.zeros((rows, PICKS), np.float32)
    bias = np.zeros(EXPERTS, np.float32)
    o.orc.orc_router_route(o.ptr(x, o.u16p), o.ptr(router, o.u16p), o.ptr(bias, o.f32p), rows, HIDDEN, EXPERTS, PICKS, 1, 0, 1.5, None,
                           o.ptr(experts, o.u32p), o.ptr(weights, o.f32p))
    want_jobs = np.zeros(rows * PICKS, dtype=o.JOB_DTYPE)
    o.orc.orc_router_jobs(o.ptr(experts, o.u32p), o.ptr(weights, o.f32p), PICKS, rows, rows, EXPERTS,
                          o.ptr(np.ascontiguousarray(layer.expert_offsets.reshape(-1)), o.u64p), want_jobs.ctypes.data)
    assert jobs.tobytes() == want_jobs.tobytes(), "the job table is the oracle's, byte for byte"
    want = exl3_oracle_rows(x, experts, weights, matrices, widths)
    error = float(np.max(np.abs(got - want)) / np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    say("  max error %.2e of the output's rms" % error)
    assert error <= 4e-3


def test_prefill_of_4096_rows(amd, workloads, exl3_layer_tensors):
    say("full shape: EXL3 prefill, 4096 rows")
    widths, matrices, router = exl3_layer_tensors
    rows = 4096
    x = workloads.activations(2, rows, HIDDEN)
    bias = (-0.05 * 1.1 * np.log(1.0 + np.arange(EXPERTS))).astype(np.float32)  # skewed loads: runs of many chunks and of few pairs
    card = amd.Card(10 << 30)
    try:
        layer = amd.Exl3Layer(card, HIDDEN, INNER, EXPERTS, PICKS, rows, matrices, widths, router_weights_bf16=router, bias=bias,
                              affinity_kind=amd.AFFINITY_SIGMOID, route_scale=1.5, limit=10.0)
        layer.set_rows(x, rows)
        card.run(layer.projection_launch())
        wide = layer.wide_router()
        card.run(wide.launches()[0:1])
        card.run(layer.tcp_launches(wide.ranges["picks"].byte_offset))
        picks = wide.read("picks", np.dtype([("expert", "<u4"), ("route_weight", "<f4")])).reshape(rows, PICKS)
        layout = layer.tcp_layout
        pairs = rows * PICKS
        sorted_pairs = card.download(layer.tcp_workspace_offset + layout["sorted"], pairs * 4, np.uint32)
        place_of = card.download(layer.tcp_workspace_offset + layout["place_of"], pairs * 4, np.uint32)
        used = int(card.download(layer.tcp_workspace_offset + layout["header"], 4, np.uint32)[0])
        chunks = card.download(layer.tcp_workspace_offset + layout["chunks"], layout["chunk_capacity"] * 16, np.uint32).reshape(-1, 4)
        got = layer.output()
    finally:
        card.close()
    experts = np.ascontiguousarray(picks["expert"])
    weights = np.ascontiguousarray(picks["route_weight"])
    # the picks of the sampled rows are the oracle's (ids and weight bits)
    sample = np.array([0, 1, 2, 3, rows - 4, rows - 3, rows - 2, rows - 1])
    want_experts, want_weights = np.zeros((len(sample), PICKS), np.uint32), np.zeros((len(sample), PICKS), np.float32)
    o.orc.orc_router_route(o.ptr(np.ascontiguousarray(x[sample]), o.u16p), o.ptr(router, o.u16p), o.ptr(bias, o.f32p), len(sample), HIDDEN, EXPERTS,
                           PICKS, 1, 0, 1.5, None, o.ptr(want_experts, o.u32p), o.ptr(want_weights, o.f32p))
    assert np.array_equal(experts[sample], want_experts) and weights[sample].tobytes() == want_weights.tobytes()
    # every sorted place: by expert, rows ascending; chunks of one expert, none longer than the GEMM's columns
    assert np.array_equal(sorted_pairs, np.argsort(experts.reshape(-1), kind="stable").astype(np.uint32))
    assert np.array_equal(place_of[sorted_pairs], np.arange(pairs, dtype=np.uint32))
    counts = np.bincount(experts.reshape(-1), minlength=EXPERTS)
    most = amd.EXL3_TCP_CHUNK_PAIRS
    assert used == int(((counts + most - 1) // most).sum()) and not chunks[used:].any()
    assert int(chunks[:used, 2].sum()) == pairs and chunks[:used, 2].max() <= most
    say("  %d chunks, the busiest expert %d pairs, %d experts idle" % (used, counts.max(), (counts == 0).sum()))
    want = exl3_oracle_rows(x[sample], experts[sample], weights[sample], matrices, widths)
    error = float(np.max(np.abs(got[sample] - want)) / np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    say("  max error of the first and last four rows %.2e of rms" % error)
    assert error <= 4e-3


WIDE_RESULTS = {}  # form -> (picks, row outputs, hidden codes): a lay-out's run is kept for the other lay-out's comparison


def run_wide_form(amd, workloads, form, rows):
    if form in WIDE_RESULTS:
        return WIDE_RESULTS[form]
    fp8, block128, native = form.startswith("fp8"), form.startswith("fp8_block128"), form.endswith("_gfx950")
    distinct_generated = 4 if fp8 else 16
    base = workloads.SEED + ((3 if fp8 else 4) << 20)
    matrix = workloads.fp8_block128_matrix if block128 else workloads.fp8_matrix if fp8 else workloads.fp4_matrix
    trios = [[matrix(base + 16 + 3 * e + 0, INNER, HIDDEN), matrix(base + 16 + 3 * e + 1, INNER, HIDDEN),
              matrix(base + 16 + 3 * e + 2, HIDDEN, INNER)] for e in range(distinct_generated)]
    matrices = [trios[e % distinct_generated] for e in range(EXPERTS)]
    router = workloads.to_bf16(workloads.normals(base + 2, EXPERTS * HIDDEN) * 0.02).reshape(EXPERTS, HIDDEN)
    x = workloads.activations(4, rows, HIDDEN)
    weight_format = (amd.WEIGHT_FORMAT_E4M3_BLOCK128_GFX950 if block128 else amd.WEIGHT_FORMAT_E4M3_GFX950 if fp8 else amd.WEIGHT_FORMAT_E2M1_GFX950) if native else \
        amd.WEIGHT_FORMAT_E4M3_BLOCK128 if block128 else amd.WEIGHT_FORMAT_E4M3_SCALED if fp8 else amd.WEIGHT_FORMAT_E2M1_SCALED
    card = amd.Card(((9 if fp8 else 5) << 30) + rows * (1 << 18))
    try:
        layer = amd.Fp4Layer(card, HIDDEN, INNER, EXPERTS, PICKS, rows, matrices, router_weights_bf16=router, gate_up_slices=4, down_slices=2,
                             weight_format=weight_format)
        layer.set_rows(x, rows)
        wide = layer.wide_router()
        experts_launches = layer.wide_expert_launches(wide)
        card.run(layer.projection_launch())
        card.run(wide.launches()[0:3])
        card.run(layer.quantize_launch())
        card.run(experts_launches)
        picks = wide.read("picks", np.dtype([("expert", "<u4"), ("route_weight", "<f4")])).reshape(rows, PICKS)
        got = layer.read("row_output", np.float32).reshape(rows, HIDDEN)
        hidden_codes = layer.read("hidden_codes").copy()
    finally:
        card.close()
    WIDE_RESULTS[form] = (x, matrices, picks, got, hidden_codes)
    return WIDE_RESULTS[form]


@pytest.mark.parametrize("form,rows", [("fp4", 8192), ("fp8", 2048), ("fp8_block128", 2048), ("fp4_gfx950", 8192), ("fp8_gfx950", 2048),
                                       ("fp8_block128_gfx950", 2048)])
def test_wide_experts_of_the_original_weights(amd, workloads, form, rows):
    say("full shape: wide", form, rows, "rows")
    fp8, block128, native = form.startswith("fp8"), form.startswith("fp8_block128"), form.endswith("_gfx950")
    x, matrices, picks, got, hidden_codes = run_wide_form(amd, workloads, form, rows)
    if native:
        # gfx950's lay-out of the same matrices: every byte the launches write is the reference lay-out's (the same sums)
        _, _, want_picks, want, want_codes = run_wide_form(amd, workloads, form[:-len("_gfx950")], rows)
        assert want_picks.tobytes() == picks.tobytes()
        assert got.tobytes() == want.tobytes(), "the row outputs differ from the reference lay-out's"
        assert hidden_codes.tobytes() == want_codes.tobytes(), "the hidden codes differ from the reference lay-out's"
    sample = np.array([0, 1, 2, rows // 2, rows - 3, rows - 2, rows - 1])
    experts = np.ascontiguousarray(picks["expert"][sample])
    weights = np.ascontiguousarray(picks["route_weight"][sample])
    pointers = (C.c_void_p * (EXPERTS * 3))(*[m.ctypes.data for trio in matrices for m in trio])  # the reference's bytes: the re-lay-out's source
    want = np.zeros((len(sample), HIDDEN), dtype=np.float32)
    o.orc.orc_linear_moe_layer(6 if block128 else 5 if fp8 else 3, o.ptr(np.ascontiguousarray(x[sample]), o.u16p), len(sample), HIDDEN, INNER, PICKS,
                               o.ptr(experts, o.u32p), o.ptr(weights, o.f32p), EXPERTS, pointers, 10.0, o.ptr(want, o.f32p), None, None, 16)
    error = float(np.sqrt(np.mean((got[sample] - want) ** 2) / np.mean(want.astype(np.float64) ** 2)))
    say("  rms error of the sampled rows %.2e" % error)
    assert error <= 2e-2
    assert np.all(np.isfinite(got)) and float(np.abs(got).max()) < 1e4, "every row of the step is written and bounded"


@pytest.mark.parametrize("form,rows", [("fp8_block128", 1), ("fp8_block128", 64), ("fp4", 32)])
def test_job_table_experts_of_the_original_weights(amd, workloads, form, rows):
    """The decode form (the router's job table, expert_gate_up_<S> / expert_down_<S> with the K slices of the measured runs)
    at the full shape: 1 and 64 rows of FP8 with float32 block scales, 32 rows of FP4; four sampled rows against the
    oracle's layer."""
    say("full shape: job-table", form, rows, "rows")
    fp8 = form != "fp4"
    distinct_generated = 4 if fp8 else 16
    base = workloads.SEED + ((3 if fp8 else 4) << 20)
    matrix = workloads.fp8_block128_matrix if fp8 else workloads.fp4_matrix
    trios = [[matrix(base + 16 + 3 * e + 0, INNER, HIDDEN), matrix(base + 16 + 3 * e + 1, INNER, HIDDEN),
              matrix(base + 16 + 3 * e + 2, HIDDEN, INNER)] for e in range(distinct_generated)]
    matrices = [trios[e % distinct_generated] for e in range(EXPERTS)]
    router = workloads.to_bf16(workloads.normals(base + 2, EXPERTS * HIDDEN) * 0.02).reshape(EXPERTS, HIDDEN)
    x = workloads.activations(4, rows, HIDDEN)
    card = amd.Card(((9 if fp8 else 5) << 30) + rows * (1 << 18))
    try:
        layer = amd.Fp4Layer(card, HIDDEN, INNER, EXPERTS, PICKS, rows, matrices, router_weights_bf16=router, gate_up_slices=4, down_slices=2,
                             weight_format=amd.WEIGHT_FORMAT_E4M3_BLOCK128 if fp8 else amd.WEIGHT_FORMAT_E2M1_SCALED)
        layer.set_rows(x, rows)
        wide = layer.wide_router() if rows > 8 else None
        routing = layer.select_launch(0) if wide is None else wide.launches(small=True)
        experts_launches = layer.expert_launches(wide)
        card.run(layer.projection_launch())
        card.run(routing)
        card.run(layer.quantize_launch())
        card.run(experts_launches)
        jobs = layer.jobs() if wide is None else wide.read("jobs", amd.JOB_DTYPE)
        got = layer.read("row_output", np.float32).reshape(rows, HIDDEN)
    finally:
        card.close()
    live = jobs[jobs["row_count"] > 0]
    experts_of, weights_of = np.zeros((rows, PICKS), np.uint32), np.zeros((rows, PICKS), np.float32)
    seen = np.zeros(rows * PICKS, dtype=int)
    for job in live:
        for c in range(job["row_count"]):
            experts_of.reshape(-1)[job["pair_index"][c]] = job["expert"]
            weights_of.reshape(-1)[job["pair_index"][c]] = job["route_weight"][c]
            seen[job["pair_index"][c]] += 1
    assert np.all(seen == 1), "every pair of the step is in exactly one job"
    # the picks are the oracle's: ids and weight bits of the sampled rows
    sample = np.unique(np.array([0, rows // 3, rows // 2, rows - 1]))
    want_experts, want_weights = np.zeros((len(sample), PICKS), np.uint32), np.zeros((len(sample), PICKS), np.float32)
    bias = np.zeros(EXPERTS, np.float32)
    o.orc.orc_router_route(o.ptr(np.ascontiguousarray(x[sample]), o.u16p), o.ptr(router, o.u16p), o.ptr(bias, o.f32p), len(sample), HIDDEN, EXPERTS,
                           PICKS, layer.affinity_kind, 0, layer.route_scale, None, o.ptr(want_experts, o.u32p), o.ptr(want_weights, o.f32p))
    assert np.array_equal(np.sort(experts_of[sample], axis=1), np.sort(want_experts, axis=1))
    pointers = (C.c_void_p * (EXPERTS * 3))(*[m.ctypes.data for trio in matrices for m in trio])
    want = np.zeros((len(sample), HIDDEN), dtype=np.float32)
    o.orc.orc_linear_moe_layer(6 if fp8 else 3, o.ptr(np.ascontiguousarray(x[sample]), o.u16p), len(sample), HIDDEN, INNER, PICKS,
                               o.ptr(np.ascontiguousarray(experts_of[sample]), o.u32p), o.ptr(np.ascontiguousarray(weights_of[sample]), o.f32p),
                               EXPERTS, pointers, 10.0, o.ptr(want, o.f32p), None, None, 16)
    error = float(np.sqrt(np.mean((got[sample] - want) ** 2) / np.mean(want.astype(np.float64) ** 2)))
    say("  rms error of the sampled rows %.2e" % error)
    assert error <= 2e-2
    assert np.all(np.isfinite(got)) and float(np.abs(got).max()) < 1e4
