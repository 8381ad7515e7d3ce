"""GPU parity of the wide select (the router of a prefill: pairs sorted by expert, runs, tiles of at most 64 pairs, jobs
of at most 8) against the CPU oracle, bit for bit, through the C ABI; the reference's hand case of its wide test
(tests/router_wide_test.c:6-11: 130 rows that pick the same six experts) among them; and a layer of the FP4 experts
driven by the wide job table."""
import ctypes as C
import sys

import numpy as np
import pytest

from _oracle import JOB_DTYPE, PAIR_DTYPE, RUN_DTYPE, TILE_DTYPE, f32p, normals, orc, ptr, to_bf16, u16p, u32p, u64p

pytestmark = pytest.mark.gpu


def say(*words):
    print(*words, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def amd():
    import anemone_amd
    return anemone_amd


@pytest.fixture(scope="module")
def card(amd):
    card = amd.Card(1 << 30)
    yield card
    card.close()


@pytest.fixture(autouse=True)
def fresh_arena(card):
    card.cursor = 256
    yield


def small_layer(amd, card, experts_n, picks, rows, hidden=128, inner=64, affinity_kind=1):
    from anemone_amd import workloads
    trio = [workloads.fp4_matrix(1, inner, hidden), workloads.fp4_matrix(2, inner, hidden), workloads.fp4_matrix(3, hidden, inner)]
    matrices = [trio] * experts_n
    router = to_bf16(normals(5, experts_n * hidden) * 0.05).reshape(experts_n, hidden)
    return amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, matrices, router_weights_bf16=router,
                        affinity_kind=affinity_kind), router


def oracle_wide(layer, scores, bias, live, order=0):
    rows, E, P = layer.rows, layer.E, layer.P
    affinities = np.array([[orc.orc_router_affinity(float(s), layer.affinity_kind) for s in row] for row in scores], dtype=np.float32)
    experts = np.zeros((rows, P), dtype=np.uint32)
    weights = np.zeros((rows, P), dtype=np.float32)
    for r in range(live):
        orc.orc_router_select(ptr(affinities[r], f32p), ptr(bias, f32p), E, P, order, layer.route_scale,
                              ptr(experts[r], u32p), ptr(weights[r], f32p))
    offsets = np.ascontiguousarray(layer.expert_offsets.reshape(-1))
    pairs = np.zeros(live * P, dtype=PAIR_DTYPE)
    runs = np.zeros(E, dtype=RUN_DTYPE)
    tiles = np.zeros(orc.orc_router_wide_tile_count(rows, P, E), dtype=TILE_DTYPE)
    jobs = np.zeros(orc.orc_router_wide_job_count(rows, P, E), dtype=JOB_DTYPE)
    orc.orc_router_wide_sort(ptr(experts, u32p), ptr(weights, f32p), P, live, rows, E, ptr(offsets, u64p),
                             pairs.ctypes.data, runs.ctypes.data, tiles.ctypes.data)
    orc.orc_router_wide_jobs(ptr(experts, u32p), ptr(weights, f32p), P, live, rows, E, ptr(offsets, u64p), jobs.ctypes.data)
    return affinities, experts, weights, pairs, runs, tiles, jobs


def run_and_compare(amd, card, layer, scores, bias, live, order=0):
    rows, E, P = layer.rows, layer.E, layer.P
    card.upload(layer.scores_offset, scores)
    card.upload(layer.bias_offset, bias)
    card.upload(layer.step_offset, amd.step_block(live))
    wide = layer.wide_router()
    wide.description.order = order
    assert wide.tile_count == orc.orc_router_wide_tile_count(rows, P, E)
    assert wide.job_count == orc.orc_router_wide_job_count(rows, P, E)
    # scratch that the kernels must overwrite or clear: fill with a pattern first
    for name in ("pairs", "runs", "tiles", "jobs"):
        r = wide.ranges[name]
        card.upload(r.byte_offset, np.full(r.byte_count, 0xA5, dtype=np.uint8))
    card.run(wide.launches())
    affinities, experts, weights, pairs, runs, tiles, jobs = oracle_wide(layer, scores, bias, live, order)
    got_aff = card.download(layer.affinities_offset, rows * E * 4, np.float32).reshape(rows, E)
    assert np.array_equal(got_aff[:live].view(np.uint32), affinities[:live].view(np.uint32))
    picks = wide.read("picks", np.dtype([("expert", "<u4"), ("route_weight", "<f4")])).reshape(rows, P)
    assert np.array_equal(picks["expert"][:live], experts[:live])
    assert np.array_equal(picks["route_weight"][:live].view(np.uint32), weights[:live].view(np.uint32))
    assert wide.read("pairs", PAIR_DTYPE)[:live * P].tobytes() == pairs.tobytes()
    assert wide.read("runs", RUN_DTYPE).tobytes() == runs.tobytes()
    assert wide.read("tiles", TILE_DTYPE).tobytes() == tiles.tobytes()
    assert wide.read("jobs", JOB_DTYPE).tobytes() == jobs.tobytes()
    return wide, experts, weights, jobs


@pytest.mark.parametrize("experts_n,picks,rows,live,kind", [(64, 4, 40, 37, 1), (256, 8, 500, 500, 1), (384, 6, 1000, 777, 0),
                                                            (64, 8, 8, 1, 1), (128, 2, 385, 385, 1)])
def test_wide_select_bit_exact(amd, card, experts_n, picks, rows, live, kind):
    say("wide select", experts_n, picks, rows, live, kind)
    layer, _ = small_layer(amd, card, experts_n, picks, rows, affinity_kind=kind)
    scores = (normals(rows * 7 + picks, rows * experts_n) * 1.5).astype(np.float32).reshape(rows, experts_n)
    bias = (normals(3, experts_n) * 0.1).astype(np.float32)
    run_and_compare(amd, card, layer, scores, bias, live)


def test_wide_select_skewed_and_hand_case(amd, card):
    """130 rows that all pick the same six experts: tiles of 64, 64 and 2 pairs an expert, 16 jobs of 8 and one of 2
    (the reference's wide test, by hand); then a Zipf-like bias: runs of very different lengths."""
    say("wide hand case")
    layer, _ = small_layer(amd, card, 384, 6, 130, affinity_kind=0)
    scores = np.zeros((130, 384), dtype=np.float32)
    bias = np.zeros(384, dtype=np.float32)
    chosen = [3, 77, 100, 200, 300, 383]
    bias[chosen] = 1.0
    wide, experts, _, jobs = run_and_compare(amd, card, layer, scores, bias, 130, order=1)
    tiles = wide.read("tiles", TILE_DTYPE)
    assert tiles["pair_count"][:18].tolist() == [64, 64, 2] * 6 and not tiles["pair_count"][18:].any()
    used = jobs[jobs["row_count"] > 0]
    assert used["row_count"].tolist() == ([8] * 16 + [2]) * 6 and used["expert"][::17].tolist() == chosen
    say("wide skewed")
    card.cursor = 256
    layer, _ = small_layer(amd, card, 256, 8, 900, affinity_kind=1)
    scores = (normals(99, 900 * 256)).astype(np.float32).reshape(900, 256)
    bias = (-1.1 * np.log(1.0 + np.arange(256))).astype(np.float32)[np.argsort(normals(5, 256))]
    wide, experts, _, _ = run_and_compare(amd, card, layer, scores, bias.astype(np.float32), 900)
    counts = np.bincount(experts.reshape(-1), minlength=256)
    say("  longest run %d pairs, %d experts without a pair" % (counts.max(), int((counts == 0).sum())))
    assert counts.max() > 400


@pytest.mark.parametrize("experts_n,picks,rows,live", [(64, 4, 40, 37), (256, 8, 384, 384), (384, 6, 130, 130), (128, 3, 1, 1)])
def test_wide_small_equals_the_four_launches(amd, card, experts_n, picks, rows, live):
    """router_wide_small (count, place and jobs of at most 384 rows in one block) writes the pairs, runs, tiles and
    jobs of the four launches, byte for byte (include/anemone/router.h:117-119 of the reference), and those are held to
    the oracle by the tests above."""
    say("wide small", experts_n, picks, rows, live)
    layer, _ = small_layer(amd, card, experts_n, picks, rows)
    scores = (normals(123, rows * experts_n) * 1.5).astype(np.float32).reshape(rows, experts_n)
    card.upload(layer.scores_offset, scores)
    card.upload(layer.bias_offset, np.zeros(experts_n, dtype=np.float32))
    card.upload(layer.step_offset, amd.step_block(live))
    wide = layer.wide_router()
    names = ("pairs", "runs", "tiles", "jobs")

    def run(launches):
        for name in names:
            card.upload(wide.ranges[name].byte_offset, np.full(wide.ranges[name].byte_count, 0xEE, dtype=np.uint8))
        card.run(launches)
        return [wide.read(name, np.uint8).copy() for name in names]
    four = run(wide.launches())
    card.upload(wide.ranges["counts"].byte_offset, np.full(wide.ranges["counts"].byte_count, 0xEE, dtype=np.uint8))
    two = run(wide.launches(small=True))
    live_pairs = live * picks
    for name, a, b in zip(names, four, two):
        count = live_pairs * 8 if name == "pairs" else a.size  # the pairs past the live rows' are not written
        assert np.array_equal(a[:count], b[:count]), name
    assert np.all(wide.read("counts", np.uint8) == 0xEE)  # the counts scratch stays unwritten


@pytest.mark.parametrize("experts_n,rows,hidden,scale", [(64, 300, 512, 1.0), (256, 257, 1024, 1.0), (64, 321, 128, 1e-18), (128, 1000, 256, 3e18), (64, 700, 384, 1.0), (64, 300, 192, 1.0), (384, 290, 5120, 1.0)])
def test_projection_of_many_rows_bit_exact(amd, card, experts_n, rows, hidden, scale):
    """router_projection_tiles (257 rows and more: the 32 chains of a score as matrix-unit products of one input each)
    against the oracle's chains, every bit; scales that put products among the subnormals and near overflow among
    the cases."""
    say("projection, many rows", experts_n, rows, hidden, scale)
    layer, _ = small_layer(amd, card, experts_n, 2, rows, hidden=hidden)
    router = to_bf16(normals(41, experts_n * hidden) * scale).reshape(experts_n, hidden)
    x = to_bf16(normals(42, rows * hidden) * scale).reshape(rows, hidden)
    card.upload(layer.router_offset, router)
    layer.set_rows(x, rows)
    launch = layer.projection_launch()
    if hidden % 128 == 0:  # a stage of the matrix-unit kernel is 128 inputs; any other width takes the thin kernel
        assert list(launch[0].block)[0] == 256 and list(launch[0].grid) == [experts_n // 16, (rows + 63) // 64, 1]
    else:
        assert list(launch[0].grid)[1] == (rows + 3) // 4
    card.upload(layer.scores_offset, np.full(rows * experts_n * 4, 0xEE, dtype=np.uint8))
    card.run(launch)
    got = card.download(layer.scores_offset, rows * experts_n * 4, np.float32).reshape(rows, experts_n)
    want = np.zeros((rows, experts_n), dtype=np.float32)
    orc.orc_router_projection(ptr(x, u16p), ptr(router, u16p), rows, hidden, experts_n, ptr(want, f32p))
    differing = np.flatnonzero(got.view(np.uint32) != want.view(np.uint32))
    say("  %d of %d scores differ" % (differing.size, got.size))
    assert differing.size == 0


def test_fp4_layer_through_the_wide_job_table(amd, card):
    """40 rows (37 live) routed by the wide select, then the FP4 experts over its job table, against the oracle."""
    say("fp4 layer, wide")
    from anemone_amd import workloads
    hidden, inner, experts_n, picks, rows, live = 512, 256, 64, 4, 40, 37
    matrices = [[workloads.fp4_matrix(7000 + 3 * e, inner, hidden), workloads.fp4_matrix(7001 + 3 * e, inner, hidden),
                 workloads.fp4_matrix(7002 + 3 * e, hidden, inner)] for e in range(experts_n)]
    router = to_bf16(normals(5, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    layer = amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, matrices, router_weights_bf16=router)
    x = to_bf16(normals(9, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x, live)
    card.run(layer.projection_launch())
    wide = layer.wide_router()
    card.run(wide.launches())
    card.run(layer.quantize_launch())
    card.run(layer.expert_launches(wide))
    scores = card.download(layer.scores_offset, rows * experts_n * 4, np.float32).reshape(rows, experts_n)
    _, experts, weights, _, _, _, jobs = oracle_wide(layer, scores, np.zeros(experts_n, dtype=np.float32), live)
    assert wide.read("jobs", JOB_DTYPE).tobytes() == jobs.tobytes()
    pointers = (C.c_void_p * (experts_n * 3))(*[m.ctypes.data for trio in matrices for m in trio])
    want = np.zeros((live, hidden), dtype=np.float32)
    orc.orc_linear_moe_layer(3, ptr(np.ascontiguousarray(x[:live]), u16p), live, hidden, inner, picks,
                             ptr(np.ascontiguousarray(experts[:live]), u32p), ptr(np.ascontiguousarray(weights[:live]), f32p),
                             experts_n, pointers, 10.0, ptr(want, f32p), None, None, 8)
    got = layer.read("row_output", np.float32).reshape(rows, hidden)[:live]
    error = np.sqrt(np.mean((got - want) ** 2) / np.mean(want.astype(np.float64) ** 2))
    say("  layer rms error vs oracle: %.2e" % error)
    assert error < 2e-2
