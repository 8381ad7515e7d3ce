"""GPU checks, through the C ABI, of the FP8 experts with float32 block scales (WEIGHT_FORMAT_E4M3_BLOCK128: E4M3
weights with one float32 scale for every 128 x 128 block, vectors quantized 128 values a float32 scale: the usual
block scaling of FP8 checkpoints). PARITY UNPINNED against the reference, which has no function of this scaling: the
checker is the CPU oracle's closed form (oracle/orc_linear.c: orc_act_quantize_128, orc_linear_products_128, which
tests/test_oracle_linear.py pins against numpy). The quantizer is held byte for byte, the products to the bound the
reference states for its own formats (tests/linear_reference.h:43-58 of the reference, with this card's allowance), the
wide form byte for byte to the job-table kernels of one slice, and whole layers to 2e-2 rms."""
import ctypes as C
import sys

import numpy as np
import pytest

from _oracle import JOB_DTYPE, f32p, f64p, normals, orc, ptr, to_bf16, u8p, u16p, u32p
from test_gpu_linear import ALLOWANCE_GFX950

pytestmark = pytest.mark.gpu
B128 = 6


def say(*words):
    print(*words, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def amd():
    import anemone_amd
    return anemone_amd


@pytest.fixture(scope="module")
def card(amd):
    card = amd.Card(2 << 30)
    yield card
    card.close()


@pytest.fixture(autouse=True)
def fresh_arena(card):
    card.cursor = 256
    yield


def build(amd, card, hidden, inner, experts_n, picks, rows, seed, distinct=4, **more):
    from anemone_amd import workloads
    trios = [[workloads.fp8_block128_matrix(seed * 1000 + 3 * e, inner, hidden), workloads.fp8_block128_matrix(seed * 1000 + 3 * e + 1, inner, hidden),
              workloads.fp8_block128_matrix(seed * 1000 + 3 * e + 2, hidden, inner)] for e in range(distinct)]
    matrices = [trios[e % distinct] for e in range(experts_n)]
    router = to_bf16(normals(seed + 5, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    layer = amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, matrices, router_weights_bf16=router, weight_format=B128, **more)
    return layer, matrices


def oracle_quantize(values):
    rows, width = values.shape
    codes, lane = np.zeros((rows, width), dtype=np.uint8), np.zeros((rows, width), dtype=np.uint8)
    scales = np.zeros((rows, width // 128), dtype=np.float32)
    for r in range(rows):
        orc.orc_act_quantize_128(ptr(values[r], u16p), width, ptr(codes[r], u8p), ptr(scales[r], f32p))
        orc.orc_codes_lane_order(ptr(codes[r], u8p), width, ptr(lane[r], u8p))
    return codes, scales, lane


def test_quantizer_byte_for_byte(amd, card):
    say("quantizer of 128 values a scale")
    rows, width = 5, 1024
    spread = np.repeat([1e-7, 1e-3, 0.2, 1.0, 30.0, 448.0, 5e3, 1e30], width // 8)
    values = to_bf16(normals(3, rows * width).reshape(rows, width) * spread)
    values[1, 128:256] = 0       # an all-zero group: the floor 1e-4
    values[2, 100] = 0x8000      # a negative zero keeps its sign
    values[3, :128] = to_bf16(np.full(128, 448.0 * 2.0 ** -5))
    layer, _ = build(amd, card, width, 128, 64, 2, rows, 1)
    layer.set_rows(values)
    card.upload(layer.ranges["operands"].byte_offset, np.full(rows * width * 2, 0xEE, dtype=np.uint8))
    card.run(layer.quantize_launch())
    _, scales, lane = oracle_quantize(values)
    assert np.array_equal(layer.read("exponents").view(np.float32).reshape(rows, -1).view(np.uint32), scales.view(np.uint32))
    assert np.array_equal(layer.read("codes").reshape(rows, width), lane)
    assert np.all(layer.read("operands") == 0xEE)  # not written


@pytest.mark.parametrize("slices", [1, 2, 8])
def test_products_within_the_bound(amd, card, slices):
    """The down kernel is the plain product: each expert's gate matrix through it, against the exact block sums."""
    say("block128 products, slices", slices)
    hidden, inner, experts_n, rows = 1024, 1024, 64, 6
    layer, matrices = build(amd, card, hidden, inner, experts_n, 1, rows, 2, gate_up_slices=1, down_slices=slices)
    x = to_bf16(normals(7, rows * hidden).reshape(rows, hidden) * np.repeat([0.01, 1.0, 100.0, 1.0], hidden // 4))
    codes, scales, lane = oracle_quantize(x)
    jobs = np.zeros(rows, dtype=JOB_DTYPE)
    plan = [(0, [0, 1, 2]), (1, [3]), (2, [4, 5])]
    for j, (expert, members) in enumerate(plan):
        jobs[j]["down_offset"] = layer.expert_offsets[expert, 0]
        jobs[j]["row_count"], jobs[j]["expert"] = len(members), expert
        jobs[j]["pair_index"][:len(members)] = members
    card.upload(layer.jobs_offset, jobs.view(np.uint8))
    card.upload(layer.ranges["hidden_codes"].byte_offset, lane)
    card.upload(layer.ranges["hidden_exponents"].byte_offset, scales)
    card.run(layer.expert_launches()[2:3])
    got = layer.read("pair_output", np.uint16).reshape(rows, hidden)
    worst = 0.0
    for expert, members in plan:
        sums, mags = np.zeros((len(members), inner)), np.zeros((len(members), inner))
        member_codes, member_scales = np.ascontiguousarray(codes[members]), np.ascontiguousarray(scales[members])
        assert orc.orc_linear_products_128(inner, hidden, ptr(matrices[expert][0], u8p), 0, inner, ptr(member_codes, u8p),
                                           ptr(member_scales, f32p), len(members), ptr(sums, f64p), ptr(mags, f64p)) == 0
        for i, row in enumerate(members):
            for o in range(inner):
                assert orc.orc_linear_within_allowance(int(got[row, o]), sums[i, o], mags[i, o], hidden, slices, ALLOWANCE_GFX950), (expert, row, o)
            worst = max(worst, float(np.mean(to_bf16(sums[i].astype(np.float32)) != got[row, :inner])))
    say("  outputs that are not the exact sum rounded once: %.4f" % worst)
    assert worst < 0.05


def routing_of(jobs, rows, picks):
    experts, weights = np.zeros((rows, picks), dtype=np.uint32), np.zeros((rows, picks), dtype=np.float32)
    for job in jobs[jobs["row_count"] > 0]:
        for c in range(job["row_count"]):
            experts.reshape(-1)[job["pair_index"][c]] = job["expert"]
            weights.reshape(-1)[job["pair_index"][c]] = job["route_weight"][c]
    return experts, weights


@pytest.mark.parametrize("rows,live,picks", [(8, 8, 4), (3, 2, 8), (1, 1, 2)])
def test_layer_against_oracle(amd, card, rows, live, picks):
    say("block128 layer", rows, live, picks)
    hidden, inner, experts_n = 512, 256, 64
    layer, matrices = build(amd, card, hidden, inner, experts_n, picks, rows, 4, distinct=64)
    x = to_bf16(normals(9, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x, live)
    card.run(layer.projection_launch())
    card.run(layer.select_launch(0))
    card.run(layer.quantize_launch())
    card.run(layer.expert_launches())
    experts, weights = routing_of(layer.jobs(), rows, picks)
    pointers = (C.c_void_p * (experts_n * 3))(*[m.ctypes.data for trio in matrices for m in trio])
    want = np.zeros((live, hidden), dtype=np.float32)
    orc.orc_linear_moe_layer(B128, ptr(np.ascontiguousarray(x[:live]), u16p), live, hidden, inner, picks, ptr(np.ascontiguousarray(experts[:live]), u32p),
                             ptr(np.ascontiguousarray(weights[:live]), f32p), experts_n, pointers, layer.limit, ptr(want, f32p), None, None, 8)
    got = layer.read("row_output", np.float32).reshape(rows, hidden)[:live]
    error = np.sqrt(np.mean((got - want) ** 2) / np.mean(want.astype(np.float64) ** 2))
    say("  layer rms error vs oracle: %.2e" % error)
    assert error < 2e-2


@pytest.mark.parametrize("hidden,inner,picks,rows,live", [(512, 256, 4, 300, 300), (640, 384, 2, 450, 449), (512, 256, 8, 1500, 1401)])
def test_wide_equals_the_job_table_kernels_byte_for_byte(amd, card, hidden, inner, picks, rows, live):
    say("block128 wide experts", hidden, inner, picks, rows, live)
    layer, _ = build(amd, card, hidden, inner, 64, picks, rows, 21)
    x = to_bf16(normals(31, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x, live)
    card.run(layer.projection_launch())
    wide = layer.wide_router()
    card.run(wide.launches())
    card.run(layer.quantize_launch())
    names = ("hidden_codes", "hidden_exponents", "pair_output", "row_output")

    def run(launches):
        for name in names + ("hidden", "hidden_operands"):
            card.upload(layer.ranges[name].byte_offset, np.full(layer.ranges[name].byte_count, 0xEE, dtype=np.uint8))
        card.run(launches)
        return [layer.read(name).copy() for name in names], layer.read("hidden").copy(), layer.read("hidden_operands").copy()
    layer.gate_up_slices = layer.down_slices = 1
    narrow, hidden_values, _ = run(layer.expert_launches(wide))
    launches = layer.wide_expert_launches(wide)
    assert len(launches) == 4
    broad, _, wide_values = run(launches)
    pairs = live * picks
    for name, a, b in zip(names, narrow, broad):
        per = a.size // (rows if name == "row_output" else rows * picks)
        count = (live if name == "row_output" else pairs) * per
        differing = np.flatnonzero(a.reshape(-1)[:count] != b.reshape(-1)[:count])
        say("  %s: %d of %d bytes differ" % (name, differing.size, count))
        assert differing.size == 0, (name, differing[:8], per)
    # the wide gate/up leaves the hidden values where the narrow chain's hidden array holds them
    assert np.array_equal(wide_values[:pairs * inner * 2], hidden_values[:pairs * inner * 2])


def test_wide_layer_against_oracle(amd, card):
    say("block128 wide layer against the oracle")
    from test_gpu_router_wide import oracle_wide
    hidden, inner, experts_n, picks, rows, live = 512, 256, 64, 4, 150, 143
    layer, matrices = build(amd, card, hidden, inner, experts_n, picks, rows, 9, distinct=64)
    x = to_bf16(normals(9, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x, live)
    card.run(layer.projection_launch())
    wide = layer.wide_router()
    card.run(wide.launches())
    card.run(layer.quantize_launch())
    card.run(layer.wide_expert_launches(wide))
    scores = card.download(layer.scores_offset, rows * experts_n * 4, np.float32).reshape(rows, experts_n)
    _, experts, weights, _, _, _, _ = oracle_wide(layer, scores, np.zeros(experts_n, dtype=np.float32), live)
    pointers = (C.c_void_p * (experts_n * 3))(*[m.ctypes.data for trio in matrices for m in trio])
    want = np.zeros((live, hidden), dtype=np.float32)
    orc.orc_linear_moe_layer(B128, ptr(np.ascontiguousarray(x[:live]), u16p), live, hidden, inner, picks,
                             ptr(np.ascontiguousarray(experts[:live]), u32p), ptr(np.ascontiguousarray(weights[:live]), f32p),
                             experts_n, pointers, 10.0, ptr(want, f32p), None, None, 8)
    got = layer.read("row_output", np.float32).reshape(rows, hidden)[:live]
    error = np.sqrt(np.mean((got - want) ** 2) / np.mean(want.astype(np.float64) ** 2))
    say("  layer rms error vs oracle: %.2e" % error)
    assert error < 2e-2
