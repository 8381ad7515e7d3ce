"""GPU parity of the FP4 (E2M1 + E8M0 per 32) and FP8 (E4M3 + E8M0 per 32 x 32) routed experts against the CPU oracle, through the C ABI: the activation
quantizer byte for byte (codes in lane order, exponents, operands), the products within the reference's own bound
(tests/linear_reference.h:43-58 of the reference: |c - y| <= ulp_bf16(c)/2 + (T + B + S) 2^-24 m + B 2^-149, T = 64),
the hidden step, the row sum bit for bit, and whole layers.

The allowance T for the rounding inside the matrix instructions is 64 in the reference (instructions of 16 products on
its cards). gfx950's v_mfma_scale_f32_16x16x128_f8f6f4 adds 128 products of four scale blocks in one instruction, and a
probe of the instruction alone shows how: exact when the products' exponents lie close together, and up to 2.7e3 x 2^-24
of the magnitude sum from the exact value (1.2e3 with E2M1 weights) when codes are drawn uniformly, every exponent as
likely as any other: the products are cut a fixed number of places below the largest of the instruction, about
2^-19 of it each. The sound bound of 128 products cut at 2^-19 of the largest is T = 4096, taken here for the stress
of uniformly random E4M3 weights; weights and vectors of the benchmark's kind (Gaussian weights under their block
scales, quantised Gaussian vectors) stay within T = 256."""
import ctypes as C
import sys

import numpy as np
import pytest

from _oracle import JOB_DTYPE, f32p, f64p, normals, orc, ptr, to_bf16, bf16_to_f32, u8p, u16p, u32p, u64p

pytestmark = pytest.mark.gpu
E2M1, E4M3 = 3, 5
ALLOWANCE_GFX950 = 256.0        # weights and vectors of the benchmark's kind
ALLOWANCE_GFX950_STRESS = 4096.0  # uniformly random codes: 128 products cut at 2^-19 of the largest


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


def build(amd, card, hidden, inner, experts_n, picks, rows, seed, fmt=E2M1, stress=False, **more):
    from anemone_amd import workloads
    matrix = workloads.fp4_matrix if fmt == E2M1 else workloads.fp8_matrix_of_random_codes if stress else workloads.fp8_matrix
    matrices = [[matrix(seed * 1000 + 3 * e + 0, inner, hidden), matrix(seed * 1000 + 3 * e + 1, inner, hidden),
                 matrix(seed * 1000 + 3 * e + 2, hidden, inner)] for e in range(experts_n)]
    router = to_bf16(normals(seed + 5, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    layer = amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, matrices, router_weights_bf16=router, weight_format=fmt, **more)
    return layer, matrices, router


def oracle_quantize(values):
    rows, width = values.shape
    codes = np.zeros((rows, width), dtype=np.uint8)
    exps = np.zeros((rows, width // 32), dtype=np.uint8)
    lane = np.zeros((rows, width), dtype=np.uint8)
    operands = np.zeros((rows, width), dtype=np.uint16)
    for r in range(rows):
        assert orc.orc_act_quantize(ptr(values[r], u16p), width, ptr(codes[r], u8p), ptr(exps[r], u8p)) == 0
        orc.orc_codes_lane_order(ptr(codes[r], u8p), width, ptr(lane[r], u8p))
        orc.orc_operands_lay_out(ptr(codes[r], u8p), ptr(exps[r], u8p), width, ptr(operands[r], u16p))
    return codes, exps, lane, operands


def lane_to_value_order(lane_codes):
    """Inverse of the lane order of a vector's codes."""
    rows, width = lane_codes.shape
    at = np.arange(width)
    j, s, t, l = at % 4, (at // 4) % 4, (at // 16) % 4, at // 64
    value = 64 * l + 16 * s + 2 * t + j // 2 + 8 * (j % 2)
    out = np.zeros_like(lane_codes)
    out[:, value] = lane_codes[:, at]
    return out


def test_quantizer_byte_for_byte(amd, card):
    say("quantizer")
    rows, width = 5, 1024
    spread = np.repeat([1e-7, 1e-3, 0.2, 1.0, 30.0, 448.0, 5e3, 1e30], width // 8)
    values = to_bf16(normals(3, rows * width).reshape(rows, width) * spread)
    values[0, :32] = to_bf16(np.full(32, 448.0 * 2.0 ** -5))      # a block whose maximum is 448 x a power of two
    values[1, 64:96] = 0                                            # an all-zero block: the floor 1e-4
    values[2, 100] = 0x8000                                         # a negative zero keeps its sign
    layer, _, _ = build(amd, card, width, 128, 64, 2, rows, 1)
    layer.set_rows(values)
    card.run(layer.quantize_launch())
    codes, exps, lane, operands = oracle_quantize(values)
    assert np.array_equal(layer.read("exponents").reshape(rows, -1), exps)
    assert np.array_equal(layer.read("codes").reshape(rows, width), lane)
    assert np.array_equal(layer.read("operands", np.uint16).reshape(rows, width), operands)


@pytest.mark.parametrize("slices,fmt,stress", [(1, E2M1, False), (2, E2M1, False), (4, E2M1, False), (8, E2M1, False),
                                               (1, E4M3, False), (2, E4M3, False), (8, E4M3, False), (4, E4M3, True)])
def test_products_within_the_reference_bound(amd, card, slices, fmt, stress):
    """The down kernel is the plain product: each expert's gate matrix through it, against the exact block sums."""
    say("products, slices", slices, "format", fmt, "stress", stress)
    hidden, inner, experts_n, rows = 1024, 1024, 64, 6
    allowance = ALLOWANCE_GFX950_STRESS if stress else ALLOWANCE_GFX950
    layer, matrices, _ = build(amd, card, hidden, inner, experts_n, 1, rows, 2, fmt=fmt, stress=stress, gate_up_slices=1, down_slices=slices)
    x = to_bf16(normals(7, rows * hidden).reshape(rows, hidden) * np.repeat([0.01, 1.0, 100.0, 1.0], hidden // 4))
    codes, exps, lane, _ = oracle_quantize(x)
    # pairs_per_row = 1: pair = row; three jobs over the first experts' GATE matrices (inner x hidden), as "down"
    jobs = np.zeros(rows, dtype=JOB_DTYPE)
    plan = [(0, [0, 1, 2]), (1, [3]), (2, [4, 5])]
    for j, (expert, members) in enumerate(plan):
        jobs[j]["down_offset"] = layer.expert_offsets[expert, 0]
        jobs[j]["row_count"], jobs[j]["expert"] = len(members), expert
        jobs[j]["pair_index"][:len(members)] = members
    card.upload(layer.jobs_offset, jobs.view(np.uint8))
    card.upload(layer.ranges["hidden_codes"].byte_offset, lane)
    card.upload(layer.ranges["hidden_exponents"].byte_offset, exps)
    launches = layer.expert_launches()
    card.run(launches[2:3])
    got = layer.read("pair_output", np.uint16).reshape(rows, hidden)
    worst = 0.0
    for expert, members in plan:
        sums, mags = np.zeros((len(members), inner)), np.zeros((len(members), inner))
        member_codes, member_exps = np.ascontiguousarray(codes[members]), np.ascontiguousarray(exps[members])
        assert orc.orc_linear_products(fmt, inner, hidden, ptr(matrices[expert][0], u8p), 0, inner, ptr(member_codes, u8p),
                                       ptr(member_exps, u8p), len(members), ptr(sums, f64p), ptr(mags, f64p)) == 0
        for i, row in enumerate(members):
            for o in range(inner):
                assert orc.orc_linear_within_allowance(int(got[row, o]), sums[i, o], mags[i, o], hidden, slices, allowance), (expert, row, o)
            exact = to_bf16(sums[i].astype(np.float32))
            worst = max(worst, float(np.mean(exact != got[row, :inner])))
    say("  outputs that are not the exact sum rounded once: %.4f" % worst)
    assert worst < (0.2 if stress else 0.02)


@pytest.mark.parametrize("rows,live,picks,fmt", [(8, 8, 4, E2M1), (3, 2, 8, E2M1), (1, 1, 2, E2M1), (8, 7, 4, E4M3), (2, 2, 8, E4M3)])
def test_layer_against_oracle(amd, card, rows, live, picks, fmt):
    say("layer", rows, live, picks, "format", fmt)
    hidden, inner, experts_n = 512, 256, 64
    layer, matrices, router = build(amd, card, hidden, inner, experts_n, picks, rows, 4, fmt=fmt)
    x = to_bf16(normals(9, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x, live)
    card.run(layer.projection_launch())
    card.run(layer.select_launch(0))
    card.run(layer.quantize_launch())
    launches = layer.expert_launches()
    card.run(launches)
    jobs = layer.jobs()
    # the oracle's routing (bit-exact with the card's, checked in test_gpu_exl3) rebuilt from the job table
    experts = np.zeros((rows, picks), dtype=np.uint32)
    weights = np.zeros((rows, picks), dtype=np.float32)
    for job in jobs[jobs["row_count"] > 0]:
        for c in range(job["row_count"]):
            experts.reshape(-1)[job["pair_index"][c]] = job["expert"]
            weights.reshape(-1)[job["pair_index"][c]] = job["route_weight"][c]
    pointers = (C.c_void_p * (experts_n * 3))(*[m.ctypes.data for trio in matrices for m in trio])
    want = np.zeros((live, hidden), dtype=np.float32)
    want_hidden = np.zeros((live * picks, inner), dtype=np.uint16)
    want_pairs = np.zeros((live * picks, hidden), dtype=np.uint16)
    orc.orc_linear_moe_layer(fmt, ptr(np.ascontiguousarray(x[:live]), u16p), live, hidden, inner, picks,
                             ptr(np.ascontiguousarray(experts[:live]), u32p), ptr(np.ascontiguousarray(weights[:live]), f32p),
                             experts_n, pointers, 10.0, ptr(want, f32p), ptr(want_hidden, u16p), ptr(want_pairs, u16p), 8)
    live_pairs = live * picks
    # hidden: the gate and up sums round to bfloat16 before the step; a flip of one last place there moves the
    # hidden value by about 2^-7 of it
    got_hidden = bf16_to_f32(layer.read("hidden", np.uint16).reshape(-1, inner)[:live_pairs]).astype(np.float64)
    ref_hidden = bf16_to_f32(want_hidden).astype(np.float64)
    assert np.all(np.abs(got_hidden - ref_hidden) <= 2.0 ** -6 * np.abs(ref_hidden) + 1e-6)
    say("  hidden values equal to the oracle's: %.4f" % float(np.mean(got_hidden == ref_hidden)))
    # down: exactly checked against the card's own hidden codes
    hidden_lane = layer.read("hidden_codes").reshape(-1, inner)[:live_pairs]
    hidden_exps = np.ascontiguousarray(layer.read("hidden_exponents").reshape(-1, inner // 32)[:live_pairs])
    hidden_bits = np.ascontiguousarray(layer.read("hidden", np.uint16).reshape(-1, inner)[:live_pairs])
    codes, exps, lane, _ = oracle_quantize(hidden_bits)
    assert np.array_equal(lane, hidden_lane) and np.array_equal(exps, hidden_exps)
    pair_out = layer.read("pair_output", np.uint16).reshape(-1, hidden)[:live_pairs]
    for pair in range(0, live_pairs, max(1, live_pairs // 6)):
        e = int(experts.reshape(-1)[pair])
        sums, mags = np.zeros(hidden), np.zeros(hidden)
        orc.orc_linear_products(fmt, hidden, inner, ptr(matrices[e][2], u8p), 0, hidden, ptr(np.ascontiguousarray(codes[pair]), u8p),
                                ptr(np.ascontiguousarray(exps[pair]), u8p), 1, ptr(sums, f64p), ptr(mags, f64p))
        assert all(orc.orc_linear_within_allowance(int(pair_out[pair, o]), sums[o], mags[o], inner, 2, ALLOWANCE_GFX950) for o in range(hidden))
    # row sum: bit for bit from the card's pair outputs
    got = layer.read("row_output", np.float32).reshape(rows, hidden)[:live]
    for r in range(live):
        rows_pairs = np.ascontiguousarray(pair_out[r * picks:(r + 1) * picks])
        for column in range(0, hidden, 37):
            assert got[r, column] == orc.orc_row_sum_bf16(ptr(rows_pairs, u16p), picks, hidden, column)
    # and the whole layer against the oracle's
    error = np.sqrt(np.mean((got - want) ** 2) / np.mean(want.astype(np.float64) ** 2))
    say("  layer rms error vs oracle: %.2e" % error)
    assert error < 2e-2


@pytest.mark.parametrize("rows,live,picks,fmt,slices", [(8, 6, 4, E2M1, 4), (8, 8, 8, E2M1, 1), (4, 3, 8, E4M3, 2), (1, 1, 2, E2M1, 2)])
def test_producer_equals_the_two_launches_byte_for_byte(amd, card, rows, live, picks, fmt, slices):
    """expert_gate_up_quantize_<S> against expert_gate_up_<S> followed by the quantizer (the reference's own bar for its
    producer, tests/expert_fused_card_test.c:2-4): the hidden values, their codes, exponents and operands of every pair,
    those of the rows beyond the live ones among them (quantized from what the hidden range holds)."""
    say("producer", rows, live, picks, fmt, slices)
    hidden, inner, experts_n = 512, 256, 64
    layer, _, _ = build(amd, card, hidden, inner, experts_n, picks, rows, 6, fmt=fmt, gate_up_slices=slices, down_slices=1)
    x = to_bf16(normals(13, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x, live)
    card.run(layer.projection_launch())
    card.run(layer.select_launch(0))
    card.run(layer.quantize_launch())
    stale = to_bf16(normals(14, rows * picks * inner) * 3.0)  # what the hidden range holds for pairs no job writes
    names = ("hidden", "hidden_codes", "hidden_exponents", "hidden_operands")

    def run(launches):
        card.upload(layer.ranges["hidden"].byte_offset, stale)
        for name in names[1:]:
            card.upload(layer.ranges[name].byte_offset, np.full(layer.ranges[name].byte_count, 0xEE, dtype=np.uint8))
        card.run(launches)
        return [layer.read(name).copy() for name in names]
    apart = run(layer.expert_launches()[0:2])
    fused = run(layer.producer_launch())
    for name, a, b in zip(names, apart, fused):
        assert np.array_equal(a, b), name
    assert not np.any(card.download(layer.arrivals.byte_offset, layer.arrivals.byte_count))  # the arrival counters stay zero
    if live < rows:  # the pairs of the rows beyond the live ones were quantized from the stale values
        want = oracle_quantize(stale.reshape(rows * picks, inner)[live * picks:])[2]
        assert np.array_equal(fused[1].reshape(rows * picks, inner)[live * picks:], want)


def branched_step(amd, layer, wide, branches):
    """A decode step of the FP4 layer through the wide select's one-block form: the rows' quantizer reads the rows alone
    and stands first; with `branches` it is a side run that opens the graph, the router's launches the main line behind
    the root, the gate/up launch the join. (Every other launch of the step reads what the one before it wrote.)"""
    routing = wide.launches(small=True)
    experts = layer.expert_launches(wide)
    order = [layer.quantize_launch()[0], layer.projection_launch()[0], routing[0], routing[1]] + [experts[i] for i in range(4)]
    step = amd.launches_of(len(order))
    for i, launch in enumerate(order):
        step[i] = launch
    if branches:
        step[0].branch, step[1].branch, step[4].branch = amd.LAUNCH_SIDE, amd.LAUNCH_RESUME, amd.LAUNCH_JOIN
    return step


def test_graph_with_a_side_run_replays_the_serial_step(amd, card):
    """A step captured with graph_capture, the rows' quantizer on a side run beside the router (LAUNCH_SIDE, RESUME,
    JOIN: include/anemone/backend_seam.h:184-195 of the reference), replayed three times with other work and waits of
    the card between the replays: every replay writes the bits of the serial launch_run; lists whose branches do not
    fit are refused before anything is captured."""
    say("graph with a side run")
    hidden, inner, experts_n, picks, rows = 512, 256, 64, 4, 32
    layer, _, _ = build(amd, card, hidden, inner, experts_n, picks, rows, 8, gate_up_slices=2, down_slices=1)
    x = to_bf16(normals(29, rows * hidden)).reshape(rows, hidden)
    other = to_bf16(normals(30, rows * hidden)).reshape(rows, hidden)
    wide = layer.wide_router()
    layer.set_rows(x, rows)
    card.run(branched_step(amd, layer, wide, False))
    serial = layer.read("row_output", np.float32).copy()
    assert np.any(serial != 0.0)
    graph = card.capture(branched_step(amd, layer, wide, True))
    for replay in range(3):
        layer.set_rows(other, rows)  # other work between the replays: a step on other rows, run launch by launch
        card.run(branched_step(amd, layer, wide, False))
        assert np.any(layer.read("row_output", np.float32) != serial)
        layer.set_rows(x, rows)
        card.run_graph(graph)
        assert np.array_equal(layer.read("row_output", np.float32).view(np.uint32), serial.view(np.uint32)), replay
    # launch_run takes the same list in its serial order
    layer.set_rows(other, rows)
    card.run(branched_step(amd, layer, wide, False))
    layer.set_rows(x, rows)
    card.run(branched_step(amd, layer, wide, True))
    assert np.array_equal(layer.read("row_output", np.float32).view(np.uint32), serial.view(np.uint32))
    for spoil in ("join without a side run", "chain behind a side launch", "resume without a side run", "unknown branch"):
        step = branched_step(amd, layer, wide, spoil == "chain behind a side launch")
        if spoil == "join without a side run":
            step[4].branch = amd.LAUNCH_JOIN
        elif spoil == "chain behind a side launch":
            step[1].branch = amd.LAUNCH_CHAIN
        elif spoil == "resume without a side run":
            step[1].branch = amd.LAUNCH_RESUME
        else:
            step[2].branch = 9
        with pytest.raises(amd.AnemoneError):
            card.capture(step)
