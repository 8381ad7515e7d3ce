"""GPU parity of the EXL3 path against the CPU oracle, through the C ABI: reconstruction (bit-exact), router
(affinity bits, expert ids, weights, job table: bit-exact), chain stages (operands bit-exact, products within
tolerance), whole layers by the chain and by the fused decode.

Tolerance of a product: the MFMA adds 32 exact fp16 x fp16 products at a time in float32; against the oracle's exact
sum rounded once, |error| <= 1e-3 x the root mean square of the outputs (stated by the path's contract: max rel err
<= 1e-3 against the float32 reference for f16 inputs and float32 accumulation)."""
import ctypes as C
import sys

import numpy as np
import pytest

from _oracle import (JOB_DTYPE, f32p, f64p, normals, orc, ptr, splitmix_words, to_bf16, bf16_to_f32, u8p, u16p, u32p, u64p,
                     exl3_matrix)

pytestmark = pytest.mark.gpu

PRODUCT_TOLERANCE = 1e-3


def say(*words):
    print(*words, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def amd():
    import anemone_amd
    return anemone_amd


@pytest.fixture(scope="module")
def card(amd):
    card = amd.Card(3 << 30)
    yield card
    card.close()


@pytest.fixture(autouse=True)
def fresh_arena(card):
    card.cursor = 256
    yield


@pytest.mark.parametrize("stored", [2, 3, 4, 40])
def test_reconstruct_bit_exact(amd, card, stored):
    say("reconstruct stored width", stored)
    inputs, outputs = 256, 384
    matrix = exl3_matrix(7 + stored, inputs, outputs, stored)
    record = amd.Exl3ReconstructRecord(card.place(matrix), card.reserve(inputs * outputs * 2), inputs, outputs, stored, 0)
    kernel = card.kernel("kernel_exl3", "exl3_reconstruct", C.sizeof(record))
    launch = amd.launches_of(1)
    amd.check(card.lib.exl3_reconstruct_prepare(C.byref(record), card.arena_bytes, kernel, launch), "prepare")
    card.run(launch)
    got = card.download(record.output_offset, inputs * outputs * 2, np.uint16).reshape(inputs, outputs)
    want = np.zeros((inputs, outputs), dtype=np.uint16)
    orc.orc_exl3_decode_matrix(ptr(matrix, u8p), inputs, outputs, stored, ptr(want, u16p))
    assert np.array_equal(got, want)


def build_layer(amd, card, hidden, inner, experts_n, picks, rows, seed, width_choices, affinity_kind=1, limit=10.0):
    draws = splitmix_words(seed, experts_n * 3) % np.uint64(len(width_choices))
    widths = np.array(width_choices, dtype=np.uint32)[draws.astype(np.int64)].reshape(experts_n, 3)
    matrices = [[exl3_matrix(seed * 1000 + 3 * e + 0, hidden, inner, int(widths[e, 0])),
                 exl3_matrix(seed * 1000 + 3 * e + 1, hidden, inner, int(widths[e, 1])),
                 exl3_matrix(seed * 1000 + 3 * e + 2, inner, hidden, int(widths[e, 2]))] for e in range(experts_n)]
    router = to_bf16(normals(seed + 5, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    layer = amd.Exl3Layer(card, hidden, inner, experts_n, picks, rows, matrices, widths, router_weights_bf16=router,
                          affinity_kind=affinity_kind, limit=limit)
    return layer, matrices, widths, router


def oracle_route(layer, x, router, live_rows, affinity_kind, order=0):
    rows, E, P, H = layer.rows, layer.E, layer.P, layer.H
    scores = np.zeros((rows, E), dtype=np.float32)
    orc.orc_router_projection(ptr(x, u16p), ptr(router, u16p), rows, H, E, ptr(scores, f32p))
    affinities = np.array([[orc.orc_router_affinity(float(s), affinity_kind) for s in row] for row in scores], dtype=np.float32)
    experts = np.zeros((rows, P), dtype=np.uint32)
    weights = np.zeros((rows, P), dtype=np.float32)
    bias = np.zeros(E, dtype=np.float32)
    for r in range(rows):
        orc.orc_router_select(ptr(affinities[r], f32p), ptr(bias, f32p), E, P, order, layer.route_scale,
                              ptr(experts[r], u32p), ptr(weights[r], f32p))
    jobs = np.zeros(rows * P, dtype=JOB_DTYPE)
    orc.orc_router_jobs(ptr(experts, u32p), ptr(weights, f32p), P, live_rows, rows, E,
                        ptr(np.ascontiguousarray(layer.expert_offsets.reshape(-1)), u64p), jobs.ctypes.data)
    return scores, affinities, experts, weights, jobs


def oracle_layer(layer, x, experts, weights, matrices, widths, live_rows, threads=8):
    rows, H, I, P, E = layer.rows, layer.H, layer.I, layer.P, layer.E
    pointers = (C.c_void_p * (E * 3))(*[m.ctypes.data for trio in matrices for m in trio])
    out = np.zeros((live_rows, H), dtype=np.float32)
    hidden = np.zeros((live_rows * P, I), dtype=np.uint16)
    pair_out = np.zeros((live_rows * P, H), dtype=np.float32)
    widths8 = np.ascontiguousarray(widths.astype(np.uint8))
    orc.orc_exl3_moe_layer(ptr(np.ascontiguousarray(x[:live_rows]), u16p), live_rows, H, I, P,
                           ptr(np.ascontiguousarray(experts[:live_rows]), u32p), ptr(np.ascontiguousarray(weights[:live_rows]), f32p),
                           E, pointers, ptr(widths8, u8p), layer.limit, ptr(out, f32p), ptr(hidden, u16p), ptr(pair_out, f32p), threads)
    return out, hidden, pair_out


@pytest.mark.parametrize("affinity_kind,experts_n,picks,order", [(1, 256, 8, 0), (0, 384, 6, 0), (0, 384, 6, 1), (1, 64, 3, 0)])
def test_router_bit_exact(amd, card, affinity_kind, experts_n, picks, order):
    say("router", affinity_kind, experts_n, picks, order)
    rows, live = 8, 7
    layer, _, _, router = build_layer(amd, card, 512, 128, experts_n, picks, rows, 3, [2], affinity_kind)
    x = to_bf16(normals(17, rows * 512)).reshape(rows, 512)
    layer.set_rows(x, live)
    card.run(layer.projection_launch())
    card.run(layer.select_launch(order))
    scores, affinities, experts, weights, jobs = oracle_route(layer, x, router, live, affinity_kind, order)
    got_scores = card.download(layer.scores_offset, rows * experts_n * 4, np.float32).reshape(rows, experts_n)
    assert np.array_equal(got_scores.view(np.uint32), scores.view(np.uint32))
    got_aff = card.download(layer.affinities_offset, rows * experts_n * 4, np.float32).reshape(rows, experts_n)
    assert np.array_equal(got_aff[:live].view(np.uint32), affinities[:live].view(np.uint32))
    assert layer.jobs().tobytes() == jobs.tobytes()


def test_router_hand_rows_on_the_card(amd, card):
    """The reference's hand rows (ties, NaN bias, -0 < +0) through the kernel: scores chosen so the affinities are
    the rows' values is not possible (affinity is computed), so the choice is exercised through the bias."""
    say("router hand rows")
    rows = 2
    layer, _, _, _ = build_layer(amd, card, 512, 128, 384, 6, rows, 4, [2], 0)
    scores = np.zeros((rows, 384), dtype=np.float32)
    bias = np.zeros(384, dtype=np.float32)
    bias[[7, 50, 100, 200, 250, 260]] = 1.0  # six equal: the lower experts first
    bias[300] = np.nan                          # a not-a-number above every number
    bias[5] = -0.0
    card.upload(layer.bias_offset, bias)
    card.upload(layer.scores_offset, scores)
    layer.set_rows(np.zeros((rows, 512), dtype=np.uint16), rows)
    card.run(layer.select_launch(0))
    jobs = layer.jobs()
    used = jobs[jobs["row_count"] > 0]
    assert used["expert"].tolist() == [7, 50, 100, 200, 250, 300]
    a = np.float32(orc.orc_router_affinity(0.0, 0))
    total = np.float32(0)
    for _ in range(6):
        total = np.float32(total + a)
    want = np.float32(np.float32(a / np.float32(total + np.float32(1e-20))) * np.float32(1.5))
    assert np.all(used["route_weight"][:, :2].view(np.uint32) == want.view(np.uint32))
    assert used["pair_index"][0, :2].tolist() == [0, 6] and used["row_count"].tolist() == [2] * 6


@pytest.mark.parametrize("width_choices,rows,live", [([2, 3, 4], 8, 8), ([3], 3, 2), ([40, 4], 4, 4), ([4], 1, 1)])
def test_chain_and_fused_decode_against_oracle(amd, card, width_choices, rows, live):
    say("layer", width_choices, rows, live)
    hidden, inner, experts_n, picks = 512, 256, 64, 4
    layer, matrices, widths, router = build_layer(amd, card, hidden, inner, experts_n, picks, rows, 11, width_choices)
    x = to_bf16(normals(23, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x, live)
    card.run(layer.projection_launch())
    card.run(layer.select_launch(0))
    _, _, experts, weights, jobs = oracle_route(layer, x, router, live, 1)
    assert layer.jobs().tobytes() == jobs.tobytes()
    want, want_hidden, want_pairs = oracle_layer(layer, x, experts, weights, matrices, widths, live)
    scale = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))

    # --- the chain, stage by stage ---
    chain = layer.chain_launches()
    record = layer.chain_record()
    card.run(chain[0:1])
    operands = card.download(record.operands_offset, 2 * layer.pairs * hidden * 2, np.uint16).reshape(2, layer.pairs, hidden)
    for job in jobs[jobs["row_count"] > 0][:5]:
        for c in range(job["row_count"]):
            pair, e = int(job["pair_index"][c]), int(job["expert"])
            for proj in range(2):
                matrix = matrices[e][proj]
                cb = int(orc.orc_exl3_code_bytes(hidden, inner, int(widths[e, proj])))
                suh = np.ascontiguousarray(matrix[cb:cb + 2 * hidden]).view(np.uint16)
                expect = np.zeros(hidden, dtype=np.uint16)
                orc.orc_exl3_operand(ptr(x[pair // picks], u16p), ptr(suh, u16p), hidden, ptr(expect, u16p))
                assert np.array_equal(operands[proj, pair], expect), "operands are bit-defined"
    card.run(chain[1:2])
    products = card.download(record.products_offset, 2 * layer.pairs * inner * 4, np.float32).reshape(2, layer.pairs, inner)
    job = jobs[0]
    pair, e = int(job["pair_index"][0]), int(job["expert"])
    for proj in range(2):
        expect = np.zeros(inner, dtype=np.float32)
        orc.orc_exl3_product_codes(ptr(matrices[e][proj], u8p), hidden, inner, int(widths[e, proj]),
                                   ptr(np.ascontiguousarray(operands[proj, pair]), u16p), 1, ptr(expect, f32p))
        rms = np.sqrt(np.mean(expect.astype(np.float64) ** 2))
        assert np.max(np.abs(products[proj, pair] - expect)) <= PRODUCT_TOLERANCE * rms
    card.run(chain[2:])
    hidden_got = card.download(layer.hidden_offset, layer.pairs * inner * 2, np.uint16).reshape(layer.pairs, inner)
    live_pairs = live * picks
    h_got, h_want = bf16_to_f32(hidden_got[:live_pairs]).astype(np.float64), bf16_to_f32(want_hidden).astype(np.float64)
    assert np.max(np.abs(h_got - h_want)) <= 2e-2 * np.sqrt(np.mean(h_want ** 2)) + 1e-6
    got = layer.output()[:live]
    assert np.max(np.abs(got - want)) <= 4e-3 * scale, "chain output"
    say("  chain max err / rms", float(np.max(np.abs(got - want)) / scale))

    # --- the fused decode ---
    card.upload(layer.out_offset, np.zeros(rows * hidden, dtype=np.float32))
    card.run(layer.tc_launches())
    fused = layer.output()[:live]
    assert np.max(np.abs(fused - want)) <= 4e-3 * scale, "fused decode output"
    say("  fused max err / rms", float(np.max(np.abs(fused - want)) / scale))
    # the combine's other form: the same sums added to the shared expert's bfloat16 rows, in place, one rounding;
    # the float32 output is then not written
    shared = to_bf16(normals(0x5A7ED, rows * hidden) * float(scale)).reshape(rows, hidden)
    shared[0, :4] = [0x0000, 0x8000, 0x7F80, 0x7FC0]
    shared_offset = card.place(shared)
    card.upload(layer.out_offset, np.full(rows * hidden * 4, 0xEE, dtype=np.uint8))
    card.run(layer.tc_launches(shared_offset))
    joined = card.download(shared_offset, rows * hidden * 2, np.uint16).reshape(rows, hidden)
    expect = to_bf16(fused + bf16_to_f32(shared[:live]))
    both_nan = np.isnan(bf16_to_f32(joined[:live])) & np.isnan(bf16_to_f32(expect))
    assert np.array_equal(joined[:live][~both_nan], expect[~both_nan]), "sum + shared row, rounded once"
    assert np.array_equal(joined[live:], shared[live:]), "rows past the live ones keep their values (a sum of nothing is +0)"
    assert np.all(card.download(layer.out_offset, rows * hidden * 4, np.uint8) == 0xEE)
    # a row alone keeps its bits: the step of one row against row 0 of the step of all
    if live > 1:
        layer.set_rows(x, 1)
        card.run(layer.select_launch(0))
        card.run(layer.tc_launches())
        assert np.array_equal(layer.output()[0].view(np.uint32), fused[0].view(np.uint32))


def test_single_linear_config0_shape(amd, card):
    """One EXL3 linear y = (((x.suh)Hb)T)Hb.svh at 4096 x 4096, K = 4, batch 1: the chain's input, down product and
    finish launches on one job whose three matrices are the same matrix, against the double-precision definition."""
    say("single linear 4096x4096 K4")
    n = 4096
    matrix = exl3_matrix(0x5EED0000, n, n, 4)
    x = to_bf16(normals(0x5EED0001, n))
    at = card.place(matrix, 256)
    jobs = np.zeros(1, dtype=JOB_DTYPE)
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
    record.bits_per_weight, record.activation_limit = 4, 10.0
    launches = amd.launches_of(5)
    amd.check(card.lib.exl3_experts_prepare(C.byref(record), card.arena_bytes, amd.backend_table(), card.handle, 950, launches), "prepare")
    linear = amd.launches_of(3)
    linear[0], linear[1], linear[2] = launches[0], launches[3], launches[4]
    linear[0].grid[2] = 1  # the gate projection alone
    card.run(linear)
    got = card.download(record.output_offset, n * 4, np.float32)
    want = np.zeros(n)
    orc.orc_exl3_linear_f64(ptr(matrix, u8p), n, n, 4, ptr(bf16_to_f32(x).astype(np.float64), f64p), ptr(want, f64p))
    rms = np.sqrt(np.mean(want ** 2))
    say("  max err / rms", float(np.max(np.abs(got - want)) / rms))
    assert np.max(np.abs(got - want)) <= 2e-3 * rms  # fp16 operand rounding (2^-11 a value) dominates



@pytest.mark.parametrize("width", [2, 40, 3, 4, (3, 2, 4)])
def test_thin_product_instances_give_the_same_bits(amd, card, width):
    """A chain of one or two jobs takes the product kernels of one output tile a block (exl3_gate_up_<k>_thin,
    exl3_down_<k>_thin: anemone_amd/host/exl3.c); the same chain with room for 64 jobs (the others empty) takes the
    kernels of eight tiles a block. Same K slices, same order of sums: every float32 product and output bit for bit."""
    say("thin product instances, width", width)
    hidden, inner, pairs = 512, 256, 2
    widths = width if isinstance(width, tuple) else (width,) * 3  # a tuple: a width a matrix, through the record's widths table
    mixed = isinstance(width, tuple)
    width = widths[0]
    matrices = [exl3_matrix(0x7100 + widths[m] * 8 + m, *((inner, hidden) if m < 2 else (hidden, inner)), widths[m]) for m in range(3)]
    widths_at = card.place(np.full(4, widths[0] | widths[1] << 8 | widths[2] << 16, dtype=np.uint32)) if mixed else 0
    places = [card.place(m, 256) for m in matrices]
    x = to_bf16(normals(0x7200 + width, pairs * hidden)).reshape(pairs, hidden)
    outputs = []
    for job_count in (1, 64):
        jobs = np.zeros(job_count, dtype=JOB_DTYPE)
        jobs[0]["gate_offset"], jobs[0]["up_offset"], jobs[0]["down_offset"] = places
        jobs[0]["row_count"], jobs[0]["expert"] = pairs, 3
        jobs[0]["pair_index"][:pairs] = np.arange(pairs)
        jobs[0]["route_weight"][:pairs] = [0.75, 1.5]
        record = amd.Exl3ExpertRecord()
        record.jobs_offset = card.place(jobs.view(np.uint8))
        record.input_offset = card.place(x)
        record.operands_offset = card.reserve(pairs * hidden * 4)
        record.products_offset = record.output_offset = card.reserve(pairs * hidden * 8)
        record.hidden_offset = card.reserve(pairs * inner * 2)
        record.input_size, record.inner_size = hidden, inner
        record.pair_count, record.pairs_per_row, record.job_count = pairs, 1, job_count
        record.bits_per_weight, record.activation_limit, record.widths_offset = width, 10.0, widths_at
        launches = amd.launches_of(5)
        amd.check(card.lib.exl3_experts_prepare(C.byref(record), card.arena_bytes, amd.backend_table(), card.handle, 950, launches), "prepare")
        assert list(launches[1].grid) == ([inner // 16, 1, 2] if job_count == 1 else [inner // 128, 64, 2])
        card.upload(record.output_offset, np.full(pairs * hidden * 8, 0xEE, dtype=np.uint8))
        card.run(launches[0:2])
        products = card.download(record.products_offset, 2 * pairs * inner * 4, np.uint32).copy()
        card.run(launches[2:5])
        outputs.append((products, card.download(record.output_offset, pairs * hidden * 4, np.uint32).copy()))
    assert np.array_equal(outputs[0][0], outputs[1][0]), "the gate and up products"
    assert np.array_equal(outputs[0][1], outputs[1][1]), "the outputs"
    assert not np.all(outputs[0][1] == 0xEEEEEEEE)


@pytest.mark.parametrize("width", [2, 40, 3, 4])
def test_a_slice_of_outputs_gives_the_whole_matrix_bits(amd, card, width):
    """The load-time slices (bb_exl3_matrix_slice_copy, include/anemone/exl3_layout.h:28-49 of the reference): a slice of
    a matrix's outputs with all of its inputs, as its own stored matrix, through the chain's input and gate product
    launches: the float32 products of the slice's outputs are the whole matrix's, bit for bit. This is what lets a card
    take a share of a layer's columns."""
    say("slice of outputs, width", width)
    import ctypes as ct
    inputs, outputs, begin, count = 1024, 768, 256, 384

    class Slice(ct.Structure):
        _fields_ = [(name, ct.c_uint32) for name in ("input_size", "output_size", "input_begin", "input_count", "output_begin", "output_count",
                                                     "bits_per_weight", "reserved_zero")]
    matrix = exl3_matrix(0x51CE0 + width, inputs, outputs, width)
    description = Slice(inputs, outputs, 0, inputs, begin, count, width, 0)
    sliced = np.zeros(int(orc.orc_exl3_code_bytes(inputs, count, width)) + 2 * (inputs + count), dtype=np.uint8)
    lib = card.lib
    lib.bb_exl3_matrix_slice_copy.restype = ct.c_int
    lib.bb_exl3_matrix_slice_copy.argtypes = [ct.POINTER(Slice), ct.c_void_p, ct.c_size_t, ct.c_void_p, ct.c_size_t]
    assert lib.bb_exl3_matrix_slice_copy(ct.byref(description), matrix.ctypes.data, matrix.nbytes, sliced.ctypes.data, sliced.nbytes) == 0
    x = to_bf16(normals(0x51CE1, inputs))
    x_at = card.place(x)

    def products_of(stored, outs):
        at = card.place(stored, 256)
        jobs = np.zeros(1, dtype=JOB_DTYPE)
        jobs[0]["gate_offset"] = jobs[0]["up_offset"] = jobs[0]["down_offset"] = at
        jobs[0]["row_count"], jobs[0]["route_weight"][0] = 1, 1.0
        record = amd.Exl3ExpertRecord()
        record.jobs_offset = card.place(jobs.view(np.uint8))
        record.input_offset = x_at
        record.operands_offset = card.reserve(inputs * 4)
        record.products_offset = record.output_offset = card.reserve(2 * max(inputs, outs) * 4)
        record.hidden_offset = card.reserve(max(inputs, outs) * 2)
        record.input_size, record.inner_size = inputs, outs
        record.pair_count = record.pairs_per_row = record.job_count = 1
        record.bits_per_weight, record.activation_limit = width, 10.0
        launches = amd.launches_of(5)
        amd.check(card.lib.exl3_experts_prepare(C.byref(record), card.arena_bytes, amd.backend_table(), card.handle, 950, launches), "prepare")
        two = amd.launches_of(2)
        two[0], two[1] = launches[0], launches[1]
        two[0].grid[2] = two[1].grid[2] = 1  # the gate projection alone
        card.run(two)
        return card.download(record.products_offset, outs * 4, np.float32)
    whole, part = products_of(matrix, outputs), products_of(sliced, count)
    assert np.array_equal(part.view(np.uint32), whole[begin:begin + count].view(np.uint32))
    assert np.any(part != 0)
