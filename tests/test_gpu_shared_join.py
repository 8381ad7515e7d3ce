"""GPU parity, through the C ABI, of the step behind the routed experts: the shared expert's trunk products
(WEIGHT_FORMAT_E4M3_SCALED) within the reference's own bound of the exact block sums, its thin, wide and interleaved
instances byte for byte equal (the reference holds its wide instances to the thin one's bits,
include/anemone/linear_records.h:114-125), the hidden step and the whole shared expert against the CPU oracle, and the
FFN site's join bit for bit against the oracle and byte for byte equal to the launches it stands for (the reference's
bar for its fused launches, include/anemone/expert_fused_records.h:10-12)."""
import ctypes as C
import sys

import numpy as np
import pytest

from _oracle import f32p, f64p, normals, orc, ptr, to_bf16, u8p, u16p, u32p
from test_gpu_linear import ALLOWANCE_GFX950, oracle_quantize

pytestmark = pytest.mark.gpu
E2M1, E4M3 = 3, 5
STREAMS = 4


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


def build(amd, card, hidden, inner, rows, picks, seed, fmt=E2M1, experts_n=64, shared_inner=None, **more):
    """A layer of a few distinct routed experts, and its shared expert of three E4M3 matrices."""
    from anemone_amd import workloads
    matrix = workloads.fp4_matrix if fmt == E2M1 else workloads.fp8_matrix
    trios = [[matrix(seed * 1000 + 3 * e, inner, hidden), matrix(seed * 1000 + 3 * e + 1, inner, hidden),
              matrix(seed * 1000 + 3 * e + 2, hidden, inner)] for e in range(4)]
    router = to_bf16(normals(seed + 5, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    layer = amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, [trios[e % 4] for e in range(experts_n)],
                         router_weights_bf16=router, weight_format=fmt)
    si = inner if shared_inner is None else shared_inner
    shared_matrices = [workloads.fp8_matrix(seed * 77 + 1, si, hidden), workloads.fp8_matrix(seed * 77 + 2, si, hidden),
                       workloads.fp8_matrix(seed * 77 + 3, hidden, si)]
    shared = amd.SharedExpert(layer, shared_matrices, inner=si, **more)
    return layer, shared, shared_matrices


def site_of(seed, rows, hidden):
    streams = to_bf16(normals(seed, rows * STREAMS * hidden)).reshape(rows, STREAMS, hidden)
    post = (normals(seed + 1, rows * STREAMS) * 0.5 + 1.0).astype(np.float32).reshape(rows, STREAMS)
    comb = (np.abs(normals(seed + 2, rows * STREAMS * STREAMS)) * 0.3).astype(np.float32).reshape(rows, STREAMS, STREAMS)
    return streams, post, comb


def trunk_launch(amd, card, layer, shared, indices, slices, rows, form, outputs):
    d = amd.TrunkQuantizedDescription()
    for m, index in enumerate(indices):
        d.matrices[m] = shared.matrix(index, slices)
        d.matrices[m].wide_form = form
        d.outputs[m] = outputs[m]
    d.codes, d.exponents, d.operands = layer.ranges["codes"], layer.ranges["exponents"], layer.ranges["operands"]
    d.matrix_count, d.row_count = len(indices), rows
    launch = amd.launches_of(1)
    amd.check(card.lib.linear_trunk_quantized_prepare(C.byref(d), card.arena_bytes, C.byref(layer.kernels), launch), "linear_trunk_quantized_prepare")
    return launch


@pytest.mark.parametrize("slices,rows", [(1, 5), (2, 8), (4, 1), (8, 7)])
def test_trunk_products_within_the_reference_bound(amd, card, slices, rows):
    say("trunk products, slices", slices, "rows", rows)
    hidden, inner = 1024, 1056  # 33 strips: the last holds one tile of its own
    layer, shared, matrices = build(amd, card, hidden, 256, rows, 1, 3, shared_inner=inner)
    x = to_bf16(normals(7, rows * hidden).reshape(rows, hidden) * np.repeat([0.01, 1.0, 100.0, 1.0], hidden // 4))
    layer.set_rows(x)
    card.run(layer.quantize_launch())
    codes, exps, _, _ = oracle_quantize(x)
    outputs = [shared.ranges["gate_output"], shared.ranges["up_output"]]
    for name in ("gate_output", "up_output"):
        card.upload(shared.ranges[name].byte_offset, np.full(shared.ranges[name].byte_count, 0xEE, dtype=np.uint8))
    card.run(trunk_launch(amd, card, layer, shared, (0, 1), slices, rows, amd.LINEAR_WIDE_GROUP_BLOCKS, outputs))
    worst = 0.0
    for m, name in enumerate(("gate_output", "up_output")):
        got = shared.read(name, np.uint16).reshape(rows, inner)
        sums, mags = np.zeros((rows, inner)), np.zeros((rows, inner))
        assert orc.orc_linear_products(E4M3, inner, hidden, ptr(matrices[m], u8p), 0, inner, ptr(codes, u8p), ptr(exps, u8p), rows,
                                       ptr(sums, f64p), ptr(mags, f64p)) == 0
        for row in range(rows):
            for o in range(inner):
                assert orc.orc_linear_within_allowance(int(got[row, o]), sums[row, o], mags[row, o], hidden, slices, ALLOWANCE_GFX950), (name, row, o)
            worst = max(worst, float(np.mean(to_bf16(sums[row].astype(np.float32)) != got[row])))
    say("  outputs that are not the exact sum rounded once: %.4f" % worst)
    assert worst < 0.05  # an informal figure; the bound above is the bar


@pytest.mark.parametrize("slices,rows,inner", [(1, 70, 1056), (1, 200, 512), (4, 21, 1056), (1, 9, 160)])
def test_wide_and_interleaved_instances_have_the_thin_bits(amd, card, slices, rows, inner):
    """Every form of a launch of many rows against thin launches of its groups of eight rows, byte for byte."""
    say("trunk forms, slices", slices, "rows", rows, "inner", inner)
    hidden = 512
    layer, shared, _ = build(amd, card, hidden, 256, rows, 1, 4, shared_inner=inner)
    x = to_bf16(normals(8, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x)
    card.run(layer.quantize_launch())
    names = ("gate_output", "up_output")
    outputs = [shared.ranges[name] for name in names]

    def run(form):
        for name in names:
            card.upload(shared.ranges[name].byte_offset, np.full(shared.ranges[name].byte_count, 0xEE, dtype=np.uint8))
        card.run(trunk_launch(amd, card, layer, shared, (0, 1), slices, rows, form, outputs))
        return [shared.read(name, np.uint16).reshape(rows, inner).copy() for name in names]
    # thin launches, eight rows at a time: the same arrays from the group's first row on
    want = [np.zeros((rows, inner), dtype=np.uint16) for _ in names]
    for first in range(0, rows, 8):
        count = min(8, rows - first)
        d = amd.TrunkQuantizedDescription()
        for m in range(2):
            d.matrices[m] = shared.matrix(m, slices)
            d.outputs[m] = amd.Range(outputs[m].byte_offset + first * inner * 2, count * inner * 2)
        d.codes = amd.Range(layer.ranges["codes"].byte_offset + first * hidden, count * hidden)
        d.exponents = amd.Range(layer.ranges["exponents"].byte_offset + first * hidden // 32, count * hidden // 32)
        d.operands = amd.Range(layer.ranges["operands"].byte_offset + first * hidden * 2, count * hidden * 2)
        d.matrix_count, d.row_count = 2, count
        launch = amd.launches_of(1)
        amd.check(card.lib.linear_trunk_quantized_prepare(C.byref(d), card.arena_bytes, C.byref(layer.kernels), launch), "thin")
        assert launch[0].grid[1] == 1 and launch[0].block[0] == 64 * slices
        card.run(launch)
    thin = [shared.read(name, np.uint16).reshape(rows, inner).copy() for name in names]
    forms = [amd.LINEAR_WIDE_GROUP_BLOCKS, amd.LINEAR_WIDE_TILE_BLOCKS] + ([amd.LINEAR_INTERLEAVED_CHUNK_BLOCKS] if slices == 1 else [])
    for form in forms:
        got = run(form)
        for m, name in enumerate(names):
            differing = int(np.count_nonzero(got[m] != thin[m]))
            say("  form %d %s: %d of %d values differ" % (form, name, differing, thin[m].size))
            assert differing == 0


@pytest.mark.parametrize("rows,form,slices", [(6, 0, (4, 2)), (8, 0, (1, 1)), (100, 2, (1, 1)), (37, 0, (2, 4))])
def test_shared_expert_against_oracle(amd, card, rows, form, slices):
    """The four launches against the oracle's layer of one expert that takes every row with a weight of 1."""
    say("shared expert", rows, form, slices)
    hidden, inner = 512, 640
    layer, shared, matrices = build(amd, card, hidden, 256, rows, 1, 6, shared_inner=inner, gate_up_slices=slices[0],
                                    down_slices=slices[1], wide_form=form)
    x = to_bf16(normals(9, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x)
    card.run(layer.quantize_launch())
    card.run(shared.launches())
    pointers = (C.c_void_p * 3)(*[m.ctypes.data for m in matrices])
    experts, weights = np.zeros((rows, 1), dtype=np.uint32), np.ones((rows, 1), dtype=np.float32)
    want_rows = np.zeros((rows, hidden), dtype=np.float32)
    want_hidden, want_output = np.zeros((rows, inner), dtype=np.uint16), np.zeros((rows, hidden), dtype=np.uint16)
    orc.orc_linear_moe_layer(E4M3, ptr(x, u16p), rows, hidden, inner, 1, ptr(experts, u32p), ptr(weights, f32p), 1, pointers,
                             layer.limit, ptr(want_rows, f32p), ptr(want_hidden, u16p), ptr(want_output, u16p), 8)
    # the hidden step bit for bit from the card's own gate and up
    gate, up = shared.read("gate_output", np.uint16), shared.read("up_output", np.uint16)
    hidden_bits = np.zeros(rows * inner, dtype=np.uint16)
    orc.orc_trunk_hidden(ptr(gate, u16p), ptr(up, u16p), layer.limit, rows * inner, ptr(hidden_bits, u16p))
    assert np.array_equal(shared.read("hidden", np.uint16), hidden_bits)
    from _oracle import bf16_to_f32
    got, want = bf16_to_f32(shared.read("output", np.uint16)).astype(np.float64), bf16_to_f32(want_output.reshape(-1)).astype(np.float64)
    error = np.sqrt(np.mean((got - want) ** 2) / np.mean(want ** 2))
    say("  output rms error vs oracle: %.2e" % error)
    assert error < 2e-2


def routed_step(card, layer, x, live=None):
    layer.set_rows(x, live)
    card.run(layer.projection_launch())
    card.run(layer.select_launch(0))
    card.run(layer.quantize_launch())
    card.run(layer.expert_launches())


@pytest.mark.parametrize("rows,picks,hidden,row_sums", [(8, 4, 1024, True), (3, 8, 2048, False), (300, 2, 1024, True), (1, 1, 1024, True)])
def test_join_bit_for_bit(amd, card, rows, picks, hidden, row_sums):
    """expert_join of arbitrary pair outputs, shared outputs and streams (infinities, not-a-numbers and signed zeros
    among them) against the oracle, every bit; and against expert_row_sum_entry + hyper_post_entry, every byte."""
    say("join", rows, picks, hidden, row_sums)
    layer, shared, _ = build(amd, card, hidden, 256, rows, picks, 12)
    pairs = to_bf16(normals(20, rows * picks * hidden) * 2.0).reshape(rows * picks, hidden)
    output = to_bf16(normals(21, rows * hidden)).reshape(rows, hidden)
    streams, post, comb = site_of(22, rows, hidden)
    pairs[0, :8] = [0x7F80, 0xFF80, 0x7FC1, 0x8000, 0x0000, 0x0001, 0x8001, 0x7F7F]
    output[0, :8] = [0x7F80, 0x7F80, 0x0000, 0x8000, 0x8000, 0x0001, 0xFFFF, 0x7F7F]
    streams[0, 1, :8] = [0x7F80, 0x0000, 0x8000, 0x8000, 0xFFC0, 0x0001, 0x7F7F, 0xFF7F]
    card.upload(layer.ranges["pair_output"].byte_offset, pairs)
    card.upload(shared.ranges["output"].byte_offset, output)
    shared.set_site(streams, post, comb)
    card.upload(shared.ranges["row_sums"].byte_offset, np.full(rows * hidden * 4, 0xEE, dtype=np.uint8))
    card.run(shared.join_launch(row_sums=row_sums))
    got_streams = shared.read("streams", np.uint16).reshape(rows, STREAMS, hidden)
    got_sums = shared.read("row_sums", np.float32).reshape(rows, hidden)
    want_streams, want_sums = streams.copy(), np.zeros((rows, hidden), dtype=np.float32)
    orc.orc_expert_join(ptr(pairs, u16p), ptr(output, u16p), ptr(want_streams, u16p), ptr(post, f32p), ptr(comb, f32p), ptr(want_sums, f32p),
                        rows, picks, hidden)
    assert np.array_equal(got_streams, want_streams)
    if row_sums:
        assert np.array_equal(got_sums.view(np.uint32), want_sums.view(np.uint32))
    else:
        assert np.all(shared.read("row_sums") == 0xEE)
    # the two launches the join stands for
    shared.set_site(streams, post, comb)
    card.run(layer.expert_launches()[3:4])
    card.run(shared.post_launch())
    assert np.array_equal(shared.read("streams", np.uint16).reshape(rows, STREAMS, hidden), want_streams)
    assert np.array_equal(layer.read("row_output", np.float32).reshape(rows, hidden).view(np.uint32), want_sums.view(np.uint32))


@pytest.mark.parametrize("rows,slices,hidden,row_sums", [(8, 1, 1024, True), (5, 4, 1056 + 992, False), (1, 2, 1024, True)])
def test_shared_join_equals_the_separate_launches(amd, card, rows, slices, hidden, row_sums):
    """expert_shared_join_<S> against trunk_linear_quantized_<S> of the down and expert_join behind it, every byte."""
    say("shared join", rows, slices, hidden, row_sums)
    picks, inner = 4, 512
    layer, shared, _ = build(amd, card, hidden, inner, rows, picks, 14, down_slices=slices)
    x = to_bf16(normals(30, rows * hidden)).reshape(rows, hidden)
    routed_step(card, layer, x)
    card.run(shared.launches())
    streams, post, comb = site_of(31, rows, hidden)
    names = ("output", "streams", "row_sums")

    def run(launches):
        shared.set_site(streams, post, comb)
        for name in ("output", "row_sums"):
            card.upload(shared.ranges[name].byte_offset, np.full(shared.ranges[name].byte_count, 0xEE, dtype=np.uint8))
        for launch in launches:
            card.run(launch)
        return [shared.read(name).copy() for name in names]
    separate = run([shared.launches()[3:4], shared.join_launch(row_sums=row_sums)])
    fused = run([shared.shared_join_launch(row_sums=row_sums)])
    for name, a, b in zip(names, separate, fused):
        differing = int(np.count_nonzero(a != b))
        say("  %s: %d of %d bytes differ" % (name, differing, a.size))
        assert differing == 0
    assert not np.all(fused[1] == streams.view(np.uint8).reshape(-1))


def test_layer_with_shared_expert_and_join_against_oracle(amd, card):
    """The whole FFN site of a wide step: routed experts in their wide form, the shared expert in its interleaved form,
    the join; streams against the oracle's join of the oracle's own routed and shared outputs."""
    say("layer with shared expert and join")
    from test_gpu_router_wide import oracle_wide
    from _oracle import bf16_to_f32
    hidden, inner, experts_n, picks, rows = 1024, 256, 64, 4, 150
    from anemone_amd import workloads
    matrices = [[workloads.fp4_matrix(9000 + 3 * e, inner, hidden), workloads.fp4_matrix(9001 + 3 * e, inner, hidden),
                 workloads.fp4_matrix(9002 + 3 * e, hidden, inner)] for e in range(experts_n)]
    router = to_bf16(normals(5, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    layer = amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, matrices, router_weights_bf16=router)
    shared_matrices = [workloads.fp8_matrix(41, inner, hidden), workloads.fp8_matrix(42, inner, hidden), workloads.fp8_matrix(43, hidden, inner)]
    shared = amd.SharedExpert(layer, shared_matrices)
    x = to_bf16(normals(9, rows * hidden)).reshape(rows, hidden)
    streams, post, comb = site_of(50, rows, hidden)
    layer.set_rows(x)
    shared.set_site(streams, post, comb)
    card.run(layer.projection_launch())
    wide = layer.wide_router()
    card.run(wide.launches())
    card.run(layer.quantize_launch())
    card.run(layer.wide_expert_launches(wide)[:2])
    card.run(shared.launches())
    card.run(shared.join_launch())
    scores = card.download(layer.scores_offset, rows * experts_n * 4, np.float32).reshape(rows, experts_n)
    _, experts, weights, _, _, _, _ = oracle_wide(layer, scores, np.zeros(experts_n, dtype=np.float32), rows)
    pointers = (C.c_void_p * (experts_n * 3))(*[m.ctypes.data for trio in matrices for m in trio])
    routed_rows, routed_pairs = np.zeros((rows, hidden), dtype=np.float32), np.zeros((rows * picks, hidden), dtype=np.uint16)
    orc.orc_linear_moe_layer(E2M1, ptr(x, u16p), rows, hidden, inner, picks, ptr(np.ascontiguousarray(experts), u32p),
                             ptr(np.ascontiguousarray(weights), f32p), experts_n, pointers, layer.limit, ptr(routed_rows, f32p), None,
                             ptr(routed_pairs, u16p), 8)
    shared_pointers = (C.c_void_p * 3)(*[m.ctypes.data for m in shared_matrices])
    one, ones = np.zeros((rows, 1), dtype=np.uint32), np.ones((rows, 1), dtype=np.float32)
    unused, shared_output = np.zeros((rows, hidden), dtype=np.float32), np.zeros((rows, hidden), dtype=np.uint16)
    orc.orc_linear_moe_layer(E4M3, ptr(x, u16p), rows, hidden, inner, 1, ptr(one, u32p), ptr(ones, f32p), 1, shared_pointers, layer.limit,
                             ptr(unused, f32p), None, ptr(shared_output, u16p), 8)
    want = streams.copy()
    orc.orc_expert_join(ptr(routed_pairs, u16p), ptr(shared_output, u16p), ptr(want, u16p), ptr(post, f32p), ptr(comb, f32p), None, rows, picks, hidden)
    got = bf16_to_f32(shared.read("streams", np.uint16)).astype(np.float64)
    wanted = bf16_to_f32(want.reshape(-1)).astype(np.float64)
    error = np.sqrt(np.mean((got - wanted) ** 2) / np.mean(wanted ** 2))
    say("  streams rms error vs oracle: %.2e" % error)
    assert error < 2e-2
    # and the join alone is exact on the card's own pair and shared outputs
    exact = streams.copy()
    pairs_card, shared_card = layer.read("pair_output", np.uint16), shared.read("output", np.uint16)
    orc.orc_expert_join(ptr(pairs_card, u16p), ptr(shared_card, u16p), ptr(exact, u16p), ptr(post, f32p), ptr(comb, f32p), None, rows, picks, hidden)
    assert np.array_equal(shared.read("streams", np.uint16).reshape(rows, STREAMS, hidden), exact)
