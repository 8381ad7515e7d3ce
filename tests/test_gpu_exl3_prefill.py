"""GPU parity of the prefill form of the EXL3 routed experts (pairs sorted by expert, grouped GEMM with the trellis
decode fused into the weight tile loads) against the CPU oracle's double-precision layer, through the C ABI. The bound
is the fused decode's: 4e-3 of the output's rms (the reference holds its tensor-core forms to 2e-3 rms of its chain,
tests/exl3_tc_card_test.c:40-41, and its probe to 2e-3 of rms against double,
tools/measure/trellis_expert_probe.cu:73)."""
import ctypes as C
import sys

import numpy as np
import pytest

from _oracle import f32p, normals, orc, ptr, splitmix_words, to_bf16, exl3_matrix, u8p, u16p, u32p

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
    card = amd.Card(2 << 30)
    yield card
    card.close()


@pytest.fixture(autouse=True)
def fresh_arena(card):
    card.cursor = 256
    yield


def build_layer(amd, card, hidden, inner, experts_n, picks, rows, seed, width_choices):
    draws = splitmix_words(seed, experts_n * 3) % np.uint64(len(width_choices))
    widths = np.array(width_choices, dtype=np.uint32)[draws.astype(np.int64)].reshape(experts_n, 3)
    matrices = [[exl3_matrix(seed * 1000 + 3 * e + 0, hidden, inner, int(widths[e, 0])),
                 exl3_matrix(seed * 1000 + 3 * e + 1, hidden, inner, int(widths[e, 1])),
                 exl3_matrix(seed * 1000 + 3 * e + 2, inner, hidden, int(widths[e, 2]))] for e in range(experts_n)]
    router = to_bf16(normals(seed + 5, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    layer = amd.Exl3Layer(card, hidden, inner, experts_n, picks, rows, matrices, widths, router_weights_bf16=router,
                          affinity_kind=1, limit=10.0)
    return layer, matrices, widths


def oracle_layer(layer, x, experts, weights, matrices, widths, threads=8):
    rows, H, I, P, E = layer.rows, layer.H, layer.I, layer.P, layer.E
    pointers = (C.c_void_p * (E * 3))(*[m.ctypes.data for trio in matrices for m in trio])
    out = np.zeros((rows, H), dtype=np.float32)
    widths8 = np.ascontiguousarray(widths.astype(np.uint8))
    orc.orc_exl3_moe_layer(ptr(x, u16p), rows, H, I, P, ptr(experts, u32p), ptr(weights, f32p), E, pointers, ptr(widths8, u8p),
                           layer.limit, ptr(out, f32p), None, None, threads)
    return out


@pytest.mark.parametrize("hidden,inner,experts_n,picks,rows,width_choices,skew", [
    (512, 256, 64, 4, 300, [2, 3, 4], 1.5),   # a few experts with more than one chunk of pairs, others ragged
    (512, 384, 64, 8, 70, [3], 0.0),          # one width; 384 outputs: a GEMM block whose last wavefronts lie past the matrix
    (256, 128, 64, 2, 9, [40, 4], 0.0),       # K = 2.5 among the widths; chunks of one or two pairs, experts without any
])
def test_prefill_layer_against_oracle(amd, card, hidden, inner, experts_n, picks, rows, width_choices, skew):
    say("prefill", hidden, inner, experts_n, picks, rows, width_choices, skew)
    layer, matrices, widths = build_layer(amd, card, hidden, inner, experts_n, picks, rows, 21, width_choices)
    x = to_bf16(normals(31, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x, rows)
    bias = (-skew * np.log(1.0 + np.arange(experts_n))).astype(np.float32)
    card.upload(layer.bias_offset, bias)
    card.run(layer.projection_launch())
    wide = layer.wide_router()
    card.run(wide.launches()[0:1])  # the picks of every row
    picks_table = wide.read("picks", np.dtype([("expert", "<u4"), ("route_weight", "<f4")])).reshape(rows, picks)
    experts = np.ascontiguousarray(picks_table["expert"])
    weights = np.ascontiguousarray(picks_table["route_weight"])
    launches = layer.tcp_launches(wide.ranges["picks"].byte_offset)
    assert len(launches) == 7
    # poison the sort's tables and the output: everything read must have been written by the call
    layout = layer.tcp_layout
    card.upload(layer.tcp_workspace_offset, np.full(layout["operands"], 0xA5, dtype=np.uint8))
    card.upload(layer.out_offset, np.full(rows * hidden * 4, 0xFF, dtype=np.uint8))
    card.run(launches)
    # the route: sorted by expert, rows ascending; place_of its inverse; chunks of at most EXL3_TCP_CHUNK_PAIRS of one expert
    pairs = rows * picks
    sorted_pairs = card.download(layer.tcp_workspace_offset + layout["sorted"], pairs * 4, np.uint32)
    place_of = card.download(layer.tcp_workspace_offset + layout["place_of"], pairs * 4, np.uint32)
    want_sorted = np.argsort(experts.reshape(-1), kind="stable").astype(np.uint32)
    assert np.array_equal(sorted_pairs, want_sorted)
    assert np.array_equal(place_of[sorted_pairs], np.arange(pairs, dtype=np.uint32))
    used = int(card.download(layer.tcp_workspace_offset + layout["header"], 4, np.uint32)[0])
    chunks = card.download(layer.tcp_workspace_offset + layout["chunks"], layout["chunk_capacity"] * 16, np.uint32).reshape(-1, 4)
    counts = np.bincount(experts.reshape(-1), minlength=experts_n)
    most = amd.EXL3_TCP_CHUNK_PAIRS
    assert used == int(((counts + most - 1) // most).sum()) and not chunks[used:].any()
    assert int(chunks[:used, 2].sum()) == pairs and chunks[:used, 2].max() <= most
    assert np.array_equal(chunks[:used, 1], np.concatenate([[0], np.cumsum(chunks[:used, 2])[:-1]]))
    say("  chunks %d, the longest run %d pairs" % (used, counts.max()))
    # the operands are bit-defined: fp16(H128(bf16 x, fp16 suh) / sqrt(128)), by place, gate then up. The down pass has
    # taken the first array since; run the route and the operands once more and read both
    card.run(launches[0:3])
    operands = card.download(layer.tcp_workspace_offset + layout["operands"], 2 * pairs * hidden * 2, np.uint16).reshape(2, pairs, hidden)
    for place in sorted(set(list(range(0, pairs, max(1, pairs // 40))) + [pairs - 1])):
        pair = int(sorted_pairs[place])
        e = int(experts.reshape(-1)[pair])
        for proj in range(2):
            cb = int(orc.orc_exl3_code_bytes(hidden, inner, int(widths[e, proj])))
            suh = np.ascontiguousarray(matrices[e][proj][cb:cb + 2 * hidden]).view(np.uint16)
            expect = np.zeros(hidden, dtype=np.uint16)
            orc.orc_exl3_operand(ptr(x[pair // picks], u16p), ptr(suh, u16p), hidden, ptr(expect, u16p))
            assert np.array_equal(operands[proj, place], expect), ("operands are bit-defined", place, proj)
    card.run(launches)
    got = layer.output()
    want = oracle_layer(layer, x, experts, weights, matrices, widths)
    scale = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    error = float(np.max(np.abs(got - want))) / scale
    say("  max error %.2e of the output's rms" % error)
    assert error <= 4e-3


def test_prefill_equals_fused_decode_on_the_same_rows(amd, card):
    """Eight rows through the fused decode and through the prefill form: the same operands, weights and float32 chains
    cut differently along k (the decode's slices against one chain): equal within float32 rounding of the sums."""
    say("prefill against the fused decode")
    hidden, inner, experts_n, picks, rows = 512, 256, 64, 4, 8
    layer, matrices, widths = build_layer(amd, card, hidden, inner, experts_n, picks, rows, 22, [2, 3, 4])
    x = to_bf16(normals(33, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x, rows)
    card.run(layer.projection_launch())
    card.run(layer.select_launch(0))
    card.run(layer.tc_launches())
    decode = layer.output().copy()
    wide = layer.wide_router()
    card.run(wide.launches()[0:1])
    card.run(layer.tcp_launches(wide.ranges["picks"].byte_offset))
    prefill = layer.output()
    scale = float(np.sqrt(np.mean(decode.astype(np.float64) ** 2)))
    error = float(np.max(np.abs(prefill - decode))) / scale
    say("  max difference %.2e of rms" % error)
    assert error <= 2e-4
