"""GPU checks, through the C ABI, of the fused fronts of a block's sites (site_front_prepare): ONE launch for a site's mix
project, mix finish and the quantization of the sublayer's input, and for the FFN front the router's scores (in the dense
product's order) and its select as well. Every output is held byte for byte against the separate launches the front stands
for (which tests/test_gpu_site_front.py, test_gpu_router.py and test_gpu_linear.py hold against the CPU oracle), and the
hidden rows against the oracle directly."""
import ctypes as C
import sys

import numpy as np
import pytest

from _oracle import f32p, normals, orc, ptr, to_bf16, u16p
from test_gpu_site_front import front_of, oracle_dense

pytestmark = pytest.mark.gpu
STREAMS, MIXES = 4, 24


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


def snapshot(card, ranges, names):
    return {name: card.download(ranges[name].byte_offset, ranges[name].byte_count).copy() for name in names}


def poison(card, ranges, names):
    for name in names:
        card.upload(ranges[name].byte_offset, np.full(ranges[name].byte_count, 0xEE, dtype=np.uint8))


SITE_OUTPUTS = ("carried_pre", "post", "comb", "hidden", "codes", "exponents", "operands")


@pytest.mark.parametrize("rows,width,live", [(8, 4096, 8), (1, 5120, 1), (3, 2048, 3), (8, 3072, 5), (2, 5120, 2)])
def test_site_front_equals_its_launches(amd, card, rows, width, live):
    say("fused site front", rows, width, live)
    front, streams, carried = front_of(amd, card, rows, width, 3 * rows + width)
    fused = front.front_launch(live)
    kernels = amd.LinearKernels()
    amd.check(card.lib.linear_kernels_prepare(amd.backend_table(), card.handle, amd.ARITHMETIC_CLASS_GFX950, C.byref(kernels)), "linear_kernels_prepare")
    q = amd.QuantizeDescription(front.ranges["hidden"], front.ranges["codes"], front.ranges["exponents"], front.ranges["operands"], width, live)
    quantize = amd.launches_of(1)
    amd.check(card.lib.linear_quantize_prepare(C.byref(q), card.arena_bytes, C.byref(kernels), quantize), "linear_quantize_prepare")
    # the separate launches
    poison(card, front.ranges, ("mixes",) + SITE_OUTPUTS[1:])
    card.run(front.mix_project_launch(live))
    card.run(front.site_launches(live)[:1])
    card.run(quantize)
    want = snapshot(card, front.ranges, SITE_OUTPUTS)
    want_mixes = front.read("mixes", np.float32).reshape(rows, MIXES)[:live].copy()
    # the fused launch on the same streams and carried pre
    front.set_streams(streams, carried)
    poison(card, front.ranges, SITE_OUTPUTS[1:])
    card.run(fused)
    got = snapshot(card, front.ranges, SITE_OUTPUTS)
    for name in SITE_OUTPUTS:
        assert got[name].tobytes() == want[name].tobytes(), (name, np.flatnonzero(got[name] != want[name])[:8])
    scratch = front.read("scratch", np.uint8)
    assert not scratch[:16].any() and not scratch[16 + 768:16 + 776].any(), "the counters are zero again; no block gave up"
    mixes = scratch[16:16 + 8 * MIXES * 4].view(np.float32).reshape(8, MIXES)
    assert np.array_equal(mixes[:live].view(np.uint32), want_mixes.view(np.uint32))
    # and the hidden rows against the oracle
    hidden = got["hidden"].view(np.uint16).reshape(rows, width)
    for r in range(live):
        pre, post, comb, want_hidden = carried[r].copy(), np.zeros(4, np.float32), np.zeros(16, np.float32), np.zeros(width, np.uint16)
        orc.orc_hyper_mix_finish(ptr(np.ascontiguousarray(streams[r]), u16p), ptr(pre, f32p), ptr(np.ascontiguousarray(want_mixes[r]), f32p),
                                 ptr(front.constants["scale"], f32p), ptr(front.constants["base"], f32p), ptr(front.constants["norm_weight"], u16p),
                                 width, ptr(post, f32p), ptr(comb, f32p), ptr(want_hidden, u16p))
        assert np.array_equal(hidden[r], want_hidden), r
    assert np.all(hidden[live:] == 0xEEEE), "rows from the live count on are not written"
    # a second run on the front's own outputs' inputs: the scratch needs no clearing between launches
    front.set_streams(streams, carried)
    card.run(fused)
    again = snapshot(card, front.ranges, SITE_OUTPUTS)
    assert all(again[name].tobytes() == want[name].tobytes() for name in SITE_OUTPUTS)


@pytest.mark.parametrize("rows,width,live", [(8, 4096, 8), (1, 5120, 1), (5, 3072, 3)])
def test_the_two_halves_equal_the_site_front(amd, card, rows, width, live):
    """The input front and then the coefficient front (site_front_records.h:24-28 of the reference): the first stores hidden,
    codes, exponents and operands and leaves pre, post and comb alone; the second the mixes, post, comb and the site's pre."""
    say("site front in two launches", rows, width, live)
    front, streams, carried = front_of(amd, card, rows, width, 5 * rows + width)
    whole = front.front_launch(live)
    first = front.front_launch(live, kind=amd.SITE_FRONT_KIND_INPUT)
    second = front.front_launch(live, kind=amd.SITE_FRONT_KIND_COEFFICIENTS)
    poison(card, front.ranges, SITE_OUTPUTS[1:])
    card.run(whole)
    want = snapshot(card, front.ranges, SITE_OUTPUTS)
    want_scratch = front.read("scratch", np.uint8).copy()
    front.set_streams(streams, carried)
    before_pre = front.read("carried_pre", np.uint8).copy()
    poison(card, front.ranges, SITE_OUTPUTS[1:])
    card.upload(front.ranges["scratch"].byte_offset, np.zeros(amd.SITE_FRONT_SCRATCH_BYTES, np.uint8))
    card.run(first)
    middle = snapshot(card, front.ranges, SITE_OUTPUTS)
    for name in ("hidden", "codes", "exponents", "operands"):
        assert middle[name].tobytes() == want[name].tobytes(), name
    assert middle["carried_pre"].tobytes() == before_pre.tobytes() and np.all(middle["post"] == 0xEE) and np.all(middle["comb"] == 0xEE)
    card.run(second)
    got = snapshot(card, front.ranges, SITE_OUTPUTS)
    for name in SITE_OUTPUTS:
        assert got[name].tobytes() == want[name].tobytes(), name
    scratch = front.read("scratch", np.uint8)
    assert not scratch[:16].any() and not scratch[16 + 768:16 + 776].any(), "the counters are zero again"
    assert scratch[16:16 + live * MIXES * 4].tobytes() == want_scratch[16:16 + live * MIXES * 4].tobytes(), "the mixes in the scratch"
    # again without clearing anything: the second half left its counter zero
    front.set_streams(streams, carried)
    card.run(first)
    card.run(second)
    again = snapshot(card, front.ranges, SITE_OUTPUTS)
    assert all(again[name].tobytes() == want[name].tobytes() for name in SITE_OUTPUTS)


def test_a_wait_that_cannot_end_gives_up_and_every_block_leaves(amd, card):
    """The waits between the front's blocks are bounded. Forced from the host: the tickets' counter starts at the row count,
    so no block takes a row and the rows' inputs never come; the block that would form the coefficients waits its bounded
    number of polls, counts itself in gave_up and leaves without writing; the last block to leave still clears the
    counters, and the next launch on a clean scratch is whole again."""
    rows, width = 4, 2048
    say("site front, a wait that cannot end", rows, width)
    front, streams, carried = front_of(amd, card, rows, width, 77)
    fused = front.front_launch(rows)
    poison(card, front.ranges, SITE_OUTPUTS[1:])
    card.run(fused)
    want = snapshot(card, front.ranges, SITE_OUTPUTS)
    front.set_streams(streams, carried)
    poison(card, front.ranges, SITE_OUTPUTS[1:])
    before_pre = front.read("carried_pre", np.uint8).copy()
    head = np.zeros(4, dtype=np.uint32)
    head[0] = rows  # tickets
    card.upload(front.ranges["scratch"].byte_offset, head.view(np.uint8))
    card.run(fused)
    scratch = front.read("scratch", np.uint8)
    counters, tail = scratch[:16].view(np.uint32), scratch[16 + 768:16 + 776].view(np.uint32)
    assert not counters.any() and tail[0] == 0, "the last block to leave cleared the counters"
    assert tail[1] == 1, "one block gave up: the one that waits for the rows before it forms the coefficients"
    got = snapshot(card, front.ranges, SITE_OUTPUTS)
    assert got["carried_pre"].tobytes() == before_pre.tobytes()
    for name in SITE_OUTPUTS[1:]:
        assert np.all(got[name] == 0xEE), name
    # gave_up is the caller's to read: site_front_check reports it as a device error and clears it; then the front is whole again
    import ctypes as C
    count = C.c_uint32(0)
    assert card.lib.site_front_check(amd.backend_table(), card.handle, front.ranges["scratch"], card.staging, 10 ** 10,
                                     C.byref(count)) == amd.STATUS_DEVICE_ERROR and count.value == 1
    assert card.lib.site_front_check(amd.backend_table(), card.handle, front.ranges["scratch"], card.staging, 10 ** 10, C.byref(count)) == 0
    card.run(fused)
    again = snapshot(card, front.ranges, SITE_OUTPUTS)
    assert all(again[name].tobytes() == want[name].tobytes() for name in SITE_OUTPUTS)
    assert not front.read("scratch", np.uint8)[16 + 768:16 + 776].any()


def fp4_layer(amd, card, hidden, inner, experts_n, picks, rows, distinct=4, **keywords):
    from anemone_amd import workloads
    trios = [[workloads.fp4_matrix(9000 + 3 * e, inner, hidden), workloads.fp4_matrix(9001 + 3 * e, inner, hidden),
              workloads.fp4_matrix(9002 + 3 * e, hidden, inner)] for e in range(distinct)]
    router = to_bf16(normals(15, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    return amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, [trios[e % distinct] for e in range(experts_n)], router_weights_bf16=router,
                        **keywords)


@pytest.mark.parametrize("rows,width,experts_n,picks,live,form", [(8, 4096, 256, 8, 8, "fp4"), (1, 4096, 256, 8, 1, "fp4"), (8, 2048, 64, 4, 5, "fp4"),
                                                                   (6, 3072, 128, 6, 6, "exl3"), (8, 5120, 384, 6, 8, "fp4-reference-order")])
def test_ffn_front_equals_its_launches(amd, card, rows, width, experts_n, picks, live, form):
    """The last case is the reference's own model: width 5,120, 384 experts, six picks in the reference's order of sums."""
    say("fused FFN front", rows, width, experts_n, picks, live, form)
    order = 1 if form.endswith("reference-order") else 0
    form = form.split("-")[0]
    inner = 256
    if form == "fp4":
        layer = fp4_layer(amd, card, width, inner, experts_n, picks, rows)
    else:
        from test_gpu_exl3 import build_layer
        layer, _, _, _ = build_layer(amd, card, width, inner, experts_n, picks, rows, 7, [2, 3, 4])
    bias = (normals(16, experts_n) * 0.1).astype(np.float32)
    card.upload(layer.bias_offset, bias)
    mix_weights = (normals(70, MIXES * STREAMS * width) * 0.02).astype(np.float32).reshape(MIXES, STREAMS * width)
    scale, base = np.array([1.0, 0.8, 1.2], np.float32), (normals(71, MIXES) * 0.5).astype(np.float32)
    norm_weight = to_bf16(normals(72, width) * 0.1 + 1.0)
    front = amd.SiteFront(card, rows, width, mix_weights, scale, base, norm_weight, hidden_range=amd.Range(layer.x_offset, rows * width * 2))
    streams = to_bf16(normals(73, rows * STREAMS * width)).reshape(rows, STREAMS, width)
    carried = (np.abs(normals(74, rows * STREAMS)) * 0.3 + 0.1).astype(np.float32).reshape(rows, STREAMS)
    layer.set_rows(np.zeros((rows, width), np.uint16), live)  # the rows are the front's to write; the step block's live rows
    fused = front.front_launch(rows, layer, order)  # the front's rows are the select's; the step block names the live ones
    scores_range = amd.Range(layer.scores_offset, rows * experts_n * 4)
    scores = front.dense_launch(amd.Range(layer.router_offset, experts_n * width * 2), amd.Range(layer.x_offset, rows * width * 2), scores_range,
                                experts_n, width, amd.DENSE_BFLOAT16, amd.DENSE_FLOAT32, 0, 1.0, 0.0, rows)
    kernels = amd.LinearKernels()
    amd.check(card.lib.linear_kernels_prepare(amd.backend_table(), card.handle, amd.ARITHMETIC_CLASS_GFX950, C.byref(kernels)), "linear_kernels_prepare")
    q = amd.QuantizeDescription(amd.Range(layer.x_offset, rows * width * 2), front.ranges["codes"], front.ranges["exponents"], front.ranges["operands"],
                                width, rows)
    quantize = amd.launches_of(1)
    amd.check(card.lib.linear_quantize_prepare(C.byref(q), card.arena_bytes, C.byref(kernels), quantize), "linear_quantize_prepare")
    ranges = dict(front.ranges)
    ranges["scores"] = scores_range
    ranges["affinities"] = amd.Range(layer.affinities_offset, rows * experts_n * 4)
    jobs_range = layer.experts_description().jobs
    ranges["jobs"] = amd.Range(jobs_range.byte_offset, jobs_range.byte_count)
    outputs = SITE_OUTPUTS + ("scores", "affinities", "jobs")

    def separate():
        card.run(front.mix_project_launch(rows))
        card.run(front.site_launches(rows)[:1])
        card.run(scores)
        card.run(layer.select_launch(order))
        card.run(quantize)

    front.set_streams(streams, carried)
    poison(card, ranges, outputs[1:])
    separate()
    want = snapshot(card, ranges, outputs)
    front.set_streams(streams, carried)
    poison(card, ranges, outputs[1:])
    card.run(fused)
    got = snapshot(card, ranges, outputs)
    for name in outputs:
        assert got[name].tobytes() == want[name].tobytes(), (name, np.flatnonzero(got[name] != want[name])[:8])
    scratch = front.read("scratch", np.uint8)
    assert not scratch[:16].any() and not scratch[16 + 768:16 + 776].any(), "the counters are zero again; no block gave up"
    # what the launches cost on the card, queued back to back
    array = amd.launches_of(5)
    array[0], array[1], array[2], array[3], array[4] = front.mix_project_launch(rows)[0], front.site_launches(rows)[0], scores[0], \
        layer.select_launch(order)[0], quantize[0]
    for name, launches in (("separate", array), ("fused", fused)):
        times = []
        for _ in range(6):
            front.set_streams(streams, carried)
            times.append(card.measure(lambda: card.run(launches, wait=False)))
        say("  %s: %.1f us (best of 6 %.1f)" % (name, float(np.median(times)), min(times)))
