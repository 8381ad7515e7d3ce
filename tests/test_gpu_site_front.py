"""GPU checks, through the C ABI, of the launches a site front stands for (the step ahead of the routed experts): the
dense product (a site's mix project with the row's scale; the router's scores in that order) and the hyper site's mix
finish and post, against the CPU oracle (oracle/orc_site.c, which tests/test_oracle_site.py pins to the reference's own
host oracles). Everything is held bit for bit: the products' sums (the definition fixes every chain and tree), the
mixes, pre, post and comb (the exponential and the reciprocal root are this build's fixed functions on both sides), the
collapse, its norm, and the streams behind the post."""
import ctypes as C
import sys

import numpy as np
import pytest

from _oracle import f32p, normals, orc, ptr, to_bf16, u16p

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
    card = amd.Card(1 << 30)
    yield card
    card.close()


@pytest.fixture(autouse=True)
def fresh_arena(card):
    card.cursor = 256
    yield


def front_of(amd, card, rows, width, seed, spread=1.0):
    mix_weights = (normals(seed, MIXES * STREAMS * width) * 0.02).astype(np.float32).reshape(MIXES, STREAMS * width)
    scale = (np.abs(normals(seed + 1, 3)) + 0.2).astype(np.float32)
    base = (normals(seed + 2, MIXES) * 0.5).astype(np.float32)
    norm_weight = to_bf16(normals(seed + 3, width) * 0.1 + 1.0)
    front = amd.SiteFront(card, rows, width, mix_weights, scale, base, norm_weight)
    streams = to_bf16(normals(seed + 4, rows * STREAMS * width) * spread).reshape(rows, STREAMS, width)
    carried = (np.abs(normals(seed + 5, rows * STREAMS)) * 0.4 + 0.05).astype(np.float32).reshape(rows, STREAMS)
    front.set_streams(streams, carried)
    return front, streams, carried


def oracle_dense(weight_type, weights, rows, flags, epsilon, scale, output_type):
    outputs, inputs = weights.shape
    out = np.zeros((rows.shape[0], outputs), np.float32 if output_type == 1 else np.uint16)
    assert orc.orc_dense_linear(weight_type, weights.ctypes.data_as(C.c_void_p), outputs, inputs, flags, epsilon, scale, output_type,
                                ptr(rows, u16p), rows.shape[0], out.ctypes.data_as(C.c_void_p)) == 0
    return out


@pytest.mark.parametrize("rows,width,live", [(8, 4096, 8), (1, 5120, 1), (5, 1024, 3), (2, 8192, 2), (37, 1024, 37), (300, 2048, 291)])
def test_mix_project_and_finish_bit_for_bit(amd, card, rows, width, live):
    say("site front: mix project, finish", rows, width, live)
    front, streams, carried = front_of(amd, card, rows, width, 10 * rows + width)
    for name in ("mixes", "post", "comb", "hidden"):
        card.upload(front.ranges[name].byte_offset, np.full(front.ranges[name].byte_count, 0xEE, dtype=np.uint8))
    card.run(front.mix_project_launch(live))
    mixes = front.read("mixes", np.float32).reshape(rows, MIXES)
    want_mixes = oracle_dense(1, front.constants["mix_weights"], np.ascontiguousarray(streams[:live].reshape(live, -1)), 1, 1e-20, 1.0, 1)
    assert np.array_equal(mixes[:live].view(np.uint32), want_mixes.view(np.uint32))
    assert np.all(mixes[live:].view(np.uint32) == 0xEEEEEEEE)
    card.run(front.site_launches(live)[:1])
    pre, post, comb = front.read("carried_pre", np.float32).reshape(rows, 4), front.read("post", np.float32).reshape(rows, 4), front.read("comb", np.float32).reshape(rows, 16)
    hidden = front.read("hidden", np.uint16).reshape(rows, width)
    for r in range(live):
        want_pre, want_post, want_comb, want_hidden = carried[r].copy(), np.zeros(4, np.float32), np.zeros(16, np.float32), np.zeros(width, np.uint16)
        orc.orc_hyper_mix_finish(ptr(np.ascontiguousarray(streams[r]), u16p), ptr(want_pre, f32p), ptr(np.ascontiguousarray(want_mixes[r]), f32p),
                                 ptr(front.constants["scale"], f32p), ptr(front.constants["base"], f32p), ptr(front.constants["norm_weight"], u16p),
                                 width, ptr(want_post, f32p), ptr(want_comb, f32p), ptr(want_hidden, u16p))
        assert np.array_equal(pre[r].view(np.uint32), want_pre.view(np.uint32)), ("pre", r)
        assert np.array_equal(post[r].view(np.uint32), want_post.view(np.uint32)), ("post", r)
        assert np.array_equal(comb[r].view(np.uint32), want_comb.view(np.uint32)), ("comb", r)
        assert np.array_equal(hidden[r], want_hidden), ("hidden", r, np.flatnonzero(hidden[r] != want_hidden)[:8])
    assert np.array_equal(pre[live:], carried[live:]) and np.all(hidden[live:] == 0xEEEE)
    say("  comb's columns sum to", comb[0].reshape(4, 4).sum(axis=0))


def test_finish_with_specials_in_the_streams(amd, card):
    """Infinities, not-a-numbers, signed zeros and the largest values among the streams; mixes that drive the
    exponentials to their ends."""
    say("site front: specials")
    rows, width = 4, 1024
    front, streams, carried = front_of(amd, card, rows, width, 5)
    streams[0, 0, :8] = [0x7F80, 0xFF80, 0x7FC1, 0x8000, 0x0000, 0x0001, 0x8001, 0x7F7F]
    streams[1] = to_bf16(normals(3, STREAMS * width) * 1e-30).reshape(STREAMS, width)
    streams[2] = to_bf16(normals(4, STREAMS * width) * 1e18).reshape(STREAMS, width)
    front.set_streams(streams, carried)
    mixes = (normals(6, rows * MIXES) * 3.0).astype(np.float32).reshape(rows, MIXES)
    mixes[1] *= 100.0
    mixes[2, :8] = [200.0, -200.0, 1e30, -1e30, 90.0, -90.0, 0.0, -0.0]
    mixes[3, 8:] = 0.0
    card.upload(front.ranges["mixes"].byte_offset, mixes)
    card.run(front.site_launches()[:1])
    pre, post, comb = front.read("carried_pre", np.float32).reshape(rows, 4), front.read("post", np.float32).reshape(rows, 4), front.read("comb", np.float32).reshape(rows, 16)
    hidden = front.read("hidden", np.uint16).reshape(rows, width)
    for r in range(rows):
        want_pre, want_post, want_comb, want_hidden = carried[r].copy(), np.zeros(4, np.float32), np.zeros(16, np.float32), np.zeros(width, np.uint16)
        orc.orc_hyper_mix_finish(ptr(np.ascontiguousarray(streams[r]), u16p), ptr(want_pre, f32p), ptr(np.ascontiguousarray(mixes[r]), f32p),
                                 ptr(front.constants["scale"], f32p), ptr(front.constants["base"], f32p), ptr(front.constants["norm_weight"], u16p),
                                 width, ptr(want_post, f32p), ptr(want_comb, f32p), ptr(want_hidden, u16p))
        for name, got, want in (("pre", pre[r], want_pre), ("post", post[r], want_post), ("comb", comb[r], want_comb)):
            same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
            assert np.all(same), (name, r, got, want)
        assert np.array_equal(hidden[r], want_hidden), ("hidden", r)


@pytest.mark.parametrize("weight_type,outputs,inputs,rows,output_type,scale", [(0, 256, 4096, 8, 1, 1.0), (0, 384, 5120, 1, 1, 1.0),
                                                                              (0, 2048, 1024, 3, 0, 0.125), (1, 64, 264, 2, 0, 1.0),
                                                                              (0, 64, 1024, 100, 1, 1.0), (1, 20, 512, 37, 0, 0.5), (1, 20, 512, 237, 0, 0.5)])
def test_dense_products_bit_for_bit(amd, card, weight_type, outputs, inputs, rows, output_type, scale):
    """The router's scores in the dense product's order (bfloat16 weights, float32 out) and the other forms: four outputs
    a block and one, one row and several, a bfloat16 output with a scale."""
    say("dense product", weight_type, outputs, inputs, rows, output_type, scale)
    front, _, _ = front_of(amd, card, 1, 1024, 9)
    raw = normals(11, outputs * inputs) * 0.05
    weights = raw.astype(np.float32).reshape(outputs, inputs) if weight_type == 1 else to_bf16(raw).reshape(outputs, inputs)
    x = to_bf16(normals(12, rows * inputs)).reshape(rows, inputs)
    w_range = amd.Range(card.place(weights, 256), weights.nbytes)
    x_range = amd.Range(card.place(x, 256), x.nbytes)
    out_bytes = rows * outputs * (4 if output_type == 1 else 2)
    out_range = amd.Range(card.reserve(out_bytes), out_bytes)
    card.run(front.dense_launch(w_range, x_range, out_range, outputs, inputs, weight_type, output_type, 0, scale, 0.0, rows))
    got = card.download(out_range.byte_offset, out_bytes, np.float32 if output_type == 1 else np.uint16).reshape(rows, outputs)
    want = oracle_dense(weight_type, weights, x, 0, 0.0, scale, output_type)
    view = np.uint32 if output_type == 1 else np.uint16
    assert np.array_equal(got.view(view), want.view(view))


def test_site_from_streams_to_streams(amd, card):
    """A whole site around a stand-in sublayer: mix project, mix finish, then the post with the combine, the streams
    against the oracle's post of the oracle's pre-sublayer state."""
    say("site front: a whole site")
    rows, width = 8, 4096
    front, streams, carried = front_of(amd, card, rows, width, 21)
    output = to_bf16(normals(31, rows * width)).reshape(rows, width)
    sums = (normals(32, rows * width) * 2.0).astype(np.float32).reshape(rows, width)
    card.upload(front.ranges["output"].byte_offset, output)
    card.upload(front.ranges["routed_sums"].byte_offset, sums)
    finish, post = front.site_launches(combined=True)
    launches = amd.launches_of(3)
    launches[0], launches[1], launches[2] = front.mix_project_launch()[0], finish, post
    card.run(launches)
    got = front.read("streams", np.uint16).reshape(rows, STREAMS, width)
    want_mixes = oracle_dense(1, front.constants["mix_weights"], np.ascontiguousarray(streams.reshape(rows, -1)), 1, 1e-20, 1.0, 1)
    for r in range(rows):
        pre, post_of, comb, hidden = carried[r].copy(), np.zeros(4, np.float32), np.zeros(16, np.float32), np.zeros(width, np.uint16)
        orc.orc_hyper_mix_finish(ptr(np.ascontiguousarray(streams[r]), u16p), ptr(pre, f32p), ptr(np.ascontiguousarray(want_mixes[r]), f32p),
                                 ptr(front.constants["scale"], f32p), ptr(front.constants["base"], f32p), ptr(front.constants["norm_weight"], u16p),
                                 width, ptr(post_of, f32p), ptr(comb, f32p), ptr(hidden, u16p))
        want = np.zeros((STREAMS, width), np.uint16)
        orc.orc_hyper_post(ptr(np.ascontiguousarray(streams[r]), u16p), ptr(post_of, f32p), ptr(comb, f32p), ptr(np.ascontiguousarray(output[r]), u16p),
                           ptr(np.ascontiguousarray(sums[r]), f32p), width, ptr(want, u16p))
        assert np.array_equal(got[r], want), r


def test_a_layer_from_streams_to_streams(amd, card):
    """A whole FFN site of a wide step on the card, streams in and streams out: the mix project and mix finish, the
    router and its wide select, the FP4 routed experts in their wide form, the shared expert, the join. The front's rows,
    post and comb bit for bit the oracle's; the streams against the oracle's composition of its own stages; and the join
    exact on the card's own pair and shared outputs."""
    say("a layer from streams to streams")
    from anemone_amd import workloads
    from test_gpu_router_wide import oracle_wide
    from _oracle import bf16_to_f32, u32p
    E2M1, E4M3 = 3, 5
    hidden, inner, experts_n, picks, rows = 1024, 256, 64, 4, 100
    matrices = [[workloads.fp4_matrix(7000 + 3 * e, inner, hidden), workloads.fp4_matrix(7001 + 3 * e, inner, hidden),
                 workloads.fp4_matrix(7002 + 3 * e, hidden, inner)] for e in range(experts_n)]
    router = to_bf16(normals(5, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    layer = amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, matrices, router_weights_bf16=router)
    shared_matrices = [workloads.fp8_matrix(61, inner, hidden), workloads.fp8_matrix(62, inner, hidden), workloads.fp8_matrix(63, hidden, inner)]
    shared = amd.SharedExpert(layer, shared_matrices)
    mix_weights = (normals(70, MIXES * STREAMS * hidden) * 0.02).astype(np.float32).reshape(MIXES, STREAMS * hidden)
    scale, base = np.array([1.0, 0.8, 1.2], np.float32), (normals(71, MIXES) * 0.5).astype(np.float32)
    norm_weight = to_bf16(normals(72, hidden) * 0.1 + 1.0)
    front = amd.SiteFront(card, rows, hidden, mix_weights, scale, base, norm_weight, hidden_range=amd.Range(layer.x_offset, rows * hidden * 2))
    for name in ("streams", "post", "comb"):
        front.ranges[name] = shared.ranges[name]
    streams = to_bf16(normals(73, rows * STREAMS * hidden)).reshape(rows, STREAMS, hidden)
    carried = (np.abs(normals(74, rows * STREAMS)) * 0.3 + 0.1).astype(np.float32).reshape(rows, STREAMS)
    front.set_streams(streams, carried)
    layer.set_rows(np.zeros((rows, hidden), np.uint16))  # the rows are the front's to write
    card.run(front.mix_project_launch())
    card.run(front.site_launches()[:1])
    card.run(layer.projection_launch())
    wide = layer.wide_router()
    card.run(wide.launches())
    card.run(layer.quantize_launch())
    card.run(layer.wide_expert_launches(wide)[:2])
    card.run(shared.launches())
    card.run(shared.join_launch())
    # the oracle's front
    mixes = oracle_dense(1, mix_weights, np.ascontiguousarray(streams.reshape(rows, -1)), 1, 1e-20, 1.0, 1)
    x, post, comb = np.zeros((rows, hidden), np.uint16), np.zeros((rows, 4), np.float32), np.zeros((rows, 16), np.float32)
    for r in range(rows):
        pre = carried[r].copy()
        orc.orc_hyper_mix_finish(ptr(np.ascontiguousarray(streams[r]), u16p), ptr(pre, f32p), ptr(np.ascontiguousarray(mixes[r]), f32p), ptr(scale, f32p),
                                 ptr(base, f32p), ptr(norm_weight, u16p), hidden, ptr(post[r], f32p), ptr(comb[r], f32p), ptr(x[r], u16p))
    assert np.array_equal(card.download(layer.x_offset, rows * hidden * 2, np.uint16).reshape(rows, hidden), x)
    assert np.array_equal(shared.read("post", np.float32).view(np.uint32), post.reshape(-1).view(np.uint32))
    assert np.array_equal(shared.read("comb", np.float32).view(np.uint32), comb.reshape(-1).view(np.uint32))
    # its routed experts (the card's own routing of those rows), its shared expert, its join
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
    exact = streams.copy()
    pairs_card, shared_card = layer.read("pair_output", np.uint16), shared.read("output", np.uint16)
    orc.orc_expert_join(ptr(pairs_card, u16p), ptr(shared_card, u16p), ptr(exact, u16p), ptr(post, f32p), ptr(comb, f32p), None, rows, picks, hidden)
    assert np.array_equal(shared.read("streams", np.uint16).reshape(rows, STREAMS, hidden), exact)


def test_exl3_decode_into_the_shared_rows_then_the_plain_post(amd, card):
    """The EXL3 site of a decode step as the reference's fused decode runs it (include/anemone/exl3_tc_records.h:52-57):
    the combine adds the routed sums to the shared expert's bfloat16 rows in place (shared_sum 1), and the site's post
    without the combine takes those rows as the sublayer's output. Against the oracle's post of bfloat16(sum + row) of the
    card's own sums (the float32 form of the same launches), bit for bit."""
    say("EXL3 decode, shared sum, plain post")
    from test_gpu_exl3 import build_layer
    hidden, inner, experts_n, picks, rows = 1024, 256, 64, 4, 8
    layer, _, _, _ = build_layer(amd, card, hidden, inner, experts_n, picks, rows, 5, [2, 3, 4])
    x = to_bf16(normals(41, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x, rows)
    card.run(layer.projection_launch())
    card.run(layer.select_launch(0))
    card.run(layer.tc_launches())
    sums = layer.output()[:rows].copy()  # float32 [rows][hidden]
    front, streams, carried = front_of(amd, card, rows, hidden, 77)
    shared_rows = to_bf16(normals(42, rows * hidden) * float(np.sqrt(np.mean(sums.astype(np.float64) ** 2)))).reshape(rows, hidden)
    card.upload(front.ranges["output"].byte_offset, shared_rows)
    post = (normals(43, rows * STREAMS) * 0.5 + 1.0).astype(np.float32).reshape(rows, STREAMS)
    comb = (np.abs(normals(44, rows * STREAMS * STREAMS)) * 0.3).astype(np.float32).reshape(rows, STREAMS, STREAMS)
    card.upload(front.ranges["post"].byte_offset, post)
    card.upload(front.ranges["comb"].byte_offset, comb)
    card.run(layer.tc_launches(front.ranges["output"].byte_offset))
    card.run(front.site_launches(combined=False)[1:])
    got = front.read("streams", np.uint16).reshape(rows, STREAMS, hidden)
    summed = to_bf16(sums + (shared_rows.astype(np.uint32) << 16).view(np.float32))
    assert np.array_equal(front.read("output", np.uint16).reshape(rows, hidden), summed)
    for r in range(rows):
        want = np.zeros((STREAMS, hidden), np.uint16)
        orc.orc_hyper_post(ptr(np.ascontiguousarray(streams[r]), u16p), ptr(post[r], f32p), ptr(np.ascontiguousarray(comb[r]), f32p),
                           ptr(np.ascontiguousarray(summed[r]), u16p), None, hidden, ptr(want, u16p))
        assert np.array_equal(got[r], want), r
