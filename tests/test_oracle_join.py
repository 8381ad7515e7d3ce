"""Pins of the CPU oracle of the FFN site's join (oracle/orc_join.c): the reference's own host oracle test_hyper_post
(built from its sources into oracle/_ref) bit for bit at its fixed width of 5,120, and what the definition fixes on
hand-made cases. No GPU."""
import numpy as np
import pytest

from _oracle import f32p, normals, orc, ptr, ref, to_bf16, u16p

STREAMS = 4


def from_bf16(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def random_row(seed, width, spread=1.0):
    streams = to_bf16(normals(seed, STREAMS * width) * spread).reshape(STREAMS, width)
    output = to_bf16(normals(seed + 1, width) * spread)
    post = (normals(seed + 2, STREAMS) * 0.7 + 1.0).astype(np.float32)
    comb = (np.abs(normals(seed + 3, STREAMS * STREAMS)) * 0.4).astype(np.float32).reshape(STREAMS, STREAMS)
    sums = (normals(seed + 4, width) * 3.0 * spread).astype(np.float32)
    return streams, output, post, comb, sums


def post_of(streams, post, comb, output, sums):
    out = np.zeros_like(streams)
    orc.orc_hyper_post(ptr(streams, u16p), ptr(post, f32p), ptr(comb, f32p), ptr(output, u16p),
                       None if sums is None else ptr(sums, f32p), streams.shape[1], ptr(out, u16p))
    return out


@pytest.mark.skipif(ref is None or not hasattr(ref, "test_hyper_post"), reason="the reference's host oracle is not built")
@pytest.mark.parametrize("seed,spread,combined", [(1, 1.0, True), (2, 1.0, False), (3, 1e-3, True), (4, 300.0, True),
                                                   (5, 1e30, True), (6, 1e-38, False)])
def test_post_equals_the_reference_oracle_bit_for_bit(seed, spread, combined):
    width = 5120
    streams, output, post, comb, sums = random_row(seed * 10, width, spread)
    if seed == 5:  # infinities, not-a-numbers and signed zeros among the inputs
        streams[0, :8] = [0x7F80, 0xFF80, 0x7FC1, 0x8000, 0x0000, 0x0001, 0x8001, 0x7F7F]
        output[:8] = [0x7F80, 0x7F80, 0x0000, 0x8000, 0x8000, 0x0001, 0xFFFF, 0x7F7F]
        sums[:8] = [np.inf, -np.inf, 1.0, -0.0, 0.0, -0.0, 1.0, 3e38]
    want = np.zeros_like(streams)
    ref.test_hyper_post(ptr(streams, u16p), ptr(post, f32p), ptr(comb, f32p), ptr(output, u16p),
                        ptr(sums, f32p) if combined else None, ptr(want, u16p))
    got = post_of(streams, post, comb, output, sums if combined else None)
    assert np.array_equal(got, want)


def test_identity_comb_and_no_post_leave_the_streams():
    width = 256
    streams, output, _, _, sums = random_row(70, width)
    got = post_of(streams, np.zeros(STREAMS, dtype=np.float32), np.eye(STREAMS, dtype=np.float32), output, sums)
    finite = streams.copy()
    finite[finite == 0x8000] = 0  # (0 + -0) is +0
    assert np.array_equal(got, finite)


def test_one_comb_entry_moves_one_stream_and_the_post_scales_the_output():
    """comb[j][k] is the weight of source stream j in target stream k; every value a small integer so each step is
    exact and the answer is the plain formula."""
    width = 64
    rng = np.random.default_rng(5)
    values = rng.integers(-8, 9, size=(STREAMS, width)).astype(np.float32)
    y = rng.integers(-8, 9, size=width).astype(np.float32)
    s = rng.integers(-8, 9, size=width).astype(np.float32)
    comb = np.zeros((STREAMS, STREAMS), dtype=np.float32)
    comb[2, 1] = 2.0  # source 2 into target 1
    comb[0, 3] = -1.0
    post = np.array([1.0, 0.5, 0.0, 4.0], dtype=np.float32)
    got = from_bf16(post_of(to_bf16(values), post, comb, to_bf16(y), s))
    joined = s + y
    want = np.zeros((STREAMS, width), dtype=np.float32)
    want[0] = post[0] * joined
    want[1] = post[1] * joined + 2.0 * values[2]
    want[2] = 0.0
    want[3] = post[3] * joined - values[0]
    assert np.array_equal(got, want)
    transposed = from_bf16(post_of(to_bf16(values), post, np.ascontiguousarray(comb.T), to_bf16(y), s))
    assert not np.array_equal(transposed, want)  # a transposed comb fails


def test_join_is_the_row_sum_then_the_post():
    rows, picks, width = 3, 5, 128
    pairs = to_bf16(normals(11, rows * picks * width)).reshape(rows * picks, width)
    shared = to_bf16(normals(12, rows * width)).reshape(rows, width)
    streams = to_bf16(normals(13, rows * STREAMS * width)).reshape(rows, STREAMS, width)
    post = (normals(14, rows * STREAMS) + 1.0).astype(np.float32).reshape(rows, STREAMS)
    comb = np.abs(normals(15, rows * 16)).astype(np.float32).reshape(rows, STREAMS, STREAMS)
    joined = streams.copy()
    sums = np.zeros((rows, width), dtype=np.float32)
    orc.orc_expert_join(ptr(pairs, u16p), ptr(shared, u16p), ptr(joined, u16p), ptr(post, f32p), ptr(comb, f32p),
                        ptr(sums, f32p), rows, picks, width)
    for row in range(rows):
        want_sums = np.zeros(width, dtype=np.float32)
        for slot in range(picks):  # ascending slot order from +0, float32
            want_sums = want_sums + from_bf16(pairs[row * picks + slot])
        assert np.array_equal(sums[row], want_sums)
        assert np.array_equal(joined[row], post_of(streams[row], post[row], comb[row], shared[row], want_sums))
    again = streams.copy()
    orc.orc_expert_join(ptr(pairs, u16p), ptr(shared, u16p), ptr(again, u16p), ptr(post, f32p), ptr(comb, f32p),
                        None, rows, picks, width)
    assert np.array_equal(again, joined)


def test_trunk_hidden_is_the_hidden_step_with_weight_one():
    count = 512
    gate, up = to_bf16(normals(21, count) * 4.0), to_bf16(normals(22, count) * 4.0)
    hidden = np.zeros(count, dtype=np.uint16)
    orc.orc_trunk_hidden(ptr(gate, u16p), ptr(up, u16p), 7.0, count, ptr(hidden, u16p))
    g, u = from_bf16(gate).astype(np.float64), from_bf16(up).astype(np.float64)
    g, u = np.minimum(g, 7.0), np.clip(u, -7.0, 7.0)
    want = g / (1.0 + np.exp(-g)) * u
    got = from_bf16(hidden).astype(np.float64)
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -7 + 1e-30)
