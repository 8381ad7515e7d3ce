"""Pins of the CPU oracle of the launches a site front stands for (oracle/orc_site.c): the reference's own host oracles
(tests/hyper_connection_reference.c, tests/dense_linear_reference.c, built from its sources into oracle/_ref) at their
fixed width of 5,120 -- the collapse, the norm's operand, the reciprocal root and the normed row bit for bit, Sinkhorn
within the places the reference states for a card, the dense product inside the reference's bound -- and what the
definitions fix on hand-made cases. No GPU."""
import ctypes as C

import numpy as np
import pytest

from _oracle import f32p, f64p, normals, orc, ptr, ref, to_bf16, u16p

STREAMS, MIXES, WIDTH = 4, 24, 5120
has_hyper = ref is not None and hasattr(ref, "test_hyper_sinkhorn")
has_dense = ref is not None and hasattr(ref, "test_dense_reference")


def site(seed, spread=1.0):
    mixes = (normals(seed, MIXES) * spread).astype(np.float32)
    scale = (np.abs(normals(seed + 1, 3)) + 0.1).astype(np.float32)
    base = (normals(seed + 2, MIXES) * 0.5).astype(np.float32)
    return mixes, scale, base


def sinkhorn(fn, mixes, scale, base):
    pre, post, comb = np.zeros(4, np.float32), np.zeros(4, np.float32), np.zeros(16, np.float32)
    fn(ptr(mixes, f32p), ptr(scale, f32p), ptr(base, f32p), ptr(pre, f32p), ptr(post, f32p), ptr(comb, f32p))
    return pre, post, comb


@pytest.mark.skipif(not has_hyper, reason="the reference's host oracle is not built")
@pytest.mark.parametrize("seed,spread", [(1, 1.0), (2, 0.05), (3, 4.0), (4, 20.0), (5, 1.0), (6, 8.0)])
def test_sinkhorn_within_the_places_the_reference_states(seed, spread):
    """tests/hyper_connection_reference.h:13-18: with an exponential within 2 places of the nearest, pre and post lie
    within TEST_HYPER_SINKHORN_PLACES (4) places and comb within TEST_HYPER_COMB_TOLERANCE (2^-20) of the reference's."""
    worst_places, worst_comb = 0, 0.0
    for trial in range(200):
        mixes, scale, base = site(seed * 1000 + trial * 7, spread)
        got, want = sinkhorn(orc.orc_hyper_sinkhorn, mixes, scale, base), sinkhorn(ref.test_hyper_sinkhorn, mixes, scale, base)
        for k in range(4):
            worst_places = max(worst_places, ref.test_hyper_float_places(float(got[0][k]), float(want[0][k])),
                               ref.test_hyper_float_places(float(got[1][k]), float(want[1][k])))
        worst_comb = max(worst_comb, float(np.max(np.abs(got[2].astype(np.float64) - want[2]))))
    print("worst places", worst_places, "worst comb difference %.3g" % worst_comb)
    assert worst_places <= 4 and worst_comb <= 2.0 ** -20


def test_sinkhorn_of_equal_mixes_is_the_uniform_matrix():
    """Every comb logit equal: each row is (1, 1, 1, 1) after the exponential and a quarter after the first division;
    rows and columns then sum to one and every later round divides by 1 + 1e-6. pre and post of a zero logit are a half
    (+ 1e-6) and one."""
    mixes, scale, base = np.zeros(MIXES, np.float32), np.ones(3, np.float32), np.zeros(MIXES, np.float32)
    pre, post, comb = sinkhorn(orc.orc_hyper_sinkhorn, mixes, scale, base)
    assert np.all(pre == np.float32(0.5) + np.float32(1e-6)) and np.all(post == 1.0)
    assert np.all(comb == comb[0]) and abs(float(comb[0]) - 0.25) < 1e-4
    assert abs(float(comb.reshape(4, 4).sum(axis=0)[0]) - 1.0) < 1e-5


@pytest.mark.skipif(not has_hyper, reason="the reference's host oracle is not built")
@pytest.mark.parametrize("seed,spread", [(1, 1.0), (2, 1e-3), (3, 300.0), (4, 1e30), (5, 1e-30)])
def test_collapse_operand_root_and_norm_equal_the_reference_bit_for_bit(seed, spread):
    streams = to_bf16(normals(seed, STREAMS * WIDTH) * spread).reshape(STREAMS, WIDTH)
    if seed == 4:
        streams[0, :6] = [0x7F80, 0xFF80, 0x7FC1, 0x8000, 0x0001, 0x7F7F]
    pre = (np.abs(normals(seed + 1, STREAMS)) * 0.5 + 0.01).astype(np.float32)
    weight = to_bf16(normals(seed + 2, WIDTH) * 0.1 + 1.0)
    got, want = np.zeros(WIDTH, np.uint16), np.zeros(WIDTH, np.uint16)
    orc.orc_hyper_collapse(ptr(streams, u16p), ptr(pre, f32p), WIDTH, ptr(got, u16p))
    ref.test_hyper_collapse(ptr(streams, u16p), ptr(pre, f32p), ptr(want, u16p))
    assert np.array_equal(got, want)
    operand, operand_ref = orc.orc_hyper_norm_operand(ptr(got, u16p), WIDTH), ref.test_hyper_norm_operand(ptr(want, u16p))
    assert np.float32(operand).view(np.uint32) == np.float32(operand_ref).view(np.uint32) or (np.isnan(operand) and np.isnan(operand_ref))
    if np.isfinite(operand) and operand >= 2.0 ** -126:
        factor, factor_ref = orc.orc_reciprocal_root(operand), ref.test_hyper_reciprocal_root(operand_ref)
        assert np.float32(factor).view(np.uint32) == np.float32(factor_ref).view(np.uint32)
        normed, normed_ref = np.zeros(WIDTH, np.uint16), np.zeros(WIDTH, np.uint16)
        orc.orc_hyper_norm_with(ptr(got, u16p), ptr(weight, u16p), factor, WIDTH, ptr(normed, u16p))
        ref.test_hyper_norm_with(ptr(want, u16p), ptr(weight, u16p), factor_ref, ptr(normed_ref, u16p))
        assert np.array_equal(normed, normed_ref)


@pytest.mark.skipif(not has_hyper, reason="the reference's host oracle is not built")
def test_reciprocal_root_equals_the_reference_over_a_sweep():
    values = np.concatenate([np.exp(np.linspace(np.log(1e-30), np.log(1e30), 20000)), [1.0, 4.0, 0.25, 2.0, 1e-20, 3.0]]).astype(np.float32)
    for value in values:
        a, b = orc.orc_reciprocal_root(float(value)), ref.test_hyper_reciprocal_root(float(value))
        assert np.float32(a).view(np.uint32) == np.float32(b).view(np.uint32), value


def test_mix_finish_puts_the_pieces_together_and_replaces_the_carried_pre():
    width = 512
    streams = to_bf16(normals(9, STREAMS * width)).reshape(STREAMS, width)
    mixes, scale, base = site(77)
    carried = np.array([1.0, 0.0, 0.0, 0.0], np.float32)
    weight = to_bf16(np.ones(width))
    post, comb, hidden = np.zeros(4, np.float32), np.zeros(16, np.float32), np.zeros(width, np.uint16)
    before = carried.copy()
    orc.orc_hyper_mix_finish(ptr(streams, u16p), ptr(carried, f32p), ptr(mixes, f32p), ptr(scale, f32p), ptr(base, f32p),
                             ptr(weight, u16p), width, ptr(post, f32p), ptr(comb, f32p), ptr(hidden, u16p))
    pre_want, post_want, comb_want = sinkhorn(orc.orc_hyper_sinkhorn, mixes, scale, base)
    assert np.array_equal(carried, pre_want) and np.array_equal(post, post_want) and np.array_equal(comb, comb_want)
    # the carried pre (1, 0, 0, 0) collapses to stream 0 (a negative zero becomes +0); the norm of weight 1 then scales
    # it to a root mean square of one
    collapsed = streams[0].copy()
    collapsed[collapsed == 0x8000] = 0
    values = (collapsed.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    want = values / np.sqrt(np.mean(values ** 2))
    got = (hidden.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    assert np.max(np.abs(got - want)) <= 2.0 ** -7 * np.max(np.abs(want)) and not np.array_equal(before, carried)


def dense(weight_type, weights, outputs, inputs, flags, epsilon, scale, output_type, rows):
    out = np.zeros((rows.shape[0], outputs), np.float32 if output_type == 1 else np.uint16)
    assert orc.orc_dense_linear(weight_type, weights.ctypes.data_as(C.c_void_p), outputs, inputs, flags, epsilon, scale, output_type,
                                ptr(rows, u16p), rows.shape[0], out.ctypes.data_as(C.c_void_p)) == 0
    return out


@pytest.mark.skipif(not has_dense, reason="the reference's host oracle is not built")
@pytest.mark.parametrize("weight_type,inputs,outputs,flags,output_type,scale", [
    (1, 20480, 24, 1, 1, 1.0),    # the mix project: float32 weights, the row's scale
    (0, 5120, 48, 0, 1, 1.0),     # the router's scores: bfloat16 weights
    (0, 2048, 16, 0, 0, 0.125),   # a bfloat16 output, scaled
    (1, 264, 8, 1, 0, 1.0),       # fewer chunks than threads
])
def test_dense_product_inside_the_reference_bound(weight_type, inputs, outputs, flags, output_type, scale):
    """tests/dense_linear_reference.h:14-21: a float32 output c holds where |c - y s| <= (2^-20 m + 2^-140) s."""
    rows_n, epsilon = 3, 1e-20
    rows = to_bf16(normals(5, rows_n * inputs)).reshape(rows_n, inputs)
    raw = normals(6, outputs * inputs) * 0.05
    weights = raw.astype(np.float32).reshape(outputs, inputs) if weight_type == 1 else to_bf16(raw).reshape(outputs, inputs)
    got = dense(weight_type, weights, outputs, inputs, flags, epsilon, scale, output_type, rows)
    sums, mags = np.zeros((rows_n, outputs)), np.zeros((rows_n, outputs))
    ref.test_dense_reference(weight_type, weights.ctypes.data_as(C.c_void_p), inputs, flags, epsilon, ptr(rows, u16p), rows_n, 0, outputs,
                             ptr(sums, f64p), ptr(mags, f64p))
    for index in range(rows_n * outputs):
        assert ref.test_dense_output_holds(output_type, scale, got.ctypes.data_as(C.c_void_p), index, float(sums.reshape(-1)[index]),
                                           float(mags.reshape(-1)[index])), index


def test_dense_product_of_small_integers_is_exact_whatever_the_order():
    inputs, outputs = 4096, 5
    rng = np.random.default_rng(3)
    rows = to_bf16(rng.integers(-4, 5, size=(2, inputs)).astype(np.float32))
    weights = rng.integers(-3, 4, size=(outputs, inputs)).astype(np.float32)
    values = (rows.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    want = values @ weights.astype(np.float64).T
    assert np.array_equal(dense(1, weights, outputs, inputs, 0, 0.0, 1.0, 1, rows).astype(np.float64), want)
    assert np.array_equal(dense(0, to_bf16(weights), outputs, inputs, 0, 0.0, 0.5, 1, rows).astype(np.float64), want * 0.5)
    # the row's scale: rows of +-2 have a mean square of 4, so every sum is halved (epsilon 0)
    twos = to_bf16(rng.choice([-2.0, 2.0], size=(1, inputs)).astype(np.float32))
    plain = dense(1, weights, outputs, inputs, 0, 0.0, 1.0, 1, twos)
    assert np.array_equal(dense(1, weights, outputs, inputs, 1, 0.0, 1.0, 1, twos), plain * np.float32(0.5))


def test_dense_product_order_is_the_definition():
    """One input a thread's chain cannot absorb: 2^24 then +1 in the same chain is lost, in another chain it is kept.
    Inputs 0 and 1 lie in thread 0's first chunk; input 8 in thread 1's."""
    inputs = 2048
    weights = np.zeros((1, inputs), np.float32)
    row = np.zeros((1, inputs), np.float32)
    weights[0, 0], weights[0, 1], weights[0, 8] = 2.0 ** 24, 1.0, 1.0
    row[0, 0] = row[0, 1] = row[0, 8] = 1.0
    got = dense(1, weights, 1, inputs, 0, 0.0, 1.0, 1, to_bf16(row))
    # chain of thread 0: fmaf(1, 1, 2^24) = 2^24 (the 1 is lost); thread 1 holds 1; lanes 0 and 1 meet at distance 1
    assert float(got[0, 0]) == 2.0 ** 24
    weights[0, 8], weights[0, 16] = 1.0, 1.0
    row[0, 16] = 1.0
    got = dense(1, weights, 1, inputs, 0, 0.0, 1.0, 1, to_bf16(row))
    # threads 1 and 2 hold 1 each: 2^24 + 1 (lane 1 at distance 1) is 2^24, then + 1 (lanes 2, 3 at distance 2) is 2^24
    # again, where an order that first adds the small ones would reach 2^24 + 2
    assert float(got[0, 0]) == 2.0 ** 24
