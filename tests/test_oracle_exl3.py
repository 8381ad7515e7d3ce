"""Pins the EXL3 part of the CPU oracle: against the reference's known answers (tests/golden/reference_kat.json),
against what the mathematics fixes (closed forms, bijections, orthogonality, an independent bit walk), and against
the reference's own C oracles (oracle/_ref) where that library was built."""
import json
import os

import numpy as np
import pytest

from _oracle import (C, f32p, f64p, orc, ptr, ref, splitmix_words, u8p, u16p, u32p, exl3_matrix, normals, to_bf16)

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kat.json")))
WIDTHS = [(2, 4), (40, 5), (3, 6), (4, 8)]


def fnv_states(states):
    digest = 0xCBF29CE484222325
    for value in states.reshape(-1):
        for byte in (int(value) & 0xFF, int(value) >> 8):
            digest = ((digest ^ byte) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return digest


def python_state(tile_bytes, bits_x2, position):
    """Independent restatement: walk the 16 bits of the window one at a time."""
    ring = 256 * bits_x2 // 2
    end = (position + 1) * bits_x2 // 2
    state = 0
    for bit in range(16):
        at = (end + ring - 16 + bit) % ring
        word = int.from_bytes(tile_bytes[at // 32 * 4: at // 32 * 4 + 4], "little")
        state = (state << 1) | ((word >> (31 - at % 32)) & 1)
    return state


@pytest.mark.parametrize("case", KAT["exl3_widths"], ids=lambda c: "stored%d" % c["stored"])
def test_known_answer_states(case):
    stored, bits_x2 = case["stored"], case["bits_x2"]
    assert orc.orc_exl3_bits_x2(stored) == bits_x2
    assert orc.orc_exl3_matrix_bytes(2304, 5120, stored) == case["expert_bytes"]
    tile_words = 256 * bits_x2 // 2 // 32
    words = (splitmix_words(0x5EED0000 + stored, 4 * tile_words) & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    states = np.zeros((32, 32), dtype=np.uint16)
    orc.orc_exl3_states(ptr(words.view(np.uint8), u8p), 32, 32, stored, ptr(states, u16p))
    assert [hex(v) for v in states.reshape(-1)[:8]] == [hex(int(v, 16)) for v in case["first"]]
    assert fnv_states(states) == int(case["digest"], 16)


def test_widths_table():
    assert [orc.orc_exl3_bits_x2(s) for s in (0, 1, 8, 9, 24, 40, 41, 56, 120, 128)] == [0, 2, 16, 0, 3, 5, 0, 7, 15, 0]


def test_codebook_closed_form():
    assert orc.orc_exl3_codebook(0) == int(KAT["codebook"]["state0_bits"], 16)
    states = np.arange(65536, dtype=np.uint64)
    product = (states * 0x83DCD12D) & 0xFFFFFFFF
    b = (product & 255) + ((product >> 8) & 255) + ((product >> 16) & 255) + (product >> 24)
    exact = (1774.0 * b.astype(np.float64) - 905216.0) / 2.0 ** 18
    expected = exact.astype(np.float16).view(np.uint16)  # numpy rounds once, to nearest even
    got = np.array([orc.orc_exl3_codebook(int(s)) for s in states], dtype=np.uint16)
    assert np.array_equal(got, expected)
    assert np.all((b >= 0) & (b <= 1020))


def test_zero_k3_tile_times_ones():
    tile = np.zeros(96, dtype=np.uint8)  # 256 * 3 bits
    weights = np.zeros((16, 16), dtype=np.uint16)
    orc.orc_exl3_decode_matrix(ptr(tile, u8p), 16, 16, 3, ptr(weights, u16p))
    assert weights.view(np.float16).astype(np.float64).sum() == KAT["codebook"]["zero_k3_tile_times_ones"]


def test_position_is_a_bijection():
    seen = set()
    for i in range(16):
        for o in range(16):
            p = orc.orc_exl3_position(i, o)
            a, b = C.c_uint32(), C.c_uint32()
            orc.orc_exl3_place(p, C.byref(a), C.byref(b))
            assert (a.value, b.value) == (i, o)
            seen.add(p)
    assert seen == set(range(256))
    # the definition: weight 8 t + m is input 2 (t % 4) + m % 2 + 8 (m / 2 % 2), output t / 4 + 8 (m / 4)
    for p in range(256):
        t, m = divmod(p, 8)
        assert orc.orc_exl3_position(2 * (t % 4) + m % 2 + 8 * (m // 2 % 2), t // 4 + 8 * (m // 4)) == p


@pytest.mark.parametrize("stored,bits_x2", WIDTHS)
def test_ring_against_bit_walk(stored, bits_x2):
    tile_bytes = 16 * bits_x2
    tiles = splitmix_words(77 + stored, 3 * tile_bytes // 8).view(np.uint8)
    for t in range(3):
        one = np.ascontiguousarray(tiles[t * tile_bytes:(t + 1) * tile_bytes])
        states = np.zeros(256, dtype=np.uint16)
        orc.orc_exl3_tile_states(bits_x2, ptr(one.view(np.uint32), u32p), ptr(states, u16p))
        expected = [python_state(bytes(one), bits_x2, p) for p in range(256)]
        assert states.tolist() == expected


def test_h128_definition_and_order():
    x = normals(5, 128)
    a = x.astype(np.float32).copy()
    orc.orc_h128_f32(ptr(a, f32p))
    d = np.zeros(128)
    orc.orc_h128_f64(ptr(x.astype(np.float32).astype(np.float64), f64p), ptr(d, f64p))
    assert np.max(np.abs(a - d)) < 4e-6
    # H . H = I
    back = np.zeros(128)
    orc.orc_h128_f64(ptr(d, f64p), ptr(back, f64p))
    assert np.max(np.abs(back - x.astype(np.float32))) < 1e-12
    # the definition against a Sylvester matrix built by Kronecker products
    h = np.array([[1.0]])
    for _ in range(7):
        h = np.kron(np.array([[1.0, 1.0], [1.0, -1.0]]), h)
    assert np.max(np.abs(d - (x.astype(np.float32).astype(np.float64) @ h) / np.sqrt(128.0))) < 1e-12
    # an impulse at index 5 gives row 5 of H: the butterfly's sign pattern, exactly
    e = np.zeros(128, dtype=np.float32)
    e[5] = 1.0
    orc.orc_h128_f32(ptr(e, f32p))
    assert np.array_equal(e, (h[5] * np.float32(0.08838834764831845)).astype(np.float32))


def test_expf_against_libm():
    xs = np.concatenate([np.linspace(-104, 89, 200001), normals(9, 50000) * 10]).astype(np.float32)
    got = np.array([orc.orc_expf(float(x)) for x in xs[::7]], dtype=np.float32)
    want64 = np.exp(xs[::7].astype(np.float64))
    finite = (want64 < 3.4e38) & (want64 > 1.2e-38)
    ulp = np.spacing(np.abs(want64[finite]).astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(got[finite].astype(np.float64) - want64[finite]) / ulp) <= 1.0
    assert orc.orc_expf(100.0) == np.inf and orc.orc_expf(-200.0) == 0.0 and orc.orc_expf(0.0) == 1.0


def test_product_modes_and_streaming_form():
    inputs, outputs = 256, 128
    for stored in (2, 3, 4, 40):
        matrix = exl3_matrix(100 + stored, inputs, outputs, stored)
        weights = np.zeros((inputs, outputs), dtype=np.uint16)
        orc.orc_exl3_decode_matrix(ptr(matrix, u8p), inputs, outputs, stored, ptr(weights, u16p))
        operand = normals(3, inputs).astype(np.float16)
        ideal = np.zeros(outputs, dtype=np.float32)
        orc.orc_exl3_product(ptr(weights, u16p), inputs, outputs, ptr(operand.view(np.uint16), u16p), 4, 0, ptr(ideal, f32p))
        want = operand.astype(np.float64) @ weights.view(np.float16).astype(np.float64)
        assert np.array_equal(ideal, want.astype(np.float32))
        ordered = np.zeros(outputs, dtype=np.float32)
        orc.orc_exl3_product(ptr(weights, u16p), inputs, outputs, ptr(operand.view(np.uint16), u16p), 4, 1, ptr(ordered, f32p))
        scale = np.abs(operand.astype(np.float64)) @ np.abs(weights.view(np.float16).astype(np.float64))
        assert np.max(np.abs(ordered - want) / scale) < 2e-6
        streamed = np.zeros(outputs, dtype=np.float32)
        orc.orc_exl3_product_codes(ptr(matrix, u8p), inputs, outputs, stored, ptr(operand.view(np.uint16), u16p), 1, ptr(streamed, f32p))
        assert np.array_equal(streamed, ideal)


def test_chain_against_the_double_precision_definition():
    """y = (((x.suh)Hb)T)Hb.svh: the float32 chain with fp16 operands stays within 1e-3 of the definition."""
    inputs, outputs, stored = 256, 384, 3
    matrix = exl3_matrix(42, inputs, outputs, stored)
    code_bytes = int(orc.orc_exl3_code_bytes(inputs, outputs, stored))
    suh = np.ascontiguousarray(matrix[code_bytes:code_bytes + 2 * inputs]).view(np.uint16)
    svh = np.ascontiguousarray(matrix[code_bytes + 2 * inputs:]).view(np.uint16)
    x = to_bf16(normals(8, inputs))
    x64 = (x.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    y = np.zeros(outputs)
    orc.orc_exl3_linear_f64(ptr(matrix, u8p), inputs, outputs, stored, ptr(x64, f64p), ptr(y, f64p))
    operand = np.zeros(inputs, dtype=np.uint16)
    orc.orc_exl3_operand(ptr(x, u16p), ptr(suh, u16p), inputs, ptr(operand, u16p))
    products = np.zeros(outputs, dtype=np.float32)
    orc.orc_exl3_product_codes(ptr(matrix, u8p), inputs, outputs, stored, ptr(operand, u16p), 1, ptr(products, f32p))
    out = np.zeros(outputs, dtype=np.float32)
    orc.orc_exl3_finish(ptr(products, f32p), ptr(svh, u16p), outputs, 1.0, ptr(out, f32p))
    assert np.max(np.abs(out - y)) / np.sqrt(np.mean(y * y)) < 2e-3


def test_activate_closed_form():
    inner = 128
    rng = normals(11, 3 * inner)
    gate, up = (rng[:inner] * 30).astype(np.float32), (rng[inner:2 * inner] * 30).astype(np.float32)
    ones = np.full(inner, 0x3C00, dtype=np.uint16)
    hidden = np.zeros(inner, dtype=np.uint16)
    operand = np.zeros(inner, dtype=np.uint16)
    orc.orc_exl3_activate(ptr(gate, f32p), ptr(up, f32p), ptr(ones, u16p), ptr(ones, u16p), ptr(ones, u16p), inner, 10.0,
                          ptr(hidden, u16p), ptr(operand, u16p))
    h = np.array([[1.0]])
    for _ in range(7):
        h = np.kron(np.array([[1.0, 1.0], [1.0, -1.0]]), h)
    g = np.minimum((gate.astype(np.float64) @ h) / np.sqrt(128), 10.0)
    u = np.clip((up.astype(np.float64) @ h) / np.sqrt(128), -10.0, 10.0)
    want = g / (1 + np.exp(-g)) * u
    got = (hidden.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-2)) < 6e-3  # one bf16 rounding + float32 noise
    back = operand.view(np.float16).astype(np.float64)
    exact = (want @ h) / np.sqrt(128)
    assert np.max(np.abs(back - exact) / np.maximum(np.abs(exact), 1.0)) < 1.5e-3  # fp16 operand rounding


def test_layer_is_the_composition_of_its_stages():
    rows, hidden, inner, picks, experts_n = 3, 256, 128, 2, 5
    widths = np.array([[2, 3, 4], [3, 3, 3], [4, 2, 40], [2, 2, 2], [3, 4, 3]], dtype=np.uint8)
    mats = []
    for e in range(experts_n):
        mats.append([exl3_matrix(1000 + 3 * e, hidden, inner, int(widths[e, 0])),
                     exl3_matrix(1001 + 3 * e, hidden, inner, int(widths[e, 1])),
                     exl3_matrix(1002 + 3 * e, inner, hidden, int(widths[e, 2]))])
    x = to_bf16(normals(21, rows * hidden)).reshape(rows, hidden)
    experts = np.array([[0, 3], [1, 3], [3, 4]], dtype=np.uint32)
    weights = np.array([[0.5, 1.0], [0.25, 0.75], [1.5, 0.125]], dtype=np.float32)
    pointers = (C.c_void_p * (experts_n * 3))(*[m.ctypes.data for trio in mats for m in trio])
    out = np.zeros((rows, hidden), dtype=np.float32)
    pair_out = np.zeros((rows * picks, hidden), dtype=np.float32)
    hidden_out = np.zeros((rows * picks, inner), dtype=np.uint16)
    orc.orc_exl3_moe_layer(ptr(x, u16p), rows, hidden, inner, picks, ptr(experts, u32p), ptr(weights, f32p), experts_n,
                           pointers, ptr(widths, u8p), 10.0, ptr(out, f32p), ptr(hidden_out, u16p), ptr(pair_out, f32p), 3)
    # by hand for pair (row 1, slot 1) -> expert 3
    row, slot, e = 1, 1, 3
    gate, up, down = mats[e]
    cb = int(orc.orc_exl3_code_bytes(hidden, inner, int(widths[e, 0])))
    g_suh, g_svh = np.ascontiguousarray(gate[cb:cb + 2 * hidden]).view(np.uint16), np.ascontiguousarray(gate[cb + 2 * hidden:]).view(np.uint16)
    cb = int(orc.orc_exl3_code_bytes(hidden, inner, int(widths[e, 1])))
    u_suh, u_svh = np.ascontiguousarray(up[cb:cb + 2 * hidden]).view(np.uint16), np.ascontiguousarray(up[cb + 2 * hidden:]).view(np.uint16)
    cb = int(orc.orc_exl3_code_bytes(inner, hidden, int(widths[e, 2])))
    d_suh, d_svh = np.ascontiguousarray(down[cb:cb + 2 * inner]).view(np.uint16), np.ascontiguousarray(down[cb + 2 * inner:]).view(np.uint16)
    operand = np.zeros(hidden, dtype=np.uint16)
    gp, up_p = np.zeros(inner, dtype=np.float32), np.zeros(inner, dtype=np.float32)
    orc.orc_exl3_operand(ptr(x[row], u16p), ptr(g_suh, u16p), hidden, ptr(operand, u16p))
    orc.orc_exl3_product_codes(ptr(gate, u8p), hidden, inner, int(widths[e, 0]), ptr(operand, u16p), 1, ptr(gp, f32p))
    orc.orc_exl3_operand(ptr(x[row], u16p), ptr(u_suh, u16p), hidden, ptr(operand, u16p))
    orc.orc_exl3_product_codes(ptr(up, u8p), hidden, inner, int(widths[e, 1]), ptr(operand, u16p), 1, ptr(up_p, f32p))
    hid, op2 = np.zeros(inner, dtype=np.uint16), np.zeros(inner, dtype=np.uint16)
    orc.orc_exl3_activate(ptr(gp, f32p), ptr(up_p, f32p), ptr(g_svh, u16p), ptr(u_svh, u16p), ptr(d_suh, u16p), inner, 10.0,
                          ptr(hid, u16p), ptr(op2, u16p))
    dp = np.zeros(hidden, dtype=np.float32)
    orc.orc_exl3_product_codes(ptr(down, u8p), inner, hidden, int(widths[e, 2]), ptr(op2, u16p), 1, ptr(dp, f32p))
    pair = np.zeros(hidden, dtype=np.float32)
    orc.orc_exl3_finish(ptr(dp, f32p), ptr(d_svh, u16p), hidden, float(weights[row, slot]), ptr(pair, f32p))
    assert np.array_equal(hidden_out[row * picks + slot], hid)
    assert np.array_equal(pair_out[row * picks + slot], pair)
    assert np.array_equal(out, (pair_out.reshape(rows, picks, hidden)[:, 0] + pair_out.reshape(rows, picks, hidden)[:, 1]))


# ---- against the reference's own C oracles, built in place ----

needs_ref = pytest.mark.skipif(ref is None, reason="oracle/_ref/libref.so was not built (no reference tree)")


@needs_ref
def test_ref_codebook_and_position():
    for state in list(range(0, 65536, 13)) + [65535]:
        assert orc.orc_exl3_codebook(state) == ref.test_exl3_codebook(state)
    for i in range(16):
        for o in range(16):
            assert orc.orc_exl3_position(i, o) == ref.test_exl3_position(i, o)


@needs_ref
@pytest.mark.parametrize("stored,bits_x2", WIDTHS)
def test_ref_states_and_decode(stored, bits_x2):
    inputs, outputs = 48, 32
    matrix = exl3_matrix(500 + stored, inputs, outputs, stored)
    states = np.zeros((inputs, outputs), dtype=np.uint16)
    orc.orc_exl3_states(ptr(matrix, u8p), inputs, outputs, stored, ptr(states, u16p))
    for i in range(inputs):
        for o in range(outputs):
            assert states[i, o] == ref.test_exl3_state(ptr(matrix, u8p), inputs, outputs, stored, i, o)
    ours = np.zeros((inputs, outputs), dtype=np.uint16)
    theirs = np.zeros((inputs, outputs), dtype=np.uint16)
    orc.orc_exl3_decode_matrix(ptr(matrix, u8p), inputs, outputs, stored, ptr(ours, u16p))
    ref.test_exl3_decode_matrix(ptr(matrix, u8p), inputs, outputs, stored, ptr(theirs, u16p))
    assert np.array_equal(ours, theirs)


@needs_ref
def test_ref_chain_product_within_its_class_tolerance():
    """The reference models NVIDIA's in-instruction truncation (class 80 / 120); the ideal sum lies within the
    bound the reference itself uses between classes: rel 1e-2 of the largest, rms 1e-3
    (tests/exl3_sm120_card_test.c:68-69)."""
    inputs, outputs, columns = 256, 64, 3
    matrix = exl3_matrix(900, inputs, outputs, 3)
    weights = np.zeros((inputs, outputs), dtype=np.uint16)
    orc.orc_exl3_decode_matrix(ptr(matrix, u8p), inputs, outputs, 3, ptr(weights, u16p))
    operands = normals(4, columns * inputs).astype(np.float16).reshape(columns, inputs)
    theirs = np.zeros((columns, outputs), dtype=np.float32)
    ref.test_exl3_chain(80, ptr(weights, u16p), inputs, outputs, 4, ptr(operands.view(np.uint16), u16p), columns, ptr(theirs, f32p))
    ours = np.zeros((columns, outputs), dtype=np.float32)
    orc.orc_exl3_product_codes(ptr(matrix, u8p), inputs, outputs, 3, ptr(operands.view(np.uint16), u16p), columns, ptr(ours, f32p))
    scale = np.sqrt(np.mean(ours.astype(np.float64) ** 2))
    assert np.max(np.abs(ours - theirs)) / scale < 1e-4
