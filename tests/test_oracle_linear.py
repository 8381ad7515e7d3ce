"""Pins the FP4 / FP8 part of the CPU oracle: value tables, lay-out / read-back round trips, hand-placed weights,
exhaustive nearest-code search, numpy float64 matmul on dequantised tensors, and the reference's own C oracles
(oracle/_ref) where built."""
import numpy as np
import pytest

from _oracle import (C, Shape, f32p, f64p, normals, orc, ptr, ref, splitmix_words, to_bf16, bf16_to_f32, u8p, u16p,
                     u32p)

E2M1, E4M3 = 3, 5
needs_ref = pytest.mark.skipif(ref is None, reason="oracle/_ref/libref.so was not built (no reference tree)")

E2M1_VALUES = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6])


def e4m3_values():
    codes = np.arange(256)
    e, m = (codes >> 3) & 15, codes & 7
    mag = np.where(e == 0, m / 8 * 2.0 ** -6, (1 + m / 8) * 2.0 ** (e.astype(float) - 7))
    return np.where(codes & 0x80, -mag, mag)


def random_matrix(fmt, outputs, inputs, seed):
    raw = splitmix_words(seed, outputs * inputs).astype(np.uint64)
    if fmt == E2M1:
        codes = (raw & np.uint64(15)).astype(np.uint8)
    else:
        codes = (raw & np.uint64(255)).astype(np.uint8)
        codes[(codes & 0x7F) == 0x7F] = 0x3A  # a pack holds no code that is no number
    n_scales = int(orc.orc_linear_scale_count(fmt, outputs, inputs))
    scales = (120 + (splitmix_words(seed + 1, n_scales) % np.uint64(12))).astype(np.uint8)
    stored = np.zeros(int(orc.orc_linear_stored_bytes(fmt, outputs, inputs)), dtype=np.uint8)
    assert orc.orc_linear_lay_out(fmt, outputs, inputs, ptr(codes, u8p), ptr(scales, u8p), ptr(stored, u8p)) == 0
    return codes.reshape(outputs, inputs), scales, stored


def dequantised(fmt, codes, scales, outputs, inputs):
    values = E2M1_VALUES[codes] if fmt == E2M1 else e4m3_values()[codes]
    if fmt == E2M1:
        s = 2.0 ** (scales.reshape(outputs, inputs // 32).astype(float) - 127)
        return values * np.repeat(s, 32, axis=1)
    s = 2.0 ** (scales.reshape((outputs + 31) // 32, inputs // 32).astype(float) - 127)
    return values * np.repeat(np.repeat(s, 32, axis=0)[:outputs], 32, axis=1)


def test_byte_counts():
    # expert of the benchmark shape: 3 x (4096 x 2048 / 2 + 4096 x 2048 / 32) = 13,369,344
    assert 3 * orc.orc_linear_stored_bytes(E2M1, 2048, 4096) == 13369344
    assert orc.orc_linear_stored_bytes(E4M3, 48, 64) == 48 * 64 + 2 * 2
    assert orc.orc_linear_lay_out(E2M1, 16, 32, None, None, None) == -1  # inputs not a multiple of 64


@pytest.mark.parametrize("fmt,outputs,inputs", [(E2M1, 32, 128), (E2M1, 16, 64), (E4M3, 48, 96), (E4M3, 16, 32)])
def test_lay_out_and_read_back(fmt, outputs, inputs):
    codes, scales, stored = random_matrix(fmt, outputs, inputs, 7)
    code, scale = C.c_uint32(), C.c_uint32()
    for o in range(outputs):
        for i in range(inputs):
            assert orc.orc_linear_read(fmt, outputs, inputs, ptr(stored, u8p), o, i, C.byref(code), C.byref(scale)) == 0
            assert code.value == codes[o, i]
            want = scales.reshape(outputs, -1)[o, i // 32] if fmt == E2M1 else scales.reshape(-1, inputs // 32)[o // 32, i // 32]
            assert scale.value == want


def test_hand_placed_weights():
    # E2M1: W[9][37] of a 16 x 64 matrix: tile 0, load 0, g = 1, r%2 = 1; step 2, j = 5: t = 2, h = 1, r/2 = 0
    codes = np.zeros((16, 64), dtype=np.uint8)
    codes[9, 37] = 0xB
    scales = np.full(16 * 2, 127, dtype=np.uint8)
    scales[9 * 2 + 1] = 130
    stored = np.zeros(16 * 64 // 2 + 32, dtype=np.uint8)
    orc.orc_linear_lay_out(E2M1, 16, 64, ptr(codes, u8p), ptr(scales, u8p), ptr(stored, u8p))
    words = stored[:512].view(np.uint32)
    lane, step, r, h = 4 * 1 + 2, 2, 1, 1
    assert words[lane * 4 + step] == 0xB << (4 * r + 16 * h) and np.count_nonzero(words) == 1
    assert stored[512 + 4 * 1 + 2 * 1 + 1] == 130  # scales word g = 1, byte 2 q + r: q = 1, r = 1
    # E4M3: W[12][21] of a 16 x 32 matrix: g = 4, b%2 = 1; 21 = 8*2 + 2*2 + 1: b/4 = 2, t = 2, (b/2)%2 = 1 -> b = 11
    codes = np.zeros((16, 32), dtype=np.uint8)
    codes[12, 21] = 0x55
    stored = np.zeros(16 * 32 + 1, dtype=np.uint8)
    orc.orc_linear_lay_out(E4M3, 16, 32, ptr(codes, u8p), ptr(np.array([127], dtype=np.uint8), u8p), ptr(stored, u8p))
    assert stored[(4 * 4 + 2) * 16 + 11] == 0x55 and np.count_nonzero(stored[:512]) == 1


def test_quantizer_exhaustive_search_and_scale_rule():
    values = to_bf16(normals(3, 256) * np.repeat([1e-6, 0.3, 7.0, 448.0, 1.0, 2.0 ** -3, 100.0, 3e4], 32))
    values[32] = to_bf16(np.array([2.0 ** -3 * 448]))[0]  # block maximum exactly 448 x a power of two
    codes = np.zeros(256, dtype=np.uint8)
    exps = np.zeros(8, dtype=np.uint8)
    assert orc.orc_act_quantize(ptr(values, u16p), 256, ptr(codes, u8p), ptr(exps, u8p)) == 0
    v = bf16_to_f32(values).astype(np.float64).reshape(8, 32)
    table = e4m3_values()[:127]
    for b in range(8):
        m = np.float32(max(np.abs(v[b]).max(), np.float32(1e-4))) * np.float32(1.0 / 448.0)
        k = int(np.ceil(np.log2(np.float64(m))))
        assert 2.0 ** k >= m > 2.0 ** (k - 1) and exps[b] == k + 127
        for i in range(32):
            scaled = min(abs(v[b, i]) / 2.0 ** k, 448.0)
            distance = np.abs(table - scaled)
            best = np.flatnonzero(distance == distance.min())
            want = best[0] if len(best) == 1 else [c for c in best if c % 2 == 0][0]
            assert codes[b * 32 + i] == (want | (0x80 if values[b * 32 + i] & 0x8000 else 0))
    assert exps[0] == 105  # the floor 1e-4 gives 2^-22


def test_vector_orders():
    codes = np.arange(128, dtype=np.uint8)
    stored = np.zeros(128, dtype=np.uint8)
    orc.orc_codes_lane_order(ptr(codes, u8p), 128, ptr(stored, u8p))
    for l in range(2):
        for t in range(4):
            for s in range(4):
                for j in range(4):
                    assert stored[((4 * l + t) * 4 + s) * 4 + j] == 64 * l + 16 * s + 2 * t + j // 2 + 8 * (j % 2)
    assert sorted(stored.tolist()) == list(range(128))
    exps = np.array([127, 120, 147, 100], dtype=np.uint8)
    codes = np.full(128, 0x38, dtype=np.uint8)  # 1.0
    codes[1] = 0xB8
    operands = np.zeros(128, dtype=np.uint16)
    orc.orc_operands_lay_out(ptr(codes, u8p), ptr(exps, u8p), 128, ptr(operands, u16p))
    f = bf16_to_f32(operands)
    assert f[0] == 2.0 ** 100 and f[1] == -2.0 ** 100  # values 0 and 1 are halves 0 and 1
    place = {64 * l + 16 * s + 2 * t + h + 8 * r: ((4 * l + t) * 4 + s) * 4 + 2 * r + h
             for l in range(2) for t in range(4) for s in range(4) for r in range(2) for h in range(2)}
    assert f[place[40]] == 2.0 ** 93 and np.isinf(f[place[70]]) and f[place[100]] == 2.0 ** 73


@pytest.mark.parametrize("fmt", [E2M1, E4M3])
def test_products_against_numpy(fmt):
    outputs, inputs, vectors = 32, 256, 3
    codes, scales, stored = random_matrix(fmt, outputs, inputs, 11)
    w = dequantised(fmt, codes, scales, outputs, inputs)
    x = to_bf16(normals(5, vectors * inputs)).reshape(vectors, inputs)
    xc = np.zeros((vectors, inputs), dtype=np.uint8)
    xe = np.zeros((vectors, inputs // 32), dtype=np.uint8)
    for v in range(vectors):
        orc.orc_act_quantize(ptr(x[v], u16p), inputs, ptr(xc[v], u8p), ptr(xe[v], u8p))
    xq = e4m3_values()[xc] * np.repeat(2.0 ** (xe.astype(float) - 127), 32, axis=1)
    assert np.max(np.abs(xq - bf16_to_f32(x)) / np.abs(bf16_to_f32(x)).max()) < 0.07
    sums, mags = np.zeros((vectors, outputs)), np.zeros((vectors, outputs))
    assert orc.orc_linear_products(fmt, outputs, inputs, ptr(stored, u8p), 0, outputs, ptr(xc, u8p), ptr(xe, u8p), vectors,
                                   ptr(sums, f64p), ptr(mags, f64p)) == 0
    assert np.allclose(sums, xq @ w.T, rtol=1e-12, atol=1e-300)
    assert np.allclose(mags, np.abs(xq) @ np.abs(w).T, rtol=1e-12)
    out = to_bf16(sums.astype(np.float32))
    assert all(orc.orc_linear_within_tolerance(int(out[v, o]), sums[v, o], mags[v, o], inputs, 4) for v in range(vectors) for o in range(outputs))
    assert not orc.orc_linear_within_tolerance(int(out[0, 0]) ^ 0x0010, sums[0, 0], mags[0, 0] * 1e-3, inputs, 4)


def test_hidden_step_and_row_sum():
    for gate, up, w in [(1.5, -2.0, 0.75), (20.0, 30.0, 1.0), (-90.0, 1.0, 1.0), (-3.0, -50.0, 0.5), (0.0, 4.0, 1.0)]:
        g, u = min(gate, 10.0), min(max(up, -10.0), 10.0)
        want = (0.0 if -g > 88.7 else g / (1 + np.exp(-g))) * u * w
        assert abs(orc.orc_hidden_value(gate, up, 10.0, w) - want) <= 1e-12 * abs(want)
        got = bf16_to_f32(np.array([orc.orc_hidden_bits(gate, up, 10.0, w)], dtype=np.uint16))[0]
        assert abs(got - want) <= abs(want) * 2.0 ** -8 + 1e-30
    pairs = to_bf16(np.array([[2.0 ** 30], [1.0], [-2.0 ** 30], [1.0], [0.0], [0.0]]))
    assert orc.orc_row_sum_bf16(ptr(pairs, u16p), 6, 1, 0) == 1.0  # ((2^30 + 1) - 2^30) + 1 in float32, in slot order


def test_block128_mode_against_numpy():
    outputs, inputs, vectors = 256, 256, 2
    w_real = normals(9, outputs * inputs).reshape(outputs, inputs) * 0.02
    w_scales = np.zeros((2, 2), dtype=np.float32)
    w_codes = np.zeros((outputs, inputs), dtype=np.uint8)
    table = e4m3_values()
    for bo in range(2):
        for bi in range(2):
            block = w_real[bo * 128:(bo + 1) * 128, bi * 128:(bi + 1) * 128]
            w_scales[bo, bi] = np.float32(np.abs(block).max() / 448.0)
            scaled = block / w_scales[bo, bi]
            idx = np.abs(table[None, None, :127] - np.abs(scaled)[:, :, None]).argmin(axis=2)
            w_codes[bo * 128:(bo + 1) * 128, bi * 128:(bi + 1) * 128] = idx | np.where(scaled < 0, 0x80, 0)
    x = to_bf16(normals(10, vectors * inputs)).reshape(vectors, inputs)
    a_codes = np.zeros((vectors, inputs), dtype=np.uint8)
    a_scales = np.zeros((vectors, inputs // 128), dtype=np.float32)
    for v in range(vectors):
        orc.orc_act_quantize_128(ptr(x[v], u16p), inputs, ptr(a_codes[v], u8p), ptr(a_scales[v], f32p))
    xf = bf16_to_f32(x).reshape(vectors, 2, 128)
    assert np.array_equal(a_scales, (np.maximum(np.abs(xf).max(axis=2), np.float32(1e-4)) / np.float32(448.0)).astype(np.float32))
    xq = table[a_codes] * np.repeat(a_scales.astype(np.float64), 128, axis=1)
    assert np.max(np.abs(xq - bf16_to_f32(x))) < 0.07 * np.abs(bf16_to_f32(x)).max()
    wq = table[w_codes] * np.repeat(np.repeat(w_scales.astype(np.float64), 128, axis=0), 128, axis=1)
    sums = np.zeros((vectors, outputs))
    orc.orc_fp8_block128_products(outputs, inputs, ptr(w_codes, u8p), ptr(w_scales, f32p), ptr(a_codes, u8p), ptr(a_scales, f32p),
                                  vectors, ptr(sums, f64p))
    assert np.allclose(sums, xq @ wq.T, rtol=1e-11)


def test_block128_stored_format_against_the_plain_arrays():
    """Format 6 (codes in E4M3_SCALED's lane order, float32 scales behind them): laid out and read back, and its
    products equal the products of the plain row-major arrays, which numpy pins above."""
    B128 = 6
    outputs, inputs, vectors = 256, 384, 3
    rng = np.random.default_rng(3)
    w_codes = rng.integers(0, 256, size=(outputs, inputs)).astype(np.uint8)
    w_codes[(w_codes & 0x7F) == 0x7F] = 0x7E
    w_scales = (rng.random((outputs // 128, inputs // 128)) * 1e-3 + 1e-5).astype(np.float32)
    assert orc.orc_linear_stored_bytes(B128, outputs, inputs) == outputs * inputs + w_scales.nbytes
    stored = np.zeros(outputs * inputs + w_scales.nbytes, dtype=np.uint8)
    assert orc.orc_linear_lay_out(B128, outputs, inputs, ptr(w_codes, u8p), ptr(w_scales.view(np.uint8).reshape(-1), u8p), ptr(stored, u8p)) == 0
    assert orc.orc_linear_lay_out(B128, 192, 384, ptr(w_codes, u8p), ptr(w_scales.view(np.uint8).reshape(-1), u8p), ptr(stored, u8p)) == -1
    same = np.zeros(outputs * inputs + outputs // 32 * (inputs // 32), dtype=np.uint8)  # the codes lie as E4M3_SCALED lays them
    assert orc.orc_linear_lay_out(E4M3, outputs, inputs, ptr(w_codes, u8p), ptr(np.zeros(outputs // 32 * inputs // 32, dtype=np.uint8), u8p), ptr(same, u8p)) == 0
    assert np.array_equal(stored[:outputs * inputs], same[:outputs * inputs])
    code, scale = C.c_uint32(0), C.c_uint32(0)
    for o, i in ((0, 0), (130, 5), (255, 383), (127, 128), (128, 127)):
        assert orc.orc_linear_read(B128, outputs, inputs, ptr(stored, u8p), o, i, C.byref(code), C.byref(scale)) == 0
        assert code.value == w_codes[o, i] and scale.value == w_scales[o // 128, i // 128].view(np.uint32)
    x = to_bf16(normals(12, vectors * inputs) * 3.0).reshape(vectors, inputs)
    a_codes, a_scales = np.zeros((vectors, inputs), dtype=np.uint8), np.zeros((vectors, inputs // 128), dtype=np.float32)
    for v in range(vectors):
        orc.orc_act_quantize_128(ptr(x[v], u16p), inputs, ptr(a_codes[v], u8p), ptr(a_scales[v], f32p))
    want, got, mags = np.zeros((vectors, outputs)), np.zeros((vectors, outputs)), np.zeros((vectors, outputs))
    orc.orc_fp8_block128_products(outputs, inputs, ptr(w_codes, u8p), ptr(w_scales, f32p), ptr(a_codes, u8p), ptr(a_scales, f32p), vectors, ptr(want, f64p))
    assert orc.orc_linear_products_128(outputs, inputs, ptr(stored, u8p), 0, outputs, ptr(a_codes, u8p), ptr(a_scales, f32p), vectors,
                                       ptr(got, f64p), ptr(mags, f64p)) == 0
    assert np.array_equal(got, want) and np.all(mags >= np.abs(got))


def test_layer_runs_and_matches_dequantised_matmul():
    rows, hidden, inner, picks, experts_n = 2, 128, 64, 2, 3
    mats, dense = [], []
    for e in range(experts_n):
        trio, dtrio = [], []
        for m, (o, i) in enumerate([(inner, hidden), (inner, hidden), (hidden, inner)]):
            codes, scales, stored = random_matrix(E2M1, o, i, 300 + 3 * e + m)
            trio.append(stored)
            dtrio.append(dequantised(E2M1, codes, (scales - 6).astype(np.uint8), o, i))
            # rewrite with the smaller scales so hidden values stay moderate
            stored2 = np.zeros_like(stored)
            orc.orc_linear_lay_out(E2M1, o, i, ptr(np.ascontiguousarray(codes), u8p), ptr((scales - 6).astype(np.uint8), u8p), ptr(stored2, u8p))
            trio[-1] = stored2
        mats.append(trio)
        dense.append(dtrio)
    x = to_bf16(normals(77, rows * hidden)).reshape(rows, hidden)
    experts = np.array([[0, 2], [1, 2]], dtype=np.uint32)
    weights = np.array([[0.5, 1.0], [0.25, 0.75]], dtype=np.float32)
    pointers = (C.c_void_p * (experts_n * 3))(*[m.ctypes.data for trio in mats for m in trio])
    out = np.zeros((rows, hidden), dtype=np.float32)
    orc.orc_linear_moe_layer(E2M1, ptr(x, u16p), rows, hidden, inner, picks, ptr(experts, u32p), ptr(weights, f32p), experts_n,
                             pointers, 10.0, ptr(out, f32p), None, None, 2)
    xf = bf16_to_f32(x).astype(np.float64)
    want = np.zeros((rows, hidden))
    for r in range(rows):
        for s in range(picks):
            g, u, d = dense[experts[r, s]]
            gg, uu = np.minimum(g @ xf[r], 10), np.clip(u @ xf[r], -10, 10)
            want[r] += d @ (gg / (1 + np.exp(-gg)) * uu * weights[r, s])
    # two E4M3 quantisations (3 fraction bits) on the way: a few percent of the root mean square
    assert np.sqrt(np.mean((out - want) ** 2) / np.mean(want ** 2)) < 0.06


@needs_ref
@pytest.mark.parametrize("fmt,outputs,inputs", [(E2M1, 32, 128), (E4M3, 48, 96)])
def test_ref_lay_out_read_and_products(fmt, outputs, inputs):
    codes, scales, stored = random_matrix(fmt, outputs, inputs, 21)
    shape = Shape(outputs, inputs, 4 if fmt == E2M1 else 8, 0)
    theirs = np.zeros_like(stored)
    flat = np.ascontiguousarray(codes.reshape(-1))
    assert ref.test_weight_format_lay_out(fmt, C.byref(shape), ptr(flat, u8p), flat.size, ptr(scales, u8p), scales.size,
                                          ptr(theirs, u8p), theirs.size) == 0
    assert np.array_equal(stored, theirs)
    vectors = 2
    x = to_bf16(normals(6, vectors * inputs)).reshape(vectors, inputs)
    xc, xe = np.zeros((vectors, inputs), dtype=np.uint8), np.zeros((vectors, inputs // 32), dtype=np.uint8)
    tc, te = np.zeros_like(xc), np.zeros_like(xe)
    for v in range(vectors):
        orc.orc_act_quantize(ptr(x[v], u16p), inputs, ptr(xc[v], u8p), ptr(xe[v], u8p))
        assert ref.test_linear_quantize(ptr(x[v], u16p), inputs, ptr(tc[v], u8p), ptr(te[v], u8p)) == 0
    assert np.array_equal(xc, tc) and np.array_equal(xe, te)
    fed = np.zeros((vectors, inputs))
    for v in range(vectors):
        ref.test_linear_fed_values_of_codes(ptr(xc[v], u8p), inputs, ptr(fed[v], f64p))
    theirs_p = np.zeros((vectors, outputs, 2))
    assert ref.test_linear_products(fmt, C.byref(shape), ptr(stored, u8p), stored.size, 0, outputs, ptr(fed, f64p), ptr(xe, u8p),
                                    vectors, 1, theirs_p.ctypes.data) == 0
    sums, mags = np.zeros((vectors, outputs)), np.zeros((vectors, outputs))
    orc.orc_linear_products(fmt, outputs, inputs, ptr(stored, u8p), 0, outputs, ptr(xc, u8p), ptr(xe, u8p), vectors, ptr(sums, f64p), ptr(mags, f64p))
    assert np.array_equal(sums, theirs_p[:, :, 0]) and np.array_equal(mags, theirs_p[:, :, 1])


@needs_ref
def test_ref_vector_orders_hidden_and_row_sum():
    width = 256
    x = to_bf16(normals(8, width) * 3)
    codes, exps = np.zeros(width, dtype=np.uint8), np.zeros(width // 32, dtype=np.uint8)
    orc.orc_act_quantize(ptr(x, u16p), width, ptr(codes, u8p), ptr(exps, u8p))
    a, b = np.zeros(width, dtype=np.uint8), np.zeros(width, dtype=np.uint8)
    orc.orc_codes_lane_order(ptr(codes, u8p), width, ptr(a, u8p))
    ref.test_linear_codes_lay_out(ptr(codes, u8p), width, ptr(b, u8p))
    assert np.array_equal(a, b)
    exps[3] = 150
    oa, ob = np.zeros(width, dtype=np.uint16), np.zeros(width, dtype=np.uint16)
    orc.orc_operands_lay_out(ptr(codes, u8p), ptr(exps, u8p), width, ptr(oa, u16p))
    ref.test_linear_operands_lay_out(ptr(codes, u8p), ptr(exps, u8p), width, ptr(ob, u16p))
    assert np.array_equal(oa, ob)
    for gate, up, w in [(1.5, -2.0, 0.75), (20.0, 30.0, 1.0), (-95.0, 1.0, 1.0), (-3.0, -50.0, 0.5)]:
        assert abs(orc.orc_hidden_value(gate, up, 10.0, w) - ref.test_linear_hidden_value(gate, up, 10.0, w)) <= 1e-12 * abs(gate * up)
    pairs = to_bf16(normals(4, 6 * 8)).reshape(6, 8)
    for column in range(8):
        assert orc.orc_row_sum_bf16(ptr(pairs, u16p), 6, 8, column) == ref.test_linear_row_sum(ptr(pairs, u16p), 6, 8, column)
