"""The weight formats in gfx950's own lane order (WEIGHT_FORMAT_E2M1_GFX950 = 7, WEIGHT_FORMAT_E4M3_GFX950 = 8) on the CPU:
the library's load-time re-lay-out (weight_format_gfx950_pack / _unpack, anemone_amd/host/weight_format.c) is a bijection of
the stored bytes (of WEIGHT_FORMAT_E4M3_BLOCK128_GFX950 = 9 too: E4M3_BLOCK128's bytes, float32 scales per 128 x 128); what
it makes is byte for byte what the oracle lays out from the plain matrix by the format's definition (oracle/orc_linear.c,
written from the definition, not from the re-lay-out); the oracle reads every weight and scale code of the re-laid-out bytes back to the plain matrix's; its products of the two lay-outs are the same numbers. No GPU."""
import ctypes as C

import numpy as np
import pytest

import anemone_amd as amd
from _oracle import orc, u8p

FORMATS = [(amd.WEIGHT_FORMAT_E2M1_GFX950, amd.WEIGHT_FORMAT_E2M1_SCALED, 4), (amd.WEIGHT_FORMAT_E4M3_GFX950, amd.WEIGHT_FORMAT_E4M3_SCALED, 8)]


def plain_matrix(seed, outputs, inputs, bits):
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 1 << bits, size=(outputs, inputs), dtype=np.uint8)
    if bits == 8:
        codes[(codes & 0x7F) == 0x7F] = 0x10  # no not-a-number codes
    count = outputs * (inputs // 32) if bits == 4 else (outputs // 32) * (inputs // 32)
    return codes, rng.integers(110, 135, size=count, dtype=np.uint8)


def laid_out(fmt, codes, scales):
    outputs, inputs = codes.shape
    stored = np.zeros(int(orc.orc_linear_stored_bytes(fmt, outputs, inputs)), dtype=np.uint8)
    assert orc.orc_linear_lay_out(fmt, outputs, inputs, codes.ctypes.data_as(u8p), scales.ctypes.data_as(u8p), stored.ctypes.data_as(u8p)) == 0
    return stored


@pytest.mark.parametrize("native,reference,bits", FORMATS)
@pytest.mark.parametrize("outputs,inputs", [(64, 128), (64, 256), (192, 640), (256, 512)])
def test_the_re_lay_out_is_the_definition_and_a_bijection(native, reference, bits, outputs, inputs):
    codes, scales = plain_matrix(outputs + inputs + bits, outputs, inputs, bits)
    stored = laid_out(reference, codes, scales)
    packed = amd.gfx950_pack(native, outputs, inputs, stored)
    assert packed.nbytes == stored.nbytes == int(orc.orc_linear_stored_bytes(native, outputs, inputs))
    assert np.array_equal(packed, laid_out(native, codes, scales)), "the library's re-lay-out is the oracle's lay-out of the definition"
    assert np.array_equal(amd.gfx950_unpack(native, outputs, inputs, packed), stored)
    # any bytes at all come back: the two maps are inverse permutations of the stored bits, both ways round
    noise = np.random.default_rng(5).integers(0, 256, size=stored.nbytes, dtype=np.uint8)
    assert np.array_equal(amd.gfx950_unpack(native, outputs, inputs, amd.gfx950_pack(native, outputs, inputs, noise)), noise)
    assert np.array_equal(amd.gfx950_pack(native, outputs, inputs, amd.gfx950_unpack(native, outputs, inputs, noise)), noise)
    if bits == 4:  # nibbles move between bytes: every nibble value is as frequent as before
        count = lambda b: np.bincount(np.concatenate([b[:outputs * inputs // 2] & 15, b[:outputs * inputs // 2] >> 4]), minlength=16)
        assert np.array_equal(count(packed), count(stored))
    else:
        assert np.array_equal(np.sort(packed), np.sort(stored))


@pytest.mark.parametrize("native,reference,bits", FORMATS)
def test_the_oracle_reads_the_same_matrix_back(native, reference, bits):
    outputs, inputs = 64, 384
    codes, scales = plain_matrix(77 + bits, outputs, inputs, bits)
    packed = amd.gfx950_pack(native, outputs, inputs, laid_out(reference, codes, scales))
    code, scale = C.c_uint32(), C.c_uint32()
    for output in range(outputs):
        for i in range(inputs):
            assert orc.orc_linear_read(native, outputs, inputs, packed.ctypes.data_as(u8p), output, i, C.byref(code), C.byref(scale)) == 0
            want_scale = scales[output * (inputs // 32) + i // 32] if bits == 4 else scales[(output // 32) * (inputs // 32) + i // 32]
            assert (code.value, scale.value) == (int(codes[output, i]), int(want_scale)), (output, i)


@pytest.mark.parametrize("native,reference,bits", FORMATS)
def test_products_of_the_two_lay_outs_are_the_same_numbers(native, reference, bits):
    outputs, inputs, vectors = 64, 256, 3
    codes, scales = plain_matrix(9 + bits, outputs, inputs, bits)
    stored = laid_out(reference, codes, scales)
    packed = amd.gfx950_pack(native, outputs, inputs, stored)
    rng = np.random.default_rng(2)
    fed = rng.integers(0, 0x7E, size=(vectors, inputs), dtype=np.uint8) | (rng.integers(0, 2, size=(vectors, inputs), dtype=np.uint8) << 7)
    exponents = rng.integers(120, 130, size=(vectors, inputs // 32), dtype=np.uint8)
    sums = [np.zeros((vectors, outputs)), np.zeros((vectors, outputs))]
    for fmt, bytes_, out in ((reference, stored, sums[0]), (native, packed, sums[1])):
        assert orc.orc_linear_products(fmt, outputs, inputs, bytes_.ctypes.data_as(u8p), 0, outputs, fed.ctypes.data_as(u8p),
                                       exponents.ctypes.data_as(u8p), vectors, out.ctypes.data_as(C.POINTER(C.c_double)), None) == 0
    assert np.array_equal(sums[0], sums[1]) and np.abs(sums[0]).max() > 0


def block128_matrix(seed, outputs, inputs):
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 256, size=(outputs, inputs), dtype=np.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x10
    scales = rng.uniform(0.002, 0.9, size=(outputs // 128) * (inputs // 128)).astype(np.float32)
    return codes, scales


@pytest.mark.parametrize("outputs,inputs", [(128, 128), (128, 384), (256, 640), (384, 256)])
def test_block128_re_lay_out_is_the_definition_and_a_bijection(outputs, inputs):
    native, reference = amd.WEIGHT_FORMAT_E4M3_BLOCK128_GFX950, amd.WEIGHT_FORMAT_E4M3_BLOCK128
    codes, scales = block128_matrix(outputs + inputs, outputs, inputs)
    stored = laid_out(reference, codes, scales.view(np.uint8))
    packed = amd.gfx950_pack(native, outputs, inputs, stored)
    assert packed.nbytes == stored.nbytes == outputs * inputs + scales.nbytes == int(orc.orc_linear_stored_bytes(native, outputs, inputs))
    assert np.array_equal(packed, laid_out(native, codes, scales.view(np.uint8))), "the library's re-lay-out is the oracle's lay-out of the definition"
    assert np.array_equal(packed[outputs * inputs:], scales.view(np.uint8)), "the float32 scales stay as they are"
    # the codes go where E4M3_GFX950's go: the same permutation of the first outputs x inputs bytes
    like = np.concatenate([stored[:outputs * inputs], np.zeros((outputs // 32) * (inputs // 32), dtype=np.uint8)])
    assert np.array_equal(amd.gfx950_pack(amd.WEIGHT_FORMAT_E4M3_GFX950, outputs, inputs, like)[:outputs * inputs], packed[:outputs * inputs])
    assert np.array_equal(amd.gfx950_unpack(native, outputs, inputs, packed), stored)
    noise = np.random.default_rng(6).integers(0, 256, size=stored.nbytes, dtype=np.uint8)
    assert np.array_equal(amd.gfx950_unpack(native, outputs, inputs, amd.gfx950_pack(native, outputs, inputs, noise)), noise)
    assert np.array_equal(amd.gfx950_pack(native, outputs, inputs, amd.gfx950_unpack(native, outputs, inputs, noise)), noise)


def test_block128_the_oracle_reads_the_same_matrix_back_and_the_same_products():
    native, reference = amd.WEIGHT_FORMAT_E4M3_BLOCK128_GFX950, amd.WEIGHT_FORMAT_E4M3_BLOCK128
    outputs, inputs, vectors = 256, 384, 3
    codes, scales = block128_matrix(31, outputs, inputs)
    stored = laid_out(reference, codes, scales.view(np.uint8))
    packed = amd.gfx950_pack(native, outputs, inputs, stored)
    code, scale = C.c_uint32(), C.c_uint32()
    bits = scales.view(np.uint32)
    for output in range(0, outputs, 3):
        for i in range(inputs):
            assert orc.orc_linear_read(native, outputs, inputs, packed.ctypes.data_as(u8p), output, i, C.byref(code), C.byref(scale)) == 0
            assert (code.value, scale.value) == (int(codes[output, i]), int(bits[(output // 128) * (inputs // 128) + i // 128])), (output, i)
    rng = np.random.default_rng(3)
    fed = rng.integers(0, 0x7E, size=(vectors, inputs), dtype=np.uint8) | (rng.integers(0, 2, size=(vectors, inputs), dtype=np.uint8) << 7)
    fed_scales = rng.uniform(0.01, 2.0, size=(vectors, inputs // 128)).astype(np.float32)
    sums = [np.zeros((vectors, outputs)), np.zeros((vectors, outputs))]
    f32p, f64p = C.POINTER(C.c_float), C.POINTER(C.c_double)
    for fmt, bytes_, out in ((reference, stored, sums[0]), (native, packed, sums[1])):
        assert orc.orc_linear_products_128_of(fmt, outputs, inputs, bytes_.ctypes.data_as(u8p), 0, outputs, fed.ctypes.data_as(u8p),
                                              fed_scales.ctypes.data_as(f32p), vectors, out.ctypes.data_as(f64p), None) == 0
    assert np.array_equal(sums[0], sums[1]) and np.abs(sums[0]).max() > 0
    # a format of E8M0 scale codes is refused by the float32-scale products
    assert orc.orc_linear_products_128_of(amd.WEIGHT_FORMAT_E4M3_GFX950, outputs, inputs, packed.ctypes.data_as(u8p), 0, outputs, fed.ctypes.data_as(u8p),
                                          fed_scales.ctypes.data_as(f32p), vectors, sums[0].ctypes.data_as(f64p), None) == -1


def test_block128_refusals():
    lib = amd.library()
    native = amd.WEIGHT_FORMAT_E4M3_BLOCK128_GFX950
    for outputs, inputs in ((64, 256), (128, 192), (128, 0), (160, 128)):  # whole blocks of 128 x 128 only
        shape = amd.Shape(outputs, inputs, 8, 0)
        stored = np.zeros(max(1, outputs * inputs + 64), dtype=np.uint8)
        out = np.full_like(stored, 0xEE)
        assert lib.weight_format_gfx950_pack(native, C.byref(shape), stored.ctypes.data, stored.nbytes, out.ctypes.data, out.nbytes) == amd.STATUS_INVALID_ARGUMENT
        assert np.all(out == 0xEE)
    shape = amd.Shape(128, 256, 4, 0)  # a width of four bits
    exact = 128 * 256 + 8
    stored, out = np.zeros(exact, dtype=np.uint8), np.full(exact, 0xEE, dtype=np.uint8)
    assert lib.weight_format_gfx950_pack(native, C.byref(shape), stored.ctypes.data, exact, out.ctypes.data, exact) == 1 and np.all(out == 0xEE)
    shape = amd.Shape(128, 256, 8, 0)
    assert lib.weight_format_gfx950_pack(native, C.byref(shape), stored.ctypes.data, exact - 1, out.ctypes.data, exact) == 1 and np.all(out == 0xEE)
    assert lib.weight_format_gfx950_pack(native, C.byref(shape), stored.ctypes.data, exact, out.ctypes.data, exact) == 0


def test_refusals_and_byte_counts():
    lib = amd.library()
    count = C.c_uint64(0)
    operations = lib.weight_format_operations_of
    operations.restype = C.c_void_p
    for native, reference, bits in FORMATS:
        for outputs, inputs, ok in ((64, 256, True), (64, 192, False), (32, 128, bits == 8), (64, 0, False)):
            shape = amd.Shape(outputs, inputs, bits, 0)
            stored = np.zeros(max(1, outputs * inputs * bits // 8 + outputs * inputs // 32), dtype=np.uint8)
            out = np.full_like(stored, 0xEE)
            status = lib.weight_format_gfx950_pack(native, C.byref(shape), stored.ctypes.data, stored.nbytes, out.ctypes.data, out.nbytes)
            if ok:
                exact = int(orc.orc_linear_stored_bytes(native, outputs, inputs))
                assert lib.weight_format_gfx950_pack(native, C.byref(shape), stored.ctypes.data, exact, out.ctypes.data, exact) == 0
            else:
                assert status == amd.STATUS_INVALID_ARGUMENT and np.all(out == 0xEE), (native, outputs, inputs)
        shape = amd.Shape(64, 256, bits, 0)
        exact = int(orc.orc_linear_stored_bytes(native, 64, 256))
        stored, out = np.zeros(exact, dtype=np.uint8), np.full(exact, 0xEE, dtype=np.uint8)
        assert lib.weight_format_gfx950_pack(native, C.byref(shape), stored.ctypes.data, exact - 1, out.ctypes.data, exact) == 1  # a source too short
        assert lib.weight_format_gfx950_pack(native, C.byref(shape), stored.ctypes.data, exact, stored.ctypes.data + 16, exact) == 1  # the two share bytes
        assert lib.weight_format_gfx950_pack(reference, C.byref(shape), stored.ctypes.data, exact, out.ctypes.data, exact) == 1  # not a GFX950 format
        assert lib.weight_format_gfx950_pack(native, C.byref(shape), None, exact, out.ctypes.data, exact) == 1
        assert np.all(out == 0xEE)
