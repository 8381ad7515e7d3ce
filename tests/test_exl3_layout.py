"""The load-time EXL3 slices (include/anemone/exl3_layout.h:15-103 of the reference): this library's
bb_exl3_matrix_slice_prepare / _copy / bb_exl3_output_shard_prepare against the reference's own source/exl3_layout.c
(built from where it lies into oracle/_ref) byte for byte and status for status, and against what the stored layout
fixes (a slice's decoded weights are the whole matrix's submatrix, by the oracle's decoder). No GPU."""
import ctypes as C

import numpy as np
import pytest

import anemone_amd as amd
from _oracle import exl3_matrix, orc, ptr, ref, u8p, u16p

u32, u64 = C.c_uint32, C.c_uint64


class Slice(C.Structure):
    _fields_ = [(name, u32) for name in ("input_size", "output_size", "input_begin", "input_count", "output_begin", "output_count",
                                         "bits_per_weight", "reserved_zero")]


class Sizes(C.Structure):
    _fields_ = [("source_bytes", u64), ("packed_bytes", u64)]


class Plan(C.Structure):
    _fields_ = [("gate_up", Slice), ("down", Slice), ("rank_count", u32), ("rank", u32), ("product_slices", u32), ("order", u32)]


def bind(lib):
    lib.bb_exl3_matrix_slice_prepare.restype = C.c_int
    lib.bb_exl3_matrix_slice_prepare.argtypes = [C.POINTER(Slice), C.POINTER(Sizes)]
    lib.bb_exl3_matrix_slice_copy.restype = C.c_int
    lib.bb_exl3_matrix_slice_copy.argtypes = [C.POINTER(Slice), C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t]
    lib.bb_exl3_output_shard_prepare.restype = C.c_int
    lib.bb_exl3_output_shard_prepare.argtypes = [u32, u32, u32, u32, u32, C.c_int, C.POINTER(Plan)]
    return lib


mine = bind(amd.library())
theirs = bind(ref) if ref is not None and hasattr(ref, "bb_exl3_matrix_slice_copy") else None
needs_ref = pytest.mark.skipif(theirs is None, reason="the reference's exl3_layout.c is not built")


def copy_by(lib, description, matrix, room=0, fill=0xEE):
    sizes = Sizes()
    assert lib.bb_exl3_matrix_slice_prepare(C.byref(description), C.byref(sizes)) == 0
    out = np.full(sizes.packed_bytes + room, fill, dtype=np.uint8)
    status = lib.bb_exl3_matrix_slice_copy(C.byref(description), matrix.ctypes.data, matrix.nbytes, out.ctypes.data, out.nbytes)
    return status, sizes, out


@needs_ref
@pytest.mark.parametrize("width", [2, 3, 4])
def test_copy_equals_the_reference_byte_for_byte(width):
    inputs, outputs = 512, 768
    matrix = exl3_matrix(100 + width, inputs, outputs, width)
    rng = np.random.default_rng(width)
    for _ in range(12):
        ib, ob = int(rng.integers(0, 4)) * 128, int(rng.integers(0, 6)) * 128
        ic, oc = int(rng.integers(1, (inputs - ib) // 128 + 1)) * 128, int(rng.integers(1, (outputs - ob) // 128 + 1)) * 128
        d = Slice(inputs, outputs, ib, ic, ob, oc, width, 0)
        a, sizes_a, out_a = copy_by(mine, d, matrix, room=64)
        b, sizes_b, out_b = copy_by(theirs, d, matrix, room=64)
        assert a == b == 0 and (sizes_a.source_bytes, sizes_a.packed_bytes) == (sizes_b.source_bytes, sizes_b.packed_bytes)
        assert sizes_a.source_bytes == matrix.nbytes and np.array_equal(out_a, out_b)
        assert np.all(out_a[sizes_a.packed_bytes:] == 0xEE)  # the room behind the slice is not touched


@needs_ref
def test_refusals_equal_the_reference():
    matrix = exl3_matrix(7, 256, 256, 3)
    good = dict(input_size=256, output_size=256, input_begin=0, input_count=128, output_begin=128, output_count=128, bits_per_weight=3, reserved_zero=0)
    cases = [dict(), dict(reserved_zero=1), dict(input_count=0), dict(output_count=0), dict(input_size=200), dict(output_begin=64),
             dict(input_begin=256, input_count=128), dict(output_begin=128, output_count=256), dict(bits_per_weight=0), dict(bits_per_weight=9),
             dict(input_count=64), dict(input_begin=128, input_count=128), dict(output_begin=0, output_count=256)]
    for changes in cases:
        d = Slice(**{**good, **changes})
        sizes_a, sizes_b = Sizes(1, 2), Sizes(1, 2)
        a, b = mine.bb_exl3_matrix_slice_prepare(C.byref(d), C.byref(sizes_a)), theirs.bb_exl3_matrix_slice_prepare(C.byref(d), C.byref(sizes_b))
        assert a == b, changes
        assert (sizes_a.source_bytes, sizes_a.packed_bytes) == (sizes_b.source_bytes, sizes_b.packed_bytes), changes
    d = Slice(**good)
    out = np.zeros(1 << 20, dtype=np.uint8)
    for lib in (mine, theirs):
        assert lib.bb_exl3_matrix_slice_copy(C.byref(d), matrix.ctypes.data, matrix.nbytes - 1, out.ctypes.data, out.nbytes) == 1   # a source too short
        assert lib.bb_exl3_matrix_slice_copy(C.byref(d), matrix.ctypes.data, matrix.nbytes, out.ctypes.data, 100) == 1            # a destination too short
        assert lib.bb_exl3_matrix_slice_copy(C.byref(d), matrix.ctypes.data, matrix.nbytes, matrix.ctypes.data + 64, matrix.nbytes - 64) == 1  # overlap
        assert lib.bb_exl3_matrix_slice_copy(None, matrix.ctypes.data, matrix.nbytes, out.ctypes.data, out.nbytes) == 1
        assert lib.bb_exl3_matrix_slice_prepare(C.byref(d), None) == 1
    assert not out.any()


@needs_ref
def test_shard_plans_equal_the_reference():
    for outer, inner in ((4096, 2048), (5120, 2560), (512, 640), (384, 512)):
        for ranks in (1, 4, 2, 0):
            for rank in range(max(ranks, 1) + 1):
                for order in (0, 1, 2):
                    for width in (3, 4):
                        a, b = Plan(), Plan()
                        C.memset(C.byref(a), 0xAB, C.sizeof(a))
                        C.memset(C.byref(b), 0xAB, C.sizeof(b))
                        sa = mine.bb_exl3_output_shard_prepare(outer, inner, width, ranks, rank, order, C.byref(a))
                        sb = theirs.bb_exl3_output_shard_prepare(outer, inner, width, ranks, rank, order, C.byref(b))
                        assert sa == sb and bytes(a) == bytes(b), (outer, inner, ranks, rank, order, width)
    assert C.sizeof(Slice) == 32 and C.sizeof(Plan) == 80


def test_a_slice_decodes_to_the_submatrix():
    """The stored layout alone fixes this: the slice of a matrix, decoded by the oracle, is the whole matrix's decoded
    weights of the slice's inputs and outputs; K2.5 (stored width 40) included."""
    for width in (2, 40, 3, 4):
        inputs, outputs = 384, 512
        matrix = exl3_matrix(300 + width, inputs, outputs, width)
        whole = np.zeros((inputs, outputs), dtype=np.uint16)
        orc.orc_exl3_decode_matrix(ptr(matrix, u8p), inputs, outputs, width, ptr(whole, u16p))
        d = Slice(inputs, outputs, 128, 256, 256, 128, width, 0)
        status, sizes, out = copy_by(mine, d, matrix)
        assert status == 0
        part = np.zeros((256, 128), dtype=np.uint16)
        orc.orc_exl3_decode_matrix(ptr(out, u8p), 256, 128, width, ptr(part, u16p))
        assert np.array_equal(part, whole[128:384, 256:384])
        # the scales behind the codes: suh of the inputs, svh of the outputs
        code_bytes = int(orc.orc_exl3_code_bytes(inputs, outputs, width))
        scales = matrix[code_bytes:].view(np.uint16)
        part_scales = out[int(orc.orc_exl3_code_bytes(256, 128, width)):].view(np.uint16)
        assert np.array_equal(part_scales[:256], scales[128:384]) and np.array_equal(part_scales[256:], scales[inputs + 256:inputs + 384])


def test_four_ranks_cover_a_layer_once():
    covered_inner, covered_outer = np.zeros(2048, int), np.zeros(4096, int)
    for rank in range(4):
        plan = Plan()
        assert mine.bb_exl3_output_shard_prepare(4096, 2048, 3, 4, rank, 0, C.byref(plan)) == 0
        covered_inner[plan.gate_up.output_begin:plan.gate_up.output_begin + plan.gate_up.output_count] += 1
        covered_outer[plan.down.output_begin:plan.down.output_begin + plan.down.output_count] += 1
        assert (plan.gate_up.input_begin, plan.gate_up.input_count) == (0, 4096) and (plan.down.input_begin, plan.down.input_count) == (0, 2048)
        assert plan.product_slices == 4
    assert np.all(covered_inner == 1) and np.all(covered_outer == 1)
