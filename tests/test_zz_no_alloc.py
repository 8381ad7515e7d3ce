"""exl3_tc_run_static (the fused EXL3 decode with its workspace in an array the library holds on the device: the entry
point for callers that cannot allocate) against exl3_tc_prepare + launch_run on the same bytes: two calls in a row,
the second of a smaller step, each bit for bit the other entry point's output. The arena the static call reads is the
caller's own memory (allocated here from the HIP runtime the library itself is linked to, through ctypes: one runtime in
the process whatever ran before), a copy of the card's arena as the select left it."""
import ctypes as C
import sys

import numpy as np
import pytest

from _oracle import normals, splitmix_words, to_bf16, exl3_matrix


def say(*words):
    print(*words, flush=True)
    sys.stdout.flush()


def hip_runtime():
    hip = C.CDLL("libamdhip64.so.7")  # the library's own: already loaded with it
    hip.hipMalloc.argtypes, hip.hipMalloc.restype = [C.POINTER(C.c_void_p), C.c_size_t], C.c_int
    hip.hipMemcpy.argtypes, hip.hipMemcpy.restype = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int], C.c_int
    hip.hipFree.argtypes, hip.hipFree.restype = [C.c_void_p], C.c_int
    hip.hipDeviceSynchronize.argtypes, hip.hipDeviceSynchronize.restype = [], C.c_int
    hip.hipMemGetInfo.argtypes, hip.hipMemGetInfo.restype = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)], C.c_int
    hip.hipStreamCreate.argtypes, hip.hipStreamCreate.restype = [C.POINTER(C.c_void_p)], C.c_int
    hip.hipStreamSynchronize.argtypes, hip.hipStreamSynchronize.restype = [C.c_void_p], C.c_int
    hip.hipStreamDestroy.argtypes, hip.hipStreamDestroy.restype = [C.c_void_p], C.c_int
    return hip


def one_step(amd, hip, rows, seed, own_stream=False):
    hidden, inner, experts_n, picks = 512, 256, 64, 4
    width_choices = [2, 3, 4, 40]
    draws = splitmix_words(seed, experts_n * 3) % np.uint64(len(width_choices))
    widths = np.array(width_choices, dtype=np.uint32)[draws.astype(np.int64)].reshape(experts_n, 3)
    matrices = [[exl3_matrix(seed * 1000 + 3 * e + 0, hidden, inner, int(widths[e, 0])),
                 exl3_matrix(seed * 1000 + 3 * e + 1, hidden, inner, int(widths[e, 1])),
                 exl3_matrix(seed * 1000 + 3 * e + 2, inner, hidden, int(widths[e, 2]))] for e in range(experts_n)]
    router = to_bf16(normals(seed + 5, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    x = to_bf16(normals(seed + 9, rows * hidden)).reshape(rows, hidden)
    card = amd.Card(1 << 30)
    try:
        layer = amd.Exl3Layer(card, hidden, inner, experts_n, picks, rows, matrices, widths, router_weights_bf16=router, affinity_kind=1, limit=10.0)
        layer.set_rows(x, rows)
        card.run(layer.projection_launch())
        card.run(layer.select_launch(0))
        launches = layer.tc_launches()
        used = (card.cursor + 255) // 256 * 256
        before = card.download(0, used).copy()  # the arena as the select left it
        card.run(launches)
        want = layer.output().copy()
        record = layer.tc_record()
    finally:
        card.close()
    out_bytes = rows * hidden * 4
    before[record.output_offset:record.output_offset + out_bytes] = 0xFF
    record.workspace_offset = 0x12345600  # ignored by the static entry point
    arena = C.c_void_p()
    assert hip.hipMalloc(C.byref(arena), before.nbytes) == 0
    try:
        assert hip.hipMemcpy(arena, before.ctypes.data, before.nbytes, 1) == 0
        lib = amd.library()
        lib.exl3_tc_run_static.restype = C.c_int
        lib.exl3_tc_run_static.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_void_p]
        stream = C.c_void_p()  # NULL: the null stream
        if own_stream:
            assert hip.hipStreamCreate(C.byref(stream)) == 0
        free_before, free_after, total = C.c_size_t(), C.c_size_t(), C.c_size_t()
        assert hip.hipDeviceSynchronize() == 0 and hip.hipMemGetInfo(C.byref(free_before), C.byref(total)) == 0
        status = lib.exl3_tc_run_static(C.byref(record), arena, before.nbytes, stream)
        assert status == 0, "exl3_tc_run_static answered %d" % status
        assert (hip.hipStreamSynchronize(stream) if own_stream else hip.hipDeviceSynchronize()) == 0
        assert hip.hipMemGetInfo(C.byref(free_after), C.byref(total)) == 0
        assert free_after.value == free_before.value, "the call changed the device's free memory: %d -> %d" % (free_before.value, free_after.value)
        if own_stream:
            assert hip.hipStreamDestroy(stream) == 0
        got = np.zeros((rows, hidden), np.float32)
        assert hip.hipMemcpy(got.ctypes.data, arena.value + record.output_offset, out_bytes, 2) == 0
    finally:
        hip.hipFree(arena)
    return got, want


@pytest.mark.gpu
def test_static_workspace_equals_the_arena_workspace_twice():
    import anemone_amd as amd
    amd.library()
    hip = hip_runtime()
    for rows, seed, own_stream in ((8, 41, False), (3, 42, True)):  # the second call of a smaller step: what the first left in the array must not show
        say("exl3_tc_run_static", rows, "rows", "on a stream of the test's" if own_stream else "on the null stream")
        got, want = one_step(amd, hip, rows, seed, own_stream)
        assert np.all(np.isfinite(want)) and float(np.abs(want).max()) > 0.0
        assert got.tobytes() == want.tobytes(), "the static workspace's output differs from the arena workspace's"


def test_a_step_above_the_array_is_refused():
    import anemone_amd as amd
    lib = amd.library()
    lib.exl3_tc_run_static.restype = C.c_int
    lib.exl3_tc_run_static.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_void_p]
    record = amd.Exl3TcRecord()
    record.row_count, record.job_capacity, record.intermediate, record.hidden, record.pairs_per_row, record.bits_x2 = 64, 512, 2048, 4096, 8, 6
    assert amd.exl3_tc_workspace_bytes(64 * 8, 4096, 2048) > amd.EXL3_TC_STATIC_SCRATCH_BYTES
    assert lib.exl3_tc_run_static(C.byref(record), C.c_void_p(4096), 1 << 30, None) == 1  # before any device call
    assert lib.exl3_tc_run_static(None, C.c_void_p(4096), 1 << 30, None) == 1
