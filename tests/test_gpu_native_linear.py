"""GPU parity of the wide routed experts whose weights lie in gfx950's own lane order (WEIGHT_FORMAT_E2M1_GFX950,
WEIGHT_FORMAT_E4M3_GFX950, WEIGHT_FORMAT_E4M3_BLOCK128_GFX950; the matrices go through the library's load-time re-lay-out, weight_format_gfx950_pack), through
the C ABI: byte for byte the outputs of the same layer in the reference's lay-out (kernel_wide_linear.hip's launches,
which tests/test_gpu_wide_linear.py holds byte for byte to the job-table kernels and those to the oracle), and the
layer's rows against the CPU oracle reading the re-laid-out bytes itself."""
import ctypes as C
import sys

import numpy as np
import pytest

from _oracle import f32p, normals, orc, ptr, to_bf16, u16p, u32p

pytestmark = pytest.mark.gpu

E2M1, E4M3, B128, E2M1_GFX950, E4M3_GFX950, B128_GFX950 = 3, 5, 6, 7, 8, 9
NATIVE_OF = {E2M1: E2M1_GFX950, E4M3: E4M3_GFX950, B128: B128_GFX950}
NAMES = ("hidden_codes", "hidden_exponents", "hidden_operands", "pair_output", "row_output")


def say(*words):
    print(*words, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def amd():
    import anemone_amd
    return anemone_amd


@pytest.fixture(scope="module")
def card(amd):
    card = amd.Card(3 << 30)
    yield card
    card.close()


@pytest.fixture(autouse=True)
def fresh_arena(card):
    card.cursor = 256
    yield


def matrices_of(hidden, inner, experts_n, seed, fmt, distinct=8):
    from anemone_amd import workloads
    matrix = workloads.fp4_matrix if fmt == E2M1 else workloads.fp8_block128_matrix if fmt == B128 else workloads.fp8_matrix
    trios = [[matrix(seed * 1000 + 3 * e + 0, inner, hidden), matrix(seed * 1000 + 3 * e + 1, inner, hidden),
              matrix(seed * 1000 + 3 * e + 2, hidden, inner)] for e in range(distinct)]
    return [trios[e % distinct] for e in range(experts_n)]


def run_wide(card, layer, x, live):
    layer.set_rows(x, live)
    card.run(layer.projection_launch())
    wide = layer.wide_router()
    card.run(wide.launches())
    card.run(layer.quantize_launch())
    for name in NAMES:
        card.upload(layer.ranges[name].byte_offset, np.full(layer.ranges[name].byte_count, 0xEE, dtype=np.uint8))
    card.run(layer.wide_expert_launches(wide))
    return [layer.read(name).copy() for name in NAMES], wide


@pytest.mark.parametrize("hidden,inner,experts_n,picks,rows,live,fmt", [
    (512, 256, 64, 4, 300, 300, E2M1),    # whole blocks of four strips
    (640, 384, 64, 4, 200, 177, E2M1),    # the last block of each product holds two live strips; rows beyond the live ones
    (512, 256, 64, 8, 40, 40, E2M1),      # most tiles hold a few pairs
    (512, 256, 64, 4, 300, 300, E4M3),
    (640, 384, 64, 2, 450, 449, E4M3),
    (512, 256, 64, 1, 700, 700, E2M1),    # one pick a row
    (512, 256, 64, 8, 1500, 1500, E2M1),  # runs of three tiles and more
    (640, 384, 64, 8, 1100, 1003, E2M1),
    (512, 256, 64, 8, 1500, 1401, E4M3),  # blocks of two tiles of one expert, a run's odd last tile alone
    (512, 256, 64, 8, 6000, 5999, E4M3),  # runs of a dozen tiles: the places of a run's tiles by the lanes' look back
    (512, 256, 64, 1, 4300, 4300, -E4M3), # one expert takes every row: a run of 68 tiles, the look back goes round again
    (512, 256, 64, 4, 300, 300, B128),    # float32 scales of 128 x 128 blocks: the quantizer between the two products
    (640, 384, 64, 2, 450, 449, B128),
    (512, 256, 64, 8, 1500, 1401, B128),
    (512, 256, 64, 1, 4300, 4300, -B128),
    # chains of one, two and three K steps: fewer steps than sets of weight registers and stages of columns
    (128, 128, 64, 4, 300, 300, E2M1),
    (256, 128, 64, 4, 300, 297, E2M1),
    (384, 256, 64, 2, 500, 500, E2M1),
    (128, 128, 64, 4, 600, 600, E4M3),
    (256, 128, 64, 8, 300, 300, E4M3),
    (384, 256, 64, 2, 500, 499, E4M3),
    (128, 128, 64, 4, 600, 600, B128),
    (256, 128, 64, 8, 300, 299, B128),
    (384, 256, 64, 2, 500, 500, B128),
])
def test_native_equals_the_reference_lay_out_byte_for_byte(amd, card, hidden, inner, experts_n, picks, rows, live, fmt):
    say("native experts", hidden, inner, experts_n, picks, rows, live, fmt)
    one_expert, fmt = fmt < 0, abs(fmt)
    matrices = matrices_of(hidden, inner, experts_n, 21, fmt)
    router = to_bf16(normals(26, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    x = to_bf16(normals(31, rows * hidden)).reshape(rows, hidden)
    bias = np.zeros(experts_n, dtype=np.float32)
    if one_expert:
        bias[5] = 100.0
    reference = amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, matrices, router_weights_bf16=router, weight_format=fmt)
    card.upload(reference.bias_offset, bias)
    want, wide = run_wide(card, reference, x, live)
    counts = np.bincount(wide.read("picks", np.dtype([("expert", "<u4"), ("route_weight", "<f4")]))["expert"][:live * picks], minlength=experts_n)
    say("  pairs of the busiest expert:", int(counts.max()))
    native = amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, matrices, router_weights_bf16=router,
                          weight_format=NATIVE_OF[fmt])
    card.upload(native.bias_offset, bias)
    got, _ = run_wide(card, native, x, live)
    pairs = live * picks
    for name, a, b in zip(NAMES, want, got):
        per = a.size // (rows if name == "row_output" else rows * picks)
        count = (live if name == "row_output" else pairs) * per
        differing = np.flatnonzero(a.reshape(-1)[:count] != b.reshape(-1)[:count])
        say("  %s: %d of %d bytes differ" % (name, differing.size, count))
        assert differing.size == 0, (name, differing[:8], per)
        assert a.reshape(-1)[:count].tobytes() != bytes([0xEE]) * count, "the launches wrote"
    if live < rows:  # nothing is written for the pairs of the rows beyond the live ones
        for name, b in zip(NAMES[:4], got[:4]):
            if fmt == B128 and name in ("hidden_codes", "hidden_exponents"):
                continue  # the quantizer of 128 values a scale is a launch over every pair the step has room for
            per = b.size // (rows * picks)
            assert np.all(b.reshape(-1)[pairs * per:] == 0xEE), name


@pytest.mark.parametrize("fmt", [E2M1, E4M3, B128])
def test_native_layer_against_oracle(amd, card, fmt):
    """The layer in gfx950's lay-out against the CPU oracle reading the SAME re-laid-out bytes (its own reading of the
    format, oracle/orc_linear.c) with the picks the card made."""
    say("native layer against the oracle", fmt)
    from test_gpu_router_wide import oracle_wide
    hidden, inner, experts_n, picks, rows, live = 512, 256, 64, 4, 150, 143
    native_format = NATIVE_OF[fmt]
    matrices = matrices_of(hidden, inner, experts_n, 33, fmt, distinct=64)
    router = to_bf16(normals(5, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    layer = amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, matrices, router_weights_bf16=router, weight_format=native_format)
    x = to_bf16(normals(9, rows * hidden)).reshape(rows, hidden)
    got, _ = run_wide(card, layer, x, live)
    scores = card.download(layer.scores_offset, rows * experts_n * 4, np.float32).reshape(rows, experts_n)
    _, experts, weights, _, _, _, _ = oracle_wide(layer, scores, np.zeros(experts_n, dtype=np.float32), live)
    packed = [[amd.gfx950_pack(native_format, *((inner, hidden) if m < 2 else (hidden, inner)), matrix) for m, matrix in enumerate(trio)] for trio in matrices]
    pointers = (C.c_void_p * (experts_n * 3))(*[m.ctypes.data for trio in packed for m in trio])
    want = np.zeros((live, hidden), dtype=np.float32)
    orc.orc_linear_moe_layer(native_format, ptr(np.ascontiguousarray(x[:live]), u16p), live, hidden, inner, picks,
                             ptr(np.ascontiguousarray(experts[:live]), u32p), ptr(np.ascontiguousarray(weights[:live]), f32p),
                             experts_n, pointers, 10.0, ptr(want, f32p), None, None, 8)
    row_output = got[4].view(np.float32).reshape(rows, hidden)[:live]
    error = np.sqrt(np.mean((row_output - want) ** 2) / np.mean(want.astype(np.float64) ** 2))
    say("  layer rms error vs oracle: %.2e" % error)
    assert error < 2e-2


def run_jobs(card, layer, x, live):
    layer.set_rows(x, live)
    card.run(layer.projection_launch())
    card.run(layer.select_launch(0))
    card.run(layer.quantize_launch())
    for name in ("hidden",) + NAMES:
        card.upload(layer.ranges[name].byte_offset, np.full(layer.ranges[name].byte_count, 0xEE, dtype=np.uint8))
    card.run(layer.expert_launches())
    return [layer.read(name).copy() for name in ("hidden",) + NAMES], layer.jobs().copy()


@pytest.mark.parametrize("hidden,inner,picks,rows,live,fmt,gate_up_slices,down_slices", [
    (512, 256, 4, 8, 8, E2M1, 4, 2),     # the slice counts the card's order takes
    (512, 256, 4, 8, 7, E2M1, 1, 1),     # one chain; a row beyond the live ones
    (1024, 512, 8, 3, 3, E2M1, 8, 4),
    (640, 384, 2, 5, 5, E2M1, 2, 1),     # five K steps over two slices: chains of two and three steps
    (512, 256, 4, 8, 8, E4M3, 4, 2),
    (640, 384, 8, 2, 2, E4M3, 1, 2),     # 40 tiles of the gate product: strips of two
    (1024, 512, 1, 8, 5, E4M3, 8, 4),
    (512, 256, 4, 8, 8, B128, 4, 2),
    (640, 384, 8, 2, 2, B128, 1, 2),
    (1024, 512, 1, 8, 5, B128, 8, 4),
    (640, 384, 2, 5, 5, B128, 2, 1),
    (128, 128, 4, 8, 8, E2M1, 1, 1),     # one K step
    (256, 128, 4, 8, 7, E4M3, 2, 1),     # two K steps over two slices: a step a chain
    (128, 128, 2, 6, 6, B128, 1, 1),
    (384, 256, 8, 4, 4, E2M1, 1, 2),
])
def test_native_job_table_kernels_equal_the_reference_lay_out(amd, card, hidden, inner, picks, rows, live, fmt, gate_up_slices, down_slices):
    """The job-table kernels (a thin step's) of the formats in gfx950's lane order, expert_gate_up_gfx950_<S> and its like:
    byte for byte what the reference-format kernels of the same slice counts write for the same matrices."""
    say("native job-table kernels", hidden, inner, picks, rows, live, fmt, gate_up_slices, down_slices)
    experts_n = 64
    matrices = matrices_of(hidden, inner, experts_n, 41, fmt, distinct=16)
    router = to_bf16(normals(43, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    x = to_bf16(normals(47, rows * hidden)).reshape(rows, hidden)
    reference = amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, matrices, router_weights_bf16=router, weight_format=fmt,
                             gate_up_slices=gate_up_slices, down_slices=down_slices)
    want, want_jobs = run_jobs(card, reference, x, live)
    native = amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, matrices, router_weights_bf16=router,
                          weight_format=NATIVE_OF[fmt], gate_up_slices=gate_up_slices, down_slices=down_slices)
    got, got_jobs = run_jobs(card, native, x, live)
    assert np.array_equal(want_jobs["expert"], got_jobs["expert"]) and np.array_equal(want_jobs["pair_index"], got_jobs["pair_index"])
    pairs = live * picks
    for name, a, b in zip(("hidden",) + NAMES, want, got):
        per = a.size // (rows if name == "row_output" else rows * picks)
        count = (live if name == "row_output" else pairs) * per
        differing = np.flatnonzero(a.reshape(-1)[:count] != b.reshape(-1)[:count])
        say("  %s: %d of %d bytes differ" % (name, differing.size, count))
        assert differing.size == 0, (name, differing[:8], per)
        if not (fmt == B128 and name == "hidden_operands"):  # the quantizer of 128 values a scale writes no operands
            assert a.reshape(-1)[:count].tobytes() != bytes([0xEE]) * count, "the launches wrote"
