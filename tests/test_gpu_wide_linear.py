"""GPU parity of the wide form of the FP4/FP8 routed experts (a grouped GEMM over the wide select's tiles of at most 64
pairs of one expert) through the C ABI. Two bars: byte for byte against the job-table kernels of one slice, which the
oracle pins (the reference holds its wide experts to the same bar against its narrow ones,
tests/expert_wide_card_test.c:3-9), and the layer's row outputs against the CPU oracle."""
import ctypes as C
import sys

import numpy as np
import pytest

from _oracle import f32p, normals, orc, ptr, to_bf16, u16p, u32p

pytestmark = pytest.mark.gpu

E2M1, E4M3 = 3, 5


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


def build(amd, card, hidden, inner, experts_n, picks, rows, seed, fmt, distinct=8):
    """A layer whose experts cycle through `distinct` trios of matrices (building 64 distinct ones is host time only)."""
    from anemone_amd import workloads
    matrix = workloads.fp4_matrix if fmt == E2M1 else workloads.fp8_matrix
    trios = [[matrix(seed * 1000 + 3 * e + 0, inner, hidden), matrix(seed * 1000 + 3 * e + 1, inner, hidden),
              matrix(seed * 1000 + 3 * e + 2, hidden, inner)] for e in range(distinct)]
    matrices = [trios[e % distinct] for e in range(experts_n)]
    router = to_bf16(normals(seed + 5, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    layer = amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, matrices, router_weights_bf16=router, weight_format=fmt)
    return layer, matrices


@pytest.mark.parametrize("hidden,inner,experts_n,picks,rows,live,fmt", [
    (512, 256, 64, 4, 300, 300, E2M1),    # whole blocks of four strips
    (640, 384, 64, 4, 200, 177, E2M1),    # the last block of each product holds two live strips; rows beyond the live ones
    (512, 256, 64, 8, 40, 40, E2M1),      # most tiles hold a few pairs
    (512, 256, 64, 4, 300, 300, E4M3),
    (640, 384, 64, 2, 450, 449, E4M3),
    (512, 256, 64, 1, 700, 700, E2M1),    # one pick a row
    (512, 256, 64, 8, 1500, 1500, E2M1),  # runs of three tiles and more: blocks of two tiles of one expert, and a run's odd last tile
    (640, 384, 64, 8, 1100, 1003, E2M1),
    (512, 256, 64, 8, 1500, 1401, E4M3),
])
def test_wide_equals_the_job_table_kernels_byte_for_byte(amd, card, hidden, inner, experts_n, picks, rows, live, fmt):
    say("wide experts", hidden, inner, experts_n, picks, rows, live, fmt)
    layer, _ = build(amd, card, hidden, inner, experts_n, picks, rows, 21, fmt)
    x = to_bf16(normals(31, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x, live)
    card.run(layer.projection_launch())
    wide = layer.wide_router()
    card.run(wide.launches())
    card.run(layer.quantize_launch())
    names = ("hidden_codes", "hidden_exponents", "hidden_operands", "pair_output", "row_output")

    def run(launches):
        for name in names:
            card.upload(layer.ranges[name].byte_offset, np.full(layer.ranges[name].byte_count, 0xEE, dtype=np.uint8))
        card.run(launches)
        return [layer.read(name).copy() for name in names]
    narrow = run(layer.expert_launches(wide))
    broad = run(layer.wide_expert_launches(wide))
    pairs = live * picks
    for name, a, b in zip(names, narrow, broad):
        per = a.size // (rows if name == "row_output" else rows * picks)
        count = (live if name == "row_output" else pairs) * per
        differing = np.flatnonzero(a.reshape(-1)[:count] != b.reshape(-1)[:count])
        say("  %s: %d of %d bytes differ" % (name, differing.size, count))
        assert differing.size == 0, (name, differing[:8], per)
    # the wide launches write nothing for the pairs of the rows beyond the live ones
    if live < rows:
        for name, b in zip(names[:4], broad[:4]):
            per = b.size // (rows * picks)
            assert np.all(b.reshape(-1)[pairs * per:] == 0xEE), name


def test_wide_layer_against_oracle(amd, card):
    """The whole layer in its wide form (projection, wide select, quantizer, wide gate/up, wide down, row sum) against
    the CPU oracle's layer of the same picks."""
    say("wide layer against the oracle")
    from anemone_amd import workloads
    from test_gpu_router_wide import oracle_wide
    hidden, inner, experts_n, picks, rows, live = 512, 256, 64, 4, 150, 143
    matrices = [[workloads.fp4_matrix(9000 + 3 * e, inner, hidden), workloads.fp4_matrix(9001 + 3 * e, inner, hidden),
                 workloads.fp4_matrix(9002 + 3 * e, hidden, inner)] for e in range(experts_n)]
    router = to_bf16(normals(5, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    layer = amd.Fp4Layer(card, hidden, inner, experts_n, picks, rows, matrices, router_weights_bf16=router)
    x = to_bf16(normals(9, rows * hidden)).reshape(rows, hidden)
    layer.set_rows(x, live)
    card.run(layer.projection_launch())
    wide = layer.wide_router()
    card.run(wide.launches())
    card.run(layer.quantize_launch())
    card.run(layer.wide_expert_launches(wide))
    scores = card.download(layer.scores_offset, rows * experts_n * 4, np.float32).reshape(rows, experts_n)
    _, experts, weights, _, _, _, _ = oracle_wide(layer, scores, np.zeros(experts_n, dtype=np.float32), live)
    pointers = (C.c_void_p * (experts_n * 3))(*[m.ctypes.data for trio in matrices for m in trio])
    want = np.zeros((live, hidden), dtype=np.float32)
    orc.orc_linear_moe_layer(3, ptr(np.ascontiguousarray(x[:live]), u16p), live, hidden, inner, picks,
                             ptr(np.ascontiguousarray(experts[:live]), u32p), ptr(np.ascontiguousarray(weights[:live]), f32p),
                             experts_n, pointers, 10.0, ptr(want, f32p), None, None, 8)
    got = layer.read("row_output", np.float32).reshape(rows, hidden)[:live]
    error = np.sqrt(np.mean((got - want) ** 2) / np.mean(want.astype(np.float64) ** 2))
    say("  layer rms error vs oracle: %.2e" % error)
    assert error < 2e-2
