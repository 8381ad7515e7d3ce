"""Pins the router part of the CPU oracle: the reference's hand vectors (tests/golden/reference_kat.json), brute
force, sort invariants, and the reference's own C oracle (oracle/_ref) at its fixed shape 384 experts / 6 picks."""
import json
import os
from decimal import Decimal

import numpy as np
import pytest

from _oracle import (C, JOB_DTYPE, PAIR_DTYPE, RUN_DTYPE, TILE_DTYPE, f32p, normals, orc, ptr, ref, splitmix_words,
                     to_bf16, bf16_to_f32, u16p, u32p, u64p)

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kat.json")))
needs_ref = pytest.mark.skipif(ref is None, reason="oracle/_ref/libref.so was not built (no reference tree)")


def select(affinities, bias, picks, reference_order=0, scale=1.5):
    experts = np.zeros(picks, dtype=np.uint32)
    weights = np.zeros(picks, dtype=np.float32)
    orc.orc_router_select(ptr(affinities, f32p), ptr(bias, f32p), len(affinities), picks, reference_order, scale,
                          ptr(experts, u32p), ptr(weights, f32p))
    return experts, weights


def test_known_affinities_within_four_places():
    for score, text in KAT["router_affinities"]:
        got = np.float32(orc.orc_router_affinity(score, 0))
        want = float(Decimal(text))
        if np.exp(np.float64(score)) < 1.1754944e-38:
            # e^score is subnormal in float32 and keeps fewer bits: the square within 2^-146 of softplus
            assert abs(float(got) ** 2 - want ** 2) <= 2.0 ** -146
        else:
            assert abs(float(got) - want) <= 4 * float(np.spacing(np.float32(want)))


def test_affinity_sweep_against_double():
    scores = np.concatenate([np.linspace(-80, 25, 40001), normals(2, 20000) * 3]).astype(np.float32)
    got = np.array([orc.orc_router_affinity(float(s), 0) for s in scores], dtype=np.float32)
    s64 = scores.astype(np.float64)
    want = np.sqrt(np.where(s64 > 20, s64, np.maximum(s64, 0) + np.log1p(np.exp(-np.abs(s64)))))
    ulp = np.spacing(want.astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(got - want) / ulp) <= 2.0
    sig = np.array([orc.orc_router_affinity(float(s), 1) for s in scores], dtype=np.float32)
    want = 1 / (1 + np.exp(-s64))
    assert np.max(np.abs(sig - want) / np.spacing(want.astype(np.float32))) <= 3.0  # exp, add, divide: three roundings
    ys = np.linspace(0, 1, 20001).astype(np.float32)
    got = np.array([orc.orc_log1pf(float(y)) for y in ys], dtype=np.float32)
    want = np.log1p(ys.astype(np.float64))
    assert np.max(np.abs(got - want) / np.maximum(np.spacing(want.astype(np.float32)), 1e-45)) <= 1.5


def test_known_rows_both_orders():
    for row in KAT["router_rows"]:
        affinities = np.full(384, row["affinity"], dtype=np.float32)
        bias = np.full(384, row["bias"], dtype=np.float32)
        for expert, a, b in row["named"]:
            affinities[expert], bias[expert] = a, b
        if row["nan_bias_expert"] is not None:
            bias[row["nan_bias_expert"]] = np.nan
        for order in (0, 1):
            experts, weights = select(affinities, bias, 6, order)
            assert experts.tolist() == row["experts"]
            assert [hex(b) for b in weights.view(np.uint32)] == [hex(int(b, 16)) for b in row["weight_bits"]]


def test_the_two_orders_of_the_sum():
    row = KAT["router_order_row"]
    affinities = np.zeros(384, dtype=np.float32)
    tiny = np.array([int(row["tiny_affinity_bits"], 16)], dtype=np.uint32).view(np.float32)[0]
    affinities[row["tiny_experts"]] = tiny
    affinities[row["big_expert"]] = 1.0
    bias = np.zeros(384, dtype=np.float32)
    for order, key in ((0, "fixed"), (1, "reference")):
        experts, weights = select(affinities, bias, 6, order)
        assert experts.tolist() == row["experts"]
        bits = weights.view(np.uint32)
        assert all(hex(b) == hex(int(row[key]["small"], 16)) for b in bits[:5])
        assert hex(bits[5]) == hex(int(row[key]["big"], 16))


def test_known_job_table():
    case = KAT["router_jobs"]
    experts = np.array(case["experts"], dtype=np.uint32)
    weights = np.array(case["weights"], dtype=np.float32)
    offsets = (4096 + 16 * np.arange(384 * 3)).astype(np.uint64)
    jobs = np.zeros(case["launch_rows"] * 6, dtype=JOB_DTYPE)
    jobs["expert"] = 0xDEAD  # every byte is written
    orc.orc_router_jobs(ptr(experts, u32p), ptr(weights, f32p), 6, 3, case["launch_rows"], 384, ptr(offsets, u64p),
                        jobs.ctypes.data)
    for job, (expert, rows, pairs, ws) in zip(jobs, case["jobs"]):
        assert job["expert"] == expert and job["row_count"] == rows
        assert job["pair_index"][:rows].tolist() == pairs and job["route_weight"][:rows].tolist() == ws
        assert job["gate_offset"] == 4096 + 16 * 3 * expert and job["down_offset"] == 4096 + 16 * (3 * expert + 2)
        assert not job["pair_index"][rows:].any() and not job["route_weight"][rows:].any()
    assert not jobs[len(case["jobs"]):].view(np.uint8).any()


def brute_force_top(affinities, bias, picks):
    biased = (affinities + bias).astype(np.float32)
    order = sorted(range(len(biased)), key=lambda e: (-biased[e], e))
    return sorted(order[:picks])


@pytest.mark.parametrize("experts_n,picks", [(256, 8), (384, 6), (128, 3), (64, 1)])
def test_select_against_brute_force(experts_n, picks):
    for seed in range(5):
        affinities = np.abs(normals(30 + seed, experts_n)).astype(np.float32)
        affinities[::7] = affinities[3]  # ties
        bias = (normals(60 + seed, experts_n) * 0.1).astype(np.float32)
        experts, weights = select(affinities, bias, picks, 0, 2.5)
        assert experts.tolist() == brute_force_top(affinities, bias, picks)
        total = np.float32(0)
        for e in experts:
            total = np.float32(total + affinities[e])
        want = (affinities[experts] / np.float32(total + np.float32(1e-20)) * np.float32(2.5)).astype(np.float32)
        assert np.array_equal(weights, want)


def test_projection_order_and_value():
    rows, hidden, experts_n = 3, 512, 16
    x = to_bf16(normals(1, rows * hidden)).reshape(rows, hidden)
    w = to_bf16(normals(2, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    scores = np.zeros((rows, experts_n), dtype=np.float32)
    orc.orc_router_projection(ptr(x, u16p), ptr(w, u16p), rows, hidden, experts_n, ptr(scores, f32p))
    exact = bf16_to_f32(x).astype(np.float64) @ bf16_to_f32(w).astype(np.float64).T
    assert np.max(np.abs(scores - exact)) < 1e-5
    # the order: chain c owns k = c mod 32 (fma), then halving folds
    xf, wf = bf16_to_f32(x), bf16_to_f32(w)
    chains = np.zeros(32, dtype=np.float64)
    for c in range(32):
        s = np.float32(0)
        for k in range(c, hidden, 32):
            s = np.float32(np.float64(wf[5, k]) * np.float64(xf[1, k]) + np.float64(s))  # product exact in double
        chains[c] = s
    chains = chains.astype(np.float32)
    d = 16
    while d:
        chains[:d] = chains[:d] + chains[d:2 * d]
        d //= 2
    assert scores[1, 5] == chains[0]


def random_choices(seed, rows, picks, experts_n):
    experts = np.zeros((rows, picks), dtype=np.uint32)
    draws = splitmix_words(seed, rows * experts_n).reshape(rows, experts_n)
    for r in range(rows):
        experts[r] = np.sort(np.argsort(draws[r] % np.uint64(1 + experts_n // 3))[:picks])  # skewed, distinct
    weights = np.abs(normals(seed + 1, rows * picks)).astype(np.float32).reshape(rows, picks)
    return experts, weights


@pytest.mark.parametrize("rows,live,picks,experts_n", [(130, 130, 6, 384), (40, 33, 8, 256), (1, 1, 8, 256), (9, 0, 8, 256)])
def test_wide_sort_invariants(rows, live, picks, experts_n):
    experts, weights = random_choices(5, rows, picks, experts_n)
    if rows == 130:
        experts[:] = np.array([3, 9, 77, 200, 201, 383], dtype=np.uint32)  # 130 rows x the same 6 experts
    offsets = (1 << 20) + 64 * np.arange(experts_n * 3, dtype=np.uint64)
    tiles_n = orc.orc_router_wide_tile_count(rows, picks, experts_n)
    jobs_n = orc.orc_router_wide_job_count(rows, picks, experts_n)
    pairs = np.zeros(max(live * picks, 1), dtype=PAIR_DTYPE)
    runs = np.zeros(experts_n, dtype=RUN_DTYPE)
    tiles = np.zeros(tiles_n, dtype=TILE_DTYPE)
    jobs = np.zeros(jobs_n, dtype=JOB_DTYPE)
    orc.orc_router_wide_sort(ptr(experts, u32p), ptr(weights, f32p), picks, live, rows, experts_n, ptr(offsets, u64p),
                             pairs.ctypes.data, runs.ctypes.data, tiles.ctypes.data)
    orc.orc_router_wide_jobs(ptr(experts, u32p), ptr(weights, f32p), picks, live, rows, experts_n, ptr(offsets, u64p),
                             jobs.ctypes.data)
    flat = experts.reshape(-1)
    assert runs["pair_count"].sum() == live * picks
    placed = pairs["pair_index"][:live * picks]
    assert sorted(placed.tolist()) == list(range(live * picks))
    keys = [(int(flat[p]), int(p)) for p in placed]
    assert keys == sorted(keys)  # stable: by expert, then row, then slot
    for e in range(experts_n):
        first, count = runs[e]["first_pair"], runs[e]["pair_count"]
        assert all(flat[p] == e for p in placed[first:first + count])
    used = tiles[tiles["pair_count"] > 0]
    assert used["pair_count"].sum() == live * picks and np.all(used["pair_count"] <= 64)
    assert not tiles[len(used):].view(np.uint8).any()
    if rows == 130:
        assert used["pair_count"].tolist() == [64, 64, 2] * 6
        assert jobs["row_count"][jobs["row_count"] > 0].tolist() == ([8] * 16 + [2]) * 6
    used_jobs = jobs[jobs["row_count"] > 0]
    assert used_jobs["row_count"].sum() == live * picks
    seen = []
    for job in used_jobs:
        assert job["gate_offset"] == offsets[3 * job["expert"]]
        seen += job["pair_index"][:job["row_count"]].tolist()
        assert np.array_equal(job["route_weight"][:job["row_count"]], weights.reshape(-1)[job["pair_index"][:job["row_count"]]])
    assert seen == placed.tolist()


@needs_ref
def test_ref_affinity_select_jobs_and_sort():
    for score in np.concatenate([np.linspace(-30, 25, 500), normals(3, 500) * 4]).astype(np.float32):
        assert ref.test_router_affinity_holds(float(score), float(orc.orc_router_affinity(float(score), 0)))
    rows = 7
    chosen = np.zeros((rows, 6), dtype=np.uint32)
    chosen_w = np.zeros((rows, 6), dtype=np.float32)
    for r in range(rows):
        affinities = np.abs(normals(100 + r, 384)).astype(np.float32)
        affinities[::5] = affinities[1]
        bias = (normals(200 + r, 384) * 0.2).astype(np.float32)
        for order in (0, 1):
            experts, weights = select(affinities, bias, 6, order)
            theirs_e, theirs_w = np.zeros(6, dtype=np.uint32), np.zeros(6, dtype=np.float32)
            ref.test_router_select(ptr(affinities, f32p), ptr(bias, f32p), bool(order), ptr(theirs_e, u32p), ptr(theirs_w, f32p))
            assert np.array_equal(experts, theirs_e) and np.array_equal(weights.view(np.uint32), theirs_w.view(np.uint32))
        chosen[r], chosen_w[r] = experts, weights
    offsets = (4096 + 16 * np.arange(384 * 3)).astype(np.uint64)
    ours, theirs = np.zeros(8 * 6, dtype=JOB_DTYPE), np.ones(8 * 6, dtype=JOB_DTYPE)
    orc.orc_router_jobs(ptr(chosen, u32p), ptr(chosen_w, f32p), 6, rows, 8, 384, ptr(offsets, u64p), ours.ctypes.data)
    ref.test_router_jobs(ptr(chosen, u32p), ptr(chosen_w, f32p), rows, 8, ptr(offsets, u64p), theirs.ctypes.data)
    assert ours.tobytes() == theirs.tobytes()
    # wide: 300 rows
    experts, weights = random_choices(9, 300, 6, 384)
    tiles_n, jobs_n = orc.orc_router_wide_tile_count(300, 6, 384), orc.orc_router_wide_job_count(300, 6, 384)
    assert tiles_n == (300 * 6 + 63) // 64 + 384 and jobs_n == min(1800, (1800 + 7 * 384) // 8)
    out = []
    for fn_sort, fn_jobs, extra in ((orc.orc_router_wide_sort, orc.orc_router_wide_jobs, (6,)), (ref.test_router_wide_sort, ref.test_router_wide_jobs, ())):
        pairs, runs = np.zeros(1800, dtype=PAIR_DTYPE), np.zeros(384, dtype=RUN_DTYPE)
        tiles, jobs = np.zeros(tiles_n, dtype=TILE_DTYPE), np.zeros(jobs_n, dtype=JOB_DTYPE)
        mid = (384,) if extra else ()
        fn_sort(ptr(experts, u32p), ptr(weights, f32p), *extra, 290, 300, *mid, ptr(offsets, u64p), pairs.ctypes.data, runs.ctypes.data, tiles.ctypes.data)
        fn_jobs(ptr(experts, u32p), ptr(weights, f32p), *extra, 290, 300, *mid, ptr(offsets, u64p), jobs.ctypes.data)
        out.append((pairs[:290 * 6].tobytes(), runs.tobytes(), tiles.tobytes(), jobs.tobytes()))
    assert out[0] == out[1]


def test_route_of_a_step_equals_the_calls_row_by_row():
    """orc_router_route (projection, affinities and the select of every row in one call) against the functions it is made of."""
    rng = np.random.default_rng(5)
    rows, hidden, experts, picks = 5, 256, 64, 4
    x = (rng.standard_normal((rows, hidden)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    w = ((rng.standard_normal((experts, hidden)) * 0.02).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    bias = (rng.standard_normal(experts) * 0.01).astype(np.float32)
    for kind in (0, 1):
        got_experts, got_weights = np.zeros((rows, picks), np.uint32), np.zeros((rows, picks), np.float32)
        got_affinities = np.zeros((rows, experts), np.float32)
        orc.orc_router_route(ptr(x, u16p), ptr(w, u16p), ptr(bias, f32p), rows, hidden, experts, picks, kind, 0, 1.5,
                               ptr(got_affinities, f32p), ptr(got_experts, u32p), ptr(got_weights, f32p))
        scores = np.zeros((rows, experts), np.float32)
        orc.orc_router_projection(ptr(x, u16p), ptr(w, u16p), rows, hidden, experts, ptr(scores, f32p))
        affinities = np.array([[orc.orc_router_affinity(float(s), kind) for s in row] for row in scores], np.float32)
        want_experts, want_weights = np.zeros((rows, picks), np.uint32), np.zeros((rows, picks), np.float32)
        for r in range(rows):
            orc.orc_router_select(ptr(affinities[r], f32p), ptr(bias, f32p), experts, picks, 0, 1.5,
                                    ptr(want_experts[r], u32p), ptr(want_weights[r], f32p))
        assert got_affinities.tobytes() == affinities.tobytes()
        assert np.array_equal(got_experts, want_experts) and got_weights.tobytes() == want_weights.tobytes()
