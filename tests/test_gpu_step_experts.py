"""A layer that keeps some of its routed experts in host memory, on the card: the select names them by tags, the expert
pause (expert_pause_run through the C ABI, over the HIP backend's copies) puts them into the card's slots and points the
jobs there, and the fused EXL3 decode then gives the bits of the same layer with every expert on the card. Over several
steps: an expert a slot holds does not go up again; the slots are taken in turn. Every pause is replayed by the oracle's
walk (oracle/orc_pause.py) from the job table the card's select wrote: the same jobs rewritten, the same experts in the
same slots, and the slots' bytes on the card are those experts'; the first step's output is also held against the
oracle's EXL3 layer."""
import ctypes as C
import os
import sys
import time

import numpy as np
import pytest

import _oracle as o
from _oracle import exl3_matrix, normals, splitmix_words, to_bf16

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import orc_pause  # noqa: E402

pytestmark = pytest.mark.gpu


def say(*words):
    print(*words, flush=True)
    sys.stdout.flush()


def test_host_experts_give_the_resident_layers_bits():
    import anemone_amd as amd
    hidden, inner, experts_n, picks, rows, seed = 512, 256, 64, 4, 4, 9
    choices = [2, 3, 4, 40]
    draws = splitmix_words(seed, experts_n * 3) % np.uint64(len(choices))
    widths = np.array(choices, dtype=np.uint32)[draws.astype(np.int64)].reshape(experts_n, 3)
    matrices = [[exl3_matrix(seed * 1000 + 3 * e + 0, hidden, inner, int(widths[e, 0])), exl3_matrix(seed * 1000 + 3 * e + 1, hidden, inner, int(widths[e, 1])),
                 exl3_matrix(seed * 1000 + 3 * e + 2, inner, hidden, int(widths[e, 2]))] for e in range(experts_n)]
    router = to_bf16(normals(seed + 5, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    host_experts = [e for e in range(experts_n) if e % 3 != 1]  # two thirds of the experts in host memory
    steps = [to_bf16(normals(100 + s, rows * hidden)).reshape(rows, hidden) for s in range(3)]
    steps.append(steps[2])  # the same rows again: nothing goes up
    want, want_jobs = [], []
    say("host experts: the resident layer")
    card = amd.Card(1 << 30)
    try:
        resident = amd.Exl3Layer(card, hidden, inner, experts_n, picks, rows, matrices, widths, router_weights_bf16=router)
        for x in steps:
            resident.set_rows(x, rows)
            card.run(resident.projection_launch())
            card.run(resident.select_launch(0))
            card.run(resident.tc_launches())
            want.append(resident.output().copy())
            want_jobs.append(resident.jobs().copy())
    finally:
        card.close()
    say("host experts: the layer with", len(host_experts), "of", experts_n, "experts in host memory")
    card = amd.Card(1 << 30)
    try:
        layer = amd.Exl3Layer(card, hidden, inner, experts_n, picks, rows, matrices, widths, router_weights_bf16=router, host_experts=host_experts)
        held = set()
        model = orc_pause.Slots(layer.pairs)
        for number, x in enumerate(steps):
            layer.set_rows(x, rows)
            card.run(layer.projection_launch())
            card.run(layer.select_launch(0))
            tagged = layer.jobs()
            live = tagged[tagged["row_count"] > 0]
            assert np.array_equal(live["expert"], want_jobs[number][want_jobs[number]["row_count"] > 0]["expert"])
            named = [int(e) for e in live["expert"] if int(e) in host_experts]
            for job in live:
                if int(job["expert"]) in host_experts:  # a tag: the three offsets equal
                    assert job["gate_offset"] == job["up_offset"] == job["down_offset"] == layer.pause.slots_offset + 16 * host_experts.index(int(job["expert"]))
            replayed = [{"gate": int(j["gate_offset"]), "up": int(j["up_offset"]), "down": int(j["down_offset"]), "rows": int(j["row_count"])} for j in tagged]
            status, want_uploads, _ = orc_pause.pause(replayed, model, int(layer.pause.slots_offset), int(layer.pause.slot_byte_count),
                                                      [int(v) for v in layer.pause.matrix_offsets], 0, len(host_experts))
            assert status == 0
            began = time.perf_counter()
            uploaded = layer.run_pause()
            took = time.perf_counter() - began
            pointed = layer.jobs()
            # the oracle's walk over the same table: the same offsets in every job, the same expert in every slot
            assert [(int(j["gate_offset"]), int(j["up_offset"]), int(j["down_offset"])) for j in pointed] == [(j["gate"], j["up"], j["down"]) for j in replayed]
            assert uploaded == len(want_uploads)
            assert [int(v) - 1 if v else None for v in layer.slot_fields[0::2]] == model.held and int(layer.slots.next_slot) == model.next_slot
            for slot, host_index in want_uploads:  # what went up is that expert, whole
                expert = host_experts[host_index]
                at = int(layer.pause.slots_offset) + slot * int(layer.pause.slot_byte_count)
                for m in range(3):
                    stored = matrices[expert][m].view(np.uint8).reshape(-1)
                    assert np.array_equal(card.download(at + int(layer.pause.matrix_offsets[m]), stored.size), stored), (slot, expert, m)
            slot_of = {}
            for job in pointed[pointed["row_count"] > 0]:
                if int(job["expert"]) in host_experts:
                    slot = (int(job["gate_offset"]) - int(layer.pause.slots_offset)) // int(layer.pause.slot_byte_count)
                    assert 0 <= slot < layer.pairs and slot not in slot_of.values()
                    slot_of[int(job["expert"])] = slot
                    assert int(job["up_offset"]) == int(job["gate_offset"]) + int(layer.pause.matrix_offsets[1])
                    assert int(job["down_offset"]) == int(job["gate_offset"]) + int(layer.pause.matrix_offsets[2])
            holding = {int(v) - 1 for v in layer.slot_fields[0::2] if v}
            fresh = [e for e in named if host_experts.index(e) not in held]
            say("  step %d: %d jobs of host experts, %d uploaded (%d bytes each) in %.0f us" % (number, len(named), uploaded, int(layer.pause.expert_byte_count),
                                                                                                    1e6 * took))
            assert uploaded == len(fresh) and set(host_experts.index(e) for e in named) <= holding
            held = holding
            card.run(layer.tc_launches())
            got = layer.output()
            assert got.tobytes() == want[number].tobytes(), "the layer's output with host experts differs from the resident layer's"
        assert uploaded == 0, "the last step's experts were all held"
        layer.release_host_experts()
    finally:
        card.close()
    # the first step against the oracle's layer (the resident layer's bits are the host-expert layer's, checked above)
    live = want_jobs[0][want_jobs[0]["row_count"] > 0]
    experts_of, weights_of = np.zeros((rows, picks), np.uint32), np.zeros((rows, picks), np.float32)
    for job in live:
        for c in range(job["row_count"]):
            experts_of.reshape(-1)[job["pair_index"][c]] = job["expert"]
            weights_of.reshape(-1)[job["pair_index"][c]] = job["route_weight"][c]
    pointers = (C.c_void_p * (experts_n * 3))(*[m.ctypes.data for trio in matrices for m in trio])
    oracle_out = np.zeros((rows, hidden), dtype=np.float32)
    o.orc.orc_exl3_moe_layer(o.ptr(steps[0], o.u16p), rows, hidden, inner, picks, o.ptr(experts_of, o.u32p), o.ptr(weights_of, o.f32p), experts_n,
                             pointers, o.ptr(np.ascontiguousarray(widths.astype(np.uint8)), o.u8p), 10.0, o.ptr(oracle_out, o.f32p), None, None, 4)
    error = float(np.max(np.abs(want[0] - oracle_out)) / np.sqrt(np.mean(oracle_out.astype(np.float64) ** 2)))
    say("  the first step against the oracle's layer: max error %.2e of rms" % error)
    assert error <= 4e-3


def test_a_pause_at_the_full_shapes_expert_size():
    """What a pause costs at the benchmark's shape (hidden 4096, intermediate 2048, 3 bits a weight: 9.4 MB an expert):
    eight rows' 64 jobs, all of host experts, then the same again (held)."""
    import anemone_amd as amd
    hidden, inner, experts_n, picks, rows = 4096, 2048, 64, 8, 8
    widths = np.full((experts_n, 3), 3, dtype=np.uint32)
    distinct = [[exl3_matrix(7000 + 3 * e + 0, hidden, inner, 3), exl3_matrix(7000 + 3 * e + 1, hidden, inner, 3), exl3_matrix(7000 + 3 * e + 2, inner, hidden, 3)]
                for e in range(4)]
    matrices = [distinct[e % 4] for e in range(experts_n)]
    router = to_bf16(normals(3, experts_n * hidden) * 0.02).reshape(experts_n, hidden)
    card = amd.Card(3 << 30)
    try:
        layer = amd.Exl3Layer(card, hidden, inner, experts_n, picks, rows, matrices, widths, router_weights_bf16=router, host_experts=list(range(experts_n)))
        layer.set_rows(to_bf16(normals(4, rows * hidden)).reshape(rows, hidden), rows)
        for attempt in range(2):
            card.run(layer.projection_launch())
            card.run(layer.select_launch(0))
            began = time.perf_counter()
            uploaded = layer.run_pause()
            took = time.perf_counter() - began
            size = int(layer.pause.expert_byte_count)
            say("  full-size pause %d: %d experts of %.1f MB uploaded in %.2f ms%s" % (attempt, uploaded, size / 1e6, 1e3 * took,
                                                                                     " = %.1f GB/s" % (uploaded * size / took / 1e9) if uploaded else ""))
            card.run(layer.tc_launches())
            assert np.all(np.isfinite(layer.output())) and float(np.abs(layer.output()).max()) > 0.0
            assert (uploaded == 0) == (attempt == 1)
    finally:
        card.close()
