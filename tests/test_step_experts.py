"""A step's expert pauses (expert_pause_plan, expert_pause_run: anemone_amd/host/step_experts.c) on the CPU: the walk over
a job table against the oracle (oracle/orc_pause.py, which tests/test_oracle_pause.py pins to the reference's own
scenario) on that scenario and on random steps, its refusals, and the whole pause over a stand-in for the backend's
copies (an arena in host memory): which bytes go where, in which order, and that a held expert does not go up again."""
import ctypes as C
import os
import sys

import numpy as np
import pytest

import anemone_amd as amd

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import orc_pause as orc  # noqa: E402
from test_oracle_pause import (CARD_EXPERTS_OFFSET, EXPERT_BYTES, FIRST_HOST_EXPERTS, HOST, LAYERS, MATRIX_OFFSETS, SLOT_BYTES, SLOTS,  # noqa: E402
                               SLOTS_OFFSET, jobs_of)

JOB = amd.JOB_DTYPE


def pause_record(layer, jobs_per_row=3, slot_count=SLOTS, **changes):
    first, count = LAYERS[layer]
    p = amd.ExpertPause()
    p.jobs_offset, p.slots_offset, p.slot_byte_count, p.expert_byte_count = 1024 * (layer + 1), SLOTS_OFFSET, SLOT_BYTES, EXPERT_BYTES
    for i, offset in enumerate(MATRIX_OFFSETS):
        p.matrix_offsets[i] = offset
    p.first_host_expert, p.host_expert_count, p.jobs_per_row, p.slot_count = first, count, jobs_per_row, slot_count
    for key, value in changes.items():
        setattr(p, key, value)
    return p


class CardSlots:
    def __init__(self, count):
        self.fields = np.zeros(2 * count, dtype=np.uint64)
        self.state = amd.ExpertSlots(self.fields.ctypes.data_as(C.POINTER(C.c_uint64)), 0, count, 0)

    def held(self):
        return [int(v) - 1 if v else None for v in self.fields[0::2]]


def table_of(jobs):
    table = np.zeros(len(jobs), dtype=JOB)
    for j, job in enumerate(jobs):
        table[j]["gate_offset"], table[j]["up_offset"], table[j]["down_offset"], table[j]["row_count"] = job["gate"], job["up"], job["down"], job["rows"]
        table[j]["expert"] = 7 + j
    return table


def plan(pause, slots, table):
    uploads = (amd.ExpertPauseUpload * max(1, len(table)))()
    n, tags = C.c_uint32(99), C.c_uint32(99)
    status = amd.library().expert_pause_plan(C.byref(pause), table.ctypes.data, len(table), C.byref(slots.state), uploads, C.byref(n), C.byref(tags))
    return status, [(uploads[i].slot, uploads[i].host_expert) for i in range(n.value)] if status == 0 else [], tags.value


def check_step(slots, model, layer, experts):
    """one pause by the library and by the oracle: the same uploads in the same order, the same job table, the same slots"""
    jobs = jobs_of(layer, experts)
    table = table_of(jobs)
    status, uploads, tags = plan(pause_record(layer), slots, table)
    want_status, want_uploads, want_tags = orc.pause(jobs, model, SLOTS_OFFSET, SLOT_BYTES, MATRIX_OFFSETS, *LAYERS[layer])
    assert status == want_status == 0 and uploads == want_uploads and tags == want_tags
    assert [(int(t["gate_offset"]), int(t["up_offset"]), int(t["down_offset"])) for t in table] == [(j["gate"], j["up"], j["down"]) for j in jobs]
    assert slots.held() == model.held and int(slots.state.next_slot) == model.next_slot
    assert [int(t["expert"]) for t in table] == [7 + j for j in range(len(table))], "nothing else of a job moves"
    return uploads


def test_plan_on_the_reference_scenario():
    slots, model = CardSlots(SLOTS), orc.Slots(SLOTS)
    assert check_step(slots, model, 0, [HOST + 2, 1, HOST + 5]) == [(0, 2), (1, 5)]
    assert check_step(slots, model, 1, [HOST + FIRST_HOST_EXPERTS + 1]) == [(2, 1)]
    assert check_step(slots, model, 0, [HOST + 5, HOST + 2]) == []
    assert check_step(slots, model, 1, [HOST + FIRST_HOST_EXPERTS + 1]) == []
    assert [s for s, _ in check_step(slots, model, 0, [HOST, HOST + 1, HOST + 3, HOST + 4, HOST + 2, HOST + 6])] == [3, 4, 5, 1, 2]
    assert check_step(slots, model, 1, [0, 3]) == []
    assert check_step(slots, model, 0, [0, 3]) == []
    assert check_step(slots, model, 1, [HOST + FIRST_HOST_EXPERTS + 1]) == [(3, 1)]


def test_plan_on_random_steps():
    rng = np.random.default_rng(5)
    slots, model = CardSlots(SLOTS), orc.Slots(SLOTS)
    for step in range(300):
        layer = int(rng.integers(0, 2))
        first, count = LAYERS[layer]
        pool = list(range(4)) + [HOST + first + i for i in range(count)]
        experts = [int(e) for e in rng.choice(pool, size=int(rng.integers(1, SLOTS + 1)), replace=False)]
        check_step(slots, model, layer, experts)


def test_plan_refusals():
    good, on_card = SLOTS_OFFSET + 3 * 16, CARD_EXPERTS_OFFSET
    for broken in ((good + 8,) * 3, (SLOTS_OFFSET + 8 * 16,) * 3, (good, good + 16, good), (good, on_card, good), (on_card, good, good)):
        table = table_of([dict(zip(("gate", "up", "down"), broken), rows=1)])
        before = table.tobytes()
        assert plan(pause_record(0), CardSlots(SLOTS), table)[0] == amd.STATUS_DEVICE_ERROR, broken
        assert table.tobytes() == before
    table = table_of(jobs_of(0, [HOST + 1]))
    assert plan(pause_record(0, slot_count=5), CardSlots(SLOTS), table)[0] == amd.STATUS_INVALID_ARGUMENT  # the card's slots are the pause's
    assert plan(pause_record(0, expert_byte_count=SLOT_BYTES + 1), CardSlots(SLOTS), table)[0] == amd.STATUS_INVALID_ARGUMENT
    seven = table_of(jobs_of(0, [HOST + i for i in range(7)]))
    assert plan(pause_record(0), CardSlots(SLOTS), seven)[0] == amd.STATUS_INVALID_ARGUMENT  # more jobs than slots
    uploads, n = (amd.ExpertPauseUpload * 1)(), C.c_uint32(0)
    assert amd.library().expert_pause_plan(None, table.ctypes.data, 1, C.byref(CardSlots(SLOTS).state), uploads, C.byref(n), C.byref(n)) == 1


# ---- the whole pause over copies into an arena in host memory ----

BEGIN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint64, C.POINTER(C.c_uint64))
WAIT = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_uint64, C.c_uint64)


class CopyBackend:
    """upload_begin, upload_wait and download_begin of struct backend_operations over a numpy arena; a download's bytes
    reach its destination only when its ticket is waited for (the seam allows a backend that)."""

    def __init__(self, arena_bytes):
        self.arena = np.zeros(arena_bytes, dtype=np.uint8)
        self.log, self.held, self.ticket = [], {}, 0
        self.fail_upload_number = 0  # the n-th upload from now answers STATUS_DEVICE_ERROR (0: none does)
        self.callbacks = (BEGIN(self.upload), WAIT(self.wait), BEGIN(self.download))
        self.operations = (C.c_void_p * 28)()
        self.operations[7] = C.cast(self.callbacks[0], C.c_void_p)
        self.operations[8] = C.cast(self.callbacks[1], C.c_void_p)
        self.operations[10] = C.cast(self.callbacks[2], C.c_void_p)
        self.card = C.c_void_p(0x2000)

    def upload(self, card, offset, source, count, ticket_out):
        if self.fail_upload_number:
            self.fail_upload_number -= 1
            if self.fail_upload_number == 0:
                self.log.append(("refused", offset, count))
                return amd.STATUS_DEVICE_ERROR
        self.arena[offset:offset + count] = np.ctypeslib.as_array((C.c_ubyte * count).from_address(source))
        self.ticket += 1
        self.log.append(("up", offset, count))
        ticket_out[0] = self.ticket
        return 0

    def download(self, card, offset, destination, count, ticket_out):
        self.ticket += 1
        self.held[self.ticket] = (destination, self.arena[offset:offset + count].copy())
        C.memset(destination, 0xA5, count)
        self.log.append(("down", offset, count))
        ticket_out[0] = self.ticket
        return 0

    def wait(self, card, ticket, limit):
        if ticket in self.held:
            destination, data = self.held.pop(ticket)
            C.memmove(destination, data.ctypes.data, data.size)
        return 0 if 0 < ticket <= self.ticket else 1


def test_run_moves_the_experts_and_the_table():
    backend = CopyBackend(32768)
    copies = np.zeros((FIRST_HOST_EXPERTS, EXPERT_BYTES), dtype=np.uint8)
    for e in range(FIRST_HOST_EXPERTS):
        copies[e] = (np.arange(EXPERT_BYTES) * 3 + 37 * e) % 251
    slots = CardSlots(SLOTS)
    pause = pause_record(0)
    staging = np.zeros(SLOTS, dtype=JOB)

    def step(experts, rows):
        jobs = jobs_of(0, experts) + [{"gate": 0, "up": 0, "down": 0, "rows": 0}] * (3 * rows - len(experts))
        backend.arena[pause.jobs_offset:pause.jobs_offset + 96 * len(jobs)] = table_of(jobs).view(np.uint8)
        backend.log.clear()
        uploaded = C.c_uint32(77)
        status = amd.library().expert_pause_run(C.addressof(backend.operations), backend.card, C.byref(pause), rows, C.byref(slots.state),
                                                staging.ctypes.data, copies.ctypes.data, 10 ** 9, C.byref(uploaded))
        assert status == 0
        return backend.arena[pause.jobs_offset:pause.jobs_offset + 96 * len(jobs)].view(JOB), uploaded.value

    table, uploaded = step([HOST + 2, 1, HOST + 5], 1)
    assert uploaded == 2 and backend.log == [("down", 1024, 288), ("up", SLOTS_OFFSET, EXPERT_BYTES), ("up", SLOTS_OFFSET + SLOT_BYTES, EXPERT_BYTES),
                                             ("up", 1024, 288)]
    assert np.array_equal(backend.arena[SLOTS_OFFSET:SLOTS_OFFSET + EXPERT_BYTES], copies[2])
    assert np.array_equal(backend.arena[SLOTS_OFFSET + SLOT_BYTES:SLOTS_OFFSET + SLOT_BYTES + EXPERT_BYTES], copies[5])
    assert (int(table[0]["gate_offset"]), int(table[0]["up_offset"]), int(table[0]["down_offset"])) == (SLOTS_OFFSET, SLOTS_OFFSET + 128, SLOTS_OFFSET + 64)
    assert int(table[1]["gate_offset"]) == CARD_EXPERTS_OFFSET + EXPERT_BYTES and int(table[2]["gate_offset"]) == SLOTS_OFFSET + SLOT_BYTES
    # held experts: nothing goes up but the job table, which held tags
    table, uploaded = step([HOST + 5, HOST + 2], 1)
    assert uploaded == 0 and backend.log == [("down", 1024, 288), ("up", 1024, 288)]
    # card experts alone: the table stays where it is
    table, uploaded = step([0, 3], 1)
    assert uploaded == 0 and backend.log == [("down", 1024, 288)]
    # two rows, six host experts
    table, uploaded = step([HOST, HOST + 1, HOST + 3, HOST + 4, HOST + 2, HOST + 6], 2)
    assert uploaded == 5 and [entry[1] for entry in backend.log[1:6]] == [SLOTS_OFFSET + s * SLOT_BYTES for s in (2, 3, 4, 5, 1)]
    for job, expert in zip(table, (0, 1, 3, 4, 2, 6)):
        at = int(job["gate_offset"])
        assert np.array_equal(backend.arena[at:at + EXPERT_BYTES], copies[expert])
    # a broken tag fails the pause before any upload
    backend.arena[pause.jobs_offset:pause.jobs_offset + 96] = table_of([{"gate": SLOTS_OFFSET + 8, "up": SLOTS_OFFSET + 8, "down": SLOTS_OFFSET + 8, "rows": 1}]).view(np.uint8)
    backend.log.clear()
    assert amd.library().expert_pause_run(C.addressof(backend.operations), backend.card, C.byref(pause), 1, C.byref(slots.state), staging.ctypes.data,
                                          copies.ctypes.data, 10 ** 9, None) == amd.STATUS_DEVICE_ERROR
    assert backend.log == [("down", 1024, 288)]
    assert amd.library().expert_pause_run(C.addressof(backend.operations), backend.card, C.byref(pause), 3, C.byref(slots.state), staging.ctypes.data,
                                          copies.ctypes.data, 10 ** 9, None) == amd.STATUS_INVALID_ARGUMENT  # nine jobs for six slots


def test_a_failed_copy_leaves_none_of_the_pause_slots_held():
    """The walk names the slots before any copy begins: when a copy fails, no slot this pause meant to fill may pass for
    holding its expert, or a later pause would run the experts on bytes that never came."""
    backend = CopyBackend(32768)
    copies = np.zeros((FIRST_HOST_EXPERTS, EXPERT_BYTES), dtype=np.uint8)
    for e in range(FIRST_HOST_EXPERTS):
        copies[e] = (np.arange(EXPERT_BYTES) * 5 + 11 * e) % 253
    slots, pause, staging = CardSlots(SLOTS), pause_record(0), np.zeros(SLOTS, dtype=JOB)

    def run(experts):
        jobs = jobs_of(0, experts)
        backend.arena[pause.jobs_offset:pause.jobs_offset + 96 * len(jobs)] = table_of(jobs).view(np.uint8)
        backend.log.clear()
        return amd.library().expert_pause_run(C.addressof(backend.operations), backend.card, C.byref(pause), 1, C.byref(slots.state),
                                              staging.ctypes.data, copies.ctypes.data, 10 ** 9, None)

    assert run([HOST + 4, 1, 2]) == 0 and slots.held() == [4, None, None, None, None, None]
    backend.fail_upload_number = 2
    assert run([HOST + 4, HOST + 1, HOST + 2]) == amd.STATUS_DEVICE_ERROR
    assert [entry[0] for entry in backend.log] == ["down", "up", "refused"], "the pause stops at the copy that fails"
    assert slots.held() == [4, None, None, None, None, None], "the held expert stays; neither of the two named slots holds one"
    # the next pause brings both up again, into the slots in turn
    assert run([HOST + 4, HOST + 1, HOST + 2]) == 0
    assert [entry[0] for entry in backend.log] == ["down", "up", "up", "up"]
    held = {expert: slot for slot, expert in enumerate(slots.held()) if expert is not None}
    assert set(held) == {4, 1, 2}
    for expert, slot in held.items():
        assert np.array_equal(backend.arena[SLOTS_OFFSET + slot * SLOT_BYTES:SLOTS_OFFSET + slot * SLOT_BYTES + EXPERT_BYTES], copies[expert])


def test_site_front_check_reads_and_clears_the_count_of_blocks_that_gave_up():
    """site_front_check over the stand-in backend: a clean scratch answers STATUS_OK and moves nothing up; a scratch whose
    gave_up counts blocks answers STATUS_DEVICE_ERROR, reports the count and leaves it zero on the card."""
    backend = CopyBackend(16384)
    scratch = amd.Range(1024, 7184)  # SITE_FRONT_SCRATCH_BYTES
    tail = 1024 + 16 + 8 * 24 * 4  # behind the four counters and the mixes of eight rows: departed, gave_up
    staging = np.zeros(2, dtype=np.uint32)
    count = C.c_uint32(99)
    lib = amd.library()
    assert lib.site_front_check(C.addressof(backend.operations), backend.card, scratch, staging.ctypes.data, 10 ** 9, C.byref(count)) == 0
    assert count.value == 0 and backend.log == [("down", tail, 8)]
    backend.arena[tail + 4:tail + 8] = np.array([3], dtype=np.uint32).view(np.uint8)
    backend.arena[tail - 4:tail] = 0x77
    backend.log.clear()
    assert lib.site_front_check(C.addressof(backend.operations), backend.card, scratch, staging.ctypes.data, 10 ** 9,
                                C.byref(count)) == amd.STATUS_DEVICE_ERROR
    assert count.value == 3 and backend.log == [("down", tail, 8), ("up", tail, 8)]
    assert not backend.arena[tail:tail + 8].any() and np.all(backend.arena[tail - 4:tail] == 0x77)
    assert lib.site_front_check(C.addressof(backend.operations), backend.card, scratch, staging.ctypes.data, 10 ** 9, None) == 0
    assert lib.site_front_check(C.addressof(backend.operations), backend.card, amd.Range(1024, 64), staging.ctypes.data, 10 ** 9,
                                None) == amd.STATUS_INVALID_ARGUMENT


# ---- the page-locked copies (expert_host_copies_attach) over a stand-in for the backend's staging memory ----

ALLOCATE = C.CFUNCTYPE(C.c_int, C.c_uint64, C.POINTER(C.c_void_p))
FREE = C.CFUNCTYPE(None, C.c_void_p)


class StagingBackend:
    def __init__(self):
        self.blocks, self.freed, self.fail_staging_allocation = {}, [], False
        self.callbacks = (ALLOCATE(self.allocate), FREE(self.free))
        self.operations = (C.c_void_p * 28)()
        self.operations[5] = C.cast(self.callbacks[0], C.c_void_p)
        self.operations[6] = C.cast(self.callbacks[1], C.c_void_p)

    def allocate(self, count, out):
        if self.fail_staging_allocation:
            return amd.STATUS_OUT_OF_MEMORY
        block = np.full(count, 0xCD, dtype=np.uint8)
        self.blocks[block.ctypes.data] = block
        out[0] = block.ctypes.data
        return 0

    def free(self, address):
        self.freed.append(address)


def test_host_copies_attach_copies_every_expert_once_and_refuses_whole():
    lib = amd.library()
    backend = StagingBackend()
    rng = np.random.default_rng(11)
    host_arena = rng.integers(0, 256, size=4096, dtype=np.uint8)
    offsets = np.array([0, 512, 100, 1800, 3000, 2400, 3600], dtype=np.uint64)  # in no order, as a loader may leave them
    pauses = (amd.ExpertPause * 2)()
    pauses[0].first_host_expert, pauses[0].host_expert_count, pauses[0].expert_byte_count = 0, 3, 200
    pauses[1].first_host_expert, pauses[1].host_expert_count, pauses[1].expert_byte_count = 3, 4, 96

    def attach(table_bytes=288, most=1 << 20, arena_bytes=host_arena.nbytes, count=len(offsets), pause_count=2):
        copies, starts = amd.ExpertHostCopies(), (C.c_uint64 * 2)(77, 77)
        status = lib.expert_host_copies_attach(C.addressof(backend.operations), pauses, pause_count, offsets.ctypes.data_as(C.POINTER(C.c_uint64)), count,
                                               host_arena.ctypes.data, arena_bytes, table_bytes, most, C.byref(copies), starts)
        return status, copies, list(starts)

    status, copies, starts = attach()
    assert status == 0 and starts == [0, 600] and copies.table_staging_offset == 1024 and copies.byte_count == 1024 + 288
    block = backend.blocks[C.cast(copies.block, C.c_void_p).value]
    for e in range(3):
        assert np.array_equal(block[200 * e:200 * e + 200], host_arena[int(offsets[e]):int(offsets[e]) + 200])
    for e in range(4):
        assert np.array_equal(block[600 + 96 * e:600 + 96 * e + 96], host_arena[int(offsets[3 + e]):int(offsets[3 + e]) + 96])
    assert np.all(block[984:] == 0xCD), "nothing is written behind the experts"
    lib.expert_host_copies_detach(C.addressof(backend.operations), C.byref(copies))
    assert backend.freed == [block.ctypes.data] and not copies.block and copies.byte_count == 0
    lib.expert_host_copies_detach(C.addressof(backend.operations), C.byref(copies))  # again: nothing to give back
    assert len(backend.freed) == 1
    # refusals allocate nothing and leave the outputs as they were
    before = len(backend.blocks)
    for keywords, want in ((dict(arena_bytes=3600 + 95), amd.STATUS_INVALID_ARGUMENT), (dict(count=6), amd.STATUS_INVALID_ARGUMENT),
                           (dict(most=1024 + 287), amd.STATUS_OUT_OF_MEMORY)):
        status, copies, starts = attach(**keywords)
        assert status == want and not copies.block and starts == [77, 77] and len(backend.blocks) == before, keywords
    pauses[1].host_expert_count = 0
    assert attach()[0] == amd.STATUS_INVALID_ARGUMENT  # a pause without host experts
    pauses[1].host_expert_count = 4
    backend.fail_staging_allocation = True
    status, copies, starts = attach()
    assert status == amd.STATUS_OUT_OF_MEMORY and not copies.block and starts == [77, 77]
    # no pauses and no table: nothing to allocate, an empty record
    backend.fail_staging_allocation = False
    status, copies, _ = attach(table_bytes=0, pause_count=0)
    assert status == 0 and not copies.block and copies.byte_count == 0 and len(backend.blocks) == before
