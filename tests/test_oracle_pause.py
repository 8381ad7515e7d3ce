"""The oracle of a step's expert pause (oracle/orc_pause.py) against the scenario the reference's own test holds
(tests/step_expert_pause_test.c:45-70, 561-631 of the reference): a card of four experts and six slots shared by two
layers of eight and four host experts, four steps whose uploads the test counts and whose slots its comments name, and
the four broken tags."""
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import orc_pause as orc  # noqa: E402

CARD_EXPERTS_OFFSET, SLOTS_OFFSET, EXPERT_BYTES, SLOT_BYTES, SLOTS = 4096, 8192, 192, 256, 6
MATRIX_OFFSETS = (0, 128, 64)  # gate, up, down: "w1, w2, w3 in the order of their names: gate, down, up" (:53-55)
FIRST_HOST_EXPERTS, SECOND_HOST_EXPERTS, HOST = 8, 4, 100
LAYERS = ((0, FIRST_HOST_EXPERTS), (FIRST_HOST_EXPERTS, SECOND_HOST_EXPERTS))  # (first_host_expert, host_expert_count)


def jobs_of(layer, experts):
    """What the test's router writes (:step_expert_pause_test.c, its stand-in): a card expert by its offsets, a host
    expert (numbered from HOST on, by its pause) by its tag."""
    first, _ = LAYERS[layer]
    jobs = []
    for expert in experts:
        if expert >= HOST:
            tag = SLOTS_OFFSET + (expert - HOST - first) * orc.TAG_BYTES
            jobs.append({"gate": tag, "up": tag, "down": tag, "rows": 1})
        else:
            at = CARD_EXPERTS_OFFSET + expert * EXPERT_BYTES
            jobs.append({"gate": at, "up": at + 128, "down": at + 64, "rows": 1})
    return jobs


def run(slots, layer, experts):
    jobs = jobs_of(layer, experts)
    first, count = LAYERS[layer]
    status, uploads, tags = orc.pause(jobs, slots, SLOTS_OFFSET, SLOT_BYTES, MATRIX_OFFSETS, first, count)
    assert status == orc.STATUS_OK
    return jobs, uploads, tags


def slot_of(job):
    return (job["gate"] - SLOTS_OFFSET) // SLOT_BYTES


def test_the_reference_scenario():
    slots = orc.Slots(SLOTS)
    # two host experts and a card expert in the first layer, one of the second's: slots 0, 1 and 2 (:575-579)
    jobs, uploads, tags = run(slots, 0, [HOST + 2, 1, HOST + 5])
    assert uploads == [(0, 2), (1, 5)] and tags == 2
    assert [slot_of(jobs[0]), slot_of(jobs[2])] == [0, 1] and jobs[1]["gate"] == CARD_EXPERTS_OFFSET + EXPERT_BYTES
    assert (jobs[0]["gate"], jobs[0]["up"], jobs[0]["down"]) == (SLOTS_OFFSET, SLOTS_OFFSET + 128, SLOTS_OFFSET + 64)
    jobs, uploads, tags = run(slots, 1, [HOST + FIRST_HOST_EXPERTS + 1])
    assert uploads == [(2, 1)] and slot_of(jobs[0]) == 2
    # the same experts again: the slots hold them, nothing goes up (:580-582)
    jobs, uploads, tags = run(slots, 0, [HOST + 5, HOST + 2])
    assert uploads == [] and tags == 2 and [slot_of(j) for j in jobs] == [1, 0]
    jobs, uploads, tags = run(slots, 1, [HOST + FIRST_HOST_EXPERTS + 1])
    assert uploads == [] and slot_of(jobs[0]) == 2
    # two rows, six host experts: expert 2 held in slot 0, five go up into the slots after it in turn (3, 4, 5, then 1
    # and 2 past the marked 0) (:583-587)
    jobs, uploads, tags = run(slots, 0, [HOST, HOST + 1, HOST + 3, HOST + 4, HOST + 2, HOST + 6])
    assert [slot for slot, _ in uploads] == [3, 4, 5, 1, 2] and [tag for _, tag in uploads] == [0, 1, 3, 4, 6]
    assert [slot_of(j) for j in jobs] == [3, 4, 5, 1, 0, 2] and tags == 6
    jobs, uploads, tags = run(slots, 1, [0, 3])  # the second layer on the card alone
    assert uploads == [] and tags == 0
    # the second layer's expert lost its slot 2: it goes up again, into the next in turn (:588-591)
    jobs, uploads, tags = run(slots, 0, [0, 3])
    assert uploads == [] and tags == 0
    jobs, uploads, tags = run(slots, 1, [HOST + FIRST_HOST_EXPERTS + 1])
    assert uploads == [(3, 1)] and slot_of(jobs[0]) == 3


def test_broken_tags():
    """:605-631: a tag off the tags' step, beyond the layer's, a job's matrices apart, a job partly a tag."""
    good = SLOTS_OFFSET + 3 * orc.TAG_BYTES
    on_card = CARD_EXPERTS_OFFSET
    for broken in ({"gate": good + 8, "up": good + 8, "down": good + 8}, {"gate": SLOTS_OFFSET + 8 * 16, "up": SLOTS_OFFSET + 8 * 16, "down": SLOTS_OFFSET + 8 * 16},
                   {"gate": good, "up": good + 16, "down": good}, {"gate": good, "up": on_card, "down": good}, {"gate": on_card, "up": good, "down": good}):
        jobs = [dict(broken, rows=1), {"gate": on_card, "up": on_card + 128, "down": on_card + 64, "rows": 1}]
        status, _, _ = orc.pause(jobs, orc.Slots(SLOTS), SLOTS_OFFSET, SLOT_BYTES, MATRIX_OFFSETS, 0, FIRST_HOST_EXPERTS)
        assert status == orc.STATUS_DEVICE_ERROR, broken
    # an empty job is not looked at, whatever its offsets
    jobs = [{"gate": good + 8, "up": 0, "down": 7, "rows": 0}]
    assert orc.pause(jobs, orc.Slots(SLOTS), SLOTS_OFFSET, SLOT_BYTES, MATRIX_OFFSETS, 0, FIRST_HOST_EXPERTS)[0] == orc.STATUS_OK
