"""CPU restatement (test infrastructure, not the product: only tests/ may import it) of a step's expert pause as the
reference's step driver runs it: source/step_experts.c:27-168, include/anemone/model_seam.h:193-214. Plain Python over
lists: a pause touches at most a few dozen jobs.

Pinned by the scenario of the reference's own tests/step_expert_pause_test.c:561-601 (test_steps: six slots shared by two
layers, which experts go up at each of four steps and into which slots) and its broken tags (:605-631), in
tests/test_oracle_pause.py.
"""

TAG_BYTES = 16  # LINEAR_OFFSET_ALIGNMENT_BYTES: the tags' step
STATUS_OK, STATUS_DEVICE_ERROR = 0, 5


class Slots:
    """A card's slots between pauses: the host expert each holds (None: none), the mark of the pause that took it last,
    the slot the next upload tries first (step_driver.h:73-77; step_experts.c:27-36)."""

    def __init__(self, count):
        self.held = [None] * count
        self.marks = [0] * count
        self.next_slot = 0
        self.pause_mark = 0


def pause(jobs, slots, slots_offset, slot_bytes, matrix_offsets, first_host_expert, host_expert_count):
    """jobs: list of dicts {gate, up, down, rows}; rewritten in place. Returns (status, uploads, tags): uploads a list of
    (slot, host expert of the pause) in the order they go up (step_experts.c:41-165)."""
    slots.pause_mark += 1
    mark = slots.pause_mark
    count = len(slots.held)
    uploads, tags = [], 0
    for second in (False, True):  # SLOT_PASSES: the slots that hold their expert, then the others'
        for job in jobs:
            offsets = (job["gate"], job["up"], job["down"])
            if job["rows"] == 0 or all(offset < slots_offset for offset in offsets):
                continue  # empty, or on the card (:69-74)
            gate = job["gate"]
            tag = (gate - slots_offset) // TAG_BYTES
            sound = (gate >= slots_offset and (gate - slots_offset) % TAG_BYTES == 0 and tag < host_expert_count and
                     job["up"] == gate and job["down"] == gate)
            if not sound:
                return STATUS_DEVICE_ERROR, uploads, tags  # :75-92
            expert = first_host_expert + tag
            slot = slots.held.index(expert) if expert in slots.held else count
            if slot < count:
                slots.marks[slot] = mark  # :96-102
            if not second:
                continue
            if slot == count:  # :106-146: the next in turn that no job of this pause marked
                slot = slots.next_slot
                tried = 1
                while tried < count and slots.marks[slot] == mark:
                    slot = (slot + 1) % count
                    tried += 1
                slots.next_slot = (slot + 1) % count
                if slots.marks[slot] == mark:
                    return STATUS_DEVICE_ERROR, uploads, tags
                uploads.append((slot, tag))
                slots.held[slot] = expert
                slots.marks[slot] = mark
            at = slots_offset + slot * slot_bytes  # :147-156
            job["gate"], job["up"], job["down"] = at + matrix_offsets[0], at + matrix_offsets[1], at + matrix_offsets[2]
            tags += 1
    return STATUS_OK, uploads, tags
