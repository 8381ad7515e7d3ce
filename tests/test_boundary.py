"""CPU tests of the boundary: the library loads without a card, exports every function its headers declare, lists its
kernels with the record sizes of anemone_records.h, and the prepare functions (pure arithmetic on a description; the
arena is a number) keep the refusal rules and launch geometry stated in anemone_ops.h. A fake backend table with a
kernel registry of names only stands in for a card, as the reference's host tests do
(tests/host_memory_backend.h:30-45 of the reference)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import anemone_amd as amd

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ARENA = 1 << 34


def declared_functions():
    names = set()
    for header in ("anemone_backend.h", "anemone_ops.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        for match in re.finditer(r"\b([a-z][a-z0-9_]+)\s*\((?!\s*\*)[^;{}]*\)\s*;", text):
            name = match.group(1)
            if name not in ("__attribute__", "warn_unused_result") and not name.startswith("result_status"):
                names.add(name)
    return names


def test_library_exports_every_declared_function():
    lib = amd.library()
    names = declared_functions()
    assert {"backend_hip_card_open", "exl3_tc_prepare", "router_select_prepare", "status_text",
            "weight_format_operations_of", "exl3_row_sum_prepare"} <= names
    missing = [name for name in sorted(names) if not hasattr(lib, name)]
    assert missing == []
    assert C.c_void_p.in_dll(lib, "backend_hip_value") is not None
    assert C.c_void_p.in_dll(lib, "exl3_weight_operations") is not None


def test_status_text_and_card_count_without_a_card():
    assert amd.status_text(0) == "ok" and amd.status_text(7) == "unsupported" and amd.status_text(99) == "unknown status"
    count = C.c_uint32(77)
    assert amd.library().backend_hip_card_count(C.byref(count)) == 0
    assert amd.library().backend_hip_card_count(None) == amd.STATUS_INVALID_ARGUMENT


def kernel_table():
    lib = amd.library()
    f, g, b = C.c_char_p(), C.c_char_p(), C.c_uint32()
    table = {}
    for i in range(lib.backend_hip_kernel_table_count()):
        assert lib.backend_hip_kernel_table_entry(i, C.byref(f), C.byref(g), C.byref(b)) == 0
        table[(f.value.decode(), g.value.decode())] = b.value
    return table


def test_kernel_table_matches_the_records():
    table = kernel_table()
    assert table[("kernel_exl3", "exl3_reconstruct")] == C.sizeof(amd.Exl3ReconstructRecord) == 32
    assert table[("kernel_exl3", "exl3_input")] == C.sizeof(amd.Exl3ExpertRecord) == 88
    assert table[("kernel_exl3", "exl3_row_sum")] == C.sizeof(amd.RowSumArguments) == 24
    assert table[("kernel_exl3_tc", "exl3_tc_products")] == C.sizeof(amd.Exl3TcRecord) == 96
    for width in ("k2", "k2_5", "k3", "k4", "mixed"):
        assert ("kernel_exl3", "exl3_gate_up_" + width) in table and ("kernel_exl3", "exl3_down_" + width) in table
    assert table[("kernel_router", "router_select_entry")] == 96
    assert C.sizeof(amd.KernelLaunch) == 232


# ---- a fake backend: kernel_prepare over the library's own kernel table, no card ----

PREPARE = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_char_p, C.c_char_p, C.c_uint32, C.POINTER(C.c_uint32))


class FakeBackend:
    def __init__(self):
        self.table = kernel_table()
        self.handles = []
        self.callback = PREPARE(self.prepare)
        # struct backend_operations: name, then 27 function pointers; kernel_prepare is the 11th member
        self.operations = (C.c_void_p * 28)()
        self.operations[11] = C.cast(self.callback, C.c_void_p)
        self.card = C.c_void_p(0x1000)  # never dereferenced by a prepare function

    def prepare(self, card, file, function, record_bytes, out):
        key = (file.decode(), function.decode())
        if key not in self.table:
            return amd.STATUS_INVALID_ARGUMENT
        if self.table[key] != record_bytes:
            return amd.STATUS_INVALID_ARGUMENT
        if key not in self.handles:
            self.handles.append(key)
        out[0] = self.handles.index(key)
        return 0

    @property
    def address(self):
        return C.addressof(self.operations)


@pytest.fixture()
def fake():
    return FakeBackend()


def chain_record(**changes):
    r = amd.Exl3ExpertRecord()
    pairs, H, I = 64, 4096, 2048
    r.jobs_offset, r.input_offset = 4096, 1 << 20
    r.operands_offset = 2 << 20
    r.products_offset = r.output_offset = (2 << 20) + pairs * H * 4
    r.hidden_offset = 16 << 20
    r.input_size, r.inner_size, r.pair_count, r.pairs_per_row, r.job_count = H, I, pairs, 8, pairs
    r.bits_per_weight, r.activation_limit = 3, 10.0
    for key, value in changes.items():
        setattr(r, key, value)
    return r


def test_chain_prepare_geometry(fake):
    lib = amd.library()
    launches = amd.launches_of(5)
    assert lib.exl3_experts_prepare(C.byref(chain_record()), ARENA, fake.address, fake.card, 950, launches) == 0
    names = [fake.handles[launch.kernel][1] for launch in launches]
    assert names == ["exl3_input", "exl3_gate_up_k3", "exl3_activate", "exl3_down_k3", "exl3_finish"]
    assert [list(l.grid) for l in launches] == [[32, 64, 2], [16, 64, 2], [16, 64, 1], [32, 64, 1], [32, 64, 1]]
    assert [l.block[0] for l in launches] == [64, 256, 64, 256, 64]
    assert all(l.argument_byte_count == 88 and not any(l.argument[88:]) for l in launches)
    mixed = amd.launches_of(5)
    assert lib.exl3_experts_prepare(C.byref(chain_record(widths_offset=1 << 30)), ARENA, fake.address, fake.card, 950, mixed) == 0
    assert fake.handles[mixed[1].kernel][1] == "exl3_gate_up_mixed" and fake.handles[mixed[3].kernel][1] == "exl3_down_mixed"
    # product launches of fewer than 256 blocks take the instances of one output tile a block (eight times the blocks)
    for jobs, pairs, names, grids in ((1, 8, ["exl3_gate_up_k3_thin", "exl3_down_k3_thin"], [[128, 1, 2], [256, 1, 1]]),
                                      (7, 8, ["exl3_gate_up_k3_thin", "exl3_down_k3_thin"], [[128, 7, 2], [256, 7, 1]]),
                                      (8, 8, ["exl3_gate_up_k3", "exl3_down_k3"], [[16, 8, 2], [32, 8, 1]])):
        few = amd.launches_of(5)
        assert lib.exl3_experts_prepare(C.byref(chain_record(job_count=jobs, pair_count=pairs)), ARENA, fake.address, fake.card, 950, few) == 0
        assert [fake.handles[few[i].kernel][1] for i in (1, 3)] == names and [list(few[i].grid) for i in (1, 3)] == grids
        assert [list(few[i].grid) for i in (0, 2, 4)] == [[32, jobs, 2], [16, jobs, 1], [32, jobs, 1]]
    assert lib.exl3_experts_prepare(C.byref(chain_record(job_count=1, pair_count=8, widths_offset=1 << 30)), ARENA, fake.address, fake.card, 950, mixed) == 0
    assert fake.handles[mixed[1].kernel][1] == "exl3_gate_up_mixed_thin" and fake.handles[mixed[3].kernel][1] == "exl3_down_mixed_thin"
    assert lib.exl3_scratch_byte_count(64, 4096) == 64 * 4096 * 12
    assert lib.exl3_width_name(6) == b"k3" and lib.exl3_width_name(5) == b"k2_5" and lib.exl3_width_name(7) is None


@pytest.mark.parametrize("changes,status", [
    (dict(reserved_zero=1), 1), (dict(pair_count=0), 1), (dict(pair_count=63), 1), (dict(job_count=0), 1),
    (dict(output_offset=64), 1), (dict(activation_limit=0.0), 1), (dict(activation_limit=float("nan")), 1),
    (dict(inner_size=8192), 1), (dict(bits_per_weight=9), 1), (dict(bits_per_weight=5), 7),
    (dict(hidden_offset=(2 << 20) + 64), 1),   # shares bytes with the operands
    (dict(jobs_offset=4100), 1),               # off the 16-byte alignment
    (dict(hidden_offset=ARENA - 4096), 1),     # leaves the arena
])
def test_chain_prepare_refusals_leave_the_launches_untouched(fake, changes, status):
    lib = amd.library()
    launches = amd.launches_of(5)
    C.memset(launches, 0xAB, C.sizeof(launches))
    before = bytes(launches)
    assert lib.exl3_experts_prepare(C.byref(chain_record(**changes)), ARENA, fake.address, fake.card, 950, launches) == status
    assert bytes(launches) == before


def test_chain_prepare_other_refusals(fake):
    lib = amd.library()
    launches = amd.launches_of(5)
    assert lib.exl3_experts_prepare(C.byref(chain_record()), ARENA, fake.address, fake.card, 80, launches) == 1  # another class
    assert lib.exl3_experts_prepare(None, ARENA, fake.address, fake.card, 950, launches) == 1
    assert lib.exl3_experts_relaxed_prepare(C.byref(chain_record()), ARENA, fake.address, fake.card, 950, launches) == 7
    assert lib.exl3_experts_fast_prepare(C.byref(chain_record()), ARENA, fake.address, fake.card, 950, launches) == 0


def tc_record(**changes):
    r = amd.Exl3TcRecord()
    r.jobs_offset, r.hidden_offset, r.workspace_offset, r.output_offset = 4096, 1 << 20, 2 << 20, 1 << 30
    r.row_count, r.job_capacity, r.intermediate, r.bits_x2 = 8, 64, 2048, 6
    r.activation_limit, r.hidden, r.pairs_per_row = 10.0, 4096, 8
    for key, value in changes.items():
        setattr(r, key, value)
    return r


def test_tc_prepare_geometry_and_refusals(fake):
    lib = amd.library()
    launches = amd.launches_of(5)
    assert lib.exl3_tc_prepare(C.byref(tc_record()), ARENA, fake.address, fake.card, launches) == 0
    assert [fake.handles[l.kernel][1] for l in launches] == ["exl3_tc_operands", "exl3_tc_products", "exl3_tc_activate",
                                                            "exl3_tc_products", "exl3_tc_combine"]
    assert [list(l.grid) for l in launches] == [[32, 64, 2], [32, 64, 2], [16, 64, 1], [64, 64, 1], [32, 8, 1]]
    passes = [amd.Exl3TcRecord.from_buffer_copy(bytes(l.argument)[:96]).pass_ for l in launches]
    assert passes == [0, 0, 0, 1, 0]
    assert amd.exl3_tc_workspace_bytes(64, 4096, 2048) == 64 * 4096 * 4 + 4 * 2 * 64 * 2048 * 4 + 4 * 64 * 4096 * 4
    for changes, status in [(dict(row_count=0), 1), (dict(row_count=65), 1), (dict(rotation=1), 7), (dict(shared_sum=2), 1),
                            (dict(shared_sum=1, shared_offset=ARENA - 4096), 1), (dict(shared_sum=1, shared_offset=1 << 20), 1),
                            (dict(intermediate=2000), 7), (dict(bits_x2=7), 7), (dict(bits_x2=0), 1), (dict(pass_=1), 1),
                            (dict(workspace_offset=(2 << 20) + 16), 1), (dict(output_offset=2 << 20), 1),
                            (dict(activation_limit=-1.0), 1), (dict(widths_offset=(2 << 20) + 256, expert_count=256), 1),
                            (dict(widths_offset=ARENA, expert_count=256), 1), (dict(widths_offset=4096 + 96, expert_count=256), 1),
                            # the table is checked for every expert's entry, not its first: its tail in the jobs, or past the arena
                            (dict(widths_offset=4096 - 1008, expert_count=256), 1), (dict(widths_offset=ARENA - 1008, expert_count=256), 1),
                            (dict(widths_offset=16384), 1), (dict(expert_count=256), 1), (dict(reserved_zero=1), 1)]:
        untouched = amd.launches_of(5)
        assert lib.exl3_tc_prepare(C.byref(tc_record(**changes)), ARENA, fake.address, fake.card, untouched) == status, changes
        assert not any(bytes(untouched))
    # a table of widths clear of the other ranges: taken
    tabled = amd.launches_of(5)
    assert lib.exl3_tc_prepare(C.byref(tc_record(widths_offset=16384, expert_count=256)), ARENA, fake.address, fake.card, tabled) == 0
    # the sum into the shared expert's rows: its own range, checked like the others
    joined = amd.launches_of(5)
    assert lib.exl3_tc_prepare(C.byref(tc_record(shared_sum=1, shared_offset=3 << 29)), ARENA, fake.address, fake.card, joined) == 0
    assert amd.Exl3TcRecord.from_buffer_copy(bytes(joined[4].argument)[:96]).shared_sum == 1
    # hidden 0 and pairs_per_row 0 stand for the reference's 5120 and 6
    default = amd.launches_of(5)
    assert lib.exl3_tc_prepare(C.byref(tc_record(hidden=0, pairs_per_row=0, intermediate=640, job_capacity=48)), ARENA,
                               fake.address, fake.card, default) == 0
    assert list(default[0].grid) == [40, 48, 2]


def test_reconstruct_and_row_sum_prepare(fake):
    lib = amd.library()
    record = amd.Exl3ReconstructRecord(4096, 1 << 24, 2304, 5120, 3, 0)
    launch = amd.launches_of(1)
    assert lib.exl3_reconstruct_prepare(C.byref(record), ARENA, 0, launch) == 0
    assert list(launch[0].grid) == [2304 * 5120 // 256, 1, 1] and launch[0].block[0] == 256
    # the output overlapping the matrix, and an arena too short: refused, the launch untouched
    for bad in (amd.Exl3ReconstructRecord(4096, 4096 + 1024, 2304, 5120, 3, 0), ):
        untouched = amd.launches_of(1)
        assert lib.exl3_reconstruct_prepare(C.byref(bad), ARENA, 0, untouched) == 1 and not any(bytes(untouched))
    untouched = amd.launches_of(1)
    assert lib.exl3_reconstruct_prepare(C.byref(record), 1 << 20, 0, untouched) == 1 and not any(bytes(untouched))
    assert lib.exl3_reconstruct_prepare(C.byref(record), ARENA, amd.BACKEND_NO_KERNEL, untouched) == 1
    row_sum = amd.RowSumArguments(1 << 20, 1 << 28, 4096, 8)
    assert lib.exl3_row_sum_prepare(C.byref(row_sum), 8, ARENA, fake.address, fake.card, launch) == 0
    assert list(launch[0].grid) == [16, 8, 1]


def test_stored_byte_counts():
    lib = amd.library()
    lib.weight_format_operations_of.restype = C.c_void_p

    class Operations(C.Structure):
        _fields_ = [("name", C.c_char_p), ("stored_byte_count", C.CFUNCTYPE(C.c_int, C.POINTER(amd.Shape), C.POINTER(C.c_uint64)))]

    def count(fmt, shape):
        operations = Operations.from_address(lib.weight_format_operations_of(fmt))
        out = C.c_uint64(0)
        return operations.stored_byte_count(C.byref(shape), C.byref(out)), out.value

    # the reference's known byte counts of a 2304 x 5120 EXL3 matrix (tests/exl3_widths_test.c:67-88)
    for stored, expected in ((2, 2963968), (40, 3701248), (3, 4438528), (4, 5913088)):
        assert count(amd.WEIGHT_FORMAT_EXL3, amd.Shape(2304, 5120, stored, 0)) == (0, expected)
    assert count(amd.WEIGHT_FORMAT_EXL3, amd.Shape(2304, 5120, 5, 0))[0] == 7       # defined, not decoded here
    assert count(amd.WEIGHT_FORMAT_EXL3, amd.Shape(2304, 5120, 9, 0))[0] == 1
    assert count(amd.WEIGHT_FORMAT_EXL3, amd.Shape(2300, 5120, 3, 0))[0] == 1
    assert count(amd.WEIGHT_FORMAT_E2M1_SCALED, amd.Shape(2048, 4096, 4, 0)) == (0, 4194304 + 262144)
    assert count(amd.WEIGHT_FORMAT_E4M3_SCALED, amd.Shape(48, 64, 8, 0)) == (0, 48 * 64 + 4)
    assert lib.weight_format_operations_of(0) is None and lib.weight_format_operations_of(1) is None


def router_description(fake, **changes):
    E, P, rows = 256, 8, 8
    experts = amd.RoutedExpertsDescription()
    experts.jobs = amd.Range(1 << 20, rows * P * 96)
    experts.expert_weights = amd.Range(1 << 24, 1 << 32)
    experts.gate_up_shape, experts.down_shape = amd.Shape(2048, 4096, 3, 0), amd.Shape(4096, 2048, 3, 0)
    experts.weight_format, experts.job_count, experts.row_count, experts.pairs_per_row = amd.WEIGHT_FORMAT_EXL3, rows * P, rows, P
    offsets = ((1 << 24) + np.arange(E * 3, dtype=np.uint64) * np.uint64(4 << 20))
    d = amd.RouterDescription()
    d.experts = C.pointer(experts)
    d.expert_offsets = offsets.ctypes.data_as(C.POINTER(C.c_uint64))
    d.step, d.scores, d.bias = amd.Range(256, 16), amd.Range(4096, rows * E * 4), amd.Range(65536, E * 4)
    d.offsets, d.affinities = amd.Range(131072, E * 24), amd.Range(262144, rows * E * 4)
    d.order, d.expert_count, d.pick_count, d.affinity_kind, d.route_scale = 0, E, P, 1, 1.5
    for key, value in changes.items():
        setattr(d, key, value)
    return d, experts, offsets


def test_router_projection_prepare_geometry(fake):
    """Which kernel takes a projection: many rows of a width in whole 128 inputs go to the matrix unit (16 experts by 64
    rows a block); any other width, and thin steps, to router_projection (eight experts a block)."""
    lib = amd.library()
    kernels = amd.RouterKernels()
    assert lib.router_kernels_prepare(fake.address, fake.card, C.byref(kernels)) == 0

    def prepared(rows, hidden, experts_n):
        d = amd.RouterProjectionDescription(amd.Range(1 << 20, experts_n * hidden * 2), amd.Range(1 << 24, rows * hidden * 2),
                                            amd.Range(1 << 27, rows * experts_n * 4), rows, hidden, experts_n, 0)
        launch = amd.launches_of(1)
        status = lib.router_projection_prepare(C.byref(d), ARENA, C.byref(kernels), launch)
        return status, (fake.handles[launch[0].kernel][1] if status == 0 else None), list(launch[0].grid), launch[0].block[0]

    assert prepared(300, 512, 64) == (0, "router_projection_tiles", [4, 5, 1], 256)
    assert prepared(4096, 4096, 256) == (0, "router_projection_tiles", [16, 64, 1], 256)
    status, name, grid, block = prepared(300, 160, 64)  # no whole number of stages of 128 inputs
    assert (status, name, grid) == (0, "router_projection", [8, 75, 1])
    status, name, grid, block = prepared(300, 512, 72)  # no whole number of 16 experts
    assert (status, name, grid) == (0, "router_projection", [9, 75, 1])
    status, name, grid, block = prepared(8, 4096, 256)  # a thin step: a row a block
    assert (status, name, grid) == (0, "router_projection", [32, 8, 1])
    assert prepared(300, 48, 64)[0] == 1 and prepared(0, 512, 64)[0] == 1  # a width that is no multiple of 32; no row


def test_router_prepare(fake):
    lib = amd.library()
    kernels = amd.RouterKernels()
    # the wide kernels may be absent: the select and the projection are required
    assert lib.router_kernels_prepare(fake.address, fake.card, C.byref(kernels)) == 0
    assert kernels.select != amd.BACKEND_NO_KERNEL and kernels.projection != amd.BACKEND_NO_KERNEL
    d, experts, offsets = router_description(fake)
    launch = amd.launches_of(1)
    assert lib.router_select_prepare(C.byref(d), ARENA, C.byref(kernels), launch) == 0
    assert list(launch[0].grid) == [1, 1, 1] and launch[0].block[0] == 512 and launch[0].argument_byte_count == 96
    for changes in (dict(expert_count=250), dict(pick_count=9), dict(order=1), dict(affinity_kind=2), dict(route_scale=0.0)):
        bad, keep, keep2 = router_description(fake, **changes)
        untouched = amd.launches_of(1)
        assert lib.router_select_prepare(C.byref(bad), ARENA, C.byref(kernels), untouched) == 1, changes
        assert not any(bytes(untouched))
    # an entry of the offsets table whose matrix leaves the experts' range
    bad, keep, table = router_description(fake)
    table[5] = (1 << 24) + (1 << 32) - 4096
    assert lib.router_select_prepare(C.byref(bad), ARENA, C.byref(kernels), launch) == 1
    # the reference order is the six-pick tree alone
    six, keep, keep2 = router_description(fake, order=1, pick_count=6, expert_count=384)
    keep.pairs_per_row, keep.job_count = 6, 48
    keep.jobs = amd.Range(1 << 20, 48 * 96)
    offsets384 = ((1 << 24) + np.arange(384 * 3, dtype=np.uint64) * np.uint64(1 << 20))
    six.expert_offsets = offsets384.ctypes.data_as(C.POINTER(C.c_uint64))
    six.scores, six.affinities, six.bias, six.offsets = amd.Range(4096, 8 * 384 * 4), amd.Range(262144, 8 * 384 * 4), amd.Range(65536, 384 * 4), amd.Range(131072, 384 * 24)
    keep.gate_up_shape, keep.down_shape = amd.Shape(512, 1024, 3, 0), amd.Shape(1024, 512, 3, 0)
    assert lib.router_select_prepare(C.byref(six), ARENA, C.byref(kernels), launch) == 0


def front_description(fake, width=4096, rows=8, ffn=False, **changes):
    d = amd.SiteFrontDescription()
    at = 1 << 21
    for name, size in (("streams", rows * 4 * width * 2), ("carried_pre", rows * 16), ("mix_weights", 24 * 4 * width * 4), ("scale", 12), ("base", 96),
                       ("norm_weight", width * 2), ("post", rows * 16), ("comb", rows * 64), ("hidden", rows * width * 2), ("codes", rows * width),
                       ("exponents", rows * width // 32), ("operands", rows * width * 2), ("scratch", amd.SITE_FRONT_SCRATCH_BYTES)):
        setattr(d, name, amd.Range(at, size))
        at += (size + 255) // 256 * 256
    d.kind, d.row_count, d.reserved_zero = (amd.SITE_FRONT_KIND_FFN if ffn else amd.SITE_FRONT_KIND_SITE), rows, width
    keep = []
    if ffn:
        router, experts, offsets = router_description(fake)
        d.router = C.pointer(router)
        d.router_weights = amd.Range(at, 256 * width * 2)
        keep = [router, experts, offsets]
    for key, value in changes.items():
        setattr(d, key, value)
    return d, keep


def test_site_front_prepare(fake):
    """One launch of blocks of width / 8 threads (the rows', the mix project's, the scores'); the FFN front's record carries the router select's record; the
    reference's refusals (site_front.h:42-75) and this build's (widths above 5,120); the two launches the site front may be cut in."""
    lib = amd.library()
    kernels, router_kernels = amd.SiteFrontKernels(), amd.RouterKernels()
    assert lib.site_front_kernels_prepare(fake.address, fake.card, C.byref(kernels)) == 0
    assert lib.router_kernels_prepare(fake.address, fake.card, C.byref(router_kernels)) == 0
    assert [fake.handles[k][1] for k in kernels.fronts[0:4]] == ["site_front_1", "site_front_8", "ffn_front_1", "ffn_front_8"]
    assert [fake.handles[k][1] for k in kernels.fronts[4:8]] == ["input_front_1", "input_front_8", "coefficient_front_1", "coefficient_front_8"]
    launch = amd.launches_of(1)
    d, keep = front_description(fake)
    assert lib.site_front_prepare(C.byref(d), ARENA, None, C.byref(kernels), launch) == 0
    assert fake.handles[launch[0].kernel][1] == "site_front_8" and list(launch[0].grid) == [8 + 6, 1, 1] and launch[0].block[0] == 512
    assert launch[0].argument_byte_count == 192
    record = np.frombuffer(bytes(launch[0].argument)[:192], dtype=np.uint64)
    assert record[9] == 8 and record[10] == d.streams.byte_offset and record[22] == d.scratch.byte_offset and record[23] == 0
    one, keep = front_description(fake, width=5120, rows=1, reserved_zero=0)
    assert lib.site_front_prepare(C.byref(one), ARENA, None, C.byref(kernels), launch) == 0
    assert fake.handles[launch[0].kernel][1] == "site_front_1" and list(launch[0].grid) == [1 + 6, 1, 1] and launch[0].block[0] == 640
    for kind, name, blocks in ((amd.SITE_FRONT_KIND_INPUT, "input_front_8", 8), (amd.SITE_FRONT_KIND_COEFFICIENTS, "coefficient_front_8", 6)):
        half, keep = front_description(fake, kind=kind)
        assert lib.site_front_prepare(C.byref(half), ARENA, None, C.byref(kernels), launch) == 0
        assert fake.handles[launch[0].kernel][1] == name and list(launch[0].grid) == [blocks, 1, 1] and launch[0].block[0] == 512
        assert bytes(launch[0].argument)[:192] == bytes(record), "the halves take the site front's record"
    f, keep = front_description(fake, ffn=True)
    assert lib.site_front_prepare(C.byref(f), ARENA, C.byref(router_kernels), C.byref(kernels), launch) == 0
    assert fake.handles[launch[0].kernel][1] == "ffn_front_8" and list(launch[0].grid) == [8 + 6 + 32, 1, 1]
    select = amd.launches_of(1)
    assert lib.router_select_prepare(C.byref(keep[0]), ARENA, C.byref(router_kernels), select) == 0
    assert bytes(launch[0].argument)[:72] == bytes(select[0].argument)[:72], "the select's nine offsets are the front's"
    words = np.frombuffer(bytes(launch[0].argument)[72:80], dtype=np.uint32)
    assert words[0] == 8 and words[1] == (0 | 256 << 1 | 8 << 11 | 1 << 15 | 0x3E00 << 16)
    assert np.frombuffer(bytes(launch[0].argument)[:192], dtype=np.uint64)[23] == f.router_weights.byte_offset
    refusals = [(dict(kind=amd.SITE_FRONT_KIND_INPUT), True, 1), (dict(kind=amd.SITE_FRONT_KIND_COEFFICIENTS), True, 1), (dict(kind=4), False, 1),
                (dict(row_count=0), False, 1), (dict(row_count=9), False, 1), (dict(reserved_zero=6144), False, 1), (dict(reserved_zero=1024), False, 1),
                (dict(reserved_zero=4100), False, 1), (dict(reserved_zero=2304), False, 1), (dict(kind=amd.SITE_FRONT_KIND_FFN), False, 1), (dict(kind=amd.SITE_FRONT_KIND_SITE), True, 1),
                (dict(hidden=amd.Range(1 << 21, 8 * 4096 * 2)), False, 1), (dict(scale=amd.Range(1 << 30, 16)), False, 1),
                (dict(scratch=amd.Range(1 << 30, 64)), False, 1), (dict(codes=amd.Range(ARENA - 256, 8 * 4096)), False, 1),
                (dict(row_count=4), True, 1), (dict(router_weights=amd.Range(4096, 256 * 4096 * 2)), True, 1)]
    for changes, ffn, status in refusals:
        bad, keep = front_description(fake, ffn=ffn, **changes)
        untouched = amd.launches_of(1)
        assert lib.site_front_prepare(C.byref(bad), ARENA, C.byref(router_kernels) if ffn else None, C.byref(kernels), untouched) == status, changes
        assert not any(bytes(untouched)), changes
    # a route scale that fp16 does not hold, a router the select refuses
    for changes in (dict(route_scale=1.1), dict(pick_count=9)):
        bad, keep = front_description(fake, ffn=True)
        setattr(keep[0], *list(changes.items())[0])
        untouched = amd.launches_of(1)
        assert lib.site_front_prepare(C.byref(bad), ARENA, C.byref(router_kernels), C.byref(kernels), untouched) == 1 and not any(bytes(untouched))
    # a front without its kernel, missing arguments
    none = amd.SiteFrontKernels()
    for i in range(8):
        none.fronts[i] = amd.BACKEND_NO_KERNEL
    d, keep = front_description(fake)
    assert lib.site_front_prepare(C.byref(d), ARENA, None, C.byref(none), launch) == 1
    assert lib.site_front_prepare(None, ARENA, None, C.byref(kernels), launch) == 1
    assert lib.site_front_kernels_prepare(fake.address, fake.card, None) == 1


# ---- the wide select, the prefill form, the FP4 / FP8 experts: geometry and refusals ----

def wide_description(**changes):
    E, P, rows = 256, 8, 4096
    offsets = ((1 << 28) + np.arange(E * 3, dtype=np.uint64) * np.uint64(4 << 20))
    d = amd.RouterWideDescription()
    d.expert_offsets = offsets.ctypes.data_as(C.POINTER(C.c_uint64))
    d.expert_weights = amd.Range(1 << 28, 1 << 32)
    d.gate_up_shape, d.down_shape, d.weight_format = amd.Shape(2048, 4096, 3, 0), amd.Shape(4096, 2048, 3, 0), amd.WEIGHT_FORMAT_EXL3
    cursor = [4096]

    def take(size):
        at = cursor[0]
        cursor[0] = (at + size + 255) // 256 * 256
        return amd.Range(at, size)
    d.step, d.scores, d.bias, d.offsets = take(16), take(rows * E * 4), take(E * 4), take(E * 24)
    d.affinities, d.picks, d.counts = take(rows * E * 4), take(rows * P * 8), take((rows + 383) // 384 * E * 4)
    d.pairs, d.runs = take(rows * P * 8), take(E * 8)
    d.tiles, d.jobs = take(amd.wide_tile_count(rows, P, E) * 32), take(amd.wide_job_count(rows, P, E) * 96)
    d.order, d.row_count, d.expert_count, d.pick_count, d.affinity_kind, d.route_scale = 0, rows, E, P, 1, 1.5
    for key, value in changes.items():
        setattr(d, key, value)
    return d, offsets


def test_wide_router_prepare(fake):
    lib = amd.library()
    kernels = amd.RouterKernels()
    assert lib.router_kernels_prepare(fake.address, fake.card, C.byref(kernels)) == 0
    assert amd.BACKEND_NO_KERNEL not in (kernels.wide_select, kernels.wide_count, kernels.wide_place, kernels.wide_jobs)
    assert kernels.wide_small != amd.BACKEND_NO_KERNEL
    d, keep = wide_description()
    launches = amd.launches_of(4)
    assert lib.router_wide_prepare(C.byref(d), ARENA, C.byref(kernels), launches) == 0
    names = [fake.handles[l.kernel][1] for l in launches]
    assert names == ["router_wide_select", "router_wide_count", "router_wide_place", "router_wide_jobs"]
    assert [list(l.grid) for l in launches] == [[512, 1, 1], [11, 1, 1], [11, 1, 1], [1, 1, 1]]
    assert all(l.block[0] == 512 and l.argument_byte_count == 136 for l in launches)
    assert amd.wide_tile_count(4096, 8, 256) == 768 and amd.wide_job_count(4096, 8, 256) == 4320  # 32768 pairs over 256 experts: at most pairs / 64 + experts tiles and (pairs + 7 experts) / 8 jobs
    for changes in (dict(row_count=0), dict(row_count=70000), dict(expert_count=100), dict(pick_count=0), dict(route_scale=-1.0),
                    dict(reserved_zero=1), dict(weight_format=1), dict(jobs=amd.Range(1 << 27, 96))):
        bad, keep = wide_description(**changes)
        untouched = amd.launches_of(4)
        assert lib.router_wide_prepare(C.byref(bad), ARENA, C.byref(kernels), untouched) == 1, changes
        assert not any(bytes(untouched))
    # two ranges of one description that share a byte
    bad, keep = wide_description()
    bad.runs = amd.Range(bad.pairs.byte_offset, 256 * 8)
    assert lib.router_wide_prepare(C.byref(bad), ARENA, C.byref(kernels), amd.launches_of(4)) == 1
    # the form of at most 384 rows: the select and one block
    two = amd.launches_of(2)
    d, keep = wide_description()
    assert lib.router_wide_small_prepare(C.byref(d), ARENA, C.byref(kernels), two) == 1  # 4096 rows
    assert not any(bytes(two))
    d, keep = wide_description(row_count=384)
    assert lib.router_wide_small_prepare(C.byref(d), ARENA, C.byref(kernels), two) == 0
    assert [fake.handles[l.kernel][1] for l in two] == ["router_wide_select", "router_wide_small"]
    assert [list(l.grid) for l in two] == [[48, 1, 1], [1, 1, 1]] and two[1].block[0] == 512 and two[1].argument_byte_count == 136
    d, keep = wide_description(row_count=385)
    assert lib.router_wide_small_prepare(C.byref(d), ARENA, C.byref(kernels), amd.launches_of(2)) == 1


def tcp_record(**changes):
    r = amd.Exl3TcpRecord()
    rows, H, I, P, E = 4096, 4096, 2048, 8, 256
    r.picks_offset, r.expert_offsets_offset, r.hidden_offset = 4096, 1 << 20, 2 << 20
    r.output_offset, r.workspace_offset = 64 << 20, 256 << 20
    r.row_count, r.intermediate, r.bits_x2, r.activation_limit = rows, I, 6, 10.0
    r.hidden, r.pairs_per_row, r.expert_count = H, P, E
    for key, value in changes.items():
        setattr(r, key, value)
    return r


def test_tcp_prepare_geometry_and_refusals(fake):
    lib = amd.library()
    launches, count = amd.launches_of(8), C.c_uint32(0)
    assert lib.exl3_tcp_prepare(C.byref(tcp_record()), ARENA, fake.address, fake.card, launches, C.byref(count)) == 0
    assert count.value == 7
    names = [fake.handles[launches[i].kernel][1] for i in range(7)]
    assert names == ["exl3_tcp_count", "exl3_tcp_place", "exl3_tcp_operands", "exl3_tcp_gemm", "exl3_tcp_activate", "exl3_tcp_gemm",
                     "exl3_tcp_combine"]
    capacity = 4096 * 8 // amd.EXL3_TCP_CHUNK_PAIRS + 256
    assert [list(launches[i].grid) for i in range(7)] == [[11, 1, 1], [11, 1, 1], [8, capacity, 10], [8, capacity, 2], [4, capacity, 10],
                                                               [16, capacity, 1], [8, 4096, 1]]  # element-wise launches: 512 channels a wavefront, 16 pairs a block
    assert [launches[i].block[0] for i in range(7)] == [512, 512, 64, 256, 64, 256, 64]
    records = [amd.Exl3TcpRecord.from_buffer_copy(bytes(launches[i].argument)[:112]) for i in range(7)]
    assert [r.pass_ for r in records] == [0, 0, 0, 0, 0, 3, 0] and all(launches[i].argument_byte_count == 112 for i in range(7))
    layout = amd.exl3_tcp_layout(4096, 8, 256, 4096, 2048)
    assert layout["total"] % 256 == 0 and layout["down"] - layout["gate_up"] == 2 * 32768 * 2048 * 4
    for changes, status in ((dict(row_count=0), 1), (dict(pairs_per_row=9), 1), (dict(expert_count=0), 1), (dict(pass_=1), 1),
                            (dict(rotation=1), 7), (dict(half_rows=5), 7), (dict(cone_layer=3), 7), (dict(intermediate=2000), 7),
                            (dict(hidden=1024, intermediate=2176), 7),  # the down operands would not fit over the gate and up operands

                            (dict(bits_x2=7), 7), (dict(bits_x2=40), 1), (dict(workspace_offset=(256 << 20) + 16), 1),
                            (dict(workspace_offset=ARENA - 4096), 1), (dict(output_offset=2 << 20), 1),
                            (dict(widths_offset=(256 << 20) + 512), 1), (dict(widths_offset=ARENA - 512), 1), (dict(widths_offset=(1 << 20) + 1024), 1)):
        untouched, n = amd.launches_of(8), C.c_uint32(99)
        assert lib.exl3_tcp_prepare(C.byref(tcp_record(**changes)), ARENA, fake.address, fake.card, untouched, C.byref(n)) == status, changes
        assert not any(bytes(untouched)) and n.value == 99


    # a table of widths of the experts' number, clear of the other ranges: taken
    assert lib.exl3_tcp_prepare(C.byref(tcp_record(widths_offset=48 << 20)), ARENA, fake.address, fake.card, launches, C.byref(count)) == 0


def experts_description(fmt=amd.WEIGHT_FORMAT_E2M1_SCALED, **changes):
    rows, P, H, I = 8, 8, 4096, 2048
    pairs = rows * P
    bits = 4 if fmt in (amd.WEIGHT_FORMAT_E2M1_SCALED, amd.WEIGHT_FORMAT_E2M1_GFX950) else 8
    d = amd.RoutedExpertsDescription()
    cursor = [4096]

    def take(size):
        at = cursor[0]
        cursor[0] = (at + size + 255) // 256 * 256
        return amd.Range(at, size)
    d.jobs, d.expert_weights = take(pairs * 96), take(1 << 30)
    d.codes, d.exponents, d.operands = take(rows * H), take(rows * H // 32), take(rows * H * 2)
    d.hidden, d.hidden_codes, d.hidden_exponents, d.hidden_operands = take(pairs * I * 2), take(pairs * I), take(pairs * I // 32), take(pairs * I * 2)
    d.pair_output, d.row_output = take(pairs * H * 2), take(rows * H * 4)
    d.gate_up_shape, d.down_shape, d.weight_format = amd.Shape(I, H, bits, 0), amd.Shape(H, I, bits, 0), fmt
    d.job_count, d.row_count, d.pairs_per_row = pairs, rows, P
    d.gate_up_slice_count, d.down_slice_count, d.activation_limit = 4, 2, 10.0
    for key, value in changes.items():
        setattr(d, key, value)
    return d


def test_linear_prepare_geometry_and_refusals(fake):
    lib = amd.library()
    kernels = amd.LinearKernels()
    assert lib.linear_kernels_prepare(fake.address, fake.card, 80, C.byref(kernels)) == 1  # a class of another card
    assert lib.linear_kernels_prepare(fake.address, fake.card, 950, C.byref(kernels)) == 0
    assert kernels.expert_gate_up[4] == amd.BACKEND_NO_KERNEL and kernels.trunk_linear_bfloat16[0] == amd.BACKEND_NO_KERNEL  # 16 slices; rows that are not quantized
    assert fake.handles[kernels.trunk_hidden][1] == "trunk_hidden_entry" and kernels.trunk_linear_quantized[4] == amd.BACKEND_NO_KERNEL
    assert fake.handles[kernels.trunk_linear_quantized_wide[2]] == ("kernel_trunk_linear", "trunk_linear_quantized_wide_4")
    assert fake.handles[kernels.trunk_linear_quantized_interleaved][1] == "trunk_linear_quantized_interleaved_1"
    launches = amd.launches_of(4)
    assert lib.linear_routed_experts_prepare(C.byref(experts_description()), ARENA, C.byref(kernels), launches) == 0
    names = [fake.handles[l.kernel][1] for l in launches]
    assert names == ["expert_gate_up_4", "activation_quantize_entry", "expert_down_2", "expert_row_sum_entry"]
    assert [list(l.grid) for l in launches] == [[32, 64, 1], [2, 64, 1], [64, 64, 1], [2, 8, 1]]  # the quantizer: 1,024 values a block
    assert [l.block[0] for l in launches] == [256, 256, 128, 256]
    assert [l.argument_byte_count for l in launches] == [64, 40, 56, 24]
    fp8 = amd.launches_of(4)
    assert lib.linear_routed_experts_prepare(C.byref(experts_description(amd.WEIGHT_FORMAT_E4M3_SCALED)), ARENA, C.byref(kernels), fp8) == 0
    assert [fake.handles[l.kernel][1] for l in fp8][::2] == ["expert_gate_up_e4m3_4", "expert_down_e4m3_2"]
    assert [list(l.grid) for l in fp8][::2] == [[64, 64, 1], [128, 64, 1]]  # strips of 32 outputs
    for changes in (dict(gate_up_slice_count=3), dict(down_slice_count=16), dict(row_count=0), dict(activation_limit=0.0),
                    dict(weight_format=amd.WEIGHT_FORMAT_EXL3), dict(reserved_zero=1), dict(gate_up_shape=amd.Shape(2048, 4000, 4, 0)),
                    dict(down_shape=amd.Shape(4096, 1024, 4, 0)), dict(gate_up_shape=amd.Shape(32, 4096, 4, 0))):
        untouched = amd.launches_of(4)
        assert lib.linear_routed_experts_prepare(C.byref(experts_description(**changes)), ARENA, C.byref(kernels), untouched) == 1, changes
        assert not any(bytes(untouched))
    quantize = amd.QuantizeDescription(amd.Range(4096, 8 * 4096 * 2), amd.Range(1 << 20, 8 * 4096), amd.Range(2 << 20, 8 * 128),
                                       amd.Range(3 << 20, 8 * 4096 * 2), 4096, 8)
    one = amd.launches_of(1)
    assert lib.linear_quantize_prepare(C.byref(quantize), ARENA, C.byref(kernels), one) == 0
    assert list(one[0].grid) == [4, 8, 1] and one[0].argument_byte_count == 40
    quantize.width = 4100
    assert lib.linear_quantize_prepare(C.byref(quantize), ARENA, C.byref(kernels), one) == 1
    shape, count = amd.Shape(2048, 4096, 4, 0), C.c_uint32(0)
    assert lib.linear_default_slice_count(1, 0, 0, C.byref(shape), 950, C.byref(count)) == 0 and count.value in (1, 2, 4, 8)


def wide_experts_description(fmt=amd.WEIGHT_FORMAT_E2M1_SCALED, **changes):
    rows, P, E = 1024, 8, 256
    tile_count = amd.wide_tile_count(rows, P, E)
    d = amd.LinearWideExpertsDescription()
    d.experts = experts_description(fmt, row_count=rows, gate_up_slice_count=1, down_slice_count=1)
    pairs, H, I = rows * P, 4096, 2048
    cursor = [3 << 30]

    def take(size):
        at = cursor[0]
        cursor[0] = (at + size + 255) // 256 * 256
        return amd.Range(at, size)
    e = d.experts
    e.codes, e.exponents = take(rows * H), take(rows * H // 32)
    e.hidden_codes, e.hidden_exponents, e.hidden_operands = take(pairs * I), take(pairs * I // 32), take(pairs * I * 2)
    e.pair_output, e.row_output = take(pairs * H * 2), take(rows * H * 4)
    d.tiles, d.pairs, d.tile_count = take(tile_count * 32), take(pairs * 8), tile_count
    for key, value in changes.items():
        if hasattr(d, key):
            setattr(d, key, value)
        else:
            setattr(d.experts, key, value)
    return d


def test_wide_linear_prepare_geometry_and_refusals(fake):
    lib = amd.library()
    arena = 8 << 30
    linear, kernels = amd.LinearKernels(), amd.LinearWideKernels()
    assert lib.linear_kernels_prepare(fake.address, fake.card, 950, C.byref(linear)) == 0
    assert lib.linear_wide_kernels_prepare(fake.address, fake.card, 90, C.byref(kernels)) == 1
    assert lib.linear_wide_kernels_prepare(fake.address, fake.card, 950, C.byref(kernels)) == 0
    table = kernel_table()
    assert table[("kernel_wide_linear", "wide_expert_gate_up_1")] == C.sizeof(amd.WideExpertGateUpArguments) == 88
    assert table[("kernel_wide_linear", "wide_expert_down_1")] == C.sizeof(amd.WideExpertDownArguments) == 64
    launches = amd.launches_of(3)
    assert lib.linear_wide_experts_prepare(C.byref(wide_experts_description()), arena, C.byref(linear), C.byref(kernels), launches) == 0
    assert [fake.handles[l.kernel][1] for l in launches] == ["wide_expert_gate_up_1", "wide_expert_down_1", "expert_row_sum_entry"]
    tiles = 1024 * 8 // 64 + 256
    assert [list(l.grid) for l in launches] == [[16, tiles, 1], [16, tiles, 1], [2, 1024, 1]]
    assert [l.block[0] for l in launches] == [256, 256, 256]
    assert [l.dynamic_shared_byte_count for l in launches] == [53760, 51712, 0]  # three blocks of either fit a CU's 160 KB
    assert [l.argument_byte_count for l in launches] == [88, 64, 24]
    record = amd.WideExpertGateUpArguments.from_buffer_copy(bytes(launches[0].argument)[:88])
    assert (record.output_size, record.input_size, record.tile_count, record.pairs_per_row, record.pair_count) == (2048, 4096, tiles, 8, 8192)
    fp8 = amd.launches_of(3)
    description = wide_experts_description(amd.WEIGHT_FORMAT_E4M3_SCALED)
    assert lib.linear_wide_experts_prepare(C.byref(description), arena, C.byref(linear), C.byref(kernels), fp8) == 0
    assert [fake.handles[l.kernel][1] for l in fp8][:2] == ["wide_expert_gate_up_e4m3_1", "wide_expert_down_e4m3_1"]
    assert [list(l.grid) for l in fp8][:2] == [[32, tiles, 1], [32, tiles, 1]]  # strips of 16 hidden outputs, of 32 outputs
    assert [l.dynamic_shared_byte_count for l in fp8] == [53760, 51712, 0]
    for changes in (dict(gate_up_slice_count=2), dict(down_slice_count=4), dict(tile_count=0), dict(tile_count=70000), dict(reserved_zero=1),
                    dict(row_count=0), dict(row_count=20000), dict(activation_limit=0.0), dict(weight_format=amd.WEIGHT_FORMAT_EXL3),
                    dict(tiles=amd.Range(3 << 30, 64)), dict(pairs=amd.Range((8 << 30) - 256, 65536)),
                    dict(gate_up_shape=amd.Shape(2048, 4000, 4, 0)), dict(down_shape=amd.Shape(4096, 1024, 4, 0))):
        untouched = amd.launches_of(3)
        status = lib.linear_wide_experts_prepare(C.byref(wide_experts_description(**changes)), arena, C.byref(linear), C.byref(kernels), untouched)
        assert status == 1, changes
        assert not any(bytes(untouched))


# ---- the shared expert and the FFN site's join ----

def shared_description(rows=8, gate_up_slices=4, down_slices=2, form=amd.LINEAR_WIDE_GROUP_BLOCKS, **changes):
    H, I = 4096, 2048
    cursor = [4096]

    def take(size):
        at = cursor[0]
        cursor[0] = (at + size + 255) // 256 * 256
        return amd.Range(at, size)

    def matrix(outputs, inputs, slices):
        return amd.LinearMatrix(take(outputs * inputs + (outputs + 31) // 32 * (inputs // 32)), amd.Shape(outputs, inputs, 8, 0),
                                amd.WEIGHT_FORMAT_E4M3_SCALED, slices, form, 0)
    d = amd.SharedExpertDescription()
    d.gate, d.up, d.down = matrix(I, H, gate_up_slices), matrix(I, H, gate_up_slices), matrix(H, I, down_slices)
    d.codes, d.exponents, d.operands = take(rows * H), take(rows * H // 32), take(rows * H * 2)
    d.gate_output, d.up_output, d.hidden = take(rows * I * 2), take(rows * I * 2), take(rows * I * 2)
    d.hidden_codes, d.hidden_exponents, d.hidden_operands = take(rows * I), take(rows * I // 32), take(rows * I * 2)
    d.output = take(rows * H * 2)
    d.row_count, d.activation_limit = rows, 10.0
    for key, value in changes.items():
        setattr(d, key, value)
    return d, cursor[0]


def join_description(rows=8, picks=8, width=4096, first=1 << 30, row_sums=True, **changes):
    cursor = [first]

    def take(size):
        at = cursor[0]
        cursor[0] = (at + size + 255) // 256 * 256
        return amd.Range(at, size)
    d = amd.ExpertJoinDescription()
    wide = 5120 if width == 0 else width
    d.pair_output, d.shared_output, d.streams = take(rows * picks * wide * 2), take(rows * wide * 2), take(rows * 4 * wide * 2)
    d.post, d.comb = take(rows * 16), take(rows * 64)
    d.row_sums = take(rows * wide * 4) if row_sums else amd.Range(0, 0)
    d.pairs_per_row, d.row_count, d.width = picks, rows, width
    for key, value in changes.items():
        setattr(d, key, value)
    return d


def test_shared_expert_prepare_geometry_and_refusals(fake):
    lib = amd.library()
    arena = 8 << 30
    kernels = amd.LinearKernels()
    assert lib.linear_kernels_prepare(fake.address, fake.card, 950, C.byref(kernels)) == 0
    table = kernel_table()
    assert table[("kernel_trunk_linear", "trunk_linear_quantized_1")] == C.sizeof(amd.TrunkLinearQuantizedArguments) == 72
    assert table[("kernel_trunk_linear", "trunk_hidden_entry")] == 32
    launches = amd.launches_of(4)
    d, _ = shared_description()
    assert lib.linear_shared_expert_prepare(C.byref(d), arena, C.byref(kernels), launches) == 0
    assert [fake.handles[l.kernel][1] for l in launches] == ["trunk_linear_quantized_4", "trunk_hidden_entry", "activation_quantize_entry",
                                                             "trunk_linear_quantized_2"]
    assert [list(l.grid) for l in launches] == [[128, 1, 1], [1, 8, 1], [2, 8, 1], [128, 1, 1]]  # strips of 32 outputs of both matrices
    assert [l.block[0] for l in launches] == [256, 256, 256, 128]
    assert [l.argument_byte_count for l in launches] == [72, 32, 40, 72]
    record = amd.TrunkLinearQuantizedArguments.from_buffer_copy(bytes(launches[0].argument)[:72])
    assert list(record.output_size) == [2048, 2048] and (record.input_size, record.row_count) == (4096, 8)
    assert list(record.weights_offset) == [d.gate.stored.byte_offset, d.up.stored.byte_offset]
    down = amd.TrunkLinearQuantizedArguments.from_buffer_copy(bytes(launches[3].argument)[:72])
    assert list(down.output_size) == [4096, 0] and down.codes_offset == d.hidden_codes.byte_offset
    # more than eight rows: the matrix's wide form
    for form, names, grids, blocks, shared_bytes in (
            (amd.LINEAR_WIDE_GROUP_BLOCKS, ["trunk_linear_quantized_wide_4", "trunk_linear_quantized_wide_2"], [[128 * 13, 1, 1], [128 * 13, 1, 1]], [256, 128], 0),
            (amd.LINEAR_WIDE_TILE_BLOCKS, ["trunk_linear_quantized_wide_4", "trunk_linear_quantized_wide_2"], [[128, 1, 1], [128, 1, 1]], [256, 128], 0)):
        wide, _ = shared_description(rows=100, form=form)
        assert lib.linear_shared_expert_prepare(C.byref(wide), arena, C.byref(kernels), launches) == 0
        assert [fake.handles[l.kernel][1] for l in launches][::3] == names
        assert [list(l.grid) for l in launches][::3] == grids and [l.block[0] for l in launches][::3] == blocks
        assert launches[0].dynamic_shared_byte_count == shared_bytes
    many, _ = shared_description(rows=8192, gate_up_slices=1, down_slices=1, form=amd.LINEAR_INTERLEAVED_CHUNK_BLOCKS)
    assert lib.linear_shared_expert_prepare(C.byref(many), arena, C.byref(kernels), launches) == 0
    assert [fake.handles[l.kernel][1] for l in launches][::3] == ["trunk_linear_quantized_interleaved_1"] * 2
    assert [list(l.grid) for l in launches] == [[32, 128, 1], [1, 8192, 1], [2, 8192, 1], [32, 128, 1]]
    assert [l.dynamic_shared_byte_count for l in launches] == [51712, 0, 0, 51712] and launches[0].block[0] == 256
    sliced, _ = shared_description(rows=100, form=amd.LINEAR_INTERLEAVED_CHUNK_BLOCKS)  # the interleaved form is of one slice
    untouched = amd.launches_of(4)
    assert lib.linear_shared_expert_prepare(C.byref(sliced), arena, C.byref(kernels), untouched) == 1 and not any(bytes(untouched))
    for changes in (dict(row_count=0), dict(row_count=20000), dict(activation_limit=0.0), dict(output=amd.Range((8 << 30) - 256, 1 << 20)),
                    dict(hidden=amd.Range(4096, 1 << 16))):
        bad, _ = shared_description(**changes)
        assert lib.linear_shared_expert_prepare(C.byref(bad), arena, C.byref(kernels), untouched) == 1, changes
        assert not any(bytes(untouched))
    for mutate in (lambda d: setattr(d.gate, "weight_format", amd.WEIGHT_FORMAT_E2M1_SCALED), lambda d: setattr(d.up, "slice_count", 2),
                   lambda d: setattr(d.down, "slice_count", 3), lambda d: setattr(d.down, "wide_form", 7),
                   lambda d: setattr(d.up, "shape", amd.Shape(1024, 4096, 8, 0)), lambda d: setattr(d.gate, "reserved_zero", 1)):
        bad, _ = shared_description()
        mutate(bad)
        assert lib.linear_shared_expert_prepare(C.byref(bad), arena, C.byref(kernels), untouched) == 1
        assert not any(bytes(untouched))
    # a trunk launch of one matrix
    one = amd.TrunkQuantizedDescription()
    one.matrices[0], one.codes, one.exponents, one.operands, one.outputs[0] = d.down, d.hidden_codes, d.hidden_exponents, d.hidden_operands, d.output
    one.matrix_count, one.row_count = 1, 8
    launch = amd.launches_of(1)
    assert lib.linear_trunk_quantized_prepare(C.byref(one), arena, C.byref(kernels), launch) == 0
    assert fake.handles[launch[0].kernel][1] == "trunk_linear_quantized_2" and list(launch[0].grid) == [128, 1, 1]
    one.matrix_count = 3
    assert lib.linear_trunk_quantized_prepare(C.byref(one), arena, C.byref(kernels), launch) == 1


def test_join_prepare_geometry_and_refusals(fake):
    lib = amd.library()
    arena = 8 << 30
    linear, kernels = amd.LinearKernels(), amd.ExpertFusedKernels()
    assert lib.linear_kernels_prepare(fake.address, fake.card, 950, C.byref(linear)) == 0
    assert lib.expert_fused_kernels_prepare(fake.address, fake.card, 950, C.byref(kernels)) == 0
    assert fake.handles[kernels.join] == ("kernel_hyper_connection", "expert_join")
    assert fake.handles[kernels.shared_join[1]] == ("kernel_trunk_linear", "expert_shared_join_2") and kernels.shared_join[4] == amd.BACKEND_NO_KERNEL
    table = kernel_table()
    assert table[("kernel_hyper_connection", "expert_join")] == C.sizeof(amd.ExpertJoinArguments) == 56
    assert table[("kernel_hyper_connection", "hyper_post_entry")] == 48 and table[("kernel_trunk_linear", "expert_shared_join_1")] == 96
    launch = amd.launches_of(1)
    d = join_description()
    assert lib.expert_join_prepare(C.byref(d), arena, C.byref(kernels), launch) == 0
    assert list(launch[0].grid) == [4, 8, 1] and launch[0].block[0] == 128 and launch[0].argument_byte_count == 56
    record = amd.ExpertJoinArguments.from_buffer_copy(bytes(launch[0].argument)[:56])
    assert (record.pair_output_offset, record.row_sums_offset, record.pairs_per_row) == (d.pair_output.byte_offset, d.row_sums.byte_offset, 8)
    none = join_description(row_sums=False)
    assert lib.expert_join_prepare(C.byref(none), arena, C.byref(kernels), launch) == 0
    assert amd.ExpertJoinArguments.from_buffer_copy(bytes(launch[0].argument)[:56]).row_sums_offset == 0xFFFFFFFFFFFFFFFF
    default = join_description(width=0, rows=3000, picks=6)  # the reference's width
    assert lib.expert_join_prepare(C.byref(default), arena, C.byref(kernels), launch) == 0 and list(launch[0].grid) == [5, 3000, 1]
    assert lib.expert_post_prepare(C.byref(d), arena, kernels.post, launch) == 0
    assert fake.handles[launch[0].kernel][1] == "hyper_post_entry" and launch[0].argument_byte_count == 48 and list(launch[0].grid) == [4, 8, 1]
    untouched = amd.launches_of(1)
    assert lib.expert_post_prepare(C.byref(none), arena, kernels.post, untouched) == 1
    for changes in (dict(row_count=0), dict(pairs_per_row=0), dict(width=4100), dict(width=512), dict(streams=amd.Range(1 << 30, 1 << 20)),
                    dict(post=amd.Range((8 << 30) - 64, 128)), dict(comb=amd.Range((1 << 30) + 8, 512))):
        assert lib.expert_join_prepare(C.byref(join_description(**changes)), arena, C.byref(kernels), untouched) == 1, changes
        assert not any(bytes(untouched))
    # the shared join: the down of a shared expert with the join behind it
    shared, end = shared_description(down_slices=2)
    s = amd.ExpertSharedJoinDescription()
    s.down, s.codes, s.exponents, s.operands = shared.down, shared.hidden_codes, shared.hidden_exponents, shared.hidden_operands
    s.join = join_description()
    assert lib.expert_shared_join_prepare(C.byref(s), arena, C.byref(linear), C.byref(kernels), launch) == 0
    assert fake.handles[launch[0].kernel][1] == "expert_shared_join_2" and list(launch[0].grid) == [128, 1, 1] and launch[0].block[0] == 128
    assert launch[0].argument_byte_count == 96
    s.join = join_description(rows=9)
    assert lib.expert_shared_join_prepare(C.byref(s), arena, C.byref(linear), C.byref(kernels), untouched) == 1 and not any(bytes(untouched))
    s.join = join_description(width=5120)
    assert lib.expert_shared_join_prepare(C.byref(s), arena, C.byref(linear), C.byref(kernels), untouched) == 1  # down has 4,096 outputs


# ---- the FP8 experts with float32 scales of 128 x 128 blocks (an extension) ----

def test_block128_prepare_geometry_and_refusals(fake):
    lib = amd.library()
    arena = 8 << 30
    B128 = amd.WEIGHT_FORMAT_E4M3_BLOCK128
    count = C.c_uint64(0)
    operations = lib.weight_format_operations_of
    operations.restype = C.c_void_p
    linear, wide_kernels = amd.LinearKernels(), amd.LinearWideKernels()
    assert lib.linear_kernels_prepare(fake.address, fake.card, 950, C.byref(linear)) == 0
    assert lib.linear_wide_kernels_prepare(fake.address, fake.card, 950, C.byref(wide_kernels)) == 0
    assert fake.handles[linear.expert_gate_up_b128[2]][1] == "expert_gate_up_b128_4" and linear.expert_down_b128[4] == amd.BACKEND_NO_KERNEL
    assert fake.handles[linear.activation_quantize_128] == ("kernel_activation_quantize", "activation_quantize_128_entry")
    assert fake.handles[wide_kernels.wide_expert_down_b128][1] == "wide_expert_down_b128_1"
    launches = amd.launches_of(4)
    assert lib.linear_routed_experts_prepare(C.byref(experts_description(B128)), ARENA, C.byref(linear), launches) == 0
    assert [fake.handles[l.kernel][1] for l in launches] == ["expert_gate_up_b128_4", "activation_quantize_128_entry", "expert_down_b128_2",
                                                             "expert_row_sum_entry"]
    assert [list(l.grid) for l in launches] == [[64, 64, 1], [2, 64, 1], [128, 64, 1], [2, 8, 1]]  # the quantizer: 1,024 values a block
    untouched = amd.launches_of(4)
    for changes in (dict(gate_up_shape=amd.Shape(2048 + 64, 4096, 8, 0)), dict(down_shape=amd.Shape(4096, 2048 + 64, 8, 0))):  # whole blocks of 128
        assert lib.linear_routed_experts_prepare(C.byref(experts_description(B128, **changes)), ARENA, C.byref(linear), untouched) == 1, changes
        assert not any(bytes(untouched))
    quantize = amd.QuantizeDescription(amd.Range(4096, 8 * 4096 * 2), amd.Range(1 << 20, 8 * 4096), amd.Range(2 << 20, 8 * 128), amd.Range(0, 0), 4096, 8)
    one = amd.launches_of(1)
    assert lib.linear_quantize_128_prepare(C.byref(quantize), ARENA, C.byref(linear), one) == 0
    assert fake.handles[one[0].kernel][1] == "activation_quantize_128_entry" and list(one[0].grid) == [4, 8, 1] and one[0].block[0] == 256
    quantize.width = 4096 + 64
    assert lib.linear_quantize_128_prepare(C.byref(quantize), ARENA, C.byref(linear), one) == 1
    # the wide form: four launches, from a prepare of its own; each prepare refuses the other's formats
    four = amd.launches_of(4)
    description = wide_experts_description(B128)
    assert lib.linear_wide_experts_block128_prepare(C.byref(description), arena, C.byref(linear), C.byref(wide_kernels), four) == 0
    assert [fake.handles[l.kernel][1] for l in four] == ["wide_expert_gate_up_b128_1", "activation_quantize_128_entry", "wide_expert_down_b128_1",
                                                         "expert_row_sum_entry"]
    tiles = 1024 * 8 // 64 + 256
    assert [list(l.grid) for l in four] == [[32, tiles, 1], [2, 8192, 1], [32, tiles, 1], [2, 1024, 1]]
    assert [l.dynamic_shared_byte_count for l in four] == [53760, 0, 51712, 0]
    quantizer = bytes(four[1].argument)[:40]
    assert int.from_bytes(quantizer[0:8], "little") == description.experts.hidden_operands.byte_offset  # the values the gate/up launch left
    assert int.from_bytes(quantizer[8:16], "little") == description.experts.hidden_codes.byte_offset
    three = amd.launches_of(4)
    assert lib.linear_wide_experts_prepare(C.byref(description), arena, C.byref(linear), C.byref(wide_kernels), three) == 1
    assert lib.linear_wide_experts_block128_prepare(C.byref(wide_experts_description(amd.WEIGHT_FORMAT_E4M3_SCALED)), arena, C.byref(linear),
                                                    C.byref(wide_kernels), three) == 1
    assert not any(bytes(three))


def test_gfx950_formats_prepare_geometry_and_refusals(fake):
    """The formats in gfx950's lane order (7, 8, 9): the job-table launches by the expert_*_gfx950_<S> kernels on the
    reference formats' grids, the wide form by linear_native_experts_prepare alone, the producer refused."""
    lib = amd.library()
    arena = 8 << 30
    linear, wide_kernels, native = amd.LinearKernels(), amd.LinearWideKernels(), amd.LinearNativeKernels()
    assert lib.linear_kernels_prepare(fake.address, fake.card, 950, C.byref(linear)) == 0
    assert lib.linear_wide_kernels_prepare(fake.address, fake.card, 950, C.byref(wide_kernels)) == 0
    assert lib.linear_native_kernels_prepare(fake.address, fake.card, 950, C.byref(native)) == 0
    assert fake.handles[linear.expert_gate_up_gfx950[0]][1] == "expert_gate_up_gfx950_1"
    assert fake.handles[linear.expert_down_e4m3_gfx950[3]][1] == "expert_down_e4m3_gfx950_8" and linear.expert_gate_up_gfx950[4] == amd.BACKEND_NO_KERNEL
    assert fake.handles[native.native_expert_gate_up][1] == "native_expert_gate_up_1" and fake.handles[native.native_expert_down_e4m3][1] == "native_expert_down_e4m3_1"
    assert fake.handles[linear.expert_gate_up_b128_gfx950[1]][1] == "expert_gate_up_b128_gfx950_2" and fake.handles[native.native_expert_down_b128][1] == "native_expert_down_b128_1"
    for fmt, like, names in ((amd.WEIGHT_FORMAT_E2M1_GFX950, amd.WEIGHT_FORMAT_E2M1_SCALED, ["expert_gate_up_gfx950_4", "expert_down_gfx950_2"]),
                             (amd.WEIGHT_FORMAT_E4M3_GFX950, amd.WEIGHT_FORMAT_E4M3_SCALED, ["expert_gate_up_e4m3_gfx950_4", "expert_down_e4m3_gfx950_2"]),
                             (amd.WEIGHT_FORMAT_E4M3_BLOCK128_GFX950, amd.WEIGHT_FORMAT_E4M3_BLOCK128, ["expert_gate_up_b128_gfx950_4", "expert_down_b128_gfx950_2"])):
        block128 = fmt == amd.WEIGHT_FORMAT_E4M3_BLOCK128_GFX950
        launches, reference = amd.launches_of(4), amd.launches_of(4)
        assert lib.linear_routed_experts_prepare(C.byref(experts_description(fmt)), ARENA, C.byref(linear), launches) == 0
        assert lib.linear_routed_experts_prepare(C.byref(experts_description(like)), ARENA, C.byref(linear), reference) == 0
        assert [fake.handles[launches[i].kernel][1] for i in (0, 2)] == names
        assert fake.handles[launches[1].kernel][1] == ("activation_quantize_128_entry" if block128 else "activation_quantize_entry")
        assert fake.handles[launches[3].kernel][1] == "expert_row_sum_entry"
        for ours, theirs in zip(launches, reference):  # the grids, blocks and records of the reference format's launches
            assert list(ours.grid) == list(theirs.grid) and list(ours.block) == list(theirs.block)
            assert bytes(ours.argument) == bytes(theirs.argument)
        # the wide form: its own prepare takes these formats, the reference formats' prepare does not, and the other way round
        three, untouched = amd.launches_of(4), amd.launches_of(4)
        description = wide_experts_description(fmt)
        assert lib.linear_native_experts_prepare(C.byref(description), arena, C.byref(linear), C.byref(native), three) == 0
        assert fake.handles[three[0].kernel][1].startswith("native_expert_gate_up") and fake.handles[three[3 if block128 else 2].kernel][1] == "expert_row_sum_entry"
        if block128:  # the hidden values' quantizer is a launch of its own, as in the E4M3_BLOCK128 wide form
            assert [fake.handles[three[i].kernel][1] for i in (0, 1, 2)] == ["native_expert_gate_up_b128_1", "activation_quantize_128_entry", "native_expert_down_b128_1"]
        else:
            assert not any(bytes(three[3]))
        assert three[0].dynamic_shared_byte_count > 0 and three[0].block[0] == 256
        assert lib.linear_wide_experts_prepare(C.byref(description), arena, C.byref(linear), C.byref(wide_kernels), untouched) == 1
        assert lib.linear_wide_experts_block128_prepare(C.byref(description), arena, C.byref(linear), C.byref(wide_kernels), untouched) == 1
        assert lib.linear_native_experts_prepare(C.byref(wide_experts_description(like)), arena, C.byref(linear), C.byref(native), untouched) == 1
        assert not any(bytes(untouched))
    # E2M1_GFX950 stores whole groups of four tiles: outputs in whole 64
    odd = amd.launches_of(4)
    assert lib.linear_routed_experts_prepare(C.byref(experts_description(amd.WEIGHT_FORMAT_E2M1_GFX950, gate_up_shape=amd.Shape(2048 + 32, 4096, 4, 0),
                                                                         down_shape=amd.Shape(4096, 2048 + 32, 4, 0))), ARENA, C.byref(linear), odd) == 1
    assert not any(bytes(odd))
    # the producer is built for the reference's two formats
    fused = amd.ExpertFusedKernels()
    assert lib.expert_fused_kernels_prepare(fake.address, fake.card, 950, C.byref(fused)) == 0
    one = amd.launches_of(1)
    for fmt in (amd.WEIGHT_FORMAT_E2M1_GFX950, amd.WEIGHT_FORMAT_E4M3_GFX950, amd.WEIGHT_FORMAT_E4M3_BLOCK128, amd.WEIGHT_FORMAT_E4M3_BLOCK128_GFX950):
        d = experts_description(fmt)
        arrivals = amd.Range(6 << 30, 64 * (2048 // 32) * 4)
        assert lib.expert_producer_prepare(C.byref(d), arrivals, arena, C.byref(linear), C.byref(fused), one) == 1, fmt
        assert not any(bytes(one))
    assert lib.expert_producer_prepare(C.byref(experts_description()), amd.Range(6 << 30, 64 * (2048 // 32) * 4), arena, C.byref(linear), C.byref(fused), one) == 0


def site_description(rows=8, width=4096, combined=True, **changes):
    d = amd.HyperSiteDescription()
    at, w = 1 << 20, width if width != 0 else 5120
    sizes = {"streams": rows * 4 * w * 2, "carried_pre": rows * 16, "mixes": rows * 96, "scale": 12, "base": 96, "norm_weight": w * 2,
             "post": rows * 16, "comb": rows * 64, "hidden": rows * w * 2, "output": rows * w * 2, "routed_sums": rows * w * 4}
    for name, size in sizes.items():
        setattr(d, name, amd.Range(at, size))
        at += (size + 255) // 256 * 256
    if not combined:
        d.routed_sums = amd.Range(0, 0)
    d.row_count, d.reserved_zero = rows, width
    for key, value in changes.items():
        setattr(d, key, value)
    return d


def dense_description(outputs=24, inputs=16384, rows=8, weight_type=1, output_type=1, flags=1, **changes):
    d = amd.DenseLinearDescription()
    d.weights = amd.Range(1 << 20, outputs * inputs * (4 if weight_type == 1 else 2))
    d.rows = amd.Range(1 << 28, rows * inputs * 2)
    d.output = amd.Range(1 << 29, rows * outputs * (4 if output_type == 1 else 2))
    d.output_size, d.input_size, d.row_count, d.weight_type, d.output_type, d.flags = outputs, inputs, rows, weight_type, output_type, flags
    d.output_scale, d.epsilon = 1.0, 1e-20
    for key, value in changes.items():
        setattr(d, key, value)
    return d


def test_site_front_launches_geometry_and_refusals(fake):
    """The dense product and the hyper site: the reference's entry points (include/anemone/dense_linear.h:70-99,
    include/anemone/hyper_connection.h:40-71), instances, geometry and refusals."""
    lib = amd.library()
    arena = 8 << 30
    dense, hyper = amd.DenseLinearKernels(), amd.HyperKernelsRecord()
    assert lib.dense_linear_kernels_prepare(fake.address, fake.card, C.byref(dense)) == 0
    assert lib.hyper_kernels_prepare(fake.address, fake.card, C.byref(hyper)) == 0
    names = [fake.handles[handle][1] for handle in dense.products]
    assert names == ["dense_linear_bfloat16_1", "dense_linear_bfloat16_8", "dense_linear_float32_1", "dense_linear_float32_8",
                     "dense_linear_bfloat16_1_narrow", "dense_linear_bfloat16_8_narrow", "dense_linear_float32_1_narrow", "dense_linear_float32_8_narrow"]
    assert fake.handles[hyper.mix_finish] == ("kernel_hyper_connection", "hyper_mix_finish") and fake.handles[hyper.post][1] == "hyper_post_entry"
    assert hyper.final_collapse == hyper.embed == hyper.draft_inputs == hyper.final_kept == amd.BACKEND_NO_KERNEL
    table = kernel_table()
    assert table[("kernel_dense_linear", "dense_linear_float32_8_narrow")] == 64 and table[("kernel_hyper_connection", "hyper_mix_finish")] == 72
    launch = amd.launches_of(1)
    # the mix project: 24 outputs are fewer than 256 blocks of four: the narrow form, a block an output
    assert lib.dense_linear_prepare(C.byref(dense_description()), arena, C.byref(dense), launch) == 0
    assert fake.handles[launch[0].kernel][1] == "dense_linear_float32_1_narrow" and list(launch[0].grid) == [24, 8, 1] and launch[0].block[0] == 256
    scores = dense_description(outputs=256, inputs=4096, weight_type=0, flags=0)  # the router's: too many blocks for a block a row
    assert lib.dense_linear_prepare(C.byref(scores), arena, C.byref(dense), launch) == 0
    assert fake.handles[launch[0].kernel][1] == "dense_linear_bfloat16_8_narrow" and list(launch[0].grid) == [256, 1, 1]
    assert lib.dense_linear_prepare(C.byref(dense_description()), arena, C.byref(dense), launch) == 0
    assert launch[0].argument_byte_count == 64
    one = dense_description(outputs=4096, inputs=2048, rows=1, weight_type=0, output_type=0, flags=0)
    assert lib.dense_linear_prepare(C.byref(one), arena, C.byref(dense), launch) == 0
    assert fake.handles[launch[0].kernel][1] == "dense_linear_bfloat16_1" and list(launch[0].grid) == [1024, 1, 1]
    # more rows: groups of 8 on grid[1], 8 outputs a block where they divide
    many = dense_description(rows=8192)
    assert lib.dense_linear_prepare(C.byref(many), arena, C.byref(dense), launch) == 0
    assert fake.handles[launch[0].kernel][1] == "dense_linear_float32_8_wide" and list(launch[0].grid) == [3, 1024, 1]
    odd = dense_description(outputs=20, rows=370)
    assert lib.dense_linear_prepare(C.byref(odd), arena, C.byref(dense), launch) == 0
    assert fake.handles[launch[0].kernel][1] == "dense_linear_float32_8" and list(launch[0].grid) == [5, 47, 1]
    middling = dense_description(rows=32)  # few outputs, some rows: still a block a row and an output
    assert lib.dense_linear_prepare(C.byref(middling), arena, C.byref(dense), launch) == 0
    assert fake.handles[launch[0].kernel][1] == "dense_linear_float32_1_narrow" and list(launch[0].grid) == [24, 32, 1]
    untouched = amd.launches_of(1)
    for changes, status in [(dict(row_count=0), 1), (dict(row_count=600000), 1), (dict(flags=3), 7), (dict(flags=8), 1), (dict(weight_type=2), 1),
                            (dict(output_size=26), 1), (dict(input_size=16388), 1), (dict(cone_layer=1), 7),
                            (dict(weights=amd.Range(1 << 20, 24 * 16384 * 4 + 16)), 1), (dict(output=amd.Range((1 << 20) + 256, 1024)), 1)]:
        assert lib.dense_linear_prepare(C.byref(dense_description(**changes)), arena, C.byref(dense), untouched) == status, changes
        assert not any(bytes(untouched))
    # a site: the mix finish and the post
    launches = amd.launches_of(2)
    d = site_description()
    assert lib.hyper_site_prepare(C.byref(d), arena, C.byref(hyper), launches) == 0
    assert [fake.handles[l.kernel][1] for l in launches] == ["hyper_mix_finish", "hyper_post_entry"]
    assert list(launches[0].grid) == [1, 8, 1] and launches[0].block[0] == 512 and launches[0].argument_byte_count == 72
    assert list(launches[1].grid) == [4, 8, 1] and launches[1].block[0] == 128 and launches[1].argument_byte_count == 48
    import struct
    finish = struct.unpack("<9Q", bytes(launches[0].argument)[:72])
    assert finish == tuple(getattr(d, name).byte_offset for name in ("streams", "carried_pre", "mixes", "scale", "base", "post", "comb", "norm_weight", "hidden"))
    post = struct.unpack("<5QII", bytes(launches[1].argument)[:48])
    assert post == (d.streams.byte_offset, d.post.byte_offset, d.comb.byte_offset, d.output.byte_offset, d.routed_sums.byte_offset, 1, 0)
    plain = site_description(combined=False, width=0, rows=3)  # the attention site's post; the reference's width
    assert lib.hyper_site_prepare(C.byref(plain), arena, C.byref(hyper), launches) == 0
    assert launches[0].block[0] == 640 and list(launches[1].grid) == [5, 3, 1]
    assert struct.unpack("<5QII", bytes(launches[1].argument)[:48])[4:] == (0, 0, 0)
    chunk = site_description(rows=2048)
    assert lib.hyper_site_prepare(C.byref(chunk), arena, C.byref(hyper), launches) == 0
    assert list(launches[0].grid) == [1, 2048, 1] and list(launches[1].grid) == [4, 2048, 1]
    untouched = amd.launches_of(2)
    for changes in (dict(row_count=0), dict(row_count=70000), dict(reserved_zero=4100), dict(reserved_zero=9216), dict(scale=amd.Range(1 << 30, 16)),
                    dict(mixes=amd.Range((1 << 20) + 64, 1024)), dict(hidden=amd.Range((8 << 30) - 256, 8 * 4096 * 2))):
        assert lib.hyper_site_prepare(C.byref(site_description(**changes)), arena, C.byref(hyper), untouched) == 1, changes
        assert not any(bytes(untouched))



def test_the_build_refuses_a_spilling_kernel_of_hand_issued_loads():
    """anemone_amd/build.py reads the compiler's resource remarks of the kernels whose loads the compiler keeps no book on
    (csrc/native_device.cuh) and names those that spill a vector register."""
    from anemone_amd import build
    remark = "/x/kernel_native_linear.hip:%d:1: remark: %s [-Rpass-analysis=kernel-resource-usage]"
    lines = []
    for at, (name, sgprs, vgprs) in enumerate([("native_expert_gate_up_1", 0, 0), ("native_expert_down_b128_1", 3, 14), ("native_expert_down_1", 9, 0)]):
        lines += [remark % (at, "Function Name: " + name), remark % (at, "    VGPRs: 168"), remark % (at, "    ScratchSize [bytes/lane]: %d" % (4 * vgprs)),
                  remark % (at, "    SGPRs Spill: %d" % sgprs), remark % (at, "    VGPRs Spill: %d" % vgprs)]
    assert build.spilling_kernels("\n".join(lines + ["warning: something else"])) == [("native_expert_down_b128_1", 14)]
    assert build.spilling_kernels("") == []
    assert "kernel_native_linear.hip" in build.NO_SPILL_SOURCES and set(build.NO_SPILL_SOURCES) <= set(build.HIP_SOURCES)
