"""The check of an EXL3 map's descriptor (include/anemone_descriptor.h, anemone_amd/host/exl3_descriptor.c) on the CPU,
through the C ABI, against the cases the reference's own test holds (tests/exl3_descriptor_test.c of the reference: its
table of one-rule-broken descriptors :95-186 and its scenarios :416-900): the same model geometry (40 layers of 384
experts, hidden 5120, intermediate 2304, layers 18 to 22 K2 and the others K3), the descriptor written member by member as
the converter writes it, one text replaced a case, and the STATUS each case must give. The lines' wording is this
library's own, so a case checks the status and that its one line names the sidecar and the field (or the thing) at fault.
The pack is a view of tensor records built here (the pack reader itself is outside this library). Also: SHA-256 against
hashlib, the JSON reader's grammar against Python's json module through members the check does not bind."""
import ctypes as C
import hashlib
import json
import os

import numpy as np
import pytest

import anemone_amd as amd

OK, INVALID, NO_MEMORY, IO_ERROR, UNSUPPORTED = 0, 1, 2, 3, 7
LAYERS, EXPERTS, HIDDEN, INNER = 40, 384, 5120, 2304
K2_LAYERS = range(18, 23)
KINDS = (("w1", INNER, HIDDEN), ("w2", HIDDEN, INNER), ("w3", INNER, HIDDEN))
SOME_DIGEST = "0123456789abcdef" * 4
TABLES = b"the front end's tables"
ESTABLISHED = '{"status": "established", "reference": "TP4_EXL3\'s default route, qualified by identity"}'
HEADER_DIGEST, FILE_BYTES, TABLES_BYTES, TABLES_DIGEST = 0x1234567890ABCDEF, 98765 * 4096, 3 * 4096, 0x0FEDCBA987654321
EXL3 = 2


def layer_width(layer):
    return "K2" if layer in K2_LAYERS else "K3"


def stored_width(name):
    whole, _, half = name[1:].partition(".")
    return int(whole) * 16 + 8 if half else int(whole)


class Pack:
    """A view of tensor records sorted by name as the pack file sorts them."""

    def __init__(self, layers=LAYERS, experts=EXPERTS, mixed_layer=None, extra=(), header_digest=HEADER_DIGEST, file_bytes=FILE_BYTES, shuffle=False):
        entries = []
        for layer in range(layers):
            for expert in range(experts):
                for kind, outputs, inputs in KINDS:
                    width = "K2" if (layer == mixed_layer and kind == "w2" and expert == 0) else layer_width(layer)
                    entries.append(("layers.%d.ffn.experts.%d.%s.weight" % (layer, expert, kind), EXL3, (outputs, inputs), stored_width(width)))
        entries += list(extra)
        entries.sort(key=lambda entry: entry[0].encode())
        if shuffle:
            entries[0], entries[-1] = entries[-1], entries[0]
        self.records = np.zeros(len(entries), dtype=amd.PACK_TENSOR_DTYPE)
        names = bytearray()
        for record, (name, weight_format, dimensions, bits) in zip(self.records, entries):
            record["name_byte_offset"], record["name_byte_count"] = len(names), len(name)
            names += name.encode()
            record["dimension_count"] = len(dimensions)
            record["dimensions"][:len(dimensions)] = dimensions
            record["weight_format"], record["bits_per_weight"], record["element_type"] = weight_format, bits, 4
        self.names = np.frombuffer(bytes(names), dtype=np.uint8).copy()
        self.view = amd.Exl3PackView(header_digest, file_bytes, self.records.ctypes.data, self.names.ctypes.data, len(entries), len(names))


def model_of(layers=LAYERS, established=(), **changes):
    m = amd.Exl3DescriptorModel()
    m.model_type, m.layers, m.experts_per_layer, m.hidden, m.intermediate = b"deepseek_v41", layers, EXPERTS, HIDDEN, INNER
    for k, (kind, outputs, inputs) in enumerate(KINDS):
        m.matrices[k] = amd.Exl3DescriptorMatrix(kind.encode(), outputs, inputs)
    m.routes_per_row, m.cone_first_layer = 6, 0
    if established:
        m._keep = (amd.Exl3EstablishedPack * len(established))(*[amd.Exl3EstablishedPack(n.encode(), d, b) for n, d, b in established])
        m.established, m.established_count = m._keep, len(established)
    for key, value in changes.items():
        setattr(m, key, value)
    return m


def descriptor(layers=LAYERS, mixed_layer=None, tables_digest="null", quality=ESTABLISHED, widths=None):
    """The descriptor as the converter writes it, member by member (the text the reference's test writes:
    tests/exl3_descriptor_test.c:222-296)."""
    text = ('{\n "format_version": 1,\n "map": {"file": "map.exl3map", "sha256": "%s", "manifest_bytes": %d, "logical_bytes": %d, '
            '"pack_header_digest": %d, "native_pack_header_digest": %d},\n' % (SOME_DIGEST, TABLES_BYTES, FILE_BYTES, HEADER_DIGEST, TABLES_DIGEST))
    text += (' "architecture": {"model_type": "deepseek_v41", "architectures": ["DeepseekV41ForCausalLM"], "config_sha256": "%s"},\n'
             ' "quantiser": {"source": "test @ 0", "index_sha256": "%s", "quantization_config_sha256": "%s"},\n'
             ' "codebook": {"mul1_multiplier": "0x83DCD12D"},\n "front_end_tables_sha256": %s,\n' % (SOME_DIGEST, SOME_DIGEST, SOME_DIGEST, tables_digest))
    text += (' "experts": {"layers": %d, "experts_per_layer": %d, "hidden": %d, "intermediate": %d, "matrices": {"w1": [%d, %d], "w2": [%d, %d], '
             '"w3": [%d, %d]}},\n "widths": ' % (layers, EXPERTS, HIDDEN, INNER, INNER, HIDDEN, HIDDEN, INNER, INNER, HIDDEN))
    k2_matrices = k2_layers = k3_layers = 0
    parts = []
    for layer in range(layers):
        kinds = []
        for kind, _, _ in KINDS:
            if layer == mixed_layer and kind == "w2":
                kinds.append('"%s": {"%s": %d, "K2": 1}' % (kind, layer_width(layer), EXPERTS - 1))
            else:
                kinds.append('"%s": {"%s": %d}' % (kind, layer_width(layer), EXPERTS))
        parts.append('"%d": {%s}' % (layer, ", ".join(kinds)))
        is_k2 = layer in K2_LAYERS
        k2_matrices += EXPERTS * 3 if is_k2 else 0
        k2_layers += 1 if is_k2 else 0
        k3_layers += 1 if not is_k2 and layer != mixed_layer else 0
    mixed = 1 if mixed_layer is not None and mixed_layer < layers else 0
    text += widths if widths is not None else "{" + ", ".join(parts) + "}"
    text += (',\n "widths_summary": {"matrices": {"K2": %d, "K3": %d}, "layers": {"K2": %d, "K3": %d%s}},\n "quality": %s\n}\n'
             % (k2_matrices + mixed, layers * EXPERTS * 3 - k2_matrices - mixed, k2_layers, k3_layers, ', "mixed": 1' if mixed else "", quality))
    return text


@pytest.fixture(scope="module")
def pack():
    return Pack()


@pytest.fixture()
def place(tmp_path):
    folder = tmp_path / "maps"
    folder.mkdir()
    map_path = folder / "map.exl3map"
    map_path.write_bytes(b"a map")
    return folder, str(map_path), str(map_path) + ".descriptor.json"


def checked(capfd, map_path, pack, model, tables=TABLES, admits=False):
    capfd.readouterr()
    status = amd.library().exl3_descriptor_check(map_path.encode() if isinstance(map_path, str) else map_path, C.byref(pack.view), C.byref(model), tables,
                                                 len(tables) if tables is not None else 0, admits)
    return status, capfd.readouterr().err


def expect(capfd, place, pack, text, status, *words, model=None, tables=TABLES, admits=False, map_path=None):
    _, default_map, sidecar = place
    if text is not None:
        with open(sidecar, "wb") as out:
            out.write(text if isinstance(text, bytes) else text.encode())
    got, log = checked(capfd, map_path or default_map, pack, model or model_of(), tables, admits)
    assert got == status, (got, status, log)
    lines = [line for line in log.splitlines() if line]
    assert len(lines) == 1, log  # one line a check, refused or served
    if map_path is None:
        assert os.path.realpath(default_map) + ".descriptor.json" in lines[0], log
    for word in words:
        assert word in lines[0], (word, log)
    return lines[0]


TABLES_HEX = '"%s"' % hashlib.sha256(TABLES).hexdigest()

# (the first `old` of the descriptor becomes `new`, the status, what the line names): tests/exl3_descriptor_test.c:95-186
REFUSALS = [
    ('"format_version": 1', '"format_version": 2', UNSUPPORTED, ["format_version", "2"]),
    ('"format_version": 1,', '', INVALID, ["format_version"]),
    ('{', '[', INVALID, ["JSON object"]),
    ('"map": {', '"map": {"file": "twice", ', INVALID, ["twice"]),
    ('"codebook": {', '"codebook": {"other": 1, ', INVALID, ["codebook", '"other"']),
    ('"native_pack_header_digest"', '"native_header_digest"', INVALID, ["map", '"native_header_digest"']),
    ('"quantiser": {"source": "test @ 0", ', '"quantiser": {', INVALID, ["quantiser", "source"]),
    ('"source": "test @ 0"', '"source": " \\t"', INVALID, ["quantiser.source", '" \\t"']),
    ('"model_type": "deepseek_v41"', '"model_type": "deepseek_v4"', UNSUPPORTED, ["architecture.model_type", '"deepseek_v4"', '"deepseek_v41"']),
    ('"model_type": "deepseek_v41"', '"model_type": null', UNSUPPORTED, ["architecture.model_type", "null"]),
    ('"0x83DCD12D"', '"0x83DCD12E"', UNSUPPORTED, ["codebook.mul1_multiplier", '"0x83DCD12E"', '"0x83DCD12D"']),
    ('"layers": 40', '"layers": 41', INVALID, ["experts.layers", "41", "40"]),
    ('"layers": 40', '"layers": "40"', INVALID, ["experts.layers", '"40"', "whole number"]),
    ('"experts_per_layer": 384', '"experts_per_layer": 256', INVALID, ["experts.experts_per_layer", "256", "384"]),
    ('"hidden": 5120', '"hidden": 4096', INVALID, ["experts.hidden", "4096", "5120"]),
    ('"intermediate": 2304', '"intermediate": 2048', INVALID, ["experts.intermediate", "2048", "2304"]),
    ('"w2": [5120, 2304]', '"w2": [2304, 5120]', INVALID, ["experts.matrices.w2", "2304", "5120"]),
    ('"w2": [5120, 2304]', '"w2": [5120, 2304, 1]', INVALID, ["experts.matrices.w2", "[outputs, inputs]"]),
    ('"w2": [5120, 2304]', '"w2": [5120]', INVALID, ["experts.matrices.w2", "[outputs, inputs]"]),
    ('"0": {"w1": {"K3": 384}', '"0": {"w1": {"K3": 383}', INVALID, ["widths.0.w1", "383", "K3", "384"]),
    ('"0": {"w1": {"K3": 384}', '"0": {"w1": {"K2": 384}', INVALID, ["widths.0.w1", "384", "K2", " 0"]),
    ('"0": {"w1": {"K3": 384}', '"0": {"w1": {"K9": 384}', INVALID, ["widths.0.w1", '"K9"', "width"]),
    ('"0": {"w1": {"K3": 384}', '"0": {"w1": {"K3": 0}', INVALID, ["widths.0.w1.K3", "0"]),
    ('"0": {', '"00": {', INVALID, ["widths", '"00"', "0 to 39"]),
    ('"39": {', '"40": {', INVALID, ["widths", '"40"', "0 to 39"]),
    ('"w2": {"K3"', '"w4": {"K3"', INVALID, ["widths.0", '"w4"']),
    ('"matrices": {"K2": 5760', '"matrices": {"K2": 5761', INVALID, ["widths_summary.matrices", "5761", "K2", "5760"]),
    ('"matrices": {"K2"', '"matrices": {"mixed": 1, "K2"', INVALID, ["widths_summary.matrices", "1 of mixed", " 0"]),
    ('"layers": {"K2": 5', '"layers": {"K2": 5, "mixed": 1', INVALID, ["widths_summary.layers", "1 of mixed", " 0"]),
    ('"codebook": {"mul1_multiplier": "0x83DCD12D"}', '"codebook": "0x83DCD12D"', INVALID, ["codebook", '"0x83DCD12D"', "object"]),
    ('"format_version": 1,', '"format_version": 1, "extra": 1,', INVALID, ["the descriptor", '"extra"']),
    ('{"w1": {"K3": 384}', '{"w1": 384', INVALID, ["widths.0.w1", "384", "object"]),
    ('"w2": [5120, 2304]', '"w2": 5120', INVALID, ["experts.matrices.w2", "[outputs, inputs]"]),
    ('"status": "established"', '"status": "measured"', UNSUPPORTED, ["quality.status", '"measured"', "established"]),
    ('"quality": {"status": "established", ', '"quality": {', INVALID, ["quality", "status"]),
    ('"reference": "TP4_EXL3', '"reference": "", "was": "TP4_EXL3', INVALID, ["quality", '"was"']),
]


@pytest.mark.parametrize("old,new,status,words", REFUSALS, ids=[str(i) for i in range(len(REFUSALS))])
def test_one_rule_broken(capfd, place, pack, old, new, status, words):
    text = descriptor(tables_digest=TABLES_HEX)
    assert old in text
    expect(capfd, place, pack, text.replace(old, new, 1), status, *words)


def test_the_descriptor_as_written_holds_and_binds_to_the_pack(capfd, place, pack):
    text = descriptor(tables_digest=TABLES_HEX)
    line = expect(capfd, place, pack, text, OK, "deepseek_v41", "test @ 0", "widths K2 5760, K3 40320", "quality established (TP4_EXL3's default route")
    assert hashlib.sha256(text.encode()).hexdigest() in line  # the sidecar's own digest is on the line
    json.loads(text)
    # the binding to the open pack: its size and its header digest
    expect(capfd, place, pack, text.replace('"logical_bytes": %d' % FILE_BYTES, '"logical_bytes": %d' % (FILE_BYTES + 4096)), INVALID, "map.logical_bytes")
    expect(capfd, place, pack, text.replace('"pack_header_digest": %d' % HEADER_DIGEST, '"pack_header_digest": %d' % (HEADER_DIGEST ^ 1)), INVALID,
           "map.pack_header_digest")
    # the tables: another digest is refused where the tables were read, and not looked at where they were not
    other = descriptor(tables_digest='"%s"' % SOME_DIGEST)
    expect(capfd, place, pack, other, INVALID, "front_end_tables_sha256", SOME_DIGEST, hashlib.sha256(TABLES).hexdigest())
    expect(capfd, place, pack, other, OK, "quality established", tables=None)
    expect(capfd, place, pack, descriptor(tables_digest="null"), OK, "quality established")
    # a layer short; a model of a layer less (the pack then holds EXL3 matrices no routed expert has); widths no object
    short = descriptor(layers=LAYERS - 1, tables_digest=TABLES_HEX).replace('"layers": %d' % (LAYERS - 1), '"layers": %d' % LAYERS)
    expect(capfd, place, pack, short, INVALID, "widths", "39", "40")
    expect(capfd, place, pack, descriptor(layers=LAYERS - 1, tables_digest=TABLES_HEX), INVALID, "46080", "44928", model=model_of(layers=LAYERS - 1))
    expect(capfd, place, pack, descriptor(tables_digest=TABLES_HEX, widths="[]"), INVALID, "widths", "object")
    # architectures is not bound: null is as good
    expect(capfd, place, pack, descriptor().replace('["DeepseekV41ForCausalLM"]', "null"), OK, "quality established", tables=None)


def test_quality(capfd, place, pack):
    folder, map_path, _ = place
    capture = folder / "capture.json"
    capture_bytes = b'{"nll": [], "scope": "test"}\n'
    capture.write_bytes(capture_bytes)
    digest = hashlib.sha256(capture_bytes).hexdigest()
    link = folder / "linked.exl3map"
    os.symlink(map_path, link)
    expect(capfd, place, pack, descriptor(), OK, "quality established")
    expect(capfd, place, pack, None, OK, "quality established", map_path=str(link))  # through a link: the sidecar is beside the map it leads to
    none = descriptor(quality='{"status": "none"}')
    expect(capfd, place, pack, none, UNSUPPORTED, "quality", '"none"', amd_opt_in(), map_path_word(map_path))
    expect(capfd, place, pack, none, OK, "quality none (%s: no quality claim)" % amd_opt_in(), admits=True)
    line = expect(capfd, place, pack, none, OK, admits=True, tables=None)
    assert line.endswith("model deepseek_v41, quantiser test @ 0, widths K2 5760, K3 40320, quality none (%s: no quality claim)" % amd_opt_in())
    expect(capfd, place, pack, descriptor(quality='{"status": "none", "reference": "x"}'), INVALID, "quality", '"reference"', admits=True)
    expect(capfd, place, pack, descriptor(quality='{"status": "established", "reference": ""}'), INVALID, "quality.reference", '""', "text")
    expect(capfd, place, pack, descriptor(quality='{"status": "established", "reference": " \\n "}'), INVALID, "quality.reference", '" \\n "', "text")
    expect(capfd, place, pack, descriptor(quality='{"status": "established", "reference": "a\\u0000b"}'), INVALID, "quality.reference", "text")
    expect(capfd, place, pack, descriptor(quality='"none"'), INVALID, "quality", '"none"', "object", admits=True)
    recorded = '{"status": "recorded", "record": "%s", "sha256": "%s"}'
    expect(capfd, place, pack, descriptor(quality=recorded % (capture, digest)), OK, "quality recorded (%s)" % capture)
    expect(capfd, place, pack, descriptor(quality=recorded % (capture, SOME_DIGEST)), INVALID, "quality.sha256", SOME_DIGEST, digest)
    expect(capfd, place, pack, descriptor(quality=recorded % (str(capture) + ".missing", digest)), IO_ERROR, ".missing", "No such file or directory")
    expect(capfd, place, pack, descriptor(quality=recorded % (capture, "xyz")), INVALID, "quality.sha256", '"xyz"')
    expect(capfd, place, pack, descriptor(quality='{"status": "recorded", "record": "%s"}' % capture), INVALID, "quality", "sha256")
    expect(capfd, place, pack, descriptor(quality=recorded % ("capture.json", digest)), INVALID, "quality.record", '"capture.json"', "absolute path")
    expect(capfd, place, pack, descriptor(quality=recorded % (folder, digest)), INVALID, "quality.record", "regular file")
    big = folder / "big.bin"  # a capture of more than one piece of the hash
    big.write_bytes(bytes(range(256)) * 9000)
    expect(capfd, place, pack, descriptor(quality=recorded % (big, hashlib.sha256(big.read_bytes()).hexdigest())), OK, "quality recorded")


def amd_opt_in():
    return "--exl3_unrated_map=1"


def map_path_word(map_path):
    return os.path.realpath(map_path)


def test_what_lies_at_the_sidecars_place(capfd, place, pack):
    folder, map_path, sidecar = place
    status, log = checked(capfd, "/" + "a" * (4096 - len(".descriptor.json") - 1), pack, model_of())
    assert status == INVALID and "sidecar" in log and len(log.splitlines()) == 1
    os.symlink(str(folder / "missing"), sidecar)
    expect(capfd, place, pack, None, IO_ERROR, "the file", "No such file or directory")
    os.unlink(sidecar)
    os.mkdir(sidecar)
    expect(capfd, place, pack, None, INVALID, "the file", "regular file", "1048576")
    os.rmdir(sidecar)
    expect(capfd, place, pack, b"", INVALID, "JSON object")
    expect(capfd, place, pack, bytes(1048576 + 1), INVALID, "the file", "regular file", "1048576")
    expect(capfd, place, pack, bytes(4096), INVALID, "JSON object")
    padded = descriptor().encode()
    padded += b" " * (1048576 - len(padded))  # exactly the most bytes: read
    expect(capfd, place, pack, padded, OK, "quality established")
    os.unlink(sidecar)
    os.mkfifo(sidecar)  # no regular file, and the open does not wait for a writer
    expect(capfd, place, pack, None, INVALID, "the file", "regular file")


def test_no_descriptor_beside_the_map(capfd, place, pack):
    folder, map_path, sidecar = place
    listed = model_of(established=[("test", HEADER_DIGEST, FILE_BYTES)])
    mismatched = model_of(established=[("another size", HEADER_DIGEST, FILE_BYTES + 4096), ("another digest", HEADER_DIGEST ^ 1, FILE_BYTES)])
    edge = [str(folder / ("m" * n)) for n in (255 - len(".descriptor.json"), 255 - len(".descriptor.json") + 1, 255)]
    for path in [map_path, str(folder / "0123456789abcdef.anemone"), str(folder / "gone" / "map.exl3map")] + edge:
        if os.path.dirname(path) == str(folder) and not os.path.exists(path):
            with open(path, "wb") as out:
                out.write(b"a map")
        for model, admits, status, words in ((listed, False, OK, ["the established pack test", "by default", str(HEADER_DIGEST), str(FILE_BYTES)]),
                                             (model_of(), False, UNSUPPORTED, ["not list", amd_opt_in(), str(HEADER_DIGEST)]),
                                             (model_of(), True, OK, ["not list as established", amd_opt_in()]),
                                             (mismatched, False, UNSUPPORTED, ["not list"])):
            status_got, log = checked(capfd, path, pack, model, admits=admits)
            assert status_got == status and len(log.splitlines()) == 1, (path, log)
            assert os.path.basename(path)[:40] in log and ".descriptor.json" in log
            for word in words:
                assert word in log, (word, log)
    # a descriptor that is there decides, listed or not: none is refused without the opt-in, established is served with its own reference
    expect(capfd, place, pack, descriptor(quality='{"status": "none"}'), UNSUPPORTED, "quality", model=listed)
    expect(capfd, place, pack, descriptor(), OK, "quality established (TP4_EXL3's default route", model=model_of())


def test_a_pack_with_one_matrix_of_another_width(capfd, place):
    mixed = Pack(mixed_layer=0)
    line = expect(capfd, place, mixed, descriptor(mixed_layer=0), OK, "widths K2 5761, K3 40319")
    assert "quality established" in line
    expect(capfd, place, mixed, descriptor(), INVALID, "widths.0.w2", "0 of K2", "the pack holds 1")
    # the summary's layers must say mixed for that layer
    expect(capfd, place, mixed, descriptor(mixed_layer=0).replace(', "mixed": 1', "").replace('"layers": {"K2": 5, "K3": 34', '"layers": {"K2": 5, "K3": 35'),
           INVALID, "widths_summary.layers")


def test_what_the_pack_holds(capfd, place):
    text = descriptor()
    # a matrix of another shape, of another format, of a width that is none; an EXL3 matrix that is no routed expert's
    def with_one(change):
        p = Pack()
        index = int(np.flatnonzero(p.records["name_byte_count"] == len("layers.7.ffn.experts.5.w2.weight"))[0])
        change(p.records[index])
        return p, bytes(p.names[p.records[index]["name_byte_offset"]:][:p.records[index]["name_byte_count"]]).decode()

    def reshape(record):
        record["dimensions"][0] += 128

    def plain(record):
        record["weight_format"] = 3

    def no_width(record):
        record["bits_per_weight"] = 9

    def three(record):
        record["dimension_count"] = 3

    for change in (reshape, plain, no_width, three):
        p, name = with_one(change)
        expect(capfd, place, p, text, INVALID, name, "EXL3 matrix")
    extra = Pack(extra=[("layers.0.attn.wq.weight", EXL3, (HIDDEN, HIDDEN), 3)])
    expect(capfd, place, extra, text, INVALID, "46081", "46080")
    plain_extra = Pack(extra=[("layers.0.attn.wq.weight", 0, (HIDDEN, HIDDEN), 0), ("embed.weight", 0, (1000, HIDDEN), 0)])
    expect(capfd, place, plain_extra, text, OK, "quality established")  # tensors that are no EXL3 matrices are not the descriptor's
    # a half width is counted under its own name
    half = Pack()
    for record in half.records:
        name = bytes(half.names[record["name_byte_offset"]:][:record["name_byte_count"]])
        if name.startswith(b"layers.18."):
            record["bits_per_weight"] = 40  # K2.5
    halves = descriptor().replace('"18": {"w1": {"K2": 384}, "w2": {"K2": 384}, "w3": {"K2": 384}}',
                                  '"18": {"w1": {"K2.5": 384}, "w2": {"K2.5": 384}, "w3": {"K2.5": 384}}')
    halves = halves.replace('"matrices": {"K2": 5760', '"matrices": {"K2": 4608, "K2.5": 1152').replace('"layers": {"K2": 5', '"layers": {"K2": 4, "K2.5": 1')
    expect(capfd, place, half, halves, OK, "widths K2 4608, K2.5 1152, K3 40320")
    # records that are not in the file's order are refused before anything is searched
    status, log = checked(capfd, place[1], Pack(shuffle=True), model_of())
    assert status == INVALID and "sorted" in log


def test_arguments():
    lib = amd.library()
    p, m = Pack(layers=1), model_of(layers=1)
    check = lambda *a: lib.exl3_descriptor_check(*a)
    assert check(None, C.byref(p.view), C.byref(m), None, 0, False) == INVALID
    assert check(b"/tmp/x", None, C.byref(m), None, 0, False) == INVALID
    assert check(b"/tmp/x", C.byref(p.view), None, None, 0, False) == INVALID
    assert check(b"/tmp/x", C.byref(p.view), C.byref(m), None, 5, False) == INVALID  # a byte count without tables
    for broken in (dict(model_type=None), dict(layers=0), dict(experts_per_layer=0), dict(established_count=1)):
        assert check(b"/tmp/x", C.byref(p.view), C.byref(model_of(**{"layers": 1, **broken})), None, 0, False) == INVALID, broken
    no_kind = model_of(layers=1)
    no_kind.matrices[1].kind = None
    assert check(b"/tmp/x", C.byref(p.view), C.byref(no_kind), None, 0, False) == INVALID


def small_descriptor(**members):
    """A descriptor of a model of one layer and two experts, for the reader's cases."""
    text = {
        "format_version": 1,
        "map": {"file": "m", "sha256": SOME_DIGEST, "manifest_bytes": 1, "logical_bytes": FILE_BYTES, "pack_header_digest": HEADER_DIGEST,
                "native_pack_header_digest": 2},
        "architecture": {"model_type": "deepseek_v41", "architectures": [], "config_sha256": SOME_DIGEST},
        "quantiser": {"source": "s", "index_sha256": SOME_DIGEST, "quantization_config_sha256": SOME_DIGEST},
        "codebook": {"mul1_multiplier": "0x83DCD12D"},
        "front_end_tables_sha256": None,
        "experts": {"layers": 1, "experts_per_layer": 2, "hidden": HIDDEN, "intermediate": INNER,
                    "matrices": {"w1": [INNER, HIDDEN], "w2": [HIDDEN, INNER], "w3": [INNER, HIDDEN]}},
        "widths": {"0": {"w1": {"K3": 2}, "w2": {"K3": 2}, "w3": {"K3": 2}}},
        "widths_summary": {"matrices": {"K3": 6}, "layers": {"K3": 1}},
        "quality": {"status": "established", "reference": "r"},
    }
    text.update(members)
    return text


def test_the_readers_grammar_is_json_loads(capfd, place):
    """Members the check does not bind carry the cases: what json.loads reads is read, what it refuses is refused (and
    what makes no UTF-8 text besides, and arrays and objects more than 128 deep: the slot is two objects down)."""
    p = Pack(layers=1, experts=2)
    m = model_of(layers=1, experts_per_layer=2)
    base = json.dumps(small_descriptor())
    expect(capfd, place, p, base, OK, "widths K3 6", model=m)
    # as the converter writes it (tools/convert/make_virtual_pack.py:350 of the reference): json.dumps(descriptor, indent=1) and a line feed
    expect(capfd, place, p, json.dumps(small_descriptor(), indent=1) + "\n", OK, "widths K3 6", model=m)
    expect(capfd, place, p, json.dumps(small_descriptor(), indent=1, ensure_ascii=False, sort_keys=True) + "\n", OK, "widths K3 6", model=m)
    slot = '"architectures": []'
    assert slot in base
    accepted = ['[1, -0, 1.5e+3, -2E-7, 0.0, NaN, Infinity, -Infinity, true, false, null]', '"\\u00e9\\ud83d\\ude00\\"\\\\\\/\\b\\f\\n\\r\\t"', '"é\U0001F600"',
                "[" * 126 + "]" * 126, '{"a": {"b": [{}, [], ""]}}', " [ \t\r\n 1 , 2 ] ", "1" * 4300, "1" * 5000 + ".0", '"\\u0000"']
    refused = ["[1,]", "[1 2]", "{'a': 1}", '{"a" 1}', "01", "1.", ".5", "+1", "1e", "- 1", "nul", "True", "-NaN", '"\\x41"', '"\\u12"', '"\t"', '"a', "[1]]",
               '"\\ud83d"', '"\\ude00"', '"\\ud83d\\u0041"', "[" * 127 + "]" * 127, "1" * 4301, "[1] 2", "\v1", ""]
    for value in accepted:
        text = base.replace(slot, '"architectures": ' + value)
        json.loads(text)
        expect(capfd, place, p, text, OK, "widths K3 6", model=m)
    reader_only = ('"\\ud83d"', '"\\ude00"', '"\\ud83d\\u0041"', "[" * 127 + "]" * 127)  # json.loads reads these; the reader's contract refuses them
    for value in refused:
        text = base.replace(slot, '"architectures": ' + value)
        if value in reader_only:
            json.loads(text)
        else:
            with pytest.raises(ValueError):
                json.loads(text)
        expect(capfd, place, p, text, INVALID, "JSON object", model=m)
    for raw in (b'"\xff"', b'"\xc0\x80"', b'"\xed\xa0\x80"', b'"\xf4\x90\x80\x80"', b'"\xe2\x82"'):  # no UTF-8: overlong, a surrogate, beyond U+10FFFF, cut short
        expect(capfd, place, p, base.encode().replace(slot.encode(), b'"architectures": ' + raw), INVALID, "JSON object", model=m)
    # a key twice, also when one of the two is written with an escape, and in an object the check does not otherwise read
    for twice in ('"architectures": {"a": 1, "\\u0061": 2}', '"architectures": [{"k": 1, "k": 1}]'):
        expect(capfd, place, p, base.replace(slot, twice), INVALID, "twice", model=m)
    expect(capfd, place, p, base.replace(slot, '"architectures": {"a": 1, "A": 2, "aa": 3, "": 4}'), OK, model=m)
    # a key that is the same text as a member's name is that member, however it is written
    expect(capfd, place, p, base.replace('"codebook"', '"code\\u0062ook"'), OK, model=m)
    # whole numbers are Python's int as str() writes it: no sign, no leading zero, no fraction
    for number in ("1.0", "1e0", "-1", "18446744073709551616"):
        expect(capfd, place, p, base.replace('"layers": 1,', '"layers": %s,' % number), INVALID, "experts.layers", "whole number", model=m)
    # a width's name is its canonical one
    for name in ("K03", "k3", "K3.0", "K0.5", "K8.5", "K", "mixed"):
        text = base.replace('"w1": {"K3": 2}', '"w1": {"%s": 2}' % name)
        expect(capfd, place, p, text, INVALID, "widths.0.w1", model=m)


def test_sha256_against_hashlib():
    lib = amd.library()
    rng = np.random.default_rng(1)
    for count in list(range(0, 130)) + [1000, 4096, 65537, 1 << 20]:
        data = rng.integers(0, 256, size=count, dtype=np.uint8).tobytes()
        out = (C.c_ubyte * 32)()
        lib.anemone_sha256(data, count, out)
        assert bytes(out) == hashlib.sha256(data).digest(), count
    out = (C.c_ubyte * 32)()
    lib.anemone_sha256(b"abc", 3, out)  # FIPS 180-4's own example
    assert bytes(out).hex() == "ba7816bf8f01cfea414140de5dae2223b00361a396177a9cb410ff61f20015ad"


def test_the_model_against_the_fused_kernels(capfd):
    """exl3_descriptor_tc_check: the model's geometry against what this build's fused EXL3 launches take (the reference's
    check, source/exl3_descriptor.c:955-1039, is against its own kernels' fixed sizes: a model that fits here is one
    exl3_tc_prepare takes)."""
    lib = amd.library()

    def tc(ranks=1, **changes):
        capfd.readouterr()
        m = model_of(**changes)
        status = lib.exl3_descriptor_tc_check(b"v41", C.byref(m), ranks, 0)
        return status, capfd.readouterr().err

    assert tc(hidden=4096, intermediate=2048, experts_per_layer=256, routes_per_row=8) == (OK, "")
    assert tc() == (OK, "")  # 5120 and 2304
    assert tc(ranks=4)[0] == OK  # 2304 = 18 blocks of 128: 5, 5, 4, 4 blocks a rank
    for changes, words in ((dict(routes_per_row=9), ["routes_per_row", "9", "8"]), (dict(routes_per_row=0), ["routes_per_row"]),
                           (dict(experts_per_layer=513), ["experts.experts_per_layer", "513", "512"]),
                           (dict(intermediate=2300), ["experts.intermediate", "2300"]), (dict(hidden=2048, intermediate=4096), ["experts.hidden", "at most"])):
        status, log = tc(**changes)
        assert status == UNSUPPORTED and len(log.splitlines()) == 1 and "v41" in log, (changes, log)
        for word in words:
            assert word in log, (word, log)
    assert tc(ranks=4, intermediate=384)[0] == UNSUPPORTED  # three blocks do not go round four ranks
    assert lib.exl3_descriptor_tc_check(None, C.byref(model_of()), 1, 0) == INVALID
    assert lib.exl3_descriptor_tc_check(b"v41", None, 1, 0) == INVALID
    assert lib.exl3_descriptor_tc_check(b"v41", C.byref(model_of()), 0, 0) == INVALID
