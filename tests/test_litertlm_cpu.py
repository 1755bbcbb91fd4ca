"""The .litertlm container reader (executor/litertlm_reader.h) against

* tests/golden/test_hf_tokenizer.litertlm, a data file the reference's own test
  holds (schema/testdata/, used by schema/core/litertlm_read_test.cc:157-170): the
  tokenizer JSON it carries must come out byte for byte (the reference compares it
  with its testdata/tokenizer.json, whose SHA-256 is recorded below);
* headers written by a small FlatBuffers writer in this file (an independent
  direction: the reader shares no code with it) covering every value type of the
  schema, several sections and the section-metadata of the reference's NOTES
  (vocab_size=10000, algorithm=bpe, quantized=true, model_size=1234567);
* damaged files: every error is a status, never a crash.
CPU only."""
import hashlib
import json
import os
import struct
import sys
import zlib

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from __graft_entry__ import load_package  # noqa: E402

X = load_package().executor
FIXTURE = os.path.join(ROOT, "tests", "golden", "test_hf_tokenizer.litertlm")
TOKENIZER_JSON_SHA256 = "9ca9acddb6525a194ec8ac7a87f24fbba7232a9a15ffa1af0c1224fcd888e47c"  # schema/testdata/tokenizer.json
TOKENIZER_JSON_BYTES = 2104556
INVALID_ARGUMENT, NOT_FOUND, UNIMPLEMENTED, INTERNAL = 3, 5, 12, 13
U8, I8, U16, I16, U32, I32, F32, BOOL, STR, U64, I64 = range(1, 12)


# ------------------------------------------------------------------ a forward-layout FlatBuffers writer
class Node:
    """table: fields = list of None | ('scalar', fmt, value) | ('ref', Node); struct: raw bytes;
    string: text; vector: list of Nodes (offsets)."""
    def __init__(self, kind, payload):
        self.kind, self.payload, self.pos = kind, payload, None


def table(*fields): return Node("table", list(fields))
def struct_(fmt, v): return Node("struct", struct.pack("<" + fmt, v))
def string(s): return Node("string", s.encode())
def vector(nodes): return Node("vector", list(nodes))
def scalar(fmt, v): return ("scalar", fmt, v)
def ref(node): return ("ref", node)


def build(root: Node) -> bytes:
    out = bytearray(8)  # root offset (+4 bytes of padding keeps 8-byte alignment)
    pending = []        # (position of the uoffset field, target node)

    def align(n):
        while len(out) % n:
            out.append(0)

    def emit(node):
        if node.kind == "table":
            sizes = []
            for f in node.payload:
                sizes.append(0 if f is None else (4 if f[0] == "ref" else struct.calcsize("<" + f[1])))
            # vtable, then the table: soffset, then the fields in order, each aligned to its size
            offs, cur = [], 4
            for sz in sizes:
                if sz == 0:
                    offs.append(0)
                    continue
                cur = (cur + sz - 1) // sz * sz
                offs.append(cur)
                cur += sz
            align(2)
            vt = len(out)
            out.extend(struct.pack("<HH", 4 + 2 * len(sizes), cur))
            for o in offs:
                out.extend(struct.pack("<H", o))
            align(8)
            node.pos = len(out)
            out.extend(struct.pack("<i", node.pos - vt))
            out.extend(bytes(cur - 4))
            for f, o in zip(node.payload, offs):
                if f is None:
                    continue
                if f[0] == "scalar":
                    struct.pack_into("<" + f[1], out, node.pos + o, f[2])
                else:
                    pending.append((node.pos + o, f[1]))
            for f in node.payload:
                if f is not None and f[0] == "ref":
                    emit(f[1])
        elif node.kind == "struct":
            align(8)
            node.pos = len(out)
            out.extend(node.payload)
        elif node.kind == "string":
            align(4)
            node.pos = len(out)
            out.extend(struct.pack("<I", len(node.payload)) + node.payload + b"\0")
        else:  # vector of offsets
            align(4)
            node.pos = len(out)
            out.extend(struct.pack("<I", len(node.payload)))
            base = len(out)
            out.extend(bytes(4 * len(node.payload)))
            for i, child in enumerate(node.payload):
                pending.append((base + 4 * i, child))
            for child in node.payload:
                emit(child)

    emit(root)
    struct.pack_into("<I", out, 0, root.pos)
    for where, node in pending:
        assert node.pos > where
        struct.pack_into("<I", out, where, node.pos - where)
    return bytes(out)


FMT = {U8: "B", I8: "b", U16: "H", I16: "h", U32: "I", I32: "i", F32: "f", BOOL: "?", U64: "Q", I64: "q"}


def kv(key, vtype, value):
    v = table(ref(string(value))) if vtype == STR else struct_(FMT[vtype], value)
    return table(ref(string(key)), scalar("B", vtype), ref(v))


def section(items, begin, end, dtype):
    return table(ref(vector(items)) if items is not None else None, scalar("Q", begin), scalar("Q", end), scalar("B", dtype))


def container(system, sections, payloads=(), version=(1, 1, 0)):
    """A whole file: preamble, header, then the payloads at the offsets the sections name."""
    fb = build(table(ref(table(ref(vector(system)))), ref(table(ref(vector(sections))))))
    head = b"LITERTLM" + struct.pack("<III", *version) + bytes(4) + struct.pack("<Q", 32 + len(fb)) + fb
    body = bytearray(head)
    for begin, data in payloads:
        assert begin >= len(body)
        body.extend(bytes(begin - len(body)))
        body.extend(data)
    return bytes(body)


def write(tmp_path, name, data):
    p = tmp_path / name
    p.write_bytes(data)
    return p


# ------------------------------------------------------------------ the reference's data file
def test_fixture_header_and_section_map():
    h = X.litertlm_header(FIXTURE)
    assert h["version"] == [1, 0, 0] and h["header_end_offset"] == 240
    assert [e["key"] for e in h["system_metadata"]] == ["arch", "version"]
    assert all(e["type"] == STR and e["value"] for e in h["system_metadata"])
    assert h["sections"] == [{"begin_offset": 16384, "end_offset": 609288, "data_type": X.SECTION_HF_TOKENIZER_ZLIB,
                              "data_type_name": "HF_Tokenizer_Zlib", "items": []}]
    with open(FIXTURE, "rb") as f:
        assert X.litertlm_header(data=f.read(4096)) == h      # from memory: the header alone is enough


def test_fixture_tokenizer_json_comes_out_byte_for_byte():
    for data in (X.litertlm_hf_tokenizer_json(FIXTURE), X.litertlm_hf_tokenizer_json(FIXTURE, 0)):
        assert len(data) == TOKENIZER_JSON_BYTES
        assert hashlib.sha256(data).hexdigest() == TOKENIZER_JSON_SHA256
    assert "model" in json.loads(data)


def test_fixture_wrong_type_bad_index_and_missing_kind():
    with pytest.raises(X.ExecutorError) as e:   # litertlm_read_test.cc: a section read as another type
        X.litertlm_section(FIXTURE, 0, X.SECTION_TFLITE)
    assert e.value.code == INVALID_ARGUMENT and "It is: HF_Tokenizer_Zlib, expected 3" in e.value.message
    for idx in (-1, 1):
        with pytest.raises(X.ExecutorError) as e:
            X.litertlm_section(FIXTURE, idx, X.SECTION_HF_TOKENIZER_ZLIB)
        assert e.value.code == INVALID_ARGUMENT and "num sections = 1" in e.value.message
    with pytest.raises(X.ExecutorError) as e:
        X.litertlm_any_binary(FIXTURE)
    assert e.value.code == NOT_FOUND
    raw = X.litertlm_section(FIXTURE, 0, X.SECTION_HF_TOKENIZER_ZLIB)
    assert len(raw) == 609288 - 16384 and struct.unpack("<Q", raw[:8])[0] == TOKENIZER_JSON_BYTES


# ------------------------------------------------------------------ written here, read there
def test_every_value_type_and_several_sections(tmp_path):
    system = [kv("arch", STR, "all"), kv("u8", U8, 200), kv("i8", I8, -100), kv("u16", U16, 60000), kv("i16", I16, -30000),
              kv("u32", U32, 4000000000), kv("i32", I32, -2000000000), kv("f32", F32, 0.25), kv("yes", BOOL, True),
              kv("no", BOOL, False), kv("u64", U64, 2 ** 63 + 5), kv("i64", I64, -(2 ** 62))]
    tok = b"not a real sentencepiece model"
    blob = b"Dummy Binary Data Content"   # schema/testdata/data.bin of the reference
    meta = bytes(range(35))
    sections = [section([kv("vocab_size", I32, 10000), kv("algorithm", STR, "bpe")], 16384, 16384 + len(tok), X.SECTION_SP_TOKENIZER),
                section([kv("quantized", BOOL, True), kv("model_size", I32, 1234567)], 32768, 32768 + 64, X.SECTION_TFLITE),
                section([kv("model", STR, "gemma3")], 49152, 49152 + len(meta), X.SECTION_LLM_METADATA),
                section([kv("type", STR, "abc")], 65536, 65536 + len(blob), X.SECTION_BINARY),
                section(None, 70000, 70000, X.SECTION_BINARY)]
    data = container(system, sections, [(16384, tok), (32768, bytes(64)), (49152, meta), (65536, blob)])
    path = write(tmp_path, "all_types.litertlm", data)
    h = X.litertlm_header(path)
    assert h["version"] == [1, 1, 0]
    got = {e["key"]: (e["type"], e["value"]) for e in h["system_metadata"]}
    assert got == {"arch": (STR, "all"), "u8": (U8, "200"), "i8": (I8, "-100"), "u16": (U16, "60000"),
                   "i16": (I16, "-30000"), "u32": (U32, "4000000000"), "i32": (I32, "-2000000000"),
                   "f32": (F32, "0.250000"), "yes": (BOOL, "true"), "no": (BOOL, "false"),
                   "u64": (U64, str(2 ** 63 + 5)), "i64": (I64, str(-(2 ** 62)))}
    assert [s["data_type_name"] for s in h["sections"]] == ["SP_Tokenizer", "TFLiteModel", "LlmMetadataProto",
                                                            "GenericBinaryData", "GenericBinaryData"]
    assert [(i["key"], i["value"]) for i in h["sections"][0]["items"]] == [("vocab_size", "10000"), ("algorithm", "bpe")]
    assert [(i["key"], i["value"]) for i in h["sections"][1]["items"]] == [("quantized", "true"), ("model_size", "1234567")]
    assert h["sections"][4]["items"] == []
    assert X.litertlm_section(path, 0, X.SECTION_SP_TOKENIZER) == tok
    assert X.litertlm_section(path, 2, X.SECTION_LLM_METADATA) == meta
    assert X.litertlm_any_binary(path) == blob                       # the first binary section
    with pytest.raises(X.ExecutorError) as e:                        # the empty one
        X.litertlm_section(path, 4, X.SECTION_BINARY)
    assert e.value.code == INVALID_ARGUMENT and "zero size" in e.value.message
    with pytest.raises(X.ExecutorError) as e:
        X.litertlm_hf_tokenizer_json(path)
    assert e.value.code == NOT_FOUND


def test_hf_tokenizer_round_trip_and_damage(tmp_path):
    text = json.dumps({"model": {"vocab": {str(i): i for i in range(500)}}}).encode()
    packed = struct.pack("<Q", len(text)) + zlib.compress(text)
    sec = [section(None, 4096, 4096 + len(packed), X.SECTION_HF_TOKENIZER_ZLIB)]
    path = write(tmp_path, "tok.litertlm", container([], sec, [(4096, packed)]))
    assert X.litertlm_hf_tokenizer_json(path) == text
    bad = bytearray(packed)
    bad[40] ^= 0xFF
    path = write(tmp_path, "tok_bad.litertlm", container([], sec, [(4096, bytes(bad))]))
    with pytest.raises(X.ExecutorError) as e:
        X.litertlm_hf_tokenizer_json(path)
    assert e.value.code == INTERNAL
    short = [section(None, 4096, 4100, X.SECTION_HF_TOKENIZER_ZLIB)]
    path = write(tmp_path, "tok_short.litertlm", container([], short, [(4096, b"abcd")]))
    with pytest.raises(X.ExecutorError) as e:
        X.litertlm_hf_tokenizer_json(path)
    assert e.value.code == INTERNAL and "too short" in e.value.message
    cut = [section(None, 4096, 8192, X.SECTION_BINARY)]                  # the file ends before the section does
    path = write(tmp_path, "cut.litertlm", container([], cut, [(4096, b"x" * 10)]))
    with pytest.raises(X.ExecutorError) as e:
        X.litertlm_section(path, 0, X.SECTION_BINARY)
    assert e.value.code == INTERNAL
    wild = [section(None, 4096, 1 << 62, X.SECTION_BINARY)]               # an end offset far past the file: a status, no allocation
    path = write(tmp_path, "wild.litertlm", container([], wild, [(4096, b"x" * 10)]))
    with pytest.raises(X.ExecutorError) as e:
        X.litertlm_section(path, 0, X.SECTION_BINARY)
    assert e.value.code == INTERNAL


# ------------------------------------------------------------------ damaged preambles and headers
def test_preamble_errors(tmp_path):
    good = open(FIXTURE, "rb").read(4096)
    with pytest.raises(X.ExecutorError) as e:
        X.litertlm_header(data=b"LITERTLX" + good[8:])
    assert e.value.code == INVALID_ARGUMENT and "Invalid magic number" in e.value.message
    with pytest.raises(X.ExecutorError) as e:
        X.litertlm_header(data=good[:8] + struct.pack("<I", 2) + good[12:])
    assert e.value.code == UNIMPLEMENTED and "doesn't support version 2, expected version 1" in e.value.message
    with pytest.raises(X.ExecutorError) as e:
        X.litertlm_header(data=good[:24] + struct.pack("<Q", 16) + good[32:])
    assert e.value.code == INVALID_ARGUMENT and "Invalid header end offset" in e.value.message
    for n in (3, 12, 22, 30, 100):   # cut inside the magic, the version, the padding, the offset, the header
        with pytest.raises(X.ExecutorError) as e:
            X.litertlm_header(data=good[:n])
        assert e.value.code == (INVALID_ARGUMENT if n < 8 else INTERNAL), n
    with pytest.raises(X.ExecutorError) as e:
        X.litertlm_header(tmp_path / "does_not_exist.litertlm")
    assert e.value.code == INTERNAL and "Could not open file" in e.value.message
    assert X.litertlm_header(write(tmp_path, "copy.litertlm", good))["header_end_offset"] == 240


def test_corrupted_offsets_are_reported_not_followed():
    good = bytearray(open(FIXTURE, "rb").read(240))
    failures = 0
    for pos in range(32, 240, 4):        # overwrite every aligned word of the header with a wild value
        for wild in (0xFFFFFFF0, 0x7FFFFFFF, 0x000F0000):
            bad = bytearray(good)
            struct.pack_into("<I", bad, pos, wild)
            try:
                X.litertlm_header(data=bytes(bad))
            except X.ExecutorError as e:
                assert e.code == INVALID_ARGUMENT, (pos, wild, e.code)
                failures += 1
    assert failures > 20
