"""What an executor takes from a .litertlm model file (executor/model_file.{h,cc}): the section map by kind, as
LitertLmLoader::MapSections files it (runtime/util/litert_lm_loader.cc:57-115), and the token capacity by the rule of
EngineSettings::MaybeUpdateAndValidate (runtime/engine/engine_settings.cc:79-88), with LlmMetadata.max_num_tokens
(runtime/proto/llm_metadata.proto:61, int32 field 5) read from the protocol-buffer wire format.

Pins: the reference's own data files (tests/golden/llm_metadata.pb = schema/testdata/llm_metadata.pb, whose text form
llm_metadata.pbtext sets a start token and two stop tokens and no capacity; tests/golden/test_hf_tokenizer.litertlm),
the published wire format restated here by an independent encoder (varints, all four wire types), and containers
written by the FlatBuffers writer of test_litertlm_cpu.py."""
import os
import struct
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from __graft_entry__ import load_package  # noqa: E402
from test_litertlm_cpu import STR, U32, container, kv, section, write  # noqa: E402

X = load_package().executor
GOLDEN = os.path.join(ROOT, "tests", "golden")
INVALID_ARGUMENT = 3
TFLITE, SP, META, HF = 3, 4, 5, 6


def varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        out.append(b | (0x80 if v else 0))
        if not v:
            return bytes(out)


def field(number, wire, payload):
    return varint(number << 3 | wire) + payload


def test_reference_metadata_file_sets_no_capacity():
    msg = open(os.path.join(GOLDEN, "llm_metadata.pb"), "rb").read()
    # start_token { token_str: "<bos>" }, stop_tokens { "<eos>" }, stop_tokens { "<end_of_turn>" }: fields 1, 2, 2
    want = (field(1, 2, varint(7) + field(2, 2, varint(5) + b"<bos>")) +
            field(2, 2, varint(7) + field(2, 2, varint(5) + b"<eos>")) +
            field(2, 2, varint(15) + field(2, 2, varint(13) + b"<end_of_turn>")))
    assert msg == want                      # the independent encoder reproduces the reference's file byte for byte
    assert X.proto_int32_field(msg, 5) == 0
    assert X.proto_int32_field(msg + field(5, 0, varint(8192)), 5) == 8192


@pytest.mark.parametrize("value", [0, 1, 127, 128, 300, 4096, 2 ** 31 - 1, -1, -(2 ** 31)])
def test_int32_field_values(value):
    noise = field(1, 2, varint(3) + b"abc") + field(9, 1, struct.pack("<Q", 7)) + field(11, 5, struct.pack("<I", 9)) + \
        field(4, 0, varint(77))
    assert X.proto_int32_field(noise + field(5, 0, varint(value)) + noise, 5) == value
    assert X.proto_int32_field(field(5, 0, varint(3)) + field(5, 0, varint(value)), 5) == value   # the last one counts
    assert X.proto_int32_field(noise, 5) == 0


@pytest.mark.parametrize("damaged", [
    b"\x28",                                   # tag of field 5 and nothing after it
    b"\x28\x80",                               # varint that never ends
    b"\x28" + b"\xff" * 11,                    # varint longer than ten bytes
    b"\x0a\x05ab",                             # length-delimited field running past the end
    b"\x09\x01\x02",                           # 64-bit field cut short
    b"\x0d\x01",                               # 32-bit field cut short
    b"\x2b",                                   # wire type 3 (groups)
    b"\x00\x00",                               # field number 0
])
def test_damaged_messages_are_invalid_argument(damaged):
    with pytest.raises(X.ExecutorError) as e:
        X.proto_int32_field(damaged, 5)
    assert e.value.code == INVALID_ARGUMENT


def test_reference_container():
    m = X.model_file(os.path.join(GOLDEN, "test_hf_tokenizer.litertlm"))
    assert m == {"sections": {"HF_Tokenizer_Zlib": [16384, 609288]}, "metadata_max_num_tokens": 0, "max_num_tokens": 4096}


def model_items(value, key="model_type"):
    return [kv(key, STR, value)]


def test_sections_are_filed_by_kind_and_model_type(tmp_path):
    meta = field(1, 2, varint(0)) + field(5, 0, varint(1280))
    payloads = [(4096, b"A" * 100), (8192, b"B" * 200), (12288, b"C" * 50), (16384, b"D" * 60), (20480, meta),
                (24576, b"E" * 10), (28672, b"F" * 70)]
    sections = [
        section(model_items("TF_LITE_PREFILL_DECODE"), 4096, 4196, TFLITE),
        section(model_items("tf_lite_embedder", key="Model_Type"), 8192, 8392, TFLITE),   # key and value in any case
        section([kv("note", STR, "x"), kv("n", U32, 3)], 12288, 12338, TFLITE),           # no model type: prefill + decode, replaces the first
        section(None, 16384, 16444, SP),
        section([], 20480, 20480 + len(meta), META),
        section(model_items("tf_lite_aux"), 24576, 24586, TFLITE),
        section(model_items("Tf_Lite_Per_Layer_Embedder"), 28672, 28742, TFLITE),
    ]
    p = write(tmp_path, "model.litertlm", container([kv("arch", STR, "all")], sections, payloads))
    m = X.model_file(p)
    assert m["sections"] == {"TF_LITE_PREFILL_DECODE": [12288, 12338], "TF_LITE_EMBEDDER": [8192, 8392],
                             "TF_LITE_PER_LAYER_EMBEDDER": [28672, 28742], "TF_LITE_AUX": [24576, 24586],
                             "SP_Tokenizer": [16384, 16444], "LlmMetadataProto": [20480, 20480 + len(meta)]}
    assert m["metadata_max_num_tokens"] == 1280 and m["max_num_tokens"] == 1280
    assert X.model_file(p, preset_max_num_tokens=512)["max_num_tokens"] == 512   # a value the caller has set stays


def test_capacity_defaults_and_errors(tmp_path):
    no_field = field(2, 2, varint(0))
    p = write(tmp_path, "a.litertlm", container([], [section([], 4096, 4096 + len(no_field), META)], [(4096, no_field)]))
    assert X.model_file(p)["max_num_tokens"] == 4096                     # metadata without the field
    zero = field(5, 0, varint(0))
    p = write(tmp_path, "b.litertlm", container([], [section([], 4096, 4096 + len(zero), META)], [(4096, zero)]))
    assert X.model_file(p)["max_num_tokens"] == 4096                     # ... or with a non-positive value
    p = write(tmp_path, "c.litertlm", container([], [section(model_items("tf_lite_gpu"), 4096, 4100, TFLITE)], [(4096, b"abcd")]))
    with pytest.raises(X.ExecutorError) as e:
        X.model_file(p)
    assert e.value.code == INVALID_ARGUMENT and e.value.message == "Unknown model type: tf_lite_gpu"
    p = write(tmp_path, "d.litertlm", container([], [section([], 4096, 9000, SP)], [(4096, b"short")]))
    with pytest.raises(X.ExecutorError) as e:
        X.model_file(p)
    assert e.value.code == INVALID_ARGUMENT and "does not lie inside the file" in e.value.message
    bad = b"\x28"
    p = write(tmp_path, "e.litertlm", container([], [section([], 4096, 4097, META)], [(4096, bad)]))
    with pytest.raises(X.ExecutorError) as e:
        X.model_file(p)
    assert e.value.code == INVALID_ARGUMENT and "protocol buffer" in e.value.message
