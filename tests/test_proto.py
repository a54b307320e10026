"""Model-file format: the protobuf writer/reader round trip, wire-level known answers
and the synthetic generator."""
import struct

import numpy as np

from lightseq_amd import proto, synthetic


def test_wire_known_answers():
    # protobuf documentation examples: field 1 varint 150 -> 08 96 01
    assert proto._tag(1, 0) + proto._varint(150) == bytes([0x08, 0x96, 0x01])
    assert proto._varint(300) == bytes([0xAC, 0x02])
    # negative int32 is ten bytes on the wire
    assert len(proto._varint(-1)) == 10
    msg = proto.encode("QuantBertModelConf", {"head_num": 12, "src_padding_id": 0, "is_post_ln": True,
                                              "use_gelu": True, "multilg_type": 0})
    assert msg == bytes([0x08, 12, 0x18, 1, 0x20, 1])  # zero-valued fields are omitted (proto3)
    emb = proto.encode("QuantBertEmbeddingLayer", {"emb_clip_max": 0.5})
    assert emb == bytes([0x2D]) + struct.pack("<f", 0.5)


def test_round_trip_quant_bert():
    cfg = synthetic.bert_config("tiny")
    msg = synthetic.make_quant_bert(cfg, seed=7)
    back = proto.decode("QuantBert", proto.encode("QuantBert", msg))
    assert back["model_conf"] == {"head_num": 2, "is_post_ln": True, "use_gelu": True}
    assert len(back["encoder_stack"]) == cfg["n_layer"]
    for a, b in zip(msg["encoder_stack"], back["encoder_stack"]):
        for k, v in a.items():
            if isinstance(v, np.ndarray):
                np.testing.assert_array_equal(np.asarray(v).reshape(-1), b[k])
            else:
                assert np.float32(v) == np.float32(b[k]), k
    np.testing.assert_array_equal(msg["src_embedding"]["token_embedding"], back["src_embedding"]["token_embedding"])


def test_unpacked_repeated_floats_are_accepted():
    raw = b"".join(proto._tag(3, 5) + struct.pack("<f", v) for v in (1.0, 2.0, 3.0))
    back = proto.decode("QuantBertEmbeddingLayer", raw)
    np.testing.assert_array_equal(back["norm_scale"], [1.0, 2.0, 3.0])


def test_stored_weight_convention():
    """uint8 = code + 127 with code = clamp(floor(x / (clip/127) + 0.5), -127, 127)
    (lightseq/training/ops/pytorch/export_quant.py:12-20)."""
    x = np.array([0.0, 0.08, -0.08, 1.0, -1.0, 0.08 / 127 * 2.5], np.float32)
    u8 = synthetic.quantize_u8(x, 0.08)
    np.testing.assert_array_equal(u8, [127, 254, 0, 254, 0, 130])


def test_token_ids_shape_and_padding():
    cfg = synthetic.bert_config("bert_base")
    ids, lens = synthetic.make_token_ids(cfg, 32, 128, seed=0, min_len=32)
    assert ids.shape == (32, 128) and ids.dtype == np.int32
    assert lens.min() >= 32 and lens.max() == 128
    for b in range(32):
        assert np.all(ids[b, :lens[b]] != cfg["padding_id"]) and np.all(ids[b, lens[b]:] == cfg["padding_id"])
    assert ids.max() < cfg["vocab"]


# --------------------------------------------------------------------------- #
# the schema tables and the C++ loaders against the reference's .proto files
# (tests/golden/proto_schema.json, written by tests/golden/make_proto_schema.py)
# --------------------------------------------------------------------------- #
def _reference_schema():
    import json
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "proto_schema.json")
    out = {}
    for _file, messages in json.load(open(path)).items():
        for name, fields in messages.items():
            assert name not in out
            out[name] = {f["name"]: f for f in fields}
    return out


def test_schema_tables_match_the_reference_proto_files():
    ref = _reference_schema()
    assert set(proto.SCHEMAS) == set(ref)
    scalar = {"float": "float", "int32": "int32", "bool": "bool", "string": "string", "bytes": "bytes"}
    for msg, table in proto.SCHEMAS.items():
        assert set(table) == set(ref[msg]), (msg, set(table) ^ set(ref[msg]))
        for field, (number, kind) in table.items():
            f = ref[msg][field]
            assert number == f["number"], (msg, field)
            if f["type"] in scalar:
                want = ("r" if f["repeated"] else "") + scalar[f["type"]]
            else:  # embedded message
                want = ("rmsg:" if f["repeated"] else "msg:") + f["type"]
            assert kind == want, (msg, field, kind, want)
        numbers = [n for n, _ in table.values()]
        assert len(set(numbers)) == len(numbers), msg


def test_cpp_loaders_switch_on_the_reference_field_numbers():
    """The C++ readers are hand-written switches over field numbers.  Every `case N:` whose
    target member carries a field name of the message it parses must use that field's number
    in the reference's .proto; each switch is matched to the message it shares most names with."""
    import os
    import re
    ref = _reference_schema()
    root = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "lightseq_amd",
                        "csrc", "model")
    case = re.compile(r"case\s+(\d+)\s*:\s*(.*?);\s*break;")
    ident = re.compile(r"[A-Za-z_]\w*")
    checked = 0
    for fname in ("quant_bert_weight.cpp", "quant_transformer_weight.cpp", "quant_gpt_weight.cpp"):
        text = open(os.path.join(root, fname)).read()
        for block in re.split(r"switch\s*\(", text)[1:]:
            block = block[:block.index("default:")] if "default:" in block else block
            cases = [(int(n), {t.lstrip("_") for t in ident.findall(body)}) for n, body in case.findall(block)]
            if len(cases) < 3:
                continue
            # the message this switch parses: the one whose field names it mentions most
            score = {m: sum(1 for _n, ids in cases if ids & set(fields)) for m, fields in ref.items()}
            msg = max(score, key=score.get)
            assert score[msg] >= 0.6 * len(cases), (fname, msg, score[msg], len(cases))
            for number, ids in cases:
                named = ids & set(ref[msg])
                for field in named:
                    assert ref[msg][field]["number"] == number, (fname, msg, field, number)
                    checked += 1
    assert checked >= 90, checked
    # the per-layer clip_max scalars are read as one contiguous range of field numbers
    for fname, msg in (("quant_bert_weight.cpp", "QuantBertEncoderLayer"),
                       ("quant_transformer_weight.cpp", "QuantEncoderLayer"),
                       ("quant_transformer_weight.cpp", "QuantDecoderLayer"),
                       ("quant_gpt_weight.cpp", "QuantGptEncoderLayer")):
        clips = sorted(f["number"] for f in ref[msg].values()
                       if f["name"].endswith("_clip_max") and f["type"] == "float" and not f["repeated"])
        assert clips == list(range(clips[0], clips[-1] + 1)), msg
        text = open(os.path.join(root, fname)).read()
        assert re.search(r"g\.number >= %d && g\.number <= %d" % (clips[0], clips[-1]), text), (fname, msg)
