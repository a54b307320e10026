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
