"""Minimal protobuf wire-format writer / reader for LightSeq's quantised model files.

The model files of the reference are proto3 messages
(lightseq/inference/proto/quant_bert.proto, quant_transformer.proto,
quant_gpt.proto).  Neither ``protoc`` nor the protobuf runtime is needed for them:
only varints, 32-bit floats and length-delimited fields occur.  The schemas below
are the data contract (field names and numbers) of those files; weights are stored
as ``uint8 = code + 127`` bytes with one ``*_clip_max`` float per tensor
(lightseq/training/ops/pytorch/export_quant.py:12-20).

Kinds: ``float`` ``int32`` ``bool`` ``string`` ``bytes`` scalar fields,
``rfloat`` / ``rint32`` repeated (written packed), ``msg:Name`` / ``rmsg:Name``
embedded messages.
"""
import struct

import numpy as np

_ENC_LAYER_COMMON = {
    "multihead_norm_scale": (1, "rfloat"), "multihead_norm_bias": (2, "rfloat"),
    "multihead_project_kernel_qkv": (3, "bytes"), "multihead_project_bias_qkv": (4, "rfloat"),
    "multihead_project_kernel_output": (5, "bytes"), "multihead_project_bias_output": (6, "rfloat"),
    "ffn_norm_scale": (7, "rfloat"), "ffn_norm_bias": (8, "rfloat"),
    "ffn_first_kernel": (9, "bytes"), "ffn_first_bias": (10, "rfloat"),
    "ffn_second_kernel": (11, "bytes"), "ffn_second_bias": (12, "rfloat"),
    "multihead_project_kernel_qkv_clip_max": (13, "float"),
    "multihead_project_kernel_output_clip_max": (14, "float"),
    "ffn_first_kernel_clip_max": (15, "float"), "ffn_second_kernel_clip_max": (16, "float"),
    "multihead_ln_clip_max": (17, "float"), "multihead_project_output_clip_max": (18, "float"),
    "ffn_ln_clip_max": (19, "float"), "ffn_first_act_clip_max": (20, "float"),
    "multihead_qkv_dense_clip_max": (21, "float"), "multihead_output_dense_clip_max": (22, "float"),
    "ffn_first_output_clip_max": (23, "float"),
}

SCHEMAS = {
    # quant_bert.proto
    "QuantBertEncoderLayer": dict(_ENC_LAYER_COMMON),
    "QuantBertEmbeddingLayer": {
        "token_embedding": (1, "bytes"), "position_embedding": (2, "rfloat"),
        "norm_scale": (3, "rfloat"), "norm_bias": (4, "rfloat"), "emb_clip_max": (5, "float"),
    },
    "QuantBertModelConf": {
        "head_num": (1, "int32"), "src_padding_id": (2, "int32"), "is_post_ln": (3, "bool"),
        "use_gelu": (4, "bool"), "multilg_type": (5, "int32"),
    },
    "QuantBert": {
        "src_embedding": (1, "msg:QuantBertEmbeddingLayer"),
        "encoder_stack": (2, "rmsg:QuantBertEncoderLayer"),
        "model_conf": (3, "msg:QuantBertModelConf"),
    },
    # quant_transformer.proto
    "QuantEncoderLayer": dict(_ENC_LAYER_COMMON, ffn_second_output_clip_max=(24, "float")),
    "QuantDecoderLayer": {
        "self_norm_scale": (1, "rfloat"), "self_norm_bias": (2, "rfloat"),
        "self_project_kernel_qkv": (3, "bytes"), "self_project_bias_qkv": (4, "rfloat"),
        "self_project_kernel_output": (5, "bytes"), "self_project_bias_output": (6, "rfloat"),
        "encdec_norm_scale": (7, "rfloat"), "encdec_norm_bias": (8, "rfloat"),
        "encdec_project_kernel_q": (9, "bytes"), "encdec_project_bias_q": (10, "rfloat"),
        "encdec_project_kernel_output": (11, "bytes"), "encdec_project_bias_output": (12, "rfloat"),
        "ffn_norm_scale": (13, "rfloat"), "ffn_norm_bias": (14, "rfloat"),
        "ffn_first_kernel": (15, "bytes"), "ffn_first_bias": (16, "rfloat"),
        "ffn_second_kernel": (17, "bytes"), "ffn_second_bias": (18, "rfloat"),
        "self_project_kernel_qkv_clip_max": (19, "float"),
        "self_project_kernel_output_clip_max": (20, "float"),
        "encdec_project_kernel_q_clip_max": (21, "float"),
        "encdec_project_kernel_output_clip_max": (22, "float"),
        "ffn_first_kernel_clip_max": (23, "float"), "ffn_second_kernel_clip_max": (24, "float"),
        "self_ln_clip_max": (25, "float"), "self_project_output_clip_max": (26, "float"),
        "encdec_ln_clip_max": (27, "float"), "encdec_project_output_clip_max": (28, "float"),
        "ffn_ln_clip_max": (29, "float"), "ffn_first_act_clip_max": (30, "float"),
        "self_qkv_dense_clip_max": (31, "float"), "self_output_dense_clip_max": (32, "float"),
        "encdec_q_dense_clip_max": (33, "float"), "encdec_output_dense_clip_max": (34, "float"),
        "ffn_first_output_clip_max": (35, "float"), "ffn_second_output_clip_max": (36, "float"),
        "self_qkv_bias_out_clip_max": (37, "float"),
    },
    "QuantEmbeddingLayer": {
        "token_embedding": (1, "bytes"), "position_embedding": (2, "rfloat"),
        "norm_scale": (3, "rfloat"), "norm_bias": (4, "rfloat"),
        "encode_output_project_kernel_kv": (5, "bytes"),
        "encode_output_project_bias_kv": (6, "rfloat"), "shared_bias": (7, "rfloat"),
        "lang_emb": (8, "rfloat"), "emb_clip_max": (9, "float"),
        "encode_output_project_kernel_kv_clip_max": (10, "rfloat"),
        "output_ln_clip_max": (11, "float"), "logits_clip_max": (12, "float"),
    },
    "QuantModelConf": {
        "head_num": (1, "int32"), "beam_size": (2, "int32"), "extra_decode_length": (3, "int32"),
        "length_penalty": (4, "float"), "src_padding_id": (5, "int32"), "trg_start_id": (6, "int32"),
        "diverse_lambda": (7, "float"), "sampling_method": (8, "string"), "topp": (9, "float"),
        "topk": (10, "int32"), "trg_end_id": (11, "int32"), "is_post_ln": (12, "bool"),
        "no_scale_embedding": (13, "bool"), "use_gelu": (14, "bool"), "multilg_type": (15, "int32"),
    },
    # quant_gpt.proto
    "QuantGptEncoderLayer": dict(_ENC_LAYER_COMMON, self_qkv_bias_out_clip_max=(24, "float")),
    "QuantGptEmbeddingLayer": {
        "token_embedding": (1, "bytes"), "position_embedding": (2, "rfloat"),
        "norm_scale": (3, "rfloat"), "norm_bias": (4, "rfloat"), "emb_clip_max": (5, "float"),
        "output_ln_clip_max": (6, "float"), "logits_clip_max": (7, "float"),
    },
    "QuantGptModelConf": {
        "head_num": (1, "int32"), "src_padding_id": (2, "int32"), "sampling_method": (3, "string"),
        "topp": (4, "float"), "topk": (5, "int32"), "eos_id": (6, "int32"),
        "extra_decode_length": (7, "int32"),
    },
    "QuantGpt": {
        "src_embedding": (1, "msg:QuantGptEmbeddingLayer"),
        "encoder_stack": (2, "rmsg:QuantGptEncoderLayer"),
        "model_conf": (3, "msg:QuantGptModelConf"),
    },
    "QuantTransformer": {
        "src_embedding": (1, "msg:QuantEmbeddingLayer"),
        "encoder_stack": (2, "rmsg:QuantEncoderLayer"),
        "trg_embedding": (3, "msg:QuantEmbeddingLayer"),
        "decoder_stack": (4, "rmsg:QuantDecoderLayer"),
        "model_conf": (5, "msg:QuantModelConf"),
    },
}


def _varint(n):
    n &= (1 << 64) - 1  # negative int32 are sign-extended to 64 bits on the wire
    out = bytearray()
    while True:
        b = n & 0x7F
        n >>= 7
        if n:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _tag(num, wire):
    return _varint((num << 3) | wire)


def encode(message, values):
    """Serialise ``values`` (dict) as protobuf message ``message``; returns bytes.

    proto3 semantics: fields that are absent, zero or empty are not written."""
    schema = SCHEMAS[message]
    chunks = []
    for name, (num, kind) in sorted(schema.items(), key=lambda kv: kv[1][0]):
        if name not in values or values[name] is None:
            continue
        v = values[name]
        if kind == "float":
            if float(v) != 0.0:
                chunks.append(_tag(num, 5) + struct.pack("<f", float(v)))
        elif kind in ("int32", "bool"):
            if int(v) != 0:
                chunks.append(_tag(num, 0) + _varint(int(v)))
        elif kind == "string":
            b = v.encode() if isinstance(v, str) else bytes(v)
            if b:
                chunks.append(_tag(num, 2) + _varint(len(b)) + b)
        elif kind == "bytes":
            b = np.ascontiguousarray(v, dtype=np.uint8).tobytes() if not isinstance(v, (bytes, bytearray)) else bytes(v)
            if b:
                chunks.append(_tag(num, 2) + _varint(len(b)) + b)
        elif kind == "rfloat":
            b = np.ascontiguousarray(v, dtype="<f4").tobytes()
            if b:
                chunks.append(_tag(num, 2) + _varint(len(b)) + b)
        elif kind == "rint32":
            b = b"".join(_varint(int(x)) for x in v)
            if b:
                chunks.append(_tag(num, 2) + _varint(len(b)) + b)
        elif kind.startswith("msg:"):
            b = encode(kind[4:], v)
            chunks.append(_tag(num, 2) + _varint(len(b)) + b)
        elif kind.startswith("rmsg:"):
            for item in v:
                b = encode(kind[5:], item)
                chunks.append(_tag(num, 2) + _varint(len(b)) + b)
        else:
            raise ValueError(kind)
    return b"".join(chunks)


def _read_varint(buf, pos):
    shift = 0
    val = 0
    while True:
        b = buf[pos]
        pos += 1
        val |= (b & 0x7F) << shift
        if not b & 0x80:
            return val, pos
        shift += 7


def decode(message, buf):
    """Parse bytes of protobuf message ``message`` into a dict (numpy arrays for
    repeated floats and bytes).  Unknown fields are skipped."""
    schema = SCHEMAS[message]
    by_num = {num: (name, kind) for name, (num, kind) in schema.items()}
    out = {}
    buf = memoryview(buf)
    pos, end = 0, len(buf)
    while pos < end:
        key, pos = _read_varint(buf, pos)
        num, wire = key >> 3, key & 7
        if wire == 0:
            val, pos = _read_varint(buf, pos)
            raw = val
        elif wire == 5:
            raw = bytes(buf[pos:pos + 4])
            pos += 4
        elif wire == 1:
            raw = bytes(buf[pos:pos + 8])
            pos += 8
        elif wire == 2:
            n, pos = _read_varint(buf, pos)
            raw = buf[pos:pos + n]
            pos += n
        else:
            raise ValueError("unsupported wire type %d" % wire)
        if num not in by_num:
            continue
        name, kind = by_num[num]
        if kind == "float":
            out[name] = struct.unpack("<f", raw)[0]
        elif kind == "int32":
            out[name] = raw - (1 << 64) if raw >= (1 << 63) else raw
        elif kind == "bool":
            out[name] = bool(raw)
        elif kind == "string":
            out[name] = bytes(raw).decode()
        elif kind == "bytes":
            out[name] = np.frombuffer(bytes(raw), dtype=np.uint8)
        elif kind == "rfloat":
            if wire == 2:
                arr = np.frombuffer(bytes(raw), dtype="<f4")
            else:  # unpacked element
                arr = np.array(struct.unpack("<f", raw), dtype=np.float32)
            out[name] = np.concatenate([out[name], arr]) if name in out else arr
        elif kind == "rint32":
            vals = []
            if wire == 2:
                p = 0
                rb = bytes(raw)
                while p < len(rb):
                    v, p = _read_varint(rb, p)
                    vals.append(v)
            else:
                vals.append(raw)
            out.setdefault(name, []).extend(vals)
        elif kind.startswith("msg:"):
            out[name] = decode(kind[4:], raw)
        elif kind.startswith("rmsg:"):
            out.setdefault(name, []).append(decode(kind[5:], raw))
    return out
