"""Extracts the data contract of the reference's quantised model files -- (message, field,
number, type, repeated) -- from the text of its three .proto files into
``tests/golden/proto_schema.json``.

Run in the build container, where /root/reference exists:

    python tests/golden/make_proto_schema.py

The fixture holds field names and numbers only (data, not source); tests/test_proto.py
compares the hand-written schema tables of lightseq_amd/proto.py and the field numbers the
C++ loaders switch on with it.
"""
import json
import os
import re
import sys

REF = "/root/reference/lightseq/inference/proto"
FILES = ["quant_bert.proto", "quant_transformer.proto", "quant_gpt.proto"]
FIELD = re.compile(r"^(repeated\s+)?([A-Za-z_][\w.]*)\s+([A-Za-z_]\w*)\s*=\s*(\d+)$")
MESSAGE = re.compile(r"message\s+(\w+)\s*\{([^{}]*)\}")


def parse(path):
    # comments off, then statements between the braces of each (flat) message
    text = "\n".join(line.split("//")[0] for line in open(path))
    messages = {}
    for name, body in MESSAGE.findall(text):
        fields = messages.setdefault(name, [])
        for stmt in body.split(";"):
            f = FIELD.match(" ".join(stmt.split()))
            if f:
                fields.append({"name": f.group(3), "number": int(f.group(4)), "type": f.group(2),
                               "repeated": bool(f.group(1))})
    return messages


def main():
    out = {}
    for name in FILES:
        out[name] = parse(os.path.join(REF, name))
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "proto_schema.json")
    with open(dst, "w") as fh:
        json.dump(out, fh, indent=1, sort_keys=True)
        fh.write("\n")
    n = sum(len(fields) for msgs in out.values() for fields in msgs.values())
    print("wrote %s: %d messages, %d fields" % (dst, sum(len(m) for m in out.values()), n))


if __name__ == "__main__":
    sys.exit(main())
