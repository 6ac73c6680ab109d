"""Writes tests/golden/einsummable_proto_fields.json: every message of the reference's
src/proto/einsummable.proto as data -- field name, number, type, label, enclosing oneof -- read
from the .proto text where it lies in the reference tree (run in the build container only;
the JSON is the committed fixture).

    python tests/golden/make_proto_fields.py [/root/reference]

tests/test_memgraph_wire.py compares the hand-restated schema its encoder is built from
(tests/memgraph_proto.py) with this table, so that a field number typed wrongly on both sides
of the wire-reader tests cannot go unnoticed.
"""
import json
import os
import re
import sys


def parse(text):
    text = re.sub(r"//[^\n]*", "", text)
    tokens = re.findall(r"[A-Za-z_][A-Za-z_0-9.]*|\d+|[{}=;]", text)
    messages, i = {}, 0
    while i < len(tokens):
        if tokens[i] == "message":
            name = tokens[i + 1]
            assert tokens[i + 2] == "{", name
            i += 3
            fields, oneof, depth = [], None, 1
            while depth:
                t = tokens[i]
                if t == "}":
                    depth -= 1
                    if depth == 1:
                        oneof = None
                    i += 1
                elif t == "oneof":
                    oneof = tokens[i + 1]
                    assert tokens[i + 2] == "{"
                    depth += 1
                    i += 3
                elif t in ("required", "optional", "repeated"):
                    typ, fname, eq, number, semi = tokens[i + 1:i + 6]
                    assert eq == "=" and semi == ";", (name, fname)
                    fields.append([fname, int(number), typ, t[:3], None])
                    i += 6
                else:  # a field inside a oneof has no label
                    typ, fname, eq, number, semi = tokens[i:i + 5]
                    assert oneof and eq == "=" and semi == ";", (name, tokens[i:i + 5])
                    fields.append([fname, int(number), typ, "opt", oneof])
                    i += 5
            messages[name] = fields
        else:
            i += 1
    return messages


if __name__ == "__main__":
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    with open(os.path.join(ref, "src", "proto", "einsummable.proto")) as f:
        table = parse(f.read())
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "einsummable_proto_fields.json")
    with open(out, "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)
        f.write("\n")
    print("%d messages -> %s" % (len(table), out))
