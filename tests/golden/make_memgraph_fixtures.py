"""Writes memgraph_sample.bin / memgraph_sample.txt: a serialized MemGraph holding one node
of every kind, encoded by the protobuf library from the schema in tests/memgraph_proto.py,
and the field-by-field text the reader must produce for it (written from the Python
description of the graph, not by the reader).

    python tests/golden/make_memgraph_fixtures.py
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import memgraph_proto as mp  # noqa: E402
from test_memgraph_wire import sample_memgraph  # noqa: E402

mg = sample_memgraph()
with open(os.path.join(HERE, "memgraph_sample.bin"), "wb") as f:
    f.write(mp.to_wire(mg))
with open(os.path.join(HERE, "memgraph_sample.txt"), "w") as f:
    f.write(mp.describe(mg))
print("wrote", len(mp.to_wire(mg)), "bytes")
