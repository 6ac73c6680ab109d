"""The reader of serialized memgraphs (es_km_memgraph_describe, es_km_graph_load_memgraph)
against bytes from Google's protobuf encoder (tests/memgraph_proto.py), hand-assembled bytes
that follow the published encoding rules, and the committed fixtures.  No device needed."""
import os

import numpy as np
import pytest

import einsummable_amd as ea
import memgraph_proto as mp
from memgraph_proto import node

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")

MATMUL = dict(join_shape=[4, 6, 5], inns=[[0, 2], [2, 1]], out_rank=2,
              join="*[hole|f32@0,hole|f32@1]", castable="+")
SCALE = dict(join_shape=[24], inns=[[0]], out_rank=1,
             join="*[variable{lr|f32},hole|f32@0]")
TOUCH = dict(selection=[(4, 8, 1, 2, 3), (6, 6, 0, 0, 6)], castable="+", dtype="f32")


def sample_memgraph(far=(1 << 40) + 16):
    """One node of every kind, negative and large numbers included; free of races, so it
    can also be run (with `far` inside the arena)."""
    nodes = [
        node("inputmem", loc=0, offset=0, size=80),                              # 0: A, 4 x 5 f32
        node("inputmem", loc=0, offset=256, size=120),                           # 1: B, 5 x 6 f32
        node("inputsto", storage_loc=0, storage_id=7, size=96),                  # 2
        node("constant", loc=0, offset=512, fill=dict(value="f32|0.5", shape=[4, 6])),
        node("constant", loc=0, offset=1024,
             fill=dict(lower="f16|0", upper="f16|NINF", nrow=3, ncol=5, start=-1)),
        node("alloc", loc=0, offset=2048, size=96),                              # 5: C, 4 x 6 f32
        node("apply", [0, 1, 5], loc=0, mems=[(2048, 96), (0, 80), (256, 120)],
             einsummable=MATMUL, group=-1),
        node("apply", [6], loc=0, mems=[(2048, 96), (2048, 96)], einsummable=SCALE, group=-1),
        node("partialize", loc=0, offset=4096, size=192),                        # 8: P, 8 x 6 f32
        node("apply", [7, 8], loc=0, mems=[(4096, 192), (2048, 96)], touch=TOUCH, group=3),
        node("apply", [3, 8, 9], loc=0, mems=[(4096, 192), (512, 96)], touch=TOUCH, group=3),
        node("evict", [7, 9], storage_loc=0, storage_id=11, loc=0, offset=2048, size=96),
        node("load", [11, 2], storage_loc=0, storage_id=11, loc=0, offset=8192, size=96),
        node("copy", [12], loc=0, size=96, src_offset=8192, offset=far),
        node("move", [12], src_loc=0, src_offset=8192, loc=0, offset=9216, size=96),
        node("del", [13, 14], loc=0, offset=8192, size=96),
        node("load", [2], storage_loc=0, storage_id=7, loc=0, offset=12288, size=96),
        node("apply", [16], loc=1, mems=[(0, 96), (96, 96)], einsummable=SCALE, group=-1),
    ]
    return dict(num_compute_locs=2, num_storage_locs=1, storage_locs=[0, 0], nodes=nodes)


def random_memgraph(r, n_nodes):
    kinds = ["inputmem", "inputsto", "constant", "apply", "move", "copy", "evict", "load",
             "partialize", "alloc", "del"]
    u64 = lambda: int(r.randint(0, 1 << 62)) >> int(r.randint(0, 62))
    i32 = lambda: int(r.randint(-(1 << 31), 1 << 31)) >> int(r.randint(0, 31))
    nodes = []
    for i in range(n_nodes):
        k = kinds[int(r.randint(len(kinds)))]
        inns = [int(x) for x in r.randint(0, i, size=int(r.randint(0, 5)))] if i else []
        f = dict(loc=i32())
        if k in ("inputmem", "partialize", "alloc", "del"):
            f.update(offset=u64(), size=u64())
        elif k == "inputsto":
            f = dict(storage_loc=i32(), storage_id=i32(), size=u64())
        elif k == "constant":
            f["offset"] = u64()
            if r.randint(2):
                f["fill"] = dict(value=["f16|1.5", "f32|-3", "f64|INF", "c64|(1,-2)"][int(r.randint(4))],
                                 shape=[int(x) for x in r.randint(1, 1000, size=int(r.randint(0, 4)))])
            else:
                f["fill"] = dict(lower="f32|1", upper="f32|NINF", nrow=int(r.randint(1, 1 << 20)),
                                 ncol=int(r.randint(1, 1 << 20)),
                                 start=int(r.randint(-(1 << 40), 1 << 40)))
        elif k == "apply":
            f["group"] = int(r.randint(-1, 5))
            if r.randint(2):
                rank = int(r.randint(1, 5))
                n_inn = int(r.randint(1, 4))
                f["einsummable"] = dict(
                    join_shape=[int(x) for x in r.randint(1, 1 << 30, size=rank)],
                    inns=[[int(x) for x in r.permutation(rank)[:int(r.randint(0, rank + 1))]]
                          for _ in range(n_inn)],
                    out_rank=int(r.randint(1, rank + 1)),
                    join="+[hole|f16@0,hole|f16@1]",
                    castable=["", "+", "x", "v", "^"][int(r.randint(5))])
                f["mems"] = [(u64(), u64()) for _ in range(n_inn + 1)]
            else:
                f["touch"] = dict(selection=[tuple(u64() for _ in range(5))
                                             for _ in range(int(r.randint(1, 5)))],
                                  castable=["", "+", "x", "v", "^"][int(r.randint(5))],
                                  dtype=["f16", "f32", "f64", "c64"][int(r.randint(4))])
                f["mems"] = [(u64(), u64()), (u64(), u64())]
        elif k == "move":
            f.update(src_loc=i32(), src_offset=u64(), offset=u64(), size=u64())
        elif k == "copy":
            f.update(size=u64(), src_offset=u64(), offset=u64())
        else:
            f.update(storage_loc=i32(), storage_id=i32(), offset=u64(), size=u64())
        nodes.append(node(k, inns, **f))
    return dict(num_compute_locs=int(r.randint(1, 9)), num_storage_locs=int(r.randint(0, 3)),
                storage_locs=[int(x) for x in r.randint(0, 3, size=int(r.randint(0, 9)))],
                nodes=nodes)


@pytest.mark.parametrize("packed", [False, True])
def test_every_node_kind_decodes_to_the_fields_protobuf_encoded(packed):
    mg = sample_memgraph()
    assert ea.memgraph_describe(mp.to_wire(mg, packed)) == mp.describe(mg)


@pytest.mark.parametrize("seed", range(8))
def test_random_memgraphs_decode_field_for_field(seed):
    r = np.random.RandomState(900 + seed)
    mg = random_memgraph(r, 40)
    # lowertri sizes are nrow * ncol * dtype size in 64 bits, as in the reader
    assert ea.memgraph_describe(mp.to_wire(mg, packed=bool(seed % 2))) == mp.describe(mg)


def varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        out.append(b | (0x80 if v else 0))
        if not v:
            return bytes(out)


def field(number, wire_type, payload):
    return varint(number << 3 | wire_type) + payload


def delimited(number, payload):
    return field(number, 2, varint(len(payload)) + payload)


def test_hand_assembled_bytes():
    # The encoding rules of the protocol-buffers documentation, applied by hand: 300 is the
    # varint AC 02; an int32 of -1 is sign-extended to ten bytes; tag = field << 3 | type.
    assert varint(300) == b"\xac\x02"
    assert varint(-1) == b"\xff" * 9 + b"\x01"
    alloc = delimited(9, b"\x08\x00" + b"\x10\xac\x02" + b"\x18\x08")      # loc 0, offset 300, size 8
    inputmem = delimited(1, b"\x08\x00\x10\x00\x18\x08")
    touch = delimited(1, b"\x08\x02\x10\x02\x18\x00\x20\x00\x28\x02") + b"\x1a\x03f32"
    apply_ = delimited(4, b"\x08\x00" + b"\x10\xac\x02\x10\x00" + b"\x18\x08\x18\x08" +
                       delimited(5, touch) + b"\x30" + b"\xff" * 9 + b"\x01")
    wire = (b"\x08\x01\x10\x00" + delimited(4, inputmem) + delimited(4, alloc) +
            delimited(4, apply_ + b"\x58\x00\x58\x01"))
    want = dict(num_compute_locs=1, num_storage_locs=0, nodes=[
        node("inputmem", loc=0, offset=0, size=8),
        node("alloc", loc=0, offset=300, size=8),
        node("apply", [0, 1], loc=0, mems=[(300, 8), (0, 8)], group=-1,
             touch=dict(selection=[(2, 2, 0, 0, 2)], castable="", dtype="f32"))])
    assert ea.memgraph_describe(wire) == mp.describe(want)
    assert wire == mp.to_wire(want)     # and Google's encoder writes the very same bytes


def test_unknown_fields_are_skipped_and_the_last_member_of_a_oneof_stays():
    mg = sample_memgraph()
    wire = mp.to_wire(mg)
    extra = (field(15, 0, varint(77)) + field(16, 1, b"\0" * 8) + field(17, 5, b"\0" * 4) +
             delimited(18, b"abc"))
    assert ea.memgraph_describe(extra + wire + extra) == mp.describe(mg)
    # a node that carries two members of its oneof: protobuf keeps the later one
    two = delimited(4, delimited(9, b"\x08\x00\x10\x10\x18\x08") +
                    delimited(10, b"\x08\x00\x10\x20\x18\x08"))
    want = dict(num_compute_locs=1, num_storage_locs=0,
                nodes=[node("del", loc=0, offset=32, size=8)])
    assert ea.memgraph_describe(b"\x08\x01\x10\x00" + two) == mp.describe(want)
    assert mp.classes()["MemGraph"].FromString(b"\x08\x01\x10\x00" + two).nodes[0].WhichOneof(
        "node") == "del"


def test_malformed_bytes_are_errors():
    wire = mp.to_wire(sample_memgraph())
    M = mp.classes()["MemGraph"]
    bad = [
        wire[:-3],                                        # cut inside the last node
        wire[:40],
        b"\x08\x01",                                      # num_storage_locs missing
        b"\x08\x01\x10\x00" + delimited(4, b""),          # node without an op
        b"\x08\x01\x10\x00" + delimited(4, delimited(9, b"\x08\x00\x10\x00")),   # alloc without size
        b"\x08\x01\x10\x00" + delimited(4, delimited(9, b"\x08\x00\x10\x00\x18\x08") + b"\x58\x00"),
        b"\x08\x01\x10\x00" + field(4, 3, b""),           # group wire type
        b"\x08\x01\x10\x00" + b"\x80" * 11,               # endless varint
    ]
    for i, b in enumerate(bad):
        with pytest.raises(ea.KmError) as ei:
            ea.memgraph_describe(b)
        assert ei.value.code == -1 and "could not parse memgraph" in str(ei.value), i
    # Truncation and missing required fields are what protobuf's own reader rejects (the
    # reference's ParseFromString returns false for either).
    for b in bad[:3] + bad[4:5]:
        try:
            ok = M.FromString(b).IsInitialized()
        except Exception:
            ok = False
        assert not ok


def test_committed_fixture_decodes():
    with open(os.path.join(GOLDEN, "memgraph_sample.bin"), "rb") as f:
        wire = f.read()
    with open(os.path.join(GOLDEN, "memgraph_sample.txt")) as f:
        want = f.read()
    assert ea.memgraph_describe(wire) == want
    assert wire == mp.to_wire(sample_memgraph())


def test_load_into_a_plan_only_graph():
    mg = sample_memgraph()
    g = ea.ApplyGraph(None)
    assert g.load_memgraph(mp.to_wire(mg), loc=0, scalar_vars={"lr": 0.25}) == len(mg["nodes"])
    kinds = [g.node_mems(i)[0] for i in range(g.num_nodes())]
    assert kinds == ["dummy", "dummy", "dummy", "constant", "lowertri", "dummy", "einsummable",
                     "einsummable", "dummy", "touch", "touch", "evict", "load", "copy", "copy",
                     "dummy", "load", "dummy"]            # the last node lives on location 1
    assert g.node_mems(0) == ("dummy", [(0, 80)])         # where the caller puts input 0
    assert g.node_mems(6) == ("einsummable", [(2048, 96), (0, 80), (256, 120)])
    assert g.node_mems(11) == ("evict", [(0, 0), (2048, 96)])
    assert g.node_mems(13) == ("copy", [((1 << 40) + 16, 96), (8192, 96)])
    assert g.arena_bytes() == (1 << 40) + 16 + 96
    g.finalize(2)
    for i, n in enumerate(mg["nodes"]):
        deps = g.node_info(i)[2]
        assert set(n["inns"]) <= set(deps)
    # the second touch of group 3 also waits for the first one
    assert 9 in g.node_info(10)[2]


def test_load_errors():
    def load(nodes, loc=0, locs=1):
        g = ea.ApplyGraph(None)
        g.load_memgraph(mp.to_wire(dict(num_compute_locs=locs, num_storage_locs=0, nodes=nodes)),
                        loc=loc)
        return g

    with pytest.raises(ea.KmError, match="only allowing touches to have a group"):
        load([node("apply", loc=0, mems=[(0, 96), (96, 96)], einsummable=SCALE, group=2)])
    with pytest.raises(ea.KmError, match="needs both devices"):
        load([node("move", src_loc=1, src_offset=0, loc=0, offset=0, size=8)], locs=2)
    with pytest.raises(ea.KmError, match="memory ranges"):
        load([node("apply", loc=0, mems=[(0, 96)], einsummable=SCALE, group=-1)])
    with pytest.raises(ea.KmError):
        load([node("apply", loc=0, mems=[(0, 96), (96, 96)], group=-1,
                   einsummable=dict(SCALE, join="*[hole|f32@0"))])
    with pytest.raises(ea.KmError):
        load([node("constant", loc=0, offset=0, fill=dict(value="f33|1", shape=[4]))])
    # the same move is fine for a process that drives neither end: it becomes a dummy
    g = load([node("move", src_loc=1, src_offset=0, loc=2, offset=0, size=8)], locs=3)
    assert g.node_mems(0)[0] == "dummy"
    g = ea.ApplyGraph(None)
    g.add_dummy()
    with pytest.raises(ea.KmError, match="must be empty"):
        g.load_memgraph(mp.to_wire(sample_memgraph()))


def test_the_restated_schema_equals_the_reference_proto_field_for_field():
    # tests/golden/einsummable_proto_fields.json is written from the reference's .proto text by
    # tests/golden/make_proto_fields.py; the encoder of these tests is built from SCHEMA
    import json
    import os

    import memgraph_proto

    with open(os.path.join(os.path.dirname(__file__), "golden",
                           "einsummable_proto_fields.json")) as f:
        reference = json.load(f)
    for message, fields in memgraph_proto.SCHEMA.items():
        assert message in reference, message
        mine = sorted((f[0], f[1], f[2], f[3], f[4] if len(f) == 5 else None) for f in fields)
        theirs = sorted(tuple(f) for f in reference[message])
        assert mine == theirs, (message, mine, theirs)
