"""Serialized memgraphs replayed on the device (es_km_graph_load_memgraph): the bytes come
from the protobuf encoder of tests/memgraph_proto.py; the results are checked against the
oracle and against the same nodes launched one by one through the kernel manager."""
import numpy as np
import pytest

import einsummable_amd as ea
import memgraph_proto as mp
import oracle
from einsummable_amd.llama_layer import DeviceRunner, LayerGraph
from helpers import assert_close, normal, rng, stream_handle
from memgraph_proto import node
from test_gpu_llama_layer import make_inputs
from test_memgraph_wire import sample_memgraph

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n_streams", [1, 3])
def test_every_node_kind_runs(km, n_streams):
    import torch

    mg = sample_memgraph(far=10240)
    g = ea.ApplyGraph(km)
    g.load_memgraph(mp.to_wire(mg), loc=0, scalar_vars={"lr": 0.25})
    assert g.arena_bytes() == 12288 + 96
    g.finalize(n_streams)

    r = rng(500)
    init = r.randint(0, 256, size=g.arena_bytes()).astype(np.uint8)
    a, b = normal(r, 20, np.float32), normal(r, 30, np.float32)
    s7 = normal(r, 24, np.float32)
    assert g.node_mems(0) == ("dummy", [(0, 80)]) and g.node_mems(1) == ("dummy", [(256, 120)])
    init[0:80] = a.view(np.uint8)
    init[256:376] = b.view(np.uint8)
    g.storage_write(7, s7.tobytes())

    arena = torch.from_numpy(init.copy()).cuda()
    for _ in range(2):           # a second run starts from the first one's arena and storage
        g.run(stream_handle(), arena.data_ptr())
        torch.cuda.synchronize()
    got = arena.cpu().numpy()

    def f32(off, n):
        return got[off:off + 4 * n].view(np.float32)

    c = f32(2048, 24).reshape(4, 6)
    want_c = 0.25 * (a.reshape(4, 5).astype(np.float64) @ b.reshape(5, 6).astype(np.float64))
    assert_close(c, want_c.astype(np.float32), ea.F32)
    # fills, through the oracle; the lowertri arrives with rows and columns exchanged
    assert np.array_equal(f32(512, 24), oracle.fill_constant(np.float32, 0.5, 24))
    tri = oracle.fill_lowertri(np.float16, 0.0, -np.inf, 5, 3, -1)
    assert np.array_equal(got[1024:1054].view(np.uint16), tri.reshape(-1).view(np.uint16))
    assert tri[0, 2] == -np.inf and tri[0, 1] == 0 and tri[1, 2] == 0
    # the group: the first touch writes rows 1..3 of C into rows 2..4 of P, the second adds
    # the constant; the other rows of P keep what the arena held
    p = init[4096:4096 + 192].view(np.float32).reshape(8, 6).copy()
    dims = [(4, 8, 1, 2, 3), (6, 6, 0, 0, 6)]
    oracle.touch(dims, None, p, np.ascontiguousarray(c))
    oracle.touch(dims, "+", p, np.full((4, 6), 0.5, np.float32))
    assert np.array_equal(f32(4096, 48).view(np.uint32), p.reshape(-1).view(np.uint32))
    # evict -> storage -> load -> copy / move; the inputsto slot loaded as it was written
    cb = c.tobytes()
    assert g.storage_read(11, 96) == cb
    for off in (8192, 10240, 9216):
        assert got[off:off + 96].tobytes() == cb, off
    assert got[12288:12288 + 96].tobytes() == s7.tobytes()
    # nothing else was written
    touched = np.zeros(len(got), bool)
    for lo, n in ((512, 96), (1024, 30), (2048, 96), (4096, 192), (8192, 96), (9216, 96),
                  (10240, 96), (12288, 96)):
        touched[lo:lo + n] = True
    assert np.array_equal(got[~touched], init[~touched])


def layer_memgraph(graph, ranges, with_dels=False):
    """The decoder layer's node list as a memgraph: an inputmem per buffer nobody writes,
    an alloc per buffer somebody writes, one apply / constant per node, and the edges the
    memory ranges imply (the memgraph carries edges, not ranges, for ordering).  `with_dels`:
    a del node, behind all its readers, for every buffer that is neither an input nor the
    layer's output (memgraph.h: del_t)."""
    def overlap(x, y):
        return x[0] < y[0] + y[1] and y[0] < x[0] + x[1]

    written = {n["out"] for n in graph.nodes}
    nodes, first = [], {}
    for name, (off, size) in ranges.items():
        first[name] = len(nodes)
        nodes.append(node("alloc" if name in written else "inputmem", loc=0, offset=off, size=size))
    history = []                                       # (id, out range, [input ranges])
    for n in graph.nodes:
        out = ranges[n["out"]]
        if n["kind"] == "einsummable":
            inn_names = list(n["inns"])
        elif n["kind"] == "touch":
            inn_names = [n["inn"]]
        else:
            inn_names = []
        inns = [ranges[b] for b in inn_names]
        deps = {first[n["out"]]} | {first[b] for b in inn_names}
        for i, o, rs in history:
            if overlap(o, out) or any(overlap(o, x) for x in inns) or any(overlap(out, x) for x in rs):
                deps.add(i)
        m = mp.layer_node(n, deps, out, inns)
        history.append((len(nodes), out, inns))
        nodes.append(m)
    if with_dels:
        for name, (off, size) in ranges.items():
            readers = {i for i, _, rs in history if any(overlap((off, size), x) for x in rs)}
            if name in written and name != graph.output and readers:
                nodes.append(node("del", readers, loc=0, offset=off, size=size))
    return dict(num_compute_locs=1, num_storage_locs=0, nodes=nodes)


@pytest.mark.parametrize("n_streams", [1, 4])
def test_llama_layer_replayed_from_wire_equals_node_by_node_launches(km, n_streams):
    import torch

    lg = LayerGraph(dim=256, n_heads=4, ffn=688, seq=128)
    vals = make_inputs(lg, 5)
    seq = DeviceRunner(km, lg)
    ranges, off = {}, 0
    for name, nbytes in lg.buffers.items():
        ranges[name] = (off, nbytes)
        off += (nbytes + 255) // 256 * 256
    wire = mp.to_wire(layer_memgraph(lg, ranges))

    g = ea.ApplyGraph(km)
    n = g.load_memgraph(wire)
    assert n == len(lg.buffers) + len(lg.nodes)
    g.finalize(n_streams)
    arena = torch.zeros(g.arena_bytes(), dtype=torch.uint8, device="cuda")
    for k, v in vals.items():
        seq.set_input(k, v)
        o, nb = ranges[k]
        arena[o:o + nb] = torch.from_numpy(np.ascontiguousarray(v).view(np.uint8).reshape(-1)).cuda()
    seq.run()
    g.run(stream_handle(), arena.data_ptr())
    torch.cuda.synchronize()
    host = arena.cpu().numpy()
    for name, (o, nb) in ranges.items():
        assert np.array_equal(seq.get(name, np.uint8), host[o:o + nb]), name


def test_llama_layer_from_wire_optimized_keeps_the_result(km):
    """The del nodes of a serialized memgraph are what the optimisation pass needs: the layer
    loaded from the wire, optimised, gives the bytes of the node-by-node run in its output."""
    import torch

    lg = LayerGraph(dim=256, n_heads=4, ffn=688, seq=128)
    vals = make_inputs(lg, 6)
    seq = DeviceRunner(km, lg)
    ranges, off = {}, 0
    for name, nbytes in lg.buffers.items():
        ranges[name] = (off, nbytes)
        off += (nbytes + 255) // 256 * 256
    g = ea.ApplyGraph(km)
    g.load_memgraph(mp.to_wire(layer_memgraph(lg, ranges, with_dels=True)))
    assert g.optimize() == 40          # as when the runner adds the del nodes itself
    g.finalize(2)
    arena = torch.zeros(g.arena_bytes(), dtype=torch.uint8, device="cuda")
    for k, v in vals.items():
        seq.set_input(k, v)
        o, nb = ranges[k]
        arena[o:o + nb] = torch.from_numpy(np.ascontiguousarray(v).view(np.uint8).reshape(-1)).cuda()
    seq.run()
    g.run(stream_handle(), arena.data_ptr())
    torch.cuda.synchronize()
    host = arena.cpu().numpy()
    for name in (lg.output, "values.f", "sm.to_f16", "gate"):
        o, nb = ranges[name]
        assert np.array_equal(seq.get(name, np.uint8), host[o:o + nb]), name


def test_storage_slot_errors(km):
    g = ea.ApplyGraph(km)
    g.add_evict((0, 64), 3)
    with pytest.raises(ea.KmError, match="after finalize"):
        g.storage_write(3, b"\0" * 64)
    g.finalize(1)
    with pytest.raises(ea.KmError, match="no storage slot 4"):
        g.storage_read(4, 8)
    with pytest.raises(ea.KmError, match="too small"):
        g.storage_write(3, b"\0" * 65)


@pytest.mark.parametrize("n_streams", [1, 4])
def test_llama_layer_with_reused_ranges_optimized(km, n_streams):
    """The reference's layout: dels right behind the last user, freed ranges handed to later
    allocs, ordering carried by the memgraph's edges alone.  Optimised and spread over
    streams, the layer's output holds the bytes of the node-by-node run."""
    import torch

    lg = LayerGraph(dim=256, n_heads=4, ffn=688, seq=128)
    vals = make_inputs(lg, 7)
    seq = DeviceRunner(km, lg)
    mg, input_ranges, out_range, top = mp.layer_memgraph_reusing(lg)
    assert top < sum((b + 255) // 256 * 256 for b in lg.buffers.values())   # ranges were reused
    g = ea.ApplyGraph(km)
    g.load_memgraph(mp.to_wire(mg))
    assert g.optimize() > 10           # fewer than with private ranges: a reused range is often still read
    assert mp.unordered_conflicts(g) == []
    g.finalize(n_streams)
    arena = torch.zeros(max(g.arena_bytes(), top), dtype=torch.uint8, device="cuda")
    for k, v in vals.items():
        seq.set_input(k, v)
        o, nb = input_ranges[k]
        arena[o:o + nb] = torch.from_numpy(np.ascontiguousarray(v).view(np.uint8).reshape(-1)).cuda()
    seq.run()
    for _ in range(3):
        g.run(stream_handle(), arena.data_ptr())
    torch.cuda.synchronize()
    o, nb = out_range
    assert np.array_equal(seq.get(lg.output, np.uint8), arena[o:o + nb].cpu().numpy())
