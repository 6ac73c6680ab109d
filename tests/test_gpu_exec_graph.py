"""The exec-node layer (es_km_graph_*): dependency graphs of apply / fill / copy nodes over
one arena, placed on several streams.  Kernels are deterministic, so whatever the placement
the arena must end up with exactly the bytes of the same nodes run one after the other."""
import numpy as np
import pytest

import einsummable_amd as ea
from einsummable_amd.llama_layer import ArenaRunner, DeviceRunner, LayerGraph
from helpers import NP, normal, rng, stream_handle
from test_gpu_llama_layer import make_inputs

pytestmark = pytest.mark.gpu

E = ea.Einsummable
SLOT = 64 * 1024          # bytes per arena slot in the random graphs
N = SLOT // 4             # f32 elements per slot


def random_graph(r, n_nodes, n_slots):
    """Node descriptions over arena slots: unary / binary elementwise, row reductions into
    the head of a slot, copies, touches (grouped accumulations included) and fills."""
    nodes = []
    group_of_slot = {}
    for _ in range(n_nodes):
        kind = r.choice(["unary", "binary", "reduce", "copy", "touch", "group", "fill"],
                        p=[0.3, 0.25, 0.1, 0.1, 0.1, 0.1, 0.05])
        out = int(r.randint(1, n_slots))
        a, b = int(r.randint(0, n_slots)), int(r.randint(0, n_slots))
        if kind in ("unary", "copy", "touch", "group", "reduce") and a == out:
            a = (a + 1) % n_slots
        if kind == "binary" and (a == out or b == out):
            kind = "fill"
        nodes.append((kind, out, a, b))
    return nodes


def add_nodes(g, nodes):
    ids = []
    groups = {}
    for kind, out, a, b in nodes:
        mo, ma, mb = (out * SLOT, SLOT), (a * SLOT, SLOT), (b * SLOT, SLOT)
        if kind == "unary":
            i = g.add_einsummable(E([N], [[0]], 1, "*[constant{f32|0.5},hole|f32@0]"), [mo, ma])
        elif kind == "binary":
            i = g.add_einsummable(E([N], [[0], [0]], 1, "+[hole|f32@0,hole|f32@1]"), [mo, ma, mb])
        elif kind == "reduce":
            i = g.add_einsummable(E([64, N // 64], [[0, 1]], 1, "hole|f32@0", "^"),
                                  [(out * SLOT, 64 * 4), ma])
        elif kind == "copy":
            i = g.add_copy(out * SLOT, a * SLOT, SLOT)
        elif kind == "touch":
            t = ea.Touch([(128, 128, 0, 0, 128), (N // 128, N // 128, 3, 5, 40)], "+", ea.F32)
            i = g.add_touch(t, -1, [mo, ma])       # no group: runs as a copy
        elif kind == "group":
            t = ea.Touch([(N, N, 0, 0, N)], "+", ea.F32)
            i = g.add_touch(t, groups.setdefault(out, len(groups)), [mo, ma])
        else:
            i = g.add_constant_fill(ea.F32, int(np.float32(1.25).view(np.uint32)), N, mo)
        ids.append(i)
    return ids


def oracle_run(nodes, init):
    """The same node list applied one after the other by the CPU oracle; returns the arena."""
    import oracle

    arena = init.copy()
    slot = lambda k: arena[k * N:(k + 1) * N]
    seen_groups = set()
    for kind, out, a, b in nodes:
        if kind == "unary":
            slot(out)[:] = oracle.einsummable([N], [[0]], 1, "*[constant{f32|0.5},hole|f32@0]",
                                              None, [slot(a).copy()], oracle.EXACT)
        elif kind == "binary":
            slot(out)[:] = oracle.einsummable([N], [[0], [0]], 1, "+[hole|f32@0,hole|f32@1]", None,
                                              [slot(a).copy(), slot(b).copy()], oracle.EXACT)
        elif kind == "reduce":
            slot(out)[:64] = oracle.einsummable([64, N // 64], [[0, 1]], 1, "hole|f32@0", "^",
                                                [slot(a).copy()], oracle.EXACT)
        elif kind == "copy":
            slot(out)[:] = slot(a)
        elif kind == "touch":
            dims = [(128, 128, 0, 0, 128), (N // 128, N // 128, 3, 5, 40)]
            o = np.ascontiguousarray(slot(out))
            oracle.touch(dims, None, o, np.ascontiguousarray(slot(a)))
            slot(out)[:] = o
        elif kind == "group":
            o = np.ascontiguousarray(slot(out))
            oracle.touch([(N, N, 0, 0, N)], "+" if out in seen_groups else None, o,
                         np.ascontiguousarray(slot(a)))
            seen_groups.add(out)
            slot(out)[:] = o
        else:
            slot(out)[:] = oracle.fill_constant(np.float32, 1.25, N)
    return arena


@pytest.mark.parametrize("seed", range(6))
def test_random_graphs_give_the_sequential_bytes_on_any_number_of_streams(km, seed):
    import torch

    r = rng(100 + seed)
    n_slots = 12
    nodes = random_graph(r, 60, n_slots)
    init = normal(r, n_slots * N, np.float32)
    results = []
    for n_streams in (1, 2, 5):
        g = ea.ApplyGraph(km)
        ids = add_nodes(g, nodes)
        g.add_memory_dependencies()
        g.finalize(n_streams)
        arena = torch.from_numpy(init.copy()).cuda()
        g.run(stream_handle(), arena.data_ptr())
        torch.cuda.synchronize()
        results.append(arena.cpu().numpy())
        streams = {g.node_info(i)[1] for i in ids}
        assert max(streams) < n_streams
        if n_streams == 1:
            assert g.cross_stream_waits() == 0
    assert np.array_equal(results[0].view(np.uint32), results[1].view(np.uint32))
    assert np.array_equal(results[0].view(np.uint32), results[2].view(np.uint32))
    assert not np.array_equal(results[0], init)
    # every operation of these graphs is a single exactly rounded f32 operation, a maximum or
    # a move: the oracle's arena must hold the same values (a product may differ in the sign
    # of a zero)
    want = oracle_run(nodes, init)
    assert np.array_equal(results[0], want)


@pytest.mark.parametrize("seed", range(4))
def test_a_host_event_loop_drives_the_nodes_one_by_one_through_completion_callbacks(km, seed):
    # what the reference's exec_state_t does (src/engine/exec_state.cc:197-219): launch a
    # node when everything it depends on has reported back, on a stream and with a workspace
    # taken from pools, and learn of its completion through a callback behind it on the stream
    import queue

    import torch

    r = rng(140 + seed)
    n_slots = 12
    nodes = random_graph(r, 60, n_slots)
    init = normal(r, n_slots * N, np.float32)
    g = ea.ApplyGraph(km)
    ids = add_nodes(g, nodes)
    g.add_memory_dependencies()
    g.finalize(1)
    deps = {i: set(g.node_info(i)[2]) for i in ids}
    users = {i: [j for j in ids if i in deps[j]] for i in ids}
    arena = torch.from_numpy(init.copy()).cuda()
    torch.cuda.synchronize()

    streams, workspaces = ea.StreamPool(0, 3), ea.WorkspacePool(0)
    done = queue.Queue()
    callback = ea.NodeCallback(lambda user: done.put(int(user) - 1))
    waiting = {i: len(deps[i]) for i in ids}
    ready = [i for i in ids if waiting[i] == 0]
    held, started_groups, in_flight, finished, order = {}, set(), 0, 0, []
    while finished != len(ids):
        while ready:
            s = streams.try_acquire()
            if not s:
                break
            i = ready.pop(int(r.randint(0, len(ready))))     # any ready node may go next
            need = g.node_workspace(i)
            ws = workspaces.acquire(need) if need else None
            group = g.node_group(i)
            first = -1
            if group >= 0:
                first = 0 if group in started_groups else 1
                started_groups.add(group)
            g.launch_node(i, s, arena.data_ptr(), ws, first, callback, i + 1)
            held[i] = (s, ws)
            in_flight += 1
            order.append(i)
        i = done.get(timeout=60)
        s, ws = held.pop(i)
        streams.release(s)
        if ws:
            workspaces.release(ws[0])
        in_flight -= 1
        finished += 1
        for j in users[i]:
            waiting[j] -= 1
            if waiting[j] == 0:
                ready.append(j)
    torch.cuda.synchronize()
    assert in_flight == 0 and sorted(order) == sorted(ids)
    assert order != sorted(order) or len(ids) < 3          # the loop did reorder independent nodes
    got = arena.cpu().numpy()
    assert np.array_equal(got, oracle_run(nodes, init))
    streams.close()
    workspaces.close()


def test_workspace_and_stream_pools(km):
    pool = ea.WorkspacePool(0)
    a, size_a = pool.acquire(1 << 20)
    b, size_b = pool.acquire(1 << 16)
    assert a != b and size_a >= 1 << 20 and size_b >= 1 << 16 and pool.blocks() == 2
    pool.release(a)
    c, size_c = pool.acquire(1 << 10)                       # the first free block that is large enough
    assert c == a and size_c == size_a and pool.blocks() == 2
    with pytest.raises(ea.KmError):
        pool.release(12345)
    pool.release(b)
    pool.release(c)
    pool.close()
    streams = ea.StreamPool(0, 2)
    s0, s1 = streams.try_acquire(), streams.try_acquire()
    assert s0 and s1 and s0 != s1 and streams.try_acquire() is None
    streams.release(s0)
    with pytest.raises(ea.KmError):
        streams.release(s0)                                 # not out
    assert streams.try_acquire() == s0
    streams.close()


def test_touch_groups_first_member_initialises_then_members_accumulate_in_order(km):
    import torch

    r = rng(120)
    n = 4096
    parts = [normal(r, n, np.float16) for _ in range(5)]
    arena = torch.zeros(6 * n, dtype=torch.float16, device="cuda")
    arena[:n] = 777.0                                   # stale bytes the first touch must replace
    for k, p in enumerate(parts):
        arena[(k + 1) * n:(k + 2) * n] = torch.from_numpy(p).cuda()
    g = ea.ApplyGraph(km)
    t = ea.Touch([(n, n, 0, 0, n)], "+", ea.F16)
    for k in range(5):
        g.add_touch(t, 7, [(0, 2 * n), ((k + 1) * 2 * n, 2 * n)])
    g.finalize(3)
    g.run(stream_handle(), arena.data_ptr())
    torch.cuda.synchronize()
    want = parts[0].copy()
    for p in parts[1:]:
        want = (want + p).astype(np.float16)            # fp16 rounding after every touch
    assert np.array_equal(arena[:n].cpu().numpy().view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("n_streams", [1, 3])
def test_a_group_of_64_touches_runs_as_one_launch_with_the_oracles_bytes(km, n_streams):
    # the memory-movement configuration as the engine would hold it: 64 accumulating touches
    # of 512 x 512 blocks into windows of one 2048 x 2048 output at odd offsets, all of one
    # group, each with its own input range; then a second group into another output
    import torch

    import oracle

    r = rng(121)
    n, blk, count = 2048, 512, 64
    out_bytes, blk_bytes = n * n * 2, blk * blk * 2
    blocks = [normal(r, blk * blk, np.float16) for _ in range(count)]
    offs = [(int(r.randint(0, n - blk + 1)), int(r.randint(0, n - blk + 1))) for _ in range(count)]
    arena = torch.empty((2 * out_bytes + count * blk_bytes) // 2, dtype=torch.float16, device="cuda")
    arena[:2 * n * n] = 777.0                      # stale bytes: the first touch of a group replaces its window only
    init = arena[:2 * n * n].cpu().numpy().copy()
    for k, b in enumerate(blocks):
        lo = (2 * out_bytes + k * blk_bytes) // 2
        arena[lo:lo + blk * blk] = torch.from_numpy(b).cuda()
    g = ea.ApplyGraph(km)
    for which in range(2):
        for k in range(count):
            ro, co = offs[k] if which == 0 else offs[count - 1 - k]
            t = ea.Touch([(blk, n, 0, ro, blk), (blk, n, 0, co, blk)], "+", ea.F16)
            g.add_touch(t, 40 + which, [(which * out_bytes, out_bytes),
                                        (2 * out_bytes + k * blk_bytes, blk_bytes)])
    g.finalize(n_streams)
    assert g.launches() == 2, g.launches()
    g.run(stream_handle(), arena.data_ptr())
    torch.cuda.synchronize()
    got = arena[:2 * n * n].cpu().numpy()
    for which in range(2):
        want = init[which * n * n:(which + 1) * n * n].copy()
        for k in range(count):
            ro, co = offs[k] if which == 0 else offs[count - 1 - k]
            dims = [(blk, n, 0, ro, blk), (blk, n, 0, co, blk)]
            want = oracle.touch(dims, None if k == 0 else "+", want, blocks[k])
        assert np.array_equal(got[which * n * n:(which + 1) * n * n].view(np.uint16),
                              want.view(np.uint16)), which


@pytest.mark.parametrize("n_streams", [1, 2, 4])
def test_llama_layer_through_the_exec_graph_equals_node_by_node_launches(km, n_streams):
    import torch

    g = LayerGraph(dim=256, n_heads=4, ffn=688, seq=128)
    vals = make_inputs(g, 3)
    seq = DeviceRunner(km, g)
    par = ArenaRunner(km, g, n_streams)
    for k, v in vals.items():
        seq.set_input(k, v)
        par.set_input(k, v)
    seq.run()
    par.run()
    torch.cuda.synchronize()
    for name in g.buffers:
        assert np.array_equal(seq.get(name, np.uint8), par.get(name, np.uint8)), name
    if n_streams > 1:
        assert par.graph.cross_stream_waits() > 0
        assert len({par.graph.node_info(i)[1] for i in par.ids}) > 1


def surviving_buffers(runner):
    """Names of the ranges some node still writes after the graph's optimisation pass."""
    by_offset = {off: name for name, (off, _) in runner.ranges.items()}
    names = set()
    for i in runner.ids:
        text = runner.graph.describe(i)
        if not text.startswith("dummy"):
            names.add(by_offset[int(text.split()[1].split(":")[0])])
    return names


@pytest.mark.parametrize("shape,n_streams", [
    (dict(dim=256, n_heads=4, ffn=688, seq=128), 1),
    (dict(dim=256, n_heads=4, ffn=688, seq=128), 4),
    (dict(dim=192, n_heads=2, ffn=520, seq=72), 2),       # extents off the vector grid
    (dict(), 4),                                          # LLaMA-7B: 4096, 32 heads, 11008, 2048
])
def test_optimized_layer_keeps_every_stored_bit(km, shape, n_streams):
    """Formation copies absorbed into their producers and single-reader elementwise nodes
    merged into their readers: fewer launches, and every range that is still written holds
    exactly the bytes of the node-by-node run."""
    import torch

    g = LayerGraph(**shape)
    vals = make_inputs(g, 11)
    plain = ArenaRunner(km, g, n_streams)
    fused = ArenaRunner(km, g, n_streams, optimize=True)
    # 13 formation copies and 17 elementwise nodes: in each of the two norms to_f32 (taken in
    # by the square and by x * rstd), the square (taken in by the row sum, which deals a row
    # of 2-byte elements to the lanes as it deals one of 4-byte elements), mean_eps, x_rstd
    # and to_f16; scores+mask, to_f32 (taken in by the row max and by x - max), x - max, exp
    # (taken in by the row sum and by the division), the division; silu; the first residual
    # (taken in by the second norm and by the second residual).  Then three chains over
    # rows: each norm's sum of squares and its (mean + eps)^-1/2 go into x * rstd * w, the
    # softmax's row max and row sum into the quotient.  And the conversions around the two
    # rotary products (to_f32 in front, to_f16 behind) go into the products, which read and
    # write pairs of f16.
    assert fused.absorbed == 13 + 17 + 6 + 4, fused.absorbed
    # (sibling projections that now follow each other may share a launch on top of that)
    assert fused.graph.launches() <= plain.graph.launches() - fused.absorbed
    for k, v in vals.items():
        plain.set_input(k, v)
        fused.set_input(k, v)
    plain.run()
    fused.run()
    torch.cuda.synchronize()
    kept = surviving_buffers(fused)
    assert g.output in kept and "sm.to_f16" in kept and "values.f" in kept
    for gone in ("scores", "sm.to_f32", "sm.sub", "sm.exp", "sm.div", "an.square", "silu", "residual1",
                 "sm.rowmax.f", "sm.rowsum.f"):
        assert gone not in kept, gone
    for name in sorted(kept):
        a, b = plain.view(name), fused.view(name)
        assert torch.equal(a, b), name


def random_ssa_graph(r, n_nodes):
    """Every node writes a slot of its own: elementwise nodes whose joins invite a fused
    multiply-add across a merge, conversions through f16, broadcasts of a row statistic, row
    maxima and sums, whole-range copies.  Returns (nodes, slot sizes, input slots)."""
    R, C = 64, 96
    n = R * C
    bounded = "*[hole|f32@0,power{-1}[+[constant{f32|1},*[hole|f32@0,hole|f32@0]]]]"   # x / (1 + x^2)
    full = [("f32", n)] * 3          # slots 0..2 are inputs
    kinds = ["f32"] * 3
    nodes = []
    def pick(kind):
        c = [i for i, k in enumerate(kinds) if k == kind]
        return int(c[r.randint(0, len(c))]) if c else None
    for _ in range(n_nodes):
        op = r.choice(["bounded", "axpy", "mul", "half", "unhalf", "rowmax", "rowsum", "bcast", "copy",
                       "scale"], p=[0.15, 0.15, 0.1, 0.1, 0.1, 0.08, 0.08, 0.1, 0.07, 0.07])
        out = len(kinds)
        a, b = pick("f32"), pick("f32")
        if op == "bounded":
            nodes.append((E([n], [[0]], 1, bounded), out, [a])); kinds.append("f32")
        elif op == "scale":
            nodes.append((E([R, C], [[0, 1]], 2, "*[constant{f32|0.75},hole|f32@0]"), out, [a])); kinds.append("f32")
        elif op == "axpy":
            nodes.append((E([n], [[0], [0]], 1, "+[*[constant{f32|1.7},hole|f32@0],hole|f32@1]"), out, [a, b]))
            kinds.append("f32")
        elif op == "mul":
            nodes.append((E([R, C], [[0, 1], [0, 1]], 2, "*[hole|f32@0,hole|f32@1]"), out, [a, b])); kinds.append("f32")
        elif op == "half":
            nodes.append((E([n], [[0]], 1, "to_f16[hole|f32@0]"), out, [a])); kinds.append("f16")
        elif op == "unhalf":
            h = pick("f16")
            if h is None:
                continue
            nodes.append((E([n], [[0]], 1, "to_f32[hole|f16@0]"), out, [h])); kinds.append("f32")
        elif op in ("rowmax", "rowsum"):
            nodes.append((E([R, C], [[0, 1]], 1, "hole|f32@0", "^" if op == "rowmax" else "+"), out, [a]))
            kinds.append("row")
        elif op == "bcast":
            row = pick("row")
            if row is None:
                continue
            nodes.append((E([R, C], [[0, 1], [0]], 2, "+[hole|f32@0,*[constant{f32|-0.01},hole|f32@1]]"), out,
                          [a, row]))
            kinds.append("f32")
        else:
            nodes.append((ea.Touch([(n, n, 0, 0, n)], None, ea.F32), out, [a])); kinds.append("f32")
    size = {"f32": 4 * n, "f16": 2 * n, "row": 4 * R}
    return nodes, [size[k] for k in kinds], 3


@pytest.mark.parametrize("seed", range(8))
def test_optimized_random_graphs_keep_every_stored_bit(km, seed):
    import torch

    r = rng(300 + seed)
    nodes, sizes, n_inputs = random_ssa_graph(r, 40)
    offs = np.concatenate([[0], np.cumsum([(s + 255) // 256 * 256 for s in sizes])]).astype(np.int64)
    mem = lambda k: (int(offs[k]), sizes[k])
    init = normal(r, int(offs[-1]) // 4, np.float32)
    arenas, graphs, ids = [], [], []
    for optimize in (False, True):
        g = ea.ApplyGraph(km)
        my = []
        last_reader = {}
        for what, out, inns in nodes:
            if isinstance(what, ea.Touch):
                i = g.add_touch(what, -1, [mem(out), mem(inns[0])])
            else:
                i = g.add_einsummable(what, [mem(out)] + [mem(k) for k in inns])
            my.append(i)
            for k in inns:
                last_reader[k] = i
        # del nodes for most of what is read at all; the rest counts as results
        rr = rng(400 + seed)
        for k, i in sorted(last_reader.items()):
            if k >= n_inputs and rr.uniform() < 0.85:
                g.add_dummy(mem(k), [i])
        g.add_memory_dependencies()
        absorbed = g.optimize() if optimize else 0
        g.finalize(2)
        arena = torch.from_numpy(init.copy()).cuda()
        g.run(stream_handle(), arena.data_ptr())
        torch.cuda.synchronize()
        arenas.append(arena.cpu().numpy().view(np.uint8))
        graphs.append(g)
        ids.append(my)
    assert absorbed > 0
    assert graphs[1].launches() == graphs[0].launches() - absorbed
    kept = 0
    for (what, out, inns), i in zip(nodes, ids[1]):
        if graphs[1].describe(i).startswith("dummy"):
            continue
        lo, nb = mem(out)
        assert np.array_equal(arenas[0][lo:lo + nb], arenas[1][lo:lo + nb]), (seed, i, graphs[1].describe(i))
        kept += 1
    assert kept > 0


@pytest.mark.parametrize("n_streams", [
    1,
    pytest.param(4, marks=pytest.mark.skip(
        reason="capturing a run that forks to and joins from pool streams ended in a "
               "host-side segmentation fault inside the HIP runtime (ROCm 7.2); no cause "
               "found in this code, so the combination is refused by ArenaRunner.capture")),
])
def test_exec_graph_captured_into_a_hip_graph_replays_the_eager_bytes(km, n_streams):
    import torch

    g = LayerGraph(dim=256, n_heads=4, ffn=688, seq=128)
    par = ArenaRunner(km, g, n_streams)
    for k, v in make_inputs(g, 5).items():
        par.set_input(k, v)
    hip_graph = par.capture()
    for seed in (6, 7, 8):
        for k, v in make_inputs(g, seed).items():
            par.set_input(k, v)
        par.run()
        torch.cuda.synchronize()
        eager = {n: par.get(n, np.uint8).copy() for n in ("residual2", "sm.div", "mask")}
        for n in eager:
            par.view(n).zero_()
        torch.cuda.synchronize()
        hip_graph.replay()
        torch.cuda.synchronize()
        for n, want in eager.items():
            assert np.array_equal(par.get(n, np.uint8), want), (seed, n)


def test_exec_graph_errors(km):
    g = ea.ApplyGraph(km)
    e = E([16], [[0]], 1, "hole|f32@0")
    with pytest.raises(ea.KmError) as ei:
        g.add_einsummable(e, [(0, 64), (64, 64)], deps=[0])      # depends on itself / later
    assert ei.value.code == -1
    with pytest.raises(ea.KmError) as ei:
        g.add_einsummable(e, [(0, 64)])                           # an input range is missing
    assert ei.value.code == -4
    a = g.add_einsummable(e, [(0, 64), (64, 64)])
    with pytest.raises(ea.KmError) as ei:
        g.run(0, 1)                                               # run before finalize
    assert ei.value.code == -2
    g.finalize(2)
    with pytest.raises(ea.KmError):
        g.add_einsummable(e, [(0, 64), (64, 64)], deps=[a])      # immutable after finalize


@pytest.mark.parametrize("m,n,k,runs", [(2048, 4096, 4096, 3), (2048, 11008, 4096, 2), (384, 512, 256, 5),
                                         (1000, 3000, 4096, 2)])
def test_sibling_products_in_one_launch(km, monkeypatch, m, n, k, runs):
    """Independent products of one shape that follow each other (q, k and v of one input; w1
    and w3) go out as one launch of the persistent kernel: the same bits as one by one."""
    import torch

    e = E.from_str("ij,kj->ik", dict(i=m, j=k, k=n), "*[hole|f16@0,hole|f16@1]", "+")
    r = rng(m + runs)
    x = normal(r, m * k, np.float16, 0.5)
    ws = [normal(r, n * k, np.float16, 0.5) for _ in range(runs)]
    sizes = [m * k * 2] + [n * k * 2] * runs + [m * n * 2] * runs
    offs = np.concatenate([[0], np.cumsum([(s + 255) // 256 * 256 + 256 for s in sizes])]).astype(np.int64)
    mem = lambda i: (int(offs[i]), sizes[i])
    results = []
    for grouped in (False, True):
        monkeypatch.setenv("ES_KM_GEMM_GROUPS", "1" if grouped else "0")
        g = ea.ApplyGraph(km)
        ids = [g.add_einsummable(e, [mem(1 + runs + j), mem(0), mem(1 + j)]) for j in range(runs)]
        g.add_memory_dependencies()
        g.finalize(1)
        if "waves=4+4 persistent" in km.describe(e) and (m // 128) * (n // 256) <= 256:
            assert g.launches() == (1 if grouped else runs)
        arena = torch.zeros(int(offs[-1]), dtype=torch.uint8, device="cuda")
        arena[offs[0]:offs[0] + sizes[0]] = torch.from_numpy(x.view(np.uint8)).cuda()
        for j, w in enumerate(ws):
            arena[offs[1 + j]:offs[1 + j] + sizes[1 + j]] = torch.from_numpy(w.view(np.uint8)).cuda()
        g.run(stream_handle(), arena.data_ptr())
        torch.cuda.synchronize()
        results.append(arena.cpu().numpy())
    assert np.array_equal(results[0], results[1])
    got = results[1][offs[1 + runs]:offs[1 + runs] + sizes[1 + runs]].view(np.float16).astype(np.float32)
    want = x.astype(np.float32).reshape(m, k) @ ws[0].astype(np.float32).reshape(n, k).T
    assert np.allclose(got.reshape(m, n), want, rtol=1e-2, atol=0.05 * np.sqrt(k) * 0.25)
