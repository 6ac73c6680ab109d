"""Chains over rows (apply_graph_t::optimize, cg_chain_t): row reductions, pointwise steps on
their per-row results and the elementwise node that uses them run as one launch that keeps a
row in registers.  The chain computes every stage as its own kernel would, in the same order
and with the same roundings, so the arena must hold, in every range that is still written,
exactly the bytes of the node-by-node run; one case is also checked against the oracle."""
import numpy as np
import pytest

import einsummable_amd as ea
from helpers import NP, assert_close, normal, oracle_einsummable, rng, stream_handle

pytestmark = pytest.mark.gpu

E = ea.Einsummable
DT = {"f16": ea.F16, "f32": ea.F32}


@pytest.fixture(scope="module")
def km():
    return ea.KernelManager(0)


def layout(sizes, misalign=0):
    """Arena offsets (256-byte aligned, plus `misalign` bytes on every one) of buffers of
    these byte sizes."""
    offs, at = [], 0
    for s in sizes:
        offs.append(at + misalign)
        at += (s + misalign + 255) // 256 * 256
    return offs, at


def run_both(km, build, arena_bytes, init, env=None):
    """build(g) adds the nodes and returns the ranges to compare; runs the graph as listed
    and optimised.  Returns (arena bytes plain, arena bytes optimised, graphs, absorbed)."""
    import torch

    arenas, graphs, absorbed = [], [], 0
    for optimize in (False, True):
        g = ea.ApplyGraph(km)
        build(g)
        g.add_memory_dependencies()
        if optimize:
            absorbed = g.optimize()
        g.finalize(1)
        arena = torch.from_numpy(init.copy()).cuda()
        assert arena.numel() >= arena_bytes
        g.run(stream_handle(), arena.data_ptr())
        torch.cuda.synchronize()
        arenas.append(arena.cpu().numpy())
        graphs.append(g)
    return arenas[0], arenas[1], graphs, absorbed


def softmax_nodes(lead, n, xdt, with_mask):
    """row max, sum of exp(x - max), exp(x - max) / sum over [lead..., n]; statistics in f32"""
    R = len(lead) + 1
    full, rows = list(range(R)), list(range(R - 1))
    x = "hole|%s@0" % xdt
    if with_mask:
        inner = "+[hole|%s@0,hole|%s@1]" % (xdt, xdt)
        k = 2
        ins = [full, [R - 2, R - 1]]
    else:
        inner = x
        k = 1
        ins = [full]
    up = inner if xdt == "f32" else "to_f32[%s]" % inner
    shifted = "+[%s,*[constant{f32|-1},hole|f32@%d]]" % (up, k)
    quotient = "*[exp[%s],power{-1}[hole|f32@%d]]" % (shifted, k + 1)
    rmax = E(lead + [n], ins, R - 1, up, "^")
    rsum = E(lead + [n], ins + [rows], R - 1, "exp[%s]" % shifted, "+")
    norm = E(lead + [n], ins + [rows, rows], R,
             quotient if xdt == "f32" else "to_f16[%s]" % quotient)
    return rmax, rsum, norm


@pytest.mark.parametrize("lead,n,xdt,with_mask,in_place", [
    ([4, 64], 2048, "f16", True, False),     # teams of 64 lanes, four vectors each
    ([3, 5], 1000, "f16", True, False),      # the last vectors of a row are missing
    ([2, 8], 8192, "f16", False, True),      # teams of 256 lanes, the output on the input
    ([1, 7], 4104, "f16", False, False),     # 513 vectors: 256 lanes, the third round nearly empty
    ([6, 32], 2048, "f32", True, False),     # 32-byte vectors
    ([2, 3], 24, "f16", True, False),        # three vectors in a row
    ([5, 16], 777, "f32", False, True),      # odd row length: one element per vector
])
def test_softmax_chain_keeps_every_bit(km, lead, n, xdt, with_mask, in_place):
    rmax, rsum, norm = softmax_nodes(lead, n, xdt, with_mask)
    rows = int(np.prod(lead))
    esz = 2 if xdt == "f16" else 4
    sizes = [rows * n * esz, lead[-1] * n * esz, rows * 4, rows * 4, rows * n * esz]
    (X, M, mx, l, P), total = layout(sizes)
    if in_place:
        P = X
    ins = [(X, sizes[0])] + ([(M, sizes[1])] if with_mask else [])

    def build(g):
        a = g.add_einsummable(rmax, [(mx, sizes[2])] + ins)
        b = g.add_einsummable(rsum, [(l, sizes[3])] + ins + [(mx, sizes[2])])
        c = g.add_einsummable(norm, [(P, sizes[4])] + ins + [(mx, sizes[2]), (l, sizes[3])])
        g.add_dummy((mx, sizes[2]), [b, c])
        g.add_dummy((l, sizes[3]), [c])

    r = rng(7 + n)
    init = np.zeros(total, np.uint8)
    x = normal(r, rows * n, NP[DT[xdt]], 2.0)
    m = np.where(r.uniform(size=lead[-1] * n) < 0.3, -30.0, 0.0).astype(NP[DT[xdt]])
    init[X:X + sizes[0]] = x.view(np.uint8)
    init[M:M + sizes[1]] = m.view(np.uint8)
    plain, fused, graphs, absorbed = run_both(km, build, total, init)
    assert absorbed == 2 and graphs[1].launches() == 1
    assert graphs[1].describe(2).startswith("chain ")
    assert np.array_equal(plain[P:P + sizes[4]], fused[P:P + sizes[4]])
    if not in_place:
        assert np.array_equal(fused[X:X + sizes[0]], init[X:X + sizes[0]])
    # the chain's result is a softmax: against the oracle's node-by-node evaluation
    if n == 2048 and xdt == "f16":
        xs = x.reshape(lead + [n])
        inputs = [xs] + ([m.reshape(lead[-1], n)] if with_mask else [])
        want_max = oracle_einsummable(rmax, inputs)
        want_sum = oracle_einsummable(rsum, inputs + [want_max])
        want = oracle_einsummable(norm, inputs + [want_max, want_sum])
        got = fused[P:P + sizes[4]].view(NP[DT[xdt]]).reshape(-1)
        assert_close(got, np.asarray(want).reshape(-1), DT[xdt], what="softmax chain")


def test_normalisation_chain_with_a_pointwise_step(km):
    """sum of squares -> (mean + eps)^-1/2 -> x * r * w: a reduction, a step on the per-row
    value and the elementwise node, with a weight that has the row's mode only."""
    T, D = 200, 4096
    sq = E([T, D], [[0, 1]], 1, "power{2}[to_f32[hole|f16@0]]", "+")
    rstd = E([T], [[0]], 1, "power{-0.5}[+[*[constant{f32|%r},hole|f32@0],constant{f32|1e-06}]]" % (1.0 / D))
    scale = E([T, D], [[0, 1], [0], [1]], 2, "*[to_f16[*[to_f32[hole|f16@0],hole|f32@1]],hole|f16@2]")
    sizes = [T * D * 2, D * 2, T * 4, T * 4, T * D * 2]
    (X, W, ss, rs, Y), total = layout(sizes)

    def build(g):
        a = g.add_einsummable(sq, [(ss, sizes[2]), (X, sizes[0])])
        b = g.add_einsummable(rstd, [(rs, sizes[3]), (ss, sizes[2])])
        c = g.add_einsummable(scale, [(Y, sizes[4]), (X, sizes[0]), (rs, sizes[3]), (W, sizes[1])])
        g.add_dummy((ss, sizes[2]), [b])
        g.add_dummy((rs, sizes[3]), [c])

    r = rng(21)
    init = np.zeros(total, np.uint8)
    init[X:X + sizes[0]] = normal(r, T * D, np.float16, 1.5).view(np.uint8)
    init[W:W + sizes[1]] = normal(r, D, np.float16, 1.0).view(np.uint8)
    plain, fused, graphs, absorbed = run_both(km, build, total, init)
    assert absorbed == 2 and graphs[1].launches() == 1
    assert np.array_equal(plain[Y:Y + sizes[4]], fused[Y:Y + sizes[4]])


def test_a_statistic_that_is_a_result_stays(km):
    """Without its del node the row maximum is a result of the graph: it keeps its node and
    its place in memory, and the chain is what follows it."""
    lead, n = [2, 16], 512
    rmax, rsum, norm = softmax_nodes(lead, n, "f16", False)
    rows = 32
    sizes = [rows * n * 2, rows * 4, rows * 4, rows * n * 2]
    (X, mx, l, P), total = layout(sizes)

    def build(g):
        a = g.add_einsummable(rmax, [(mx, sizes[1]), (X, sizes[0])])
        b = g.add_einsummable(rsum, [(l, sizes[2]), (X, sizes[0]), (mx, sizes[1])])
        c = g.add_einsummable(norm, [(P, sizes[3]), (X, sizes[0]), (mx, sizes[1]), (l, sizes[2])])
        g.add_dummy((l, sizes[2]), [c])       # the maximum is kept, the sum is deleted

    r = rng(5)
    init = np.zeros(total, np.uint8)
    init[X:X + sizes[0]] = normal(r, rows * n, np.float16, 2.0).view(np.uint8)
    plain, fused, graphs, absorbed = run_both(km, build, total, init)
    # the sum goes into the chain (a reduction that reads the stored maximum), the maximum stays
    assert absorbed == 1 and graphs[1].launches() == 2
    assert graphs[1].describe(0).startswith("einsummable ")
    for lo, nb in ((mx, sizes[1]), (P, sizes[3])):
        assert np.array_equal(plain[lo:lo + nb], fused[lo:lo + nb])


def test_chain_on_buffers_that_are_not_16_byte_aligned_is_left_alone(km):
    lead, n = [2, 16], 512
    rmax, rsum, norm = softmax_nodes(lead, n, "f16", False)
    rows = 32
    sizes = [rows * n * 2, rows * 4, rows * 4, rows * n * 2]
    (X, mx, l, P), total = layout(sizes, misalign=8)

    def build(g):
        a = g.add_einsummable(rmax, [(mx, sizes[1]), (X, sizes[0])])
        b = g.add_einsummable(rsum, [(l, sizes[2]), (X, sizes[0]), (mx, sizes[1])])
        c = g.add_einsummable(norm, [(P, sizes[3]), (X, sizes[0]), (mx, sizes[1]), (l, sizes[2])])
        g.add_dummy((mx, sizes[1]), [b, c])
        g.add_dummy((l, sizes[2]), [c])

    r = rng(6)
    init = np.zeros(total, np.uint8)
    init[X:X + sizes[0]] = normal(r, rows * n, np.float16, 2.0).view(np.uint8)
    plain, fused, graphs, absorbed = run_both(km, build, total, init)
    assert absorbed == 0 and graphs[1].launches() == 3
    assert np.array_equal(plain[P:P + sizes[3]], fused[P:P + sizes[3]])


def test_chain_switched_off_by_the_environment(km, monkeypatch):
    monkeypatch.setenv("ES_KM_ROW_CHAINS", "0")
    lead, n = [2, 16], 512
    rmax, rsum, norm = softmax_nodes(lead, n, "f16", False)
    g = ea.ApplyGraph(km)
    sizes = [32 * n * 2, 128, 128, 32 * n * 2]
    (X, mx, l, P), total = layout(sizes)
    a = g.add_einsummable(rmax, [(mx, sizes[1]), (X, sizes[0])])
    b = g.add_einsummable(rsum, [(l, sizes[2]), (X, sizes[0]), (mx, sizes[1])])
    c = g.add_einsummable(norm, [(P, sizes[3]), (X, sizes[0]), (mx, sizes[1]), (l, sizes[2])])
    g.add_dummy((mx, sizes[1]), [b, c])
    g.add_dummy((l, sizes[2]), [c])
    g.add_memory_dependencies()
    assert g.optimize() == 0


def chain_case(kind, lead, n, xdt):
    """(nodes, buffers): nodes as (einsummable, out buffer, [input buffers]); buffers as
    name -> (dtype, element count, is a statistic that is deleted)."""
    R = len(lead) + 1
    full, rows = list(range(R)), list(range(R - 1))
    nrows = int(np.prod(lead))
    x = "hole|%s@0" % xdt
    up = x if xdt == "f32" else "to_f32[%s]" % x
    down = (lambda t: t) if xdt == "f32" else (lambda t: "to_f16[%s]" % t)
    bufs = {"X": (xdt, nrows * n, False), "Y": (xdt, nrows * n, False)}
    nodes = []
    if kind == "layernorm":
        # mean, sum of squared deviations, (var + eps)^-1/2, (x - mean) * rstd * w + b
        bufs.update(mean=("f32", nrows, True), dev=("f32", nrows, True), rstd=("f32", nrows, True),
                    W=(xdt, n, False), B=(xdt, n, False))
        centred = "+[%s,*[constant{f32|-1},hole|f32@1]]" % up
        nodes.append((E(lead + [n], [full], R - 1, "*[constant{f32|%r},%s]" % (1.0 / n, up), "+"),
                      "mean", ["X"]))
        nodes.append((E(lead + [n], [full, rows], R - 1, "power{2}[%s]" % centred, "+"),
                      "dev", ["X", "mean"]))
        nodes.append((E(lead, [rows], R - 1,
                        "power{-0.5}[+[*[constant{f32|%r},hole|f32@0],constant{f32|1e-05}]]" % (1.0 / n)),
                      "rstd", ["dev"]))
        w = "hole|%s@3" % xdt if xdt == "f32" else "to_f32[hole|%s@3]" % xdt
        b = "hole|%s@4" % xdt if xdt == "f32" else "to_f32[hole|%s@4]" % xdt
        nodes.append((E(lead + [n], [full, rows, rows, [R - 1], [R - 1]], R,
                        down("+[*[*[%s,hole|f32@2],%s],%s]" % (centred, w, b))),
                      "Y", ["X", "mean", "rstd", "W", "B"]))
    elif kind == "minmax":
        # (x - min) / (max - min + 1)
        bufs.update(lo=("f32", nrows, True), hi=("f32", nrows, True))
        nodes.append((E(lead + [n], [full], R - 1, up, "v"), "lo", ["X"]))
        nodes.append((E(lead + [n], [full], R - 1, up, "^"), "hi", ["X"]))
        span = "power{-1}[+[+[hole|f32@2,*[constant{f32|-1},hole|f32@1]],constant{f32|1}]]"
        nodes.append((E(lead + [n], [full, rows, rows], R,
                        down("*[+[%s,*[constant{f32|-1},hole|f32@1]],%s]" % (up, span))),
                      "Y", ["X", "lo", "hi"]))
    else:
        # statistics in f16, as C4 has them: max, sum of exp(x - max), quotient
        assert xdt == "f16"
        bufs.update(m=("f16", nrows, True), l=("f16", nrows, True))
        sub = "exp[+[hole|f16@0,*[constant{f16|-1},hole|f16@1]]]"
        nodes.append((E(lead + [n], [full], R - 1, "hole|f16@0", "^"), "m", ["X"]))
        nodes.append((E(lead + [n], [full, rows], R - 1, sub, "+"), "l", ["X", "m"]))
        nodes.append((E(lead + [n], [full, rows, rows], R, "*[%s,power{-1}[hole|f16@2]]" % sub),
                      "Y", ["X", "m", "l"]))
    return nodes, bufs


@pytest.mark.parametrize("kind,lead,n,xdt", [
    ("layernorm", [7, 9], 768, "f16"),
    ("layernorm", [33], 4096, "f32"),
    ("layernorm", [2, 3, 4], 1000, "f16"),
    ("minmax", [5, 5], 2048, "f16"),
    ("minmax", [64], 333, "f32"),
    ("f16stats", [8, 16], 2048, "f16"),
    ("f16stats", [3], 16384, "f16"),         # eight vectors per lane
])
def test_other_chains_keep_every_bit(km, kind, lead, n, xdt):
    nodes, bufs = chain_case(kind, lead, n, xdt)
    names = list(bufs)
    esz = {"f16": 2, "f32": 4}
    sizes = [bufs[k][1] * esz[bufs[k][0]] for k in names]
    offs, total = layout(sizes)
    mem = {k: (o, s) for k, o, s in zip(names, offs, sizes)}

    def build(g):
        last_reader = {}
        for e, out, ins in nodes:
            i = g.add_einsummable(e, [mem[out]] + [mem[k] for k in ins])
            for k in ins:
                last_reader.setdefault(k, []).append(i)
        for k in names:
            if bufs[k][2]:
                g.add_dummy(mem[k], last_reader[k])

    r = rng(len(kind) * 100003 + n)
    init = np.zeros(total, np.uint8)
    for k in names:
        if not bufs[k][2] and k != "Y":
            lo, nb = mem[k]
            init[lo:lo + nb] = normal(r, bufs[k][1], NP[DT[bufs[k][0]]], 1.5).view(np.uint8)
    plain, fused, graphs, absorbed = run_both(km, build, total, init)
    assert absorbed == len(nodes) - 1 and graphs[1].launches() == 1, (absorbed, graphs[1].launches())
    lo, nb = mem["Y"]
    assert np.array_equal(plain[lo:lo + nb], fused[lo:lo + nb])
    assert np.isfinite(fused[lo:lo + nb].view(NP[DT[xdt]]).astype(np.float64)).all()


@pytest.mark.parametrize("seq,heads,half", [(2048, 32, 64), (77, 5, 24), (3, 1, 1)])
def test_conversions_around_a_complex_view_are_absorbed(km, seq, heads, half):
    """Rotary embeddings as the reference's graph spells them: to_f32, the product with the
    frequencies on the buffer seen as complex numbers, to_f16.  Optimised, the complex node
    reads and writes pairs of f16 itself: one launch, the same bits."""
    n = seq * heads * half * 2                       # f16 elements
    up = E([n], [[0]], 1, "to_f32[hole|f16@0]")
    rot = E([1, seq, heads, half], [[0, 1, 2, 3], [1, 3]], 4, "*[hole|c64@0,hole|c64@1]")
    down = E([n], [[0]], 1, "to_f16[hole|f32@0]")
    sizes = [n * 2, seq * half * 8, n * 4, n * 4, n * 2]
    (X, F, A, B, Y), total = layout(sizes)

    def build(g):
        a = g.add_einsummable(up, [(A, sizes[2]), (X, sizes[0])])
        b = g.add_einsummable(rot, [(B, sizes[3]), (A, sizes[2]), (F, sizes[1])])
        c = g.add_einsummable(down, [(Y, sizes[4]), (B, sizes[3])])
        g.add_dummy((A, sizes[2]), [b])
        g.add_dummy((B, sizes[3]), [c])

    r = rng(seq)
    init = np.zeros(total, np.uint8)
    init[X:X + sizes[0]] = normal(r, n, np.float16, 1.0).view(np.uint8)
    ang = r.uniform(0, 6.28, seq * half)
    init[F:F + sizes[1]] = (np.cos(ang) + 1j * np.sin(ang)).astype(np.complex64).view(np.uint8)
    plain, fused, graphs, absorbed = run_both(km, build, total, init)
    assert absorbed == 2 and graphs[1].launches() == 1
    assert "f16 pairs: out in0" in graphs[1].describe(2)
    assert np.array_equal(plain[Y:Y + sizes[4]], fused[Y:Y + sizes[4]])
    got = fused[Y:Y + sizes[4]].view(np.float16).astype(np.float32).reshape(seq, heads, half, 2)
    x = init[X:X + sizes[0]].view(np.float16).astype(np.float32).reshape(seq, heads, half, 2)
    want = (x[..., 0] + 1j * x[..., 1]) * (np.cos(ang) + 1j * np.sin(ang)).reshape(seq, 1, half)
    assert np.allclose(got[..., 0], want.real, atol=4e-3) and np.allclose(got[..., 1], want.imag, atol=4e-3)
