"""Parity of the generated elementwise / reduction kernels with the CPU oracle, through the
C ABI.  The forms are the ones the LLaMA layer and the benchmark configurations use (the
reference exercises the same forms in exps/gpuexec_kernelmanager.cc and
exps/cpuexec_kernels.cc:88-318) plus ragged shapes that force the scalar paths."""
import numpy as np
import pytest

import einsummable_amd as ea
import oracle
from helpers import (NP, assert_bits_equal, assert_close, assert_values_equal, empty_device, normal,
                     oracle_einsummable, rng, run_einsummable, stream_handle, to_device, to_host, uniform)

pytestmark = pytest.mark.gpu

E = ea.Einsummable

RELU_MUL = "*[ite_>=[constant{f16|0},hole|f16@0,constant{f16|0},hole|f16@0],hole|f16@1]"
EXP_SUB = "exp[+[hole|f16@0,*[constant{f16|-1},hole|f16@1]]]"
SILU = "*[hole|f16@0,power{-1}[+[constant{f16|1},exp[*[constant{f16|-1},hole|f16@0]]]]]"


def inputs_for(e, r, sd=1.0, positive=False):
    _, dts = oracle.scalarop_info(e.join)
    xs = []
    for k, dt in enumerate(dts):
        n = int(np.prod(e.inn_shape(k)))
        x = normal(r, n, NP[dt], sd)
        if positive:
            x = np.abs(x) + np.asarray(0.5, dtype=x.dtype)
        xs.append(x)
    return xs


def check(km, e, seed=0, positive=False, sd=1.0, exact=False, scale=None):
    xs = inputs_for(e, rng(seed), sd, positive)
    got = run_einsummable(km, e, xs)
    od, _ = oracle.scalarop_info(e.join)
    if exact == "bits":
        want = oracle_einsummable(e, xs, oracle.EXACT)
        assert_bits_equal(got, want, "%s %s" % (e.join_shape, e.join))
    elif exact:
        want = oracle_einsummable(e, xs, oracle.EXACT)
        assert_values_equal(got, want, "%s %s" % (e.join_shape, e.join))
    else:
        want = oracle_einsummable(e, xs, oracle.WIDE)
        assert_close(got, want, od, scale=scale, what="%s %s" % (e.join_shape, e.join))
    return got


UNARY = [
    ("to_f32[hole|f16@0]", "bits"),
    ("to_f16[hole|f32@0]", "bits"),
    ("to_f64[hole|f32@0]", "bits"),
    ("to_f32[hole|f64@0]", "bits"),
    ("power{2}[hole|f32@0]", False),
    ("power{-0.5}[hole|f32@0]", False),
    ("power{-1}[hole|f32@0]", False),
    ("power{0.5}[hole|f64@0]", False),
    ("power{1.7}[hole|f32@0]", False),
    ("exp[hole|f32@0]", False),
    ("exp[hole|f64@0]", False),
    ("log[hole|f32@0]", False),
    ("+[*[constant{f32|0.000244141},hole|f32@0],constant{f32|1e-06}]", False),
    ("*[constant{f16|0.0883789},hole|f16@0]", True),
    (SILU, False),
    ("ite_<[hole|f32@0,constant{f32|0},constant{f32|0},hole|f32@0]", True),
    ("conj[hole|c64@0]", True),
    ("real[hole|c64@0]", True),
    ("imag[hole|c64@0]", True),
]


@pytest.mark.parametrize("join,exact", UNARY)
@pytest.mark.parametrize("n", [1, 5, 1000, 4099, 65536])
def test_unary(km, join, exact, n):
    positive = "log" in join or "power{-0.5}" in join or "power{0.5}" in join or "power{1.7}" in join
    check(km, E([n], [[0]], 1, join), seed=n, positive=positive, exact=exact)


BINARY = [
    ("+[hole|f16@0,hole|f16@1]", True),
    ("*[hole|f16@0,hole|f16@1]", True),
    ("+[hole|f32@0,hole|f32@1]", True),
    ("*[hole|f64@0,hole|f64@1]", True),
    ("*[hole|f32@0,power{-1}[hole|f32@1]]", False),
    ("+[hole|f32@0,*[constant{f32|-1},hole|f32@1]]", True),
    (RELU_MUL, True),
    (EXP_SUB, False),
    ("*[hole|c64@0,hole|c64@1]", False),
    ("+[hole|c64@0,hole|c64@1]", True),
    ("complex[hole|f32@0,hole|f32@1]", True),
    ("ite_==[hole|f32@0,hole|f32@1,constant{f32|1},constant{f32|0}]", True),
]


@pytest.mark.parametrize("join,exact", BINARY)
def test_binary_straight_and_broadcast(km, join, exact):
    positive = "power{-1}" in join
    for shape in ([37], [4096], [3, 5], [64, 96], [7, 1024]):
        R = len(shape)
        full = list(range(R))
        check(km, E(shape, [full, full], R, join), seed=R, positive=positive, exact=exact)
    # ab,a->ab and ab,b->ab and a,ab->ab
    for a, b in ((5, 7), (64, 256), (33, 1000)):
        check(km, E([a, b], [[0, 1], [0]], 2, join), seed=a, positive=positive, exact=exact)
        check(km, E([a, b], [[0, 1], [1]], 2, join), seed=b, positive=positive, exact=exact)
        check(km, E([a, b], [[0], [0, 1]], 2, join), seed=a + b, positive=positive, exact=exact)


def test_softmax_elementwise_three_inputs(km):
    # ab,a,a->ab : exp(x - m[a]) / s[a]
    join = "*[exp[+[hole|f32@0,*[constant{f32|-1},hole|f32@1]]],power{-1}[hole|f32@2]]"
    check(km, E([48, 512], [[0, 1], [0], [0]], 2, join), seed=3, positive=True)


def test_rotary_complex_broadcast(km):
    # abcd,bd->abcd complex multiply (src/engine/cpu/kernel_executor.cc:272-314)
    check(km, E([2, 16, 4, 32], [[0, 1, 2, 3], [1, 3]], 4, "*[hole|c64@0,hole|c64@1]"), seed=11)


def test_outer_product_and_pure_broadcast(km):
    check(km, E([40, 72], [[0], [1]], 2, "*[hole|f32@0,hole|f32@1]"), seed=1, exact=True)
    check(km, E([6, 40], [[1]], 2, "hole|f32@0"), seed=2, exact="bits")   # b->ab
    check(km, E([40, 6], [[0]], 2, "hole|f16@0"), seed=3, exact="bits")   # a->ab


@pytest.mark.parametrize("dt", ["f16", "f32", "f64"])
def test_permute_inner_preserved(km, dt):
    # abcd->acbd: the innermost mode stays innermost (a strided row copy)
    check(km, E([4, 6, 5, 64], [[0, 2, 1, 3]], 4, "hole|%s@0" % dt), seed=4, exact="bits")
    check(km, E([3, 5, 4, 7], [[0, 2, 1, 3]], 4, "hole|%s@0" % dt), seed=5, exact="bits")


def test_transposed_input_elementwise(km):
    # ba,ab->ab: the first input is read transposed
    check(km, E([24, 40], [[1, 0], [0, 1]], 2, "+[hole|f32@0,hole|f32@1]"), seed=6, exact=True)


def test_output_may_alias_input(km):
    """Straight elementwise ops may be run in place (donation, memgraph.h:278-287)."""
    import torch
    from helpers import stream_handle, to_device, to_host

    e = E([10000], [[0], [0]], 1, "+[hole|f16@0,hole|f16@1]")
    km.build(e)
    r = rng(8)
    x, y = normal(r, 10000, np.float16), normal(r, 10000, np.float16)
    dx, dy = to_device(x), to_device(y)
    km(e, stream_handle(), dx.data_ptr(), [dx.data_ptr(), dy.data_ptr()])
    torch.cuda.synchronize()
    assert_bits_equal(to_host(dx, np.float16), (x + y).astype(np.float16), "in-place add")


REDUCTIONS = ["+", "x", "v", "^"]


@pytest.mark.parametrize("castable", REDUCTIONS)
@pytest.mark.parametrize("dt", ["f16", "f32", "f64"])
def test_row_reduction_ab_a(km, castable, dt):
    for a, b in ((1, 1), (3, 5), (17, 64), (9, 1000), (130, 4096), (4, 20000)):
        sd = 1.0
        if castable == "x":
            if b > 1000:
                continue
            sd = 0.05  # products stay in range
        e = E([a, b], [[0, 1]], 1, "hole|%s@0" % dt, castable)
        xs = inputs_for(e, rng(a * 7 + b), sd)
        if castable == "x":
            xs = [np.asarray(1.0, xs[0].dtype) + xs[0]]
        got = run_einsummable(km, e, xs)
        od, _ = oracle.scalarop_info(e.join)
        if castable in ("v", "^"):
            assert_bits_equal(got, oracle_einsummable(e, xs, oracle.EXACT), "min/max reduce")
        else:
            assert_close(got, oracle_einsummable(e, xs, oracle.WIDE), od, what="reduce %s" % castable)


def test_fused_exp_sub_row_sum(km):
    # ab,a->a : sum_b exp(x[a,b] - m[a])
    for dt, shape in (("f16", (64, 2048)), ("f32", (33, 1000)), ("f32", (8, 8))):
        join = "exp[+[hole|%s@0,*[constant{%s|-1},hole|%s@1]]]" % (dt, dt, dt)
        check(km, E(list(shape), [[0, 1], [0]], 1, join, "+"), seed=9)


def test_column_and_middle_reductions(km):
    check(km, E([64, 40], [[1, 0]], 1, "hole|f32@0", "+"), seed=10)             # ba->a
    check(km, E([6, 32, 20], [[0, 2, 1]], 2, "hole|f32@0", "+"), seed=11)       # acb->ab
    check(km, E([6, 32, 20], [[0, 2, 1]], 2, "hole|f16@0", "^"), seed=12, exact=True)
    check(km, E([5, 7, 3, 4], [[0, 2, 1, 3]], 2, "hole|f64@0", "+"), seed=13)   # two agg modes
    check(km, E([5, 3, 4], [[0, 1, 2], [0, 1, 2]], 1, "*[hole|f32@0,hole|f32@1]", "+"), seed=14)


def test_generic_contractions_through_codegen(km):
    """Contractions in dtypes without a matrix-core kernel fall back to generated code."""
    check(km, E([6, 5, 7], [[0, 2], [2, 1]], 2, "*[hole|c64@0,hole|c64@1]", "+"), seed=15)


def test_merged_and_unmerged_descriptors_agree(km):
    r = rng(16)
    x = normal(r, 3 * 4 * 5 * 6, np.float32)
    y = normal(r, 3 * 4, np.float32)
    full = E([3, 4, 5, 6], [[0, 1, 2, 3], [0, 1]], 4, "*[hole|f32@0,hole|f32@1]")
    merged = E([12, 30], [[0, 1], [0]], 2, "*[hole|f32@0,hole|f32@1]")
    assert oracle.merge_adjacent_dims(full.join_shape, full.inns, 4) == ([12, 30], [[0, 1], [0]], 2)
    a = run_einsummable(km, full, [x, y])
    b = run_einsummable(km, merged, [x, y])
    assert_bits_equal(a, b, "merge_adjacent_dims invariance")


def test_error_contract(km):
    import torch

    e = E([123], [[0]], 1, "exp[hole|f32@0]")
    d = torch.zeros(123, device="cuda")
    with pytest.raises(ea.KmError) as ei:   # not built
        km(e, 0, d.data_ptr(), [d.data_ptr()])
    assert ei.value.code == -2
    with pytest.raises(ea.KmError) as ei:
        km.workspace_size(e)
    assert ei.value.code == -2
    assert km.build(e) == 0
    assert km.workspace_size(e) == 0
    with pytest.raises(ea.KmError) as ei:   # wrong number of inputs
        km(e, 0, d.data_ptr(), [d.data_ptr(), d.data_ptr()])
    assert ei.value.code == -4
    with pytest.raises(ea.KmError) as ei:   # malformed join
        km.build(E([4], [[0]], 1, "exp[hole|f32@0"))
    assert ei.value.code == -1
    with pytest.raises(ea.KmError):         # aggregation without castable
        km.build(E([4, 4], [[0, 1]], 1, "hole|f32@0"))
    # scalar variables must be substituted by the caller: unsupported, not an error
    assert km.build(E([4], [[0]], 1, "*[variable{lr|f32},hole|f32@0]")) is None


SPLIT_REDUCTIONS = [
    # few outputs, long aggregation over an outer mode: slices of the aggregated range run
    # side by side and a second kernel folds their partial results (needs a workspace)
    (E([64, 4096], [[1, 0]], 1, "hole|f32@0", "+"), False),                 # ba->a
    (E([256, 1000], [[1, 0]], 1, "hole|f16@0", "+"), False),
    (E([256, 1000], [[1, 0]], 1, "hole|f16@0", "^"), True),
    (E([3, 40, 777], [[0, 2, 1]], 2, "hole|f32@0", "v"), True),             # acb->ab
    (E([24, 300, 5], [[1, 2, 0]], 1, "hole|f32@0", "+"), False),            # two aggregated modes
    (E([128, 513], [[1, 0], [0]], 1, "*[hole|f32@0,hole|f32@1]", "+"), False),  # ba,a->a
    (E([16, 3000], [[1, 0]], 1, "hole|f64@0", "+"), False),
    (E([8, 2048], [[1, 0]], 1, "hole|c64@0", "+"), False),
]


@pytest.mark.parametrize("case", range(len(SPLIT_REDUCTIONS)))
def test_split_column_reductions(km, case):
    e, exact = SPLIT_REDUCTIONS[case]
    ws = km.build(e)
    assert ws is not None and ws > 0, "expected a two-pass plan"
    assert "splits=" in km.describe(e) and km.workspace_size(e) == ws
    check(km, e, seed=60 + case, exact=exact)


def test_sliced_column_reduction_on_a_used_workspace(km):
    """The slices of a column reduction leave their partial results in the workspace, which
    holds whatever the last user left: the same workspace, first filled with a byte pattern,
    serves launches with different inputs one after the other, and each result is right."""
    import torch

    for e, exact in ((E([4096, 2048], [[1, 0]], 1, "hole|f16@0", "^"), True),
                     (E([64, 4096], [[1, 0]], 1, "hole|f32@0", "+"), False),
                     (E([3, 1000, 72], [[0, 2, 1]], 2, "hole|f32@0", "+"), False)):
        ws = km.build(e)
        assert ws > 0 and "splits=" in km.describe(e)
        od, _ = oracle.scalarop_info(e.join)
        d_ws = torch.full((ws,), 0xAB, dtype=torch.uint8, device="cuda")
        for rep in range(3):
            xs = inputs_for(e, rng(900 + rep), 1.0, False)
            d_in = [to_device(x) for x in xs]
            d_out = empty_device(e.out_nelem(), NP[od])
            km(e, stream_handle(), d_out.data_ptr(), [t.data_ptr() for t in d_in], (d_ws.data_ptr(), ws))
            torch.cuda.synchronize()
            got = to_host(d_out, NP[od])
            if exact:
                assert_values_equal(got, oracle_einsummable(e, xs, oracle.EXACT), "launch %d" % rep)
            else:
                assert_close(got, oracle_einsummable(e, xs, oracle.WIDE), od, what="launch %d" % rep)


def test_workspace_contract_of_a_two_pass_reduction(km):
    import torch

    e = E([64, 4096], [[1, 0]], 1, "hole|f32@0", "+")
    ws = km.build(e)
    assert ws > 0
    x = torch.zeros(64 * 4096, device="cuda")
    y = torch.zeros(64, device="cuda")
    w = torch.zeros(ws, dtype=torch.uint8, device="cuda")
    with pytest.raises(ea.KmError) as ei:          # no workspace
        km(e, 0, y.data_ptr(), [x.data_ptr()])
    assert ei.value.code == -3
    with pytest.raises(ea.KmError) as ei:          # too small
        km(e, 0, y.data_ptr(), [x.data_ptr()], (w.data_ptr(), ws - 1))
    assert ei.value.code == -3
    km(e, 0, y.data_ptr(), [x.data_ptr()], (w.data_ptr(), ws))
    torch.cuda.synchronize()


def test_two_pass_reduction_inside_an_exec_graph(km):
    import torch

    e = E([64, 4096], [[1, 0]], 1, "hole|f32@0", "+")
    r = rng(70)
    x = normal(r, 64 * 4096, np.float32)
    arena = torch.zeros(64 * 4096 + 64, device="cuda")
    arena[:64 * 4096] = torch.from_numpy(x).cuda()
    g = ea.ApplyGraph(km)
    g.add_einsummable(e, [(64 * 4096 * 4, 256), (0, 64 * 4096 * 4)])
    g.finalize(2)
    g.run(0, arena.data_ptr())
    torch.cuda.synchronize()
    want = x.reshape(4096, 64).astype(np.float64).sum(axis=0)
    assert_close(arena[64 * 4096:].cpu().numpy(), want, ea.F32, what="exec graph two-pass")


SPLIT_ROW_REDUCTIONS = [
    # a handful of very long rows: each row is cut into slices that run side by side
    (E([3, 131072], [[0, 1]], 1, "hole|f16@0", "+"), False),
    (E([1, 262144], [[0, 1]], 1, "hole|f32@0", "^"), True),
    (E([5, 140000], [[0, 1]], 1, "hole|f32@0", "+"), False),                     # ragged last slice
    (E([2, 64, 2048], [[0, 1, 2]], 1, "hole|f16@0", "v"), True),                 # two aggregated modes
    (E([2, 131072], [[0, 1], [0]], 1, "exp[+[hole|f16@0,*[constant{f16|-1},hole|f16@1]]]", "+"),
     False),                                                                      # ab,a->a
    (E([3, 40000], [[0, 1]], 1, "hole|f64@0", "+"), False),
]


@pytest.mark.parametrize("case", range(len(SPLIT_ROW_REDUCTIONS)))
def test_split_row_reductions(km, case):
    e, exact = SPLIT_ROW_REDUCTIONS[case]
    ws = km.build(e)
    assert ws is not None and ws > 0 and "splits=" in km.describe(e), km.describe(e)
    check(km, e, seed=80 + case, exact=exact, sd=0.5)


STAGED = [
    ("ab,ba->ab", dict(a=136, b=72), "+[hole|f16@0,hole|f16@1]"),
    ("ab,ba->ab", dict(a=33, b=50), "*[hole|f32@0,hole|f32@1]"),                  # ragged: scalar paths
    ("abc,acb->abc", dict(a=3, b=40, c=24), "*[hole|f16@0,hole|f16@1]"),
    ("abcd,dcba,ab->abcd", dict(a=4, b=6, c=8, d=16), "+[hole|f32@0,*[hole|f32@1,hole|f32@2]]"),
    ("ba->ab", dict(a=64, b=48), "*[constant{f16|2},hole|f16@0]"),
    ("abc,cb->abc", dict(a=5, b=16, c=32), "+[hole|f64@0,hole|f64@1]"),           # transposed and broadcast
    ("ab,ba,ba->ab", dict(a=40, b=56), "+[hole|c64@0,*[hole|c64@1,hole|c64@2]]"),
]


@pytest.mark.parametrize("case", range(len(STAGED)))
def test_inputs_with_another_inner_mode_are_transposed_into_the_workspace(monkeypatch, case):
    spec, sizes, join = STAGED[case]
    monkeypatch.setenv("ES_KM_EW_STAGE_MIN", "1")       # by itself only from 2 M elements on
    staged = ea.KernelManager(0)
    e = E.from_str(spec, sizes, join)
    ws = staged.build(e)
    assert ws > 0 and staged.describe(e).startswith("staged ["), staged.describe(e)
    got = check(staged, e, seed=120 + case)
    monkeypatch.setenv("ES_KM_EW_STAGE_MIN", "0")
    direct = ea.KernelManager(0)
    assert direct.build(e) == 0 and direct.describe(e).startswith("elementwise")
    # the same arithmetic on the same values, whichever way they were fetched
    xs = inputs_for(e, rng(120 + case))
    assert_bits_equal(got, run_einsummable(direct, e, xs), spec)


def test_large_transposed_input_is_staged_by_default(km):
    e = E.from_str("ab,ba->ab", dict(a=2048, b=1536), "+[hole|f16@0,hole|f16@1]")
    ws = km.build(e)
    assert ws == 2048 * 1536 * 2 and km.describe(e).startswith("staged ["), km.describe(e)
    r = rng(130)
    xs = [normal(r, 2048 * 1536, np.float16) for _ in range(2)]
    got = run_einsummable(km, e, xs)
    want = (xs[0].reshape(2048, 1536).astype(np.float32) +
            xs[1].reshape(1536, 2048).T.astype(np.float32)).astype(np.float16)
    assert_bits_equal(got, want.reshape(-1), "ab,ba->ab")
    import torch
    from helpers import stream_handle
    d = torch.zeros(16, device="cuda", dtype=torch.float16)
    with pytest.raises(ea.KmError) as ei:
        km(e, stream_handle(), d.data_ptr(), [d.data_ptr(), d.data_ptr()])
    assert ei.value.code == -3


# ------------------------------------------------------------------ buffers off the vector grid

def run_at_offsets(km, e, xs, shift):
    """Every buffer starts `shift` bytes behind a 256-byte boundary of one byte arena (the
    engine hands out arena offsets aligned to 16 bytes only, memgraph.cc:58-62)."""
    import torch

    from helpers import stream_handle

    od, dts = oracle.scalarop_info(e.join)
    ws = km.build(e)
    assert ws is not None
    sizes = [x.nbytes for x in xs] + [e.out_nelem() * np.dtype(NP[od]).itemsize, max(ws, 1)]
    offs, off = [], 0
    for nb in sizes:
        offs.append(off + shift)
        off += (nb + shift + 255) // 256 * 256 + 256
    arena = torch.zeros(off, dtype=torch.uint8, device="cuda")
    for x, o in zip(xs, offs):
        arena[o:o + x.nbytes] = torch.from_numpy(np.ascontiguousarray(x).view(np.uint8).reshape(-1)).cuda()
    base = arena.data_ptr()
    assert base % 256 == 0
    km(e, stream_handle(), base + offs[len(xs)], [base + o for o in offs[:len(xs)]],
       (base + offs[-1], ws) if ws else None)
    torch.cuda.synchronize()
    o = offs[len(xs)]
    return arena[o:o + sizes[len(xs)]].cpu().numpy().view(NP[od])


OFF_GRID = [
    E([96, 512], [[0, 1]], 2, "to_f32[hole|f16@0]"),                                   # 8 f16 in, 32 bytes out
    E([96, 512], [[0, 1], [0]], 2, "to_f16[*[hole|f32@0,hole|f32@1]]"),               # f32 row statistic
    E([40, 2048], [[0, 1]], 1, "hole|f32@0", "+"),                                     # 32 bytes per lane and step
    E([40, 2048], [[0, 1], [1]], 1, "to_f32[+[hole|f16@0,hole|f16@1]]", "+"),
    E([3, 131072], [[0, 1]], 1, "hole|f32@0", "+"),                                    # slices and fold
    E([512, 96], [[1, 0]], 1, "to_f32[hole|f16@0]", "+"),                              # column sum, f32 out
    E([4, 64, 128], [[0, 1, 2], [1, 2], [0, 1]], 3, "exp[+[to_f32[+[hole|f16@0,hole|f16@1]],*[constant{f32|-1},hole|f32@2]]]"),
]


@pytest.mark.parametrize("case", range(len(OFF_GRID)))
def test_generated_kernels_at_buffers_off_the_vector_grid(km, case):
    """At 16 bytes behind a 256-byte boundary the vector kernels still apply (a 32-byte vector
    moves as two 16-byte pieces) and a reduction adds in the same order as at the boundary;
    at one element's size behind it the scalar variant runs: every result against the oracle."""
    e = OFF_GRID[case]
    od, dts = oracle.scalarop_info(e.join)
    xs = inputs_for(e, rng(140 + case), 0.5)
    want = oracle_einsummable(e, xs, oracle.WIDE)
    at0 = run_at_offsets(km, e, xs, 0)
    at16 = run_at_offsets(km, e, xs, 16)
    assert_close(at0, want, od, what="on the grid")
    assert_bits_equal(at16, at0, "16 bytes off: same kernel, same bits")
    smallest = min([np.dtype(NP[d]).itemsize for d in dts] + [np.dtype(NP[od]).itemsize])
    assert_close(run_at_offsets(km, e, xs, smallest), want, od, what="one element off")
