"""Pins the CPU oracle: against the reference's own known-answer vector, against golden
vectors written from the reference's scalarop_t / permute_t (tests/golden/), live against
oracle/_ref where that was built, and against what the mathematics fixes (numpy closed
forms, brute force, invariants).  No GPU."""
import hashlib
import itertools
import json
import os

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = json.load(open(os.path.join(HERE, "golden", "scalarop_golden.json")))
needs_ref = pytest.mark.skipif(not oracle.ref_available(), reason="oracle/_ref was not built")


# ------------------------------------------------------------------ fp16 arithmetic

def test_f16_conversion_exhaustive_against_numpy():
    allh = np.arange(65536, dtype=np.uint16)
    f = allh.view(np.float16)
    # widening is exact
    wide = np.array([oracle._lib.es_oracle_f16_to_f32(int(h)) for h in allh[::7]], np.float32)
    assert np.array_equal(wide[~np.isnan(wide)], f[::7].astype(np.float32)[~np.isnan(wide)])
    # narrowing: every half, its neighbours' midpoints and random doubles, ties to even
    rs = np.random.RandomState(0)
    finite = f[np.isfinite(f)].astype(np.float64)
    mids = (finite[:-1] + finite[1:]) / 2
    cands = np.concatenate([finite, mids, np.nextafter(mids, np.inf), np.nextafter(mids, -np.inf),
                            rs.normal(0, 100, 20000), rs.normal(0, 1e-5, 20000),
                            [65504.0, 65519.999, 65520.0, 1e6, -1e6, 2.0 ** -25, 2.0 ** -24,
                             np.nextafter(2.0 ** -25, 1.0), 0.0, -0.0, np.inf, -np.inf]])
    with np.errstate(over="ignore"):
        want = cands.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f64_to_f16_bits(v) for v in cands], np.uint16)
    assert np.array_equal(got, want)


def _digest(u16):
    u16 = np.ascontiguousarray(u16).view(np.uint16)
    f = u16.view(np.float16)
    u16 = np.where(np.isnan(f), np.uint16(0x7E00), u16)
    return hashlib.sha256(np.ascontiguousarray(u16).tobytes()).hexdigest()


@pytest.mark.parametrize("text", sorted(GOLDEN["f16_unary_sha256"]))
def test_f16_unary_ops_exhaustive_against_golden(text):
    """All 65536 half inputs through exp / log / power / silu must reproduce the reference's
    half_float results bit for bit (digest written from the reference)."""
    allh = np.arange(65536, dtype=np.uint16).view(np.float16)
    got = oracle.scalarop_map(text, [allh])
    assert _digest(got) == GOLDEN["f16_unary_sha256"][text]


@pytest.mark.parametrize("text", sorted(GOLDEN["f16_binary_seed0_sha256"]))
def test_f16_binary_ops_against_golden(text):
    # same draws as tests/golden/make_golden.py, which come after its eval points
    rs2 = _replay_golden_rng()
    xs = rs2.randint(0, 65536, 1 << 20).astype(np.uint16)
    ys = rs2.randint(0, 65536, 1 << 20).astype(np.uint16)
    got = oracle.scalarop_map(text, [xs.view(np.float16), ys.view(np.float16)])
    assert _digest(got) == GOLDEN["f16_binary_seed0_sha256"][text]
    # and IEEE: numpy's float16 add / mul are correctly rounded
    with np.errstate(all="ignore"):
        ref = (xs.view(np.float16) + ys.view(np.float16)) if text[0] == "+" else (
            xs.view(np.float16) * ys.view(np.float16))
    assert _digest(got) == _digest(ref)


def _replay_golden_rng():
    """make_golden.py draws its eval points from RandomState(0) before the binary tables;
    replay those draws so the tables use the same inputs."""
    rs = np.random.RandomState(0)
    for entry in GOLDEN["eval"]:
        _, holes = oracle.scalarop_info(entry["op"])
        for _ in entry["points"]:
            for dt in holes:
                rs.normal(0, 2.0)
                if dt == oracle.C64:
                    rs.normal()
    return rs


# ------------------------------------------------------------------ scalarop text + eval

LITERALS = [  # spelled out in src/engine/gpu/gpu_kernel_manager.cc / exps/gpuexec_kernelmanager.cc
    "*[*[hole|f32@0,power{-1}[hole|f32@1]],hole|f32@2]",
    "*[constant{f16|0.0883789},hole|f16@0]",
    "*[hole|c64@0,hole|c64@1]",
    "*[hole|f16@0,power{-1}[+[constant{f16|1},exp[*[constant{f16|-1},hole|f16@0]]]]]",
    "*[hole|f32@0,*[hole|f32@1,*[constant{f32|-1},power{-1}[*[hole|f32@2,hole|f32@2]]]]]",
    "*[hole|f32@0,*[hole|f32@1,*[constant{f32|-1},power{-2}[hole|f32@2]]]]",
    "+[*[constant{f32|0.000244141},hole|f32@0],constant{f32|1e-06}]",
    "+[*[constant{f32|0.5},hole|f32@0],*[constant{f32|-500},hole|f32@1]]",
    "+[hole|f32@0,*[constant{f32|-1},hole|f32@1]]",
    "exp[hole|f32@0]",
    "power{2}[hole|f32@0]",
    "ite_>=[constant{f16|0},hole|f16@0,constant{f16|0},hole|f16@0]",
    "ite_==[hole|f32@0,hole|f32@1,constant{f32|1},constant{f32|0}]",
    "constant{f32|INF}", "constant{f16|NINF}", "constant{f64|NAN}", "constant{c64|(1.5,-2)}",
    "variable{lr|f32}",
    "to_f16[to_f32[hole|f64@0]]",
    "complex[real[hole|c64@0],imag[conj[hole|c64@1]]]",
]


@pytest.mark.parametrize("text", LITERALS)
def test_text_round_trip(text):
    assert oracle.scalarop_roundtrip(text) == text


def test_canonical_constructor_texts_round_trip():
    for text in GOLDEN["make"].values():
        assert oracle.scalarop_roundtrip(text) == text
    for entry in GOLDEN["make_scale"]:
        assert oracle.scalarop_roundtrip(entry["text"]) == entry["text"]
    for text in GOLDEN["simplify"].values():
        assert oracle.scalarop_roundtrip(text) == text


@pytest.mark.parametrize("bad", ["", "hole|f32", "+[hole|f32@0]", "+[hole|f32@0,hole|f16@1]",
                                 "exp[hole|c64@0]", "to_f32[hole|f32@0]", "frob[hole|f32@0]",
                                 "ite_<[hole|f32@0,hole|f32@1,hole|f32@0,hole|f16@1]",
                                 "exp[hole|f32@0]]", "complex[hole|f64@0,hole|f64@1]"])
def test_malformed_or_ill_typed_text_is_rejected(bad):
    with pytest.raises(oracle.OracleError):
        oracle.scalarop_roundtrip(bad)


@pytest.mark.parametrize("entry", GOLDEN["eval"], ids=lambda e: e["op"][:40])
def test_eval_against_golden_points(entry):
    text = entry["op"]
    od, holes = oracle.scalarop_info(text)
    for bits, want in entry["points"]:
        vals = [oracle._from_bits(b, dt) for b, dt in zip(bits, holes)]
        got = oracle._to_bits(oracle.scalarop_eval(text, vals), od)
        if od == oracle.C64 or not np.isnan(oracle._from_bits(want, od)):
            assert got == want, (text, vals, hex(got), hex(want))


def test_six_digit_constants_are_taken_from_text():
    # 1/sqrt(128) printed with 6 significant digits, then stored in the op's dtype
    assert oracle.scalarop_eval("*[constant{f32|0.0883883},hole|f32@0]", [1.0]) == np.float32(0.0883883)
    assert oracle.scalarop_eval("*[constant{f16|0.0883789},hole|f16@0]", [1.0]) == np.float16(0.0883789)
    assert np.float32(0.0883883) != np.float32(1 / np.sqrt(128))


def test_relu_forms_quirk():
    """make_relu evaluates as max(x, 0); the simplified form of max(x, const) is a min
    (normalize_order, scalarop.cc:1442-1493).  Texts as written by the reference."""
    relu = GOLDEN["make"]["relu|f32"]
    assert relu == "ite_>=[constant{f32|0},hole|f32@0,constant{f32|0},hole|f32@0]"
    assert oracle.scalarop_eval(relu, [-2.0]) == 0.0 and oracle.scalarop_eval(relu, [3.0]) == 3.0
    flipped = GOLDEN["simplify"]["ite_>[hole|f32@0,constant{f32|0},hole|f32@0,constant{f32|0}]"]
    assert flipped == "ite_<=[constant{f32|0},hole|f32@0,constant{f32|0},hole|f32@0]"
    assert oracle.scalarop_eval(flipped, [-2.0]) == -2.0 and oracle.scalarop_eval(flipped, [3.0]) == 0.0


def test_eval_closed_forms_against_numpy():
    rs = np.random.RandomState(1)
    x = rs.normal(0, 2, 4000).astype(np.float32)
    y = rs.normal(0, 2, 4000).astype(np.float32)
    xp = np.abs(x) + np.float32(0.25)
    f = oracle.scalarop_map
    assert np.array_equal(f("+[hole|f32@0,hole|f32@1]", [x, y]), x + y)
    assert np.array_equal(f("*[hole|f32@0,hole|f32@1]", [x, y]), x * y)
    np.testing.assert_allclose(f("power{2}[hole|f32@0]", [x]), x.astype(np.float64) ** 2, rtol=2e-7)
    np.testing.assert_allclose(f("exp[hole|f32@0]", [x]), np.exp(x.astype(np.float64)), rtol=2e-7)
    np.testing.assert_allclose(f("log[hole|f32@0]", [xp]), np.log(xp.astype(np.float64)), rtol=2e-7,
                               atol=1e-7)
    np.testing.assert_allclose(f("power{-0.5}[hole|f32@0]", [xp]), xp.astype(np.float64) ** -0.5,
                               rtol=2e-7)
    assert np.array_equal(f("ite_<[hole|f32@0,hole|f32@1,hole|f32@0,hole|f32@1]", [x, y]),
                          np.minimum(x, y))
    assert np.array_equal(f("ite_>[hole|f32@0,hole|f32@1,hole|f32@0,hole|f32@1]", [x, y]),
                          np.maximum(x, y))
    assert np.array_equal(f("to_f16[hole|f32@0]", [x]), x.astype(np.float16))
    xd = rs.normal(0, 300, 4000)
    assert np.array_equal(f("to_f16[hole|f64@0]", [xd]), xd.astype(np.float16))
    assert np.array_equal(f("to_f32[hole|f64@0]", [xd]), xd.astype(np.float32))
    c = (x + 1j * y).astype(np.complex64)
    d = (y - 1j * x).astype(np.complex64)
    got = f("*[hole|c64@0,hole|c64@1]", [c, d])
    np.testing.assert_allclose(got, c.astype(np.complex128) * d.astype(np.complex128), rtol=1e-6)
    assert np.array_equal(f("conj[hole|c64@0]", [c]), np.conj(c))
    assert np.array_equal(f("real[hole|c64@0]", [c]), c.real)
    assert np.array_equal(f("complex[hole|f32@0,hole|f32@1]", [x, y]), c)
    # WIDE mode does not round intermediates
    h = rs.normal(0, 1, 1000).astype(np.float16)
    silu = GOLDEN["make"]["silu|f16"]
    wide = f(silu, [h], oracle.WIDE)
    hd = h.astype(np.float64)
    assert np.array_equal(wide, (hd / (1 + np.exp(-hd))).astype(np.float16))


@needs_ref
def test_live_against_reference_scalarop():
    """Same checks as the golden file, live against the compiled reference."""
    for key, text in GOLDEN["make"].items():
        which, dt = key.split("|")
        assert oracle.ref_scalarop_make(which, {"f16": 0, "f32": 1, "f64": 2}[dt]) == text
    for src, want in GOLDEN["simplify"].items():
        assert oracle.ref_scalarop_simplify(src) == want
    rs = np.random.RandomState(3)
    for text in ["*[exp[+[hole|f32@0,*[constant{f32|-1},hole|f32@1]]],power{-1}[hole|f32@2]]",
                 "+[*[constant{f16|0.5},hole|f16@0],hole|f16@1]",
                 "ite_<=[hole|f64@0,hole|f64@1,power{3}[hole|f64@0],log[hole|f64@1]]"]:
        od, holes = oracle.scalarop_info(text)
        for _ in range(200):
            vals = [oracle._from_bits(oracle._to_bits(abs(rs.normal(0, 2)) + 0.1, dt), dt)
                    for dt in holes]
            a = oracle._to_bits(oracle.scalarop_eval(text, vals), od)
            b = oracle._to_bits(oracle.ref_scalarop_eval(text, vals), od)
            assert a == b, (text, vals)


# ------------------------------------------------------------------ einsummable

def test_reference_matmul_known_answer():
    # tests/reference.h:4-49
    lhs = np.arange(8, 20, dtype=np.float64)
    rhs = np.arange(100, 120, dtype=np.float64)
    out = oracle.einsummable([3, 5, 4], [[0, 2], [2, 1]], 2, "*[hole|f64@0,hole|f64@1]", "+",
                             [lhs, rhs])
    assert out.tolist() == [4110.0, 4148.0, 4186.0, 4224.0, 4262.0, 5830.0, 5884.0, 5938.0,
                            5992.0, 6046.0, 7550.0, 7620.0, 7690.0, 7760.0, 7830.0]


SPECS = ["ij,jk->ik", "ij,kj->ik", "bij,bjk->bik", "acbe,adbe->abcd", "abce,aebd->abcd",
         "adbe,cde->abc", "ab,a->ab", "ab,b->ab", "ab->a", "ba->a", "abc->ac", "a,b->ab",
         "abcd->acbd", "abcd,bd->abcd", "ab,ab,a->a", "ij,kl->ik"]


@pytest.mark.parametrize("spec", SPECS)
def test_interpreter_against_numpy_einsum(spec):
    rs = np.random.RandomState(abs(hash(spec)) % 1000)
    inns, out_rank = oracle.einsummable_parse(spec)
    letters = sorted(set(spec) - set(",->"))
    sizes = {c: int(rs.randint(2, 6)) for c in letters}
    lhs, outw = spec.split("->")
    words = lhs.split(",")
    # join_shape in mode-id order
    ids = {}
    for c in outw:
        ids.setdefault(c, len(ids))
    for w in words:
        for c in w:
            ids.setdefault(c, len(ids))
    join_shape = [0] * len(ids)
    for c, i in ids.items():
        join_shape[i] = sizes[c]
    xs = [rs.normal(0, 1, [sizes[c] for c in w]) for w in words]
    n = len(words)
    join = "hole|f64@0"
    for k in range(1, n):
        join = "*[%s,hole|f64@%d]" % (join, k)
    has_agg = len(ids) > out_rank
    got = oracle.einsummable(join_shape, inns, out_rank, join, "+" if has_agg else None, xs)
    want = np.einsum(spec, *xs)
    np.testing.assert_allclose(got.reshape(want.shape), want, rtol=1e-12, atol=1e-12)
    assert oracle.einsummable_str(inns, out_rank).count(",") == n - 1


def test_exact_mode_accumulates_in_output_dtype_in_order():
    rs = np.random.RandomState(5)
    x = rs.normal(0, 1, (3, 500)).astype(np.float16)
    got = oracle.einsummable([3, 500], [[0, 1]], 1, "hole|f16@0", "+", [x], oracle.EXACT)
    want = []
    for r in range(3):
        acc = x[r, 0]
        for v in x[r, 1:]:
            acc = np.float16(acc + v)
        want.append(acc)
    assert np.array_equal(got, np.array(want, np.float16))
    wide = oracle.einsummable([3, 500], [[0, 1]], 1, "hole|f16@0", "+", [x], oracle.WIDE)
    assert np.array_equal(wide, x.astype(np.float64).sum(axis=1).astype(np.float16))
    for c, fn in (("v", np.min), ("^", np.max)):
        got = oracle.einsummable([3, 500], [[0, 1]], 1, "hole|f16@0", c, [x])
        assert np.array_equal(got, fn(x, axis=1))
    p = (1 + rs.normal(0, 0.01, (4, 50))).astype(np.float32)
    got = oracle.einsummable([4, 50], [[0, 1]], 1, "hole|f32@0", "x", [p], oracle.WIDE)
    np.testing.assert_allclose(got, np.prod(p.astype(np.float64), axis=1), rtol=1e-6)


def test_aggregation_modes_are_renumbered_by_first_appearance():
    # bij,bjk->ik : "203 231->01" is the canonical form (einsummable.cc:45-72)
    assert oracle.einsummable_str([[3, 0, 2], [3, 2, 1]], 2) == "cad,cdb->ab"
    assert oracle.einsummable_str([[2, 0, 3], [2, 3, 1]], 2) == "cad,cdb->ab"
    rs = np.random.RandomState(6)
    a, b = rs.normal(size=(2, 3, 4)), rs.normal(size=(2, 4, 5))
    got = oracle.einsummable([3, 5, 2, 4], [[2, 0, 3], [2, 3, 1]], 2, "*[hole|f64@0,hole|f64@1]",
                             "+", [a, b])
    np.testing.assert_allclose(got.reshape(3, 5), np.einsum("bij,bjk->ik", a, b), rtol=1e-12)


MERGE_CASES = [
    # (join_shape, inns, out_rank) -> merged ; exps/einsummable_test.cc:8-41, einsummable.h:19-37
    (([3, 4, 5, 6], [[0, 1, 2, 3], [0, 1]], 4), ([12, 30], [[0, 1], [0]], 2)),
    (([3, 4, 5, 6], [[0, 1, 2, 3]], 2), ([12, 30], [[0, 1]], 1)),
    # nothing merges; the aggregated modes come back renumbered by first appearance
    (([5, 6, 4, 8, 3], [[0, 2, 1, 4], [0, 1, 3, 4]], 3), ([5, 6, 4, 8, 3], [[0, 2, 1, 3], [0, 1, 4, 3]], 3)),
    (([5, 6, 4, 8, 3], [[0, 1, 3, 4], [0, 2, 1, 4]], 3), ([5, 6, 4, 8, 3], [[0, 1, 3, 4], [0, 2, 1, 4]], 3)),
    (([4, 5, 6], [[0, 1, 2], [0, 1, 2]], 3), ([120], [[0], [0]], 1)),
    (([1, 32, 2048, 2048, 128], [[0, 2, 1, 4], [0, 3, 1, 4]], 4),
     ([1, 32, 2048, 2048, 128], [[0, 2, 1, 4], [0, 3, 1, 4]], 4)),
    (([1, 2048, 4096, 32, 128], [[0, 3, 1, 4], [2, 3, 4]], 3),
     ([1, 2048, 4096, 32, 128], [[0, 3, 1, 4], [2, 3, 4]], 3)),
    (([32, 32, 2048, 128], [[0, 2, 1, 3]], 4), ([32, 32, 2048, 128], [[0, 2, 1, 3]], 4)),
    (([8, 16, 4], [[0, 1, 2]], 1), ([8, 64], [[0, 1]], 1)),
]


@pytest.mark.parametrize("case,want", MERGE_CASES)
def test_merge_adjacent_dims_known_answers(case, want):
    got = oracle.merge_adjacent_dims(*case)
    assert got == want


def test_merge_adjacent_dims_keeps_results():
    rs = np.random.RandomState(7)
    x = rs.normal(size=3 * 4 * 5 * 6)
    y = rs.normal(size=3 * 4)
    join = "*[hole|f64@0,hole|f64@1]"
    full = oracle.einsummable([3, 4, 5, 6], [[0, 1, 2, 3], [0, 1]], 4, join, None, [x, y])
    js, inns, orank = oracle.merge_adjacent_dims([3, 4, 5, 6], [[0, 1, 2, 3], [0, 1]], 4)
    merged = oracle.einsummable(js, inns, orank, join, None, [x, y])
    assert np.array_equal(full, merged)


def test_einsummable_constructor_errors():
    with pytest.raises(oracle.OracleError):   # aggregation without castable
        oracle.einsummable([2, 3], [[0, 1]], 1, "hole|f32@0", None, [np.zeros(6, np.float32)])
    with pytest.raises(oracle.OracleError):   # join arity mismatch
        oracle.einsummable([2], [[0], [0]], 1, "hole|f32@0", None, [np.zeros(2, np.float32)] * 2)
    with pytest.raises(oracle.OracleError):   # wrong join rank
        oracle.einsummable([2, 3, 4], [[0, 1]], 2, "hole|f32@0", None, [np.zeros(6, np.float32)])
    with pytest.raises(oracle.OracleError):   # duplicate mode in an input
        oracle.einsummable([2], [[0, 0]], 1, "hole|f32@0", None, [np.zeros(4, np.float32)])


# ------------------------------------------------------------------ permute, touch, fill

def test_permute_all_orders_against_numpy_and_golden():
    t = np.arange(3 * 4 * 5 * 6, dtype=np.float32).reshape(3, 4, 5, 6)
    for perm in itertools.permutations(range(4)):
        # out mode z is input mode perm[z]: join_shape is the out shape, the input lists, for
        # each of its own positions, the out mode it maps to
        out_shape = [t.shape[p] for p in perm]
        inn = [perm.index(i) for i in range(4)]
        got = oracle.einsummable(out_shape, [inn], 4, "hole|f32@0", None, [t])
        want = np.ascontiguousarray(np.transpose(t, perm))
        assert np.array_equal(got.reshape(want.shape), want)
        key = "".join(map(str, perm))
        assert hashlib.sha256(want.tobytes()).hexdigest() == GOLDEN["permute_3x4x5x6_sha256"][key]


@needs_ref
def test_permute_live_against_reference():
    t = np.arange(10 * 11 * 12 * 13, dtype=np.float32).reshape(10, 11, 12, 13)
    for perm in [(0, 2, 1, 3), (3, 2, 1, 0), (1, 0, 3, 2), (2, 3, 0, 1)]:
        assert np.array_equal(oracle.ref_permute(t, perm), np.transpose(t, perm))


def _numpy_touch(dims, castable, out, inn):
    o = out.reshape([d[1] for d in dims])
    i = inn.reshape([d[0] for d in dims])
    so = tuple(slice(d[3], d[3] + d[4]) for d in dims)
    si = tuple(slice(d[2], d[2] + d[4]) for d in dims)
    if castable is None:
        o[so] = i[si]
    elif castable == "+":
        o[so] = o[so] + i[si]
    elif castable == "x":
        o[so] = o[so] * i[si]
    elif castable == "v":
        o[so] = np.minimum(o[so], i[si])
    else:
        o[so] = np.maximum(o[so], i[si])
    return out


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.float64, np.complex64])
@pytest.mark.parametrize("castable", [None, "+", "x", "v", "^"])
def test_touch_against_numpy_slicing(dtype, castable):
    if dtype == np.complex64 and castable in ("v", "^"):
        with pytest.raises(oracle.OracleError):
            oracle.touch([(2, 2, 0, 0, 2)], castable, np.zeros(2, dtype), np.zeros(2, dtype))
        return
    rs = np.random.RandomState(8)
    for rank in (1, 2, 3, 4):
        for _ in range(6):
            dims = []
            for _ in range(rank):
                size = int(rs.randint(1, 5))
                oi, oo = int(rs.randint(0, 3)), int(rs.randint(0, 3))
                dims.append((size + oi + int(rs.randint(0, 3)), size + oo + int(rs.randint(0, 3)),
                             oi, oo, size))
            n_in = int(np.prod([d[0] for d in dims]))
            n_out = int(np.prod([d[1] for d in dims]))
            inn = rs.normal(size=n_in).astype(dtype)
            out = rs.normal(size=n_out).astype(dtype)
            if dtype == np.complex64:
                inn = (inn + 1j * rs.normal(size=n_in)).astype(dtype)
            want = _numpy_touch(dims, castable, out.copy(), inn)
            got = oracle.touch(dims, castable, out.copy(), inn)
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (dims, castable)
            # simplify() does not change the result
            simp = oracle.touch_simplify(dims)
            got2 = oracle.touch(simp, castable, out.copy(), inn)
            assert np.array_equal(got2.view(np.uint8), want.view(np.uint8))


def test_touch_simplify_known_answer():
    assert oracle.touch_simplify([(10, 10, 3, 3, 2), (20, 20, 0, 0, 20)]) == [(200, 200, 60, 60, 40)]
    assert oracle.touch_simplify([(4, 4, 0, 0, 4), (5, 5, 0, 0, 5)]) == [(20, 20, 0, 0, 20)]
    assert oracle.touch_simplify([(4, 6, 0, 1, 4), (5, 5, 0, 0, 5)]) == [(20, 30, 0, 5, 20)]
    keep = [(4, 6, 0, 1, 3), (5, 5, 1, 0, 4)]
    assert oracle.touch_simplify(keep) == keep
    with pytest.raises(oracle.OracleError):
        oracle.touch([(4, 4, 2, 0, 3)], None, np.zeros(4, np.float32), np.zeros(4, np.float32))


def test_fills_closed_form():
    c = oracle.fill_constant(np.float16, -1.5, 33)
    assert c.dtype == np.float16 and np.all(c == np.float16(-1.5))
    for nrow, ncol, start in [(5, 7, 0), (7, 5, 2), (6, 6, -2), (4, 4, 10), (4, 4, -10)]:
        m = oracle.fill_lowertri(np.float32, 0.0, -np.inf, nrow, ncol, start)
        i, j = np.indices((nrow, ncol))
        assert np.array_equal(m == 0.0, i - start >= j)
        assert np.array_equal(np.isneginf(m), ~(i - start >= j))
    # start == 0 on a square is numpy's tril
    m = oracle.fill_lowertri(np.float64, 1.0, 0.0, 6, 6, 0)
    assert np.array_equal(m, np.tril(np.ones((6, 6))))


def test_cpu_baseline_loops_agree_with_the_oracle():
    # the -O3 loops that bench.py times as the CPU baseline compute what the oracle computes
    r = np.random.RandomState(5)
    x = r.normal(0, 1, (37, 523)).astype(np.float16)
    y = r.normal(0, 1, (37, 523)).astype(np.float16)
    relu_mul = "*[ite_>=[constant{f16|0},hole|f16@0,constant{f16|0},hole|f16@0],hole|f16@1]"
    want = oracle.einsummable([37, 523], [[0, 1], [0, 1]], 2, relu_mul, None, [x, y], oracle.EXACT)
    for threads in (1, 3):
        got = oracle.loops_relu_mul(x, y, threads)
        assert np.array_equal(got.astype(np.float32), want.reshape(37, 523).astype(np.float32))
        m = oracle.loops_rowmax(x, threads)
        assert np.array_equal(m, x.max(axis=1))
        e = oracle.loops_exp_sub(x, m, threads)
        ref = np.exp(x.astype(np.float64) - m.astype(np.float64)[:, None])
        assert np.allclose(e.astype(np.float64), ref, rtol=1e-2, atol=1e-7)
        s = oracle.loops_rowsum(e, threads)
        assert np.allclose(s.astype(np.float64), e.astype(np.float64).sum(axis=1), rtol=2e-3)
        t = r.normal(0, 1, (3, 5, 4, 16)).astype(np.float16)
        assert np.array_equal(oracle.loops_permute_acbd(t, threads), t.transpose(0, 2, 1, 3))
        acc = r.normal(0, 1, (64, 96)).astype(np.float16)
        blk = r.normal(0, 1, (20, 33)).astype(np.float16)
        want_acc = oracle.touch([(20, 64, 0, 7, 20), (33, 96, 0, 11, 33)], "+", acc.copy(), blk)
        assert np.array_equal(oracle.loops_touch_add(acc.copy(), blk, 7, 11, threads).view(np.uint16),
                              want_acc.view(np.uint16))
