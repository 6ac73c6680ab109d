"""Parity of the MFMA contraction path with the CPU oracle (computed in double, rounded once):
every b/i/j/k mode arrangement the planner distinguishes, ragged sizes that exercise the tile
edges, and the LLaMA layer's forms at reduced sizes.  fp32 within 1e-4, fp16 within 1e-2 of
the higher-precision result; f64 to 1e-10."""
import numpy as np
import pytest

import einsummable_amd as ea
import oracle
from helpers import NP, assert_close, normal, oracle_einsummable, rng, run_einsummable, uniform

pytestmark = pytest.mark.gpu

E = ea.Einsummable
DT = {"f16": ea.F16, "f32": ea.F32, "f64": ea.F64, "c64": ea.C64}


def contraction(spec, sizes, dt):
    join = "*[hole|%s@0,hole|%s@1]" % (dt, dt)
    return E.from_str(spec, sizes, join, "+")


def check(km, spec, sizes, dt, seed=0, expect_mfma=True):
    e = contraction(spec, sizes, dt)
    r = rng(seed)
    xs = [uniform(r, int(np.prod(e.inn_shape(k))), NP[DT[dt]]) for k in range(2)]
    got = run_einsummable(km, e, xs)
    if expect_mfma and dt == "c64":
        # the complex product runs as an fp32 product of twice the depth on the matrix cores
        d = km.describe(e)
        assert d.startswith("contraction_c64_as_f32") and "contraction_mfma_f32" in d, d
    elif expect_mfma:
        assert km.describe(e).startswith("contraction_mfma_" + dt), km.describe(e)
    want = oracle_einsummable(e, xs, oracle.WIDE)
    assert_close(got, want, DT[dt], what="%s %s %s [%s]" % (spec, sizes, dt, km.describe(e)))


@pytest.mark.parametrize("dt", ["f16", "f32", "f64"])
def test_reference_known_answer_shape(km, dt):
    # tests/reference.h:4-49: 3x4 times 4x5 with iota(8) / iota(100)
    e = contraction("ij,jk->ik", dict(i=3, j=4, k=5), dt)
    lhs = np.arange(8, 20, dtype=NP[DT[dt]])
    rhs = np.arange(100, 120, dtype=NP[DT[dt]])
    got = run_einsummable(km, e, [lhs, rhs])
    want = np.array([4110, 4148, 4186, 4224, 4262, 5830, 5884, 5938, 5992, 6046, 7550, 7620, 7690,
                     7760, 7830], dtype=np.float64)
    assert_close(got, want, DT[dt], what="known-answer matmul")


MATMULS = ["ij,jk->ik", "ij,kj->ik", "ji,jk->ik", "ji,kj->ik",
           "jk,ij->ik", "kj,ij->ik", "jk,ji->ik", "kj,ji->ik"]


@pytest.mark.parametrize("dt", ["f16", "f32", "f64"])
@pytest.mark.parametrize("spec", MATMULS)
def test_all_matmul_spellings(km, spec, dt):
    check(km, spec, dict(i=64, j=96, k=80), dt, seed=1)       # vector paths
    check(km, spec, dict(i=37, j=51, k=29), dt, seed=2)       # ragged: elementwise paths


@pytest.mark.parametrize("dt", ["f16", "f32"])
def test_tile_edges_and_deep_k(km, dt):
    check(km, "ij,kj->ik", dict(i=130, j=264, k=136), dt, seed=3)
    check(km, "ij,kj->ik", dict(i=256, j=1024, k=128), dt, seed=4)
    check(km, "ij,jk->ik", dict(i=200, j=72, k=392), dt, seed=5)
    check(km, "ij,jk->ik", dict(i=1, j=512, k=8), dt, seed=6)
    check(km, "ij,jk->ik", dict(i=8, j=8, k=1), dt, seed=7)


BATCHED = [
    ("bij,bjk->bik", dict(b=3, i=40, j=48, k=56)),
    ("bij,jk->bik", dict(b=3, i=40, j=48, k=56)),        # b is an m mode here
    ("ibj,bjk->bik", dict(b=3, i=40, j=48, k=56)),       # batch in the middle of lhs
    ("bij,bjk->ikb", dict(b=4, i=24, j=16, k=40)),       # batch innermost in out
    ("bij,bkj->bki", dict(b=2, i=40, j=32, k=24)),       # lhs owns the innermost out mode
    ("abij,abkj->abik", dict(a=2, b=3, i=24, j=32, k=40)),
    ("aibj,akbj->abik", dict(a=2, b=3, i=24, j=32, k=40)),
]


@pytest.mark.parametrize("dt", ["f16", "f32", "f64"])
@pytest.mark.parametrize("spec,sizes", BATCHED)
def test_batched_forms(km, spec, sizes, dt):
    check(km, spec, sizes, dt, seed=8)


@pytest.mark.parametrize("dt", ["f16", "f32"])
def test_llama_attention_forms(km, dt):
    # scores acbe,adbe->abcd ; P.V abce,aebd->abcd ; out-proj adbe,cde->abc and adbe,dec->abc
    # (exps/gpuexec_kernelmanager.cc:993, 3120-3132; llama/modules.cc:315-352), reduced sizes
    check(km, "acbe,adbe->abcd", dict(a=1, b=4, c=72, d=88, e=64), dt, seed=9)
    check(km, "abce,aebd->abcd", dict(a=1, b=4, c=72, e=88, d=64), dt, seed=10)
    check(km, "adbe,cde->abc", dict(a=1, d=4, b=72, e=64, c=96), dt, seed=11)
    check(km, "adbe,dec->abc", dict(a=1, d=4, b=72, e=64, c=96), dt, seed=12)
    check(km, "bhid,bhjd->bhij", dict(b=2, h=3, i=40, j=56, d=128), dt, seed=13)
    check(km, "bhij,bhjd->bhid", dict(b=2, h=3, i=40, j=56, d=128), dt, seed=14)


@pytest.mark.parametrize("dt", ["f16", "f32"])
def test_multi_mode_groups(km, dt):
    # two k modes whose order differs between the operands, two m modes, two n modes
    check(km, "ipq,qpk->ik", dict(i=24, p=6, q=16, k=40), dt, seed=15)
    check(km, "xiyj,jk->xyik", dict(x=3, y=5, i=8, j=32, k=24), dt, seed=16)
    check(km, "ij,xjyk->iyxk", dict(x=3, y=5, i=8, j=32, k=24), dt, seed=17)


@pytest.mark.parametrize("spec", MATMULS)
def test_complex_matmul_spellings_run_on_the_matrix_cores(km, spec):
    # every spelling: the left operand in place (summed mode innermost) or split into planes,
    # the right one expanded along k or along n; the known-answer shape of tests/reference.h
    check(km, spec, dict(i=64, j=96, k=80), "c64", seed=31)
    check(km, spec, dict(i=37, j=51, k=29), "c64", seed=32)
    check(km, spec, dict(i=3, j=4, k=5), "c64", seed=33)
    check(km, spec, dict(i=130, j=264, k=136), "c64", seed=34)


def test_complex_matmul_closed_form(km):
    # (1 + i) times ones times (2 - i) ones: every entry is j * (1 + i)(2 - i) = j * (3 + i)
    e = contraction("ij,jk->ik", dict(i=40, j=48, k=56), "c64")
    lhs = np.full(40 * 48, 1 + 1j, np.complex64)
    rhs = np.full(48 * 56, 2 - 1j, np.complex64)
    got = run_einsummable(km, e, [lhs, rhs])
    assert np.array_equal(got, np.full(40 * 56, 48 * (3 + 1j), np.complex64))


COMPLEX_FORMS = [
    ("bij,bjk->bik", dict(b=3, i=40, j=48, k=56), True),
    ("bij,jk->bik", dict(b=3, i=40, j=48, k=56), True),
    ("ibj,bjk->bik", dict(b=3, i=40, j=48, k=56), True),
    ("bij,bkj->bki", dict(b=2, i=40, j=32, k=24), True),       # the left operand is expanded
    ("aibj,akbj->abik", dict(a=2, b=3, i=24, j=32, k=40), True),
    ("ipq,qpk->ik", dict(i=24, p=6, q=16, k=40), True),         # two summed modes, orders differ
    ("xiyj,jk->xyik", dict(x=3, y=5, i=8, j=32, k=24), True),
    ("ij,xjyk->iyxk", dict(x=3, y=5, i=8, j=32, k=24), True),
    ("acbe,adbe->abcd", dict(a=1, b=4, c=72, d=88, e=64), True),
    ("abce,aebd->abcd", dict(a=1, b=4, c=72, e=88, d=64), True),
    ("bij,bjk->ikb", dict(b=4, i=24, j=16, k=40), False),       # batch innermost: generated kernel
]


@pytest.mark.parametrize("spec,sizes,mfma", COMPLEX_FORMS)
def test_complex_contraction_forms(km, spec, sizes, mfma):
    check(km, spec, sizes, "c64", seed=35, expect_mfma=mfma)
    if not mfma:
        assert not km.describe(contraction(spec, sizes, "c64")).startswith("contraction_c64")


def test_complex_contraction_with_operands_off_the_vector_grid(km):
    """Operands and output 8 bytes off a 16-byte boundary (a complex element's own alignment):
    the expansion reads them as they lie, the fp32 product falls to its element paths."""
    import torch
    from helpers import stream_handle

    e = contraction("ij,kj->ik", dict(i=72, j=40, k=56), "c64")
    r = rng(36)
    xs = [uniform(r, 72 * 40, np.complex64), uniform(r, 56 * 40, np.complex64)]
    ws = km.build(e)
    bufs = []
    for x in xs:
        t = torch.zeros(x.size + 1, dtype=torch.complex64, device="cuda")
        t[1:] = torch.from_numpy(x).cuda()
        bufs.append(t)
    out = torch.zeros(72 * 56 + 1, dtype=torch.complex64, device="cuda")
    w = torch.empty(max(ws, 1), dtype=torch.uint8, device="cuda")
    km(e, stream_handle(), out.data_ptr() + 8, [b.data_ptr() + 8 for b in bufs], (w.data_ptr(), ws))
    torch.cuda.synchronize()
    want = oracle_einsummable(e, xs, oracle.WIDE)
    assert_close(out[1:].cpu().numpy(), want, ea.C64, what="c64 off the vector grid")
    assert out[0].item() == 0


def test_one_sided_aggregation_is_not_a_gemm(km):
    # j is summed over lhs only, l over rhs only: handled by the generated reduce kernel
    e = E.from_str("ij,kl->ik", dict(i=6, j=5, k=7, l=4), "*[hole|f32@0,hole|f32@1]", "+")
    r = rng(18)
    xs = [uniform(r, 30, np.float32), uniform(r, 28, np.float32)]
    got = run_einsummable(km, e, xs)
    assert not km.describe(e).startswith("contraction")
    assert_close(got, oracle_einsummable(e, xs, oracle.WIDE), ea.F32, what="one-sided agg")


def test_misaligned_operands_fall_back_to_elementwise_loads(km):
    import torch
    from helpers import stream_handle, to_host

    e = contraction("ij,kj->ik", dict(i=64, j=64, k=64), "f16")
    km.build(e)
    r = rng(19)
    a, b = uniform(r, 64 * 64, np.float16), uniform(r, 64 * 64, np.float16)
    da = torch.zeros(64 * 64 + 8, dtype=torch.float16, device="cuda")
    db = torch.zeros(64 * 64 + 8, dtype=torch.float16, device="cuda")
    dc = torch.zeros(64 * 64 + 8, dtype=torch.float16, device="cuda")
    da[1:1 + 4096] = torch.from_numpy(a).cuda()
    db[3:3 + 4096] = torch.from_numpy(b).cuda()
    km(e, stream_handle(), dc.data_ptr() + 2, [da.data_ptr() + 2, db.data_ptr() + 6])
    torch.cuda.synchronize()
    got = dc[1:1 + 4096].cpu().numpy()
    assert_close(got, oracle_einsummable(e, [a, b], oracle.WIDE), ea.F16, what="misaligned")


BIG_TILE_CASES = [
    # (spec, sizes, dtype, taken by the direct-to-LDS kernel)
    # k-contiguous operands: K a multiple of the 64-byte slice and at least four slices
    ("ij,kj->ik", dict(i=256, j=128, k=256), "f16", True),   # one tile, the minimum depth
    ("ij,kj->ik", dict(i=512, j=160, k=256), "f16", True),   # five slices: one steady-loop trip
    ("ij,kj->ik", dict(i=264, j=448, k=520), "f16", True),   # ragged m and n: clamped rows
    ("ij,kj->ik", dict(i=40, j=256, k=24), "f16", True),     # one partial tile
    ("bij,bkj->bik", dict(b=3, i=272, j=192, k=136), "f16", True),
    ("adbe,cde->abc", dict(a=2, d=4, b=136, e=64, c=264), "f16", True),  # two k modes
    ("acbe,adbe->abcd", dict(a=1, b=2, c=264, d=136, e=128), "f16", True),
    ("ij,kj->ik", dict(i=264, j=80, k=520), "f32", True),
    # B contiguous along n: kept [k][n] in LDS, read transposed
    ("ij,jk->ik", dict(i=264, j=160, k=264), "f16", True),
    ("ij,jk->ik", dict(i=264, j=128, k=520), "f16", True),
    ("ij,jk->ik", dict(i=40, j=256, k=24), "f16", True),
    ("bhij,bhjd->bhid", dict(b=2, h=2, i=264, j=192, d=128), "f16", True),
    ("abce,aebd->abcd", dict(a=1, b=3, c=136, e=160, d=64), "f16", True),
    ("ij,jk->ik", dict(i=264, j=80, k=264), "f32", True),
    ("ij,jk->ik", dict(i=130, j=64, k=520), "f32", True),
    ("bij,bjk->bik", dict(b=2, i=40, j=112, k=72), "f32", True),
    # A contiguous along m (a transposed lhs), with B along n or along k
    ("ji,jk->ik", dict(i=264, j=160, k=264), "f16", True),
    ("ji,kj->ik", dict(i=520, j=128, k=264), "f16", True),
    ("ji,jk->ik", dict(i=24, j=256, k=40), "f16", True),
    ("bji,bjk->bik", dict(b=3, i=136, j=192, k=264), "f16", True),
    ("jk,ji->ik", dict(i=264, j=160, k=136), "f16", True),      # operands swapped by the planner
    ("ji,jk->ik", dict(i=264, j=80, k=264), "f32", True),
    ("ji,kj->ik", dict(i=132, j=64, k=520), "f32", True),
    # K not a whole number of slices, or too short: the register-staged kernels
    ("ij,kj->ik", dict(i=264, j=72, k=264), "f16", False),
    ("ij,kj->ik", dict(i=264, j=296, k=264), "f16", False),
    ("ij,jk->ik", dict(i=264, j=100, k=264), "f32", False),
]
BIG_TILES = ["256x256", "128x256", "256x128"]


@pytest.mark.parametrize("tile", BIG_TILES)
@pytest.mark.parametrize("case", range(len(BIG_TILE_CASES)))
def test_big_tile_kernels(km, monkeypatch, case, tile):
    # a second manager (after the session's, which initialises the device) whose planner is
    # told which tile to use: left alone it keeps the large ones for problems too big for
    # the oracle
    monkeypatch.setenv("ES_KM_GEMM_TILE", tile)
    big = ea.KernelManager(0)
    spec, sizes, dt, direct = BIG_TILE_CASES[case]
    check(big, spec, sizes, dt, seed=20)
    d = big.describe(contraction(spec, sizes, dt))
    assert ("load=direct_to_lds" in d) == direct, d
    if direct or tile == "256x256":
        assert "tile=" + tile in d, d


EIGHT_WAVE_CASES = [
    # K a whole number of 128-byte slices: the eight-wavefront kernels, each operand along k
    # or along its own mode
    ("ij,jk->ik", dict(i=520, j=448, k=264)),                    # B along n
    ("ji,kj->ik", dict(i=264, j=448, k=520)),                    # A along m
    ("ji,jk->ik", dict(i=272, j=192, k=264)),                    # both
    ("bij,bjk->bik", dict(b=2, i=264, j=256, k=136)),
    ("ij,kj->ik", dict(i=512, j=512, k=512)),                    # full tiles
    ("ij,kj->ik", dict(i=264, j=448, k=520)),                    # ragged m and n, seven slices
    ("ij,kj->ik", dict(i=40, j=192, k=24)),                      # one partial tile, three slices
    ("bij,bkj->bik", dict(b=3, i=272, j=256, k=136)),
    ("adbe,cde->abc", dict(a=2, d=4, b=136, e=64, c=264)),       # two k modes
    ("ij,kj->ik", dict(i=8, j=4096, k=264)),                     # split-K, partial tiles folded
]


@pytest.mark.parametrize("tile", BIG_TILES)
@pytest.mark.parametrize("case", range(len(EIGHT_WAVE_CASES)))
def test_eight_wavefront_kernels_match_the_four_wavefront_ones_bitwise(km, monkeypatch, case, tile):
    # same products summed in the same order: the bits must agree on random data, and both
    # must agree with the oracle.  The default plan is a third kernel where both operands lie
    # along k (persistent workgroups, accumulators in named registers): the same bits again.
    spec, sizes = EIGHT_WAVE_CASES[case]
    e = contraction(spec, sizes, "f16")
    monkeypatch.setenv("ES_KM_GEMM_TILE", tile)
    default = ea.KernelManager(0)
    default.build(e)  # the planner reads its tuning variables when it plans
    monkeypatch.setenv("ES_KM_GEMM_WAVES", "8")
    eight = ea.KernelManager(0)
    eight.build(e)
    monkeypatch.setenv("ES_KM_GEMM_WAVES", "4")
    four = ea.KernelManager(0)
    four.build(e)
    r = rng(90 + case)
    xs = [uniform(r, int(np.prod(e.inn_shape(k))), np.float16) for k in range(2)]
    a = run_einsummable(eight, e, xs)
    b = run_einsummable(four, e, xs)
    c = run_einsummable(default, e, xs)
    assert "waves=8" in eight.describe(e), eight.describe(e)
    assert "waves=" not in four.describe(e) and "tile=" + tile in four.describe(e), four.describe(e)
    d = default.describe(e)
    along_k = " A=k B=k " in d and "split_k" not in d
    assert ("persistent" in d) == along_k, d
    if along_k:
        assert ("waves=4 persistent" if tile == "256x256" else "waves=4+4 persistent") in d, d
    np.testing.assert_array_equal(a.view(np.uint16), b.view(np.uint16))
    np.testing.assert_array_equal(a.view(np.uint16), c.view(np.uint16))
    assert_close(a, oracle_einsummable(e, xs, oracle.WIDE), ea.F16, what=eight.describe(e))


PERSISTENT_CASES = [
    # several tiles per workgroup, ragged edges (the output's inner extent in whole 16-byte
    # vectors: the wide epilogue), K not a multiple of the stage count
    ("ij,kj->ik", dict(i=2300, j=448, k=4504), "256x256"),
    ("ij,kj->ik", dict(i=2300, j=448, k=4504), "128x256"),
    ("ij,kj->ik", dict(i=4500, j=320, k=2296), "256x128"),
    # a batch of products walked across its entries; two k modes stepped by the slice walker
    ("bij,bkj->bik", dict(b=40, i=520, j=192, k=776), "128x256"),
    ("bij,bkj->bik", dict(b=9, i=1030, j=256, k=1288), "256x256"),
    ("adbe,cde->abc", dict(a=2, d=4, b=1100, e=64, c=2056), "128x256"),
    ("adbe,cde->abc", dict(a=1, d=3, b=2100, e=128, c=2056), "256x256"),
    # the scale applied to the fp32 sums in the epilogue
    ("ij,kj->ik", dict(i=1500, j=512, k=3000), "256x128"),
]


@pytest.mark.parametrize("case", range(len(PERSISTENT_CASES)))
def test_persistent_kernels_walk_many_tiles(km, monkeypatch, case):
    """More tiles than compute units: every workgroup of the persistent kernels computes
    several tiles, with the next tile's first slices loaded under the current one's last.
    Bitwise equal to the eight-wavefront kernel (same order of summation) and within the
    f16 tolerance of the oracle."""
    spec, sizes, tile = PERSISTENT_CASES[case]
    scaled = case == len(PERSISTENT_CASES) - 1
    e = contraction(spec, sizes, "f16")
    if scaled:
        e = ea.Einsummable(e.join_shape, e.inns, e.out_rank,
                           "*[constant{f16|0.0883789},*[hole|f16@0,hole|f16@1]]", "+")
    monkeypatch.setenv("ES_KM_GEMM_TILE", tile)
    pers = ea.KernelManager(0)
    pers.build(e)
    monkeypatch.setenv("ES_KM_GEMM_WAVES", "8")
    eight = ea.KernelManager(0)
    eight.build(e)
    assert "persistent" in pers.describe(e) and "tile=" + tile in pers.describe(e), pers.describe(e)
    assert "waves=8" in eight.describe(e), eight.describe(e)
    r = rng(300 + case)
    xs = [uniform(r, int(np.prod(e.inn_shape(k))), np.float16) for k in range(2)]
    a = run_einsummable(pers, e, xs)
    b = run_einsummable(eight, e, xs)
    np.testing.assert_array_equal(a.view(np.uint16), b.view(np.uint16))
    # the oracle on a sample of rows (the whole product would take it minutes)
    if not scaled and spec == "ij,kj->ik":
        i, j, k = sizes["i"], sizes["j"], sizes["k"]
        rows = np.array([0, 1, 127, 128, 255, 256, i // 2, i - 2, i - 1])
        sub = contraction(spec, dict(i=len(rows), j=j, k=k), "f16")
        want = oracle_einsummable(sub, [xs[0].reshape(i, j)[rows].reshape(-1), xs[1]], oracle.WIDE)
        assert_close(a.reshape(i, k)[rows].reshape(-1), want, ea.F16, what=pers.describe(e))


def test_big_tile_matches_small_tile_bitwise_on_exact_data(km, monkeypatch):
    # small integers: every product and partial sum is exact in fp32, so both tilings must
    # give the same bits whatever their summation order
    e = contraction("ij,kj->ik", dict(i=520, j=256, k=392), "f16")
    km.build(e)  # planned with the default tile rule
    monkeypatch.setenv("ES_KM_GEMM_TILE", "256x256")
    km_big_tiles = ea.KernelManager(0)
    r = rng(21)
    xs = [r.randint(-4, 5, size=520 * 256).astype(np.float16),
          r.randint(-4, 5, size=392 * 256).astype(np.float16)]
    a = run_einsummable(km, e, xs)
    b = run_einsummable(km_big_tiles, e, xs)
    assert "tile=128x128" in km.describe(e) and "tile=256x256" in km_big_tiles.describe(e)
    want = (xs[0].astype(np.float64).reshape(520, 256) @
            xs[1].astype(np.float64).reshape(392, 256).T).astype(np.float16)
    np.testing.assert_array_equal(a.view(np.uint16), b.view(np.uint16))
    np.testing.assert_array_equal(a.reshape(520, 392), want)


SPLIT_K_CASES = [
    # few tiles and a long reduction: several workgroups per tile, fp32 partial tiles in the
    # workspace, a fold kernel; all four operand layouts, batch, ragged m / n, a one-row lhs
    ("ij,kj->ik", dict(i=8, j=2048, k=264), "f16"),
    ("ij,jk->ik", dict(i=1, j=1024, k=256), "f16"),
    ("ji,jk->ik", dict(i=136, j=1536, k=72), "f16"),
    ("ji,kj->ik", dict(i=40, j=1024, k=136), "f16"),
    ("bij,bkj->bik", dict(b=3, i=24, j=1024, k=40), "f16"),
    ("ij,kj->ik", dict(i=130, j=1008, k=136), "f32"),
    ("ij,jk->ik", dict(i=8, j=4096, k=64), "f32"),
]


@pytest.mark.parametrize("case", range(len(SPLIT_K_CASES)))
def test_split_k_contractions(km, case):
    spec, sizes, dt = SPLIT_K_CASES[case]
    e = contraction(spec, sizes, dt)
    ws = km.build(e)
    assert ws and "split_k=" in km.describe(e), km.describe(e)
    check(km, spec, sizes, dt, seed=40 + case)


def test_split_k_is_deterministic_and_checks_its_workspace(km):
    import torch
    from helpers import stream_handle

    e = contraction("ij,kj->ik", dict(i=8, j=2048, k=264), "f16")
    ws = km.build(e)
    assert ws > 0
    r = rng(50)
    xs = [uniform(r, 8 * 2048, np.float16), uniform(r, 264 * 2048, np.float16)]
    a = run_einsummable(km, e, xs)
    b = run_einsummable(km, e, xs)
    np.testing.assert_array_equal(a.view(np.uint16), b.view(np.uint16))
    d = torch.zeros(264 * 2048, dtype=torch.float16, device="cuda")
    with pytest.raises(ea.KmError) as ei:
        km(e, stream_handle(), d.data_ptr(), [d.data_ptr(), d.data_ptr()])
    assert ei.value.code == -3


RESIDENT_A_CASES = [
    # reductions of exactly 128 fp16 elements over enough rows of tiles: the lhs rows
    # stay in registers and a workgroup walks along n.  Full tiles, ragged m and n, a batch
    # of two modes with strides (heads stored between sequence and head dimension), more
    # than 16 tiles along n (several walks per row of tiles)
    ("bid,bjd->bij", dict(b=128, i=1024, j=1024, d=128)),
    ("bid,bjd->bij", dict(b=130, i=1000, j=1016, d=128)),
    ("bihd,bjhd->bhij", dict(b=8, h=16, i=1024, j=1024, d=128)),
    ("bid,bjd->bij", dict(b=43, i=1024, j=5000, d=128)),
]


@pytest.mark.parametrize("case", range(len(RESIDENT_A_CASES)))
def test_resident_lhs_kernel_for_head_dimension_reductions(km, monkeypatch, case):
    spec, sizes = RESIDENT_A_CASES[case]
    e = contraction(spec, sizes, "f16")
    km.build(e)
    assert "resident_a" in km.describe(e), km.describe(e)
    monkeypatch.setenv("ES_KM_GEMM_RESIDENT_A", "0")
    per_tile = ea.KernelManager(0)
    per_tile.build(e)
    assert "resident_a" not in per_tile.describe(e)
    r = rng(60 + case)
    xs = [normal(r, int(np.prod(e.inn_shape(k))), np.float16) for k in range(2)]
    a = run_einsummable(km, e, xs)
    b = run_einsummable(per_tile, e, xs)
    # both kernels add the same eight 16-wide products per output in the same order
    np.testing.assert_array_equal(a.view(np.uint16), b.view(np.uint16))
    # and a slice of it against the oracle (the whole product is billions of flops)
    lhs_shape, rhs_shape = e.inn_shape(0), e.inn_shape(1)
    if spec.startswith("bid"):
        L = xs[0].reshape(lhs_shape)[-1:, -136:, :]
        R = xs[1].reshape(rhs_shape)[-1:, -264:, :]
        sub = contraction(spec, dict(b=1, i=136, j=264, d=128), "f16")
        got = a.reshape(sizes["b"], sizes["i"], sizes["j"])[-1:, -136:, -264:]
    else:
        L = xs[0].reshape(lhs_shape)[-1:, -136:, -1:, :]
        R = xs[1].reshape(rhs_shape)[-1:, -264:, -1:, :]
        sub = contraction(spec, dict(b=1, h=1, i=136, j=264, d=128), "f16")
        got = a.reshape(sizes["b"], sizes["h"], sizes["i"], sizes["j"])[-1:, -1:, -136:, -264:]
    want = oracle_einsummable(sub, [np.ascontiguousarray(L).reshape(-1),
                                    np.ascontiguousarray(R).reshape(-1)], oracle.WIDE)
    assert_close(np.ascontiguousarray(got).reshape(-1), want, DT["f16"], what=spec)


@pytest.mark.parametrize("grid,resident_min", [(24, 1), (8, 1), (4096, 1)])
def test_resident_lhs_kernel_streams_of_walks(monkeypatch, grid, resident_min):
    """The resident-lhs kernel with a forced number of workgroups: few (every workgroup works
    through many walks, among them the short last walk of a row of 19 tiles), and more than
    there are walks (workgroups without work).  Bitwise against the kernel that takes a
    workgroup per tile."""
    spec, sizes = "bid,bjd->bij", dict(b=5, i=300, j=2400, d=128)
    e = contraction(spec, sizes, "f16")
    monkeypatch.setenv("ES_KM_GEMM_RESIDENT_MIN", str(resident_min))
    monkeypatch.setenv("ES_KM_GEMM_RESIDENT_GRID", str(grid))
    streamed = ea.KernelManager(0)
    streamed.build(e)
    assert "resident_a" in streamed.describe(e), streamed.describe(e)
    monkeypatch.setenv("ES_KM_GEMM_RESIDENT_A", "0")
    per_tile = ea.KernelManager(0)
    per_tile.build(e)
    assert "resident_a" not in per_tile.describe(e)
    r = rng(77)
    xs = [normal(r, int(np.prod(e.inn_shape(k))), np.float16) for k in range(2)]
    a = run_einsummable(streamed, e, xs)
    b = run_einsummable(per_tile, e, xs)
    np.testing.assert_array_equal(a.view(np.uint16), b.view(np.uint16))


def scaled(spec, sizes, dt, const, form=0):
    c = "constant{%s|%s}" % (dt, const)
    prod = ["*[hole|%s@0,hole|%s@1]", "*[hole|%s@1,hole|%s@0]"][form & 1] % (dt, dt)
    join = ("*[%s,%s]" % (c, prod)) if form < 2 else ("*[%s,%s]" % (prod, c))
    return E.from_str(spec, sizes, join, "+")


SCALED_CASES = [
    # (spec, sizes, dtype, constant, what it must run on); the constant is the attention
    # scale 1/sqrt(128) as the reference prints it (six digits, then rounded to the dtype)
    ("bid,bjd->bij", dict(b=130, i=1000, j=1016, d=128), "f16", "0.0883789", "resident_a"),
    ("bid,bjd->bij", dict(b=3, i=136, j=264, d=128), "f16", "0.0883789", "direct_to_lds"),
    ("ij,kj->ik", dict(i=8, j=2048, k=264), "f16", "0.0883789", "split_k="),
    ("ij,jk->ik", dict(i=130, j=264, k=136), "f32", "0.0883883", "C=wide"),
    ("ij,jk->ik", dict(i=130, j=256, k=136), "f32", "0.0883883", "direct_to_lds"),
    ("ij,kj->ik", dict(i=130, j=1008, k=136), "f32", "-2.5", "split_k="),
    ("ij,jk->ik", dict(i=37, j=51, k=29), "f16", "0.0883789", "A=elem"),
    ("ji,jk->ik", dict(i=64, j=96, k=80), "f64", "0.3", "contraction_mfma_f64"),
]


@pytest.mark.parametrize("case", range(len(SCALED_CASES)))
def test_product_times_a_constant_is_one_contraction(km, case):
    spec, sizes, dt, const, path = SCALED_CASES[case]
    for form in range(4 if case == 1 else 1):
        e = scaled(spec, sizes, dt, const, form)
        r = rng(70 + case)
        xs = [normal(r, int(np.prod(e.inn_shape(k))), NP[DT[dt]]) for k in range(2)]
        got = run_einsummable(km, e, xs)
        d = km.describe(e)
        assert d.startswith("contraction_mfma_" + dt) and path in d and d.endswith(" scaled"), d
        if case == 0:
            # a slice against the oracle, and the whole against the unscaled product times
            # the constant in fp32 (one rounding apart at most)
            L = xs[0].reshape(130, 1000, 128)[-1:, -136:, :]
            R = xs[1].reshape(130, 1016, 128)[-1:, -264:, :]
            sub = scaled(spec, dict(b=1, i=136, j=264, d=128), dt, const, form)
            want = oracle_einsummable(sub, [np.ascontiguousarray(L).reshape(-1),
                                            np.ascontiguousarray(R).reshape(-1)], oracle.WIDE)
            part = got.reshape(130, 1000, 1016)[-1:, -136:, -264:]
            assert_close(np.ascontiguousarray(part).reshape(-1), want, DT[dt], what=spec)
            plain = run_einsummable(km, contraction(spec, sizes, dt), xs).astype(np.float32)
            assert_close(got, plain * np.float32(np.float16(float(const))), DT[dt], what="scaled")
        else:
            want = oracle_einsummable(e, xs, oracle.WIDE)
            assert_close(got, want, DT[dt], what="%s %s [%s]" % (spec, e.join, d))


def test_scale_of_one_and_swapped_holes_are_the_plain_product(km):
    sizes = dict(i=136, j=256, k=72)
    r = rng(80)
    xs = [normal(r, 136 * 256, np.float16), normal(r, 256 * 72, np.float16)]
    plain = run_einsummable(km, contraction("ij,jk->ik", sizes, "f16"), xs)
    swapped = E.from_str("ij,jk->ik", sizes, "*[hole|f16@1,hole|f16@0]", "+")
    got = run_einsummable(km, swapped, xs)
    assert km.describe(swapped).startswith("contraction_mfma_f16")
    np.testing.assert_array_equal(got.view(np.uint16), plain.view(np.uint16))
    one = scaled("ij,jk->ik", sizes, "f16", "1")
    got = run_einsummable(km, one, xs)
    assert not km.describe(one).endswith(" scaled")
    np.testing.assert_array_equal(got.view(np.uint16), plain.view(np.uint16))


WIDE_SLICE_CASES = [
    # products bound by the reads of one large operand take 128-byte slices by themselves;
    # ragged m and n, both layouts of the small operand, a reduction of exactly two slices
    ("bij,bjd->bid", dict(b=40, i=1000, j=1984, d=120)),
    ("ij,kj->ik", dict(i=40000, j=1024, k=72)),
    ("bij,bjd->bid", dict(b=300, i=136, j=128, d=64)),
    ("abce,aebd->abcd", dict(a=2, b=24, c=520, e=576, d=128)),
]


@pytest.mark.parametrize("stages", ["", "2", "3"])
@pytest.mark.parametrize("case", range(len(WIDE_SLICE_CASES)))
def test_whole_cache_line_slices_equal_half_line_slices_bitwise(monkeypatch, case, stages):
    spec, sizes = WIDE_SLICE_CASES[case]
    e = contraction(spec, sizes, "f16")
    r = rng(90 + case)
    xs = [normal(r, int(np.prod(e.inn_shape(k))), np.float16) for k in range(2)]
    if stages:
        monkeypatch.setenv("ES_KM_GEMM_WIDE_SLICES", stages)
    wide = ea.KernelManager(0)
    wide.build(e)
    if stages != "2" and case == 2:
        # two slices cannot fill three stages, and by itself the planner keeps reductions
        # this short on half-line slices
        assert "slices=128B" not in wide.describe(e)
        return
    assert "slices=128B" in wide.describe(e), wide.describe(e)
    monkeypatch.setenv("ES_KM_GEMM_WIDE_SLICES", "0")
    half = ea.KernelManager(0)
    half.build(e)
    assert "slices=128B" not in half.describe(e)
    a = run_einsummable(wide, e, xs)
    b = run_einsummable(half, e, xs)
    # the k-steps run in the same order through the same matrix instructions
    np.testing.assert_array_equal(a.view(np.uint16), b.view(np.uint16))
    if case == 2:
        want = oracle_einsummable(e, xs, oracle.WIDE)
        assert_close(a, want, DT["f16"], what=spec)


@pytest.mark.parametrize("spec", ["ij,jk->ik", "ij,kj->ik"])
@pytest.mark.parametrize("stages", ["", "2", "3"])
def test_whole_cache_line_slices_fp32(monkeypatch, spec, stages):
    # at most one tile per compute unit and no split-K: four stages by default
    sizes = dict(i=1500, j=1056, k=1700)
    e = contraction(spec, sizes, "f32")
    r = rng(95)
    xs = [uniform(r, int(np.prod(e.inn_shape(k))), np.float32) for k in range(2)]
    monkeypatch.setenv("ES_KM_GEMM_TILE", "128x128")    # 168 tiles: no split-K
    if stages:
        monkeypatch.setenv("ES_KM_GEMM_WIDE_SLICES", stages)
    wide = ea.KernelManager(0)
    wide.build(e)
    assert "slices=128B" in wide.describe(e) and "split_k" not in wide.describe(e), wide.describe(e)
    monkeypatch.setenv("ES_KM_GEMM_WIDE_SLICES", "0")
    half = ea.KernelManager(0)
    half.build(e)
    assert "slices=128B" not in half.describe(e)
    a = run_einsummable(wide, e, xs)
    b = run_einsummable(half, e, xs)
    np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))
    if not stages:
        want = oracle_einsummable(e, xs, oracle.WIDE)
        assert_close(a, want, DT["f32"], what=spec)
