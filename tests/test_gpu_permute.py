"""N-D permutes through the C ABI, bit-exact against numpy's transpose and the oracle
(procedure of exps/cpuexec_permute.cc:33-77: every permutation of a 10x11x12x130 iota tensor
compared exactly with the interpreter)."""
import itertools

import numpy as np
import pytest

import einsummable_amd as ea
import oracle
from helpers import NP, assert_bits_equal, normal, rng, run_einsummable

pytestmark = pytest.mark.gpu


def permute_einsummable(in_shape, perm, dt):
    """out mode z is input mode perm[z] (numpy.transpose convention)."""
    out_shape = [in_shape[p] for p in perm]
    inn = [perm.index(i) for i in range(len(in_shape))]
    return ea.Einsummable(out_shape, [inn], len(in_shape), "hole|%s@0" % dt)


@pytest.mark.parametrize("perm", list(itertools.permutations(range(4))))
def test_all_permutations_of_a_4d_iota_tensor(km, perm):
    shape = (10, 11, 12, 130)
    t = np.arange(int(np.prod(shape)), dtype=np.float32).reshape(shape)
    e = permute_einsummable(shape, perm, "f32")
    got = run_einsummable(km, e, [t])
    want = np.ascontiguousarray(np.transpose(t, perm)).reshape(-1)
    assert_bits_equal(got, want, "permute %s [%s]" % (perm, km.describe(e)))


@pytest.mark.parametrize("dt,npdt", [("f16", np.float16), ("f64", np.float64), ("c64", np.complex64)])
def test_transposes_of_other_widths_and_ragged_tiles(km, dt, npdt):
    r = rng(50)
    for shape, perm in [((70, 33), (1, 0)), ((64, 64), (1, 0)), ((1, 200), (1, 0)),
                        ((5, 65, 67), (2, 1, 0)), ((3, 4, 129, 2), (3, 0, 2, 1)),
                        ((257, 3, 66), (2, 0, 1))]:
        x = normal(r, int(np.prod(shape)), npdt).reshape(shape)
        e = permute_einsummable(shape, perm, dt)
        got = run_einsummable(km, e, [x])
        want = np.ascontiguousarray(np.transpose(x, perm)).reshape(-1)
        assert_bits_equal(got, want, "permute %s %s" % (shape, perm))
        od, _ = oracle.scalarop_info(e.join)
        ref = oracle.einsummable(e.join_shape, e.inns, e.out_rank, e.join, None, [x])
        assert_bits_equal(ref, want, "oracle permute")


def test_kernel_choice(km):
    # innermost mode preserved: generated row copy; innermost mode changed: LDS transpose
    e1 = permute_einsummable((8, 16, 4, 64), (0, 2, 1, 3), "f16")
    e2 = permute_einsummable((8, 16, 4, 64), (0, 3, 2, 1), "f16")
    km.build(e1)
    km.build(e2)
    assert km.describe(e1).startswith("elementwise")
    assert km.describe(e2).startswith("transpose_lds")


@pytest.mark.parametrize("dt,npdt", [("f16", np.float16), ("f32", np.float32), ("f64", np.float64),
                                     ("c64", np.complex64)])
def test_transposes_with_16_byte_rows_use_vector_accesses(km, dt, npdt):
    r = rng(51)
    v = 16 // np.dtype(npdt).itemsize
    for shape, perm in [((9 * v, 17 * v), (1, 0)), ((3, 9 * v, 17 * v), (0, 2, 1)),
                        ((8 * v, 3, 5, 8 * v), (3, 1, 2, 0)), ((2 * v, 7, 11 * v), (2, 1, 0)),
                        ((64, 64), (1, 0)), ((128, 192), (1, 0))]:
        x = normal(r, int(np.prod(shape)), npdt).reshape(shape)
        e = permute_einsummable(shape, perm, dt)
        got = run_einsummable(km, e, [x])
        assert "vec16" in km.describe(e), km.describe(e)
        want = np.ascontiguousarray(np.transpose(x, perm)).reshape(-1)
        assert_bits_equal(got, want, "permute %s %s" % (shape, perm))


def test_vector_transpose_falls_back_when_a_buffer_is_misaligned(km):
    import torch
    from helpers import stream_handle

    x = normal(rng(52), 72 * 136, np.float16).reshape(72, 136)
    e = permute_einsummable((72, 136), (1, 0), "f16")
    km.build(e)
    din = torch.zeros(72 * 136 + 8, dtype=torch.float16, device="cuda")
    dout = torch.zeros(72 * 136 + 8, dtype=torch.float16, device="cuda")
    din[1:1 + 72 * 136] = torch.from_numpy(x.reshape(-1)).cuda()
    km(e, stream_handle(), dout.data_ptr() + 6, [din.data_ptr() + 2])
    torch.cuda.synchronize()
    got = dout[3:3 + 72 * 136].cpu().numpy()
    assert_bits_equal(got, np.ascontiguousarray(x.T).reshape(-1), "misaligned transpose")


def test_wide_tile_of_4_byte_transposes_with_ragged_edges(km):
    # enough tiles for the 128 x 64 tile; neither extent is a multiple of the tile
    shape, perm = (3, 3000, 2008), (0, 2, 1)
    x = normal(rng(53), int(np.prod(shape)), np.float32).reshape(shape)
    e = permute_einsummable(shape, perm, "f32")
    got = run_einsummable(km, e, [x])
    assert "tile=128x64 vec16 cached_stores" in km.describe(e), km.describe(e)
    want = np.ascontiguousarray(np.transpose(x, perm)).reshape(-1)
    assert_bits_equal(got, want, "permute %s %s" % (shape, perm))


def test_transpose_beyond_a_gibibyte_takes_the_long_tile(km):
    import torch
    from helpers import stream_handle

    # 2-byte elements: 256 x 64 tile; 23176 x 23176 is just past 1 GiB in + out, ragged
    n_a, n_b = 23176, 23184
    e = permute_einsummable((n_a, n_b), (1, 0), "f16")
    km.build(e)
    d = km.describe(e)
    assert "tile=256x64 vec16 cached_stores" in d, d
    g = torch.Generator(device="cuda").manual_seed(54)
    x = torch.randint(0, 1 << 15, (n_a, n_b), device="cuda", dtype=torch.int16, generator=g)
    y = torch.full((n_b, n_a), -1, device="cuda", dtype=torch.int16)
    km(e, stream_handle(), y.data_ptr(), [x.data_ptr()])
    torch.cuda.synchronize()
    assert torch.equal(y, x.t())


@pytest.mark.parametrize("stores,order", [("stream", 0), ("cached", 1), ("cached", 2), ("stream", 2)])
@pytest.mark.parametrize("dt,npdt,tile", [("f16", np.float16, "256x64"), ("f32", np.float32, "128x64")])
def test_long_tiles_forced_on_small_ragged_transposes(monkeypatch, dt, npdt, tile, stores, order):
    # the switches are read when a plan is made: a manager of its own, so that no plan made
    # under them stays in the session's manager.  `order`: the tile a workgroup takes (launch
    # order; one run of tiles per XCD; the same with the output-inner mode first), on tile
    # counts that do not divide by the eight XCDs
    monkeypatch.setenv("ES_KM_TRANSPOSE_TILE", "long")
    monkeypatch.setenv("ES_KM_TRANSPOSE_STORES", stores)
    monkeypatch.setenv("ES_KM_TRANSPOSE_ORDER", str(order))
    km = ea.KernelManager(0)
    r = rng(55)
    for shape, perm in [((264, 72), (1, 0)), ((2, 520, 136), (0, 2, 1)), ((8, 3, 776), (2, 1, 0)),
                        ((1032, 1160), (1, 0))]:
        x = normal(r, int(np.prod(shape)), npdt).reshape(shape)
        e = permute_einsummable(shape, perm, dt)
        got = run_einsummable(km, e, [x])
        d = km.describe(e)
        assert ("tile=%s vec16" % tile) in d and ("cached_stores" in d) == (stores == "cached"), d
        assert ("xcd_runs" in d) == (order != 0) and ("out_first" in d) == (order == 2), d
        want = np.ascontiguousarray(np.transpose(x, perm)).reshape(-1)
        assert_bits_equal(got, want, "permute %s %s" % (shape, perm))


@pytest.mark.parametrize("dt,npdt", [("f16", np.float16), ("f32", np.float32), ("c64", np.complex64)])
def test_row_permutes_in_pairs_of_input_neighbours(monkeypatch, dt, npdt):
    """A permutation that keeps the innermost mode is a copy of rows; for large ones a thread
    moves the same vector of two rows that are neighbours in the input.  Forced here at small
    sizes: inner extents that are and are not powers of two (shift and division), a last
    workgroup that is not full, and shapes whose mode next to the innermost one in the input
    has an odd extent, which keep the plain mapping."""
    monkeypatch.setenv("ES_KM_EW_PAIR", "2")
    km = ea.KernelManager(0)
    r = rng(57)
    v = 16 // np.dtype(npdt).itemsize
    cases = [((3, 64, 4, 8 * v), (0, 2, 1, 3), True),       # abcd->acbd, inner count a power of two
             ((2, 6, 10, 3 * v), (0, 2, 1, 3), True),       # 6 x 3 vectors under the pair: division
             ((5, 7, 2, v), (2, 0, 1, 3), True),            # the paired mode is outermost in the output
             ((4, 3, 6, 5 * v), (1, 2, 0, 3), True),
             ((3, 8, 5, 4 * v), (0, 2, 1, 3), False),       # 5 rows next to each other: odd
             ((6, 4, 2 * v), (1, 0, 2), True),
             ((2, 3, 4, 2 * v), (1, 0, 2, 3), False)]       # c and d merge; next to them in the input: 3 rows
    for shape, perm, paired in cases:
        x = normal(r, int(np.prod(shape)), npdt).reshape(shape)
        e = permute_einsummable(shape, perm, dt)
        got = run_einsummable(km, e, [x])
        d = km.describe(e)
        assert d.startswith("elementwise") and ("row_pairs" in d) == paired, (shape, perm, d)
        want = np.ascontiguousarray(np.transpose(x, perm)).reshape(-1)
        assert_bits_equal(got, want, "permute %s %s" % (shape, perm))
