"""Bit-exact parity of touch / fill kernels with the CPU oracle (procedure of the reference's
exps/cpuexec_touch.cc:18-114: random 1-4-D touches, every dtype and castable, exact
equality)."""
import numpy as np
import pytest

import einsummable_amd as ea
import oracle
from helpers import NP, assert_bits_equal, empty_device, normal, rng, stream_handle, to_device, to_host

pytestmark = pytest.mark.gpu

CASTABLES = [None, "+", "x", "v", "^"]


def random_touch(r, rank, aligned):
    dims = []
    for i in range(rank):
        q = 8 if (aligned and i == rank - 1) else 1
        size = int(r.randint(1, 6)) * q
        off_i = int(r.randint(0, 4)) * q
        off_o = int(r.randint(0, 4)) * q
        d_inn = size + off_i + int(r.randint(0, 3)) * q
        d_out = size + off_o + int(r.randint(0, 3)) * q
        dims.append((d_inn, d_out, off_i, off_o, size))
    return dims


def run_touch(km, dims, castable, dt, r):
    n_inn = int(np.prod([d[0] for d in dims]))
    n_out = int(np.prod([d[1] for d in dims]))
    inn = normal(r, n_inn, NP[dt])
    out0 = normal(r, n_out, NP[dt])
    want = oracle.touch(dims, castable, out0.copy(), inn)
    d_inn, d_out = to_device(inn), to_device(out0)
    km.touch(ea.Touch(dims, castable, dt), stream_handle(), d_out.data_ptr(), d_inn.data_ptr())
    got = to_host(d_out, NP[dt])
    assert_bits_equal(got, want, "touch %s castable=%s dtype=%d" % (dims, castable, dt))


@pytest.mark.parametrize("dt", [ea.F16, ea.F32, ea.F64, ea.C64])
@pytest.mark.parametrize("castable", CASTABLES)
def test_random_touches(km, dt, castable):
    if dt == ea.C64 and castable in ("v", "^"):
        pytest.skip("min/max of complex values is not defined (engine/touch.cc:228-234)")
    r = rng(1000 + dt * 10 + CASTABLES.index(castable))
    for rank in (1, 2, 3, 4):
        for aligned in (False, True):
            for _ in range(3):
                run_touch(km, random_touch(r, rank, aligned), castable, dt, r)


def test_touch_simplify_merges_full_dims(km):
    # X[3:5, 0:20] = Y[3:5, 0:20] for (10, 20) matrices becomes a 1-D touch
    # (example in src/einsummable/touch.h:30-37)
    dims = [(10, 10, 3, 3, 2), (20, 20, 0, 0, 20)]
    assert oracle.touch_simplify(dims) == [(200, 200, 60, 60, 40)]
    run_touch(km, dims, None, ea.F32, rng(5))
    # six dimensions that simplify to two
    dims6 = [(4, 5, 1, 2, 2), (3, 3, 0, 0, 3), (2, 2, 0, 0, 2), (6, 7, 1, 0, 4), (2, 2, 0, 0, 2),
             (8, 8, 0, 0, 8)]
    assert len(oracle.touch_simplify(dims6)) == 2
    run_touch(km, dims6, "+", ea.F16, rng(6))


def test_touch_errors(km):
    d = to_device(np.zeros(64, np.float32))
    with pytest.raises(ea.KmError) as ei:
        km.touch(ea.Touch([(4, 4, 2, 0, 3)], None, ea.F32), 0, d.data_ptr(), d.data_ptr())
    assert ei.value.code == -1
    five = [(3, 4, 0, 1, 2)] * 5
    with pytest.raises(ea.KmError):
        km.touch(ea.Touch(five, None, ea.F32), 0, d.data_ptr(), d.data_ptr())


def test_overlapping_accumulate_windows_in_order(km):
    """64 sum-accumulate touches of 512x512 blocks into random windows of a zeroed
    4096x4096 f16 matrix, applied in list order (the memory-movement configuration)."""
    r = rng(7)
    n, b, count = 4096, 512, 64
    out_ref = np.zeros(n * n, np.float16)
    d_out = empty_device(n * n, np.float16, 0.0)
    for _ in range(count):
        ro, co = int(r.randint(0, n - b + 1)), int(r.randint(0, n - b + 1))
        blk = normal(r, b * b, np.float16)
        dims = [(b, n, 0, ro, b), (b, n, 0, co, b)]
        oracle.touch(dims, "+", out_ref, blk)
        d_blk = to_device(blk)
        km.touch(ea.Touch(dims, "+", ea.F16), stream_handle(), d_out.data_ptr(), d_blk.data_ptr())
    assert_bits_equal(to_host(d_out, np.float16), out_ref, "64 accumulate touches")


@pytest.mark.parametrize("dt", [ea.F16, ea.F32, ea.F64, ea.C64])
def test_constant_fill(km, dt):
    value = {ea.F16: -1.5, ea.F32: 3.25, ea.F64: 1e-300, ea.C64: 1.5 - 2.5j}[dt]
    bits = oracle._to_bits(value, dt)
    for n in (1, 7, 8, 9, 1000, 4097):
        for shift in (0, 1):
            buf = empty_device(n + 16, NP[dt], 0.0)
            ptr = buf.data_ptr() + shift * np.dtype(NP[dt]).itemsize
            km.constant_fill(dt, bits, n, stream_handle(), ptr)
            got = to_host(buf, NP[dt])
            want = np.zeros(n + 16, NP[dt])
            want[shift:shift + n] = oracle.fill_constant(NP[dt], value, n)
            assert_bits_equal(got, want, "constant fill n=%d shift=%d" % (n, shift))


@pytest.mark.parametrize("dt", [ea.F16, ea.F32, ea.F64])
def test_lowertri_fill(km, dt):
    lower, upper = 0.0, -np.inf
    lb, ub = oracle._to_bits(lower, dt), oracle._to_bits(upper, dt)
    for nrow, ncol, start in [(8, 8, 0), (5, 7, 0), (7, 5, 2), (16, 24, -3), (9, 16, 20), (6, 8, -20),
                              (2048, 2048, 0)]:
        buf = empty_device(nrow * ncol, NP[dt], 1.0)
        km.lowerTri_fill(dt, lb, ub, nrow, ncol, start, stream_handle(), buf.data_ptr())
        got = to_host(buf, NP[dt]).reshape(nrow, ncol)
        want = oracle.fill_lowertri(NP[dt], lower, upper, nrow, ncol, start)
        assert_bits_equal(got, want, "lowertri %dx%d start=%d" % (nrow, ncol, start))
        # closed form (src/einsummable/fill.h:17-19)
        i, j = np.indices((nrow, ncol))
        assert np.array_equal(np.isinf(want), ~(i - start >= j))


def _apply_sequentially(touches, blocks, out0):
    ref = out0.copy()
    for t, blk in zip(touches, blocks):
        oracle.touch(t.selection, t.castable, ref, blk)
    return ref


@pytest.mark.parametrize("dt", [ea.F16, ea.F32, ea.C64])
def test_touch_batch_equals_sequential_touches(km, dt):
    """One call for a whole group of touches into the same output: bit-identical to applying
    them one by one in list order, also where windows overlap and castables are mixed."""
    r = rng(40 + dt)
    for rank, aligned in ((1, True), (2, True), (2, False), (3, False), (4, True)):
        d_out = [int(r.randint(6, 14)) for _ in range(rank)]
        if aligned:
            d_out[-1] = 8 * int(r.randint(4, 9))
        touches, blocks = [], []
        for _ in range(int(r.randint(1, 70))):
            dims = []
            for i, do in enumerate(d_out):
                q = 8 if (aligned and i == rank - 1) else 1
                size = q * int(r.randint(1, do // q + 1))
                off_o = q * int(r.randint(0, (do - size) // q + 1))
                off_i = q * int(r.randint(0, 3))
                dims.append((size + off_i + q * int(r.randint(0, 2)), do, off_i, off_o, size))
            castable = [None, "+", "x", "v", "^"][int(r.randint(0, 5 if dt != ea.C64 else 3))]
            touches.append(ea.Touch(dims, castable, dt))
            blocks.append(normal(r, int(np.prod([d[0] for d in dims])), NP[dt], 0.5))
        out0 = normal(r, int(np.prod(d_out)), NP[dt], 0.5)
        want = _apply_sequentially(touches, blocks, out0)
        d_out_t = to_device(out0)
        d_blocks = [to_device(b) for b in blocks]
        km.touch_batch(touches, stream_handle(), d_out_t.data_ptr(), [b.data_ptr() for b in d_blocks])
        assert_bits_equal(to_host(d_out_t, NP[dt]), want, "touch batch rank %d" % rank)


def test_touch_batch_memory_movement_configuration(km):
    """The 64 accumulate touches of 512x512 blocks into a zeroed 4096x4096 f16 matrix as one
    batch, against the sequential oracle."""
    r = rng(41)
    n, b, count = 4096, 512, 64
    touches, blocks = [], []
    for _ in range(count):
        ro, co = int(r.randint(0, n - b + 1)), int(r.randint(0, n - b + 1))
        touches.append(ea.Touch([(b, n, 0, ro, b), (b, n, 0, co, b)], "+", ea.F16))
        blocks.append(normal(r, b * b, np.float16))
    want = _apply_sequentially(touches, blocks, np.zeros(n * n, np.float16))
    d_out = empty_device(n * n, np.float16, 0.0)
    d_blocks = [to_device(x) for x in blocks]
    km.touch_batch(touches, stream_handle(), d_out.data_ptr(), [x.data_ptr() for x in d_blocks])
    assert_bits_equal(to_host(d_out, np.float16), want, "64 accumulate touches, batched")


@pytest.mark.parametrize("dt", [ea.F16, ea.F32, ea.C64])
def test_touch_batch_disjoint_windows_that_share_output_vectors(km, dt):
    """Windows laid side by side with odd widths: neighbours meet inside 16-byte output
    vectors, and being disjoint they run in the same launch.  Each must leave the other's
    elements alone."""
    r = rng(60 + dt)
    rows, cols = 37, 256
    touches, blocks = [], []
    c = 0
    while c < cols:
        w = min(int(r.randint(1, 23)), cols - c)
        h = int(r.randint(1, rows + 1))
        r0 = int(r.randint(0, rows - h + 1))
        oi = int(r.randint(0, 5))
        touches.append(ea.Touch([(h, rows, 0, r0, h), (w + oi + 2, cols, oi, c, w)],
                                [None, "+", "x"][int(r.randint(0, 3))], dt))
        blocks.append(normal(r, h * (w + oi + 2), NP[dt], 0.5))
        c += w
    out0 = normal(r, rows * cols, NP[dt], 0.5)
    want = _apply_sequentially(touches, blocks, out0)
    d_out = to_device(out0)
    d_blocks = [to_device(b) for b in blocks]
    km.touch_batch(touches, stream_handle(), d_out.data_ptr(), [b.data_ptr() for b in d_blocks])
    assert_bits_equal(to_host(d_out, NP[dt]), want, "side-by-side windows")


@pytest.mark.parametrize("dt", [ea.F16, ea.F32])
def test_touch_batch_stacked_partial_sums(km, dt):
    """The fan-in of partial sums: 40 inputs accumulated into the same window, in order."""
    r = rng(70 + dt)
    n, b = 96, 64
    touches = [ea.Touch([(b, n, 0, 16, b), (b, n, 0, 8, b)], None if i == 0 else "+", dt)
               for i in range(40)]
    blocks = [normal(r, b * b, NP[dt]) for _ in touches]
    out0 = normal(r, n * n, NP[dt])
    want = _apply_sequentially(touches, blocks, out0)
    d_out = to_device(out0)
    d_blocks = [to_device(x) for x in blocks]
    km.touch_batch(touches, stream_handle(), d_out.data_ptr(), [x.data_ptr() for x in d_blocks])
    assert_bits_equal(to_host(d_out, NP[dt]), want, "stacked partial sums")


@pytest.mark.parametrize("castable", [None, "+"])
def test_touch_batch_of_one_op_with_aligned_rows(km, castable):
    """Every touch of the batch has the same op and an input whose rows are 16-byte aligned
    (the form the batch kernel specialises on): overlapping windows at odd column offsets,
    more than one launch's worth of touches, in list order (with plain copies the last writer
    of an element wins)."""
    r = rng(91 if castable else 90)
    n, touches, blocks = 520, [], []
    for _ in range(90):
        h, w = int(r.randint(1, 200)), 8 * int(r.randint(1, 30))
        ro, co = int(r.randint(0, n - h + 1)), int(r.randint(0, n - w + 1))
        touches.append(ea.Touch([(h, n, 0, ro, h), (w, n, 0, co, w)], castable, ea.F16))
        blocks.append(normal(r, h * w, np.float16))
    out0 = normal(r, n * n, np.float16)
    want = _apply_sequentially(touches, blocks, out0)
    d_out = to_device(out0)
    d_blocks = [to_device(x) for x in blocks]
    km.touch_batch(touches, stream_handle(), d_out.data_ptr(), [x.data_ptr() for x in d_blocks])
    assert_bits_equal(to_host(d_out, np.float16), want, "one-op batch")


def test_touch_batch_errors(km):
    d = to_device(np.zeros(64, np.float32))
    a = ea.Touch([(4, 8, 0, 0, 4)], None, ea.F32)
    b = ea.Touch([(4, 16, 0, 0, 4)], None, ea.F32)     # another output extent
    with pytest.raises(ea.KmError) as ei:
        km.touch_batch([a, b], 0, d.data_ptr(), [d.data_ptr(), d.data_ptr()])
    assert ei.value.code == -1
    km.touch_batch([], 0, d.data_ptr(), [])


@pytest.mark.parametrize("dt,castable", [(ea.F16, "+"), (ea.F16, None), (ea.F32, "^"), (ea.C64, "+")])
def test_large_touch_whose_window_is_not_vector_aligned(km, dt, castable):
    """Windows of a few million elements at odd offsets (input and output phases differ):
    they run on 16-byte output vectors with element-wise edges; bit-identical to the oracle."""
    r = rng(90 + dt)
    rows, cols = 1500, 2048
    t = ea.Touch([(rows + 3, rows + 8, 2, 5, rows), (cols + 24, cols + 32, 7, 13, cols - 11)],
                 castable, dt)
    blk = normal(r, (rows + 3) * (cols + 24), NP[dt], 0.5)
    out0 = normal(r, (rows + 8) * (cols + 32), NP[dt], 0.5)
    want = _apply_sequentially([t], [blk], out0)
    d_out, d_blk = to_device(out0), to_device(blk)
    km.touch(t, stream_handle(), d_out.data_ptr(), d_blk.data_ptr())
    assert_bits_equal(to_host(d_out, NP[dt]), want, "large unaligned touch")
