"""Generated kernels with 64-bit indices: an einsummable with 2^32 - 1 or more elements in
its output or in an input is compiled with `unsigned long long` index arithmetic
(csrc/codegen.cc, fits32).  These run that variant at 2^32 + 2^20 elements and check it two
ways: on the device against torch's own operators over the same buffers (an independent
restatement: every element), and on the host against the oracle on slices at the start,
across element 2^32 and at the end."""
import numpy as np
import pytest

import einsummable_amd as ea
import oracle
from helpers import assert_close, assert_values_equal, stream_handle

pytestmark = pytest.mark.gpu

ROWS, COLS = (1 << 20) + 256, 4096          # ROWS * COLS = 2^32 + 2^20
N = ROWS * COLS
CHUNK = 1 << 28


@pytest.fixture(scope="module")
def big():
    """8 GiB of seeded f16 values on the device, made chunk by chunk."""
    import torch

    assert N > (1 << 32)
    g = torch.Generator(device="cuda").manual_seed(64)
    x = torch.empty(N, dtype=torch.float16, device="cuda")
    for lo in range(0, N, CHUNK):
        hi = min(lo + CHUNK, N)
        x[lo:hi] = torch.randn(hi - lo, generator=g, device="cuda", dtype=torch.float32).half()
    torch.cuda.synchronize()
    yield x
    del x
    torch.cuda.empty_cache()


def run(km, e, out, inns):
    import torch

    ws = km.build(e)
    assert ws is not None
    assert " idx64" in km.describe(e), km.describe(e)
    d_ws = torch.empty(max(ws, 1), dtype=torch.uint8, device="cuda")
    km(e, stream_handle(), out.data_ptr(), [t.data_ptr() for t in inns],
       (d_ws.data_ptr(), ws) if ws else None)
    torch.cuda.synchronize()


# element ranges checked on the host: the first vectors, both sides of element 2^32, the tail
SLICES = [(0, 4096), ((1 << 32) - 4096, (1 << 32) + 4096), (N - 4096, N)]


def test_elementwise_beyond_2_to_32_elements(km, big):
    import torch

    e = ea.Einsummable([N], [[0]], 1, "ite_<[hole|f16@0,constant{f16|0},constant{f16|0},hole|f16@0]")
    out = torch.full((N,), 7.0, dtype=torch.float16, device="cuda")
    run(km, e, out, [big])
    for lo in range(0, N, CHUNK):
        hi = min(lo + CHUNK, N)
        assert bool((out[lo:hi] == torch.relu(big[lo:hi])).all()), (lo, hi)
    for lo, hi in SLICES:
        x = big[lo:hi].cpu().numpy()
        want = oracle.einsummable([hi - lo], [[0]], 1, e.join, None, [x], oracle.EXACT)
        assert_values_equal(out[lo:hi].cpu().numpy(), want, "relu [%d, %d)" % (lo, hi))
    del out


def test_broadcast_beyond_2_to_32_elements(km, big):
    import torch

    e = ea.Einsummable([ROWS, COLS], [[0, 1], [0]], 2, "+[hole|f16@0,hole|f16@1]")
    g = torch.Generator(device="cuda").manual_seed(65)
    v = torch.randn(ROWS, generator=g, device="cuda", dtype=torch.float32).half()
    out = torch.empty(N, dtype=torch.float16, device="cuda")
    run(km, e, out, [big, v])
    rows_per = CHUNK // COLS
    for r0 in range(0, ROWS, rows_per):
        r1 = min(r0 + rows_per, ROWS)
        want = big[r0 * COLS:r1 * COLS].view(r1 - r0, COLS) + v[r0:r1, None]
        assert bool((out[r0 * COLS:r1 * COLS].view(r1 - r0, COLS) == want).all()), (r0, r1)
    for r0, r1 in [(0, 2), ((1 << 20) - 1, (1 << 20) + 1), (ROWS - 2, ROWS)]:
        x = big[r0 * COLS:r1 * COLS].cpu().numpy()
        want = oracle.einsummable([r1 - r0, COLS], [[0, 1], [0]], 2, e.join, None,
                                  [x, v[r0:r1].cpu().numpy()], oracle.EXACT)
        assert_values_equal(out[r0 * COLS:r1 * COLS].cpu().numpy(), want, "rows %d..%d" % (r0, r1))
    del out


@pytest.mark.parametrize("castable", ["^", "+"])
def test_row_reduction_beyond_2_to_32_elements(km, big, castable):
    import torch

    e = ea.Einsummable([ROWS, COLS], [[0, 1]], 1, "hole|f16@0", castable)
    out = torch.full((ROWS,), 7.0, dtype=torch.float16, device="cuda")
    run(km, e, out, [big])
    x = big.view(ROWS, COLS)
    if castable == "^":
        assert bool((out == x.amax(dim=1)).all())
    else:
        # fp32 sums of 4096 values of N(0, 1) rounded to f16 (|sum| ~ 64, spacing 2^-4):
        # another order of addition moves the sum by far less than one spacing
        want = torch.empty(ROWS, dtype=torch.float32, device="cuda")
        rows_per = CHUNK // COLS
        for r0 in range(0, ROWS, rows_per):
            r1 = min(r0 + rows_per, ROWS)
            want[r0:r1] = x[r0:r1].float().sum(dim=1)
        err = (out.float() - want).abs()
        assert bool((err <= 1e-2 * want.abs().clamp(min=64.0)).all()), float(err.max())
    for r0, r1 in [(0, 4), ((1 << 20) - 2, (1 << 20) + 2), (ROWS - 4, ROWS)]:
        rows = big[r0 * COLS:r1 * COLS].cpu().numpy()
        want = oracle.einsummable([r1 - r0, COLS], [[0, 1]], 1, e.join, castable, [rows], oracle.WIDE)
        got = out[r0:r1].cpu().numpy()
        if castable == "^":
            assert_values_equal(got, want.astype(np.float16), "row max %d..%d" % (r0, r1))
        else:
            assert_close(got, want, ea.F16, what="row sum %d..%d" % (r0, r1))
    del out
