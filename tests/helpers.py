"""Shared plumbing of the parity tests: device buffers through torch (memory and streams
only), calls through the C ABI, comparisons against the CPU oracle."""
import numpy as np

import einsummable_amd as ea
import oracle

NP = {ea.F16: np.float16, ea.F32: np.float32, ea.F64: np.float64, ea.C64: np.complex64}
ES = {np.dtype(v): k for k, v in NP.items()}

# tolerances of the parity contract: f32 relative 1e-4, f16 relative 1e-2 (against the
# result computed in higher precision), with an absolute floor for outputs near zero.
RTOL = {ea.F16: 1e-2, ea.F32: 1e-4, ea.F64: 1e-10, ea.C64: 1e-4}


def rng(seed):
    # MT19937, the generator family the reference seeds (src/base/setup.cc:28-38)
    return np.random.RandomState(seed)


def uniform(r, shape, dtype, lo=-1.0, hi=1.0):
    if np.dtype(dtype) == np.complex64:
        return (r.uniform(lo, hi, shape) + 1j * r.uniform(lo, hi, shape)).astype(np.complex64)
    return r.uniform(lo, hi, shape).astype(dtype)


def normal(r, shape, dtype, sd=1.0):
    if np.dtype(dtype) == np.complex64:
        return (r.normal(0, sd, shape) + 1j * r.normal(0, sd, shape)).astype(np.complex64)
    return r.normal(0, sd, shape).astype(dtype)


def to_device(a):
    import torch

    a = np.ascontiguousarray(a)
    if a.dtype == np.complex64:
        return torch.view_as_complex(torch.from_numpy(a.view(np.float32).reshape(-1, 2)).cuda())
    return torch.from_numpy(a.reshape(-1)).cuda()


def to_host(t, np_dtype):
    import torch

    if np.dtype(np_dtype) == np.complex64:
        return torch.view_as_real(t).cpu().numpy().view(np.complex64).reshape(-1)
    return t.cpu().numpy().reshape(-1)


def empty_device(n, np_dtype, fill=None):
    import torch

    tdt = {
        np.dtype(np.float16): torch.float16,
        np.dtype(np.float32): torch.float32,
        np.dtype(np.float64): torch.float64,
        np.dtype(np.complex64): torch.complex64,
    }[np.dtype(np_dtype)]
    t = torch.empty(n, dtype=tdt, device="cuda")
    if fill is not None:
        t.fill_(fill)
    return t


def stream_handle():
    import torch

    return torch.cuda.current_stream().cuda_stream


def run_einsummable(km, e, inputs, check_build=True):
    """Build + execute through the C ABI; returns the flat output as numpy."""
    import torch

    ws = km.build(e)
    assert ws is not None, "build returned unsupported for %s %s" % (e.join_shape, e.join)
    od, _ = oracle.scalarop_info(e.join)
    d_in = [to_device(x) for x in inputs]
    d_out = empty_device(e.out_nelem(), NP[od])
    d_ws = torch.empty(max(ws, 1), dtype=torch.uint8, device="cuda")
    km(e, stream_handle(), d_out.data_ptr(), [t.data_ptr() for t in d_in],
       (d_ws.data_ptr(), ws) if ws else None)
    torch.cuda.synchronize()
    return to_host(d_out, NP[od])


def oracle_einsummable(e, inputs, mode=oracle.WIDE):
    return oracle.einsummable(e.join_shape, e.inns, e.out_rank, e.join, e.castable, inputs, mode)


def assert_close(got, want, es_dtype, scale=None, what=""):
    """|got - want| <= rtol * max(|want|, floor) elementwise.  `floor` defaults to the
    root-mean-square magnitude of `want` (sums of many terms are compared against the
    magnitude of the result, not of the cancellations inside it)."""
    got = np.asarray(got).astype(np.complex128 if es_dtype == ea.C64 else np.float64)
    want = np.asarray(want).astype(got.dtype)
    assert got.shape == want.shape, (got.shape, want.shape)
    both_nan = np.isnan(got) & np.isnan(want)
    both_inf = np.isinf(want) & (got == want)
    fine = both_nan | both_inf
    finite = np.isfinite(want) & ~fine
    if scale is None:
        mag = np.abs(want[finite])
        scale = float(np.sqrt(np.mean(mag * mag))) if mag.size else 1.0
        scale = max(scale, 1e-30)
    with np.errstate(invalid="ignore"):   # inf - inf where both sides overflowed alike
        err = np.abs(got - want)
    bound = RTOL[es_dtype] * np.maximum(np.abs(want), scale)
    # an infinite (or NaN) expectation is only met by that very value: `err <= bound` would
    # read inf <= inf there and accept anything
    bad = ~fine & (~np.isfinite(want) | ~(err <= bound))
    if bad.any():
        i = int(np.argmax(np.where(bad, err, 0)))
        raise AssertionError(
            "%s: %d of %d elements outside tolerance; worst at %d: got %r want %r (bound %g)"
            % (what, int(bad.sum()), got.size, i, got[i], want[i], float(bound[i]))
        )


def assert_bits_equal(got, want, what=""):
    got = np.ascontiguousarray(got)
    want = np.ascontiguousarray(want)
    assert got.dtype == want.dtype and got.shape == want.shape, (got.dtype, want.dtype)
    a = got.view(np.uint8)
    b = want.view(np.uint8)
    if not np.array_equal(a, b):
        isz = got.dtype.itemsize
        idx = np.nonzero((a.reshape(-1, isz) != b.reshape(-1, isz)).any(axis=1))[0]
        raise AssertionError(
            "%s: %d of %d elements differ bitwise; first at %d: got %r want %r"
            % (what, idx.size, got.size, idx[0], got.reshape(-1)[idx[0]], want.reshape(-1)[idx[0]])
        )


def assert_values_equal(got, want, what=""):
    """Exact equality of values: bitwise, except that +0 and -0 compare equal and any NaN
    matches any NaN.  Used for computed results whose single rounding is fully determined
    (the GPU compiler may fuse a multiply into an fma with a +0 addend, which only changes
    the sign of a zero result)."""
    got = np.ascontiguousarray(got)
    want = np.ascontiguousarray(want)
    assert got.dtype == want.dtype and got.shape == want.shape, (got.dtype, want.dtype)
    g = got.view(np.float32) if got.dtype == np.complex64 else got
    w = want.view(np.float32) if want.dtype == np.complex64 else want
    same = (g == w) | (np.isnan(g) & np.isnan(w))
    if not same.all():
        idx = np.nonzero(~same)[0]
        raise AssertionError(
            "%s: %d of %d values differ; first at %d: got %r want %r"
            % (what, idx.size, g.size, idx[0], g[idx[0]], w[idx[0]])
        )
