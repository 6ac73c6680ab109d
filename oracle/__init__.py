"""ctypes front-end of the CPU oracle (test infrastructure only).

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package.  It loads ``libes_oracle.so`` (the C restatement of the reference's
apply-node semantics, see ``es_oracle.h``) and, when it has been built, the
reference-backed checker ``_ref/libes_ref.so``.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

F16, F32, F64, C64 = 0, 1, 2, 3
EXACT, WIDE = 0, 1
DTYPE_NAMES = {F16: "f16", F32: "f32", F64: "f64", C64: "c64"}
NP_DTYPES = {F16: np.float16, F32: np.float32, F64: np.float64, C64: np.complex64}
_NP_TO_ES = {np.dtype(v): k for k, v in NP_DTYPES.items()}


def es_dtype(np_dtype):
    return _NP_TO_ES[np.dtype(np_dtype)]


def build(force=False):
    """Compile libes_oracle.so (and oracle/_ref when the reference tree is present)."""
    args = ["make", "-C", _HERE]
    if force:
        args.append("-B")
    subprocess.run(args + ["all"], check=True, capture_output=True)


def _load():
    path = os.path.join(_HERE, "libes_oracle.so")
    if not os.path.exists(path):
        build()
    lib = ctypes.CDLL(path)
    lib.es_oracle_last_error.restype = ctypes.c_char_p
    lib.es_oracle_f64_to_f16.restype = ctypes.c_uint16
    lib.es_oracle_f64_to_f16.argtypes = [ctypes.c_double]
    lib.es_oracle_f16_to_f32.restype = ctypes.c_float
    lib.es_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
    return lib


_lib = _load()


class OracleError(RuntimeError):
    pass


def _check(rc):
    if rc < 0:
        raise OracleError(_lib.es_oracle_last_error().decode())
    return rc


def _u64(xs):
    return (ctypes.c_uint64 * len(xs))(*[int(x) for x in xs])


def _ints(xs):
    return (ctypes.c_int * max(len(xs), 1))(*[int(x) for x in xs])


def _flatten(inns):
    flat, offs = [], [0]
    for inn in inns:
        flat.extend(inn)
        offs.append(len(flat))
    return flat, offs


def _castable_char(castable):
    return ctypes.c_char(castable.encode() if castable else b"\0")


def f64_to_f16_bits(v):
    return _lib.es_oracle_f64_to_f16(float(v))


def scalarop_roundtrip(text):
    buf = ctypes.create_string_buffer(8192)
    _check(_lib.es_oracle_scalarop_roundtrip(text.encode(), buf, ctypes.c_size_t(8192)))
    return buf.value.decode()


def scalarop_info(text):
    """(out_dtype, [hole dtypes])"""
    od, n = ctypes.c_int(), ctypes.c_int()
    dts = (ctypes.c_int * 16)()
    _check(_lib.es_oracle_scalarop_info(text.encode(), ctypes.byref(od), ctypes.byref(n), dts, 16))
    return od.value, [dts[i] for i in range(n.value)]


def _to_bits(x, dt):
    a = np.array([x], dtype=NP_DTYPES[dt])
    raw = a.tobytes() + b"\0" * 8
    return int.from_bytes(raw[:8], "little")


def _from_bits(bits, dt):
    raw = int(bits).to_bytes(8, "little")
    return np.frombuffer(raw[: np.dtype(NP_DTYPES[dt]).itemsize], dtype=NP_DTYPES[dt])[0]


def scalarop_eval(text, inputs, mode=EXACT):
    """Evaluate at one point; inputs are python/numpy scalars (cast to each hole's dtype)."""
    _, hole_dts = scalarop_info(text)
    bits = [_to_bits(x, dt if dt >= 0 else F32) for x, dt in zip(inputs, hole_dts)]
    out, od = ctypes.c_uint64(), ctypes.c_int()
    _check(
        _lib.es_oracle_scalarop_eval(
            text.encode(), len(bits), _u64(bits), mode, ctypes.byref(out), ctypes.byref(od)
        )
    )
    return _from_bits(out.value, od.value)


def scalarop_map(text, inputs, mode=EXACT):
    od, hole_dts = scalarop_info(text)
    arrs = [np.ascontiguousarray(x, dtype=NP_DTYPES[dt]) for x, dt in zip(inputs, hole_dts)]
    n = arrs[0].size
    out = np.empty(n, dtype=NP_DTYPES[od])
    ptrs = (ctypes.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])
    _check(
        _lib.es_oracle_scalarop_map(
            text.encode(), len(arrs), ptrs, ctypes.c_uint64(n), mode, ctypes.c_void_p(out.ctypes.data)
        )
    )
    return out


def einsummable(join_shape, inns, out_rank, join, castable, inputs, mode=EXACT):
    """Run the interpreter; returns a flat array of the join's output dtype."""
    od, hole_dts = scalarop_info(join)
    arrs = [np.ascontiguousarray(x, dtype=NP_DTYPES[dt]) for x, dt in zip(inputs, hole_dts)]
    # aggregated modes are renumbered by first appearance (einsummable.cc:32-93); sizes
    # follow join_shape under the new numbers, and every input must hold exactly that many
    renamed = {}
    for a, inn in zip(arrs, inns):
        n = 1
        for m in inn:
            if m >= out_rank:
                m = renamed.setdefault(m, out_rank + len(renamed))
            if 0 <= m < len(join_shape):
                n *= int(join_shape[m])
        if a.size != n:
            raise ValueError("input of %d elements where modes %s of %s need %d"
                             % (a.size, list(inn), list(join_shape), n))
    flat, offs = _flatten(inns)
    n_out = int(np.prod([join_shape[i] for i in range(out_rank)], dtype=np.int64))
    out = np.empty(n_out, dtype=NP_DTYPES[od])
    ptrs = (ctypes.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])
    _check(
        _lib.es_oracle_einsummable(
            _u64(join_shape), len(join_shape), _ints(flat), _ints(offs), len(inns), out_rank,
            join.encode(), _castable_char(castable), mode, ctypes.c_void_p(out.ctypes.data), ptrs,
        )
    )
    return out


def merge_adjacent_dims(join_shape, inns, out_rank):
    flat, offs = _flatten(inns)
    njs = (ctypes.c_uint64 * len(join_shape))()
    nflat = (ctypes.c_int * max(len(flat), 1))()
    noffs = (ctypes.c_int * (len(inns) + 1))()
    nor = ctypes.c_int()
    r = _check(
        _lib.es_oracle_merge_adjacent_dims(
            _u64(join_shape), len(join_shape), _ints(flat), _ints(offs), len(inns), out_rank,
            njs, nflat, noffs, ctypes.byref(nor),
        )
    )
    new_inns = [[nflat[i] for i in range(noffs[k], noffs[k + 1])] for k in range(len(inns))]
    return [int(njs[i]) for i in range(r)], new_inns, nor.value


def einsummable_str(inns, out_rank):
    flat, offs = _flatten(inns)
    buf = ctypes.create_string_buffer(256)
    _check(_lib.es_oracle_einsummable_str(_ints(flat), _ints(offs), len(inns), out_rank, buf,
                                          ctypes.c_size_t(256)))
    return buf.value.decode()


def einsummable_parse(s):
    flat = (ctypes.c_int * 64)()
    offs = (ctypes.c_int * 17)()
    n, orank = ctypes.c_int(), ctypes.c_int()
    _check(_lib.es_oracle_einsummable_parse(s.encode(), flat, offs, ctypes.byref(n),
                                            ctypes.byref(orank), 64))
    return [[flat[i] for i in range(offs[k], offs[k + 1])] for k in range(n.value)], orank.value


def touch(dims, castable, out, inn):
    """dims: list of (d_inn, d_out, offset_inn, offset_out, size); updates `out` in place."""
    assert out.flags["C_CONTIGUOUS"] and inn.flags["C_CONTIGUOUS"] and out.dtype == inn.dtype
    flat = [v for d in dims for v in d]
    _check(
        _lib.es_oracle_touch(
            _u64(flat), len(dims), _castable_char(castable), es_dtype(out.dtype),
            ctypes.c_void_p(out.ctypes.data), ctypes.c_void_p(inn.ctypes.data),
        )
    )
    return out


def touch_simplify(dims):
    flat = [v for d in dims for v in d]
    od = (ctypes.c_uint64 * len(flat))()
    r = ctypes.c_int()
    _check(_lib.es_oracle_touch_simplify(_u64(flat), len(dims), od, ctypes.byref(r)))
    return [tuple(int(od[5 * i + j]) for j in range(5)) for i in range(r.value)]


def fill_constant(np_dtype, value, nelem):
    dt = es_dtype(np_dtype)
    out = np.empty(nelem, dtype=np_dtype)
    _check(_lib.es_oracle_fill_constant(dt, ctypes.c_uint64(_to_bits(value, dt)),
                                        ctypes.c_uint64(nelem), ctypes.c_void_p(out.ctypes.data)))
    return out


def fill_lowertri(np_dtype, lower, upper, nrow, ncol, start):
    dt = es_dtype(np_dtype)
    out = np.empty(nrow * ncol, dtype=np_dtype)
    _check(
        _lib.es_oracle_fill_lowertri(
            dt, ctypes.c_uint64(_to_bits(lower, dt)), ctypes.c_uint64(_to_bits(upper, dt)),
            ctypes.c_uint64(nrow), ctypes.c_uint64(ncol), ctypes.c_int64(start),
            ctypes.c_void_p(out.ctypes.data),
        )
    )
    return out.reshape(nrow, ncol)


# ----------------------------------------------------------------------------------------
# Reference-backed checker (oracle/_ref/libes_ref.so): the reference's own scalarop_t and
# permute_t compiled from the reference tree.  Present only where that tree was available
# at build time; never required by the product.


def ref_available():
    return os.path.exists(os.path.join(_HERE, "_ref", "libes_ref.so"))


_ref = None


def _ref_lib():
    global _ref
    if _ref is None:
        _ref = ctypes.CDLL(os.path.join(_HERE, "_ref", "libes_ref.so"))
        _ref.es_ref_last_error.restype = ctypes.c_char_p
    return _ref


def _ref_check(rc):
    if rc < 0:
        raise OracleError("reference: " + _ref_lib().es_ref_last_error().decode())
    return rc


def ref_scalarop_roundtrip(text):
    buf = ctypes.create_string_buffer(8192)
    _ref_check(_ref_lib().es_ref_scalarop_roundtrip(text.encode(), buf, ctypes.c_size_t(8192)))
    return buf.value.decode()


def ref_scalarop_simplify(text):
    buf = ctypes.create_string_buffer(8192)
    _ref_check(_ref_lib().es_ref_scalarop_simplify(text.encode(), buf, ctypes.c_size_t(8192)))
    return buf.value.decode()


def ref_scalarop_make(which, dt):
    buf = ctypes.create_string_buffer(8192)
    _ref_check(_ref_lib().es_ref_scalarop_make(which.encode(), dt, buf, ctypes.c_size_t(8192)))
    return buf.value.decode()


def ref_scalarop_make_scale(dt, value, increment=False):
    buf = ctypes.create_string_buffer(8192)
    _ref_check(_ref_lib().es_ref_scalarop_make_scale(dt, ctypes.c_double(value), int(increment),
                                                     buf, ctypes.c_size_t(8192)))
    return buf.value.decode()


def ref_scalarop_eval(text, inputs):
    _, hole_dts = scalarop_info(text)
    bits = [_to_bits(x, dt if dt >= 0 else F32) for x, dt in zip(inputs, hole_dts)]
    out, od = ctypes.c_uint64(), ctypes.c_int()
    _ref_check(_ref_lib().es_ref_scalarop_eval(text.encode(), len(bits), _u64(bits),
                                               ctypes.byref(out), ctypes.byref(od)))
    return _from_bits(out.value, od.value)


def ref_scalarop_map_f16(text, x, y=None):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty_like(x)
    if y is None:
        _ref_check(_ref_lib().es_ref_scalarop_map_f16_unary(
            text.encode(), ctypes.c_void_p(x.ctypes.data), ctypes.c_uint64(x.size),
            ctypes.c_void_p(out.ctypes.data)))
    else:
        y = np.ascontiguousarray(y, dtype=np.uint16)
        _ref_check(_ref_lib().es_ref_scalarop_map_f16_binary(
            text.encode(), ctypes.c_void_p(x.ctypes.data), ctypes.c_void_p(y.ctypes.data),
            ctypes.c_uint64(x.size), ctypes.c_void_p(out.ctypes.data)))
    return out


def ref_permute(inn, out_perm):
    """inn: numpy array; out_perm = (2,0,1) means ijk->kij (permute_t's convention)."""
    inn = np.ascontiguousarray(inn)
    out = np.empty(inn.size, dtype=inn.dtype)
    _ref_check(_ref_lib().es_ref_permute(
        _u64(inn.shape), inn.ndim, _ints(out_perm), inn.dtype.itemsize,
        ctypes.c_void_p(out.ctypes.data), ctypes.c_void_p(inn.ctypes.data)))
    return out.reshape([inn.shape[p] for p in out_perm])


# ---- optimised CPU loops for the reported CPU baseline (es_cpu_loops.c); benchmark
# infrastructure like the rest of this package

_loops = None


def cpu_loops():
    """The -O3 / AVX2 / OpenMP loops library (built on demand)."""
    global _loops
    if _loops is None:
        path = os.path.join(_HERE, "libes_cpu_loops.so")
        if not os.path.exists(path):
            subprocess.run(["make", "-C", _HERE, "libes_cpu_loops.so"], check=True,
                           capture_output=True)
        lib = ctypes.CDLL(path)
        P, Z, I = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
        lib.es_cpu_max_threads.restype = I
        lib.es_cpu_relu_mul_f16.argtypes = [P, P, P, Z, I]
        lib.es_cpu_rowmax_f16.argtypes = [P, P, Z, Z, I]
        lib.es_cpu_exp_sub_f16.argtypes = [P, P, P, Z, Z, I]
        lib.es_cpu_rowsum_f16.argtypes = [P, P, Z, Z, I]
        lib.es_cpu_permute_acbd_2byte.argtypes = [P, P, Z, Z, Z, Z, I]
        lib.es_cpu_touch_add_f16.argtypes = [P, Z, P, Z, Z, Z, Z, I]
        _loops = lib
    return _loops


def _p(a):
    assert a.flags["C_CONTIGUOUS"]
    return ctypes.c_void_p(a.ctypes.data)


def loops_relu_mul(x, y, threads=0):
    out = np.empty_like(x)
    cpu_loops().es_cpu_relu_mul_f16(_p(x), _p(y), _p(out), x.size, threads)
    return out


def loops_rowmax(x, threads=0):
    out = np.empty(x.shape[0], np.float16)
    cpu_loops().es_cpu_rowmax_f16(_p(x), _p(out), x.shape[0], x.shape[1], threads)
    return out


def loops_exp_sub(x, m, threads=0):
    out = np.empty_like(x)
    cpu_loops().es_cpu_exp_sub_f16(_p(x), _p(m), _p(out), x.shape[0], x.shape[1], threads)
    return out


def loops_rowsum(x, threads=0):
    out = np.empty(x.shape[0], np.float16)
    cpu_loops().es_cpu_rowsum_f16(_p(x), _p(out), x.shape[0], x.shape[1], threads)
    return out


def loops_permute_acbd(x, threads=0):
    a, b, c, d = x.shape
    out = np.empty((a, c, b, d), x.dtype)
    cpu_loops().es_cpu_permute_acbd_2byte(_p(x), _p(out), a, b, c, d, threads)
    return out


def loops_touch_add(out, inn, ro, co, threads=0):
    cpu_loops().es_cpu_touch_add_f16(_p(out), out.shape[1], _p(inn), inn.shape[0], inn.shape[1],
                                     ro, co, threads)
    return out
