"""The reference's own cases, literally: the einsummables its kernel-manager harness runs
(exps/gpuexec_kernelmanager.cc:18-3443, `kernelNN`: join shape, inns, out rank, join and
castable as written there, at the harness's sizes) and the joins its GPU manager tells apart
by text (src/engine/gpu/gpu_kernel_manager.cc:180-470: custom kernels 1-5, the
large-workspace forms 1, 2 and 4, the two softmax-v3 forms with the folded
`constant{f32|0.0883883}`, the special max / sum reductions).  Each one through the C ABI
against the oracle; tolerance f32 1e-4, f16 1e-2 (the harness itself only asks for
`is_close`'s 0.03)."""
import numpy as np
import pytest

import einsummable_amd as ea
import oracle
from helpers import NP, assert_bits_equal, assert_close, oracle_einsummable, rng, run_einsummable, uniform

pytestmark = pytest.mark.gpu

E = ea.Einsummable
DT = {"f16": ea.F16, "f32": ea.F32, "f64": ea.F64, "c64": ea.C64}


def mul(dt):
    return "*[hole|%s@0,hole|%s@1]" % (dt, dt)


SILU16 = "*[hole|f16@0,power{-1}[+[constant{f16|1},exp[*[constant{f16|-1},hole|f16@0]]]]]"

# (name, join_shape, inns, out_rank, join, castable, line in exps/gpuexec_kernelmanager.cc)
KERNELS = []
for dt in ("f16", "f32", "f64"):
    KERNELS += [
        ("kernel23 " + dt, [147], [[0], [0]], 1, mul(dt), "+", 41),
        ("kernel27 " + dt, [88], [[0], [0]], 1, mul(dt), "+", 182),
        ("kernel9 " + dt, [4, 16, 16], [[0, 2], [1, 2]], 2, mul(dt), "+", 432),
        ("kernel24 " + dt, [4, 16, 64], [[0, 2], [1, 2]], 2, mul(dt), "+", 572),
        ("kernel28 " + dt, [4, 128, 16], [[0, 2], [1, 2]], 2, mul(dt), "+", 710),
        ("kernel29 " + dt, [4, 32, 64], [[0, 2], [1, 2]], 2, mul(dt), "+", 848),
        ("kernel11 " + dt, [4, 16, 8, 8, 16], [[0, 2, 1, 4], [0, 3, 1, 4]], 4, mul(dt), "+", 993),
        ("kernel21 " + dt, [4, 16, 8, 16, 8], [[0, 1, 2, 4], [0, 4, 1, 3]], 4, mul(dt), "+", 1133),
        ("kernel22 " + dt, [2, 4, 8, 4, 4], [[0, 3, 1, 4], [2, 3, 4]], 3, mul(dt), "+", 1274),
        ("kernel15 " + dt, [128, 4], [[0, 1]], 1, "hole|%s@0" % dt, "+", 1399),
        ("kernel3 " + dt, [32, 256], [[0, 1]], 1, "hole|%s@0" % dt, "+", 1571),
        ("kernel2 " + dt, [32], [[0]], 1, "power{2}[hole|%s@0]" % dt, "+", 1656),
        ("kernel5 " + dt, [32], [[0]], 1, "power{-0.5}[hole|%s@0]" % dt, "+", 1718),
        ("kernel13 " + dt, [8, 4], [[0, 1], [1]], 2, "+[hole|%s@0,hole|%s@1]" % (dt, dt), "+", 2040),
    ]
for src, dst, n, name in (("f16", "f32", 8192, "kernel1"), ("f32", "f16", 8192, "kernel7"),
                          ("f32", "f64", 512, "kernel14"), ("f64", "f32", 512, "kernel20")):
    KERNELS.append(("%s %s->%s" % (name, src, dst), [n], [[0]], 1,
                    "to_%s[hole|%s@0]" % (dst, src), "+", 1780))
KERNELS += [
    ("kernel10 c64", [2, 4, 4, 2], [[0, 1, 2, 3], [1, 3]], 4, "*[hole|c64@0,hole|c64@1]", "+", 310),
    ("kernel10 f32", [2, 8, 4, 2], [[0, 1, 2, 3], [1, 3]], 4, mul("f32"), "+", 323),
    ("kernel4", [16], [[0]], 1,
     "+[*[constant{f32|0.000244141},hole|f32@0],constant{f32|1e-06}]", "+", 2127),
    ("kernel19", [128, 4], [[0, 1], [0]], 2, "*[hole|f32@0,power{-1}[hole|f32@1]]", "+", 2191),
    ("kernel26", [16], [[0]], 1, SILU16, "+", 2285),
    ("kernel17", [16], [[0]], 1, "exp[hole|f32@0]", "+", 2352),
    ("kernel12", [16], [[0]], 1, "*[constant{f16|0.0883789},hole|f16@0]", "+", 2418),
    ("kernel6", [32, 256], [[0, 1], [0]], 2, mul("f32"), "+", 2485),
    ("kernel16", [128, 4], [[0, 1], [0]], 2, "+[hole|f32@0,*[constant{f32|-1},hole|f32@1]]", "+", 2582),
    ("kernel8", [128, 4], [[0, 1], [1]], 2, mul("f16"), "+", 2677),
    ("kernel30", [32, 4], [[0, 1], [0, 1], [0]], 1,
     "*[hole|f32@0,*[hole|f32@1,*[constant{f32|-1},power{-2}[hole|f32@2]]]]", "+", 2775),
    ("kernel31", [2, 2], [[0, 1], [0, 1], [0]], 2,
     "*[hole|f32@0,*[hole|f32@1,*[constant{f32|-1},power{-1}[*[hole|f32@2,hole|f32@2]]]]]", None, 2863),
    ("kernel32", [100], [[0]], 1, "power{2}[hole|f32@0]", None, 2959),
    ("kernel33", [256, 32], [[0, 1], [0], [0]], 2,
     "*[*[hole|f32@0,power{-1}[hole|f32@1]],hole|f32@2]", None, 3028),
    ("kernel34", [1, 4, 8, 2, 32], [[0, 3, 1, 4], [3, 4, 2]], 3, mul("f32"), "+", 3131),
    ("kernel35", [32, 4], [[0, 1], [0]], 2, "+[hole|f32@0,*[constant{f32|-1},hole|f32@1]]", None, 3211),
    ("kernel36", [128, 16], [[0, 1]], 1, "hole|f32@0", "+", 3284),
    ("kernel37", [256, 32], [[0, 1], [0], [0]], 2,
     "*[*[hole|f32@0,power{-1}[hole|f32@1]],hole|f32@2]", None, 3354),
]

# (name, join_shape, inns, out_rank, join, castable, line in gpu_kernel_manager.cc)
MANAGER_FORMS = [
    ("custom_kernel1 (silu)", [4096], [[0]], 1, SILU16, None, 189),
    ("custom_kernel2 (is_equal)", [64, 8000], [[0, 1], [0]], 2,
     "ite_==[hole|f32@0,hole|f32@1,constant{f32|1},constant{f32|0}]", None, 202),
    ("custom_kernel3 (sum of negatives) f32", [64, 8000], [[0, 1]], 1,
     "*[constant{f32|-1},hole|f32@0]", "+", 229),
    ("custom_kernel3 (sum of negatives) f16", [64, 8000], [[0, 1]], 1,
     "*[constant{f16|-1},hole|f16@0]", "+", 239),
    ("custom_kernel4 / large_workspace1", [512, 4096], [[0, 1], [0, 1], [0]], 1,
     "*[hole|f32@0,*[hole|f32@1,*[constant{f32|-1},power{-2}[hole|f32@2]]]]", "+", 330),
    ("custom_kernel5", [32768], [[0], [0]], 1,
     "+[*[constant{f32|0.999},hole|f32@0],*[constant{f32|0.000999987},power{2}[hole|f32@1]]]",
     None, 285),
    ("large_workspace2", [512, 4096], [[0, 1], [0], [0]], 2,
     "*[*[hole|f32@0,power{-1}[hole|f32@1]],hole|f32@2]", None, 345),
    ("large_workspace4", [32768], [[0], [0]], 1,
     "+[*[constant{f32|0.5},hole|f32@0],*[constant{f32|-500},hole|f32@1]]", None, 370),
    ("softmax_v3 reduction", [512, 2048], [[0, 1], [0]], 1,
     "exp[*[constant{f32|0.0883883},+[hole|f32@0,*[constant{f32|-1},hole|f32@1]]]]", "+", 377),
    ("softmax_v3 elementwise", [512, 2048], [[0, 1], [0], [0]], 2,
     "*[exp[*[constant{f32|0.0883883},+[hole|f32@0,*[constant{f32|-1},hole|f32@1]]]],"
     "power{-1}[hole|f32@2]]", None, 430),
    ("special max reduction", [512, 2048], [[0, 1]], 1, "hole|f32@0", "^", 441),
    ("special sum reduction", [512, 2048], [[0, 1]], 1, "hole|f32@0", "+", 456),
]


def inputs_for(e, r, name):
    xs = []
    for k in range(len(e.inns)):
        dt = NP[oracle.scalarop_info(e.join)[1][k]]
        n = int(np.prod(e.inn_shape(k)))
        if "power{-" in e.join or "is_equal" in name:
            # divisors and roots away from zero; for the comparison, values that do collide
            x = np.round(r.uniform(1.0, 3.0, n), 0 if "is_equal" in name else 3).astype(dt)
        else:
            x = uniform(r, n, dt)
        xs.append(x)
    return xs


def run_case(km, case, seed):
    name, shape, inns, out_rank, join, castable, _ = case
    e = E(shape, inns, out_rank, join, castable)
    xs = inputs_for(e, rng(seed), name)
    got = run_einsummable(km, e, xs)
    out_dt = oracle.scalarop_info(e.join)[0]
    want = oracle_einsummable(e, xs, oracle.WIDE)
    assert_close(got, want, out_dt, what=name + " | " + km.describe(e))
    return e, xs, got


@pytest.mark.parametrize("case", KERNELS, ids=[c[0].replace(" ", "_") for c in KERNELS])
def test_harness_kernels(km, case):
    e, xs, got = run_case(km, case, 7000 + case[6])
    if case[0].startswith(("kernel1 ", "kernel7 ", "kernel14", "kernel20")):
        # a conversion is one rounding: the bits of the oracle's
        assert_bits_equal(got, oracle_einsummable(e, xs, oracle.EXACT), case[0])


@pytest.mark.parametrize("case", MANAGER_FORMS, ids=[c[0].replace(" ", "_") for c in MANAGER_FORMS])
def test_joins_the_gpu_manager_tells_apart(km, case):
    run_case(km, case, 8000 + case[6])


def test_special_max_reduction_is_exact(km):
    e = E([512, 2048], [[0, 1]], 1, "hole|f16@0", "^")
    xs = [uniform(rng(5), 512 * 2048, np.float16)]
    assert_bits_equal(run_einsummable(km, e, xs), oracle_einsummable(e, xs, oracle.EXACT), "row max")
