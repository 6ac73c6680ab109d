"""Randomly generated einsummables against the CPU oracle, through the C ABI: every mode
layout the planner can meet (straight, broadcast, permuted, aggregated, contraction-shaped),
every dtype and castable, with extents that are ragged against every tile and vector width.
The reference checks its kernels the same way, random inputs against its interpreter
(exps/cpuexec_kernels.cc:88-318, exps/gpuexec_kernelmanager.cc:60-120)."""
import random

import numpy as np
import pytest

import einsummable_amd as ea
import oracle
from helpers import NP, assert_close, assert_values_equal, normal, oracle_einsummable, rng, run_einsummable

pytestmark = pytest.mark.gpu

DIMS = [1, 2, 3, 4, 5, 7, 8, 9, 16, 17, 24, 31, 32, 33, 40, 64, 65, 96, 130]


def join_for(r, n, dt):
    h = ["hole|%s@%d" % (dt, i) for i in range(n)]
    if n == 1:
        if dt == "c64":
            return r.choice([h[0], "conj[%s]" % h[0]])
        return r.choice([h[0], "*[constant{%s|0.5},%s]" % (dt, h[0]),
                         "+[constant{%s|1},*[%s,%s]]" % (dt, h[0], h[0]),
                         "ite_<[%s,constant{%s|0},constant{%s|0},%s]" % (h[0], dt, dt, h[0])])
    if n == 2:
        if dt == "c64":
            return r.choice(["*[%s,%s]", "+[%s,%s]"]) % (h[0], h[1])
        return r.choice(["*[%s,%s]" % (h[0], h[1]), "+[%s,%s]" % (h[0], h[1]),
                         "ite_>[%s,%s,%s,%s]" % (h[0], h[1], h[0], h[1]),
                         "*[%s,+[%s,constant{%s|-0.25}]]" % (h[0], h[1], dt)])
    return "+[%s,*[%s,%s]]" % tuple(h)


def random_einsummable(r):
    R = r.randint(1, 4)
    out_rank = r.randint(1, R)
    # keep the join space small enough for the oracle's loops
    while True:
        shape = [r.choice(DIMS) for _ in range(R)]
        if int(np.prod(shape)) <= 300000:
            break
    n_inn = r.choice([1, 1, 2, 2, 2, 3])
    kind = r.random()
    inns = []
    for k in range(n_inn):
        if kind < 0.35 and n_inn == 2 and out_rank < R and out_rank >= 2:
            # contraction-shaped: each input holds the aggregated modes and part of the output
            part = [m for m in range(out_rank) if (m % 2 == k) or r.random() < 0.2]
            modes = part + list(range(out_rank, R))
        else:
            modes = [m for m in range(R) if r.random() < 0.7]
        if not modes:
            modes = [r.randrange(R)]
        r.shuffle(modes)
        inns.append(modes)
    # every mode must appear somewhere (aggregated ones by definition, output ones as a rule
    # of the kernels' callers: a mode nobody reads would be a pure broadcast, allowed too)
    for m in range(out_rank, R):
        if not any(m in i for i in inns):
            inns[r.randrange(n_inn)].append(m)
    dt = r.choice(["f16", "f32", "f32", "f64", "c64"])
    castable = None
    if out_rank < R:
        castable = r.choice(["+", "v", "^", "x"]) if dt != "c64" else "+"
    return ea.Einsummable(shape, inns, out_rank, join_for(r, n_inn, dt), castable), dt


@pytest.mark.parametrize("seed", [100, 101, 102])
def test_random_einsummables_with_every_transposed_input_staged(monkeypatch, seed):
    # elementwise nodes bring inputs with another inner mode into the output's order through
    # the workspace, by themselves only when the input is large: here always
    monkeypatch.setenv("ES_KM_EW_STAGE_MIN", "1")
    test_random_einsummables_match_the_oracle(ea.KernelManager(0), seed)


@pytest.mark.parametrize("seed", range(12))
def test_random_einsummables_match_the_oracle(km, seed):
    r = random.Random(1000 + seed)
    nr = rng(2000 + seed)
    done = 0
    for _ in range(40):
        e, dt = random_einsummable(r)
        _, dts = oracle.scalarop_info(e.join)
        # products of many factors: keep magnitudes near one so that neither side overflows
        sd = 1.0 if e.castable != "x" else 0.05
        xs = []
        for k, d in enumerate(dts):
            x = normal(nr, int(np.prod(e.inn_shape(k))), NP[d], sd)
            if e.castable == "x":
                x = (x + np.asarray(1.0, dtype=x.dtype)).astype(NP[d])
            xs.append(x)
        what = "%s %s out_rank=%d %s %s" % (e.join_shape, e.inns, e.out_rank, e.join, e.castable)
        if km.build(e) is None:
            continue
        got = run_einsummable(km, e, xs)
        od, _ = oracle.scalarop_info(e.join)
        selects_only = e.join.startswith("hole") or e.join.startswith("ite_")
        if selects_only and e.castable in (None, "v", "^"):
            want = oracle_einsummable(e, xs, oracle.EXACT)
            assert_values_equal(got, want, what + " [" + km.describe(e) + "]")
        else:
            want = oracle_einsummable(e, xs, oracle.WIDE)
            assert_close(got, want, od, what=what + " [" + km.describe(e) + "]")
        done += 1
    assert done >= 30
