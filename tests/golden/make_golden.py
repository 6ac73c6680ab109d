#!/usr/bin/env python3
"""Writes tests/golden/scalarop_golden.json from the reference's own scalarop_t and permute_t
(compiled from the reference tree into oracle/_ref/libes_ref.so by oracle/Makefile).

Run in a container that has the reference tree:   python tests/golden/make_golden.py

The fixture holds inputs and the reference's outputs only: canonical texts written by
operator<<, simplify() results, eval() results as raw bit patterns, SHA-256 digests of
exhaustive f16 tables, and permute outputs of a small iota tensor."""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

assert oracle.ref_available(), "build oracle/_ref first (make -C oracle ref)"

out = {}

# 1. canonical text of the constructors the configurations rely on
out["make"] = {}
for which in ["relu", "silu", "sub", "div", "max", "min", "exp", "square", "inverse_sqrt",
              "sigmoid", "neg", "relu_mul", "exp_sub"]:
    for dt in (oracle.F16, oracle.F32, oracle.F64):
        out["make"]["%s|%s" % (which, oracle.DTYPE_NAMES[dt])] = oracle.ref_scalarop_make(which, dt)

# 2. scalars travel through 6-significant-digit text
out["make_scale"] = []
for dt, v, inc in [(oracle.F16, 1 / np.sqrt(128), False), (oracle.F32, 1 / np.sqrt(128), False),
                   (oracle.F32, 1 / 4096.0, False), (oracle.F32, 1e-6, True),
                   (oracle.F64, np.pi, False), (oracle.F32, 0.001, False)]:
    out["make_scale"].append({"dtype": dt, "value": float(v), "increment": inc,
                              "text": oracle.ref_scalarop_make_scale(dt, float(v), inc)})

# 3. parse -> simplify -> print of hand-written inputs (includes the literals quoted in
#    src/engine/gpu/gpu_kernel_manager.cc and exps/gpuexec_kernelmanager.cc)
SIMPLIFY_INPUTS = [
    "+[*[constant{f32|0.000244141},hole|f32@0],constant{f32|1e-06}]",
    "*[hole|f32@0,power{-1}[hole|f32@1]]",
    "*[*[hole|f32@0,power{-1}[hole|f32@1]],hole|f32@2]",
    "*[hole|f32@0,*[hole|f32@1,*[constant{f32|-1},power{-2}[hole|f32@2]]]]",
    "+[*[constant{f32|0.5},hole|f32@0],*[constant{f32|-500},hole|f32@1]]",
    "ite_>[hole|f32@0,constant{f32|0},hole|f32@0,constant{f32|0}]",
    "ite_>[constant{f32|0},hole|f32@0,constant{f32|0},hole|f32@0]",
    "*[constant{f32|2},constant{f32|3}]",
    "+[hole|f32@1,hole|f32@0]",
    "*[hole|f16@0,constant{f16|0.0883789}]",
    "exp[+[hole|f16@0,*[constant{f16|-1},hole|f16@1]]]",
    "to_f32[hole|f16@0]",
    "*[hole|c64@0,hole|c64@1]",
    "power{2}[hole|f32@0]",
    "+[constant{f32|0},hole|f32@0]",
    "*[constant{f32|1},hole|f32@0]",
]
# joins as they stand right after their variables were replaced by constants (what
# einsummable_t::replace_scalar_variables hands to the scalarop_t constructor), and forms
# that exercise every rule of simplify_once / normalize_order
SIMPLIFY_INPUTS += [
    "*[*[constant{f32|-1},constant{f32|0.25}],hole|f32@0]",
    "+[hole|f32@0,*[*[constant{f32|-1},constant{f32|0.001}],hole|f32@1]]",
    "+[*[constant{f32|0.9},hole|f32@0],*[+[constant{f32|1},*[constant{f32|-1},constant{f32|0.9}]],hole|f32@1]]",
    "*[constant{f32|0.333333},*[constant{f32|0.142857},hole|f32@0]]",
    "*[constant{f16|0.333252},*[constant{f16|0.142822},hole|f16@0]]",
    "*[constant{f64|0.333333},*[constant{f64|0.142857},hole|f64@0]]",
    "*[hole|f32@1,hole|f32@0]",
    "*[hole|f32@0,constant{f32|0}]",
    "+[hole|f32@0,constant{f32|INF}]",
    "+[constant{f32|NINF},hole|f32@0]",
    "power{0}[hole|f32@0]",
    "power{1}[exp[hole|f32@0]]",
    "power{-0.5}[constant{f32|2}]",
    "power{2}[constant{f16|1.5}]",
    "exp[constant{f32|1}]",
    "exp[constant{f16|1}]",
    "log[constant{f64|10}]",
    "to_f16[constant{f32|0.1}]",
    "to_f32[*[constant{f16|0.1},constant{f16|3}]]",
    "ite_<[constant{f32|1},constant{f32|2},hole|f32@0,hole|f32@1]",
    "ite_==[hole|f32@0,hole|f32@0,hole|f32@1,constant{f32|7}]",
    "ite_<[hole|f32@0,hole|f32@1,hole|f32@2,hole|f32@2]",
    "ite_<[hole|f32@1,hole|f32@0,constant{f32|1},constant{f32|0}]",
    "ite_>=[hole|f32@1,hole|f32@0,hole|f32@1,hole|f32@0]",
    "ite_<=[hole|f32@0,constant{f32|0},constant{f32|0},hole|f32@0]",
    "conj[conj[hole|c64@0]]",
    "*[constant{c64|(1,0)},hole|c64@0]",
    "*[constant{c64|(0,1)},constant{c64|(0,1)}]",
    "+[real[hole|c64@0],*[constant{f32|2},constant{f32|0.5}]]",
    "complex[constant{f32|1},constant{f32|2}]",
    "*[+[constant{f32|1},constant{f32|-1}],hole|f32@0]",
    "+[*[constant{f32|1},hole|f32@1],*[hole|f32@0,constant{f32|1}]]",
    "*[hole|f16@0,power{-1}[+[constant{f16|1},exp[*[constant{f16|-1},hole|f16@0]]]]]",
    "exp[*[constant{f32|0.0883883},+[hole|f32@0,*[constant{f32|-1},hole|f32@1]]]]",
]
out["simplify"] = {t: oracle.ref_scalarop_simplify(t) for t in SIMPLIFY_INPUTS}

# 4. eval at sampled points, bit patterns in and out
rs = np.random.RandomState(0)
EVAL_OPS = [
    "+[hole|f16@0,hole|f16@1]", "*[hole|f16@0,hole|f16@1]",
    "+[hole|f32@0,hole|f32@1]", "*[hole|f32@0,hole|f32@1]",
    "+[hole|f64@0,hole|f64@1]", "*[hole|f64@0,hole|f64@1]",
    "*[hole|c64@0,hole|c64@1]", "+[hole|c64@0,hole|c64@1]",
    "exp[hole|f32@0]", "log[hole|f32@0]", "power{-0.5}[hole|f32@0]", "power{2}[hole|f32@0]",
    "exp[hole|f64@0]", "power{1.7}[hole|f64@0]",
    "ite_<[hole|f32@0,hole|f32@1,hole|f32@0,hole|f32@1]",
    "ite_>=[constant{f16|0},hole|f16@0,constant{f16|0},hole|f16@0]",
    "to_f16[hole|f32@0]", "to_f16[hole|f64@0]", "to_f32[hole|f64@0]", "to_f64[hole|f16@0]",
    "*[hole|f16@0,power{-1}[+[constant{f16|1},exp[*[constant{f16|-1},hole|f16@0]]]]]",
    "+[*[constant{f32|0.000244141},hole|f32@0],constant{f32|1e-06}]",
    "*[exp[+[hole|f32@0,*[constant{f32|-1},hole|f32@1]]],power{-1}[hole|f32@2]]",
    "conj[hole|c64@0]", "real[hole|c64@0]", "imag[hole|c64@0]", "complex[hole|f32@0,hole|f32@1]",
]
out["eval"] = []
for text in EVAL_OPS:
    _, holes = oracle.scalarop_info(text)
    rows = []
    for _ in range(48):
        vals = []
        for dt in holes:
            v = rs.normal(0, 2.0)
            if "log" in text or "power{-0.5}" in text or "power{1.7}" in text:
                v = abs(v) + 0.1
            vals.append(complex(v, rs.normal()) if dt == oracle.C64 else v)
        bits = [oracle._to_bits(v, dt) for v, dt in zip(vals, holes)]
        cast = [oracle._from_bits(b, dt) for b, dt in zip(bits, holes)]
        r = oracle.ref_scalarop_eval(text, cast)
        od, _ = oracle.scalarop_info(text)
        rows.append([bits, oracle._to_bits(r, od)])
    out["eval"].append({"op": text, "points": rows})

# 5. exhaustive f16 tables as digests (all 65536 inputs; NaN results canonicalised)
allh = np.arange(65536, dtype=np.uint16)


def digest(u16):
    f = u16.view(np.float16)
    u16 = np.where(np.isnan(f), np.uint16(0x7E00), u16)
    return hashlib.sha256(np.ascontiguousarray(u16).tobytes()).hexdigest()


out["f16_unary_sha256"] = {}
for text in ["exp[hole|f16@0]", "log[hole|f16@0]", "power{-1}[hole|f16@0]", "power{2}[hole|f16@0]",
             "power{-0.5}[hole|f16@0]", "power{0.5}[hole|f16@0]", "power{0.3}[hole|f16@0]",
             "*[constant{f16|0.0883789},hole|f16@0]",
             "*[hole|f16@0,power{-1}[+[constant{f16|1},exp[*[constant{f16|-1},hole|f16@0]]]]]"]:
    out["f16_unary_sha256"][text] = digest(oracle.ref_scalarop_map_f16(text, allh))
xs = rs.randint(0, 65536, 1 << 20).astype(np.uint16)
ys = rs.randint(0, 65536, 1 << 20).astype(np.uint16)
out["f16_binary_seed0_sha256"] = {
    text: digest(oracle.ref_scalarop_map_f16(text, xs, ys))
    for text in ["+[hole|f16@0,hole|f16@1]", "*[hole|f16@0,hole|f16@1]"]
}

# 6. permute_t on a 3x4x5x6 iota tensor, every permutation (exps/cpuexec_permute.cc:33-77)
import itertools  # noqa: E402

t = np.arange(3 * 4 * 5 * 6, dtype=np.float32).reshape(3, 4, 5, 6)
out["permute_3x4x5x6_sha256"] = {}
for perm in itertools.permutations(range(4)):
    r = oracle.ref_permute(t, perm)
    out["permute_3x4x5x6_sha256"]["".join(map(str, perm))] = hashlib.sha256(
        np.ascontiguousarray(r).tobytes()).hexdigest()

path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "scalarop_golden.json")
with open(path, "w") as f:
    json.dump(out, f, indent=1, sort_keys=True)
print("wrote", path, os.path.getsize(path), "bytes")
