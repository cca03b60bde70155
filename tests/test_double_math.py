"""The base-2 exponential and logarithm that float64 kernels carry with them, checked on the CPU:
their text is cut out of a generated kernel, compiled as plain C and compared with libm."""
import ctypes
import os
import re
import subprocess

import numpy as np

from conftest import compile_spn
from test_packed_rows_host import ASM, _statement


def _routines(native, tmp_path, marginal=False):
    from spnc import synthetic as syn
    k = compile_spn(native, syn.c2_spn(), "float32", marginal=marginal, **{"hip-compute-type": "float64"})
    src = k.source()
    os.remove(k.fileName())
    assert src.count("spn_exp2(") > 200 and src.count("spn_log2(") > 70 and "spn_exp(" not in src and "spn_log(" not in src
    parts = ["#define SPN_EXP2_TABLE spn_exp2_table\n#define SPN_LOG2_TABLE spn_log2_table\n#define SPN_POLY spn_poly\n"]
    for name in ("spn_exp2_table", "spn_log2_table", "spn_poly"):   # the kernel copies these into LDS; on the CPU they are read where they are
        m = re.search(r"__device__ const (?:real_t|unsigned long long) " + name + r"\[\d+\] = \{.*?\};\n", src, re.S)
        assert m, name
        parts.append(m.group(0).replace("__device__ ", "static "))
    for name in ("spn_exp2", "spn_log2"):
        m = re.search(r"static __device__ \S+ real_t " + name + r"\(real_t x\) \{.*?\n\}\n", src, re.S)
        assert m, name
        parts.append(ASM.sub(_statement, re.sub(r"static __device__ \S+ ", "", m.group(0))))   # assembler statements as the C they stand for
    c = tmp_path / ("m%d.c" % marginal)
    c.write_text("typedef double real_t;\ntypedef _Bool bool;\n" + "".join(parts))
    so = tmp_path / ("m%d.so" % marginal)
    subprocess.check_call(["gcc", "-O2", "-shared", "-fPIC", "-ffp-contract=off", "-o", str(so), str(c), "-lm"])
    lib = ctypes.CDLL(str(so))
    for f in (lib.spn_exp2, lib.spn_log2):
        f.restype, f.argtypes = ctypes.c_double, [ctypes.c_double]
    return lib


import pytest


@pytest.mark.parametrize("marginal", [False, True])
def test_double_exp2_log2_against_libm(native, tmp_path, marginal):
    """Kernels with marginalisation handle missing (NaN) features at the leaves, so their routines guard their ranges
    without keeping NaN; the others pass NaN through."""
    lib = _routines(native, tmp_path, marginal)
    rng = np.random.default_rng(5)
    xs = np.concatenate([rng.uniform(-70, 0, 20000), rng.uniform(-1070, 1000, 4000), [0.0, -0.5, 0.5, -1.0, -1022.0]])
    got = np.array([lib.spn_exp2(float(x)) for x in xs])
    want = np.exp2(xs)
    normal = want > 1e-300
    # the polynomial stops at the fourth power of the remainder (at most 1/128): 4e-14 of the result, against 1e-10 that results are held to
    assert np.max(np.abs(got[normal] - want[normal]) / want[normal]) < 5e-14
    assert np.all(got[~normal] <= 1e-299)
    assert lib.spn_exp2(float("-inf")) == 0.0 and lib.spn_exp2(-5000.0) == 0.0
    assert marginal or np.isnan(lib.spn_exp2(float("nan")))
    ss = np.concatenate([rng.uniform(1, 700, 20000), np.exp2(rng.uniform(-1000, 1000, 4000)), [1.0, 2.0, 0.5, 1.4142135623730951, 0.7071067811865476]])
    got = np.array([lib.spn_log2(float(s)) for s in ss])
    want = np.log2(ss)
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-3)) < 3e-15   # the polynomial stops at the fifth power of u < 1/256: 1e-15
    near = rng.uniform(1.0, 1.001, 5000)            # sums dominated by one term: absolute accuracy matters
    assert max(abs(lib.spn_log2(float(s)) - np.log2(s)) for s in near) < 1e-17 * 50
    assert lib.spn_log2(1.0) == 0.0 and lib.spn_log2(0.0) == float("-inf")
    assert marginal or np.isnan(lib.spn_log2(float("nan")))
