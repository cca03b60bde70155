"""Generated straight-line kernels run on the CPU: the evaluation function of every kernel (of every task, for graphs cut
by maxTaskSize) is cut out of the generated source, compiled for the host and driven sample by sample, with the
intermediate buffer between tasks laid out as on the device ([rows][samples]). Checks code generation and the
partitioner against the oracle and the reference's expected outputs without a GPU."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from conftest import GOLDEN, compile_query, compile_spn, load_golden, model_as_query, oracle_model
from oracle import evaluate as ev
from test_packed_rows_host import ASM, CLANG, _statement, lane_constants_on_the_host, needs_clang

PRELUDE = """#include <cmath>
#define __device__
#define __forceinline__ inline
#define __restrict__
static inline float __builtin_amdgcn_exp2f(float x) { return exp2f(x); }
static inline float __builtin_amdgcn_logf(float x) { return log2f(x); }
"""
TABLES = "#define SPN_EXP2_TABLE spn_exp2_table\n#define SPN_LOG2_TABLE spn_log2_table\n#define SPN_POLY spn_poly\n#define SPN_CTAB spn_ctab\n"


def _host_part(text, name, task):
    """Everything of one kernel's source before the kernel itself, plus a loop over samples around its evaluation function."""
    body = text[:text.index('extern "C" __global__')]
    body = lane_constants_on_the_host(ASM.sub(_statement, body)).replace("__builtin_amdgcn_sched_barrier(0);", "")
    body = body.replace("__device__ __attribute__((aligned(32))) const real_t spn_tables", "alignas(32) const real_t spn_tables")
    assert "asm" not in body
    tab = "spn_tables" if "spn_tables[SPN_NTAB]" in body else "nullptr"
    by_row = "spn_eval(const feat_t* __restrict__ row" in body
    final = "__builtin_nontemporal_store(value, out + i)" in text or not task
    args = "in + i * SPN_F, " + tab if by_row else "x, " + tab
    if task:
        args += ", ext + i, res + i, (unsigned long long)n"
    load = "" if by_row else "feat_t x[SPN_F]; spn_load_row(in, i, x);"
    return body + """
extern "C" void %s(const feat_t* in, real_t* out, long n, const real_t* ext, real_t* res) {
  for (long i = 0; i < n; ++i) {
    %s
    const real_t value = spn_eval(%s);
    %s
  }
}
""" % (name, load, args, "out[i] = value;" if final else "(void)value;")


def host_kernel(source, info, tmp_path):
    """-> function(X) that evaluates the kernel (all its tasks, one after the other) on the host."""
    tasks = info["num_tasks"]
    if tasks == 1:
        text = PRELUDE + TABLES + _host_part(source, "task0", False)
    else:
        text = PRELUDE
        parts = re.split(r"// task \d+ of \d+:[^\n]*\n", source)[1:]
        assert len(parts) == tasks
        for t, part in enumerate(parts):
            scope, rest = part.split("{\n", 1)
            inner = rest[:rest.rindex("}  // task")]
            text += TABLES + scope + "{\n" + _host_part(inner, "task%d" % t, True) + "}\n" + "".join(
                "#undef %s\n" % m for m in ("SPN_LOAD", "SPN_LOAD_TILE", "SPN_F", "SPN_BLOCK", "SPN_U", "SPN_NTAB", "SPN_DOUBLE_TABLES",
                                            "SPN_EXP2_TABLE", "SPN_LOG2_TABLE", "SPN_POLY", "SPN_NCTAB", "SPN_CTAB"))
    cpp, so = tmp_path / "k.cpp", tmp_path / "k.so"
    cpp.write_text(text)
    subprocess.check_call([CLANG, "-O1", "-shared", "-fPIC", "-std=c++17", "-ffp-contract=fast", "-w", "-o", str(so), str(cpp)])
    lib = ctypes.CDLL(str(so))
    real = np.float64 if info["dtype"] == "float64" else np.float32

    def run(X):
        X = np.ascontiguousarray(X)
        n = X.shape[0]
        out = np.zeros(n, real)
        inter = np.full((max(1, info["task_rows"]), n), np.nan, real)   # a row read before it is written shows as NaN
        for t in range(tasks):
            getattr(lib, "task%d" % t)(X.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(n),
                                       inter.ctypes.data_as(ctypes.c_void_p), inter.ctypes.data_as(ctypes.c_void_p))
        return out
    return run


def _partition_example():
    from spnc.structure import Histogram, Product, Sum
    h1 = Histogram([0., 1., 2.], [0.25, 0.75], [1, 1], scope=0)
    h2 = Histogram([0., 1., 2.], [0.45, 0.55], [1, 1], scope=1)
    h3 = Histogram([0., 1., 2.], [0.33, 0.67], [1, 1], scope=0)
    h4 = Histogram([0., 1., 2.], [0.875, 0.125], [1, 1], scope=1)
    return Sum([0.3, 0.7], [Product(children=[h1, h2]), Product(children=[h3, h4])])


@needs_clang
@pytest.mark.parametrize("opts", [{}, {"hip-compute-type": "float64"}, {"use-log-space": "false"}], ids=["log-f32", "log-f64", "linear-f64"])
@pytest.mark.parametrize("size", [0, 1, 2, 5])
def test_reference_partitioning_example_on_the_host(native, tmp_path, opts, size):
    """The SPN of the reference's partitioning tests (python-interface/test/vector/test_log_vector_graph_partitioning.py:22-42),
    uncut and cut at 1, 2 and 5 operations."""
    rng = np.random.default_rng(30)
    X = np.column_stack((rng.integers(0, 2, 30), rng.integers(0, 2, 30))).astype("float64")
    spn = _partition_example()
    k = compile_spn(native, spn, "float64", marginal=False, **dict(opts, **({"maxTaskSize": size} if size else {})))
    info, src = k.info(), k.source()
    os.remove(k.fileName())
    assert (info["num_tasks"] > 1) == (size > 0)
    got = host_kernel(src, info, tmp_path)(X)
    ref = ev.ll_closed_f64(oracle_model(spn, "float64"), X, marginal=False)
    assert np.abs(got - ref).max() <= (1e-4 if got.dtype == np.float32 else 1e-10)


@needs_clang
@pytest.mark.parametrize("name,opts", [("NIPS5", {"use-log-space": "false"}), ("NIPS5", {"use-log-space": "false", "maxTaskSize": 3}),
                                        ("NIPS5", {"use-log-space": "false", "maxTaskSize": 10}), ("NIPS5", {"maxTaskSize": 7}),
                                        ("plants", {"maxTaskSize": 64, "hip-kernel": "jit"}), ("plants", {"maxTaskSize": 400, "hip-compute-type": "float64", "hip-kernel": "jit"})],
                         ids=["nips5-linear", "nips5-linear-3", "nips5-linear-10", "nips5-log-7", "plants-64", "plants-400-f64"])
def test_golden_models_on_the_host(native, tmp_path, name, opts):
    """The reference's expected outputs (NIPS5 as in test_partitioned_cuda_NIPS5.py:34 and test_partitioned_vector_NIPS5.py:35)
    from the generated code of whole and cut graphs."""
    X, ref = load_golden(name)
    if name == "NIPS5":
        path, X = os.path.join(GOLDEN, "NIPS5.bin"), X.astype(np.uint32)
    else:
        path, X, ref = model_as_query(os.path.join(GOLDEN, name + ".bin"), "float64", str(tmp_path / "q.bin")), X[:400], ref[:400]
    k = compile_query(native, path, **opts)
    info, src = k.info(), k.source()
    os.remove(k.fileName())
    assert info["kernel_kind"] == 1 and (info["num_tasks"] > 1) == ("maxTaskSize" in opts)
    got = host_kernel(src, info, tmp_path)(X)
    assert np.abs(got - ref).max() <= (1e-4 if got.dtype == np.float32 else 1e-10)


@needs_clang
@pytest.mark.parametrize("cfg,opts", [("c1", {}), ("c1", {"maxTaskSize": 3}), ("c2", {"hip-samples-per-lane": 1}), ("c2", {"maxTaskSize": 300}),
                                       ("c5", {}), ("c5", {"hip-compute-type": "float64"}), ("c5", {"hip-compute-type": "float64", "maxTaskSize": 150}),
                                       ("c5", {"hip-compute-type": "float64", "hip-nan-masks": "false"}), ("c3", {"hip-packed-rows": "false", "maxTaskSize": 300}),
                                       ("c5", {"hip-compute-type": "float64", "hip-gauss-expanded": "false"}),
                                       ("c5", {"hip-compute-type": "float64", "hip-lane-constants": "false"}),
                                       ("c5", {"hip-compute-type": "float64", "hip-marginal-tables-kib": 0}),
                                       ("c5", {"hip-compute-type": "float64", "hip-marginal-tables-kib": 3}),
                                       ("c2", {"hip-compute-type": "float64"}), ("c2", {"hip-compute-type": "float64", "hip-lane-constants": "false"}),
                                       ("c5", {"hip-marginal-offsets": "false"}), ("c5", {"maxTaskSize": 150}), ("c5", {"hip-marginal-tables-kib": 1})],
                         ids=["c1", "c1-cut", "c2", "c2-cut", "c5", "c5-f64", "c5-f64-cut", "c5-f64-selects", "c3-cut", "c5-f64-factored",
                              "c5-f64-scalar-constants", "c5-f64-no-pattern-tables", "c5-f64-few-pattern-tables", "c2-f64", "c2-f64-scalar-constants",
                              "c5-selects", "c5-cut", "c5-few-offset-tables"])
def test_benchmark_graphs_on_the_host(native, tmp_path, cfg, opts):
    from spnc import synthetic as syn
    c = syn.CONFIGS[cfg]
    spn, X = c["spn"](), c["inputs"](500)
    k = compile_spn(native, spn, c["dtype"], marginal=c["marginal"], **dict(opts, **{"hip-kernel": "jit"}))
    info, src = k.info(), k.source()
    os.remove(k.fileName())
    got = host_kernel(src, info, tmp_path)(X)
    ref = ev.ll_closed_f64(oracle_model(spn, c["dtype"]), X, marginal=c["marginal"])
    fin = np.isfinite(ref)
    assert np.array_equal(np.isneginf(got), np.isneginf(ref))
    assert np.abs(got[fin] - ref[fin]).max() <= (1e-4 if got.dtype == np.float32 else 1e-10)


def _wide_marginal_products(seed=3):
    """A sum over five products of eleven Gaussian leaves each, some of them narrow and far from the others (their value
    at the stand-in for a missing feature is large, so they keep their select), with rows that miss none, some and all
    of their features."""
    from spnc.structure import Gaussian, Product, Sum
    rng = np.random.default_rng(seed)
    products = []
    for _ in range(5):
        leaves = []
        for f in range(11):
            narrow = rng.random() < 0.25
            leaves.append(Gaussian(mean=float(rng.normal(0, 3 if narrow else 1)), stdev=float(rng.uniform(0.05, 0.2) if narrow else rng.uniform(0.5, 2.0)), scope=f))
        products.append(Product(children=leaves))
    spn = Sum([float(v) for v in rng.dirichlet(np.ones(5))], products)
    X = rng.normal(0, 1.5, (600, 11)).astype(np.float32)
    X[rng.random(X.shape) < 0.3] = np.nan
    X[0, :] = np.nan
    X[1, :10] = np.nan
    X[2, 1:] = np.nan
    X[3, :] = 0.25
    return spn, X


@pytest.mark.parametrize("opts", [{}, {"hip-marginal-offsets": "false"}, {"hip-marginal-tables-kib": 1}, {"maxTaskSize": 20}],
                         ids=["offsets", "selects", "few-tables", "cut"])
def test_missing_features_in_wide_products_on_the_host(native, tmp_path, opts):
    spn, X = _wide_marginal_products()
    k = compile_spn(native, spn, "float32", marginal=True, **dict(opts, **{"hip-kernel": "jit"}))
    info, src = k.info(), k.source()
    os.remove(k.fileName())
    if not opts:
        assert "SPN_CTAB[" in src and " != g" in src   # both forms in one kernel: table offsets, and selects for the narrow leaves
    got = host_kernel(src, info, tmp_path)(X)
    ref = ev.ll_closed_f64(oracle_model(spn, "float32"), X, marginal=True)
    assert np.isfinite(ref).all() and abs(ref[0]) < 1e-12   # every feature missing: log 1
    # the narrow leaves put results at -100 to -3000, where a float's own spacing is up to 2.4e-4: 1e-4 plus three such steps
    assert (np.abs(got - ref) <= 1e-4 + 4e-7 * np.abs(ref)).all()
    near = np.abs(ref) < 60
    assert near.sum() > 50 and np.abs(got[near] - ref[near]).max() <= 1e-4


def _narrow_leaf_next_to_the_stand_in():
    """Two products over two features; on feature 0 one leaf is very narrow (stddev 0.003) and sits 0.01 from the value
    that stands in for a missing input (the middle of the two means). Its value there is small, so it goes through the
    table, but it moves by 1e-4 when the mean moves by one float rounding: the table entry has to come from the rounded
    constants the kernel computes with."""
    from spnc.structure import Gaussian, Product, Sum
    spn = Sum([0.3, 0.7], [Product(children=[Gaussian(mean=1.0, stdev=0.5, scope=0), Gaussian(mean=0.2, stdev=1.0, scope=1)]),
                           Product(children=[Gaussian(mean=1.02, stdev=0.003, scope=0), Gaussian(mean=-0.4, stdev=0.8, scope=1)])])
    rng = np.random.default_rng(8)
    X = np.column_stack((rng.normal(1.01, 0.01, 400), rng.normal(0, 1, 400))).astype(np.float32)
    X[::2, 0] = np.nan
    X[::5, 1] = np.nan
    return spn, X


def test_narrow_leaf_next_to_the_stand_in_on_the_host(native, tmp_path):
    spn, X = _narrow_leaf_next_to_the_stand_in()
    k = compile_spn(native, spn, "float32", marginal=True, **{"hip-kernel": "jit"})
    info, src = k.info(), k.source()
    os.remove(k.fileName())
    assert "SPN_CTAB[" in src and ") ? 0x" not in src   # both leaves of both products through tables, no select of a constant
    got = host_kernel(src, info, tmp_path)(X)
    ref = ev.ll_closed_f64(oracle_model(spn, "float32"), X, marginal=True)
    missing = np.isnan(X[:, 0])
    assert np.abs(got[missing] - ref[missing]).max() <= 2e-6   # nothing of the narrow leaf is left when its feature is missing
    assert (np.abs(got - ref) <= 1e-4 + 4e-7 * np.abs(ref)).all()
