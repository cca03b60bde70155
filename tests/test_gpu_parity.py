"""Parity of the HIP kernels with the CPU oracle, through the C-ABI, on a real MI355X.

Tolerances: |delta| <= 1e-4 absolute log-likelihood for f32 kernels, <= 1e-10 for f64 kernels
(the bars the path is specified to), checked against the oracle's restatement of the reference's
CPU kernel (``ll_reforder``) and against the float64 closed form.
"""
import math
import os

import numpy as np
import pytest

import rawfile as rf
from conftest import GOLDEN, ROOT, compile_query, compile_spn, load_golden, model_as_query, oracle_model, quiet
from oracle import c_oracle, evaluate as ev, spn_model as sm

pytestmark = pytest.mark.gpu

F32_TOL = 1e-4
F64_TOL = 1e-10

VARIANTS = {
    "jit": {},
    "jit-pairwise": {"hip-sum-form": "pairwise"},
    "jit-strict": {"hip-sum-form": "pairwise", "hip-log2-domain": "false"},
    "interp": {"hip-kernel": "interpreter"},
    "interp-natural": {"hip-kernel": "interpreter", "hip-log2-domain": "false"},
}


def within_f32(got, want, tol=F32_TOL):
    """Float32 results against float64 expectations, row by row: the strict absolute bar wherever |LL| <= 100, and the
    same number of float32 digits beyond (a float32 near 1000 is spaced 6e-5 apart; 1e-4 absolute means nothing there)."""
    return bool(np.all(np.abs(got - want) <= tol * np.maximum(1.0, np.abs(want) / 100)))


def run(kernel, X):
    out = kernel.execute(X.shape[0], X)
    os.remove(kernel.fileName()) if os.path.isfile(kernel.fileName()) else None
    return out


def check_f32(got, model, X, marginal):
    assert got.dtype == np.float32 and got.shape == (X.shape[0],)
    ref32 = ev.ll_reforder(model, X, np.float32, marginal=marginal)
    ref64 = ev.ll_closed_f64(model, X, marginal=marginal)
    finite = np.isfinite(ref64)
    assert np.array_equal(np.isneginf(got), np.isneginf(ref64))
    assert np.abs(got[finite] - ref64[finite]).max(initial=0) <= F32_TOL
    ok = finite & np.isfinite(ref32)
    assert np.abs(got[ok] - ref32[ok]).max(initial=0) <= F32_TOL


# ---- the reference's own CUDA test cases (python-interface/test/cuda/*.py), run through HIPCompiler ----

def _reference_test_spns():
    from spnc import synthetic as syn
    from spnc.structure import Gaussian, Histogram, Product, Sum
    cat = syn.c1_spn()
    gauss = Product(children=[Gaussian(mean=m, stdev=s, scope=i) for i, (m, s) in enumerate(
        [(0.5, 1.0), (0.125, 0.25), (0.345, 0.24), (0.456, 0.1), (0.94, 0.48), (0.56, 0.42), (0.76, 0.14), (0.32, 0.58), (0.58, 0.219),
         (0.14, 0.28)])])
    h1 = Histogram([0., 1., 2.], [0.25, 0.75], [1, 1], scope=0)
    h2 = Histogram([0., 1., 2.], [0.45, 0.55], [1, 1], scope=1)
    h3 = Histogram([0., 1., 2.], [0.33, 0.67], [1, 1], scope=0)
    h4 = Histogram([0., 1., 2.], [0.875, 0.125], [1, 1], scope=1)
    hist = Sum(children=[Product(children=[h1, h2]), Product(children=[h3, h4])], weights=[0.3, 0.7])
    return cat, gauss, hist


@pytest.mark.parametrize("marginal", [False, True])
def test_reference_cuda_test_cases(native, marginal):
    from spnc.hip import HIPCompiler
    rng = np.random.default_rng(7)
    cat, gauss, hist = _reference_test_spns()
    cases = [(cat, rng.integers(0, 3, (30, 6)).astype("float64")), (gauss, rng.normal(0.5, 1.0, (30, 10)).astype("float64")),
             (hist, rng.integers(0, 2, (30, 2)).astype("float64"))]
    for spn, X in cases:
        if marginal:
            X[rng.random(X.shape) < 0.3] = np.nan
        for preload in (False, True):
            with quiet():
                got = HIPCompiler(preloadToSharedMem=preload).log_likelihood(spn, X, supportMarginal=marginal)
            m = oracle_model(spn, "float64")
            want = ev.ll_closed_f64(m, X, marginal=marginal)
            # the reference's own acceptance criterion ...
            assert np.all(np.isclose(got, want)) or np.all(np.isclose(np.exp(got), np.exp(want)))
            # ... and the absolute bar of this path
            check_f32(got, m, X, marginal)


def test_integer_inputs_readme_example(native):
    from spnc import synthetic as syn
    from spnc.hip import HIPCompiler
    X = syn.c1_inputs(30)
    with quiet():
        got = HIPCompiler().log_likelihood(syn.c1_spn(), X, supportMarginal=False)
    check_f32(got, oracle_model(syn.c1_spn(), "int32"), X, False)


@pytest.mark.parametrize("name", ["mini-example", "categorical-example", "gaussian-example"])
def test_known_answers(native, name):
    from test_oracle_pins import KNOWN
    X, expected = KNOWN[name]
    for opts in VARIANTS.values():
        got = run(compile_query(native, os.path.join(GOLDEN, name + ".bin"), **opts), X)
        assert np.allclose(got, expected, rtol=0, atol=6e-6)


@pytest.mark.parametrize("variant", sorted(VARIANTS))
@pytest.mark.parametrize("name", ["NIPS5", "nltcs", "plants"])
def test_golden_outputs_f32(native, tmp_path, name, variant):
    X, ref = load_golden(name)
    if name == "NIPS5":
        path, X = os.path.join(GOLDEN, "NIPS5.bin"), X.astype(np.uint32)
    else:
        path = model_as_query(os.path.join(GOLDEN, name + ".bin"), "float64", str(tmp_path / "q.bin"))
    got = run(compile_query(native, path, **VARIANTS[variant]), X)
    assert got.dtype == np.float32
    assert np.abs(got - ref).max() <= F32_TOL


@pytest.mark.parametrize("opts", [{"hip-compute-type": "float64"}, {"hip-compute-type": "float64", "hip-sum-form": "pairwise"},
                                  {"hip-compute-type": "float64", "hip-kernel": "interpreter"},
                                  {"hip-compute-type": "float64", "hip-kernel": "interpreter", "hip-log2-domain": "false"}, {"use-log-space": "false"},
                                  {"use-log-space": "false", "hip-kernel": "interpreter"}, {"use-log-space": "false", "hip-kernel": "jit", "maxTaskSize": 2000}],
                         ids=["log-f64", "log-f64-pairwise", "log-f64-interp", "log-f64-interp-natural", "linear-f64", "linear-f64-interp", "linear-f64-tasks"])
@pytest.mark.parametrize("name", ["NIPS5", "nltcs", "plants"])
def test_golden_outputs_f64(native, tmp_path, name, opts):
    if name == "nltcs" and "hip-sum-form" in opts:
        # one straight-line float64 kernel of the 3641-node model takes minutes of hipRTC time: cut into tasks it builds in seconds
        opts = dict(opts, maxTaskSize=300, **{"hip-kernel": "jit"})
    X, ref = load_golden(name)
    if name == "NIPS5":
        path, X = os.path.join(GOLDEN, "NIPS5.bin"), X.astype(np.uint32)
    else:
        path = model_as_query(os.path.join(GOLDEN, name + ".bin"), "float64", str(tmp_path / "q.bin"))
    k = compile_query(native, path, **opts)
    if name == "nltcs" and "use-log-space" in opts:
        # a graph this size in linear space: the interpreter unless the caller asks for straight-line kernels, then cut into tasks
        if opts.get("hip-kernel") == "jit":
            assert k.info()["kernel_kind"] == 1 and k.info()["num_tasks"] > 1
        else:
            assert k.info()["kernel_kind"] == 2
    got = run(k, X)
    assert got.dtype == np.float64
    assert np.abs(got - ref).max() <= F64_TOL


def _partition_example():
    """The SPN of the reference's partitioning tests (python-interface/test/vector/test_log_vector_graph_partitioning.py:22-31,
    test/cpu/test_graph_partitioning.py): two products of two histograms under one sum."""
    from spnc.structure import Histogram, Product, Sum
    h1 = Histogram([0., 1., 2.], [0.25, 0.75], [1, 1], scope=0)
    h2 = Histogram([0., 1., 2.], [0.45, 0.55], [1, 1], scope=1)
    h3 = Histogram([0., 1., 2.], [0.33, 0.67], [1, 1], scope=0)
    h4 = Histogram([0., 1., 2.], [0.875, 0.125], [1, 1], scope=1)
    return Sum([0.3, 0.7], [Product(children=[h1, h2]), Product(children=[h3, h4])])


@pytest.mark.parametrize("opts", [{}, {"hip-compute-type": "float64"}, {"use-log-space": "false"}, {"hip-sum-form": "pairwise", "hip-log2-domain": "false"}],
                         ids=["log-f32", "log-f64", "linear-f64", "strict-f32"])
@pytest.mark.parametrize("size", [1, 2, 5])
def test_reference_partitioning_example(native, opts, size):
    """maxTaskSize=5 on the reference's seven-node example, as its tests run it (and the smallest bounds there are): the
    graph becomes several kernels that pass values through device memory, and the results are those of the uncut graph."""
    rng = np.random.default_rng(30)
    X = np.column_stack((rng.integers(0, 2, 30), rng.integers(0, 2, 30))).astype("float64")
    spn = _partition_example()
    k = compile_spn(native, spn, "float64", marginal=False, maxTaskSize=size, **opts)
    assert k.info()["num_tasks"] > 1
    got = run(k, X)
    ref = ev.ll_closed_f64(oracle_model(spn, "float64"), X, marginal=False)
    assert np.abs(got - ref).max() <= (F32_TOL if got.dtype == np.float32 else F64_TOL)


@pytest.mark.parametrize("cfg,size", [("c1", 3), ("c2", 400), ("c3", 300), ("c5", 150), ("c5", 1200)])
def test_partitioned_benchmark_configurations(native, cfg, size):
    """The benchmark graphs cut into tasks: integer and float features, table leaves with their own LDS pool per task,
    Gaussian leaves with missing values, sums split into trees where one sum alone exceeds the bound."""
    from spnc import synthetic as syn
    c = syn.CONFIGS[cfg]
    spn, X = c["spn"](), c["inputs"](3000)
    k = compile_spn(native, spn, c["dtype"], marginal=c["marginal"], maxTaskSize=size, **{"hip-kernel": "jit"})
    assert k.info()["num_tasks"] > 1
    check_f32(run(k, X), oracle_model(spn, c["dtype"]), X, c["marginal"])


@pytest.mark.parametrize("size", [3, 10, 17])
def test_partitioned_nips5_in_linear_space(native, size):
    """The reference's partitioned NIPS5 runs (python-interface/test/examples/NIPS5/test_partitioned_cuda_NIPS5.py:34 with
    maxTaskSize=10, test_partitioned_vector_NIPS5.py:35 with 3): linear space, float64, against its expected outputs."""
    X, ref = load_golden("NIPS5")
    k = compile_query(native, os.path.join(GOLDEN, "NIPS5.bin"), maxTaskSize=size, **{"use-log-space": "false"})
    assert k.info()["num_tasks"] > 1
    got = run(k, X.astype(np.uint32))
    assert got.dtype == np.float64 and np.abs(got - ref).max() <= F64_TOL


@pytest.mark.parametrize("opts", [{"maxTaskSize": 64}, {"maxTaskSize": 1000}, {"maxTaskSize": 250, "hip-sum-form": "pairwise"},
                                  {"maxTaskSize": 400, "hip-compute-type": "float64"}, {"maxTaskSize": 120, "hip-task-buffer-mib": 1}],
                         ids=["64", "1000", "250-pairwise", "400-f64", "120-small-buffer"])
@pytest.mark.parametrize("name", ["nltcs", "plants"])
def test_partitioned_golden_models(native, tmp_path, name, opts):
    """nltcs (3641 nodes) and plants cut into tasks of different sizes reproduce the reference's expected outputs; with a
    1 MiB buffer for the values between tasks the batch runs in several passes (1024 rows at a time at least)."""
    X, ref = load_golden(name)
    path = model_as_query(os.path.join(GOLDEN, name + ".bin"), "float64", str(tmp_path / "q.bin"))
    k = compile_query(native, path, **dict(opts, **{"hip-kernel": "jit"}))
    assert k.info()["num_tasks"] > 1
    if "hip-task-buffer-mib" in opts:
        reps = -(-12000 // X.shape[0])
        X, ref = np.tile(X, (reps, 1)), np.tile(ref, reps)
        assert k.info()["task_rows"] * 4 * X.shape[0] > (1 << 20)   # more than one pass
    got = run(k, X)
    assert np.abs(got - ref).max() <= (F64_TOL if got.dtype == np.float64 else F32_TOL)


def test_partitioned_kernel_on_two_streams_and_reloaded(native, tmp_path):
    """A partitioned kernel keeps one buffer of intermediate values: calls on different streams take turns on it; the
    kernel file restores all tasks."""
    import torch
    X, ref = load_golden("plants")
    path = model_as_query(os.path.join(GOLDEN, "plants.bin"), "float64", str(tmp_path / "q.bin"))
    k = compile_query(native, path, maxTaskSize=150, **{"hip-kernel": "jit"})
    k2 = native.Kernel(k.fileName(), k.kernelName(), k.queryType(), k.target(), k.batchSize(), k.numFeatures(), k.bytesPerFeature(), k.numResults(),
                       k.bytesPerResult(), k.dataType())
    assert k2.info()["num_tasks"] == k.info()["num_tasks"] > 1
    Xd = torch.from_numpy(np.ascontiguousarray(X)).cuda()
    outs = [torch.empty(X.shape[0], dtype=torch.float32, device="cuda") for _ in range(4)]
    streams = [torch.cuda.Stream() for _ in range(2)]
    torch.cuda.synchronize()
    for rep in range(4):
        s = streams[rep % 2]
        k2.execute_device(X.shape[0], Xd.data_ptr(), outs[rep].data_ptr(), s.cuda_stream)
    torch.cuda.synchronize()
    for o in outs:
        assert np.abs(o.cpu().numpy() - ref).max() <= F32_TOL
    os.remove(k.fileName())


def test_interpreter_kernel_on_two_streams(native):
    """An interpreter handle keeps one buffer of spilled value slots: launches on different streams take turns on it
    (as the reference's generated host code is re-entrant, mlir/lib/Conversion/LoSPNtoGPU/GPUStructurePatterns.cpp:96-146).
    Four launches over different inputs alternate between two streams with nothing between them."""
    import torch
    from spnc import synthetic as syn
    c = syn.CONFIGS["c4"]
    spn = c["spn"]()
    k = compile_spn(native, spn, c["dtype"])
    assert k.info()["kernel_kind"] == 2 and "long-lived" in k.source()     # values in the spill tier
    n = 400_003
    base = c["inputs"](4001)
    xs = []
    for rep in range(4):
        idx = (torch.arange(n, device="cuda") * (rep + 1) + rep) % 4001
        xs.append(torch.from_numpy(base).cuda()[idx].contiguous())
    serial = []
    for x in xs:
        out = torch.empty(n, dtype=torch.float32, device="cuda")
        k.execute_device(n, x.data_ptr(), out.data_ptr(), torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        serial.append(out)
    outs = [torch.full((n,), float("nan"), dtype=torch.float32, device="cuda") for _ in range(4)]
    streams = [torch.cuda.Stream() for _ in range(2)]
    torch.cuda.synchronize()
    for rep in range(4):
        k.execute_device(n, xs[rep].data_ptr(), outs[rep].data_ptr(), streams[rep % 2].cuda_stream)
    torch.cuda.synchronize()
    want = ev.ll_closed_f64(oracle_model(spn, c["dtype"]), base, marginal=False)
    for rep in range(4):
        assert torch.equal(outs[rep], serial[rep]), rep
        idx = ((np.arange(2000) * (rep + 1) + rep) % 4001)
        assert np.abs(outs[rep][:2000].cpu().numpy() - want[idx]).max() <= F32_TOL
    os.remove(k.fileName())


def _speaker_inputs(n, seed=5):
    """Inputs as the reference's speaker test draws them (python-interface/test/examples/speaker/test_vector_slp_speaker.py:20-47):
    feature i ~ N(0.01 (i + 1), s_i) with s = 1.0, 0.9, ..., 0.1 repeating."""
    rng = np.random.default_rng(seed)
    return np.column_stack([rng.normal(0.01 * (i + 1), 1.0 - 0.1 * (i % 10), n) for i in range(26)]).astype("float64")


@pytest.mark.parametrize("opts", [{}, {"hip-kernel": "interpreter"}, {"hip-sum-form": "pairwise", "hip-log2-domain": "false"},
                                  {"hip-compute-type": "float64"}, {"hip-compute-type": "float64", "hip-kernel": "interpreter"},
                                  {"use-log-space": "false"}],
                         ids=["f32", "f32-interp", "f32-strict", "f64", "f64-interp", "linear-f64"])
@pytest.mark.parametrize("name", ["speaker_FADG0", "NIPS10"])
def test_reference_queries_without_expected_outputs(native, name, opts):
    """speaker_FADG0.bin (26 Gaussian features, 1326 leaves) and NIPS10.bin (ten histogram features) ship without expected
    outputs; the reference's own test compares with SPFlow's closed-form inference, here the oracle's float64 closed form."""
    path = os.path.join(GOLDEN, name + ".bin")
    m = sm.load_model(path)
    if name == "NIPS10":
        X = np.random.default_rng(3).integers(0, 72, (5000, 10)).astype(np.uint32)
        X[:3000] = np.minimum(X[:3000], np.random.default_rng(4).integers(0, 6, (3000, 10))).astype(np.uint32)   # the dense low bins
    else:
        X = _speaker_inputs(5000)
    want = ev.ll_closed_f64(m, X, marginal=False)
    assert np.isfinite(want).all()
    got = run(compile_query(native, path, **opts), X)
    if got.dtype == np.float64:
        assert np.abs(got - want).max() <= (1e-9 if "use-log-space" in opts else F64_TOL)
    else:
        assert within_f32(got, want), np.abs(got - want).max()


def test_the_47k_node_model_in_linear_space(native, tmp_path):
    """fashion_mnist.bin computed with probabilities instead of logarithms (the reference's computeInLogSpace=False, which
    yields float64): the interpreter takes it, so compiling is a matter of a second. The product of 784 densities leaves
    the double range (log-likelihoods near -1000 even at the leaves' means), where the reference's arithmetic ends in
    log(0) = -inf as well: that is what the oracle's restatement of the reference's linear kernel gives for every row."""
    import time
    path = model_as_query(os.path.join(GOLDEN, "fashion_mnist.bin"), "float64", str(tmp_path / "q.bin"))
    m = sm.load_model(path)
    X = np.random.default_rng(12).random((200, 784))
    t0 = time.time()
    k = compile_query(native, path, **{"use-log-space": "false"})
    assert time.time() - t0 < 10 and k.info()["kernel_kind"] == 2 and k.info()["dtype"] == "float64"
    got = run(k, X)
    want = ev.ll_linear_f64(m, X, marginal=False)
    assert got.dtype == np.float64 and np.array_equal(np.isneginf(got), np.isneginf(want)) and not np.isnan(got).any()


@pytest.mark.parametrize("cfg", ["c2", "c3", "c4", "c5"])
def test_benchmark_configurations_in_linear_space_on_the_interpreter(native, cfg):
    """Linear space (probabilities, float64) on the interpreter against the oracle's restatement of the reference's linear
    kernel (mlir/lib/Conversion/LoSPNtoCPU/NodePatterns.cpp:242-304): Gaussian and table leaves, missing features, sums
    over outer products, the region graph that the interpreter takes by itself."""
    from spnc import synthetic as syn
    c = syn.CONFIGS[cfg]
    spn, X = c["spn"](), c["inputs"](1500)
    opts = {"use-log-space": "false"} if cfg == "c4" else {"use-log-space": "false", "hip-kernel": "interpreter"}
    k = compile_spn(native, spn, c["dtype"], marginal=c["marginal"], **opts)
    assert k.info()["kernel_kind"] == 2 and "linear space" in k.source()
    got = run(k, X)
    want = ev.ll_linear_f64(oracle_model(spn, c["dtype"]), X, marginal=c["marginal"])
    finite = np.isfinite(want)
    assert got.dtype == np.float64 and finite.sum() > 1000
    assert np.array_equal(np.isneginf(got), np.isneginf(want))
    assert np.abs(got[finite] - want[finite]).max() <= F64_TOL


@pytest.mark.parametrize("opts", [{}, {"hip-compute-type": "float64"}, {"hip-log2-domain": "false"}], ids=["f32", "f64", "f32-natural"])
def test_the_47k_node_model(native, tmp_path, opts):
    """fashion_mnist.bin of the reference's test resources (784 features, 47466 nodes, 39200 Gaussian leaves): the
    reference ships no expected outputs for it, so the oracle's closed form in float64 is the yardstick. |LL| is in the
    thousands: float64 must agree to 1e-9 absolute, float32 to a few units in the last place of the result."""
    path = model_as_query(os.path.join(GOLDEN, "fashion_mnist.bin"), "float64", str(tmp_path / "q.bin"))
    m = sm.load_model(path)
    X = np.random.default_rng(11).random((300, 784))
    X[7] = 0.0
    X[8] = 1.0
    ref = ev.ll_closed_f64(m, X, marginal=False)
    k = compile_query(native, path, **opts)
    assert k.info()["kernel_kind"] == 2   # interpreter-sized
    got = run(k, X)
    if opts.get("hip-compute-type") == "float64":
        assert got.dtype == np.float64
        assert np.abs(got - ref).max() <= 1e-9
    else:
        assert got.dtype == np.float32
        assert (np.abs(got - ref) / np.abs(ref)).max() <= 4 * np.finfo(np.float32).eps


@pytest.mark.parametrize("variant", sorted(VARIANTS))
@pytest.mark.parametrize("cfg", ["c1", "c2", "c3", "c3_deep", "c4", "c5"])
def test_benchmark_configurations(native, cfg, variant):
    from spnc import synthetic as syn
    c = syn.CONFIGS[cfg]
    opts = dict(VARIANTS[variant])
    if cfg == "c4" and variant == "jit-strict":
        # the 8881-node region graph as one straight-line kernel with library exp/log takes minutes of hipRTC time; cut into
        # tasks of 2000 operations it builds in seconds
        opts.update({"maxTaskSize": 2000, "hip-kernel": "jit"})
    n = 1500 if cfg == "c4" else 5000
    spn, X = c["spn"](), c["inputs"](n)
    got = run(compile_spn(native, spn, c["dtype"], marginal=c["marginal"], **opts), X)
    m = oracle_model(spn, c["dtype"])
    check_f32(got, m, X, c["marginal"])
    assert np.abs(got - c_oracle.ll_f32(m, X, marginal=c["marginal"])).max() <= F32_TOL


GROUPED = {
    "default": {},                                        # blocks of four columns, packed indices, one block of 1024 threads
    "plain": {"hip-grouped-tables": "false"},
    "singles": {"hip-table-group-window": 0},             # blocks of four columns, every table read on its own
    "wide-window": {"hip-table-group-window": 1000},
    "no-room": {"hip-table-pad-kib": 0},                  # blocks do not fit: plain tables
    "no-joint": {"hip-joint-tables": "false"},
    "small-pool": {"hip-table-budget-kib": 30},           # no pairing, and the blocks outgrow 30 + 18 KiB: plain tables
    "block-256": {"hip-block-size": 256},
    "float64": {"hip-compute-type": "float64"},           # 32-byte entries: offsets do not fit eight bits, plain tables
}


@pytest.mark.parametrize("cfg", ["c3", "c3_deep"])
@pytest.mark.parametrize("variant", sorted(GROUPED))
def test_grouped_tables_on_the_discrete_configuration(native, variant, cfg):
    """Tables read with the same index interleaved in blocks of four columns (one 16-byte read for up to four leaves):
    the layout, the packed indices and every fallback to plain tables give the oracle's values."""
    from spnc import synthetic as syn
    c = syn.CONFIGS[cfg]
    spn, X = c["spn"](), c["inputs"](4099)
    X[5, :] = 77            # out of every feature's range
    X[6, 3] = 9
    k = compile_spn(native, spn, c["dtype"], marginal=False, **GROUPED[variant], **{"hip-packed-rows": "false"})
    src = k.source()
    grouped = variant not in ("plain", "no-room", "small-pool", "float64")
    if cfg == "c3":   # products of up to fifty leaves: which layout the generator picks is its own business, the values count
        src = None
    assert src is None or ("v_bfe_u32" in src) == grouped and ("spn_r4*" in src) == (grouped and variant != "singles"), variant
    got = run(k, X)
    m = oracle_model(spn, c["dtype"])
    if variant == "float64":
        assert got.dtype == np.float64
        ref = ev.ll_closed_f64(m, X, marginal=False)
        assert np.array_equal(np.isneginf(got), np.isneginf(ref)) and np.isneginf(got[5]) and np.isneginf(got[6])
        assert np.abs(got[np.isfinite(ref)] - ref[np.isfinite(ref)]).max() <= F64_TOL
    else:
        check_f32(got, m, X, False)
        assert np.isneginf(got[5]) and np.isneginf(got[6])


PACKED = {
    "default": {},                                        # rows packed to bytes, sibling products fused, leaves over two categories as multiply-adds
    "unbatched": {"hip-fused-batch": 0},
    "batch-7": {"hip-fused-batch": 7},
    "all-lds": {"hip-one-hot-max-domain": 0},
    "one-hot-3": {"hip-one-hot-max-domain": 3},           # leaves over three categories as quadratic polynomials
    "one-hot-5": {"hip-one-hot-max-domain": 5},
    "no-joint": {"hip-joint-tables": "false"},
    "small-budget": {"hip-table-budget-kib": 24},         # pairs are split again until the tables fit
    "float64": {"hip-compute-type": "float64"},
    "block-256": {"hip-block-size": 256},
    "per-lane-rows": {"hip-wave-transpose": "false"},     # no per-wavefront transposed load: rows stay unpacked
}


@pytest.mark.parametrize("cfg", ["c3", "c3_deep"])
@pytest.mark.parametrize("variant", sorted(PACKED))
def test_packed_rows_on_the_discrete_configuration(native, variant, cfg):
    """Wide rows of small integers kept four features to a register, the table leaves of sibling products evaluated
    together (joint tables over pairs of features, one-hot multiply-adds for small domains): every variant gives the
    oracle's values, inputs outside a feature's range included (they make the result log 0)."""
    from spnc import synthetic as syn
    c = syn.CONFIGS[cfg]
    spn, X = c["spn"](), c["inputs"](4099)
    X[5, :] = 77            # out of every feature's range
    X[6, 3] = 9             # out of one feature's range
    X[7, 97] = 2 ** 31 - 1  # far out (a feature of the last register)
    X[8, 0] = 255
    X[9, 1] = 256           # does not fit a byte
    # Left to itself the compiler drops packed rows when the kernel spills registers (the deeper graph does): the
    # variants ask for them outright, "default" leaves the choice to the compiler.
    opts = dict(PACKED[variant])
    if variant != "default":
        opts.setdefault("hip-packed-rows", "true")
    k = compile_spn(native, spn, c["dtype"], marginal=False, **opts)
    src = k.source()
    packed = "unsigned PK0 = R[0]" in src and "spn_rows" in src
    assert packed == (variant != "per-lane-rows" and not (variant == "default" and cfg == "c3_deep"))
    got = run(k, X)
    m = oracle_model(spn, c["dtype"])
    if variant == "float64":
        assert got.dtype == np.float64
        ref = ev.ll_closed_f64(m, X, marginal=False)
        assert np.array_equal(np.isneginf(got), np.isneginf(ref))
        assert np.abs(got[np.isfinite(ref)] - ref[np.isfinite(ref)]).max() <= F64_TOL
    else:
        check_f32(got, m, X, False)
    assert all(np.isneginf(got[r]) for r in (5, 6, 7, 8, 9)) and np.isfinite(got[10])


@pytest.mark.parametrize("opts", [{}, {"hip-prefetch-rows": "false"}, {"hip-hoist-feature-values": "false"}, {"hip-fused-batch": 0}, {"hip-table-planes": "true"}],
                         ids=["default", "no-prefetch", "no-hoist", "unbatched", "planes"])
def test_packed_rows_with_long_tables(native, opts):
    """One sum over nine products of 32 categorical leaves, one feature with 120 categories: the padding that would make
    unclamped packed bytes safe is too large here, so the kernel clamps every byte to its table's length and puts the
    register together again. Inputs outside the
    ranges, next to them and far away, give log 0."""
    from spnc.structure import Categorical, Product, Sum
    rng = np.random.default_rng(17)
    domains = [120] + [int(d) for d in rng.integers(2, 7, 31)]
    products = []
    for _ in range(9):
        products.append(Product(children=[Categorical(p=[float(v) for v in rng.dirichlet(np.ones(d))], scope=f) for f, d in enumerate(domains)]))
    spn = Sum([float(v) for v in rng.dirichlet(np.ones(9))], products)
    X = np.column_stack([rng.integers(0, d, 3000) for d in domains]).astype(np.int32)
    X[3, 0] = 120
    X[4, 0] = 127
    X[5, 0] = 128
    X[6, 0] = 255
    X[7, 0] = 256
    X[8, 5] = domains[5]
    X[9, 31] = 2 ** 31 - 1
    X[10, :] = [d - 1 for d in domains]
    planes = opts.get("hip-table-planes") == "true"   # the siblings' tables one after the other: the padding stays small, nothing is clamped
    k = compile_spn(native, spn, "int32", marginal=False, **dict({"hip-table-planes": "false"}, **dict(opts, **{"hip-packed-rows": "true"})))
    src = k.source()
    assert "unsigned PK0 = R[0]" in src and ("PK0 = spn_q;" in src) == (not planes)   # packed rows, bytes clamped
    got = run(k, X)
    check_f32(got, oracle_model(spn, "int32"), X, False)
    assert all(np.isneginf(got[r]) for r in range(3, 10)) and np.isfinite(got[10]) and np.isfinite(got[:3]).all()


def test_narrow_leaf_next_to_the_stand_in(native):
    """A very narrow Gaussian leaf 0.01 from the value that stands in for its feature when it is missing: the table entry
    that takes the leaf's value off again comes from the rounded constants the kernel computes with (from the unrounded
    ones it would be 3e-5 off)."""
    from test_generated_code_host import _narrow_leaf_next_to_the_stand_in
    spn, X = _narrow_leaf_next_to_the_stand_in()
    k = compile_spn(native, spn, "float32", marginal=True, **{"hip-kernel": "jit"})
    assert "SPN_CTAB[" in k.source()
    got = run(k, X)
    ref = ev.ll_closed_f64(oracle_model(spn, "float32"), X, marginal=True)
    missing = np.isnan(X[:, 0])
    assert np.abs(got[missing] - ref[missing]).max() <= 2e-6
    assert (np.abs(got - ref) <= F32_TOL + 4e-7 * np.abs(ref)).all()


def test_discrete_graph_whose_tables_do_not_fit_lds(native):
    """10 k nodes over 64 integer features: the table pool is too large for LDS, so the kernel reads its tables from
    global memory with one index per feature (packed rows address their tables inside LDS and are not used)."""
    from spnc import synthetic as syn
    spn = syn.c3_spn(64, 33, sum_levels=3, inner_fan_in=(2, 9))
    X = syn.c3_inputs(3000, 64, 33, data_seed=933)
    X[5, :] = 77
    X[6, 3] = 9
    X[2999, 0] = -1
    k = compile_spn(native, spn, "int32", marginal=False)
    assert "unsigned PK0 = R[0]" not in k.source()
    got = run(k, X)
    check_f32(got, oracle_model(spn, "int32"), X, False)
    assert np.isneginf(got[5]) and np.isneginf(got[6]) and np.isneginf(got[2999])


@pytest.mark.parametrize("opts", [{}, {"hip-marginal-offsets": "false"}, {"hip-marginal-tables-kib": 1}, {"maxTaskSize": 20, "hip-kernel": "jit"},
                                  {"hip-kernel": "interpreter"}, {"hip-samples-per-lane": 2}, {"hip-block-size": 256, "gpu-shared-mem": "true"}],
                         ids=["offsets", "selects", "few-tables", "cut", "interpreter", "two-samples-per-lane", "staged-rows"])
def test_missing_features_in_wide_products(native, opts):
    """Products of eleven Gaussian leaves under one sum, a quarter of the leaves narrow and far from the others, rows that
    miss none, some and all of their features: float kernels take what leaves over missing features add off again with a
    table value per four leaves, and keep a select for the leaves whose value at the stand-in is large."""
    from test_generated_code_host import _wide_marginal_products
    spn, X = _wide_marginal_products()
    X = np.tile(X, (9, 1))[:5000]
    k = compile_spn(native, spn, "float32", marginal=True, **opts)
    if not opts:
        src = k.source()
        assert "SPN_CTAB[" in src and " != g" in src
    got = run(k, X)
    ref = ev.ll_closed_f64(oracle_model(spn, "float32"), X, marginal=True)
    assert got.dtype == np.float32 and np.isfinite(ref).all() and abs(got[0]) < 1e-6   # every feature missing: log 1
    # the narrow leaves put results at -100 to -3000, where a float's own spacing is up to 2.4e-4: 1e-4 plus three such steps
    assert (np.abs(got - ref) <= F32_TOL + 4e-7 * np.abs(ref)).all()
    near = np.abs(ref) < 60
    assert near.sum() > 400 and np.abs(got[near] - ref[near]).max() <= F32_TOL


@pytest.mark.parametrize("dtype,marginal", [("uint8", False), ("int32", False), ("float32", True), ("float64", True)])
def test_grouped_tables_feature_types_and_marginals(native, dtype, marginal):
    """Small graph, grouping forced: every feature has five or six table leaves (one index each), joint tables for the
    pairs inside the products; NaN selects the marginal entry, out-of-range values the impossible one."""
    from spnc.structure import Categorical, Histogram, Product, Sum
    rng = np.random.default_rng(23)
    doms = [2, 3, 5, 4]
    def product():
        kids = [Categorical(p=list(rng.dirichlet(np.ones(d))), scope=f) for f, d in enumerate(doms)]
        kids.append(Histogram(breaks=[0, 2, 3, 6], densities=list(rng.dirichlet(np.ones(3)) / np.array([2, 1, 3])), bin_repr_points=[1, 2, 4], scope=4))
        return Product(children=kids)
    spn = Sum(weights=list(rng.dirichlet(np.ones(2))), children=[
        Sum(weights=list(rng.dirichlet(np.ones(3))), children=[product() for _ in range(3)]),
        Sum(weights=list(rng.dirichlet(np.ones(2))), children=[product() for _ in range(2)])])
    X = np.column_stack([rng.integers(0, d + 2, 700) for d in doms + [7]]).astype(dtype)
    if marginal:
        X[rng.random(X.shape) < 0.2] = np.nan
        X[0, :] = np.nan
    for opts in ({"hip-table-group-min-reads": 0}, {"hip-table-group-min-reads": 0, "hip-joint-tables": "false"}, {}):
        k = compile_spn(native, spn, dtype, marginal=marginal, **opts)
        assert ("spn_r4*" in k.source()) == bool(opts)
        got = run(k, X)
        check_f32(got, oracle_model(spn, dtype), X, marginal)
        if marginal:
            assert abs(got[0]) < 1e-6


@pytest.mark.parametrize("kernel", ["jit", "interpreter"])
def test_c5_marginal_in_f64(native, kernel):
    from spnc import synthetic as syn
    c = syn.CONFIGS["c5"]
    spn, X = c["spn"](), c["inputs"](5000)
    got = run(compile_spn(native, spn, "float32", marginal=True, **{"hip-compute-type": "float64", "hip-kernel": kernel}), X)
    assert got.dtype == np.float64
    m = oracle_model(spn, "float32")
    assert np.abs(got - ev.ll_closed_f64(m, X, marginal=True)).max() <= F64_TOL
    # linear-space float64 (the reference's own f64 kernel) on the same inputs
    if kernel == "jit":
        lin = run(compile_spn(native, spn, "float32", marginal=True, **{"use-log-space": "false"}), X)
        assert np.abs(lin - ev.ll_linear_f64(m, X, marginal=True)).max() <= F64_TOL


@pytest.mark.parametrize("dtype", ["uint8", "uint16", "int32", "uint32", "int64", "float32", "float64"])
@pytest.mark.parametrize("kernel", ["jit", "interpreter"])
def test_feature_types_and_out_of_range_inputs(native, dtype, kernel):
    from spnc.structure import Categorical, Gaussian, Histogram, Product, Sum
    spn = Sum(weights=[0.4, 0.6], children=[
        Product(children=[Categorical(p=[0.2, 0.5, 0.3], scope=0), Gaussian(1.0, 2.0, scope=1),
                          Histogram(breaks=[0, 2, 3, 6], densities=[0.1, 0.5, 0.1], bin_repr_points=[1, 2, 4], scope=2)]),
        Product(children=[Categorical(p=[0.7, 0.3], scope=0), Gaussian(3.0, 1.5, scope=1),
                          Histogram(breaks=[1, 4], densities=[1 / 3], bin_repr_points=[2], scope=2)])])
    rng = np.random.default_rng(11)
    X = np.column_stack([rng.integers(0, 5, 400), rng.integers(0, 7, 400), rng.integers(0, 8, 400)]).astype(dtype)
    got = run(compile_spn(native, spn, dtype, **{"hip-kernel": kernel}), X)
    check_f32(got, oracle_model(spn, dtype), X, False)
    assert np.isneginf(got).any() and np.isfinite(got).any()


def test_nan_handling(native):
    from spnc import synthetic as syn
    spn = syn.c2_spn()
    X = syn.c2_inputs(64)
    X[0, :] = np.nan          # everything marginalised: log 1
    X[1, :8] = np.nan
    for kernel in ("jit", "interpreter"):
        got = run(compile_spn(native, spn, "float32", marginal=True, **{"hip-kernel": kernel}), X)
        assert abs(got[0]) < 1e-6     # log of the weights summing to 1, in float32
        check_f32(got, oracle_model(spn, "float32"), X, True)
    # table leaves: NaN marginalises, a fractional value truncates, negative / too large is impossible
    from spnc.structure import Categorical, Product
    spn = Product(children=[Categorical(p=[0.25, 0.75], scope=0), Categorical(p=[0.1, 0.9], scope=1)])
    X = np.array([[np.nan, 1.0], [1.9, np.nan], [np.nan, np.nan], [-0.5, 0.0], [-1.0, 0.0], [2.0, 0.0]])
    want = [math.log(0.9), math.log(0.75), 0.0, math.log(0.25 * 0.1), -math.inf, -math.inf]
    for kernel in ("jit", "interpreter"):
        got = run(compile_spn(native, spn, "float64", marginal=True, **{"hip-kernel": kernel}), X)
        assert np.allclose(got, want, rtol=0, atol=1e-6)


def test_impossible_evidence_gives_minus_infinity(native):
    """Zero-probability evidence under every child of a sum: -inf. (The reference's pairwise log-add
    yields NaN for -inf + -inf, mlir/lib/Conversion/LoSPNtoCPU/NodePatterns.cpp:233-239; the n-ary form does not.)"""
    from spnc.structure import Categorical, Product, Sum
    spn = Sum(weights=[0.5, 0.25, 0.25], children=[Product(children=[Categorical(p=[1.0, 0.0], scope=0), Categorical(p=[q, 1 - q], scope=1)])
                                                   for q in (0.5, 0.25, 0.125)])
    X = np.array([[1, 0], [0, 1]], dtype=np.int32)
    for kernel in ("jit", "interpreter"):
        got = run(compile_spn(native, spn, "int32", **{"hip-kernel": kernel}), X)
        assert np.isneginf(got[0]) and abs(got[1] - math.log(0.5 * 0.5 + 0.25 * 0.75 + 0.25 * 0.875)) < 1e-6


@pytest.mark.parametrize("n", [1, 63, 64, 255, 256, 257, 1023, 1025, 4097])
def test_ragged_sizes(native, n):
    from spnc import synthetic as syn
    for cfg, opts in (("c1", {}), ("c2", {}), ("c2", {"hip-kernel": "interpreter"})):
        c = syn.CONFIGS[cfg]
        spn = c["spn"]()
        X = c["inputs"](4097)[:n]
        got = run(compile_spn(native, spn, c["dtype"], **opts), X)
        full = ev.ll_reforder(oracle_model(spn, c["dtype"]), X, np.float32, marginal=False)
        assert got.shape == (n,) and np.abs(got - full).max() <= F32_TOL


@pytest.mark.parametrize("cfg", ["c2", "c5"])
def test_ragged_sizes_in_float64(native, cfg):
    """float64 kernels whose Gaussian leaves read their constants from other lanes of their row of sixteen: a batch that ends
    inside a row, inside a wavefront, or before the first row is full must not show (every lane stays at work, the ones
    past the end on the last row). With and without marginalisation, one and several tasks."""
    from spnc import synthetic as syn
    c = syn.CONFIGS[cfg]
    spn = c["spn"]()
    X = c["inputs"](1300)
    want = ev.ll_closed_f64(oracle_model(spn, c["dtype"]), X, marginal=c["marginal"])
    for opts in ({}, {"maxTaskSize": 700, "hip-kernel": "jit"}, {"hip-samples-per-lane": 2}):
        k = compile_spn(native, spn, c["dtype"], marginal=c["marginal"], **dict(opts, **{"hip-compute-type": "float64"}))
        assert "row_newbcast" in k.source()
        for n in (1, 7, 15, 16, 17, 63, 65, 255, 520, 991, 1000, 1300):
            got = k.execute(n, X[:n])
            assert got.shape == (n,) and np.abs(got - want[:n]).max() <= F64_TOL, (opts, n)
        os.remove(k.fileName())


def test_ragged_sizes_with_packed_rows(native):
    """The per-wavefront transposed load with its prefetch: batches smaller than one wavefront's tile (nothing to
    prefetch at all), exact tiles, one row more or less, partial last blocks."""
    from spnc import synthetic as syn
    c = syn.CONFIGS["c3"]
    spn = c["spn"]()
    k = compile_spn(native, spn, c["dtype"])
    assert "unsigned PK0 = R[0]" in k.source()
    X = c["inputs"](70000)
    full = ev.ll_closed_f64(oracle_model(spn, c["dtype"]), X, marginal=False)
    for n in (1, 2, 63, 64, 65, 127, 128, 511, 512, 513, 1000, 4096, 65535, 65536, 65537, 70000):
        got = k.execute(n, X[:n])
        assert got.shape == (n,) and np.abs(got - full[:n]).max() <= F32_TOL, n
    os.remove(k.fileName())


def test_packed_rows_over_several_rounds_of_tiles(native):
    """More tiles than the resident grid holds: every block runs its loop over tiles several times, so the tile that was
    prefetched during one round (fetched in two halves, parked in the wavefront's row buffer) is the one evaluated in
    the next. A 4096-row block repeats over the batch; an out-of-range row and the ragged tail sit in late tiles."""
    import torch
    from spnc import synthetic as syn
    c = syn.CONFIGS["c3"]
    spn = c["spn"]()
    k = compile_spn(native, spn, c["dtype"])
    assert "unsigned PK0 = R[0]" in k.source()
    block = c["inputs"](4096)
    n = 1_500_000 + 37                      # above 256 CUs x 2 blocks x 512 rows x 4 rounds
    idx = torch.arange(n, device="cuda") % 4096
    x = torch.from_numpy(block).cuda()[idx].contiguous()
    bad = [n - 5, n - 70_000, 1_234_567]
    for r in bad:
        x[r, 17] = 77                       # outside every table
    out = torch.empty(n, dtype=torch.float32, device="cuda")
    k.execute_device(n, x.data_ptr(), out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    small = torch.from_numpy(k.execute(4096, block)).cuda()
    want = ev.ll_closed_f64(oracle_model(spn, c["dtype"]), block, marginal=False)
    assert np.abs(small.cpu().numpy() - want).max() <= F32_TOL
    expect = small[idx]
    for r in bad:
        assert float(out[r]) == float("-inf")
        expect[r] = float("-inf")
    assert torch.equal(out, expect)
    os.remove(k.fileName())


def test_empty_batch_and_reuse(native):
    from spnc import synthetic as syn
    k = compile_spn(native, syn.c1_spn(), "int32")
    assert k.execute(0, np.zeros((0, 6), dtype=np.int32)).shape == (0,)
    X = syn.c1_inputs(100)
    a, b = k.execute(100, X), k.execute(50, X[:50])      # compile once, execute many
    assert np.array_equal(a[:50], b)
    os.remove(k.fileName())


def test_kernel_reloaded_from_file_computes_the_same(native):
    from spnc import synthetic as syn
    for cfg, opts in (("c3", {}), ("c3", {"hip-kernel": "interpreter"})):
        c = syn.CONFIGS[cfg]
        k = compile_spn(native, c["spn"](), c["dtype"], **opts)
        X = c["inputs"](1000)
        first = k.execute(1000, X)
        again = native.Kernel(k.fileName()).execute(1000, X)
        assert np.array_equal(first, again)
        os.remove(k.fileName())


def test_host_path_streams_large_batches_in_chunks(native):
    """More rows than one staging chunk (32 MiB of input): chunk boundaries must not show."""
    from spnc import synthetic as syn
    spn = syn.c2_spn()
    n = 1_300_000
    X = np.tile(syn.c2_inputs(4096), (n // 4096 + 1, 1))[:n]
    for opts in ({}, {"hip-kernel": "interpreter"}):
        k = compile_spn(native, spn, "float32", **opts)
        got = k.execute(n, X)
        small = k.execute(4096, X[:4096])
        os.remove(k.fileName())
        assert np.abs(small - ev.ll_reforder(oracle_model(spn, "float32"), X[:4096], np.float32, marginal=False)).max() <= F32_TOL
        reps = got[: (n // 4096) * 4096].reshape(-1, 4096)
        assert np.array_equal(reps, np.broadcast_to(small, reps.shape))
        assert np.array_equal(got[(n // 4096) * 4096:], small[: n % 4096])


def test_device_pointer_checks(native):
    import torch
    from spnc import synthetic as syn
    k = compile_spn(native, syn.c2_spn(), "float32")
    x = torch.zeros(1024 * 16 + 4, dtype=torch.float32, device="cuda")
    out = torch.empty(1024, dtype=torch.float32, device="cuda")
    with pytest.raises(RuntimeError, match="input pointer must be aligned to 16 bytes"):
        k.execute_device(1024, x.data_ptr() + 4, out.data_ptr())
    k.execute_device(1024, x.data_ptr(), out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    os.remove(k.fileName())


# ---- full benchmark sizes: properties that do not need the oracle at that size ----

def test_c1_at_64m_rows_matches_the_729_state_table(native):
    import torch
    from spnc import synthetic as syn
    k = compile_spn(native, syn.c1_spn(), "int32")
    states = np.array(np.meshgrid(*[range(3)] * 6, indexing="ij")).reshape(6, -1).T.astype(np.int32)   # all 3^6 inputs
    table = ev.ll_closed_f64(oracle_model(syn.c1_spn(), "int32"), states, marginal=False)
    n = 64 * 2 ** 20
    idx = torch.arange(n, device="cuda") % 729
    x = torch.from_numpy(states).cuda()[idx].contiguous()
    out = torch.empty(n, dtype=torch.float32, device="cuda")
    k.execute_device(n, x.data_ptr(), out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    first = out[:729].cpu().numpy()
    assert np.abs(first - table).max() <= F32_TOL
    assert abs(np.exp(first.astype(np.float64)).sum() - 1.0) < 1e-5        # the distribution is normalised
    assert bool((out == out[:729][idx]).all())                              # every row, bit for bit
    os.remove(k.fileName())


@pytest.mark.parametrize("cfg,opts", [("c2", {}), ("c5", {}), ("c3", {}), ("c4", {})])
def test_full_size_batches_repeat_a_checked_block(native, cfg, opts):
    import torch
    from spnc import synthetic as syn
    c = syn.CONFIGS[cfg]
    spn = c["spn"]()
    block = 3001 if cfg != "c4" else 1001          # odd, so repeats straddle tile and wave boundaries
    Xb = c["inputs"](block)
    n = c["n"]
    k = compile_spn(native, spn, c["dtype"], marginal=c["marginal"], **opts)
    want = ev.ll_reforder(oracle_model(spn, c["dtype"]), Xb, np.float32, marginal=c["marginal"])
    idx = torch.arange(n, device="cuda") % block
    x = torch.from_numpy(Xb).cuda()[idx].contiguous()
    out = torch.empty(n, dtype=torch.float32, device="cuda")
    k.execute_device(n, x.data_ptr(), out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert np.abs(out[:block].cpu().numpy() - want).max() <= F32_TOL
    assert bool((out == out[:block][idx]).all())
    os.remove(k.fileName())


# ---- randomly generated SPNs: DAGs with shared sub-graphs, mixed leaf kinds, uneven fan-in ----

def _random_spn(seed, num_features, marginal):
    from spnc.structure import Categorical, Gaussian, Histogram, Product, Sum
    rng = np.random.default_rng(seed)
    kinds = rng.integers(0, 3, num_features)        # per feature: 0 Gaussian, 1 Categorical, 2 Histogram
    domains = rng.integers(2, 7, num_features)
    pool = {}                                        # scope -> already built sub-SPNs, reused to make the graph a DAG

    def leaf(f):
        if kinds[f] == 0:
            return Gaussian(float(rng.normal()), float(rng.uniform(0.2, 2.0)), scope=int(f))
        p = rng.dirichlet(np.ones(domains[f]))
        if rng.random() < 0.2:
            p[rng.integers(0, len(p))] = 0.0         # an impossible category / empty bin
            p = p / p.sum()
        if kinds[f] == 1:
            return Categorical(p=[float(v) for v in p], scope=int(f))
        return Histogram(breaks=list(range(len(p) + 1)), densities=[float(v) for v in p], bin_repr_points=[0.5] * len(p), scope=int(f))

    def build(scope, depth):
        key = tuple(scope)
        if key in pool and rng.random() < 0.4:
            return pool[key][rng.integers(0, len(pool[key]))]
        if len(scope) == 1:
            node = leaf(scope[0])
        elif depth >= 4 or rng.random() < 0.3:
            node = Product(children=[leaf(f) for f in scope])
        elif rng.random() < 0.5:
            k = int(rng.integers(1, 20 if depth == 0 else 6))
            node = Sum(weights=[float(w) for w in rng.dirichlet(np.ones(k))], children=[build(scope, depth + 1) for _ in range(k)])
        else:
            parts = int(rng.integers(2, min(4, len(scope)) + 1))
            perm = [scope[i] for i in rng.permutation(len(scope))]
            node = Product(children=[build(sorted(int(v) for v in part), depth + 1) for part in np.array_split(np.array(perm), parts)])
        pool.setdefault(key, []).append(node)
        return node

    spn = build(list(range(num_features)), 0)
    n = 257
    X = np.empty((n, num_features), dtype=np.float64)
    for f in range(num_features):
        X[:, f] = rng.normal(0, 1.5, n) if kinds[f] == 0 else rng.integers(-1, domains[f] + 2, n)
    if marginal:
        X[rng.random(X.shape) < 0.15] = np.nan
    return spn, X


@pytest.mark.parametrize("seed", range(12))
def test_random_spns(native, seed):
    marginal = seed % 2 == 0
    spn, X = _random_spn(1000 + seed, num_features=3 + seed, marginal=marginal)
    m = oracle_model(spn, "float64")
    want64 = ev.ll_closed_f64(m, X, marginal=marginal)
    for opts in ({}, {"hip-kernel": "interpreter"}, {"hip-sum-form": "pairwise"}, {"hip-compute-type": "float64"},
                 {"hip-compute-type": "float64", "hip-kernel": "interpreter"}):
        got = run(compile_spn(native, spn, "float64", marginal=marginal, **opts), X)
        finite = np.isfinite(want64)
        if opts.get("hip-sum-form") != "pairwise":
            assert np.array_equal(np.isneginf(got), np.isneginf(want64)), opts
            assert np.isfinite(got[finite]).all(), opts
        else:
            # the pairwise tree turns (-inf) + (-inf) into NaN, like the reference: NaN only where the reference's operation
            # order gives it, and never on a row that order evaluates to a finite value
            ref = ev.ll_reforder(m, X, np.float32, marginal=marginal)
            assert not np.any(np.isnan(got) & ~np.isnan(ref)), opts
            assert np.isfinite(got[np.isfinite(ref)]).all(), opts
        ok = finite & np.isfinite(got)
        tol = F64_TOL if got.dtype == np.float64 else F32_TOL
        if got.dtype == np.float32:
            assert within_f32(got[ok], want64[ok], tol), opts
        else:
            assert np.abs(got[ok] - want64[ok]).max(initial=0) <= tol, opts
    if not marginal:                                    # integer inputs of the same values (negative ones wrap to huge unsigned: impossible)
        Xi = np.where(np.isnan(X), 0, X).astype(np.int32)
        has_gauss = any(n.kind == sm.GAUSSIAN for n in m.nodes)
        if not has_gauss:
            got = run(compile_spn(native, spn, "int32", **{}), Xi)
            check_f32(got, oracle_model(spn, "int32"), Xi.astype(np.uint32), False)


def _region_graph(seed, shapes, num_features=12, marginal=False):
    """Region graph whose sum groups cover given (left, right) operand counts: `shapes` lists, from
    the root region down, how many nodes the left child region holds; the right child is the rest of
    the chain and always holds eight sums (the last one: `shapes[-1][1]` leaf products)."""
    from spnc.structure import Gaussian, Product, Sum
    rng = np.random.default_rng(seed)

    def leaves(scope, count):
        return [Product(children=[Gaussian(mean=float(rng.normal()), stdev=float(rng.uniform(0.3, 1.4)), scope=int(f)) for f in scope])
                for _ in range(count)]

    def sums_over(left, right):
        products = [Product(children=[a, b]) for a in left for b in right]
        return [Sum(weights=[float(v) for v in rng.dirichlet(np.ones(len(products)))], children=products) for _ in range(8)]

    def chain(scope, level):
        na, nb_last = shapes[level]
        left = leaves(scope[:2], na)
        if level + 1 == len(shapes):
            return sums_over(left, leaves(scope[2:], nb_last))
        return sums_over(left, chain(scope[2:], level + 1))

    def mirrored(scope, level):   # the same with the operands swapped: (8, na) groups
        na, nb_last = shapes[level]
        right = leaves(scope[:2], na)
        if level + 1 == len(shapes):
            return sums_over(leaves(scope[2:], nb_last), right)
        return sums_over(mirrored(scope[2:], level + 1), right)

    roots = chain(list(range(num_features)), 0) + mirrored(list(range(num_features))[::-1], 0)
    spn = Sum(weights=[float(v) for v in rng.dirichlet(np.ones(len(roots)))], children=roots)
    X = rng.normal(0, 1.2, (700, num_features))
    if marginal:
        X[rng.random(X.shape) < 0.2] = np.nan
    return spn, X


@pytest.mark.parametrize("case", [
    ((2, 8), (4, 8), (8, 8), (4, 4)),        # groups of 2x8, 4x8, 8x8 and 4x4 products, and 8x2, 8x4, ... mirrored
    ((4, 8), (2, 8), (8, 4)),
    ((8, 8), (8, 8), (8, 8), (2, 8)),
])
@pytest.mark.parametrize("marginal", [False, True])
def test_matrix_form_outer_sums(native, case, marginal):
    """Every operand-count pair the matrix-core outer sum exists for, with slot lists in either tier."""
    spn, X = _region_graph(77 + len(case), case, num_features=2 * len(case) + 2, marginal=marginal)
    want64 = ev.ll_closed_f64(oracle_model(spn, "float64"), X, marginal=marginal)
    # LDS limits below the program's slot count put the long-lived pool (tiered access) or any slot (select-the-base
    # access) into the spill tier.
    for opts in ({}, {"hip-interp-short-slots": 12, "hip-interp-lds-slots": 24},
                 {"hip-interp-staged-features": "spill", "hip-interp-long-range": 4, "hip-interp-lds-slots": 24},
                 {"hip-interp-short-slots": 12, "hip-interp-long-range": 2, "hip-interp-lds-slots": 20},
                 {"hip-interp-matrix-core": "false"}, {"hip-interp-lds-slots": 6}):
        k = compile_spn(native, spn, "float64", marginal=marginal, **dict(opts, **{"hip-kernel": "interpreter"}))
        if opts.get("hip-interp-matrix-core") != "false":
            assert "outersum(8 sums x" in k.source()
        got = run(k, X)
        assert got.dtype == np.float32
        assert within_f32(got, want64), opts


def _leaf_region_graph(seed, count, leaves_per_product, regions, marginal, paired=False):
    """Sums over pairs of leaf regions: each leaf region holds `count` products of `leaves_per_product`
    Gaussians over features of its own; `regions` pairs are combined by outer products and eight sums each.
    paired: two such sum vectors at a time are combined the same way once more (2: and the results again)."""
    from spnc.structure import Gaussian, Product, Sum
    rng = np.random.default_rng(seed)
    G = leaves_per_product
    num_features = 2 * G * regions

    def leaf_region(scope):
        return [Product(children=[Gaussian(mean=float(rng.normal()), stdev=float(rng.uniform(0.3, 1.4)), scope=int(f)) for f in scope])
                for _ in range(count)]

    def sums_over(left, right):
        products = [Product(children=[a, b]) for a in left for b in right]
        return [Sum(weights=[float(v) for v in rng.dirichlet(np.ones(len(products)))], children=products) for _ in range(8)]

    vectors = []
    for r in range(regions):
        scope = list(range(2 * G * r, 2 * G * (r + 1)))
        vectors.append(sums_over(leaf_region(scope[:G]), leaf_region(scope[G:])))
    for _ in range(int(paired)):
        vectors = [sums_over(vectors[i], vectors[i + 1]) for i in range(0, len(vectors) - 1, 2)] + (vectors[-1:] if len(vectors) % 2 else [])
    tops = [Sum(weights=[float(v) for v in rng.dirichlet(np.ones(8))], children=v) for v in vectors]
    spn = Product(children=tops) if len(tops) > 1 else tops[0]
    X = rng.normal(0, 1.2, (600, num_features))
    if marginal:
        X[rng.random(X.shape) < 0.2] = np.nan
    return spn, X


@pytest.mark.parametrize("count,leaves", [(4, 2), (8, 2), (4, 4), (8, 4), (8, 1), (4, 1)])
@pytest.mark.parametrize("marginal", [False, True])
def test_leaf_regions_inside_the_outer_sum(native, count, leaves, marginal):
    """Outer sums over two leaf regions compute the leaf products themselves (4x4 and 8x8 products of one, two or
    four Gaussians), with the features and the results in either tier; the unfused program gives the same."""
    spn, X = _leaf_region_graph(500 + 10 * count + leaves, count, leaves, 3, marginal)
    want64 = ev.ll_closed_f64(oracle_model(spn, "float64"), X, marginal=marginal)
    for opts in ({}, {"hip-interp-staged-features": "spill", "hip-interp-long-range": 4, "hip-interp-lds-slots": 30},
                 {"hip-interp-staged-features": "lds", "hip-interp-short-slots": 12, "hip-interp-long-range": 2, "hip-interp-lds-slots": 40},
                 {"hip-interp-lds-slots": 6}, {"hip-interp-leaf-regions": "false"}):
        k = compile_spn(native, spn, "float64", marginal=marginal, **dict(opts, **{"hip-kernel": "interpreter"}))
        assert ("leafregion(8 sums x" in k.source()) == (opts.get("hip-interp-leaf-regions") != "false"), k.source()[:2000]
        got = run(k, X)
        assert got.dtype == np.float32
        assert within_f32(got, want64), opts


@pytest.mark.parametrize("count,leaves", [(4, 2), (8, 2), (4, 4), (8, 1), (4, 1)])
@pytest.mark.parametrize("marginal", [False, True])
def test_pairs_of_leaf_regions_inside_the_outer_sum(native, count, leaves, marginal):
    """An 8x8 outer sum over the result vectors of two leaf regions takes both in; five leaf regions give two such
    pairs and one leaf region on its own."""
    spn, X = _leaf_region_graph(900 + 10 * count + leaves, count, leaves, 5, marginal, paired=True)
    want64 = ev.ll_closed_f64(oracle_model(spn, "float64"), X, marginal=marginal)
    for opts in ({}, {"hip-interp-staged-features": "spill", "hip-interp-long-range": 4, "hip-interp-lds-slots": 30},
                 {"hip-interp-staged-features": "lds", "hip-interp-short-slots": 12, "hip-interp-long-range": 2, "hip-interp-lds-slots": 40},
                 {"hip-interp-lds-slots": 6}, {"hip-interp-scaled-vectors": "false"}):
        k = compile_spn(native, spn, "float64", marginal=marginal, **dict(opts, **{"hip-kernel": "interpreter"}))
        src = k.source()
        pairs = 2 if count == 4 and "hip-interp-scaled-vectors" not in opts else 0   # only 4x4 leaf regions are taken in as pairs
        assert src.count("leafpair(") == pairs and src.count("leafregion(") == 5 - 2 * pairs, src[:2000]
        got = run(k, X)
        assert got.dtype == np.float32
        assert within_f32(got, want64), opts


@pytest.mark.parametrize("count,leaves,regions,want", [
    (4, 2, 9, (2, 0, 1)), (4, 1, 9, (2, 0, 1)),
    (4, 4, 5, (0, 2, 1)),     # four leaves per product: pairs, no quads
    (8, 2, 9, (0, 0, 9)),     # 8x8 leaf regions stay single
    (4, 2, 13, (3, 0, 1)),    # 52 features: not staged, the fused instructions read the input row
    (4, 4, 9, (0, 4, 1)),     # 72 features, likewise
])
@pytest.mark.parametrize("marginal", [False, True])
def test_quads_of_leaf_regions_inside_the_outer_sum(native, count, leaves, regions, want, marginal):
    """Two levels of 8x8 outer sums over 4x4 leaf regions of one or two leaves per product become one instruction
    (`want`: instructions over four, two and one leaf region); other shapes stop at pairs or single regions."""
    spn, X = _leaf_region_graph(1300 + 10 * count + leaves + regions, count, leaves, regions, marginal, paired=2)
    want64 = ev.ll_closed_f64(oracle_model(spn, "float64"), X, marginal=marginal)
    for opts in ({}, {"hip-interp-staged-features": "spill", "hip-interp-long-range": 4, "hip-interp-lds-slots": 30},
                 {"hip-interp-staged-features": "lds", "hip-interp-short-slots": 12, "hip-interp-long-range": 2, "hip-interp-lds-slots": 50},
                 {"hip-interp-lds-slots": 6}):
        k = compile_spn(native, spn, "float64", marginal=marginal, **dict(opts, **{"hip-kernel": "interpreter"}))
        src = k.source()
        assert ("features direct" in src) == (2 * leaves * regions > 48)
        assert (src.count("leafquad("), src.count("leafpair("), src.count("leafregion(")) == want, src[:2000]
        got = run(k, X)
        assert got.dtype == np.float32
        assert within_f32(got, want64), opts


@pytest.mark.parametrize("count,leaves,regions,paired,want", [
    (4, 2, 9, 2, (2, 0, 1)), (4, 1, 9, 2, (2, 0, 1)), (4, 4, 5, 2, (0, 2, 1)), (8, 2, 3, 0, (0, 0, 3)), (8, 4, 3, 0, (0, 0, 3)),
    (4, 1, 5, 1, (0, 2, 1)), (4, 2, 13, 2, (3, 0, 1)),
])
@pytest.mark.parametrize("marginal", [False, True])
def test_fused_leaf_instructions_in_float64(native, count, leaves, regions, paired, want, marginal):
    """The instructions over one, two and four leaf regions in a double program: the weights reach the multiply-adds
    through lanes (v_fmac_f64 with a cross-lane operand), the vectors inside an instruction stay linear, its result is
    written as log2 values. Against the closed form to 1e-10, with the slots in either tier and with staged features."""
    spn, X = _leaf_region_graph(1700 + 10 * count + leaves + regions, count, leaves, regions, marginal, paired=paired)
    want64 = ev.ll_closed_f64(oracle_model(spn, "float64"), X, marginal=marginal)
    for opts in ({}, {"hip-interp-lds-slots": 6}, {"hip-interp-staged-features": "spill"}, {"hip-interp-staged-features": "lds", "hip-interp-lds-slots": 40},
                 {"hip-interp-leaf-regions": "false"}):
        k = compile_spn(native, spn, "float64", marginal=marginal, **dict(opts, **{"hip-kernel": "interpreter", "hip-compute-type": "float64"}))
        src = k.source()
        assert "compute f64" in src and ("features direct" in src) == (2 * leaves * regions > 48)
        fused = (src.count("leafquad("), src.count("leafpair("), src.count("leafregion("))
        assert fused == (want if "hip-interp-leaf-regions" not in opts else (0, 0, 0)), src[:2000]
        got = run(k, X)
        assert got.dtype == np.float64
        assert np.abs(got - want64).max() <= F64_TOL, opts


_LOAD_ORDER_SCRIPT = r"""
import os, sys
import numpy as np
root = sys.argv[1]
sys.path.insert(0, os.path.join(root, "spn-compiler_amd")); sys.path.insert(0, os.path.join(root, "tests")); sys.path.insert(0, root)
from spnc import spncpy as native
from spnc.hip import HIPCompiler
from spnc.structure import Categorical, Product
assert "torch" not in sys.modules
p = Product(children=[Categorical(p=[.35, .55, .1], scope=0), Categorical(p=[.25, .625, .125], scope=1)])
X = np.array([[0, 1], [2, 2], [1, 0]], dtype=np.int32)
k = HIPCompiler().compile_ll(p, "int32", supportMarginal=False)
first = k.execute(3, X)                       # the library's HIP runtime is up before torch is even imported
import torch
t = torch.arange(1000, device="cuda", dtype=torch.float32)
assert float(t.sum()) == 499500.0
second = k.execute(3, X)
Xd = torch.from_numpy(X).cuda()
out = torch.empty(3, dtype=torch.float32, device="cuda")
torch.cuda.synchronize()
k.execute_device(3, Xd.data_ptr(), out.data_ptr(), torch.cuda.current_stream().cuda_stream)
torch.cuda.synchronize()
want = np.log(np.array([.35 * .625, .1 * .125, .55 * .25]))
for got in (first, second, out.cpu().numpy()):
    assert np.abs(got - want).max() < 1e-6, got
os.remove(k.fileName())
print("load order ok")
"""


def test_library_loaded_before_torch(native):
    """The library brought up first, PyTorch imported and used afterwards, in a fresh process: both must work on the one
    GPU whichever HIP runtime library the loader picked for the process."""
    import subprocess, sys
    r = subprocess.run([sys.executable, "-c", _LOAD_ORDER_SCRIPT, ROOT], capture_output=True, text=True, timeout=280)
    assert r.returncode == 0 and "load order ok" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
