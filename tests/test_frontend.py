"""Python front end without a GPU: xspn writer/reader round trip, HIPCompiler argument checks, CPU baseline generator."""
import os

import numpy as np
import pytest

from conftest import GOLDEN, oracle_model, quiet, write_query


def _same(a, b):
    from spnc.structure import node_kind
    assert node_kind(a) == node_kind(b)
    kind = node_kind(a)
    if kind in ("product", "sum"):
        assert len(a.children) == len(b.children)
        if kind == "sum":
            assert list(a.weights) == list(b.weights)
        for x, y in zip(a.children, b.children):
            _same(x, y)
    elif kind == "gaussian":
        assert (a.mean, a.stdev, a.scope) == (b.mean, b.stdev, b.scope)
    elif kind == "categorical":
        assert (list(a.p), a.scope) == (list(b.p), b.scope)
    else:
        assert (list(a.breaks), list(a.densities), a.scope) == (list(b.breaks), list(b.densities), b.scope)


def test_round_trip_of_query_and_model(tmp_path):
    """Mirrors xspn/test/serialization/binary/test_binary_serialization_roundtrip.py of the reference."""
    from spnc import synthetic as syn
    from xspn.serialization.binary.BinarySerialization import BinaryDeserializer, BinarySerializer
    from xspn.structure.Model import SPNModel
    from xspn.structure.Query import ErrorKind, ErrorModel, JointProbability
    for spn, dtype in ((syn.c3_spn(), "int32"), (syn.c2_spn(), "float32")):
        path = str(tmp_path / "q.bin")
        with quiet():
            BinarySerializer(path).serialize_to_file(JointProbability(SPNModel(spn, dtype, "rt"), batchSize=17, supportMarginal=dtype != "int32",
                                                                      rootError=ErrorModel(ErrorKind.RELATIVE, 0.125)))
            q = BinaryDeserializer(path).deserialize_from_file()
        assert (q.batchSize, q.supportsMarginal(), q.errorModel.kind, q.errorModel.error) == (17, dtype != "int32", ErrorKind.RELATIVE, 0.125)
        assert (q.graph.featureType, q.graph.name) == (dtype, "rt")
        _same(q.graph.root, spn)
        with quiet():
            BinarySerializer(path).serialize_to_file(SPNModel(spn, dtype, "rt"))
            m = BinaryDeserializer(path).deserialize_from_file()
        assert isinstance(m, SPNModel)
        _same(m.root, spn)


def test_reader_accepts_multi_segment_files_of_the_reference():
    from oracle import spn_model as sm
    from xspn.serialization.binary.BinarySerialization import BinaryDeserializer
    from spnc.structure import node_kind, topological_nodes
    for name in ("nltcs", "plants", "speaker_FADG0", "NIPS10"):
        with quiet():
            got = BinaryDeserializer(os.path.join(GOLDEN, name + ".bin")).deserialize_from_file()
        root = got.root if hasattr(got, "root") else got.graph.root
        want = sm.load_model(os.path.join(GOLDEN, name + ".bin"))
        nodes = topological_nodes(root)
        assert len(nodes) == len(sm.reachable_topo(want))
        assert sorted(node_kind(n) for n in nodes) == sorted(sm.KIND_NAMES[n.kind] for n in sm.reachable_topo(want))


def test_writer_output_is_read_identically_by_the_oracle_reader(tmp_path):
    from spnc import synthetic as syn
    from oracle import spn_model as sm
    q = sm.load(write_query(syn.c4_spn(), "float32", str(tmp_path / "q.bin"), marginal=True, batch_size=99, name="c4"))
    assert (q.batch_size, q.support_marginal, q.model.name, q.model.feature_type, q.model.num_features) == (99, True, "c4", "float32", 32)
    assert len(q.model.nodes) == 8881 and sorted(q.model.scope) == list(range(32))


def test_invalid_spn_is_refused_before_serialization(tmp_path):
    from spnc.structure import Categorical, Product, Sum
    from xspn.serialization.binary.BinarySerialization import BinarySerializer
    from xspn.structure.Model import SPNModel
    overlapping = Product(children=[Categorical(p=[.5, .5], scope=0), Categorical(p=[.5, .5], scope=0)])
    incomplete = Sum(weights=[.5, .5], children=[Categorical(p=[.5, .5], scope=0), Categorical(p=[.5, .5], scope=1)])
    for bad in (overlapping, incomplete):
        with pytest.raises(AssertionError, match="SPN invalid before serialization"):
            BinarySerializer(str(tmp_path / "x.bin")).serialize_to_file(SPNModel(bad, "int32", "bad"))
    with pytest.raises(NotImplementedError):
        BinarySerializer(str(tmp_path / "x.bin")).serialize_to_file("not a model")


def test_hipcompiler_argument_checks(native):
    """Same errors as python-interface/spnc/gpu.py:172-175,205-208 of the reference."""
    from spnc import synthetic as syn
    from spnc.hip import HIPCompiler
    c = HIPCompiler()
    with pytest.raises(RuntimeError, match="Input is not an numpy array"):
        c.log_likelihood(syn.c1_spn(), [[0, 1, 2, 0, 1, 2]])
    with pytest.raises(RuntimeError, match="Input must be a two-dimensional array"):
        c.log_likelihood(syn.c1_spn(), np.zeros(6, dtype=np.int32))
    with quiet():
        k = c.compile_ll(syn.c1_spn(), "int32", supportMarginal=False)
    assert os.path.isfile(k.fileName()) and k.kernelName() == "spn_hip" and k.batchSize() == 64
    with pytest.raises(RuntimeError, match="Input is not an numpy array"):
        c.execute(k, "nope")
    with pytest.raises(RuntimeError, match="Input must be a two-dimensional array"):
        c.execute(k, np.zeros((2, 3, 6), dtype=np.int32))
    with pytest.raises(RuntimeError, match="does not match the kernel's feature type int32"):
        c.execute(k, np.zeros((4, 6), dtype=np.float64))
    with pytest.raises(RuntimeError, match=r"Input must have shape \[4, 6\]"):
        c.execute(k, np.zeros((4, 5), dtype=np.int32))
    os.remove(k.fileName())
    with quiet(), pytest.raises(RuntimeError, match="floating-point to support marginal"):
        c.compile_ll(syn.c1_spn(), "int32")  # supportMarginal defaults to True, as in the reference
    with quiet(), pytest.raises(RuntimeError, match="Unknown compile option"):
        HIPCompiler(notAnOption=1).compile_ll(syn.c1_spn(), "float64")
    assert HIPCompiler.isAvailable() in (True, False)
    assert native.SPNCompiler.isTargetSupported("CUDA") is False


def test_cpu_baseline_kernel_follows_the_oracle(tmp_path):
    from oracle import cgen, evaluate as ev
    from spnc import synthetic as syn
    from spnc.structure import Gaussian, Product, Sum
    small = Sum(weights=[0.3, 0.2, 0.5], children=[Product(children=[Gaussian(0.1 * i, 0.5 + 0.1 * j, scope=j) for j in range(3)])
                                                  for i in range(3)])
    for spn, dtype, X, marginal in ((syn.c1_spn(), "int32", syn.c1_inputs(1000), False),
                                    (small, "float32", np.random.default_rng(0).standard_normal((1000, 3)).astype(np.float32), True)):
        if marginal:
            X[::7, 1] = np.nan
        m = oracle_model(spn, dtype)
        so, _ = cgen.build(m, marginal, workdir=str(tmp_path / dtype))
        got = cgen.load(so, dtype)(X)
        assert np.abs(got - ev.ll_reforder(m, X, np.float32, marginal=marginal)).max() < 2e-6


def test_bench_refuses_more_than_one_gpu():
    """The benchmark measures one GPU; asking for more exits with a message instead of a number."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in (r.stdout + r.stderr)
