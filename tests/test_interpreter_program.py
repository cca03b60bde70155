"""The interpreter's node program, checked on the CPU: a bounds-checked emulator (tests/interp_emulator.cpp)
builds the program with the library's own sources, verifies its structural invariants and evaluates it;
results must agree with the oracle. No GPU involved."""
import os
import subprocess

import numpy as np
import pytest

from conftest import GOLDEN, ROOT, load_golden, model_as_query, oracle_model, write_query
from oracle import evaluate as ev, spn_model as sm

CSRC = os.path.join(ROOT, "spn-compiler_amd", "csrc")


@pytest.fixture(scope="module")
def emulator(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("emu") / "interp_emulator")
    srcs = [os.path.join(CSRC, f) for f in ("spn_graph.cpp", "capnp_reader.cpp", "interp_program.cpp", "options.cpp")]
    subprocess.run(["g++", "-O1", "-std=c++17", "-o", exe, os.path.join(ROOT, "tests", "interp_emulator.cpp")] + srcs, check=True)

    def run(query, X, *options):
        path = query + ".f64"
        np.ascontiguousarray(X, dtype=np.float64).tofile(path)
        r = subprocess.run([exe, query, path, str(X.shape[0])] + list(options), capture_output=True, text=True)
        assert r.returncode == 0, r.stderr
        return np.array([float(v) for v in r.stdout.split()], dtype=np.float64), r.stderr

    return run


@pytest.mark.parametrize("cfg", ["c1", "c2", "c3", "c4", "c5"])
def test_program_of_benchmark_configuration(emulator, tmp_path, cfg):
    from spnc import synthetic as syn
    c = syn.CONFIGS[cfg]
    spn = c["spn"]()
    q = write_query(spn, c["dtype"], str(tmp_path / "q.bin"), marginal=c["marginal"])
    X = c["inputs"](24)
    got, info = emulator(q, X)
    want = ev.ll_closed_f64(oracle_model(spn, c["dtype"]), X, marginal=c["marginal"])
    assert np.abs(got - want).max() < 1e-4
    if cfg == "c4":   # region graph: the 64-product layers are never materialised and the short pool fits four blocks per CU
        words = dict(zip(info.split()[::2], info.split()[1::2]))
        assert int(words["instructions"]) < 1000 and int(words["short"]) <= 40 < int(words["slots"])


@pytest.mark.parametrize("name", ["nltcs", "plants"])
def test_program_of_reference_models(emulator, tmp_path, name):
    X, ref = load_golden(name)
    q = model_as_query(os.path.join(GOLDEN, name + ".bin"), "float64", str(tmp_path / "q.bin"))
    got, _ = emulator(q, X[:40])
    assert np.abs(got - ref[:40]).max() < 1e-4
    got, _ = emulator(q, X[:10], "hip-log2-domain=false")
    assert np.abs(got - ref[:10]).max() < 1e-4


def test_program_of_the_47k_node_model_is_well_formed(emulator, tmp_path):
    q = model_as_query(os.path.join(GOLDEN, "fashion_mnist.bin"), "float64", str(tmp_path / "q.bin"))
    m = sm.load_model(q)
    X = np.random.default_rng(5).random((2, 784))
    got, _ = emulator(q, X)
    assert np.abs(got - ev.ll_closed_f64(m, X, marginal=False)).max() < 2e-3   # |LL| is in the thousands here
