import contextlib
import io
import os
import sys
import tempfile

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")
for p in (os.path.join(ROOT, "spn-compiler_amd"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@contextlib.contextmanager
def quiet():
    """Silences the serializer's INFO prints."""
    with contextlib.redirect_stdout(io.StringIO()):
        yield


def write_query(spn, dtype, path, marginal=False, batch_size=64, name="spn_test"):
    """Serializes `spn` with the product's own xspn writer."""
    from xspn.serialization.binary.BinarySerialization import BinarySerializer
    from xspn.structure.Model import SPNModel
    from xspn.structure.Query import JointProbability
    with quiet():
        BinarySerializer(path).serialize_to_file(JointProbability(SPNModel(spn, dtype, name), batchSize=batch_size,
                                                                  supportMarginal=marginal))
    return path


def oracle_model(spn, dtype="float64"):
    """SPN -> oracle model record, through the wire format (writer of the product, reader of the oracle)."""
    from oracle import spn_model as sm
    with tempfile.TemporaryDirectory() as td:
        return sm.load_model(write_query(spn, dtype, os.path.join(td, "q.bin")))


def load_golden(name):
    """(inputs, expected) of a golden data set shipped with the reference's tests."""
    if name == "NIPS5":
        X = np.genfromtxt(os.path.join(GOLDEN, "NIPS5_inputdata.txt"), delimiter=";", dtype="float64")
        ref = np.genfromtxt(os.path.join(GOLDEN, "NIPS5_outputdata.txt"), dtype="float64")
    else:
        X = np.genfromtxt(os.path.join(GOLDEN, name + "_input.csv"), delimiter=",", dtype="float64")
        ref = np.genfromtxt(os.path.join(GOLDEN, name + "_output.csv"), delimiter=",", dtype="float64")
    return X, ref.reshape(-1)


@pytest.fixture(scope="session")
def native():
    """The ctypes binding of libspnc_hip.so; fails (does not skip) when the library is missing."""
    # PyTorch ships its own HIP runtime: when a test also uses torch tensors, torch has to
    # initialise first so that one runtime serves both it and libspnc_hip.so.
    try:
        import torch
        if torch.cuda.is_available():
            torch.cuda.init()
    except ImportError:
        pass
    from spnc import spncpy
    spncpy._load()
    return spncpy


def compile_query(native, path, **options):
    opts = {"target": "HIP", "use-log-space": "true"}
    opts.update({k.replace("_", "-"): str(v) for k, v in options.items()})
    with quiet():
        return native.SPNCompiler().compileQuery(path, opts)


def compile_spn(native, spn, dtype, marginal=False, **options):
    with tempfile.TemporaryDirectory() as td:
        return compile_query(native, write_query(spn, dtype, os.path.join(td, "q.bin"), marginal=marginal), **options)


def model_as_query(model_bin, dtype, path, marginal=False):
    """Wraps a serialized raw model (nltcs, plants, ...) into a joint query, as the reference's
    example tests do (python-interface/test/examples/nltcs/test_vector_nltcs.py:24-33)."""
    from xspn.serialization.binary.BinarySerialization import BinaryDeserializer
    with quiet():
        model = BinaryDeserializer(model_bin).deserialize_from_file()
    return write_query(model.root, dtype, path, marginal=marginal, name=model.name or "spn_test")
