"""ctypes front end of oracle/spn_oracle.c (test infrastructure, see oracle/__init__.py)."""
import ctypes
import os
import subprocess

import numpy as np

from . import spn_model as sm
from .evaluate import histogram_table

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "spn_oracle.so")


class _Flat(ctypes.Structure):
    _fields_ = [("num_nodes", ctypes.c_int), ("num_features", ctypes.c_int)] + [
        (name, ctypes.c_void_p) for name in ("kind", "column", "mean", "stddev", "table_off", "table_len", "tables", "child_off",
                                             "child_cnt", "children", "weights")]


def build():
    subprocess.run(["make", "-s", "-C", _HERE, "spn_oracle.so"], check=True)
    return _SO


def threads(set_to=None):
    """OpenMP threads the evaluator runs on; ``set_to`` changes the number for later calls."""
    if not os.path.isfile(_SO):
        build()
    lib = ctypes.CDLL(_SO)
    lib.spn_oracle_threads.restype = ctypes.c_int
    if set_to is not None:
        lib.spn_oracle_set_threads.argtypes = [ctypes.c_int]
        lib.spn_oracle_set_threads(int(set_to))
    return lib.spn_oracle_threads()


def ll_f32(model, X, marginal=True):
    """f32 log-likelihoods in the reference's operation order, evaluated by the C restatement."""
    if not os.path.isfile(_SO):
        build()
    lib = ctypes.CDLL(_SO)
    lib.spn_oracle_f32.argtypes = [ctypes.POINTER(_Flat), ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p]
    nodes = sm.reachable_topo(model)
    index = {n.id: i for i, n in enumerate(nodes)}
    col = model.column_of()
    N = len(nodes)
    kind = np.zeros(N, np.int32)
    column = np.zeros(N, np.int32)
    mean = np.zeros(N)
    std = np.ones(N)
    toff = np.zeros(N, np.int32)
    tlen = np.zeros(N, np.int32)
    coff = np.zeros(N, np.int32)
    ccnt = np.zeros(N, np.int32)
    tables, children, weights = [], [], []
    for i, n in enumerate(nodes):
        kind[i] = n.kind
        if n.kind in (sm.GAUSSIAN, sm.CATEGORICAL, sm.HISTOGRAM):
            column[i] = col[n.scope]
        if n.kind == sm.GAUSSIAN:
            mean[i], std[i] = n.mean, n.stddev
        elif n.kind in (sm.CATEGORICAL, sm.HISTOGRAM):
            t = list(n.probabilities) if n.kind == sm.CATEGORICAL else list(histogram_table(n))
            toff[i], tlen[i] = len(tables), len(t)
            tables.extend(t)
        else:
            coff[i], ccnt[i] = len(children), len(n.children)
            children.extend(index[c] for c in n.children)
            weights.extend(n.weights if n.kind == sm.SUM else [1.0] * len(n.children))
    tables = np.asarray(tables or [1.0], np.float64)
    children = np.asarray(children or [0], np.int32)
    weights = np.asarray(weights or [1.0], np.float64)
    keep = [kind, column, mean, std, toff, tlen, tables, coff, ccnt, children, weights]
    flat = _Flat(N, model.num_features, *[a.ctypes.data for a in keep])
    Xd = np.ascontiguousarray(X, dtype=np.float64)
    out = np.empty(Xd.shape[0], np.float32)
    rc = lib.spn_oracle_f32(ctypes.byref(flat), Xd.ctypes.data, Xd.shape[0], int(bool(marginal)), out.ctypes.data)
    if rc != 0:
        raise MemoryError("spn_oracle_f32 could not allocate its work buffers")
    return out
