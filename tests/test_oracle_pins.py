"""Pins the CPU oracle (oracle/) against everything the reference's own files fix for this path."""
import json
import math
import os

import numpy as np
import pytest

from conftest import GOLDEN, load_golden, oracle_model
from oracle import c_oracle, evaluate as ev, spn_model as sm

# Known answers in the comments of the reference's CLI driver, execute/src/main.cpp:32-52.
KNOWN = {
    "mini-example": (np.array([[0, 0], [0, 1], [1, 0], [1, 1]], dtype=np.uint32), [-1.44445, -2.65748, -0.670163, -1.70169]),
    "categorical-example": (np.array([[0, 0], [0, 1], [1, 0], [1, 1]], dtype=np.uint8), [-2.43612, -1.51983, -1.98413, -1.06784]),
    "gaussian-example": (np.array([[0.5, 0.125], [0.125, 0.5], [0.25, 0.25], [0.325, 0.275]], dtype=np.float32),
                         [-0.451583, -1.6469, -0.607833, -0.646895]),
}


@pytest.mark.parametrize("name", sorted(KNOWN))
def test_known_answers_of_reference_cli(name):
    X, expected = KNOWN[name]
    m = sm.load_model(os.path.join(GOLDEN, name + ".bin"))
    # printed with 6 significant digits
    for got in (ev.ll_closed_f64(m, X, marginal=False), ev.ll_reforder(m, X, np.float32, marginal=False),
                ev.ll_linear_f64(m, X, marginal=False), c_oracle.ll_f32(m, X, marginal=False)):
        assert np.allclose(got, expected, rtol=0, atol=6e-6)


@pytest.mark.parametrize("name,f32_bound", [("NIPS5", 5e-6), ("nltcs", 1e-5), ("plants", 4e-5)])
def test_golden_outputs(name, f32_bound):
    X, ref = load_golden(name)
    m = sm.load_model(os.path.join(GOLDEN, name + ".bin"))
    assert np.abs(ev.ll_closed_f64(m, X, marginal=False) - ref).max() < 1e-12
    assert np.abs(ev.ll_reforder(m, X, np.float64, marginal=False) - ref).max() < 1e-12
    assert np.abs(ev.ll_linear_f64(m, X, marginal=False) - ref).max() < 1e-11
    assert np.abs(ev.ll_reforder(m, X, np.float32, marginal=False) - ref).max() < f32_bound
    assert np.abs(c_oracle.ll_f32(m, X, marginal=False) - ref).max() < f32_bound


def test_fixture_census():
    # node counts by kind as decoded from the reference's files: [product, sum, histogram, gaussian, categorical]
    expect = {
        "categorical-example": (3, [1, 0, 0, 0, 2]), "gaussian-example": (3, [1, 0, 0, 2, 0]), "mini-example": (7, [2, 1, 4, 0, 0]),
        "categorical6": (7, [1, 0, 0, 0, 6]), "gaussian10": (11, [1, 0, 0, 10, 0]), "histogram4": (7, [2, 1, 4, 0, 0]),
        "NIPS5": (13, [2, 1, 10, 0, 0]), "NIPS10": (31, [5, 2, 24, 0, 0]), "nltcs": (3641, [2232, 161, 0, 1248, 0]),
        "plants": (1297, [549, 127, 0, 621, 0]), "speaker_FADG0": (1378, [51, 1, 0, 1326, 0]),
        "fashion_mnist": (47466, [7635, 631, 0, 39200, 0]),
    }
    for name, (total, kinds) in expect.items():
        m = sm.load_model(os.path.join(GOLDEN, name + ".bin"))
        got = [0] * 5
        for n in m.nodes:
            got[n.kind] += 1
        assert (len(m.nodes), got) == (total, kinds), name
    q = sm.load(os.path.join(GOLDEN, "mini-example.bin"))
    assert isinstance(q, sm.Query) and q.model.scope == [1, 2] and q.model.feature_type == "uint32" and not q.support_marginal
    assert isinstance(sm.load(os.path.join(GOLDEN, "nltcs.bin")), sm.Model)
    assert sm.load(os.path.join(GOLDEN, "categorical6.bin")).batch_size == 12


def test_bin_matches_json_twin():
    """execute/examples/NIPS5.json describes the same model as NIPS5.bin in JSON."""
    doc = json.load(open(os.path.join(GOLDEN, "NIPS5.json")))
    m = sm.load_model(os.path.join(GOLDEN, "NIPS5.bin"))

    def walk(node, out):
        (kind, body), = node.items()
        if kind == "Histogram":
            out.append((body["scope"][0] if isinstance(body["scope"], list) else body["scope"], body["breaks"], body["densities"]))
        for c in body.get("children", []):
            walk(c, out)

    hists = []
    walk(doc, hists)
    by_key = {}
    for n in m.nodes:
        if n.kind == sm.HISTOGRAM:
            by_key.setdefault((n.scope, tuple(n.breaks)), []).append(n.densities)
    assert len(hists) == 10
    for scope, breaks, dens in hists:
        cands = [d for (s, b), ds in by_key.items() for d in ds if tuple(breaks) == b]
        assert any(np.allclose(dens, d) for d in cands), scope


def test_filecheck_constants():
    """f32 constants pinned by mlir/test/lowering/lospn-to-cpu/lower-to-cpu-nodes-scalar-log.mlir:3-7,133-160."""
    f32 = lambda v: np.asarray(v, dtype=np.float32)
    assert np.array_equal(np.log([.35, .55, .1]).astype(np.float32), f32([-1.04982209, -0.597836971, -2.30258512]))
    assert np.array_equal(np.log([.25, .625, .125]).astype(np.float32), f32([-1.38629436, -0.470003635, -2.07944155]))
    from spnc.structure import Gaussian, Product
    m = oracle_model(Product(children=[Gaussian(0.0, 1.0, scope=0), Gaussian(0.25, 0.1, scope=1)]), "float32")
    X = np.array([[0.0, 0.25]], dtype=np.float32)  # at the means the leaf value is its coefficient
    coef = np.float32(-0.918938517) + np.float32(1.38364661)
    assert ev.ll_reforder(m, X, np.float32, marginal=False)[0] == coef
    # denominators -0.5 and -50: one unit away from the mean adds exactly den
    X1 = np.array([[1.0, 0.25], [0.0, 1.25]], dtype=np.float32)
    got = ev.ll_reforder(m, X1, np.float32, marginal=False)
    assert np.allclose(got - coef, [-0.5, -50.0], rtol=1e-6)


def test_sum_tree_order():
    """k=5 weighted sum lowers to ((t0+t1)+t2)+(t3+t4), mlir/test/lowering/hispn-to-lospn/lower-to-lospn-sum.mlir:27-41."""
    shape = ev._balanced(list("abcde"), lambda x, y: f"({x}{y})")
    assert shape == "(((ab)c)(de))"
    assert ev._balanced(list("abcdef"), lambda x, y: f"({x}{y})") == "(((ab)c)((de)f))"


def test_normalisation_and_marginal_invariants():
    from spnc import synthetic as syn
    m = oracle_model(syn.c1_spn(), "float64")
    states = np.array(np.meshgrid(*[range(3)] * 6)).reshape(6, -1).T.astype(np.float64)
    for f in (ev.ll_closed_f64, lambda mm, X, marginal: ev.ll_reforder(mm, X, np.float64, marginal)):
        assert abs(np.exp(f(m, states, marginal=True)).sum() - 1.0) < 1e-12
    # all-NaN row: every leaf marginalised, LL = log 1 = 0
    nan_row = np.full((1, 6), np.nan)
    assert ev.ll_closed_f64(m, nan_row)[0] == 0.0 and ev.ll_reforder(m, nan_row, np.float32)[0] == 0.0
    # marginalising feature 2 of a product drops its term
    X = states[:50].copy()
    full = ev.ll_closed_f64(m, X)
    X[:, 2] = np.nan
    dropped = full - np.log(np.array(syn.C1_PROBS[2]))[states[:50, 2].astype(int)]
    assert np.allclose(ev.ll_closed_f64(m, X), dropped, atol=1e-13)
    assert np.allclose(ev.ll_reforder(m, X, np.float32), dropped, atol=2e-6)
    # a mixture: sum over a binary feature of exp(LL) of the marginalised remainder
    m2 = oracle_model(syn.c2_spn(), "float32")
    Xn = np.full((3, 16), np.nan, dtype=np.float32)
    assert np.allclose(ev.ll_closed_f64(m2, Xn), 0.0, atol=1e-12)


@pytest.mark.parametrize("cfg", ["c2", "c3", "c5"])
def test_restatements_agree_on_synthetic_spns(cfg):
    from spnc import synthetic as syn
    c = syn.CONFIGS[cfg]
    m = oracle_model(c["spn"](), c["dtype"])
    X = c["inputs"](300)
    f64 = ev.ll_closed_f64(m, X, marginal=c["marginal"])
    f32 = ev.ll_reforder(m, X, np.float32, marginal=c["marginal"])
    cc = c_oracle.ll_f32(m, X, marginal=c["marginal"])
    lin = ev.ll_linear_f64(m, X, marginal=c["marginal"])
    assert np.abs(f32 - f64).max() < 1e-4 and np.abs(cc - f64).max() < 1e-4
    assert np.abs(cc - f32).max() < 3e-5
    ok = np.isfinite(lin)
    assert ok.all() and np.abs(lin - f64).max() < 1e-9


def test_out_of_range_and_gaps():
    from spnc.structure import Categorical, Histogram, Product
    spn = Product(children=[Categorical(p=[0.2, 0.8], scope=0),
                            Histogram(breaks=[0, 2, 4], densities=[0.25, 0.25], bin_repr_points=[1, 3], scope=1)])
    m = oracle_model(spn, "float64")
    X = np.array([[0, 1], [1, 3], [2, 0], [0, 4], [-1, 0], [0.9, 1.9]])
    want = [math.log(0.2 * 0.25), math.log(0.8 * 0.25), -math.inf, -math.inf, -math.inf, math.log(0.2 * 0.25)]
    for got in (ev.ll_closed_f64(m, X, marginal=False), ev.ll_reforder(m, X, np.float32, marginal=False),
                c_oracle.ll_f32(m, X, marginal=False)):
        assert np.allclose(got, want, rtol=1e-6)
