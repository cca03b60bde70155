"""CPU evaluators for joint log-likelihood (test infrastructure, see oracle/__init__.py).

``ll_closed_f64``  textbook closed forms in float64 (SciPy ``norm.logpdf`` and
                   ``logsumexp``); the ground truth both the reference kernel
                   and the HIP kernels approximate.
``ll_reforder``    restates the reference's CPU kernel: operation order,
                   tree shapes and rounding points of
                   mlir/lib/Conversion/HiSPNtoLoSPN/NodePatterns.cpp:17-88 and
                   mlir/lib/Conversion/LoSPNtoCPU/NodePatterns.cpp:216-529,
                   evaluated with NumPy in the requested compute type.
``ll_linear_f64``  the reference's linear-space float64 kernel
                   (NodePatterns.cpp:242-304 Gaussian, MulLowering/AddLowering,
                   root log at HiSPNtoLoSPN/NodePatterns.cpp:140-152).

Out-of-range indices of table leaves evaluate to log 0 = -inf (the reference's
GPU lowering, mlir/lib/Conversion/LoSPNtoGPU/GPUNodePatterns.cpp:385-395; its
CPU lowering reads out of bounds there).
"""
import math

import numpy as np

from . import spn_model as sm


def _columns(model, X):
    col = model.column_of()
    return {s: X[:, c] for s, c in col.items()}


def _to_index(x):
    """fptoui-like truncation for float features, identity for integer ones; NaN -> 0 (masked later)."""
    if np.issubdtype(x.dtype, np.floating):
        xi = np.where(np.isnan(x), 0.0, x)
        return np.trunc(xi).astype(np.int64)
    return x.astype(np.int64)


def histogram_table(node):
    """Flat table [0, maxUB) of densities, 0 in gaps (LoSPNtoCPU/NodePatterns.cpp:447-493)."""
    max_ub = max(node.breaks[1:]) if len(node.breaks) > 1 else 0
    if min(node.breaks[:-1]) < 0:
        raise ValueError("histogram with negative lower bound")
    tab = np.zeros(max_ub, dtype=np.float64)
    for i in range(len(node.breaks) - 1):
        tab[node.breaks[i]:node.breaks[i + 1]] = node.densities[i]
    return tab


def _table_lookup(tab, x):
    idx = _to_index(x)
    ok = (idx >= 0) & (idx < len(tab))
    safe = np.where(ok, idx, 0)
    return tab[safe], ok


def ll_closed_f64(model, X, marginal=True):
    from scipy.special import logsumexp
    from scipy.stats import norm

    cols = _columns(model, X)
    val = {}
    for n in sm.reachable_topo(model):
        if n.kind == sm.GAUSSIAN:
            x = cols[n.scope].astype(np.float64)
            r = norm.logpdf(x, n.mean, n.stddev)
        elif n.kind in (sm.CATEGORICAL, sm.HISTOGRAM):
            x = cols[n.scope]
            tab = np.asarray(n.probabilities, dtype=np.float64) if n.kind == sm.CATEGORICAL else histogram_table(n)
            p, ok = _table_lookup(tab, x)
            with np.errstate(divide="ignore"):
                r = np.where(ok, np.log(p), -np.inf)
        elif n.kind == sm.PRODUCT:
            r = np.sum([val[c] for c in n.children], axis=0)
        elif n.kind == sm.SUM:
            with np.errstate(divide="ignore"):
                lw = np.log(np.asarray(n.weights, dtype=np.float64))
            r = logsumexp(np.stack([val[c] for c in n.children], axis=1) + lw[None, :], axis=1)
        else:
            raise ValueError(n.kind)
        if n.kind in (sm.GAUSSIAN, sm.CATEGORICAL, sm.HISTOGRAM) and marginal and np.issubdtype(cols[n.scope].dtype, np.floating):
            r = np.where(np.isnan(cols[n.scope]), 0.0, r)
        val[n.id] = r
    return np.asarray(val[model.root], dtype=np.float64)


def _balanced(items, combine):
    """Balanced binary tree with pivot ceil(k/2), left first (HiSPNtoLoSPN/NodePatterns.cpp:17-40,49-88)."""
    if len(items) == 1:
        return items[0]
    if len(items) == 2:
        return combine(items[0], items[1])
    pivot = (len(items) + 1) // 2
    return combine(_balanced(items[:pivot], combine), _balanced(items[pivot:], combine))


def _logadd(x, y):
    """a + log1p(exp(b - a)), a = x if x > y else y (LoSPNtoCPU/NodePatterns.cpp:216-240)."""
    gt = x > y
    a = np.where(gt, x, y)
    b = np.where(gt, y, x)
    with np.errstate(invalid="ignore", over="ignore"):
        return a + np.log1p(np.exp(b - a))


def ll_reforder(model, X, dtype=np.float32, marginal=True):
    T = np.dtype(dtype).type
    cols = _columns(model, X)
    val = {}
    for n in sm.reachable_topo(model):
        if n.kind == sm.GAUSSIAN:
            x_in = cols[n.scope]
            x = x_in.astype(T)  # uitofp / fpext / fptrunc
            coef = T(-math.log(n.stddev) + -0.5 * math.log(2 * math.pi))
            den = T(-(1.0 / (2.0 * n.stddev * n.stddev)))
            d = x - T(n.mean)
            r = coef + (d * d) * den
            if marginal:
                r = np.where(np.isnan(x), T(0), r)
        elif n.kind in (sm.CATEGORICAL, sm.HISTOGRAM):
            x = cols[n.scope]
            p = np.asarray(n.probabilities, dtype=np.float64) if n.kind == sm.CATEGORICAL else histogram_table(n)
            with np.errstate(divide="ignore"):
                tab = np.log(p).astype(T)  # log in double, rounded to the compute type
            v, ok = _table_lookup(tab, x)
            r = np.where(ok, v, T(-np.inf))
            if marginal and np.issubdtype(x.dtype, np.floating):
                r = np.where(np.isnan(x), T(0), r)
        elif n.kind == sm.PRODUCT:
            r = _balanced([val[c] for c in n.children], lambda a, b: a + b)
        elif n.kind == sm.SUM:
            with np.errstate(divide="ignore"):
                terms = [val[c] + T(math.log(w)) if w > 0 else val[c] + T(-np.inf) for c, w in zip(n.children, n.weights)]
            r = _balanced(terms, _logadd)
        else:
            raise ValueError(n.kind)
        val[n.id] = r.astype(T)
    return val[model.root]


def ll_linear_f64(model, X, marginal=True):
    cols = _columns(model, X)
    val = {}
    for n in sm.reachable_topo(model):
        if n.kind == sm.GAUSSIAN:
            x = cols[n.scope].astype(np.float64)
            var = n.stddev * n.stddev
            coef = 1.0 / math.sqrt(2.0 * math.pi * var)
            den = -1.0 / (2.0 * var)
            d = x - n.mean
            r = coef * np.exp((d * d) * den)
            if marginal:
                r = np.where(np.isnan(x), 1.0, r)
        elif n.kind in (sm.CATEGORICAL, sm.HISTOGRAM):
            x = cols[n.scope]
            tab = np.asarray(n.probabilities, dtype=np.float64) if n.kind == sm.CATEGORICAL else histogram_table(n)
            v, ok = _table_lookup(tab, x)
            r = np.where(ok, v, 0.0)
            if marginal and np.issubdtype(x.dtype, np.floating):
                r = np.where(np.isnan(x), 1.0, r)
        elif n.kind == sm.PRODUCT:
            r = _balanced([val[c] for c in n.children], lambda a, b: a * b)
        elif n.kind == sm.SUM:
            r = _balanced([val[c] * w for c, w in zip(n.children, n.weights)], lambda a, b: a + b)
        val[n.id] = r
    with np.errstate(divide="ignore"):
        return np.log(val[model.root])
