"""Seeded synthetic SPNs and input batches for the five benchmark configurations.

Each ``cN_spn()`` returns the root of an SPN built from ``spnc.structure`` classes and each
``cN_inputs(n)`` the matching ``[n, F]`` array; seeds are fixed so that tests, the benchmark and
the CPU baseline all see the same network and data.

C1  the 6-leaf Categorical product of the reference's README (README.md:57-63 of the reference,
    also python-interface/test/cuda/test_cuda_categorical.py:27-33), int32 inputs in {0,1,2}.
C2  random sum/product tree over 16 Gaussian features, depth 6, sums with 4 Dirichlet(1) children.
C3  discrete SPN over 100 features: Categorical (2-5 categories) and Histogram (8 integer bins) leaves.
C4  RAT-SPN-style region graph over 32 Gaussian features, 10 repetitions (interpreter-sized).
C5  C2 with 20 % of the inputs set to NaN (marginalised).
"""
import numpy as np

from .structure import Categorical, Gaussian, Histogram, Product, Sum

C1_PROBS = [[.35, .55, .1], [.25, .625, .125], [.5, .2, .3], [.6, .15, .25], [.7, .11, .19], [.8, .14, .06]]


def c1_spn():
    return Product(children=[Categorical(p=p, scope=i) for i, p in enumerate(C1_PROBS)])


def c1_inputs(n, seed=1):
    return np.random.default_rng(seed).integers(0, 3, size=(n, 6), dtype=np.int32)


def c2_spn(num_features=16, depth=6, sum_children=4, seed=2):
    """Alternating sum/product layers from a sum root. A product halves its scope; the last
    product layer factorises its scope completely into univariate Gaussian leaves."""
    rng = np.random.default_rng(seed)

    def leaf(f):
        return Gaussian(mean=float(rng.normal()), stdev=float(rng.uniform(0.1, 2.0)), scope=int(f))

    def make_sum(scope, level):
        weights = rng.dirichlet(np.ones(sum_children))
        return Sum(weights=[float(w) for w in weights], children=[make_product(scope, level + 1) for _ in range(sum_children)])

    def make_product(scope, level):
        if level >= depth - 1 or len(scope) <= 2:
            return Product(children=[leaf(f) for f in scope])
        half = len(scope) // 2
        return Product(children=[make_sum(scope[:half], level + 1), make_sum(scope[half:], level + 1)])

    return make_sum(list(range(num_features)), 0)


def c2_inputs(n, num_features=16, seed=102):
    return np.random.default_rng(seed).standard_normal((n, num_features)).astype(np.float32)


def c5_inputs(n, num_features=16, seed=102, nan_seed=105, nan_fraction=0.2):
    x = c2_inputs(n, num_features, seed)
    mask = np.random.default_rng(nan_seed).random(x.shape) < nan_fraction
    x[mask] = np.nan
    return x


def c3_domains(num_features=100, seed=3):
    """Per feature: ('hist', 8) or ('cat', d) with d in 2..5."""
    rng = np.random.default_rng(seed)
    doms = []
    for _ in range(num_features):
        if rng.random() < 0.3:
            doms.append(("hist", 8))
        else:
            doms.append(("cat", int(rng.integers(2, 6))))
    return doms


def c3_spn(num_features=100, seed=3, sum_levels=2, inner_fan_in=(2, 9)):
    """Discrete SPN over `num_features` features: sums and products alternate from a sum root; every sum draws
    2 to 8 children with Dirichlet(1) weights; a product splits its scope into 2 or 3 random parts, one sum (or a
    single leaf) per part, until `sum_levels` levels of sums exist or the scope is small, where the product factorises
    into the leaves of its scope. Defaults: 1651 nodes (10 sums, 40 products, 1601 leaves).
    ``c3_deep_spn`` is the deeper, narrower variant (68 sums of 2 to 4 children, 2640 nodes)."""
    doms = c3_domains(num_features, seed)
    rng = np.random.default_rng(seed + 1000)
    max_level = 2 * sum_levels - 1

    def leaf(f):
        kind, d = doms[f]
        p = rng.dirichlet(np.ones(d))
        if kind == "hist":
            return Histogram(breaks=list(range(d + 1)), densities=[float(v) for v in p], bin_repr_points=[i + 0.5 for i in range(d)],
                             scope=int(f))
        return Categorical(p=[float(v) for v in p], scope=int(f))

    def make_product(scope, level):
        if len(scope) <= 6 or level >= max_level:
            return Product(children=[leaf(f) for f in scope])
        parts = int(rng.integers(2, 4))
        perm = [scope[i] for i in rng.permutation(len(scope))]
        cuts = np.array_split(np.array(perm), parts)
        children = []
        for part in cuts:
            part = sorted(int(v) for v in part)
            children.append(leaf(part[0]) if len(part) == 1 else make_sum(part, level + 1))
        return Product(children=children)

    def make_sum(scope, level):
        k = int(rng.integers(2, 9)) if level == 0 else int(rng.integers(*inner_fan_in))
        weights = rng.dirichlet(np.ones(k))
        return Sum(weights=[float(w) for w in weights], children=[make_product(scope, level + 1) for _ in range(k)])

    return make_sum(list(range(num_features)), 0)


def c3_deep_spn(num_features=100, seed=3):
    """Three levels of sums, inner sums of 2 or 3 children: 68 sums, 174 products, 2398 leaves."""
    return c3_spn(num_features, seed, sum_levels=3, inner_fan_in=(2, 4))


def c3_inputs(n, num_features=100, seed=3, data_seed=103):
    doms = c3_domains(num_features, seed)
    rng = np.random.default_rng(data_seed)
    x = np.empty((n, num_features), dtype=np.int32)
    for j, (_, d) in enumerate(doms):
        x[:, j] = rng.integers(0, d, size=n, dtype=np.int32)
    return x


def c4_spn(num_features=32, repetitions=10, split_depth=4, sums_per_region=8, leaves_per_region=4, seed=4):
    """RAT-SPN-style: per repetition a random balanced binary region tree of the given depth;
    leaf regions hold `leaves_per_region` fully factorised Gaussian distributions; an inner region
    holds `sums_per_region` sums over all pairwise products of its two children's nodes; the root
    is one sum over the root-region nodes of all repetitions."""
    rng = np.random.default_rng(seed)

    def region(scope, level):
        if level == split_depth:
            nodes = []
            for _ in range(leaves_per_region):
                nodes.append(Product(children=[
                    Gaussian(mean=float(rng.normal()), stdev=float(rng.uniform(0.2, 1.5)), scope=int(f)) for f in scope]))
            return nodes
        half = len(scope) // 2
        left, right = region(scope[:half], level + 1), region(scope[half:], level + 1)
        products = [Product(children=[a, b]) for a in left for b in right]
        sums = []
        for _ in range(sums_per_region):
            w = rng.dirichlet(np.ones(len(products)))
            sums.append(Sum(weights=[float(v) for v in w], children=products))
        return sums

    roots = []
    for _ in range(repetitions):
        perm = [int(v) for v in rng.permutation(num_features)]
        roots.extend(region(perm, 0))
    w = rng.dirichlet(np.ones(len(roots)))
    return Sum(weights=[float(v) for v in w], children=roots)


def c4_inputs(n, num_features=32, seed=104):
    return np.random.default_rng(seed).standard_normal((n, num_features)).astype(np.float32)


CONFIGS = {
    "c1": dict(spn=c1_spn, inputs=c1_inputs, dtype="int32", marginal=False, n=64 * 2 ** 20, features=6,
               desc="README product of 6 Categorical(3) leaves, int32 [N,6]"),
    "c2": dict(spn=c2_spn, inputs=c2_inputs, dtype="float32", marginal=False, n=16 * 2 ** 20, features=16,
               desc="random depth-6 sum/product tree, 16 Gaussian features, float32 [N,16]"),
    "c3": dict(spn=c3_spn, inputs=c3_inputs, dtype="int32", marginal=False, n=8 * 2 ** 20, features=100,
               desc="discrete SPN, 100 features, Categorical + Histogram leaves, int32 [N,100]"),
    "c3_deep": dict(spn=c3_deep_spn, inputs=c3_inputs, dtype="int32", marginal=False, n=8 * 2 ** 20, features=100,
                    desc="discrete SPN, 100 features, three levels of narrow sums (2640 nodes), int32 [N,100]"),
    "c4": dict(spn=c4_spn, inputs=c4_inputs, dtype="float32", marginal=False, n=4 * 2 ** 20, features=32,
               desc="RAT-SPN-style region graph, 32 Gaussian features, 10 repetitions, float32 [N,32]"),
    "c5": dict(spn=c2_spn, inputs=c5_inputs, dtype="float32", marginal=True, n=16 * 2 ** 20, features=16,
               desc="C2 with 20% NaN inputs (marginal query), float32 [N,16]"),
}
