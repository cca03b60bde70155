"""Plain SPN node classes with the attribute names of SPFlow's node types.

SPFlow (``spn.structure.Base`` / ``spn.structure.leaves``) is what the reference's Python front
end consumes (python-interface/spnc/gpu.py:79-119, xspn/xspn/serialization/binary/
BinarySerialization.py:139-247). These classes carry the same attributes (``children``,
``weights``, ``scope``, ``p``, ``mean``, ``stdev``, ``breaks``, ``densities``,
``bin_repr_points``) so that SPNs can be built where SPFlow is not installed; the serializer
accepts either kind of object.
"""


class Node:
    def __init__(self):
        self.id = 0
        self.scope = []


class Sum(Node):
    def __init__(self, weights=None, children=None):
        super().__init__()
        self.weights = list(weights) if weights is not None else []
        self.children = list(children) if children is not None else []


class Product(Node):
    def __init__(self, children=None):
        super().__init__()
        self.children = list(children) if children is not None else []


class Leaf(Node):
    def __init__(self, scope=None):
        super().__init__()
        if scope is not None:
            self.scope = list(scope) if isinstance(scope, (list, tuple)) else [scope]


class Gaussian(Leaf):
    def __init__(self, mean=None, stdev=None, scope=None):
        super().__init__(scope)
        self.mean = mean
        self.stdev = stdev


class Categorical(Leaf):
    def __init__(self, p=None, scope=None):
        super().__init__(scope)
        self.p = list(p) if p is not None else []


class Histogram(Leaf):
    def __init__(self, breaks, densities, bin_repr_points=None, scope=None, type_=None, meta_type=None):
        super().__init__(scope)
        self.breaks = list(breaks)
        self.densities = list(densities)
        self.bin_repr_points = list(bin_repr_points) if bin_repr_points is not None else []
        self.type = type_
        self.meta_type = meta_type


def node_kind(node):
    """'product' | 'sum' | 'histogram' | 'gaussian' | 'categorical' for these classes and SPFlow's."""
    for cls in type(node).__mro__:
        name = cls.__name__
        if name in ("Product", "Sum", "Histogram", "Gaussian", "Categorical"):
            return name.lower()
    raise NotImplementedError(f"No serialization defined for node {node} of type {type(node)}")


def leaf_scope(node):
    s = node.scope
    if isinstance(s, (list, tuple)):
        assert len(s) == 1, "Expecting leaf to be univariate"
        s = s[0]
    return int(s)


def topological_nodes(root):
    """All nodes reachable from root, children before parents, each once."""
    order, seen = [], set()
    stack = [(root, 0)]
    while stack:
        node, ci = stack.pop()
        if ci == 0 and id(node) in seen:
            continue
        children = getattr(node, "children", None) or []
        if ci < len(children):
            stack.append((node, ci + 1))
            if id(children[ci]) not in seen:
                stack.append((children[ci], 0))
            continue
        if id(node) not in seen:
            seen.add(id(node))
            order.append(node)
    return order


def rebuild_scopes_bottom_up(root):
    for n in topological_nodes(root):
        kind = node_kind(n)
        if kind in ("product", "sum"):
            scope = set()
            for c in n.children:
                scope.update(c.scope)
            n.scope = sorted(scope)
        elif not isinstance(n.scope, list):
            n.scope = [leaf_scope(n)]
    return root


def assign_ids(root, assigned=None):
    assigned = assigned if assigned is not None else {}
    next_id = max(assigned.values(), default=-1) + 1
    # Breadth-first from the root, as SPFlow numbers nodes: the root gets the lowest id.
    queue, seen = [root], {id(root)}
    while queue:
        n = queue.pop(0)
        if id(n) not in assigned:
            assigned[id(n)] = next_id
            next_id += 1
        n.id = assigned[id(n)]
        for c in getattr(n, "children", None) or []:
            if id(c) not in seen:
                seen.add(id(c))
                queue.append(c)
    return root


def is_valid(root):
    """Completeness (sum children share a scope) and decomposability (product children are disjoint)."""
    rebuild_scopes_bottom_up(root)
    for n in topological_nodes(root):
        kind = node_kind(n)
        if kind == "sum":
            if len(n.children) == 0 or len(n.children) != len(n.weights):
                return False
            if any(set(c.scope) != set(n.scope) for c in n.children):
                return False
        elif kind == "product":
            if len(n.children) == 0:
                return False
            total = sum(len(c.scope) for c in n.children)
            if total != len(n.scope):
                return False
    return True
