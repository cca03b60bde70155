"""Decode the reference's serialized SPN files into plain records (test infrastructure).

Field positions follow the schema
xspn/xspn/serialization/binary/capnproto/spflow.capnp:27-102 laid out by the
standard Cap'n Proto struct-layout rules; the semantic rules (sorted scope ->
input column, children referenced by id, default kernel name) follow
compiler/src/pipeline/steps/frontend/SPFlowToMLIRDeserializer.cpp:63-223.
"""
from dataclasses import dataclass, field
from typing import List, Optional

from .capnp_lite import Message, CapnpError

PRODUCT, SUM, HISTOGRAM, GAUSSIAN, CATEGORICAL = range(5)
KIND_NAMES = ["product", "sum", "histogram", "gaussian", "categorical"]


@dataclass
class Node:
    id: int
    kind: int
    root: bool = False
    children: List[int] = field(default_factory=list)
    weights: List[float] = field(default_factory=list)
    scope: int = -1
    mean: float = 0.0
    stddev: float = 1.0
    probabilities: List[float] = field(default_factory=list)
    breaks: List[int] = field(default_factory=list)
    densities: List[float] = field(default_factory=list)


@dataclass
class Model:
    root: int
    name: str
    feature_type: str
    num_features: int
    scope: List[int]
    nodes: List[Node]

    def by_id(self):
        return {n.id: n for n in self.nodes}

    def column_of(self):
        """scope value -> input column: ascending scope order (SPFlowToMLIRDeserializer.cpp:120-130)."""
        return {s: i for i, s in enumerate(sorted(self.scope))}


@dataclass
class Query:
    batch_size: int
    error_kind: int
    max_error: float
    support_marginal: bool
    model: Model


def _decode_node(s) -> Node:
    nid = s.get("i", 0)
    is_root = s.get_bool(32)
    which = s.get("H", 6)
    body = s.ptr_struct(0)
    n = Node(id=nid, kind=which, root=is_root)
    if which == PRODUCT:
        n.children = body.ptr_list(0).primitives("i")
    elif which == SUM:
        n.children = body.ptr_list(0).primitives("i")
        n.weights = body.ptr_list(1).primitives("d")
    elif which == HISTOGRAM:
        n.breaks = body.ptr_list(0).primitives("i")
        n.densities = body.ptr_list(1).primitives("d")
        n.scope = body.get("i", 4)
    elif which == GAUSSIAN:
        n.mean = body.get("d", 0)
        n.stddev = body.get("d", 8)
        n.scope = body.get("i", 16)
    elif which == CATEGORICAL:
        n.probabilities = body.ptr_list(0).primitives("d")
        n.scope = body.get("i", 0)
    else:
        raise CapnpError("unknown node kind %d" % which)
    return n


def _decode_model(m) -> Model:
    return Model(
        root=m.get("i", 0),
        num_features=m.get("i", 4),
        name=m.ptr_text(0),
        feature_type=m.ptr_text(1),
        scope=m.ptr_list(2).primitives("i"),
        nodes=[_decode_node(s) for s in m.ptr_list(3).structs()],
    )


def load(path):
    """Returns a Query or a bare Model depending on the Header union."""
    msg = Message.from_file(path)
    hdr = msg.root()
    which = hdr.get("H", 0)
    if which == 0:
        return _decode_model(hdr.ptr_struct(0))
    if which != 1:
        raise CapnpError("unknown header kind")
    q = hdr.ptr_struct(0)
    if not q.has_ptr(0):
        raise CapnpError("query without joint")
    j = q.ptr_struct(0)
    return Query(
        batch_size=q.get("i", 0),
        error_kind=q.get("H", 4),
        max_error=q.get("d", 8),
        support_marginal=j.get_bool(0),
        model=_decode_model(j.ptr_struct(0)),
    )


def load_model(path) -> Model:
    r = load(path)
    return r.model if isinstance(r, Query) else r


def reachable_topo(model: Model) -> List[Node]:
    """Nodes reachable from the root, children before parents, in first-visit DFS order."""
    by_id = model.by_id()
    order, seen = [], set()
    stack = [(model.root, 0)]
    while stack:
        nid, ci = stack.pop()
        n = by_id[nid]
        if ci == 0 and nid in seen:
            continue
        if ci < len(n.children):
            stack.append((nid, ci + 1))
            c = n.children[ci]
            if c not in seen:
                stack.append((c, 0))
            continue
        if nid not in seen:
            seen.add(nid)
            order.append(n)
    return order
