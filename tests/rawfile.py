"""Writes query files field by field (no validation), to feed the compiler malformed or unusual inputs."""
from xspn.serialization.binary.BinarySerialization import _Segment

KIND = {"product": 0, "sum": 1, "histogram": 2, "gaussian": 3, "categorical": 4}


def write(path, nodes, scope, feature_type="float64", root=0, marginal=False, num_features=None, name="raw", batch_size=8,
          header_kind=1, with_joint=True, with_model=True, joint_data_words=1):
    seg = _Segment()
    header = seg.new_struct(0, 1, 1)
    seg.put(header, 0, "H", header_kind)
    if header_kind == 0:
        _model(seg, header + 1, nodes, scope, feature_type, root, num_features, name)
    else:
        q = seg.new_struct(header + 1, 2, 1)
        seg.put(q, 0, "i", batch_size)
        seg.put(q, 8, "d", 0.02)
        if with_joint:
            joint = seg.new_struct(q + 2, joint_data_words, 1)
            if joint_data_words:
                seg.put(joint, 0, "B", 1 if marginal else 0)
            if with_model:
                _model(seg, joint + joint_data_words, nodes, scope, feature_type, root, num_features, name)
    with open(path, "wb") as f:
        f.write(seg.stream())
    return path


def _model(seg, at, nodes, scope, feature_type, root, num_features, name):
    m = seg.new_struct(at, 1, 4)
    seg.put(m, 0, "i", root)
    seg.put(m, 4, "i", len(scope) if num_features is None else num_features)
    seg.text(m + 1, name)
    seg.text(m + 2, feature_type)
    seg.prim_list(m + 3, "i", 4, list(scope))
    slots = seg.struct_list(m + 4, len(nodes), 1, 1)
    for n, at in zip(nodes, slots):
        seg.put(at, 0, "i", n["id"])
        seg.put(at, 4, "B", 1 if n["id"] == root else 0)
        seg.put(at, 6, "H", KIND[n["kind"]])
        if n["kind"] == "product":
            b = seg.new_struct(at + 1, 0, 1)
            seg.prim_list(b, "i", 4, n["children"])
        elif n["kind"] == "sum":
            b = seg.new_struct(at + 1, 0, 2)
            seg.prim_list(b, "i", 4, n["children"])
            seg.prim_list(b + 1, "d", 5, n["weights"])
        elif n["kind"] == "histogram":
            b = seg.new_struct(at + 1, 1, 3)
            seg.put(b, 4, "i", n["scope"])
            seg.prim_list(b + 1, "i", 4, n["breaks"])
            seg.prim_list(b + 2, "d", 5, n["densities"])
            seg.prim_list(b + 3, "d", 5, [])
        elif n["kind"] == "gaussian":
            b = seg.new_struct(at + 1, 3, 0)
            seg.put(b, 0, "d", n["mean"])
            seg.put(b, 8, "d", n["stddev"])
            seg.put(b, 16, "i", n["scope"])
        else:
            b = seg.new_struct(at + 1, 1, 1)
            seg.put(b, 0, "i", n["scope"])
            seg.prim_list(b + 1, "d", 5, n["p"])


def cat(i, scope, p=(0.5, 0.5)):
    return {"id": i, "kind": "categorical", "scope": scope, "p": list(p)}


def gauss(i, scope, mean=0.0, stddev=1.0):
    return {"id": i, "kind": "gaussian", "scope": scope, "mean": mean, "stddev": stddev}


def hist(i, scope, breaks=(0, 1, 2), densities=(0.5, 0.5)):
    return {"id": i, "kind": "histogram", "scope": scope, "breaks": list(breaks), "densities": list(densities)}


def prod(i, children):
    return {"id": i, "kind": "product", "children": list(children)}


def wsum(i, children, weights):
    return {"id": i, "kind": "sum", "children": list(children), "weights": list(weights)}
