"""Binary (Cap'n Proto) serialization of SPN models and queries without pycapnp or SPFlow.

Produces and consumes the wire format of the reference's schema
(xspn/xspn/serialization/binary/capnproto/spflow.capnp:27-102) with the class and method names
of its serializer (xspn/xspn/serialization/binary/BinarySerialization.py:53-370):
``BinarySerializer(fileName).serialize_to_file(content)`` and
``BinaryDeserializer(fileName).deserialize_from_file()``. Messages are written as one segment in
Cap'n Proto's unpacked stream framing; the reader also accepts multi-segment files with far
pointers, which pycapnp emits for large models.
"""
import struct

from spnc import structure as st
from xspn.structure.Model import SPNModel
from xspn.structure.Query import ErrorKind, ErrorModel, JointProbability, Query

_TYPE_ENUM = ["REAL", "INTERVAL", "POSITIVE", "CATEGORICAL", "ORDINAL", "COUNT", "BINARY"]
_META_ENUM = ["REAL", "BINARY", "DISCRETE"]
_KIND_TAG = {"product": 0, "sum": 1, "histogram": 2, "gaussian": 3, "categorical": 4}


def _enum_ordinal(value, names, default=0):
    """Ordinal of an SPFlow Type/MetaType-like value (enum member, name or ordinal)."""
    if value is None:
        return default
    name = getattr(value, "name", value)
    if isinstance(name, str) and name.upper() in names:
        return names.index(name.upper())
    if isinstance(value, int) and 0 <= value < len(names):
        return value
    return default


def _plain(value):
    return value.item() if hasattr(value, "item") else value


# --------------------------------------------------------------------------------------------
# writer
# --------------------------------------------------------------------------------------------
class _Segment:
    """A growing array of 64-bit words; word 0 is the root pointer."""

    def __init__(self):
        self.buf = bytearray(8)

    def alloc(self, nwords):
        at = len(self.buf) // 8
        self.buf.extend(bytes(8 * nwords))
        return at

    def put(self, word, byte_off, fmt, value):
        struct.pack_into("<" + fmt, self.buf, 8 * word + byte_off, value)

    def point_struct(self, at, target, dwords, pwords):
        off = (target - at - 1) & 0x3FFFFFFF
        self.put(at, 0, "Q", (off << 2) | (dwords << 32) | (pwords << 48))

    def point_list(self, at, target, elem_code, count):
        off = (target - at - 1) & 0x3FFFFFFF
        self.put(at, 0, "Q", 1 | (off << 2) | (elem_code << 32) | (count << 35))

    def new_struct(self, at, dwords, pwords):
        target = self.alloc(dwords + pwords)
        self.point_struct(at, target, dwords, pwords)
        return target

    def prim_list(self, at, fmt, elem_code, values):
        size = struct.calcsize(fmt)
        nbytes = size * len(values)
        target = self.alloc((nbytes + 7) // 8)
        struct.pack_into("<%d%s" % (len(values), fmt), self.buf, 8 * target, *values)
        self.point_list(at, target, elem_code, len(values))

    def text(self, at, s):
        raw = s.encode("utf-8") + b"\0"
        target = self.alloc((len(raw) + 7) // 8)
        self.buf[8 * target:8 * target + len(raw)] = raw
        self.point_list(at, target, 2, len(raw))

    def struct_list(self, at, count, dwords, pwords):
        stride = dwords + pwords
        tag = self.alloc(1 + count * stride)
        self.put(tag, 0, "Q", (count << 2) | (dwords << 32) | (pwords << 48))
        self.point_list(at, tag, 7, count * stride)
        return [tag + 1 + i * stride for i in range(count)]

    def stream(self):
        return struct.pack("<II", 0, len(self.buf) // 8) + bytes(self.buf)


class BinarySerializer:
    """Serialize SPN models / queries into the binary format the compiler reads."""

    def __init__(self, fileName, bufferSize=10 * (2 ** 10), clearFile=True):
        self.assignedIDs = {}
        self.fileName = fileName
        self.bufferSize = bufferSize
        if clearFile:
            open(fileName, "w").close()

    def serialize_to_file(self, content):
        seg = _Segment()
        header = seg.new_struct(0, 1, 1)
        if isinstance(content, SPNModel):
            seg.put(header, 0, "H", 0)
            self._write_model(seg, header + 1, content)
        elif isinstance(content, Query):
            seg.put(header, 0, "H", 1)
            self._write_query(seg, header + 1, content)
        else:
            raise NotImplementedError(f"No serialization defined for content {content} of type {type(content)}")
        with open(self.fileName, "a+b") as out:
            out.write(seg.stream())

    def _write_query(self, seg, at, query):
        q = seg.new_struct(at, 2, 1)
        seg.put(q, 0, "i", int(query.batchSize))
        if query.errorModel.kind == ErrorKind.ABSOLUTE:
            seg.put(q, 4, "H", 0)
        elif query.errorModel.kind == ErrorKind.RELATIVE:
            seg.put(q, 4, "H", 1)
        else:
            raise NotImplementedError(f"No serialization defined for error kind {query.errorModel.kind}")
        seg.put(q, 8, "d", float(query.errorModel.error))
        if not isinstance(query, JointProbability):
            raise NotImplementedError(f"No serialization defined for query {query} of type {type(query)}")
        joint = seg.new_struct(q + 2, 1, 1)
        seg.put(joint, 0, "B", 1 if query.supportsMarginal() else 0)
        self._write_model(seg, joint + 1, query.graph)

    def _write_model(self, seg, at, model):
        root = model.root
        assert st.is_valid(root), "SPN invalid before serialization"
        st.assign_ids(root, self.assignedIDs)
        st.rebuild_scopes_bottom_up(root)
        m = seg.new_struct(at, 1, 4)
        seg.put(m, 0, "i", int(root.id))
        seg.put(m, 4, "i", len(root.scope))
        seg.text(m + 1, model.name if model.name is not None else "")
        seg.text(m + 2, str(model.featureType))
        seg.prim_list(m + 3, "i", 4, [int(_plain(v)) for v in root.scope])
        nodes = st.topological_nodes(root)  # children before parents
        slots = seg.struct_list(m + 4, len(nodes), 1, 1)
        for node, slot in zip(nodes, slots):
            self._write_node(seg, slot, node, node is root)
        print(f"INFO: Serialized {len(nodes)} nodes to {self.fileName}")

    def _write_node(self, seg, at, node, is_root):
        kind = st.node_kind(node)
        seg.put(at, 0, "i", int(node.id))
        seg.put(at, 4, "B", 1 if is_root else 0)
        seg.put(at, 6, "H", _KIND_TAG[kind])
        ptr = at + 1
        if kind == "product":
            body = seg.new_struct(ptr, 0, 1)
            seg.prim_list(body, "i", 4, [int(c.id) for c in node.children])
        elif kind == "sum":
            body = seg.new_struct(ptr, 0, 2)
            seg.prim_list(body, "i", 4, [int(c.id) for c in node.children])
            seg.prim_list(body + 1, "d", 5, [float(_plain(w)) for w in node.weights])
        elif kind == "histogram":
            body = seg.new_struct(ptr, 1, 3)
            seg.put(body, 0, "H", _enum_ordinal(getattr(node, "type", None), _TYPE_ENUM))
            seg.put(body, 2, "H", _enum_ordinal(getattr(node, "meta_type", None), _META_ENUM))
            seg.put(body, 4, "i", st.leaf_scope(node))
            seg.prim_list(body + 1, "i", 4, [int(b) for b in node.breaks])
            seg.prim_list(body + 2, "d", 5, [float(_plain(d)) for d in node.densities])
            seg.prim_list(body + 3, "d", 5, [float(_plain(r)) for r in (getattr(node, "bin_repr_points", None) or [])])
        elif kind == "gaussian":
            body = seg.new_struct(ptr, 3, 0)
            seg.put(body, 0, "d", float(_plain(node.mean)))
            seg.put(body, 8, "d", float(_plain(node.stdev)))
            seg.put(body, 16, "i", st.leaf_scope(node))
        elif kind == "categorical":
            body = seg.new_struct(ptr, 1, 1)
            seg.put(body, 0, "i", st.leaf_scope(node))
            seg.prim_list(body + 1, "d", 5, [float(_plain(p)) for p in node.p])


# --------------------------------------------------------------------------------------------
# reader
# --------------------------------------------------------------------------------------------
class _Msg:
    def __init__(self, data):
        (nseg,) = struct.unpack_from("<I", data, 0)
        nseg += 1
        sizes = struct.unpack_from("<%dI" % nseg, data, 4)
        pos = 4 + 4 * nseg
        pos += pos % 8
        self.segs = []
        for s in sizes:
            self.segs.append(data[pos:pos + 8 * s])
            pos += 8 * s

    def w(self, seg, idx):
        return struct.unpack_from("<Q", self.segs[seg], 8 * idx)[0]

    def deref(self, seg, idx):
        """-> (pointer word, segment, word index of the target) following far pointers; None for null."""
        p = self.w(seg, idx)
        if p == 0:
            return None
        if p & 3 != 2:
            off = (p >> 2) & 0x3FFFFFFF
            off -= (off & 0x20000000) << 1
            return p, seg, idx + 1 + off
        pad_seg, pad = p >> 32, (p >> 3) & 0x1FFFFFFF
        if not (p >> 2) & 1:
            q = self.w(pad_seg, pad)
            off = (q >> 2) & 0x3FFFFFFF
            off -= (off & 0x20000000) << 1
            return q, pad_seg, pad + 1 + off
        far, tag = self.w(pad_seg, pad), self.w(pad_seg, pad + 1)
        return tag, far >> 32, (far >> 3) & 0x1FFFFFFF


class _S:
    """Struct view with default-zero reads beyond the encoded size."""

    def __init__(self, msg, seg=0, at=0, dw=0, pw=0):
        self.m, self.seg, self.at, self.dw, self.pw = msg, seg, at, dw, pw

    @classmethod
    def at_pointer(cls, msg, seg, idx):
        r = msg.deref(seg, idx)
        if r is None:
            return cls(msg)
        p, tseg, target = r
        return cls(msg, tseg, target, (p >> 32) & 0xFFFF, (p >> 48) & 0xFFFF)

    def get(self, fmt, off):
        if off + struct.calcsize(fmt) > 8 * self.dw:
            return 0
        return struct.unpack_from("<" + fmt, self.m.segs[self.seg], 8 * self.at + off)[0]

    def struct(self, i):
        return _S.at_pointer(self.m, self.seg, self.at + self.dw + i) if i < self.pw else _S(self.m)

    def has(self, i):
        return i < self.pw and self.m.w(self.seg, self.at + self.dw + i) != 0

    def prims(self, i, fmt):
        if i >= self.pw:
            return []
        r = self.m.deref(self.seg, self.at + self.dw + i)
        if r is None:
            return []
        p, tseg, target = r
        count = p >> 35
        return list(struct.unpack_from("<%d%s" % (count, fmt), self.m.segs[tseg], 8 * target))

    def text(self, i):
        raw = bytes(self.prims(i, "B"))
        return raw[:-1].decode("utf-8") if raw else ""

    def structs(self, i):
        if i >= self.pw:
            return []
        r = self.m.deref(self.seg, self.at + self.dw + i)
        if r is None:
            return []
        p, tseg, target = r
        tag = self.m.w(tseg, target)
        count, dw, pw = (tag >> 2) & 0x3FFFFFFF, (tag >> 32) & 0xFFFF, (tag >> 48) & 0xFFFF
        return [_S(self.m, tseg, target + 1 + k * (dw + pw), dw, pw) for k in range(count)]


class BinaryDeserializer:
    """Read SPN models / queries back from the binary format."""

    def __init__(self, fileName):
        self.fileName = fileName

    def deserialize_from_file(self):
        with open(self.fileName, "rb") as f:
            msg = _Msg(f.read())
        header = _S.at_pointer(msg, 0, 0)
        which = header.get("H", 0)
        if which == 1:
            return self._query(header.struct(0))
        if which == 0:
            return self._model(header.struct(0))
        raise NotImplementedError("No deserialization defined for this header")

    def _query(self, q):
        kind = ErrorKind.ABSOLUTE if q.get("H", 4) == 0 else ErrorKind.RELATIVE
        joint = q.struct(0)
        model = self._model(joint.struct(0))
        return JointProbability(model, q.get("i", 0), bool(joint.get("B", 0) & 1), ErrorModel(kind, q.get("d", 8)))

    def _model(self, m):
        root_id = m.get("i", 0)
        name = m.text(0) or None
        nodes = {}
        for s in m.structs(3):
            tag, body = s.get("H", 6), s.struct(0)
            if tag == 0:
                n = st.Product(children=[nodes[c] for c in body.prims(0, "i")])
            elif tag == 1:
                n = st.Sum(weights=body.prims(1, "d"), children=[nodes[c] for c in body.prims(0, "i")])
            elif tag == 2:
                n = st.Histogram(body.prims(0, "i"), body.prims(1, "d"), body.prims(2, "d"), scope=body.get("i", 4),
                                 type_=_TYPE_ENUM[body.get("H", 0)], meta_type=_META_ENUM[body.get("H", 2)])
            elif tag == 3:
                n = st.Gaussian(body.get("d", 0), body.get("d", 8), scope=body.get("i", 16))
            elif tag == 4:
                n = st.Categorical(p=body.prims(0, "d"), scope=body.get("i", 0))
            else:
                raise NotImplementedError(f"No deserialization defined for node kind {tag}")
            n.id = s.get("i", 0)
            nodes[n.id] = n
        print(f"Deserialized {len(nodes)} nodes from {self.fileName}")
        root = nodes[root_id]
        st.rebuild_scopes_bottom_up(root)
        assert st.is_valid(root), "SPN invalid after deserialization"
        return SPNModel(root, m.text(1), name)
