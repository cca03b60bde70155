"""Minimal read-only Cap'n Proto decoder (test infrastructure, see oracle/__init__.py).

Implements just what the public Cap'n Proto encoding specification fixes and
what the reference's fixtures need: the unpacked stream framing that
``StreamFdMessageReader`` consumes
(compiler/src/pipeline/steps/frontend/SPFlowToMLIRDeserializer.cpp:38-41),
struct/list/far/double-far pointers, composite lists, and default values for
fields beyond a struct's encoded size.

Written independently of the C++ reader in ``spn-compiler_amd/csrc`` so that
each can check the other.
"""
import struct


class CapnpError(ValueError):
    pass


class Message:
    def __init__(self, data: bytes):
        if len(data) < 8:
            raise CapnpError("message too short")
        nseg = struct.unpack_from("<I", data, 0)[0] + 1
        if nseg > 512:
            raise CapnpError("implausible segment count %d" % nseg)
        sizes = struct.unpack_from("<%dI" % nseg, data, 4)
        hdr = 4 + 4 * nseg
        if hdr % 8:
            hdr += 4
        self.segments = []
        off = hdr
        for s in sizes:
            end = off + 8 * s
            if end > len(data):
                raise CapnpError("segment exceeds file")
            self.segments.append(memoryview(data)[off:end])
            off = end

    @classmethod
    def from_file(cls, path):
        with open(path, "rb") as f:
            return cls(f.read())

    def word(self, seg, idx):
        s = self.segments[seg]
        if idx < 0 or 8 * idx + 8 > len(s):
            raise CapnpError("word index out of segment")
        return struct.unpack_from("<Q", s, 8 * idx)[0]

    def root(self):
        return self._resolve_struct(0, 0)

    # -- pointer resolution -------------------------------------------------
    def _follow_far(self, seg, idx):
        """Returns (pointer word, segment, word index *after* the pointer) with far pointers resolved.

        For a double-far the returned position is the content start and the
        pointer word is the tag (offset treated as zero by the caller through
        the returned base).
        """
        p = self.word(seg, idx)
        if p & 3 != 2:
            return p, seg, idx + 1, False
        double = (p >> 2) & 1
        off = (p >> 3) & 0x1FFFFFFF
        tseg = p >> 32
        if tseg >= len(self.segments):
            raise CapnpError("far pointer to unknown segment")
        if not double:
            q = self.word(tseg, off)
            if q & 3 == 2:
                raise CapnpError("far pointer landing pad is itself far")
            return q, tseg, off + 1, False
        pad = self.word(tseg, off)
        tag = self.word(tseg, off + 1)
        if pad & 3 != 2 or (pad >> 2) & 1:
            raise CapnpError("malformed double-far landing pad")
        cseg = pad >> 32
        coff = (pad >> 3) & 0x1FFFFFFF
        return tag, cseg, coff, True

    @staticmethod
    def _soff(p):
        o = (p >> 2) & 0x3FFFFFFF
        return o - (1 << 30) if o & (1 << 29) else o

    def _resolve_struct(self, seg, idx):
        p, tseg, base, dbl = self._follow_far(seg, idx)
        if p == 0:
            return Struct(self, 0, 0, 0, 0)
        if p & 3 != 0:
            raise CapnpError("expected struct pointer")
        start = base if dbl else base + self._soff(p)
        return Struct(self, tseg, start, (p >> 32) & 0xFFFF, (p >> 48) & 0xFFFF)

    def _resolve_list(self, seg, idx):
        p, tseg, base, dbl = self._follow_far(seg, idx)
        if p == 0:
            return List(self, 0, 0, 0, 0, 0, 0)
        if p & 3 != 1:
            raise CapnpError("expected list pointer")
        start = base if dbl else base + self._soff(p)
        esz = (p >> 32) & 7
        cnt = p >> 35
        if esz == 7:
            tag = self.word(tseg, start)
            n = (tag >> 2) & 0x3FFFFFFF
            dw, pw = (tag >> 32) & 0xFFFF, (tag >> 48) & 0xFFFF
            if n * (dw + pw) > cnt:
                raise CapnpError("composite list overruns its word count")
            return List(self, tseg, start + 1, 7, n, dw, pw)
        return List(self, tseg, start, esz, cnt, 0, 0)


class Struct:
    def __init__(self, msg, seg, start, dwords, pwords):
        self.msg, self.seg, self.start, self.dw, self.pw = msg, seg, start, dwords, pwords

    def _bytes(self, off, n):
        if off + n > 8 * self.dw:
            return None
        s = self.msg.segments[self.seg]
        b = 8 * self.start + off
        if b + n > len(s):
            raise CapnpError("struct data out of segment")
        return s[b:b + n]

    def get(self, fmt, byte_off, default=0):
        b = self._bytes(byte_off, struct.calcsize(fmt))
        if b is None:
            return default
        return struct.unpack("<" + fmt, b)[0]

    def get_bool(self, bit, default=False):
        b = self._bytes(bit // 8, 1)
        if b is None:
            return default
        return bool((b[0] >> (bit % 8)) & 1) != default

    def has_ptr(self, i):
        return i < self.pw and self.msg.word(self.seg, self.start + self.dw + i) != 0

    def ptr_struct(self, i):
        if i >= self.pw:
            return Struct(self.msg, 0, 0, 0, 0)
        return self.msg._resolve_struct(self.seg, self.start + self.dw + i)

    def ptr_list(self, i):
        if i >= self.pw:
            return List(self.msg, 0, 0, 0, 0, 0, 0)
        return self.msg._resolve_list(self.seg, self.start + self.dw + i)

    def ptr_text(self, i):
        l = self.ptr_list(i)
        if l.count == 0:
            return ""
        raw = bytes(l.raw_bytes())
        return raw[:-1].decode("utf-8")


_ELEM = {2: ("b", 1), 3: ("h", 2), 4: ("i", 4), 5: ("q", 8)}


class List:
    def __init__(self, msg, seg, start, esz, count, dw, pw):
        self.msg, self.seg, self.start, self.esz, self.count, self.dw, self.pw = msg, seg, start, esz, count, dw, pw

    def __len__(self):
        return self.count

    def raw_bytes(self):
        if self.esz not in _ELEM:
            raise CapnpError("not a primitive list")
        n = _ELEM[self.esz][1] * self.count
        s = self.msg.segments[self.seg]
        if 8 * self.start + n > len(s):
            raise CapnpError("list out of segment")
        return s[8 * self.start:8 * self.start + n]

    def primitives(self, fmt):
        if self.count == 0:
            return []
        size = struct.calcsize(fmt)
        if self.esz not in _ELEM or _ELEM[self.esz][1] != size:
            raise CapnpError("list element size mismatch")
        return list(struct.unpack("<%d%s" % (self.count, fmt), self.raw_bytes()))

    def structs(self):
        if self.count == 0:
            return []
        if self.esz != 7:
            raise CapnpError("not a composite list")
        stride = self.dw + self.pw
        return [Struct(self.msg, self.seg, self.start + i * stride, self.dw, self.pw) for i in range(self.count)]
