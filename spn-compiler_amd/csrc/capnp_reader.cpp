#include "capnp_reader.h"

#include <cstdio>

namespace spnc_hip {
namespace capnp {

namespace {
[[noreturn]] void fail(const char* what) { throw std::runtime_error(std::string("malformed Cap'n Proto message: ") + what); }

inline int64_t signedOffset(uint64_t p) {
  // bits 2..31, two's complement 30-bit
  int64_t o = int64_t((p >> 2) & 0x3FFFFFFFu);
  if (o & (int64_t(1) << 29)) o -= (int64_t(1) << 30);
  return o;
}
}  // namespace

Message::Message(std::vector<uint8_t> bytes) : data_(std::move(bytes)) {
  if (data_.size() < 8) fail("shorter than a segment table");
  uint32_t nsegM1;
  std::memcpy(&nsegM1, data_.data(), 4);
  uint64_t nseg = uint64_t(nsegM1) + 1;
  if (nseg > 512) fail("implausible segment count");
  size_t hdr = 4 + 4 * nseg;
  if (hdr % 8) hdr += 4;
  if (hdr > data_.size()) fail("segment table exceeds file");
  size_t off = hdr;
  for (uint64_t s = 0; s < nseg; ++s) {
    uint32_t words;
    std::memcpy(&words, data_.data() + 4 + 4 * s, 4);
    size_t nbytes = size_t(words) * 8;
    if (off + nbytes > data_.size()) fail("segment exceeds file");
    segs_.push_back({off, words});
    off += nbytes;
  }
}

Message Message::fromFile(const std::string& path) {
  FILE* f = std::fopen(path.c_str(), "rb");
  if (!f) throw std::runtime_error("cannot open query file '" + path + "'");
  std::vector<uint8_t> buf;
  uint8_t tmp[1 << 16];
  size_t n;
  while ((n = std::fread(tmp, 1, sizeof(tmp), f)) > 0) buf.insert(buf.end(), tmp, tmp + n);
  std::fclose(f);
  return Message(std::move(buf));
}

uint64_t Message::word(uint32_t seg, uint64_t idx) const {
  if (seg >= segs_.size() || idx >= segs_[seg].words) fail("pointer outside segment");
  uint64_t v;
  std::memcpy(&v, data_.data() + segs_[seg].byteOffset + idx * 8, 8);
  return v;
}

const uint8_t* Message::bytes(uint32_t seg, uint64_t wordIdx, uint64_t nbytes) const {
  if (seg >= segs_.size()) fail("unknown segment");
  uint64_t total = segs_[seg].words * 8;
  if (wordIdx * 8 > total || nbytes > total - wordIdx * 8) fail("object outside segment");
  return data_.data() + segs_[seg].byteOffset + wordIdx * 8;
}

Message::Resolved Message::follow(uint32_t seg, uint64_t idx) const {
  uint64_t p = word(seg, idx);
  if ((p & 3) != 2) return {p, seg, idx + 1, false};
  bool doubleFar = (p >> 2) & 1;
  uint64_t off = (p >> 3) & 0x1FFFFFFFu;
  uint32_t tseg = uint32_t(p >> 32);
  if (!doubleFar) {
    uint64_t q = word(tseg, off);
    if ((q & 3) == 2) fail("far pointer lands on a far pointer");
    return {q, tseg, off + 1, false};
  }
  uint64_t pad = word(tseg, off);
  uint64_t tag = word(tseg, off + 1);
  if ((pad & 3) != 2 || ((pad >> 2) & 1)) fail("bad double-far landing pad");
  return {tag, uint32_t(pad >> 32), (pad >> 3) & 0x1FFFFFFFu, true};
}

StructReader Message::resolveStruct(uint32_t seg, uint64_t idx) const {
  Resolved r = follow(seg, idx);
  if (r.ptr == 0) return StructReader(this, 0, 0, 0, 0);
  if ((r.ptr & 3) != 0) fail("expected a struct pointer");
  int64_t start = r.contentAtBase ? int64_t(r.base) : int64_t(r.base) + signedOffset(r.ptr);
  if (start < 0) fail("negative struct offset");
  uint16_t dw = uint16_t(r.ptr >> 32), pw = uint16_t(r.ptr >> 48);
  bytes(r.seg, uint64_t(start), (uint64_t(dw) + pw) * 8);
  return StructReader(this, r.seg, uint64_t(start), dw, pw);
}

ListReader Message::resolveList(uint32_t seg, uint64_t idx) const {
  Resolved r = follow(seg, idx);
  if (r.ptr == 0) return ListReader(this, 0, 0, 0, 0, 0, 0);
  if ((r.ptr & 3) != 1) fail("expected a list pointer");
  int64_t start = r.contentAtBase ? int64_t(r.base) : int64_t(r.base) + signedOffset(r.ptr);
  if (start < 0) fail("negative list offset");
  unsigned esz = unsigned((r.ptr >> 32) & 7);
  uint64_t cnt = r.ptr >> 35;
  if (esz == 7) {
    uint64_t tag = word(r.seg, uint64_t(start));
    uint64_t n = (tag >> 2) & 0x3FFFFFFFu;
    uint16_t dw = uint16_t(tag >> 32), pw = uint16_t(tag >> 48);
    if (n * (uint64_t(dw) + pw) > cnt) fail("composite list overruns its word count");
    bytes(r.seg, uint64_t(start) + 1, cnt * 8);
    return ListReader(this, r.seg, uint64_t(start) + 1, 7, n, dw, pw);
  }
  static const unsigned bits[7] = {0, 1, 8, 16, 32, 64, 64};
  bytes(r.seg, uint64_t(start), (cnt * bits[esz] + 7) / 8);
  return ListReader(this, r.seg, uint64_t(start), esz, cnt, 0, 0);
}

StructReader Message::root() const { return resolveStruct(0, 0); }

const uint8_t* StructReader::dataPtr(size_t byteOffset, size_t n) const {
  return msg_->bytes(seg_, start_, size_t(dw_) * 8) + byteOffset + 0 * n;
}

bool StructReader::hasPointer(unsigned i) const {
  if (!msg_ || i >= pw_) return false;
  return msg_->word(seg_, start_ + dw_ + i) != 0;
}

StructReader StructReader::getStruct(unsigned i) const {
  if (!msg_ || i >= pw_) return StructReader(msg_, 0, 0, 0, 0);
  return msg_->resolveStruct(seg_, start_ + dw_ + i);
}

ListReader StructReader::getList(unsigned i) const {
  if (!msg_ || i >= pw_) return ListReader(msg_, 0, 0, 0, 0, 0, 0);
  return msg_->resolveList(seg_, start_ + dw_ + i);
}

std::string StructReader::getText(unsigned i) const {
  ListReader l = getList(i);
  if (l.size() == 0) return std::string();
  if (l.elementCode() != 2) fail("text is not a byte list");
  const char* p = reinterpret_cast<const char*>(l.raw());
  return std::string(p, l.size() - 1);  // drop the trailing NUL
}

const uint8_t* ListReader::raw() const {
  static const unsigned bits[8] = {0, 1, 8, 16, 32, 64, 64, 0};
  return msg_->bytes(seg_, start_, (count_ * bits[esz_] + 7) / 8);
}

void ListReader::checkPrimitive(size_t bytes, size_t i) const {
  static const unsigned sz[8] = {0, 0, 1, 2, 4, 8, 0, 0};
  if (esz_ > 5 || sz[esz_] != bytes) fail("list element width mismatch");
  if (i >= count_) fail("list index out of range");
}

StructReader ListReader::getStruct(size_t i) const {
  if (esz_ != 7) fail("not a struct list");
  if (i >= count_) fail("list index out of range");
  return StructReader(msg_, seg_, start_ + i * (uint64_t(dw_) + pw_), dw_, pw_);
}

}  // namespace capnp
}  // namespace spnc_hip
