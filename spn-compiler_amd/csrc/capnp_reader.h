// Dependency-free, read-only Cap'n Proto decoder for the serialized SPN queries.
//
// Replaces the capnp C++ runtime the reference links for its frontend
// (compiler/src/pipeline/steps/frontend/SPFlowToMLIRDeserializer.cpp:38-41 reads the file
// through StreamFdMessageReader).  Supports exactly the encoding features the query files use:
// unpacked stream framing, single and multi-segment messages, far and double-far pointers,
// composite lists, and default values for fields beyond a struct's encoded size.
// Every access is bounds-checked; malformed input raises std::runtime_error.
#pragma once
#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

namespace spnc_hip {
namespace capnp {

class Message;
class ListReader;

class StructReader {
 public:
  StructReader() = default;
  StructReader(const Message* m, uint32_t seg, uint64_t start, uint16_t dw, uint16_t pw)
      : msg_(m), seg_(seg), start_(start), dw_(dw), pw_(pw) {}

  template <typename T>
  T get(size_t byteOffset, T def = T()) const {
    if (byteOffset + sizeof(T) > size_t(dw_) * 8) return def;
    T v;
    std::memcpy(&v, dataPtr(byteOffset, sizeof(T)), sizeof(T));
    return v;
  }
  bool getBool(size_t bit) const {
    if (bit / 8 + 1 > size_t(dw_) * 8) return false;
    return (*dataPtr(bit / 8, 1) >> (bit % 8)) & 1;
  }
  bool hasPointer(unsigned i) const;
  StructReader getStruct(unsigned i) const;
  ListReader getList(unsigned i) const;
  std::string getText(unsigned i) const;

 private:
  const uint8_t* dataPtr(size_t byteOffset, size_t n) const;
  const Message* msg_ = nullptr;
  uint32_t seg_ = 0;
  uint64_t start_ = 0;  // word index of the data section inside the segment
  uint16_t dw_ = 0, pw_ = 0;
};

class ListReader {
 public:
  ListReader() = default;
  ListReader(const Message* m, uint32_t seg, uint64_t start, unsigned esz, uint64_t count, uint16_t dw, uint16_t pw)
      : msg_(m), seg_(seg), start_(start), esz_(esz), count_(count), dw_(dw), pw_(pw) {}
  size_t size() const { return count_; }
  template <typename T>
  T get(size_t i) const {
    checkPrimitive(sizeof(T), i);
    T v;
    std::memcpy(&v, raw() + i * sizeof(T), sizeof(T));
    return v;
  }
  template <typename T>
  std::vector<T> toVector() const {
    std::vector<T> out(count_);
    for (size_t i = 0; i < count_; ++i) out[i] = get<T>(i);
    return out;
  }
  StructReader getStruct(size_t i) const;
  const uint8_t* raw() const;
  unsigned elementCode() const { return esz_; }

 private:
  void checkPrimitive(size_t bytes, size_t i) const;
  const Message* msg_ = nullptr;
  uint32_t seg_ = 0;
  uint64_t start_ = 0;
  unsigned esz_ = 0;
  uint64_t count_ = 0;
  uint16_t dw_ = 0, pw_ = 0;
};

class Message {
 public:
  // Takes ownership of the raw stream bytes (segment table + segments).
  explicit Message(std::vector<uint8_t> bytes);
  static Message fromFile(const std::string& path);
  StructReader root() const;

  size_t numSegments() const { return segs_.size(); }

 private:
  friend class StructReader;
  friend class ListReader;
  struct Seg {
    size_t byteOffset;
    uint64_t words;
  };
  uint64_t word(uint32_t seg, uint64_t idx) const;
  const uint8_t* bytes(uint32_t seg, uint64_t wordIdx, uint64_t nbytes) const;
  struct Resolved {
    uint64_t ptr;
    uint32_t seg;
    uint64_t base;  // word index the pointer's offset is relative to (or the content start for double-far)
    bool contentAtBase;
  };
  Resolved follow(uint32_t seg, uint64_t idx) const;
  StructReader resolveStruct(uint32_t seg, uint64_t idx) const;
  ListReader resolveList(uint32_t seg, uint64_t idx) const;

  std::vector<uint8_t> data_;
  std::vector<Seg> segs_;
};

}  // namespace capnp
}  // namespace spnc_hip
