// Minimal FlatBuffers codec (reader + builder) for the TTNN binary format.  No flatc, no
// generated accessors: tables are read through their vtable by field slot number
// (schema_generated.h) and written with a small back-to-front builder that produces the standard
// wire format (size prefix, root offset, file identifier, vtables, uoffsets).
#pragma once
#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <string_view>
#include <vector>

namespace ttmlir_amd::fb {

// ------------------------------------------------------------------------------------- reader
struct Bounds {
  const uint8_t *begin = nullptr, *end = nullptr;
  void check(const uint8_t *p, size_t n) const {
    if (p < begin || p > end || n > static_cast<size_t>(end - p)) throw std::runtime_error("flatbuffer: read out of bounds");
  }
};

template <typename T>
inline T readScalar(const uint8_t *p) {
  T v;
  std::memcpy(&v, p, sizeof(T));
  return v;
}

class Table;

template <typename T>
class ScalarVector {
public:
  ScalarVector() = default;
  ScalarVector(const uint8_t *p, Bounds b) : b_(b) {
    b_.check(p, 4);
    n_ = readScalar<uint32_t>(p);
    data_ = p + 4;
    b_.check(data_, static_cast<size_t>(n_) * sizeof(T));
  }
  uint32_t size() const { return n_; }
  T operator[](uint32_t i) const {
    if (i >= n_) throw std::runtime_error("flatbuffer: vector index out of range");
    return readScalar<T>(data_ + static_cast<size_t>(i) * sizeof(T));
  }
  const uint8_t *data() const { return data_; }
  std::vector<T> toVector() const {
    std::vector<T> v(n_);
    if (n_) std::memcpy(v.data(), data_, static_cast<size_t>(n_) * sizeof(T));
    return v;
  }

private:
  const uint8_t *data_ = nullptr;
  uint32_t n_ = 0;
  Bounds b_;
};

class TableVector;

class Table {
public:
  Table() = default;
  Table(const uint8_t *p, Bounds b) : p_(p), b_(b) {
    b_.check(p_, 4);
    int32_t so = readScalar<int32_t>(p_);
    vt_ = p_ - so;
    b_.check(vt_, 4);
    vtSize_ = readScalar<uint16_t>(vt_);
    if (vtSize_ < 4) throw std::runtime_error("flatbuffer: bad vtable");
    b_.check(vt_, vtSize_);
  }
  explicit operator bool() const { return p_ != nullptr; }
  bool has(int slot) const { return fieldOffset(slot) != 0; }

  template <typename T>
  T scalar(int slot, T def) const {
    uint16_t o = fieldOffset(slot);
    if (!o) return def;
    b_.check(p_ + o, sizeof(T));
    return readScalar<T>(p_ + o);
  }
  // inline struct: pointer to its bytes (or null)
  const uint8_t *structPtr(int slot, size_t size) const {
    uint16_t o = fieldOffset(slot);
    if (!o) return nullptr;
    b_.check(p_ + o, size);
    return p_ + o;
  }
  Table table(int slot) const {
    const uint8_t *t = indirect(slot);
    return t ? Table(t, b_) : Table();
  }
  std::string_view string(int slot) const {
    const uint8_t *s = indirect(slot);
    if (!s) return {};
    b_.check(s, 4);
    uint32_t n = readScalar<uint32_t>(s);
    b_.check(s + 4, n);
    return std::string_view(reinterpret_cast<const char *>(s + 4), n);
  }
  template <typename T>
  ScalarVector<T> scalars(int slot) const {
    const uint8_t *v = indirect(slot);
    return v ? ScalarVector<T>(v, b_) : ScalarVector<T>();
  }
  TableVector tables(int slot) const;

private:
  uint16_t fieldOffset(int slot) const {
    if (!p_) return 0;
    size_t at = 4 + static_cast<size_t>(slot) * 2;
    if (at + 2 > vtSize_) return 0;
    return readScalar<uint16_t>(vt_ + at);
  }
  const uint8_t *indirect(int slot) const {
    uint16_t o = fieldOffset(slot);
    if (!o) return nullptr;
    b_.check(p_ + o, 4);
    return p_ + o + readScalar<uint32_t>(p_ + o);
  }
  const uint8_t *p_ = nullptr, *vt_ = nullptr;
  uint16_t vtSize_ = 0;
  Bounds b_;
};

class TableVector {
public:
  TableVector() = default;
  TableVector(const uint8_t *p, Bounds b) : b_(b) {
    b_.check(p, 4);
    n_ = readScalar<uint32_t>(p);
    data_ = p + 4;
    b_.check(data_, static_cast<size_t>(n_) * 4);
  }
  uint32_t size() const { return n_; }
  Table operator[](uint32_t i) const {
    if (i >= n_) throw std::runtime_error("flatbuffer: vector index out of range");
    const uint8_t *e = data_ + static_cast<size_t>(i) * 4;
    return Table(e + readScalar<uint32_t>(e), b_);
  }

private:
  const uint8_t *data_ = nullptr;
  uint32_t n_ = 0;
  Bounds b_;
};

inline TableVector Table::tables(int slot) const {
  const uint8_t *v = indirect(slot);
  return v ? TableVector(v, b_) : TableVector();
}

// Root of a size-prefixed buffer; checks the size prefix and (optionally) the file identifier.
inline Table sizePrefixedRoot(const uint8_t *buf, size_t len, const char *identifier) {
  if (len < 12) throw std::runtime_error("flatbuffer: buffer too small");
  uint32_t size = readScalar<uint32_t>(buf);
  if (static_cast<size_t>(size) + 4 > len) throw std::runtime_error("flatbuffer: size prefix exceeds the buffer");
  const uint8_t *body = buf + 4;
  if (identifier && std::memcmp(body + 4, identifier, 4) != 0)
    throw std::runtime_error(std::string("flatbuffer: file identifier is not '") + identifier + "'");
  Bounds b{body, body + size};
  uint32_t root = readScalar<uint32_t>(body);
  return Table(body + root, b);
}

// ------------------------------------------------------------------------------------- builder
// Back-to-front builder.  Offsets handed out are distances from the END of the buffer, as in the
// reference implementation of the format, so they stay valid while the buffer grows.
class Builder {
public:
  using Off = uint32_t;  // 0 = null

  Off createString(std::string_view s) {
    preAlign(s.size() + 1, 4);
    pushZeros(1);
    pushBytes(s.data(), s.size());
    pushScalar<uint32_t>(static_cast<uint32_t>(s.size()));
    return size();
  }
  template <typename T>
  Off createScalarVector(const T *data, size_t n) {
    preAlign(n * sizeof(T), 4);
    preAlign(n * sizeof(T), sizeof(T));
    pushBytes(data, n * sizeof(T));
    pushScalar<uint32_t>(static_cast<uint32_t>(n));
    return size();
  }
  template <typename T>
  Off createScalarVector(const std::vector<T> &v) { return createScalarVector(v.data(), v.size()); }
  Off createOffsetVector(const std::vector<Off> &offs) {
    preAlign(offs.size() * 4, 4);
    for (size_t i = offs.size(); i-- > 0;) pushOffset(offs[i]);
    pushScalar<uint32_t>(static_cast<uint32_t>(offs.size()));
    return size();
  }

  void startTable(int numFields) {
    fields_.assign(static_cast<size_t>(numFields), 0);
    tableStart_ = size();
    inTable_ = true;
  }
  template <typename T>
  void addScalar(int slot, T v) {
    align(sizeof(T));
    pushScalarNoAlign(v);
    fields_.at(slot) = size();
  }
  template <typename T>
  void addScalarDefault(int slot, T v, T def) {
    if (v != def) addScalar(slot, v);
  }
  void addStruct(int slot, const void *bytes, size_t n, size_t alignment) {
    align(alignment);
    pushBytes(bytes, n);
    fields_.at(slot) = size();
  }
  void addOffset(int slot, Off target) {
    if (!target) return;
    align(4);
    pushOffsetNoAlign(target);
    fields_.at(slot) = size();
  }
  Off endTable() {
    align(4);
    pushScalarNoAlign<int32_t>(0);  // soffset placeholder
    const Off tableOff = size();
    // trim trailing absent fields
    size_t n = fields_.size();
    while (n > 0 && fields_[n - 1] == 0) --n;
    const uint16_t vtBytes = static_cast<uint16_t>(4 + 2 * n);
    for (size_t i = n; i-- > 0;) {
      uint16_t o = fields_[i] ? static_cast<uint16_t>(tableOff - fields_[i]) : 0;
      pushScalarNoAlign<uint16_t>(o);
    }
    pushScalarNoAlign<uint16_t>(static_cast<uint16_t>(tableOff - tableStart_));
    pushScalarNoAlign<uint16_t>(vtBytes);
    const Off vtOff = size();
    // soffset = table position - vtable position (vtable sits before the table in memory)
    int32_t so = static_cast<int32_t>(vtOff - tableOff);
    std::memcpy(&buf_[buf_.size() - tableOff], &so, 4);
    inTable_ = false;
    return tableOff;
  }

  // Finish with size prefix and 4-character identifier; returns the complete file image.
  std::vector<uint8_t> finishSizePrefixed(Off root, const char *identifier) {
    preAlign(4 + 4 + 4, maxAlign_);
    pushBytes(identifier, 4);
    pushOffset(root);
    pushScalarNoAlign<uint32_t>(size());
    return std::vector<uint8_t>(buf_.end() - size(), buf_.end());
  }

  Off size() const { return used_; }

private:
  // buf_ is filled from its end toward its start
  void grow(size_t need) {
    if (buf_.size() - used_ >= need) return;
    size_t ns = buf_.size() ? buf_.size() : 1024;
    while (ns - used_ < need) ns *= 2;
    std::vector<uint8_t> nb(ns, 0);
    if (used_) std::memcpy(nb.data() + ns - used_, buf_.data() + buf_.size() - used_, used_);
    buf_.swap(nb);
  }
  void pushBytes(const void *p, size_t n) {
    if (!n) return;
    grow(n);
    used_ += static_cast<Off>(n);
    std::memcpy(&buf_[buf_.size() - used_], p, n);
  }
  void pushZeros(size_t n) {
    if (!n) return;
    grow(n);
    used_ += static_cast<Off>(n);
    std::memset(&buf_[buf_.size() - used_], 0, n);
  }
  void align(size_t a) {
    if (a > maxAlign_) maxAlign_ = a;
    pushZeros((a - (used_ % a)) % a);
  }
  // make (size() + len) a multiple of `a` once `len` more bytes have been pushed
  void preAlign(size_t len, size_t a) {
    if (a > maxAlign_) maxAlign_ = a;
    pushZeros((a - ((used_ + len) % a)) % a);
  }
  template <typename T>
  void pushScalarNoAlign(T v) { pushBytes(&v, sizeof(T)); }
  template <typename T>
  void pushScalar(T v) {
    align(sizeof(T));
    pushScalarNoAlign(v);
  }
  void pushOffsetNoAlign(Off target) {
    // the stored uoffset is the distance from the offset field to its target
    uint32_t rel = (used_ + 4) - target;
    pushScalarNoAlign<uint32_t>(rel);
  }
  void pushOffset(Off target) {
    align(4);
    pushOffsetNoAlign(target);
  }

  std::vector<uint8_t> buf_;
  Off used_ = 0;
  std::vector<Off> fields_;
  Off tableStart_ = 0;
  bool inTable_ = false;
  size_t maxAlign_ = 4;
};

}  // namespace ttmlir_amd::fb
