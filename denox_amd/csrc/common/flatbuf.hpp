// FlatBuffers wire format, written and read without the FlatBuffers library.
//
// The reference stores compiled models and its timing database as FlatBuffers (dnx.fbs:1-195, db.fbs:1-150, written
// through flatc-generated code: compiler/src/denox/compiler/serialize/serialize.cpp:598-633).  Neither flatc nor the
// library's headers exist on this platform, so this header restates the published binary layout:
//
//   buffer  := uoffset32 root, [4-byte file identifier], objects...            (little endian throughout)
//   table   := soffset32 (table position - vtable position), fields inline, each aligned to its own size
//   vtable  := u16 vtable bytes, u16 table bytes, u16 field offset from the table start per field id (0 = absent)
//   uoffset := u32, relative to its own position, always pointing to a HIGHER address
//   vector  := u32 element count, elements (scalars, structs inline, or uoffsets to tables / strings)
//   string  := u32 byte count, bytes, one 0 byte that the count does not include
//   union   := two fields: a u8 member index (0 = NONE) and a uoffset to the member table
//
// `Builder` writes back to front (children first), as the library's own builder does, so every uoffset is positive by
// construction; identical vtables are shared.  `Table` / `Vector` are views that check every access against the buffer
// (position, size, alignment, string terminator) and throw Error(InvalidModel): reading a table is verifying it, which
// replaces the separate flatbuffers::Verifier pass of runtime/src/denox/runtime/model.cpp:639-644.
#pragma once
#include "error.hpp"
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

namespace denox::fb {

using Off = uint32_t; // distance from the END of the buffer under construction to the start of an object; 0 = none

class Builder {
public:
  explicit Builder(size_t initial = 1u << 16) : m_buf(initial < 64 ? 64 : initial), m_head(m_buf.size()) {}

  Off createString(const std::string &s) {
    prep(4, s.size() + 1);
    push8(0);
    push(s.data(), s.size());
    place<uint32_t>(static_cast<uint32_t>(s.size()));
    return used();
  }
  // [ubyte] / [uint32] / ... : `count` elements of `elemSize` bytes, element alignment `align`, already little endian
  Off createVector(const void *data, size_t elemSize, size_t align, size_t count) {
    if (count > 0x7FFFFFFFu / (elemSize ? elemSize : 1)) fail(Status::Internal, "vector too large for a flatbuffer");
    const size_t bytes = elemSize * count;
    prep(4, bytes);
    prep(align, bytes);
    push(data, bytes);
    place<uint32_t>(static_cast<uint32_t>(count));
    return used();
  }
  Off createOffsetVector(const std::vector<Off> &offs) {
    prep(4, 4 * offs.size());
    for (size_t i = offs.size(); i-- > 0;) placeUOffset(offs[i]);
    place<uint32_t>(static_cast<uint32_t>(offs.size()));
    return used();
  }

  void startTable(unsigned fields) {
    m_slots.assign(fields, 0);
    m_objEnd = used();
  }
  template <typename T> void addScalar(unsigned slot, T v, T def) {
    if (v == def) return; // a field equal to its schema default is left out, as the library does
    prep(sizeof(T), 0);
    place<T>(v);
    m_slots.at(slot) = used();
  }
  void addOffset(unsigned slot, Off o) {
    if (!o) return;
    prep(4, 0);
    placeUOffset(o);
    m_slots.at(slot) = used();
  }
  Off endTable() {
    prep(4, 0);
    place<int32_t>(0); // soffset to the vtable, patched below
    const Off table = used();
    size_t n = m_slots.size();
    while (n > 0 && m_slots[n - 1] == 0) --n;
    std::vector<uint16_t> vt(2 + n);
    if (4 + 2 * n > 0xFFFF || table - m_objEnd > 0xFFFF) fail(Status::Internal, "table too large for a flatbuffer");
    vt[0] = static_cast<uint16_t>(4 + 2 * n);
    vt[1] = static_cast<uint16_t>(table - m_objEnd);
    for (size_t i = 0; i < n; ++i) vt[2 + i] = m_slots[i] ? static_cast<uint16_t>(table - m_slots[i]) : 0;
    Off vtOff = 0;
    for (Off cand : m_vtables) {
      const uint8_t *p = m_buf.data() + (m_buf.size() - cand);
      uint16_t len;
      std::memcpy(&len, p, 2);
      if (len == vt[0] && std::memcmp(p, vt.data(), len) == 0) { vtOff = cand; break; }
    }
    if (!vtOff) {
      push(vt.data(), vt.size() * 2);
      vtOff = used();
      m_vtables.push_back(vtOff);
    }
    const int32_t soff = static_cast<int32_t>(static_cast<int64_t>(vtOff) - static_cast<int64_t>(table));
    std::memcpy(m_buf.data() + (m_buf.size() - table), &soff, 4);
    return table;
  }

  // Ends the buffer: root offset, file identifier; the total size is a multiple of the largest alignment used.
  // `identifier` may be null for a schema that declares none.
  std::vector<uint8_t> finish(Off root, const char *identifier) {
    prep(m_minAlign, identifier ? 8 : 4);
    if (identifier) push(identifier, 4);
    placeUOffset(root);
    return std::vector<uint8_t>(m_buf.begin() + static_cast<std::ptrdiff_t>(m_head), m_buf.end());
  }

private:
  Off used() const { return static_cast<Off>(m_buf.size() - m_head); }
  void ensure(size_t n) {
    if (m_head >= n) return;
    const size_t usedBytes = m_buf.size() - m_head;
    size_t cap = m_buf.size();
    while (cap - usedBytes < n) cap *= 2;
    if (cap > 0x7FFFFFFFu) fail(Status::Internal, "flatbuffer exceeds 2 GiB");
    std::vector<uint8_t> nb(cap);
    std::memcpy(nb.data() + (cap - usedBytes), m_buf.data() + m_head, usedBytes);
    m_buf.swap(nb);
    m_head = cap - usedBytes;
  }
  // after `additional` more bytes the write position is aligned to `size`
  void prep(size_t size, size_t additional) {
    if (size > m_minAlign) m_minAlign = size;
    const size_t pad = (~(static_cast<size_t>(used()) + additional) + 1) & (size - 1);
    ensure(pad + size + additional);
    for (size_t i = 0; i < pad; ++i) m_buf[--m_head] = 0;
  }
  void push8(uint8_t v) { ensure(1); m_buf[--m_head] = v; }
  void push(const void *p, size_t n) {
    ensure(n);
    m_head -= n;
    if (n) std::memcpy(m_buf.data() + m_head, p, n);
  }
  template <typename T> void place(T v) { push(&v, sizeof(T)); }
  void placeUOffset(Off target) {
    if (target == 0 || target > used()) fail(Status::Internal, "flatbuffer offset to an object that is not written yet");
    place<uint32_t>(used() + 4 - target);
  }

  std::vector<uint8_t> m_buf;
  size_t m_head;
  size_t m_minAlign = 4;
  std::vector<Off> m_slots;
  Off m_objEnd = 0;
  std::vector<Off> m_vtables;
};

// ------------------------------------------------------------------------------------------------ checked reading

struct Buf {
  const uint8_t *p = nullptr;
  size_t n = 0;
  // Bytes of tables, vectors and strings handed out so far.  Offsets may legally point at shared objects, so a small
  // file can describe a huge object graph (a long vector whose elements all name one large table); a reader that
  // copies what it visits would be made to allocate without bound.  Every object visited is charged here and the walk
  // stops at a multiple of the buffer size that no honest file, whose objects are visited a few times each, reaches.
  size_t *spent = nullptr;
  void charge(size_t bytes) const {
    if (!spent) return;
    *spent += bytes + 4;
    if (*spent > 16 * n + (1u << 16)) fail(Status::InvalidModel, "flatbuffer: object graph larger than the buffer allows");
  }
  void check(size_t pos, size_t len, size_t align) const {
    if (pos > n || len > n - pos) fail(Status::InvalidModel, "flatbuffer: object outside the buffer");
    if (align > 1 && (pos & (align - 1))) fail(Status::InvalidModel, "flatbuffer: misaligned object");
  }
  template <typename T> T rd(size_t pos) const {
    check(pos, sizeof(T), sizeof(T));
    T v;
    std::memcpy(&v, p + pos, sizeof(T));
    return v;
  }
  // position an uoffset at `loc` points to
  size_t follow(size_t loc) const {
    const uint32_t u = rd<uint32_t>(loc);
    if (u == 0 || u > n - loc) fail(Status::InvalidModel, "flatbuffer: offset outside the buffer");
    return loc + u;
  }
};

class Table;

class Vector {
public:
  Vector() = default;
  Vector(Buf b, size_t pos, size_t elemSize, size_t align) : m_b(b), m_elem(elemSize), m_present(true) {
    m_len = b.rd<uint32_t>(pos);
    m_data = pos + 4;
    if (elemSize && m_len > (b.n - m_data) / elemSize) fail(Status::InvalidModel, "flatbuffer: vector longer than the buffer");
    b.check(m_data, static_cast<size_t>(m_len) * elemSize, align);
    b.charge(static_cast<size_t>(m_len) * elemSize);
  }
  bool present() const { return m_present; }
  uint32_t size() const { return m_len; }
  const uint8_t *data() const { return m_b.p + m_data; }
  template <typename T> T get(uint32_t i) const {
    if (i >= m_len || sizeof(T) > m_elem) fail(Status::InvalidModel, "flatbuffer: vector index out of range");
    T v;
    std::memcpy(&v, m_b.p + m_data + static_cast<size_t>(i) * m_elem, sizeof(T));
    return v;
  }
  // byte `off` of struct element i
  template <typename T> T member(uint32_t i, size_t off) const {
    if (i >= m_len || off + sizeof(T) > m_elem) fail(Status::InvalidModel, "flatbuffer: struct member out of range");
    T v;
    std::memcpy(&v, m_b.p + m_data + static_cast<size_t>(i) * m_elem + off, sizeof(T));
    return v;
  }
  inline Table table(uint32_t i) const;

private:
  Buf m_b;
  size_t m_data = 0, m_elem = 0;
  uint32_t m_len = 0;
  bool m_present = false;
};

class Table {
public:
  Table() = default;
  Table(Buf b, size_t pos) : m_b(b), m_pos(pos), m_present(true) {
    const int32_t soff = b.rd<int32_t>(pos);
    const int64_t vt = static_cast<int64_t>(pos) - soff;
    if (vt < 0 || static_cast<uint64_t>(vt) > b.n) fail(Status::InvalidModel, "flatbuffer: vtable outside the buffer");
    m_vt = static_cast<size_t>(vt);
    m_vtSize = b.rd<uint16_t>(m_vt);
    if (m_vtSize < 4 || (m_vtSize & 1)) fail(Status::InvalidModel, "flatbuffer: bad vtable size");
    b.check(m_vt, m_vtSize, 2);
    m_tblSize = b.rd<uint16_t>(m_vt + 2);
    if (m_tblSize < 4) fail(Status::InvalidModel, "flatbuffer: bad table size");
    b.check(pos, m_tblSize, 4);
    b.charge(m_tblSize);
  }
  // `identifier` may be null for a schema that declares none.
  // `spent` (optional) is the caller's counter for Buf::charge; it must outlive every view made from the root.
  static Table root(const void *data, size_t size, const char *identifier, size_t *spent = nullptr) {
    Buf b{static_cast<const uint8_t *>(data), size, spent};
    if (spent) *spent = 0;
    if (!data || size < 12) fail(Status::InvalidModel, "flatbuffer: buffer too short");
    if (size > 0x7FFFFFFFu) fail(Status::InvalidModel, "flatbuffer: buffer exceeds 2 GiB");
    if (identifier && std::memcmp(b.p + 4, identifier, 4) != 0) fail(Status::InvalidModel, std::string("flatbuffer: file identifier is not '") + std::string(identifier, 4) + "'");
    return Table(b, b.follow(0));
  }
  bool present() const { return m_present; }
  bool has(unsigned slot) const { return m_present && fieldOffset(slot) != 0; }
  template <typename T> T scalar(unsigned slot, T def) const {
    const size_t o = m_present ? fieldOffset(slot) : 0;
    if (!o) return def;
    if (o + sizeof(T) > m_tblSize) fail(Status::InvalidModel, "flatbuffer: field outside its table");
    return m_b.rd<T>(m_pos + o);
  }
  Table table(unsigned slot) const {
    const size_t loc = offsetField(slot);
    return loc ? Table(m_b, m_b.follow(loc)) : Table();
  }
  Vector vector(unsigned slot, size_t elemSize, size_t align) const {
    const size_t loc = offsetField(slot);
    return loc ? Vector(m_b, m_b.follow(loc), elemSize, align) : Vector();
  }
  // "" when absent
  std::string str(unsigned slot) const {
    const size_t loc = offsetField(slot);
    if (!loc) return {};
    const size_t pos = m_b.follow(loc);
    const uint32_t len = m_b.rd<uint32_t>(pos);
    m_b.check(pos + 4, static_cast<size_t>(len) + 1, 1);
    if (m_b.p[pos + 4 + len] != 0) fail(Status::InvalidModel, "flatbuffer: string without terminator");
    m_b.charge(len);
    return std::string(reinterpret_cast<const char *>(m_b.p + pos + 4), len);
  }
  Buf buf() const { return m_b; }

private:
  size_t fieldOffset(unsigned slot) const {
    const size_t e = 4 + 2 * static_cast<size_t>(slot);
    if (e + 2 > m_vtSize) return 0;
    uint16_t o;
    std::memcpy(&o, m_b.p + m_vt + e, 2);
    if (o != 0 && (o < 4 || o >= m_tblSize)) fail(Status::InvalidModel, "flatbuffer: field offset outside its table");
    return o;
  }
  size_t offsetField(unsigned slot) const {
    const size_t o = m_present ? fieldOffset(slot) : 0;
    if (!o) return 0;
    if (o + 4 > m_tblSize) fail(Status::InvalidModel, "flatbuffer: field outside its table");
    return m_pos + o;
  }
  Buf m_b;
  size_t m_pos = 0, m_vt = 0;
  uint16_t m_vtSize = 0, m_tblSize = 0;
  bool m_present = false;
};

inline Table Vector::table(uint32_t i) const {
  if (i >= m_len || m_elem != 4) fail(Status::InvalidModel, "flatbuffer: vector index out of range");
  return Table(m_b, m_b.follow(m_data + 4 * static_cast<size_t>(i)));
}

} // namespace denox::fb
