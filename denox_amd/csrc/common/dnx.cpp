#include "dnx.hpp"
#include <cstring>

namespace denox::dnx {

namespace {
constexpr uint32_t MAGIC = 0x48584E44u; // "DNXH"
constexpr uint32_t FORMAT = 1;

struct Writer {
  std::vector<uint8_t> b;
  void raw(const void *p, size_t n) { const uint8_t *c = static_cast<const uint8_t *>(p); b.insert(b.end(), c, c + n); }
  void u8(uint8_t v) { b.push_back(v); }
  void u16(uint16_t v) { raw(&v, 2); }
  void u32(uint32_t v) { raw(&v, 4); }
  void i64(int64_t v) { raw(&v, 8); }
  void str(const std::string &s) { u32(static_cast<uint32_t>(s.size())); raw(s.data(), s.size()); }
  void bytes(const std::vector<uint8_t> &v) { i64(static_cast<int64_t>(v.size())); raw(v.data(), v.size()); }
  void src(const ScalarSource &s) { u8(s.symbolic ? 1 : 0); u8(static_cast<uint8_t>(s.dtype)); i64(s.value); }
};

struct Reader {
  const uint8_t *p; size_t n, pos = 0;
  void need(size_t k) { if (k > n - pos) fail(Status::InvalidModel, "dnx stream truncated"); }
  void raw(void *d, size_t k) { need(k); std::memcpy(d, p + pos, k); pos += k; }
  uint8_t u8() { uint8_t v; raw(&v, 1); return v; }
  uint16_t u16() { uint16_t v; raw(&v, 2); return v; }
  uint32_t u32() { uint32_t v; raw(&v, 4); return v; }
  int64_t i64() { int64_t v; raw(&v, 8); return v; }
  // element counts are bounded by the bytes left, so a corrupt count cannot trigger a huge allocation
  uint32_t count(size_t minElemBytes) { uint32_t c = u32(); if (static_cast<size_t>(c) * minElemBytes > n - pos) fail(Status::InvalidModel, "dnx element count exceeds stream"); return c; }
  std::string str() { uint32_t k = u32(); need(k); std::string s(reinterpret_cast<const char *>(p + pos), k); pos += k; return s; }
  std::vector<uint8_t> bytes() { int64_t k = i64(); if (k < 0) fail(Status::InvalidModel, "negative blob size"); need(static_cast<size_t>(k)); std::vector<uint8_t> v(p + pos, p + pos + k); pos += static_cast<size_t>(k); return v; }
  ScalarSource src() {
    ScalarSource s; uint8_t sym = u8(); uint8_t dt = u8();
    if (sym > 1 || dt > 8) fail(Status::InvalidModel, "bad scalar source");
    s.symbolic = sym != 0; s.dtype = static_cast<ScalarType>(dt); s.value = i64(); return s;
  }
};
} // namespace

std::vector<uint8_t> serialize(const Model &m) {
  Writer w;
  w.u32(MAGIC); w.u32(FORMAT); w.u16(m.version);
  w.str(m.info.producer); w.str(m.info.producer_version); w.str(m.info.model_version);
  w.u32(m.sym_ir.varCount); w.u32(static_cast<uint32_t>(m.sym_ir.ops.size()));
  for (const auto &o : m.sym_ir.ops) { w.u16(o.opcode); w.i64(o.lhs); w.i64(o.rhs); }
  w.u32(static_cast<uint32_t>(m.value_names.size()));
  for (const auto &v : m.value_names) { w.str(v.name); w.src(v.value); }
  w.u32(static_cast<uint32_t>(m.buffers.size()));
  for (const auto &b : m.buffers) { w.src(b.size); w.u16(b.alignment); }
  w.u32(static_cast<uint32_t>(m.tensors.size()));
  for (const auto &t : m.tensors) {
    w.u32(t.buffer); w.src(t.offset); w.src(t.size);
    w.u8(t.info.has_extent ? 1 : 0); w.src(t.info.width); w.src(t.info.height); w.src(t.info.channels);
    w.u16(static_cast<uint16_t>(t.info.format)); w.u16(static_cast<uint16_t>(t.info.storage));
    w.u8(static_cast<uint8_t>(t.info.type)); w.str(t.info.name);
  }
  w.u32(static_cast<uint32_t>(m.initializers.size()));
  for (const auto &i : m.initializers) { w.u32(i.tensor); w.bytes(i.data); }
  w.u32(static_cast<uint32_t>(m.inputs.size())); for (uint32_t i : m.inputs) w.u32(i);
  w.u32(static_cast<uint32_t>(m.outputs.size())); for (uint32_t o : m.outputs) w.u32(o);
  w.u32(static_cast<uint32_t>(m.shader_binaries.size()));
  for (const auto &s : m.shader_binaries) w.bytes(s.code_object);
  w.u32(static_cast<uint32_t>(m.dispatches.size()));
  for (const auto &d : m.dispatches) {
    w.u32(d.binary_id); w.src(d.workgroup_count_x); w.src(d.workgroup_count_y); w.src(d.workgroup_count_z);
    for (int i = 0; i < 3; ++i) w.u32(d.workgroup_size[i]);
    w.str(d.entry_point);
    w.u32(static_cast<uint32_t>(d.bindings.size()));
    for (const auto &s : d.bindings) {
      w.u16(s.set); w.u32(static_cast<uint32_t>(s.bindings.size()));
      for (const auto &b : s.bindings) { w.u16(b.binding); w.u8(static_cast<uint8_t>(b.access)); w.u32(b.tensor); }
    }
    w.u16(d.push_constant.size); w.u32(static_cast<uint32_t>(d.push_constant.fields.size()));
    for (const auto &f : d.push_constant.fields) { w.u8(static_cast<uint8_t>(f.dtype)); w.u16(f.offset); w.src(f.source); }
    w.str(d.info.name); w.str(d.info.debug_info); w.str(d.info.src_path);
    w.u8(d.info.has_reads); w.src(d.info.memory_reads);
    w.u8(d.info.has_writes); w.src(d.info.memory_writes);
    w.u8(d.info.has_flops); w.src(d.info.flops);
  }
  w.u32(MAGIC); // trailer: catches truncation at a record boundary
  return std::move(w.b);
}

Model deserialize(const void *data, size_t size) {
  if (!data || size < 12) fail(Status::InvalidModel, "dnx stream too short");
  Reader r{static_cast<const uint8_t *>(data), size};
  if (r.u32() != MAGIC) fail(Status::InvalidModel, "not a dnx stream (bad magic)");
  if (r.u32() != FORMAT) fail(Status::InvalidModel, "unsupported dnx format version");
  Model m;
  m.version = r.u16();
  m.info.producer = r.str(); m.info.producer_version = r.str(); m.info.model_version = r.str();
  m.sym_ir.varCount = r.u32();
  if (m.sym_ir.varCount > 0xFFFF) fail(Status::InvalidModel, "var_count exceeds uint16");
  uint32_t n = r.count(18);
  m.sym_ir.ops.resize(n);
  for (auto &o : m.sym_ir.ops) { o.opcode = r.u16(); o.lhs = r.i64(); o.rhs = r.i64(); }
  n = r.count(14); m.value_names.resize(n);
  for (auto &v : m.value_names) { v.name = r.str(); v.value = r.src(); }
  n = r.count(12); m.buffers.resize(n);
  for (auto &b : m.buffers) { b.size = r.src(); b.alignment = r.u16(); }
  n = r.count(64); m.tensors.resize(n);
  for (auto &t : m.tensors) {
    t.buffer = r.u32(); t.offset = r.src(); t.size = r.src();
    t.info.has_extent = r.u8() != 0; t.info.width = r.src(); t.info.height = r.src(); t.info.channels = r.src();
    uint16_t f = r.u16(), s = r.u16(); uint8_t ty = r.u8();
    if (f > 7 || s > 2 || ty > 8) fail(Status::InvalidModel, "bad tensor enum");
    t.info.format = static_cast<TensorFormat>(f); t.info.storage = static_cast<TensorStorage>(s); t.info.type = static_cast<ScalarType>(ty);
    t.info.name = r.str();
  }
  n = r.count(12); m.initializers.resize(n);
  for (auto &i : m.initializers) { i.tensor = r.u32(); i.data = r.bytes(); }
  n = r.count(4); m.inputs.resize(n); for (auto &i : m.inputs) i = r.u32();
  n = r.count(4); m.outputs.resize(n); for (auto &o : m.outputs) o = r.u32();
  n = r.count(8); m.shader_binaries.resize(n);
  for (auto &s : m.shader_binaries) s.code_object = r.bytes();
  n = r.count(64); m.dispatches.resize(n);
  for (auto &d : m.dispatches) {
    d.binary_id = r.u32(); d.workgroup_count_x = r.src(); d.workgroup_count_y = r.src(); d.workgroup_count_z = r.src();
    for (int i = 0; i < 3; ++i) d.workgroup_size[i] = r.u32();
    d.entry_point = r.str();
    uint32_t ns = r.count(6); d.bindings.resize(ns);
    for (auto &s : d.bindings) {
      s.set = r.u16(); uint32_t nb = r.count(7); s.bindings.resize(nb);
      for (auto &b : s.bindings) { b.binding = r.u16(); uint8_t a = r.u8(); if (a > 2) fail(Status::InvalidModel, "bad access"); b.access = static_cast<Access>(a); b.tensor = r.u32(); }
    }
    d.push_constant.size = r.u16(); uint32_t nf = r.count(13); d.push_constant.fields.resize(nf);
    for (auto &f : d.push_constant.fields) { uint8_t dt = r.u8(); if (dt > 8) fail(Status::InvalidModel, "bad field dtype"); f.dtype = static_cast<ScalarType>(dt); f.offset = r.u16(); f.source = r.src(); }
    d.info.name = r.str(); d.info.debug_info = r.str(); d.info.src_path = r.str();
    d.info.has_reads = r.u8() != 0; d.info.memory_reads = r.src();
    d.info.has_writes = r.u8() != 0; d.info.memory_writes = r.src();
    d.info.has_flops = r.u8() != 0; d.info.flops = r.src();
  }
  if (r.u32() != MAGIC) fail(Status::InvalidModel, "dnx trailer missing");
  if (r.pos != size) fail(Status::InvalidModel, "trailing bytes after dnx stream");
  validate(m);
  return m;
}

void validate(const Model &m) {
  const size_t nsym = m.sym_ir.varCount + m.sym_ir.ops.size();
  auto chk = [&](const ScalarSource &s) {
    if (s.symbolic && (s.value < 0 || static_cast<size_t>(s.value) >= nsym)) fail(Status::InvalidModel, "symbol reference out of range");
  };
  for (size_t pc = 0; pc < m.sym_ir.ops.size(); ++pc) {
    const auto &o = m.sym_ir.ops[pc];
    const uint16_t base = o.opcode & 0x3FFF;
    if (base < SYM_ADD || base > SYM_MAX) fail(Status::InvalidModel, "SymIR opcode invalid");
    const size_t lim = m.sym_ir.varCount + pc;
    if ((o.opcode & SYM_LHSC) && (o.opcode & SYM_RHSC)) fail(Status::InvalidModel, "SymIR op with two constants");
    if (!(o.opcode & SYM_LHSC) && (o.lhs < 0 || static_cast<size_t>(o.lhs) >= lim)) fail(Status::InvalidModel, "SymIR forward reference");
    if (!(o.opcode & SYM_RHSC) && (o.rhs < 0 || static_cast<size_t>(o.rhs) >= lim)) fail(Status::InvalidModel, "SymIR forward reference");
  }
  for (const auto &v : m.value_names) chk(v.value);
  for (const auto &b : m.buffers) { chk(b.size); if (b.alignment == 0) fail(Status::InvalidModel, "zero buffer alignment"); }
  for (const auto &t : m.tensors) {
    if (t.buffer >= m.buffers.size()) fail(Status::InvalidModel, "tensor references missing buffer");
    chk(t.offset); chk(t.size); chk(t.info.width); chk(t.info.height); chk(t.info.channels);
  }
  for (const auto &i : m.initializers) if (i.tensor >= m.tensors.size()) fail(Status::InvalidModel, "initializer references missing tensor");
  for (uint32_t i : m.inputs) if (i >= m.tensors.size()) fail(Status::InvalidModel, "input references missing tensor");
  for (uint32_t o : m.outputs) if (o >= m.tensors.size()) fail(Status::InvalidModel, "output references missing tensor");
  for (const auto &d : m.dispatches) {
    if (d.binary_id >= m.shader_binaries.size()) fail(Status::InvalidModel, "dispatch references missing binary");
    if (d.entry_point.empty()) fail(Status::InvalidModel, "dispatch without entry point");
    chk(d.workgroup_count_x); chk(d.workgroup_count_y); chk(d.workgroup_count_z);
    const uint64_t threads = static_cast<uint64_t>(d.workgroup_size[0]) * d.workgroup_size[1] * d.workgroup_size[2];
    if (threads == 0 || threads > 1024) fail(Status::InvalidModel, "workgroup size outside 1..1024");
    for (const auto &s : d.bindings) for (const auto &b : s.bindings) if (b.tensor >= m.tensors.size()) fail(Status::InvalidModel, "binding references missing tensor");
    for (const auto &f : d.push_constant.fields) {
      chk(f.source);
      if (f.offset + scalarSize(f.dtype) > d.push_constant.size) fail(Status::InvalidModel, "push constant field outside range");
    }
    chk(d.info.memory_reads); chk(d.info.memory_writes); chk(d.info.flops);
  }
}

} // namespace denox::dnx
