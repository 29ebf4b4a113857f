#include "dnx.hpp"
#include "flatbuf.hpp"
#include <cstring>

namespace denox::dnx {

namespace {

// Field ids: the declaration order of each table in dnx.fbs; a union field takes two (its member index, then the member).
namespace id {
enum SymRef { SymRef_sid = 0 };                                                   // dnx.fbs:18-20
enum ScalarLiteral { Lit_dtype = 0, Lit_bytes = 1 };                              // dnx.fbs:22-25
enum PushConstantField { PCF_dtype = 0, PCF_offset = 1, PCF_source_type = 2, PCF_source = 3 }; // dnx.fbs:32-36
enum PushConstant { PC_size = 0, PC_fields = 1 };                                 // dnx.fbs:38-41
enum DescriptorBinding { DB_binding = 0, DB_access = 1, DB_tensor = 2 };          // dnx.fbs:49-53
enum DescriptorSetBinding { DSB_set = 0, DSB_bindings = 1 };                      // dnx.fbs:55-58
enum DispatchInfo { DI_name = 0, DI_debug_info = 1, DI_src_path = 2, DI_reads_type = 3, DI_reads = 4, DI_writes_type = 5, DI_writes = 6, DI_flops_type = 7, DI_flops = 8 }; // dnx.fbs:59-66
enum ComputeDispatch { CD_binary_id = 0, CD_wgx_type = 1, CD_wgx = 2, CD_wgy_type = 3, CD_wgy = 4, CD_wgz_type = 5, CD_wgz = 6, CD_entry_point = 7, CD_bindings = 8,
                       CD_push_constant = 9, CD_info = 10, CD_wgsize_x = 11, CD_wgsize_y = 12, CD_wgsize_z = 13, CD_count = 14 }; // dnx.fbs:68-78 + workgroup size
enum Buffer { Buf_size_type = 0, Buf_size = 1, Buf_alignment = 2 };               // dnx.fbs:82-85
enum TensorInfo { TI_width_type = 0, TI_width = 1, TI_height_type = 2, TI_height = 3, TI_channels_type = 4, TI_channels = 5, TI_format = 6, TI_storage = 7, TI_type = 8, TI_name = 9 }; // dnx.fbs:104-112
enum Tensor { T_buffer = 0, T_offset_type = 1, T_offset = 2, T_size_type = 3, T_size = 4, T_info = 5 }; // dnx.fbs:114-119
enum SymIR { SI_var_count = 0, SI_ops = 1 };                                      // dnx.fbs:140-143
enum TensorInitializer { TIn_tensor = 0, TIn_data = 1 };                          // dnx.fbs:145-148
enum ModelInfo { MI_producer = 0, MI_producer_version = 1, MI_model_version = 2 };// dnx.fbs:154-158
enum ValueName { VN_name = 0, VN_value_type = 1, VN_value = 2 };                  // dnx.fbs:164-167
enum ShaderBinary { SB_spirv = 0, SB_code_object = 1 };                           // dnx.fbs:169-171 + code object
enum Model { M_version = 0, M_required_features = 1, M_info = 2, M_tensors = 3, M_initializers = 4, M_inputs = 5, M_outputs = 6, M_buffers = 7, M_dispatches = 8,
             M_shader_binaries = 9, M_sym_ir = 10, M_value_names = 11, M_requirements = 12 }; // dnx.fbs:173-192 + requirements
enum Requirement { RQ_lhs_type = 0, RQ_lhs = 1, RQ_rhs_type = 2, RQ_rhs = 3, RQ_relation = 4, RQ_what = 5 }; // (not in dnx.fbs)
} // namespace id
constexpr uint8_t SRC_NONE = 0, SRC_LITERAL = 1, SRC_SYMBOLIC = 2;                // union ScalarSource, dnx.fbs:27-30
constexpr char IDENTIFIER[4] = {'d', 'n', 'x', 'x'};                               // dnx.fbs:4
constexpr size_t SYMOP_BYTES = 24;                                                // struct SymIROp {u16, pad, i64, i64}, dnx.fbs:134-138

struct Writer {
  fb::Builder b{1u << 20};
  // the member table of a ScalarSource: a literal keeps its dtype and little-endian bytes (serialize.cpp:137-186 of the reference)
  fb::Off source(const ScalarSource &s) {
    if (s.symbolic) {
      b.startTable(1);
      b.addScalar<uint32_t>(id::SymRef_sid, static_cast<uint32_t>(s.value), 0);
      return b.endTable();
    }
    if (s.dtype == ScalarType::F16 || s.dtype == ScalarType::F32 || s.dtype == ScalarType::F64) fail(Status::Internal, "floating-point literal in a scalar source");
    uint8_t bytes[8];
    const uint64_t v = static_cast<uint64_t>(s.value);
    for (int i = 0; i < 8; ++i) bytes[i] = static_cast<uint8_t>(v >> (8 * i));
    const fb::Off data = b.createVector(bytes, 1, 1, scalarSize(s.dtype));
    b.startTable(2);
    b.addScalar<uint8_t>(id::Lit_dtype, static_cast<uint8_t>(s.dtype), 0);
    b.addOffset(id::Lit_bytes, data);
    return b.endTable();
  }
  void addSource(unsigned typeSlot, const ScalarSource &s, fb::Off member) {
    b.addScalar<uint8_t>(typeSlot, s.symbolic ? SRC_SYMBOLIC : SRC_LITERAL, SRC_NONE);
    b.addOffset(typeSlot + 1, member);
  }
  template <typename T, typename F> fb::Off tables(const std::vector<T> &items, F &&one) {
    std::vector<fb::Off> offs(items.size());
    for (size_t i = 0; i < items.size(); ++i) offs[i] = one(items[i]);
    return b.createOffsetVector(offs);
  }
};

struct Reader {
  ScalarSource source(const fb::Table &t, unsigned typeSlot, bool *present = nullptr) {
    const uint8_t kind = t.scalar<uint8_t>(typeSlot, SRC_NONE);
    const fb::Table m = t.table(typeSlot + 1);
    if (present) *present = kind != SRC_NONE;
    ScalarSource s;
    if (kind == SRC_NONE) {
      if (!present) fail(Status::InvalidModel, "dnx: scalar source missing");
      return s;
    }
    if (!m.present()) fail(Status::InvalidModel, "dnx: scalar source without a value");
    if (kind == SRC_SYMBOLIC) {
      s.symbolic = true;
      s.value = m.scalar<uint32_t>(id::SymRef_sid, 0);
      return s;
    }
    if (kind != SRC_LITERAL) fail(Status::InvalidModel, "dnx: unknown scalar source kind");
    const uint8_t dt = m.scalar<uint8_t>(id::Lit_dtype, 0);
    if (dt > 5) fail(Status::InvalidModel, "dnx: literal of a non-integer type");
    s.dtype = static_cast<ScalarType>(dt);
    const fb::Vector bytes = m.vector(id::Lit_bytes, 1, 1);
    const size_t n = scalarSize(s.dtype);
    if (!bytes.present() || bytes.size() < n) fail(Status::InvalidModel, "dnx: literal shorter than its type");
    uint64_t v = 0;
    for (size_t i = 0; i < n; ++i) v |= static_cast<uint64_t>(bytes.get<uint8_t>(static_cast<uint32_t>(i))) << (8 * i);
    const bool isSigned = s.dtype == ScalarType::I16 || s.dtype == ScalarType::I32 || s.dtype == ScalarType::I64;
    if (isSigned && n < 8 && (v >> (8 * n - 1)) & 1) v |= ~uint64_t(0) << (8 * n);
    if (!isSigned && v > static_cast<uint64_t>(INT64_MAX)) fail(Status::InvalidModel, "dnx: literal exceeds int64");
    s.value = static_cast<int64_t>(v);
    return s;
  }
  template <typename E> E enumOf(uint64_t v, uint64_t maxValue, const char *what) {
    if (v > maxValue) fail(Status::InvalidModel, std::string("dnx: bad ") + what);
    return static_cast<E>(v);
  }
};
} // namespace

std::vector<uint8_t> serialize(const Model &m) {
  Writer w;
  fb::Builder &b = w.b;

  // children before parents: every offset in a FlatBuffer points towards the end of the buffer
  const fb::Off valueNames = w.tables(m.value_names, [&](const ValueName &v) {
    const fb::Off name = b.createString(v.name), val = w.source(v.value);
    b.startTable(3);
    b.addOffset(id::VN_name, name);
    w.addSource(id::VN_value_type, v.value, val);
    return b.endTable();
  });

  const fb::Off requirements = w.tables(m.requirements, [&](const Requirement &q) {
    const fb::Off what = b.createString(q.what), lhs = w.source(q.lhs), rhs = w.source(q.rhs);
    b.startTable(6);
    w.addSource(id::RQ_lhs_type, q.lhs, lhs);
    w.addSource(id::RQ_rhs_type, q.rhs, rhs);
    b.addScalar<uint8_t>(id::RQ_relation, q.relation, 0);
    b.addOffset(id::RQ_what, what);
    return b.endTable();
  });

  std::vector<uint8_t> ops(m.sym_ir.ops.size() * SYMOP_BYTES, 0);
  for (size_t i = 0; i < m.sym_ir.ops.size(); ++i) {
    const SymIROp &o = m.sym_ir.ops[i];
    std::memcpy(&ops[i * SYMOP_BYTES], &o.opcode, 2);
    std::memcpy(&ops[i * SYMOP_BYTES + 8], &o.lhs, 8);
    std::memcpy(&ops[i * SYMOP_BYTES + 16], &o.rhs, 8);
  }
  const fb::Off opsVec = b.createVector(ops.data(), SYMOP_BYTES, 8, m.sym_ir.ops.size());
  b.startTable(2);
  b.addScalar<uint16_t>(id::SI_var_count, static_cast<uint16_t>(m.sym_ir.varCount), 0);
  b.addOffset(id::SI_ops, opsVec);
  const fb::Off symIr = b.endTable();

  const fb::Off binaries = w.tables(m.shader_binaries, [&](const ShaderBinary &s) {
    const fb::Off spirv = b.createVector(nullptr, 4, 4, 0); // no SPIR-V: the vector the original schema declares stays empty
    const fb::Off code = b.createVector(s.code_object.data(), 1, 1, s.code_object.size());
    b.startTable(2);
    b.addOffset(id::SB_spirv, spirv);
    b.addOffset(id::SB_code_object, code);
    return b.endTable();
  });

  const fb::Off dispatches = w.tables(m.dispatches, [&](const ComputeDispatch &d) {
    const fb::Off name = b.createString(d.info.name), dbg = b.createString(d.info.debug_info), src = b.createString(d.info.src_path);
    const fb::Off reads = d.info.has_reads ? w.source(d.info.memory_reads) : 0, writes = d.info.has_writes ? w.source(d.info.memory_writes) : 0,
                  flops = d.info.has_flops ? w.source(d.info.flops) : 0;
    b.startTable(9);
    b.addOffset(id::DI_name, name);
    b.addOffset(id::DI_debug_info, dbg);
    b.addOffset(id::DI_src_path, src);
    if (reads) w.addSource(id::DI_reads_type, d.info.memory_reads, reads);
    if (writes) w.addSource(id::DI_writes_type, d.info.memory_writes, writes);
    if (flops) w.addSource(id::DI_flops_type, d.info.flops, flops);
    const fb::Off info = b.endTable();

    const fb::Off fields = w.tables(d.push_constant.fields, [&](const PushConstantField &f) {
      const fb::Off val = w.source(f.source);
      b.startTable(4);
      b.addScalar<uint8_t>(id::PCF_dtype, static_cast<uint8_t>(f.dtype), 0);
      b.addScalar<uint16_t>(id::PCF_offset, f.offset, 0);
      w.addSource(id::PCF_source_type, f.source, val);
      return b.endTable();
    });
    b.startTable(2);
    b.addScalar<uint16_t>(id::PC_size, d.push_constant.size, 0);
    b.addOffset(id::PC_fields, fields);
    const fb::Off pc = b.endTable();

    const fb::Off sets = w.tables(d.bindings, [&](const DescriptorSetBinding &s) {
      const fb::Off bs = w.tables(s.bindings, [&](const DescriptorBinding &x) {
        b.startTable(3);
        b.addScalar<uint16_t>(id::DB_binding, x.binding, 0);
        b.addScalar<uint8_t>(id::DB_access, static_cast<uint8_t>(x.access), 0);
        b.addScalar<uint32_t>(id::DB_tensor, x.tensor, 0);
        return b.endTable();
      });
      b.startTable(2);
      b.addScalar<uint16_t>(id::DSB_set, s.set, 0);
      b.addOffset(id::DSB_bindings, bs);
      return b.endTable();
    });
    const fb::Off entry = b.createString(d.entry_point);
    const fb::Off gx = w.source(d.workgroup_count_x), gy = w.source(d.workgroup_count_y), gz = w.source(d.workgroup_count_z);
    b.startTable(id::CD_count);
    b.addScalar<uint32_t>(id::CD_binary_id, d.binary_id, 0);
    w.addSource(id::CD_wgx_type, d.workgroup_count_x, gx);
    w.addSource(id::CD_wgy_type, d.workgroup_count_y, gy);
    w.addSource(id::CD_wgz_type, d.workgroup_count_z, gz);
    b.addOffset(id::CD_entry_point, entry);
    b.addOffset(id::CD_bindings, sets);
    b.addOffset(id::CD_push_constant, pc);
    b.addOffset(id::CD_info, info);
    b.addScalar<uint32_t>(id::CD_wgsize_x, d.workgroup_size[0], 0);
    b.addScalar<uint32_t>(id::CD_wgsize_y, d.workgroup_size[1], 0);
    b.addScalar<uint32_t>(id::CD_wgsize_z, d.workgroup_size[2], 0);
    return b.endTable();
  });

  const fb::Off buffers = w.tables(m.buffers, [&](const Buffer &x) {
    const fb::Off size = w.source(x.size);
    b.startTable(3);
    w.addSource(id::Buf_size_type, x.size, size);
    b.addScalar<uint16_t>(id::Buf_alignment, x.alignment, 0);
    return b.endTable();
  });
  const fb::Off outputs = b.createVector(m.outputs.data(), 4, 4, m.outputs.size());
  const fb::Off inputs = b.createVector(m.inputs.data(), 4, 4, m.inputs.size());
  const fb::Off initializers = w.tables(m.initializers, [&](const TensorInitializer &x) {
    const fb::Off data = b.createVector(x.data.data(), 1, 1, x.data.size());
    b.startTable(2);
    b.addScalar<uint32_t>(id::TIn_tensor, x.tensor, 0);
    b.addOffset(id::TIn_data, data);
    return b.endTable();
  });
  const fb::Off tensors = w.tables(m.tensors, [&](const Tensor &t) {
    const fb::Off name = b.createString(t.info.name);
    fb::Off wd = 0, ht = 0, ch = 0;
    if (t.info.has_extent) { wd = w.source(t.info.width); ht = w.source(t.info.height); ch = w.source(t.info.channels); }
    b.startTable(10);
    if (t.info.has_extent) {
      w.addSource(id::TI_width_type, t.info.width, wd);
      w.addSource(id::TI_height_type, t.info.height, ht);
      w.addSource(id::TI_channels_type, t.info.channels, ch);
    }
    b.addScalar<uint16_t>(id::TI_format, static_cast<uint16_t>(t.info.format), 0);
    b.addScalar<uint16_t>(id::TI_storage, static_cast<uint16_t>(t.info.storage), 0);
    b.addScalar<uint8_t>(id::TI_type, static_cast<uint8_t>(t.info.type), 0);
    b.addOffset(id::TI_name, name);
    const fb::Off info = b.endTable();
    const fb::Off off = w.source(t.offset), size = w.source(t.size);
    b.startTable(6);
    b.addScalar<uint32_t>(id::T_buffer, t.buffer, 0);
    w.addSource(id::T_offset_type, t.offset, off);
    w.addSource(id::T_size_type, t.size, size);
    b.addOffset(id::T_info, info);
    return b.endTable();
  });
  const fb::Off producer = b.createString(m.info.producer), producerVersion = b.createString(m.info.producer_version), modelVersion = b.createString(m.info.model_version);
  b.startTable(3);
  b.addOffset(id::MI_producer, producer);
  b.addOffset(id::MI_producer_version, producerVersion);
  b.addOffset(id::MI_model_version, modelVersion);
  const fb::Off info = b.endTable();
  const fb::Off features = b.createVector(m.required_features.data(), 4, 4, m.required_features.size());

  b.startTable(13);
  b.addScalar<uint16_t>(id::M_version, m.version, 0);
  b.addOffset(id::M_required_features, features);
  b.addOffset(id::M_info, info);
  b.addOffset(id::M_tensors, tensors);
  b.addOffset(id::M_initializers, initializers);
  b.addOffset(id::M_inputs, inputs);
  b.addOffset(id::M_outputs, outputs);
  b.addOffset(id::M_buffers, buffers);
  b.addOffset(id::M_dispatches, dispatches);
  b.addOffset(id::M_shader_binaries, binaries);
  b.addOffset(id::M_sym_ir, symIr);
  b.addOffset(id::M_value_names, valueNames);
  if (!m.requirements.empty()) b.addOffset(id::M_requirements, requirements);
  return b.finish(b.endTable(), IDENTIFIER);
}

void Model::checkRequirements(const std::vector<int64_t> &dp) const {
  for (const auto &q : requirements) {
    const int64_t a = q.lhs.eval(dp), b = q.rhs.eval(dp);
    if (q.relation == 0 ? a != b : a > b)
      fail(Status::InvalidArgument, q.what + ": " + std::to_string(a) + (q.relation == 0 ? " != " : " > ") + std::to_string(b) + " at these extents");
  }
}

Model deserialize(const void *data, size_t size) {
  size_t spent = 0;
  const fb::Table root = fb::Table::root(data, size, IDENTIFIER, &spent);
  Reader r;
  Model m;
  m.version = root.scalar<uint16_t>(id::M_version, 0);
  if (m.version != 0) fail(Status::InvalidModel, "dnx: unknown format version");
  auto u32s = [](const fb::Vector &v, std::vector<uint32_t> &out) {
    out.resize(v.size());
    for (uint32_t i = 0; i < v.size(); ++i) out[i] = v.get<uint32_t>(i);
  };
  u32s(root.vector(id::M_required_features, 4, 4), m.required_features);
  const fb::Table info = root.table(id::M_info);
  m.info.producer = info.str(id::MI_producer);
  m.info.producer_version = info.str(id::MI_producer_version);
  m.info.model_version = info.str(id::MI_model_version);

  const fb::Table symIr = root.table(id::M_sym_ir);
  m.sym_ir.varCount = symIr.scalar<uint16_t>(id::SI_var_count, 0);
  const fb::Vector ops = symIr.vector(id::SI_ops, SYMOP_BYTES, 8);
  m.sym_ir.ops.resize(ops.size());
  for (uint32_t i = 0; i < ops.size(); ++i) {
    m.sym_ir.ops[i].opcode = ops.member<uint16_t>(i, 0);
    m.sym_ir.ops[i].lhs = ops.member<int64_t>(i, 8);
    m.sym_ir.ops[i].rhs = ops.member<int64_t>(i, 16);
  }

  const fb::Vector valueNames = root.vector(id::M_value_names, 4, 4);
  m.value_names.resize(valueNames.size());
  for (uint32_t i = 0; i < valueNames.size(); ++i) {
    const fb::Table t = valueNames.table(i);
    m.value_names[i].name = t.str(id::VN_name);
    m.value_names[i].value = r.source(t, id::VN_value_type);
  }

  const fb::Vector requirements = root.vector(id::M_requirements, 4, 4);
  m.requirements.resize(requirements.size());
  for (uint32_t i = 0; i < requirements.size(); ++i) {
    const fb::Table t = requirements.table(i);
    m.requirements[i].lhs = r.source(t, id::RQ_lhs_type);
    m.requirements[i].rhs = r.source(t, id::RQ_rhs_type);
    m.requirements[i].relation = t.scalar<uint8_t>(id::RQ_relation, 0);
    m.requirements[i].what = t.str(id::RQ_what);
  }

  const fb::Vector buffers = root.vector(id::M_buffers, 4, 4);
  m.buffers.resize(buffers.size());
  for (uint32_t i = 0; i < buffers.size(); ++i) {
    const fb::Table t = buffers.table(i);
    m.buffers[i].size = r.source(t, id::Buf_size_type);
    m.buffers[i].alignment = t.scalar<uint16_t>(id::Buf_alignment, 0);
  }

  const fb::Vector tensors = root.vector(id::M_tensors, 4, 4);
  m.tensors.resize(tensors.size());
  for (uint32_t i = 0; i < tensors.size(); ++i) {
    const fb::Table t = tensors.table(i);
    Tensor &x = m.tensors[i];
    x.buffer = t.scalar<uint32_t>(id::T_buffer, 0);
    x.offset = r.source(t, id::T_offset_type);
    x.size = r.source(t, id::T_size_type);
    const fb::Table ti = t.table(id::T_info);
    if (ti.present()) {
      bool hw = false, hh = false, hc = false;
      x.info.width = r.source(ti, id::TI_width_type, &hw);
      x.info.height = r.source(ti, id::TI_height_type, &hh);
      x.info.channels = r.source(ti, id::TI_channels_type, &hc);
      x.info.has_extent = hw && hh && hc;
      x.info.format = r.enumOf<TensorFormat>(ti.scalar<uint16_t>(id::TI_format, 0), 7, "tensor format");
      x.info.storage = r.enumOf<TensorStorage>(ti.scalar<uint16_t>(id::TI_storage, 0), 2, "tensor storage");
      x.info.type = r.enumOf<ScalarType>(ti.scalar<uint8_t>(id::TI_type, 0), 8, "tensor type");
      x.info.name = ti.str(id::TI_name);
    }
  }

  const fb::Vector initializers = root.vector(id::M_initializers, 4, 4);
  m.initializers.resize(initializers.size());
  for (uint32_t i = 0; i < initializers.size(); ++i) {
    const fb::Table t = initializers.table(i);
    m.initializers[i].tensor = t.scalar<uint32_t>(id::TIn_tensor, 0);
    const fb::Vector d = t.vector(id::TIn_data, 1, 1);
    if (d.present()) m.initializers[i].data.assign(d.data(), d.data() + d.size());
  }
  u32s(root.vector(id::M_inputs, 4, 4), m.inputs);
  u32s(root.vector(id::M_outputs, 4, 4), m.outputs);

  const fb::Vector binaries = root.vector(id::M_shader_binaries, 4, 4);
  m.shader_binaries.resize(binaries.size());
  for (uint32_t i = 0; i < binaries.size(); ++i) {
    const fb::Table t = binaries.table(i);
    m.shader_binaries[i].spirv_words = t.vector(id::SB_spirv, 4, 4).size();
    const fb::Vector code = t.vector(id::SB_code_object, 1, 1);
    if (code.present()) m.shader_binaries[i].code_object.assign(code.data(), code.data() + code.size());
  }

  const fb::Vector dispatches = root.vector(id::M_dispatches, 4, 4);
  m.dispatches.resize(dispatches.size());
  for (uint32_t i = 0; i < dispatches.size(); ++i) {
    const fb::Table t = dispatches.table(i);
    ComputeDispatch &d = m.dispatches[i];
    d.binary_id = t.scalar<uint32_t>(id::CD_binary_id, 0);
    d.workgroup_count_x = r.source(t, id::CD_wgx_type);
    d.workgroup_count_y = r.source(t, id::CD_wgy_type);
    d.workgroup_count_z = r.source(t, id::CD_wgz_type);
    d.workgroup_size[0] = t.scalar<uint32_t>(id::CD_wgsize_x, 0);
    d.workgroup_size[1] = t.scalar<uint32_t>(id::CD_wgsize_y, 0);
    d.workgroup_size[2] = t.scalar<uint32_t>(id::CD_wgsize_z, 0);
    d.entry_point = t.str(id::CD_entry_point);
    const fb::Vector sets = t.vector(id::CD_bindings, 4, 4);
    d.bindings.resize(sets.size());
    for (uint32_t s = 0; s < sets.size(); ++s) {
      const fb::Table st = sets.table(s);
      d.bindings[s].set = st.scalar<uint16_t>(id::DSB_set, 0);
      const fb::Vector bs = st.vector(id::DSB_bindings, 4, 4);
      d.bindings[s].bindings.resize(bs.size());
      for (uint32_t k = 0; k < bs.size(); ++k) {
        const fb::Table bt = bs.table(k);
        DescriptorBinding &x = d.bindings[s].bindings[k];
        x.binding = bt.scalar<uint16_t>(id::DB_binding, 0);
        x.access = r.enumOf<Access>(bt.scalar<uint8_t>(id::DB_access, 0), 2, "access");
        x.tensor = bt.scalar<uint32_t>(id::DB_tensor, 0);
      }
    }
    const fb::Table pc = t.table(id::CD_push_constant);
    d.push_constant.size = pc.scalar<uint16_t>(id::PC_size, 0);
    const fb::Vector fields = pc.vector(id::PC_fields, 4, 4);
    d.push_constant.fields.resize(fields.size());
    for (uint32_t k = 0; k < fields.size(); ++k) {
      const fb::Table ft = fields.table(k);
      PushConstantField &f = d.push_constant.fields[k];
      f.dtype = r.enumOf<ScalarType>(ft.scalar<uint8_t>(id::PCF_dtype, 0), 8, "push constant type");
      f.offset = ft.scalar<uint16_t>(id::PCF_offset, 0);
      f.source = r.source(ft, id::PCF_source_type);
    }
    const fb::Table di = t.table(id::CD_info);
    d.info.name = di.str(id::DI_name);
    d.info.debug_info = di.str(id::DI_debug_info);
    d.info.src_path = di.str(id::DI_src_path);
    if (di.present()) {
      d.info.memory_reads = r.source(di, id::DI_reads_type, &d.info.has_reads);
      d.info.memory_writes = r.source(di, id::DI_writes_type, &d.info.has_writes);
      d.info.flops = r.source(di, id::DI_flops_type, &d.info.has_flops);
    }
  }
  validate(m);
  return m;
}

void requireExecutable(const Model &m) {
  for (const auto &d : m.dispatches) {
    const ShaderBinary &s = m.shader_binaries[d.binary_id]; // index checked by validate
    if (s.code_object.empty())
      fail(Status::Unsupported, s.spirv_words ? "dnx: dispatch '" + d.info.name + "' is compiled to SPIR-V; this runtime launches gfx950 code objects only"
                                              : "dnx: dispatch '" + d.info.name + "' has no code object");
    const uint64_t threads = static_cast<uint64_t>(d.workgroup_size[0]) * d.workgroup_size[1] * d.workgroup_size[2];
    if (threads == 0 || threads > 1024) fail(Status::InvalidModel, "workgroup size outside 1..1024");
  }
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
  for (const auto &q : m.requirements) {
    chk(q.lhs);
    chk(q.rhs);
    if (q.relation > 1) fail(Status::InvalidModel, "dnx: unknown relation in a requirement");
  }
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
    for (const auto &s : d.bindings) for (const auto &b : s.bindings) if (b.tensor >= m.tensors.size()) fail(Status::InvalidModel, "binding references missing tensor");
    for (const auto &f : d.push_constant.fields) {
      chk(f.source);
      if (f.offset + scalarSize(f.dtype) > d.push_constant.size) fail(Status::InvalidModel, "push constant field outside range");
    }
    chk(d.info.memory_reads); chk(d.info.memory_writes); chk(d.info.flops);
  }
}

} // namespace denox::dnx
