// In-memory form and byte serialisation of a compiled model ("dnx").
//
// The bytes are a FlatBuffer of the reference's schema dnx.fbs:1-195 (file identifier "dnxx", root table Model), written
// and read by hand over common/flatbuf.hpp: field ids are the declaration order of each table, a union takes two ids
// (member index, then the member).  A HIP backend needs two things the schema does not hold, and both are added the way
// FlatBuffers schemas evolve -- new fields at the end of a table, which a reader generated from the original schema skips:
//   * ShaderBinary.code_object:[ubyte] (id 1, after spirv): a gfx950 code object instead of SPIR-V words
//     (dnx.fbs:169-171);
//   * ComputeDispatch.workgroup_size_{x,y,z}:uint (ids 11-13, after info): SPIR-V bakes the workgroup size into the
//     module as local_size, a HIP launch takes it as an argument;
//   * RuntimeFeature gains HipCodeObject = 1 (dnx.fbs:160-162), listed in required_features of every model written here.
// A model written by the reference (SPIR-V only) parses and can be described; running it reports UNSUPPORTED.
#pragma once
#include "error.hpp"
#include "sym.hpp"
#include <cstdint>
#include <string>
#include <vector>

namespace denox::dnx {

enum class ScalarType : uint8_t { I16 = 0, U16 = 1, I32 = 2, U32 = 3, I64 = 4, U64 = 5, F16 = 6, F32 = 7, F64 = 8 };
enum class Access : uint8_t { ReadOnly = 0, WriteOnly = 1, ReadWrite = 2 };
enum class TensorFormat : uint16_t { UNKNOWN = 0, SSBO_HWC = 1, SSBO_CHW = 2, SSBO_CHWC8 = 3, TEX_RGBA = 4, TEX_RGB = 5, TEX_RG = 6, TEX_R = 7 };
enum class TensorStorage : uint16_t { StorageBuffer = 0, StorageImage = 1, SampledStorageImage = 2 };

inline size_t scalarSize(ScalarType t) {
  switch (t) {
  case ScalarType::I16: case ScalarType::U16: case ScalarType::F16: return 2;
  case ScalarType::I32: case ScalarType::U32: case ScalarType::F32: return 4;
  default: return 8;
  }
}

// union ScalarSource { literal, symbolic } (dnx.fbs:16-29).  Literals are kept
// as int64 (all literals this backend emits are integers).
struct ScalarSource {
  bool symbolic = false;
  ScalarType dtype = ScalarType::I64; // dtype of a literal
  int64_t value = 0;                  // literal value or SymRef.sid
  static ScalarSource fromSym(Sym s, ScalarType t = ScalarType::I64) { return ScalarSource{s.symbolic, t, s.v}; }
  int64_t eval(const std::vector<int64_t> &dp) const {
    if (!symbolic) return value;
    if (value < 0 || static_cast<size_t>(value) >= dp.size()) fail(Status::InvalidModel, "SymRef out of range");
    return dp[static_cast<size_t>(value)];
  }
};

struct PushConstantField { ScalarType dtype; uint16_t offset; ScalarSource source; };
struct PushConstant { uint16_t size = 0; std::vector<PushConstantField> fields; };
struct DescriptorBinding { uint16_t binding; Access access; uint32_t tensor; };
struct DescriptorSetBinding { uint16_t set; std::vector<DescriptorBinding> bindings; };
struct DispatchInfo {
  std::string name, debug_info, src_path;
  bool has_reads = false, has_writes = false, has_flops = false;
  ScalarSource memory_reads, memory_writes, flops;
};
struct ComputeDispatch {
  uint32_t binary_id = 0;
  ScalarSource workgroup_count_x, workgroup_count_y, workgroup_count_z;
  uint32_t workgroup_size[3] = {1, 1, 1}; // HIP addition: threads per workgroup
  std::string entry_point;
  std::vector<DescriptorSetBinding> bindings;
  PushConstant push_constant;
  DispatchInfo info;
};
struct Buffer { ScalarSource size; uint16_t alignment = 16; };
struct TensorInfo {
  bool has_extent = false;
  ScalarSource width, height, channels;
  TensorFormat format = TensorFormat::UNKNOWN;
  TensorStorage storage = TensorStorage::StorageBuffer;
  ScalarType type = ScalarType::F16;
  std::string name;
};
struct Tensor { uint32_t buffer = 0; ScalarSource offset, size; TensorInfo info; };
struct TensorInitializer { uint32_t tensor; std::vector<uint8_t> data; };
struct ValueName { std::string name; ScalarSource value; };
// A relation between two extents that the model's graph needs and that symbolic extents only settle when an instance gets its
// values: lhs == rhs (relation 0) or lhs <= rhs (1).  `what` names the layer for the error message.  (No counterpart in dnx.fbs:
// the reference leaves such extents to the caller; a trailing field of `Model`, skipped by readers of the unchanged schema.)
struct Requirement { ScalarSource lhs, rhs; uint8_t relation = 0; std::string what; };
struct ShaderBinary { std::vector<uint8_t> code_object; uint32_t spirv_words = 0; };
struct ModelInfo { std::string producer, producer_version, model_version; };

struct Model {
  uint16_t version = 0;
  std::vector<uint32_t> required_features; // RuntimeFeature: 0 CooperativeMatrix (reference), 1 HipCodeObject
  ModelInfo info;
  std::vector<Tensor> tensors;
  std::vector<TensorInitializer> initializers;
  std::vector<uint32_t> inputs, outputs;
  std::vector<Buffer> buffers;
  std::vector<ComputeDispatch> dispatches;
  std::vector<ShaderBinary> shader_binaries;
  SymIR sym_ir;
  std::vector<ValueName> value_names;
  std::vector<Requirement> requirements;
  // Error(InvalidArgument) naming the first requirement that the evaluated symbol table `dp` violates
  void checkRequirements(const std::vector<int64_t> &dp) const;
};

std::vector<uint8_t> serialize(const Model &m);
// Throws Error(InvalidModel) on a truncated, corrupt or inconsistent buffer
// (the role of the FlatBuffers verifier in runtime/src/denox/runtime/model.cpp:639-644).
Model deserialize(const void *data, size_t size);
// Index / reference consistency checks shared by the reader and the compiler.
void validate(const Model &m);
// What a model needs on top of `validate` before it can be launched: a code object behind every binary a dispatch names
// and a workgroup size of 1..1024 threads.  Error(Unsupported) for a model that holds SPIR-V only.
void requireExecutable(const Model &m);

} // namespace denox::dnx
