// The plug-in side of the compiler: kernel families ("shaders") match patterns
// in the layer graph and register dispatches for them; every (match,
// configuration) becomes one hyper-edge of the super graph from which the
// schedule is selected.
//
// Interfaces follow the reference:
//   IShader                 compiler/src/denox/compiler/implement/shaders/IShader.hpp:33-71
//   OpImpl                  compiler/src/denox/compiler/implement/OpImpl.cpp:9-80
//   ComputeDispatchBuilder  compiler/src/denox/compiler/implement/ComputeDispatchBuilder.cpp:18-176
//   ComputeDispatch         compiler/src/denox/compiler/implement/ComputeDispatch.hpp:29-40
//   SuperGraphBuilder       compiler/src/denox/compiler/implement/SuperGraphBuilder.hpp:15-107
//   implement()             compiler/src/denox/compiler/implement/implement.cpp:11-68
// A dispatch names a HIP kernel variant (source + definitions, identified by
// its SHA-256) where the reference names a GLSL variant.
#pragma once
#include "../common/dnx.hpp"
#include "../hip/hip_compiler.hpp"
#include "model.hpp"
#include "options.hpp"
#include <algorithm>
#include <functional>
#include <memory>
#include <string>
#include <vector>

namespace denox::compiler {

struct TensorId { uint32_t index; };

enum class BindingType { Input = 0, Output = 1, Param = 2, Read = 3, Write = 4 };

struct PushConstantDesc { Sym value; dnx::ScalarType dtype; };

struct TensorBinding {
  uint16_t set = 0, binding = 0;
  dnx::Access access;
  TensorId tensor;
  BindingType type;
  // bytes the kernel may touch from the bound address, when that is not the tensor's own size (a channel range
  // written with the pixel pitch of a wider tensor); the timing table sizes its scratch buffers with it
  bool hasSpan = false;
  Sym span;
};

struct ComputeDispatchInfo {
  std::string name, operation, config, srcPath;
  bool hasReads = false, hasWrites = false, hasFlops = false;
  Sym memoryReads, memoryWrites, flops;
};

struct ComputeDispatch {
  hip::HipCompilerInstance kernel;
  std::string entryPoint;
  std::vector<PushConstantDesc> pushConstants;
  Sym workgroupCountX, workgroupCountY, workgroupCountZ;
  uint32_t workgroupSize[3] = {1, 1, 1};
  std::vector<TensorBinding> bindings;
  ComputeDispatchInfo info;
  // index of a push constant whose bit 0 selects a reversed tile walk, -1 if the kernel has none;
  // the compiler alternates it along the selected schedule (it is 0 in every table row)
  int traversalFlagIndex = -1;
};

struct SuperTensor {
  Sym byteSize;
  uint16_t alignment = 16;
  bool isParam = false;
  // for graph tensors
  int modelTensor = -1;
  dnx::TensorFormat format = dnx::TensorFormat::SSBO_HWC;
  dnx::ScalarType type = dnx::ScalarType::F16;
  std::string name;
};

struct Parameter { TensorId tensor; std::function<std::vector<uint8_t>()> lazyValue; };
struct MemoryConstrain { TensorId src0, src1, dst; };
// `src` lives inside `dst`, `byteOffset` from its start, with dst's pixel pitch (pixel-major concat without a copy)
struct ViewConstrain { TensorId src, dst; uint64_t byteOffset; };

// A tensor that may be produced directly as a channel range of a concat's output: its only consumer is that concat,
// it is neither a model input nor output, and the concat's result is an ordinary tensor.  The reference restricts its
// implicit concat the same way (each source feeds exactly one concat, CopyTransformShader.cpp:198-237).
struct ConcatView {
  bool valid = false;
  int concatOp = -1;
  TensorHandle parent = -1;
  unsigned pitch = 0, channelOffset = 0;
};
ConcatView concatViewOf(const Model &model, TensorHandle t);

struct SuperGraphEdge {
  std::vector<int> inputs; // model tensor handles
  int output = -1;
  std::vector<int> coveredOps;
  std::vector<ComputeDispatch> dispatches;
  std::vector<Parameter> parameters;
  std::vector<MemoryConstrain> memoryConstrains;
  std::vector<ViewConstrain> viewConstrains;
  // 0: the tensor as a buffer of its own; 1: the tensor as a channel range of its concat's output (ConcatView).
  // The two are different nodes of the hyper-graph the schedule is selected from.
  int outputVariant = 0;
  std::vector<int> inputVariants; // one per input, empty = all 0
  // Activation layout of the output / of each input (empty = all 0): 0 pixel-major (HWC), 1 channel-block-major (CHWC8).
  // As in the reference, where every tensor exists once per candidate layout and the edges are the cross product
  // (compiler/src/denox/compiler/specialization/specialization.cpp:13-16,112-121,282-306), the two layouts of a tensor
  // are different nodes of the hyper-graph; a dispatch that reads one layout and writes the other is the conversion.
  int outputFormat = 0;
  std::vector<int> inputFormats;
  std::string shader, config;
  float speedup = 1.0f;
};

struct SuperGraph {
  // [0, N) mirror the model's N tensors in HWC, [N, 2N) the same tensors in CHWC8 (a buffer of its own each), parameters follow
  std::vector<SuperTensor> tensors;
  std::vector<SuperGraphEdge> edges;
  size_t modelTensorCount = 0;
};

class OpImpl;

class ComputeDispatchBuilder {
public:
  void addBinding(dnx::Access access, TensorHandle modelTensor);
  void addBinding(dnx::Access access, TensorHandle modelTensor, Sym span); // see TensorBinding::span
  void addParamBinding(TensorId tensor);
  void addPushConstant(Sym value, dnx::ScalarType dtype = dnx::ScalarType::U32);
  void addTraversalFlag(); // a U32 push constant, 0 here, set per position in the schedule
  void setName(const std::string &n) { self().info.name = n; }
  void setConfig(const std::string &c) { self().info.config = c; }
  void setOperation(const std::string &o) { self().info.operation = o; }
  void setSourcePath(const std::string &p) { self().info.srcPath = p; }
  void setMemoryReads(Sym s) { self().info.memoryReads = s; self().info.hasReads = true; }
  void setMemoryWrites(Sym s) { self().info.memoryWrites = s; self().info.hasWrites = true; }
  void setFlops(Sym s) { self().info.flops = s; self().info.hasFlops = true; }
  // assigns binding numbers in class order Input < Output < Param < Read < Write
  // (ComputeDispatchBuilder.cpp:100-176 of the reference); all in descriptor set 0
  ~ComputeDispatchBuilder();
  ComputeDispatchBuilder(ComputeDispatchBuilder &&o) : m_index(o.m_index), m_impl(o.m_impl) { o.m_impl = nullptr; }

private:
  friend class OpImpl;
  ComputeDispatchBuilder(size_t index, OpImpl *impl) : m_index(index), m_impl(impl) {}
  ComputeDispatch &self();
  size_t m_index;
  OpImpl *m_impl;
};

class OpImpl {
public:
  OpImpl(SuperGraph *g, const Model *model, std::vector<int> inputs, int output, std::vector<int> coveredOps)
      : m_graph(g), m_model(model) { m_edge.inputs = std::move(inputs); m_edge.output = output; m_edge.coveredOps = std::move(coveredOps); }

  ComputeDispatchBuilder registerDispatch(hip::HipCompilerInstance kernel, const std::string &entryPoint,
                                          Sym wgX, Sym wgY, Sym wgZ, uint32_t blockX, uint32_t blockY = 1, uint32_t blockZ = 1);
  TensorId createParameter(size_t byteSize, dnx::ScalarType dtype, std::function<std::vector<uint8_t>()> value, uint16_t alignment = 256);
  void createImplicitConcatConstrain(TensorHandle src0, TensorHandle src1, TensorHandle dst);
  void createViewConstrain(TensorHandle src, TensorHandle dst, uint64_t byteOffset);
  SuperGraphEdge &edge() { return m_edge; }
  void finish();

private:
  friend class ComputeDispatchBuilder;
  SuperGraph *m_graph;
  const Model *m_model;
  SuperGraphEdge m_edge;
};

struct Match {
  unsigned pattern = 0;
  std::vector<int> ops;      // covered op indices, in execution order
  std::vector<int> inputs;   // tensor handles read
  int output = -1;           // tensor handle written
  int outputVariant = 0;     // as SuperGraphEdge::outputVariant
  std::vector<int> inputVariants;
  int outputFormat = 0;      // as SuperGraphEdge::outputFormat
  std::vector<int> inputFormats;
  bool blocked() const { return outputFormat != 0 || std::any_of(inputFormats.begin(), inputFormats.end(), [](int f) { return f != 0; }); }
};

class IShader {
public:
  virtual ~IShader() = default;
  virtual std::string name() const = 0;
  // every place in the graph this kernel family can implement
  virtual std::vector<Match> matchAll(const Model &model, const CompileOptions &opt) const = 0;
  // configuration ids valid for a match
  virtual std::vector<unsigned> acceptMatch(const Model &model, const Match &m, const CompileOptions &opt) const = 0;
  virtual size_t parameterMemorySize(const Model &, const Match &) const { return 0; }
  virtual float speedup(unsigned /*config*/) const { return 1.0f; }
  virtual void implement(OpImpl &impl, const Model &model, const Match &m, unsigned config, SymGraph &sym, const CompileOptions &opt) const = 0;
};

std::vector<std::unique_ptr<IShader>> get_all_shaders(const hip::HipCompiler *compiler);
// every name `CompileOptions::forceConvConfig` accepts: the convolution shaders' configuration tables
std::vector<std::string> conv_config_names();

// Build the super graph: every shader x match x configuration.
SuperGraph implement(const Model &model, SymGraph &sym, const std::vector<std::unique_ptr<IShader>> &shaders, const CompileOptions &opt);

} // namespace denox::compiler
