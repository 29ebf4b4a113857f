#include "implement.hpp"
#include <algorithm>

namespace denox::compiler {

ComputeDispatch &ComputeDispatchBuilder::self() { return m_impl->m_edge.dispatches[m_index]; }

void ComputeDispatchBuilder::addBinding(dnx::Access access, TensorHandle t) {
  const auto &e = m_impl->m_edge;
  TensorBinding b;
  b.access = access;
  b.tensor = TensorId{static_cast<uint32_t>(t)};
  const bool isSrc = std::find(e.inputs.begin(), e.inputs.end(), t) != e.inputs.end();
  const bool isDst = e.output == t;
  if (isSrc && access == dnx::Access::ReadOnly) b.type = BindingType::Input;
  else if (isDst && access != dnx::Access::ReadOnly) b.type = BindingType::Output;
  else b.type = access == dnx::Access::ReadOnly ? BindingType::Read : BindingType::Write;
  self().bindings.push_back(b);
}

void ComputeDispatchBuilder::addBinding(dnx::Access access, TensorHandle t, Sym span) {
  addBinding(access, t);
  self().bindings.back().hasSpan = true;
  self().bindings.back().span = span;
}

void ComputeDispatchBuilder::addParamBinding(TensorId tensor) {
  TensorBinding b;
  b.access = dnx::Access::ReadOnly;
  b.tensor = tensor;
  b.type = BindingType::Param;
  self().bindings.push_back(b);
}

void ComputeDispatchBuilder::addPushConstant(Sym value, dnx::ScalarType dtype) { self().pushConstants.push_back(PushConstantDesc{value, dtype}); }

void ComputeDispatchBuilder::addTraversalFlag() {
  self().traversalFlagIndex = static_cast<int>(self().pushConstants.size());
  self().pushConstants.push_back(PushConstantDesc{Sym::Const(0), dnx::ScalarType::U32});
}

ComputeDispatchBuilder::~ComputeDispatchBuilder() {
  if (!m_impl) return;
  auto &bs = self().bindings;
  // kernels take their arguments in registration order within a class, classes in
  // the order Input < Output < Param < Read < Write
  std::stable_sort(bs.begin(), bs.end(), [](const TensorBinding &a, const TensorBinding &b) { return static_cast<int>(a.type) < static_cast<int>(b.type); });
  uint16_t n = 0;
  for (auto &b : bs) { b.set = 0; b.binding = n++; }
}

ComputeDispatchBuilder OpImpl::registerDispatch(hip::HipCompilerInstance kernel, const std::string &entryPoint, Sym wgX, Sym wgY, Sym wgZ,
                                                uint32_t bx, uint32_t by, uint32_t bz) {
  ComputeDispatch d;
  d.kernel = std::move(kernel);
  d.entryPoint = entryPoint;
  d.workgroupCountX = wgX; d.workgroupCountY = wgY; d.workgroupCountZ = wgZ;
  d.workgroupSize[0] = bx; d.workgroupSize[1] = by; d.workgroupSize[2] = bz;
  d.info.srcPath = d.kernel.sourcePath();
  m_edge.dispatches.push_back(std::move(d));
  return ComputeDispatchBuilder(m_edge.dispatches.size() - 1, this);
}

TensorId OpImpl::createParameter(size_t byteSize, dnx::ScalarType dtype, std::function<std::vector<uint8_t>()> value, uint16_t alignment) {
  SuperTensor t;
  t.byteSize = Sym::Const(static_cast<int64_t>(byteSize));
  t.alignment = alignment;
  t.isParam = true;
  t.type = dtype;
  t.format = dnx::TensorFormat::UNKNOWN;
  m_graph->tensors.push_back(std::move(t));
  TensorId id{static_cast<uint32_t>(m_graph->tensors.size() - 1)};
  m_edge.parameters.push_back(Parameter{id, std::move(value)});
  return id;
}

void OpImpl::createImplicitConcatConstrain(TensorHandle src0, TensorHandle src1, TensorHandle dst) {
  const size_t n = m_model->tensors().size();
  if (src0 < 0 || src1 < 0 || dst < 0 || static_cast<size_t>(src0) >= n || static_cast<size_t>(src1) >= n || static_cast<size_t>(dst) >= n)
    fail(Status::Internal, "Failed to create memory constrain, invalid node ids.");
  m_edge.memoryConstrains.push_back(MemoryConstrain{TensorId{static_cast<uint32_t>(src0)}, TensorId{static_cast<uint32_t>(src1)}, TensorId{static_cast<uint32_t>(dst)}});
}

void OpImpl::createViewConstrain(TensorHandle src, TensorHandle dst, uint64_t byteOffset) {
  const size_t n = m_model->tensors().size();
  if (src < 0 || dst < 0 || static_cast<size_t>(src) >= n || static_cast<size_t>(dst) >= n) fail(Status::Internal, "Failed to create memory constrain, invalid node ids.");
  m_edge.viewConstrains.push_back(ViewConstrain{TensorId{static_cast<uint32_t>(src)}, TensorId{static_cast<uint32_t>(dst)}, byteOffset});
}

ConcatView concatViewOf(const Model &model, TensorHandle t) {
  ConcatView v;
  const TensorNode &n = model.tensors()[static_cast<size_t>(t)];
  if (n.isInput || n.isOutput || n.consumers.size() != 1) return v;
  const Op &cat = model.ops()[static_cast<size_t>(n.consumers[0])];
  if (cat.kind != OpKind::Concat || cat.inputs.size() != 2 || cat.inputs[0] == cat.inputs[1]) return v;
  v.valid = true;
  v.concatOp = n.consumers[0];
  v.parent = cat.output;
  v.pitch = model.tensors()[static_cast<size_t>(cat.output)].channels;
  v.channelOffset = cat.inputs[0] == t ? 0 : model.tensors()[static_cast<size_t>(cat.inputs[0])].channels;
  return v;
}

void OpImpl::finish() { m_graph->edges.push_back(std::move(m_edge)); }

SuperGraph implement(const Model &model, SymGraph &sym, const std::vector<std::unique_ptr<IShader>> &shaders, const CompileOptions &opt) {
  SuperGraph g;
  g.tensors.reserve(model.tensors().size() + 64);
  for (size_t i = 0; i < model.tensors().size(); ++i) {
    const TensorNode &t = model.tensors()[i];
    SuperTensor st;
    st.byteSize = sym.mul(sym.mul(t.width, t.height), static_cast<int64_t>(t.channels) * 2);
    st.alignment = 256;
    st.modelTensor = static_cast<int>(i);
    st.name = t.name;
    g.tensors.push_back(std::move(st));
  }
  // the same tensors stored channel-block-major
  const size_t N = model.tensors().size();
  g.modelTensorCount = N;
  for (size_t i = 0; i < N; ++i) {
    SuperTensor st = g.tensors[i];
    st.format = dnx::TensorFormat::SSBO_CHWC8;
    g.tensors.push_back(std::move(st));
  }
  for (const auto &shader : shaders) {
    for (const Match &m : shader->matchAll(model, opt)) {
      for (unsigned config : shader->acceptMatch(model, m, opt)) {
        OpImpl impl(&g, &model, m.inputs, m.output, m.ops);
        impl.edge().shader = shader->name();
        impl.edge().speedup = shader->speedup(config);
        impl.edge().outputVariant = m.outputVariant;
        impl.edge().inputVariants = m.inputVariants;
        impl.edge().outputFormat = m.outputFormat;
        impl.edge().inputFormats = m.inputFormats;
        shader->implement(impl, model, m, config, sym, opt);
        if (m.blocked()) {
          // The shaders bind model tensors by handle; an input or output the match takes in CHWC8 is that tensor's second
          // super-graph tensor.
          auto blockedTensor = [&](uint32_t t) -> uint32_t {
            if (t >= N) return t; // a parameter
            if (static_cast<int>(t) == m.output && m.outputFormat) return t + static_cast<uint32_t>(N);
            for (size_t i = 0; i < m.inputs.size(); ++i)
              if (m.inputs[i] == static_cast<int>(t) && i < m.inputFormats.size() && m.inputFormats[i]) return t + static_cast<uint32_t>(N);
            return t;
          };
          for (auto &d : impl.edge().dispatches)
            for (auto &b : d.bindings) b.tensor.index = blockedTensor(b.tensor.index);
          for (auto &mc : impl.edge().memoryConstrains) {
            mc.src0.index = blockedTensor(mc.src0.index);
            mc.src1.index = blockedTensor(mc.src1.index);
            mc.dst.index = blockedTensor(mc.dst.index);
          }
        }
        impl.finish();
      }
    }
  }
  return g;
}

} // namespace denox::compiler
