#include "runtime.hpp"
#include "arena_plan.hpp"
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace denox::runtime {

void hipCheck(hipError_t e, const char *what) {
  if (e != hipSuccess) fail(Status::HipError, std::string(what) + ": " + hipGetErrorString(e));
}

// ---------------------------------------------------------------- Context
Context::Context(int device) : m_device(device) {
  int n = 0;
  hipCheck(hipGetDeviceCount(&n), "hipGetDeviceCount");
  if (device < 0 || device >= n) fail(Status::InvalidArgument, "no HIP device with index " + std::to_string(device));
  hipCheck(hipSetDevice(device), "hipSetDevice");
  hipCheck(hipGetDeviceProperties(&m_props, device), "hipGetDeviceProperties");
  // default priority, non-blocking with respect to the null stream
  hipCheck(hipStreamCreateWithFlags(&m_stream, hipStreamNonBlocking), "hipStreamCreateWithFlags");
  try {
    m_staticScratch = staticScratchAddress(device); // set-up time: the allocation-free entry point must not have to ask
    hipCheck(hipEventCreateWithFlags(&m_staticDone, hipEventDisableTiming), "hipEventCreateWithFlags");
  } catch (...) {
    (void)hipStreamDestroy(m_stream);
    throw;
  }
}

Context::~Context() {
  if (m_stream) (void)hipStreamSynchronize(m_stream);
  staticScratchForget(m_device, this);
  if (m_staticDone) (void)hipEventDestroy(m_staticDone);
  if (m_stream) (void)hipStreamDestroy(m_stream);
}

void Context::makeCurrent() const { hipCheck(hipSetDevice(m_device), "hipSetDevice"); }

// ---------------------------------------------------------------- Model
Model::Model(ContextHandle ctx, const void *dnxbuf, size_t size) : m_ctx(std::move(ctx)), m_dnx(dnx::deserialize(dnxbuf, size)) {
  dnx::requireExecutable(m_dnx);
  m_ctx->makeCurrent();
  m_modules.resize(m_dnx.shader_binaries.size(), nullptr);
  try {
    for (size_t i = 0; i < m_modules.size(); ++i) {
      if (m_dnx.shader_binaries[i].code_object.empty()) continue; // a binary no dispatch names
      hipCheck(hipModuleLoadData(&m_modules[i], m_dnx.shader_binaries[i].code_object.data()), "hipModuleLoadData");
    }
    m_dispatches.reserve(m_dnx.dispatches.size());
    for (const auto &d : m_dnx.dispatches) {
      ModelDispatch md;
      md.dnx = &d;
      hipCheck(hipModuleGetFunction(&md.function, m_modules[d.binary_id], d.entry_point.c_str()), "hipModuleGetFunction");
      // kernel arguments follow (set, binding) order
      std::vector<const dnx::DescriptorSetBinding *> sets;
      for (const auto &s : d.bindings) sets.push_back(&s);
      std::sort(sets.begin(), sets.end(), [](auto *a, auto *b) { return a->set < b->set; });
      for (const auto *s : sets) {
        std::vector<dnx::DescriptorBinding> bs = s->bindings;
        std::sort(bs.begin(), bs.end(), [](const auto &a, const auto &b) { return a.binding < b.binding; });
        for (const auto &b : bs) md.tensors.emplace_back(b.tensor, b.access);
      }
      // On one in-order stream program order resolves every RAW/WAW/WAR hazard the
      // reference inserts barriers for; what remains to check is that no single
      // dispatch reads a tensor through one binding and writes it through another.
      for (size_t a = 0; a < md.tensors.size(); ++a)
        for (size_t b = a + 1; b < md.tensors.size(); ++b)
          if (md.tensors[a].first == md.tensors[b].first &&
              (md.tensors[a].second != dnx::Access::ReadOnly || md.tensors[b].second != dnx::Access::ReadOnly))
            fail(Status::InvalidModel, "dispatch '" + d.info.name + "' binds a tensor it writes more than once");
      m_dispatches.push_back(std::move(md));
    }
  } catch (...) {
    for (auto m : m_modules) if (m) (void)hipModuleUnload(m);
    throw;
  }
}

Model::~Model() {
  for (auto m : m_modules) if (m) (void)hipModuleUnload(m);
}

// ---------------------------------------------------------------- Instance
static void putScalar(std::vector<uint8_t> &buf, size_t off, dnx::ScalarType t, int64_t v) {
  switch (t) {
  case dnx::ScalarType::I16: { int16_t x = static_cast<int16_t>(v); std::memcpy(buf.data() + off, &x, 2); break; }
  case dnx::ScalarType::U16: { uint16_t x = static_cast<uint16_t>(v); std::memcpy(buf.data() + off, &x, 2); break; }
  case dnx::ScalarType::I32: { int32_t x = static_cast<int32_t>(v); std::memcpy(buf.data() + off, &x, 4); break; }
  case dnx::ScalarType::U32: { uint32_t x = static_cast<uint32_t>(v); std::memcpy(buf.data() + off, &x, 4); break; }
  case dnx::ScalarType::I64: std::memcpy(buf.data() + off, &v, 8); break;
  case dnx::ScalarType::U64: { uint64_t x = static_cast<uint64_t>(v); std::memcpy(buf.data() + off, &x, 8); break; }
  default: fail(Status::Unsupported, "floating-point push constants are not supported"); // instance.cpp:196-199 of the reference
  }
}

Instance::Instance(ModelHandle model, const std::vector<ValueSpec> &specs) : m_model(std::move(model)) {
  const dnx::Model &m = m_model->dnx();
  m_model->context()->makeCurrent();
  // name -> variable, unknown names are ignored (instance.cpp:308-318 of the reference)
  std::vector<int64_t> vars(m.sym_ir.varCount, 0);
  std::vector<bool> set(m.sym_ir.varCount, false);
  for (const auto &spec : specs)
    for (const auto &vn : m.value_names)
      if (vn.name == spec.name && vn.value.symbolic && vn.value.value >= 0 && static_cast<uint64_t>(vn.value.value) < vars.size()) {
        vars[static_cast<size_t>(vn.value.value)] = spec.value;
        set[static_cast<size_t>(vn.value.value)] = true;
      }
  // every named variable needs a value (unnamed table slots are unused)
  for (const auto &vn : m.value_names)
    if (vn.value.symbolic && vn.value.value >= 0 && static_cast<uint64_t>(vn.value.value) < vars.size() && !set[static_cast<size_t>(vn.value.value)])
      fail(Status::InvalidArgument, "no value given for dynamic extent '" + vn.name + "'");
  m_sym = m.sym_ir.eval(vars);
  m.checkRequirements(m_sym); // extents the graph needs to agree (concat sources, slice bounds)

  // tensors must fit their buffers
  m_bufferSizes.resize(m.buffers.size());
  for (size_t i = 0; i < m.buffers.size(); ++i) {
    const int64_t sz = m.buffers[i].size.eval(m_sym);
    if (sz < 0 || sz > (int64_t(1) << 40)) fail(Status::InvalidArgument, "buffer " + std::to_string(i) + " evaluates to an unusable size (" + std::to_string(sz) + " bytes)");
    m_bufferSizes[i] = static_cast<uint64_t>(sz);
  }
  for (const auto &t : m.tensors) {
    const int64_t off = t.offset.eval(m_sym), sz = t.size.eval(m_sym);
    if (off < 0 || sz < 0 || static_cast<uint64_t>(off) + static_cast<uint64_t>(sz) > m_bufferSizes[t.buffer])
      fail(Status::InvalidModel, "tensor '" + t.info.name + "' does not fit its buffer");
    // the kernels address a tensor with 32-bit byte offsets (buffer resources); offsets from 0xFFFFF000 up mean "no access"
    if (static_cast<uint64_t>(sz) >= 0xFFFFF000ull)
      fail(Status::Unsupported, "tensor '" + t.info.name + "' is " + std::to_string(sz) + " bytes at these extents; tensors of 4 GiB and more are not supported");
  }
  try {
    m_buffers.assign(m.buffers.size(), nullptr);
    // slack so that 16-byte vector accesses at the very end of a tensor stay inside the allocation
    auto padded = [&](size_t i) { return (std::max<uint64_t>(m_bufferSizes[i], 16) + 256 + 255) / 256 * 256; };
    // Buffers that only hold intermediate results live from the first to the last dispatch that binds one of their
    // tensors (the dispatches run in order on one stream) and share one arena: two buffers overlap in memory only when
    // their lifetimes do not.  The reference keeps one allocation per buffer (placement.cpp:276-300 records first / last
    // use, instance.cpp allocates each); here the smaller working set matters for speed too: a dead tensor's lines are
    // overwritten while they still sit in the memory-side cache instead of being written back to HBM.
    // Interface tensors (filled and read outside the dispatches) and parameters keep allocations of their own.
    std::vector<int> first(m.buffers.size(), INT32_MAX), last(m.buffers.size(), -1);
    std::vector<char> own(m.buffers.size(), 0);
    for (uint32_t t : m.inputs) own[m.tensors[t].buffer] = 1;
    for (uint32_t t : m.outputs) own[m.tensors[t].buffer] = 1;
    for (const auto &init : m.initializers) own[m.tensors[init.tensor].buffer] = 1;
    {
      int di = 0;
      for (const auto &md : m_model->dispatches()) {
        for (const auto &tb : md.tensors) {
          const uint32_t b = m.tensors[tb.first].buffer;
          first[b] = std::min(first[b], di);
          last[b] = std::max(last[b], di);
        }
        ++di;
      }
    }
    std::vector<size_t> shared;
    for (size_t i = 0; i < m.buffers.size(); ++i)
      if (!own[i] && last[i] >= 0 && !std::getenv("DENOX_HIP_NO_ALIAS")) shared.push_back(i);
    // (placing in order of first use with a preference for ranges that died just before was measured too: 16 % more
    // memory and 1 % slower than the largest-first placement of plan_arena)
    std::vector<ArenaItem> items;
    for (size_t i : shared) items.push_back(ArenaItem{padded(i), first[i], last[i]});
    uint64_t arenaBytes = 0;
    const std::vector<uint64_t> at = plan_arena(items, arenaBytes, static_cast<int>(m_model->dispatches().size()));
    m_arenaBytes = arenaBytes;
    if (arenaBytes) {
      hipCheck(hipMalloc(&m_arena, arenaBytes), "hipMalloc(arena)");
      m_deviceBytes += arenaBytes;
      for (size_t k = 0; k < shared.size(); ++k) m_buffers[shared[k]] = static_cast<uint8_t *>(m_arena) + at[k];
    }
    m_ownBuffer.assign(m.buffers.size(), 0);
    for (size_t i = 0; i < m.buffers.size(); ++i) {
      if (m_buffers[i]) continue;
      hipCheck(hipMalloc(&m_buffers[i], padded(i)), "hipMalloc");
      m_ownBuffer[i] = 1;
      m_deviceBytes += padded(i);
    }
    // parameters (instance.cpp:65-113 of the reference)
    hipStream_t s = m_model->context()->stream();
    if (std::getenv("DENOX_HIP_POISON")) { // debugging: every activation byte starts as 0xFF (binary16 NaN), so a kernel that
                                           // lets memory nobody wrote reach its result shows up in the output
      if (m_arena) hipCheck(hipMemsetAsync(m_arena, 0xFF, arenaBytes, s), "hipMemsetAsync(poison)");
      for (size_t i = 0; i < m.buffers.size(); ++i)
        if (m_ownBuffer[i]) hipCheck(hipMemsetAsync(m_buffers[i], 0xFF, padded(i), s), "hipMemsetAsync(poison)");
    }
    for (const auto &init : m.initializers) {
      const auto &t = m.tensors[init.tensor];
      const uint64_t sz = static_cast<uint64_t>(t.size.eval(m_sym));
      if (init.data.size() > sz) fail(Status::InvalidModel, "initializer larger than its tensor");
      hipCheck(hipMemcpyAsync(tensorPtr(init.tensor), init.data.data(), init.data.size(), hipMemcpyHostToDevice, s), "hipMemcpyAsync(initializer)");
    }
    hipCheck(hipStreamSynchronize(s), "hipStreamSynchronize");

    // launches (instance.cpp:121-229 of the reference)
    for (const auto &md : m_model->dispatches()) {
      const dnx::ComputeDispatch &d = *md.dnx;
      Launch l;
      l.fn = md.function;
      const int64_t g[3] = {d.workgroup_count_x.eval(m_sym), d.workgroup_count_y.eval(m_sym), d.workgroup_count_z.eval(m_sym)};
      for (int i = 0; i < 3; ++i) {
        if (g[i] < 0 || g[i] > (i == 0 ? 0x7FFFFFFF : 65535)) fail(Status::InvalidArgument, "dispatch '" + d.info.name + "' workgroup count out of range");
        l.grid[i] = static_cast<unsigned>(g[i]);
        l.block[i] = d.workgroup_size[i];
      }
      const size_t ptrBytes = md.tensors.size() * sizeof(void *);
      // push constants start at the next multiple of their strictest field alignment (at most 8)
      size_t pcAlign = 4;
      for (const auto &f : d.push_constant.fields) pcAlign = std::max(pcAlign, dnx::scalarSize(f.dtype));
      const size_t pcOff = (ptrBytes + pcAlign - 1) / pcAlign * pcAlign;
      l.args.assign(pcOff + d.push_constant.size, 0);
      for (size_t i = 0; i < md.tensors.size(); ++i) {
        const uint32_t tensor = md.tensors[i].first;
        void *p = tensorPtr(tensor);
        std::memcpy(l.args.data() + i * sizeof(void *), &p, sizeof(void *));
        Launch::Slot slot{i * sizeof(void *), tensor, -1, false, 0};
        // Everything in an interface tensor's buffer moves with the address the caller binds: the tensor itself and
        // the tensors placed inside it (concat sources that their producers write in place, compile.cpp view constrains).
        const uint32_t buffer = m.tensors[tensor].buffer;
        const int64_t off = m.tensors[tensor].offset.eval(m_sym);
        for (size_t k = 0; k < m.inputs.size() && slot.iface < 0; ++k)
          if (m.tensors[m.inputs[k]].buffer == buffer) slot = Launch::Slot{slot.offset, tensor, static_cast<int>(k), true, off - m.tensors[m.inputs[k]].offset.eval(m_sym)};
        for (size_t k = 0; k < m.outputs.size() && slot.iface < 0; ++k)
          if (m.tensors[m.outputs[k]].buffer == buffer) slot = Launch::Slot{slot.offset, tensor, static_cast<int>(k), false, off - m.tensors[m.outputs[k]].offset.eval(m_sym)};
        l.ptrSlots.push_back(slot);
      }
      for (const auto &f : d.push_constant.fields) putScalar(l.args, pcOff + f.offset, f.dtype, f.source.eval(m_sym));
      // the argument buffer of the allocation-free path: arena addresses become static-scratch addresses
      l.staticArgs = l.args;
      if (m_arena && m_arenaBytes <= kStaticScratchBytes && m_model->context()->staticScratch())
        for (const auto &slot : l.ptrSlots) {
          uint8_t *p = static_cast<uint8_t *>(tensorPtr(slot.tensor));
          uint8_t *a = static_cast<uint8_t *>(m_arena);
          if (p < a || p >= a + m_arenaBytes) continue;
          void *q = static_cast<uint8_t *>(m_model->context()->staticScratch()) + (p - a);
          std::memcpy(l.staticArgs.data() + slot.offset, &q, sizeof(void *));
        }
      m_launches.push_back(std::move(l));
    }
    m_boundInputs.assign(m.inputs.size(), nullptr);
    m_boundOutputs.assign(m.outputs.size(), nullptr);
    m_useGraph = !std::getenv("DENOX_HIP_NO_GRAPH");
    if (m_useGraph) selectGraph();
  } catch (...) {
    freeBuffers();
    destroyGraphs();
    throw;
  }
}

Instance::~Instance() {
  if (m_model) {
    (void)hipSetDevice(m_model->context()->device());
    (void)hipStreamSynchronize(m_model->context()->stream());
  }
  destroyPipeline();
  destroyGraphs();
  freeBuffers();
}

void Instance::destroyGraphs() {
  bool current = false;
  for (auto &c : m_graphCache) {
    current |= c.exec == m_graphExec;
    if (c.exec) (void)hipGraphExecDestroy(c.exec);
    if (c.graph) (void)hipGraphDestroy(c.graph);
  }
  m_graphCache.clear();
  if (!current) { // captured but not filed yet (a failure in between)
    if (m_graphExec) (void)hipGraphExecDestroy(m_graphExec);
    if (m_graph) (void)hipGraphDestroy(m_graph);
  }
  m_graphExec = nullptr;
  m_graph = nullptr;
}

void Instance::freeBuffers() {
  for (size_t i = 0; i < m_buffers.size(); ++i)
    if (m_buffers[i] && i < m_ownBuffer.size() && m_ownBuffer[i]) (void)hipFree(m_buffers[i]);
  if (m_arena) (void)hipFree(m_arena);
  m_arena = nullptr;
  m_buffers.clear();
}

void Instance::destroyPipeline() {
  if (m_pipe.exec) (void)hipGraphExecDestroy(m_pipe.exec);
  if (m_pipe.graph) (void)hipGraphDestroy(m_pipe.graph);
  for (void *p : m_pipe.in) if (p) (void)hipFree(p);
  for (void *p : m_pipe.out) if (p) (void)hipFree(p);
  for (int s = 0; s < 2; ++s) {
    if (m_pipe.inReady[s]) (void)hipEventDestroy(m_pipe.inReady[s]);
    if (m_pipe.computed[s]) (void)hipEventDestroy(m_pipe.computed[s]);
    if (m_pipe.outRead[s]) (void)hipEventDestroy(m_pipe.outRead[s]);
  }
  if (m_pipe.h2d) (void)hipStreamDestroy(m_pipe.h2d);
  if (m_pipe.d2h) (void)hipStreamDestroy(m_pipe.d2h);
  m_pipe = Pipeline{};
}

void *Instance::tensorPtr(uint32_t tensor) const {
  const auto &t = m_model->dnx().tensors.at(tensor);
  return static_cast<uint8_t *>(m_buffers[t.buffer]) + t.offset.eval(m_sym);
}

TensorDesc Instance::describe(uint32_t tensor) const {
  const auto &t = m_model->dnx().tensors.at(tensor);
  TensorDesc d;
  if (t.info.has_extent) {
    d.width = t.info.width.eval(m_sym);
    d.height = t.info.height.eval(m_sym);
    d.channels = t.info.channels.eval(m_sym);
  }
  d.format = t.info.format;
  d.dtype = t.info.type;
  d.byteSize = static_cast<uint64_t>(t.size.eval(m_sym));
  d.name = t.info.name;
  return d;
}

static void launchOne(hipFunction_t fn, const unsigned grid[3], const unsigned block[3], std::vector<uint8_t> &args, hipStream_t s) {
  if (grid[0] == 0 || grid[1] == 0 || grid[2] == 0) return; // empty extent: nothing to do
  size_t size = args.size();
  void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, args.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
  hipCheck(hipModuleLaunchKernel(fn, grid[0], grid[1], grid[2], block[0], block[1], block[2], 0, s, nullptr, config), "hipModuleLaunchKernel");
}

void Instance::launchAll(hipStream_t s) {
  for (auto &l : m_launches) launchOne(l.fn, l.grid, l.block, l.args, s);
}

void Instance::buildGraph() {
  // Whole-network capture: one graph launch per frame instead of one driver
  // call per dispatch.
  hipStream_t s = m_model->context()->stream();
  hipCheck(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
  try {
    launchAll(s);
  } catch (...) {
    hipGraph_t g = nullptr;
    (void)hipStreamEndCapture(s, &g);
    if (g) (void)hipGraphDestroy(g);
    throw;
  }
  hipCheck(hipStreamEndCapture(s, &m_graph), "hipStreamEndCapture");
  const hipError_t e = hipGraphInstantiate(&m_graphExec, m_graph, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGraphDestroy(m_graph);
    m_graph = nullptr;
    m_graphExec = nullptr;
    hipCheck(e, "hipGraphInstantiate");
  }
}

void Instance::rebind(const void *const *inputs, void *const *outputs) {
  // Patch external input/output addresses into the argument buffers.  A graph is captured only for a set of addresses
  // not seen before (the last few are kept).
  const dnx::Model &m = m_model->dnx();
  bool changed = false;
  std::vector<void *> in(m.inputs.size()), out(m.outputs.size());
  for (size_t i = 0; i < m.inputs.size(); ++i) {
    void *p = inputs ? const_cast<void *>(inputs[i]) : nullptr;
    if (p != m_boundInputs[i]) { changed = true; m_boundInputs[i] = p; }
    in[i] = p ? p : tensorPtr(m.inputs[i]);
  }
  for (size_t i = 0; i < m.outputs.size(); ++i) {
    void *p = outputs ? outputs[i] : nullptr;
    if (p != m_boundOutputs[i]) { changed = true; m_boundOutputs[i] = p; }
    out[i] = p ? p : tensorPtr(m.outputs[i]);
  }
  if (!changed && !m_graphStale) return;
  patchInterface(in, out);
  if (!m_useGraph) return; // plain launches read the argument buffers at launch time
  // Until a graph for these addresses is in place the bindings count as unfinished: if the capture fails, the next call with
  // the same addresses tries again instead of taking "nothing changed" for "a graph exists".
  m_graphStale = true;
  selectGraph();
  m_graphStale = false;
}

// Makes m_graph / m_graphExec the captured dispatch list for the interface addresses bound now (m_boundInputs /
// m_boundOutputs, which the argument buffers already hold): from the cache, or captured and filed there.
void Instance::selectGraph() {
  std::vector<void *> key = m_boundInputs;
  key.insert(key.end(), m_boundOutputs.begin(), m_boundOutputs.end());
  for (auto &c : m_graphCache)
    if (c.key == key) {
      m_graph = c.graph;
      m_graphExec = c.exec;
      c.lastUse = ++m_graphUse;
      return;
    }
  constexpr size_t kCachedGraphs = 4;
  if (m_graphCache.size() >= kCachedGraphs) {
    // The one used longest ago goes.  An earlier launch of it may still be running (inferDevice does not wait), and
    // an executable graph must not be destroyed under a running launch.
    hipCheck(hipStreamSynchronize(m_model->context()->stream()), "hipStreamSynchronize");
    auto victim = std::min_element(m_graphCache.begin(), m_graphCache.end(), [](const CachedGraph &a, const CachedGraph &b) { return a.lastUse < b.lastUse; });
    (void)hipGraphExecDestroy(victim->exec);
    (void)hipGraphDestroy(victim->graph);
    m_graphCache.erase(victim);
  }
  m_graph = nullptr;
  m_graphExec = nullptr; // until the capture below succeeds, inferDevice would fall back to plain launches
  buildGraph();
  m_graphCache.push_back(CachedGraph{std::move(key), m_graph, m_graphExec, ++m_graphUse});
}

// Writes the given interface addresses into the argument buffers (no graph is touched): every bound tensor that lives
// in an interface tensor's buffer follows that tensor's address.
void Instance::patchInterface(const std::vector<void *> &inputs, const std::vector<void *> &outputs, bool staticArgs) {
  for (auto &l : m_launches)
    for (const auto &slot : l.ptrSlots) {
      if (slot.iface < 0) continue;
      void *base = slot.isInput ? inputs[static_cast<size_t>(slot.iface)] : outputs[static_cast<size_t>(slot.iface)];
      void *p = static_cast<uint8_t *>(base) + slot.delta;
      std::memcpy((staticArgs ? l.staticArgs : l.args).data() + slot.offset, &p, sizeof(void *));
    }
}

void Instance::preparePipeline() {
  if (m_pipe.ready) return;
  const dnx::Model &m = m_model->dnx();
  try {
    // default-priority streams that do not synchronise with the legacy stream
    hipCheck(hipStreamCreateWithFlags(&m_pipe.h2d, hipStreamNonBlocking), "hipStreamCreateWithFlags");
    hipCheck(hipStreamCreateWithFlags(&m_pipe.d2h, hipStreamNonBlocking), "hipStreamCreateWithFlags");
    for (int s = 0; s < 2; ++s) {
      hipCheck(hipEventCreateWithFlags(&m_pipe.inReady[s], hipEventDisableTiming), "hipEventCreate");
      hipCheck(hipEventCreateWithFlags(&m_pipe.computed[s], hipEventDisableTiming), "hipEventCreate");
      hipCheck(hipEventCreateWithFlags(&m_pipe.outRead[s], hipEventDisableTiming), "hipEventCreate");
    }
    auto alloc = [&](uint32_t tensor) {
      void *p = nullptr;
      const uint64_t bytes = std::max<uint64_t>(static_cast<uint64_t>(m.tensors[tensor].size.eval(m_sym)), 16) + 256;
      hipCheck(hipMalloc(&p, bytes), "hipMalloc(second interface tensor)");
      m_deviceBytes += bytes;
      return p;
    };
    m_pipe.in.assign(m.inputs.size(), nullptr);
    m_pipe.out.assign(m.outputs.size(), nullptr);
    for (size_t i = 0; i < m.inputs.size(); ++i) m_pipe.in[i] = alloc(m.inputs[i]);
    for (size_t i = 0; i < m.outputs.size(); ++i) m_pipe.out[i] = alloc(m.outputs[i]);
    if (m_graphExec) {
      // the same dispatch list captured once more with the second set's addresses
      std::vector<void *> in0, out0;
      for (uint32_t t : m.inputs) in0.push_back(tensorPtr(t));
      for (uint32_t t : m.outputs) out0.push_back(tensorPtr(t));
      hipGraph_t g0 = m_graph;
      hipGraphExec_t e0 = m_graphExec;
      m_graph = nullptr;
      m_graphExec = nullptr;
      patchInterface(m_pipe.in, m_pipe.out);
      try {
        buildGraph();
      } catch (...) {
        patchInterface(in0, out0);
        m_graph = g0;
        m_graphExec = e0;
        throw;
      }
      m_pipe.graph = m_graph;
      m_pipe.exec = m_graphExec;
      m_graph = g0;
      m_graphExec = e0;
      patchInterface(in0, out0);
    }
    m_pipe.ready = true;
  } catch (...) {
    destroyPipeline();
    throw;
  }
}

void Instance::inferMany(size_t frames, const void *const *inputs, void *const *outputs) {
  const dnx::Model &m = m_model->dnx();
  if (frames == 0) return;
  if (!inputs || !outputs) fail(Status::InvalidArgument, "infer: null pointer array");
  const size_t nin = m.inputs.size(), nout = m.outputs.size();
  for (size_t i = 0; i < frames * nin; ++i) if (!inputs[i]) fail(Status::InvalidArgument, "infer: null input pointer");
  for (size_t i = 0; i < frames * nout; ++i) if (!outputs[i]) fail(Status::InvalidArgument, "infer: null output pointer");
  m_model->context()->makeCurrent();
  rebind(nullptr, nullptr); // set 0 is the instance's own interface tensors
  preparePipeline();
  hipStream_t cs = m_model->context()->stream();
  std::vector<void *> in0, out0;
  for (uint32_t t : m.inputs) in0.push_back(tensorPtr(t));
  for (uint32_t t : m.outputs) out0.push_back(tensorPtr(t));
  // nothing enqueued earlier on the context's stream may still use the interface tensors
  hipCheck(hipStreamSynchronize(cs), "hipStreamSynchronize");
  bool patched = false;
  try {
    for (size_t f = 0; f < frames; ++f) {
      const int s = static_cast<int>(f & 1);
      const std::vector<void *> &din = s ? m_pipe.in : in0, &dout = s ? m_pipe.out : out0;
      // upload: the dispatches of frame f-2 have read this set's inputs
      if (f >= 2) hipCheck(hipStreamWaitEvent(m_pipe.h2d, m_pipe.computed[s], 0), "hipStreamWaitEvent");
      for (size_t i = 0; i < nin; ++i)
        hipCheck(hipMemcpyAsync(din[i], inputs[f * nin + i], static_cast<uint64_t>(m.tensors[m.inputs[i]].size.eval(m_sym)), hipMemcpyHostToDevice, m_pipe.h2d), "hipMemcpyAsync(input)");
      hipCheck(hipEventRecord(m_pipe.inReady[s], m_pipe.h2d), "hipEventRecord");
      // dispatches: inputs are up, and the download of frame f-2 has read this set's outputs
      hipCheck(hipStreamWaitEvent(cs, m_pipe.inReady[s], 0), "hipStreamWaitEvent");
      if (f >= 2) hipCheck(hipStreamWaitEvent(cs, m_pipe.outRead[s], 0), "hipStreamWaitEvent");
      if (m_graphExec) {
        hipCheck(hipGraphLaunch(s ? m_pipe.exec : m_graphExec, cs), "hipGraphLaunch");
      } else { // without a graph the argument buffers are read at launch time: patch them per frame
        patchInterface(din, dout);
        patched = s != 0;
        launchAll(cs);
      }
      hipCheck(hipEventRecord(m_pipe.computed[s], cs), "hipEventRecord");
      // download
      hipCheck(hipStreamWaitEvent(m_pipe.d2h, m_pipe.computed[s], 0), "hipStreamWaitEvent");
      for (size_t i = 0; i < nout; ++i)
        hipCheck(hipMemcpyAsync(outputs[f * nout + i], dout[i], static_cast<uint64_t>(m.tensors[m.outputs[i]].size.eval(m_sym)), hipMemcpyDeviceToHost, m_pipe.d2h), "hipMemcpyAsync(output)");
      hipCheck(hipEventRecord(m_pipe.outRead[s], m_pipe.d2h), "hipEventRecord");
    }
  } catch (...) {
    (void)hipStreamSynchronize(m_pipe.h2d);
    (void)hipStreamSynchronize(cs);
    (void)hipStreamSynchronize(m_pipe.d2h);
    if (patched) patchInterface(in0, out0);
    throw;
  }
  hipCheck(hipStreamSynchronize(m_pipe.h2d), "hipStreamSynchronize");
  hipCheck(hipStreamSynchronize(cs), "hipStreamSynchronize");
  hipCheck(hipStreamSynchronize(m_pipe.d2h), "hipStreamSynchronize");
  if (patched) patchInterface(in0, out0);
}

void Instance::inferDevice(const void *const *inputs, void *const *outputs) {
  m_model->context()->makeCurrent();
  rebind(inputs, outputs);
  hipStream_t s = m_model->context()->stream();
  if (m_graphExec)
    hipCheck(hipGraphLaunch(m_graphExec, s), "hipGraphLaunch");
  else
    launchAll(s);
}

void Instance::inferDeviceStatic(const void *const *inputs, void *const *outputs) {
  // No allocation on this path: no graph is captured or instantiated, nothing is malloc'ed on the device; the
  // argument buffers exist since the instance was made and are only overwritten in place.
  const dnx::Model &m = m_model->dnx();
  if (m_arenaBytes > kStaticScratchBytes)
    fail(Status::Unsupported, "this instance needs " + std::to_string(m_arenaBytes) + " bytes for its intermediate tensors; the static scratch array holds " +
                                  std::to_string(kStaticScratchBytes));
  if (m_arenaBytes && !m_arena) fail(Status::Unsupported, "the allocation-free path needs the intermediate buffers in one arena (DENOX_HIP_NO_ALIAS is set)");
  if (!m_model->context()->staticScratch()) fail(Status::HipError, "the static scratch array has no device address");
  m_model->context()->makeCurrent();
  const Context *ctx = m_model->context().get();
  if (m_arenaBytes) staticScratchAcquire(ctx->device(), ctx);
  for (auto &l : m_launches)
    for (const auto &slot : l.ptrSlots) {
      if (slot.iface < 0) continue;
      void *ext = slot.isInput ? (inputs ? const_cast<void *>(inputs[slot.iface]) : nullptr) : (outputs ? outputs[slot.iface] : nullptr);
      void *base = ext ? ext : tensorPtr(slot.isInput ? m.inputs[static_cast<size_t>(slot.iface)] : m.outputs[static_cast<size_t>(slot.iface)]);
      void *p = static_cast<uint8_t *>(base) + slot.delta;
      std::memcpy(l.staticArgs.data() + slot.offset, &p, sizeof(void *));
    }
  hipStream_t s = m_model->context()->stream();
  for (auto &l : m_launches) launchOne(l.fn, l.grid, l.block, l.staticArgs, s);
  if (m_arenaBytes) staticScratchRecord(ctx->device(), ctx, ctx->staticScratchDone(), s);
}

void Instance::synchronize() {
  m_model->context()->makeCurrent();
  hipCheck(hipStreamSynchronize(m_model->context()->stream()), "hipStreamSynchronize");
}

void Instance::infer(const void *const *inputs, void *const *outputs) {
  const dnx::Model &m = m_model->dnx();
  if (!inputs || !outputs) fail(Status::InvalidArgument, "infer: null pointer array");
  m_model->context()->makeCurrent();
  hipStream_t s = m_model->context()->stream();
  for (size_t i = 0; i < m.inputs.size(); ++i) {
    if (!inputs[i]) fail(Status::InvalidArgument, "infer: null input pointer");
    const uint64_t sz = static_cast<uint64_t>(m.tensors[m.inputs[i]].size.eval(m_sym));
    hipCheck(hipMemcpyAsync(tensorPtr(m.inputs[i]), inputs[i], sz, hipMemcpyHostToDevice, s), "hipMemcpyAsync(input)");
  }
  inferDevice(nullptr, nullptr);
  for (size_t i = 0; i < m.outputs.size(); ++i) {
    if (!outputs[i]) fail(Status::InvalidArgument, "infer: null output pointer");
    const uint64_t sz = static_cast<uint64_t>(m.tensors[m.outputs[i]].size.eval(m_sym));
    hipCheck(hipMemcpyAsync(outputs[i], tensorPtr(m.outputs[i]), sz, hipMemcpyDeviceToHost, s), "hipMemcpyAsync(output)");
  }
  hipCheck(hipStreamSynchronize(s), "hipStreamSynchronize");
}

// One dispatch timed where it runs: `frames` whole inferences as plain launches on the instance's stream, with an event
// in front of and behind dispatch `index` only, so that the kernel finds the caches, clocks and memory traffic of the
// frame around it (launched several times back to back, as bench() does, a matrix-bound kernel runs 4 % slower than
// after a lighter neighbour).  The interval holds one launch gap; returns the mean over the frames in milliseconds.
float Instance::benchInFrame(uint32_t index, int frames, int warmup) {
  if (index >= m_launches.size()) fail(Status::InvalidArgument, "dispatch index out of range");
  if (frames < 1) fail(Status::InvalidArgument, "frames must be at least 1");
  m_model->context()->makeCurrent();
  rebind(nullptr, nullptr);
  hipStream_t s = m_model->context()->stream();
  for (int i = 0; i < warmup; ++i) launchAll(s);
  hipCheck(hipStreamSynchronize(s), "hipStreamSynchronize");
  std::vector<hipEvent_t> ev(2 * static_cast<size_t>(frames), nullptr);
  double sum = 0.0;
  try {
    for (auto &e : ev) hipCheck(hipEventCreate(&e), "hipEventCreate");
    for (int f = 0; f < frames; ++f)
      for (size_t i = 0; i < m_launches.size(); ++i) {
        auto &l = m_launches[i];
        if (i == index) hipCheck(hipEventRecord(ev[2 * static_cast<size_t>(f)], s), "hipEventRecord");
        launchOne(l.fn, l.grid, l.block, l.args, s);
        if (i == index) hipCheck(hipEventRecord(ev[2 * static_cast<size_t>(f) + 1], s), "hipEventRecord");
      }
    hipCheck(hipStreamSynchronize(s), "hipStreamSynchronize");
    for (int f = 0; f < frames; ++f) {
      float ms = 0.0f;
      hipCheck(hipEventElapsedTime(&ms, ev[2 * static_cast<size_t>(f)], ev[2 * static_cast<size_t>(f) + 1]), "hipEventElapsedTime");
      sum += ms;
    }
  } catch (...) {
    for (auto e : ev) if (e) (void)hipEventDestroy(e);
    throw;
  }
  for (auto e : ev) if (e) (void)hipEventDestroy(e);
  return static_cast<float>(sum / frames);
}

std::vector<DispatchTiming> Instance::bench(int warmup) {
  const dnx::Model &m = m_model->dnx();
  m_model->context()->makeCurrent();
  rebind(nullptr, nullptr);
  hipStream_t s = m_model->context()->stream();
  for (int i = 0; i < warmup; ++i) {
    if (m_graphExec) hipCheck(hipGraphLaunch(m_graphExec, s), "hipGraphLaunch");
    else launchAll(s);
  }
  hipCheck(hipStreamSynchronize(s), "hipStreamSynchronize");
  std::vector<hipEvent_t> ev(m_launches.size() + 1, nullptr);
  std::vector<DispatchTiming> out;
  try {
    for (auto &e : ev) hipCheck(hipEventCreate(&e), "hipEventCreate");
    hipCheck(hipEventRecord(ev[0], s), "hipEventRecord");
    // Each dispatch runs kReps times back to back between its two events (every kernel is a pure function of its
    // inputs, so repeating it changes nothing): the cost of recording an event and of the launch gap, several
    // microseconds, is spread over the repetitions instead of being charged to one launch.
    constexpr int kReps = 4;
    for (size_t i = 0; i < m_launches.size(); ++i) {
      auto &l = m_launches[i];
      for (int r = 0; r < kReps; ++r) launchOne(l.fn, l.grid, l.block, l.args, s);
      hipCheck(hipEventRecord(ev[i + 1], s), "hipEventRecord");
    }
    hipCheck(hipStreamSynchronize(s), "hipStreamSynchronize");
    auto fmt = [&](uint32_t t) {
      const auto &ti = m.tensors[t].info;
      const char *f = ti.format == dnx::TensorFormat::SSBO_HWC ? "HWC" : ti.format == dnx::TensorFormat::SSBO_CHW ? "CHW" : ti.format == dnx::TensorFormat::SSBO_CHWC8 ? "CHWC8" : "?";
      return std::string(f) + "[" + (ti.has_extent ? std::to_string(ti.channels.eval(m_sym)) : std::string("-")) + "]";
    };
    for (size_t i = 0; i < m_launches.size(); ++i) {
      const auto &md = m_model->dispatches()[i];
      const auto &d = *md.dnx;
      DispatchTiming t;
      t.name = d.info.name;
      for (const auto &[tensor, access] : md.tensors) {
        const bool param = std::any_of(m.initializers.begin(), m.initializers.end(), [&](const auto &in) { return in.tensor == tensor; });
        if (param) continue;
        if (access == dnx::Access::ReadOnly) t.input += (t.input.empty() ? "" : "+") + fmt(tensor);
        else t.output += (t.output.empty() ? "" : "+") + fmt(tensor);
      }
      if (d.info.has_reads) t.memoryReads = static_cast<uint64_t>(d.info.memory_reads.eval(m_sym));
      if (d.info.has_writes) t.memoryWrites = static_cast<uint64_t>(d.info.memory_writes.eval(m_sym));
      if (d.info.has_flops) t.flops = static_cast<uint64_t>(d.info.flops.eval(m_sym));
      hipCheck(hipEventElapsedTime(&t.latencyMs, ev[i], ev[i + 1]), "hipEventElapsedTime");
      t.latencyMs /= static_cast<float>(kReps);
      out.push_back(std::move(t));
    }
  } catch (...) {
    for (auto e : ev) if (e) (void)hipEventDestroy(e);
    throw;
  }
  for (auto e : ev) if (e) (void)hipEventDestroy(e);
  return out;
}

} // namespace denox::runtime
