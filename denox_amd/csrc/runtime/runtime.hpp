// Run-time half of the backend: load a compiled model, bind it to concrete
// image extents, execute it on one HIP stream.
//
// Same object model as the reference runtime --
//   Context  : runtime/src/denox/runtime/context.hpp:113-252 (device + queue)
//   Model    : runtime/src/denox/runtime/model.hpp:107-170, model.cpp:80-239,637-659
//   Instance : runtime/src/denox/runtime/instance.hpp:44-63, instance.cpp:25-430
// -- with Vulkan replaced by the HIP module API: one hipModule_t per shader
// binary, one hipFunction_t per dispatch, kernel arguments = bound tensor
// addresses in (set, binding) order followed by the push-constant bytes, all
// launches in program order on a single stream (which makes the reference's
// barrier insertion, model.cpp:247-340, unnecessary), and the whole dispatch
// list captured once per Instance into a hipGraph.
#pragma once
#include "../common/dnx.hpp"
#include <hip/hip_runtime_api.h>
#include <memory>
#include <string>
#include <vector>

namespace denox::runtime {

void hipCheck(hipError_t e, const char *what);

class Context {
public:
  explicit Context(int device);
  ~Context();
  Context(const Context &) = delete;
  Context &operator=(const Context &) = delete;
  int device() const { return m_device; }
  hipStream_t stream() const { return m_stream; }
  void makeCurrent() const;
  const hipDeviceProp_t &props() const { return m_props; }
  // this device's copy of the library's static scratch array (static_scratch.hip); resolved when the context is made
  void *staticScratch() const { return m_staticScratch; }
  // recorded behind every call of the allocation-free entry point (created with the context: that call creates nothing)
  hipEvent_t staticScratchDone() const { return m_staticDone; }

private:
  int m_device;
  hipStream_t m_stream = nullptr;
  hipDeviceProp_t m_props;
  void *m_staticScratch = nullptr;
  hipEvent_t m_staticDone = nullptr;
};

// The library's allocation-free path keeps intermediate results in a file-scope device array of this many bytes per GPU.
constexpr uint64_t kStaticScratchBytes = 64ull << 20;
// Device address of that array on `device`, which must be current (hipGetSymbolAddress once per device, then cached).
void *staticScratchAddress(int device);
// One user at a time per GPU.  Acquire: refuses (InvalidArgument) while a call made through another context is still running.
// Record: marks `context` as the user, with `done` recorded on `stream` behind the launches.  Forget: a context that is being
// destroyed (its stream already synchronized) gives the array up.
void staticScratchAcquire(int device, const void *context);
void staticScratchRecord(int device, const void *context, hipEvent_t done, hipStream_t stream);
void staticScratchForget(int device, const void *context);
using ContextHandle = std::shared_ptr<Context>;

struct ModelDispatch {
  const dnx::ComputeDispatch *dnx = nullptr;
  hipFunction_t function = nullptr;
  std::vector<std::pair<uint32_t, dnx::Access>> tensors; // flattened in (set, binding) order
};

class Model {
public:
  Model(ContextHandle ctx, const void *dnxbuf, size_t size);
  ~Model();
  Model(const Model &) = delete;
  Model &operator=(const Model &) = delete;
  const ContextHandle &context() const { return m_ctx; }
  const dnx::Model &dnx() const { return m_dnx; }
  const std::vector<ModelDispatch> &dispatches() const { return m_dispatches; }

private:
  ContextHandle m_ctx;
  dnx::Model m_dnx;
  std::vector<hipModule_t> m_modules;
  std::vector<ModelDispatch> m_dispatches;
};
using ModelHandle = std::shared_ptr<Model>;

struct ValueSpec { std::string name; int64_t value; };

struct TensorDesc {
  int64_t width = 0, height = 0, channels = 0;
  dnx::TensorFormat format = dnx::TensorFormat::UNKNOWN;
  dnx::ScalarType dtype = dnx::ScalarType::F16;
  uint64_t byteSize = 0;
  std::string name;
};

struct DispatchTiming {
  std::string name, input, output;
  uint64_t memoryReads = 0, memoryWrites = 0, flops = 0;
  float latencyMs = 0.0f;
};

class Instance {
public:
  Instance(ModelHandle model, const std::vector<ValueSpec> &specs);
  ~Instance();
  Instance(const Instance &) = delete;
  Instance &operator=(const Instance &) = delete;

  // Host pointers, arrays in model input / output order, tightly packed in the
  // tensor's declared format; blocking (instance.cpp:322-430 of the reference).
  void infer(const void *const *inputs, void *const *outputs);
  // Device pointers (inputs already resident in HBM); enqueues on the context's
  // stream and returns without synchronising.  A null entry means "use the
  // instance's own buffer for that tensor" (see inputDevicePtr/outputDevicePtr).
  void inferDevice(const void *const *inputs, void *const *outputs);
  // inferDevice without any allocation: plain launches (no graph is built or instantiated) with the intermediate
  // buffers placed in the library's static scratch array instead of this instance's arena.  Fails when the arena
  // would not fit.  Every instance on one GPU shares that array: calls that overlap in time race.
  void inferDeviceStatic(const void *const *inputs, void *const *outputs);
  uint64_t arenaBytes() const { return m_arenaBytes; }
  // A sequence of frames from host memory, arrays frame-major (inputs[f * inputCount() + i]); blocking.
  // Upload of frame f+1, the dispatches of frame f and the download of frame f-1 run at the same time on three
  // streams: the interface tensors exist twice, everything in between once (the dispatches of consecutive frames
  // are serialised on the context's stream anyway).  The copies overlap only when the host memory is pinned
  // (hipHostMalloc); with pageable memory the result is the same and the transfers are staged by the driver.
  // The reference has no counterpart: its infer() is one blocking frame (instance.cpp:322-430).
  void inferMany(size_t frames, const void *const *inputs, void *const *outputs);
  void synchronize();
  // Per-dispatch timings with hipEvents after warm-up passes (instance.cpp:432-654).
  std::vector<DispatchTiming> bench(int warmup);
  float benchInFrame(uint32_t index, int frames, int warmup);

  size_t inputCount() const { return m_model->dnx().inputs.size(); }
  size_t outputCount() const { return m_model->dnx().outputs.size(); }
  TensorDesc inputDesc(size_t i) const { return describe(m_model->dnx().inputs.at(i)); }
  TensorDesc outputDesc(size_t i) const { return describe(m_model->dnx().outputs.at(i)); }
  void *inputDevicePtr(size_t i) const { return tensorPtr(m_model->dnx().inputs.at(i)); }
  void *outputDevicePtr(size_t i) const { return tensorPtr(m_model->dnx().outputs.at(i)); }
  uint64_t deviceBytes() const { return m_deviceBytes; }
  bool usesGraph() const { return m_graphExec != nullptr; } // false while plain launches stand in (no graph wanted, or none captured yet)

private:
  struct Launch {
    hipFunction_t fn;
    unsigned grid[3], block[3];
    std::vector<uint8_t> args;              // pointers then push constants
    std::vector<uint8_t> staticArgs;        // the same with arena addresses replaced by static-scratch addresses
    // One per bound tensor.  A tensor that lives in the buffer of an interface tensor (that tensor itself, or a channel
    // range of it written in place) follows the interface address: iface = index into inputs (isInput) / outputs,
    // delta = byte distance from the interface tensor's start; iface < 0 otherwise.
    struct Slot { size_t offset; uint32_t tensor; int iface; bool isInput; int64_t delta; };
    std::vector<Slot> ptrSlots;
  };
  TensorDesc describe(uint32_t tensor) const;
  void *tensorPtr(uint32_t tensor) const;
  void launchAll(hipStream_t s);
  void buildGraph();
  void rebind(const void *const *inputs, void *const *outputs);
  void patchInterface(const std::vector<void *> &inputs, const std::vector<void *> &outputs, bool staticArgs = false);
  void preparePipeline();

  ModelHandle m_model;
  std::vector<int64_t> m_sym;
  std::vector<void *> m_buffers;
  std::vector<char> m_ownBuffer; // 1: an allocation of its own, 0: a range of m_arena
  void *m_arena = nullptr;       // memory shared by the intermediate buffers
  uint64_t m_arenaBytes = 0;
  void freeBuffers();
  std::vector<uint64_t> m_bufferSizes;
  std::vector<Launch> m_launches;
  std::vector<void *> m_boundInputs, m_boundOutputs; // external overrides currently patched in
  hipGraph_t m_graph = nullptr;       // the captured dispatch list for the interface addresses bound now
  hipGraphExec_t m_graphExec = nullptr;
  // Captured graphs of interface addresses used before (a caller that alternates between a few sets of buffers
  // finds its graph again instead of paying a capture per frame); m_graph / m_graphExec are one of these.
  struct CachedGraph { std::vector<void *> key; hipGraph_t graph; hipGraphExec_t exec; uint64_t lastUse; };
  std::vector<CachedGraph> m_graphCache;
  uint64_t m_graphUse = 0;
  bool m_useGraph = false;
  bool m_graphStale = false; // the bound interface addresses have no captured graph yet (a capture failed)
  void selectGraph();
  void destroyGraphs();
  uint64_t m_deviceBytes = 0;
  // inferMany: the second set of interface tensors with its own captured graph, copy streams, per-set events
  struct Pipeline {
    std::vector<void *> in, out;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hipStream_t h2d = nullptr, d2h = nullptr;
    hipEvent_t inReady[2] = {nullptr, nullptr}, computed[2] = {nullptr, nullptr}, outRead[2] = {nullptr, nullptr};
    bool ready = false;
  } m_pipe;
  void destroyPipeline();
};

} // namespace denox::runtime
