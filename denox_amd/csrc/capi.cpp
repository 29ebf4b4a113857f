// C ABI over the compiler, database and runtime classes (include/denox_hip.h).
#pragma GCC visibility push(default)
#include "../../include/denox_hip.h"
#pragma GCC visibility pop
#include "common/sha256.hpp"
#include "compiler/compile.hpp"
#include "database/db.hpp"
#include "device_info/device_info.hpp"
#include "frontend/onnx_import.hpp"
#include "hip/hip_compiler.hpp"
#include "runtime/db_bench.hpp"
#include "runtime/runtime.hpp"
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <sstream>

using namespace denox;

struct denox_hip_context { runtime::ContextHandle ctx; };
struct denox_hip_model { runtime::ModelHandle model; };
struct denox_hip_instance { std::unique_ptr<runtime::Instance> inst; };
struct denox_hip_builder { compiler::Model model; };
struct denox_hip_db { Db db; };

namespace {
thread_local std::string g_lastError;
thread_local std::string g_lastReport;
std::mutex g_pathMutex;
std::string g_kernelDir, g_cacheDir;
bool g_cacheDirSet = false;

int fail_with(Status s, const std::string &msg) {
  g_lastError = msg;
  return static_cast<int>(s);
}

template <class F> int guarded(F &&f) {
  try {
    f();
    return DENOX_HIP_OK;
  } catch (const Error &e) {
    return fail_with(e.status, e.what());
  } catch (const std::bad_alloc &) {
    return fail_with(Status::Internal, "out of host memory");
  } catch (const std::exception &e) {
    return fail_with(Status::Internal, e.what());
  } catch (...) {
    return fail_with(Status::Internal, "unknown failure");
  }
}

void need(const void *p, const char *what) {
  if (!p) fail(Status::InvalidArgument, std::string(what) + " is null");
}

hip::HipCompiler makeCompiler() {
  std::lock_guard<std::mutex> lock(g_pathMutex);
  return hip::HipCompiler(g_kernelDir.empty() ? hip::defaultKernelDir() : g_kernelDir, g_cacheDirSet ? g_cacheDir : hip::defaultCacheDir());
}

Sym symFromHandle(int64_t h) {
  // handles: bit 62 set = symbolic reference, else constant (constants are limited to +-2^61)
  if (h & (int64_t(1) << 62)) return Sym::Ref(h & ~(int64_t(1) << 62));
  return Sym::Const(h >= (int64_t(1) << 61) ? h - (int64_t(1) << 62) : h);
}
int64_t handleFromSym(Sym s) {
  if (s.symbolic) return s.v | (int64_t(1) << 62);
  if (s.v >= (int64_t(1) << 61) || s.v < -(int64_t(1) << 61)) fail(Status::InvalidArgument, "symbolic constant out of range");
  return s.v < 0 ? s.v + (int64_t(1) << 62) : s.v;
}

compiler::CompileOptions toOptions(const denox_hip_compile_options *o) {
  compiler::CompileOptions opt;
  if (!o) return opt;
  opt.features.enableConvReluFusion = o->enable_conv_relu_fusion != 0;
  opt.features.enableConcatConvFusion = o->enable_concat_conv_fusion != 0;
  opt.features.enableUpsampleFusion = o->enable_upsample_fusion != 0;
  opt.features.enablePoolFusion = o->enable_pool_fusion != 0;
  opt.features.enablePadFusion = o->enable_pad_fusion != 0;
  opt.features.enableSliceFusion = o->enable_slice_fusion != 0;
  opt.features.enableAlternatingTraversal = o->enable_alternating_traversal != 0;
  opt.features.enableUpsampleFold = o->enable_upsample_fold != 0;
  opt.features.enableImplicitConcat = o->enable_implicit_concat != 0;
  opt.features.enableConvConvFusion = o->enable_conv_conv_fusion != 0;
  opt.features.enableBlockedLayout = o->enable_blocked_layout != 0;
  opt.layoutPreference = o->layout_preference;
  auto fmt = [](int f) {
    switch (f) {
    case 0: case DENOX_HIP_FORMAT_HWC: return dnx::TensorFormat::SSBO_HWC;
    case DENOX_HIP_FORMAT_CHW: return dnx::TensorFormat::SSBO_CHW;
    case DENOX_HIP_FORMAT_CHWC8: return dnx::TensorFormat::SSBO_CHWC8;
    default: fail(Status::InvalidArgument, "unknown tensor format");
    }
  };
  // one unnamed descriptor applies to every interface tensor of that side
  const dnx::TensorFormat inF = fmt(o->input_format), outF = fmt(o->output_format);
  for (int i = 0; i < 16; ++i) {
    opt.inputDescriptors.push_back(compiler::InterfaceTensorDescriptor{"", inF});
    opt.outputDescriptors.push_back(compiler::InterfaceTensorDescriptor{"", outF});
  }
  for (uint32_t i = 0; i < o->assumption_count; ++i) {
    need(o->assumption_names, "assumption_names");
    need(o->assumption_values, "assumption_values");
    opt.assumptions[o->assumption_names[i]] = o->assumption_values[i];
  }
  if (o->force_conv_config) opt.forceConvConfig = o->force_conv_config;
  opt.deviceInfo = o->device >= 0 ? query_driver_device_info(o->device) : cdna4_device_info();
  return opt;
}

void copyStr(char *dst, size_t cap, const std::string &s) {
  const size_t n = std::min(cap - 1, s.size());
  std::memcpy(dst, s.data(), n);
  dst[n] = '\0';
}
} // namespace

extern "C" {

const char *denox_hip_last_error(void) { return g_lastError.c_str(); }
const char *denox_hip_version(void) { return "denox-hip 0.1 (gfx950)"; }

int denox_hip_set_kernel_paths(const char *kernel_dir, const char *cache_dir) {
  return guarded([&] {
    std::lock_guard<std::mutex> lock(g_pathMutex);
    g_kernelDir = kernel_dir ? kernel_dir : "";
    g_cacheDirSet = cache_dir != nullptr;
    g_cacheDir = cache_dir ? cache_dir : "";
  });
}

int denox_hip_query_device_info(int device, denox_hip_device_info *out) {
  return guarded([&] {
    need(out, "out");
    const DeviceInfo d = device >= 0 ? query_driver_device_info(device) : cdna4_device_info();
    std::memset(out, 0, sizeof(*out));
    copyStr(out->name, sizeof(out->name), d.name);
    copyStr(out->arch, sizeof(out->arch), d.arch);
    out->subgroup_size = d.subgroupSize;
    out->max_workgroup_invocations = d.maxComputeWorkGroupInvocations;
    for (int i = 0; i < 3; ++i) { out->max_workgroup_size[i] = d.maxComputeWorkGroupSize[i]; out->max_workgroup_count[i] = d.maxComputeWorkGroupCount[i]; }
    out->max_shared_memory = d.maxComputeSharedMemory;
    out->compute_units = d.computeUnits;
    out->xcd_count = d.xcdCount;
    out->hbm_bytes = d.hbmBytes;
    out->hbm_bytes_per_second = d.hbmBytesPerSecond;
    out->fp16_mfma_flops = d.fp16MfmaFlops;
    out->matrix_shape_count = static_cast<uint32_t>(std::min<size_t>(4, d.matrixShapes.size()));
    for (uint32_t i = 0; i < out->matrix_shape_count; ++i) { out->matrix_shapes[i][0] = d.matrixShapes[i].m; out->matrix_shapes[i][1] = d.matrixShapes[i].n; out->matrix_shapes[i][2] = d.matrixShapes[i].k; }
    out->from_device = d.fromDevice ? 1 : 0;
  });
}

// ---------------------------------------------------------------- builder
int denox_hip_builder_create(denox_hip_builder **out) {
  return guarded([&] { need(out, "out"); *out = new denox_hip_builder(); });
}
void denox_hip_builder_destroy(denox_hip_builder *b) { delete b; }

int denox_hip_builder_sym_const(denox_hip_builder *b, int64_t value, int64_t *out_sym) {
  return guarded([&] { need(b, "builder"); need(out_sym, "out_sym"); *out_sym = handleFromSym(Sym::Const(value)); });
}
int denox_hip_builder_sym_var(denox_hip_builder *b, const char *name, int64_t *out_sym) {
  return guarded([&] { need(b, "builder"); need(name, "name"); need(out_sym, "out_sym"); *out_sym = handleFromSym(b->model.requireValueOfName(name)); });
}
int denox_hip_builder_sym_op(denox_hip_builder *b, int op, int64_t lhs, int64_t rhs, int64_t *out_sym) {
  return guarded([&] {
    need(b, "builder"); need(out_sym, "out_sym");
    if (op < DENOX_HIP_SYM_ADD || op > DENOX_HIP_SYM_MAX) fail(Status::InvalidArgument, "unknown symbolic op");
    *out_sym = handleFromSym(b->model.symGraph().op(static_cast<uint16_t>(op), symFromHandle(lhs), symFromHandle(rhs)));
  });
}
int denox_hip_builder_input(denox_hip_builder *b, const char *name, int64_t w, int64_t h, uint32_t channels, int *out_tensor) {
  return guarded([&] { need(b, "builder"); need(name, "name"); need(out_tensor, "out_tensor"); *out_tensor = b->model.input(name, symFromHandle(w), symFromHandle(h), channels); });
}
int denox_hip_builder_conv2d(denox_hip_builder *b, int src, uint32_t K, uint32_t C, uint32_t R, uint32_t S, const uint16_t *w, const uint16_t *bias,
                             uint32_t sx, uint32_t sy, uint32_t px, uint32_t py, uint32_t dx, uint32_t dy, int *out_tensor) {
  return guarded([&] { need(b, "builder"); need(w, "weights"); need(out_tensor, "out_tensor"); *out_tensor = b->model.conv2d(src, K, C, R, S, w, bias, sx, sy, px, py, dx, dy); });
}
int denox_hip_builder_activation(denox_hip_builder *b, int src, int func, float alpha, int *out_tensor) {
  return guarded([&] {
    need(b, "builder"); need(out_tensor, "out_tensor");
    if (func != DENOX_HIP_ACT_RELU && func != DENOX_HIP_ACT_LEAKY_RELU) fail(Status::InvalidArgument, "unknown activation function");
    *out_tensor = b->model.activation(src, func == DENOX_HIP_ACT_RELU ? compiler::ActivationFunction::ReLU : compiler::ActivationFunction::LeakyReLU, alpha);
  });
}
int denox_hip_builder_upsample(denox_hip_builder *b, int src, uint32_t scale, int *out_tensor) {
  return guarded([&] { need(b, "builder"); need(out_tensor, "out_tensor"); *out_tensor = b->model.upsample(src, scale, compiler::FilterMode::Nearest); });
}
int denox_hip_builder_pool(denox_hip_builder *b, int src, uint32_t kx, uint32_t ky, uint32_t px, uint32_t py, uint32_t sx, uint32_t sy, int *out_tensor) {
  return guarded([&] { need(b, "builder"); need(out_tensor, "out_tensor"); *out_tensor = b->model.pool(src, kx, ky, px, py, sx, sy, compiler::PoolFunction::Max); });
}
int denox_hip_builder_avg_pool(denox_hip_builder *b, int src, uint32_t kx, uint32_t ky, uint32_t px, uint32_t py, uint32_t sx, uint32_t sy, int *out_tensor) {
  return guarded([&] { need(b, "builder"); need(out_tensor, "out_tensor"); *out_tensor = b->model.pool(src, kx, ky, px, py, sx, sy, compiler::PoolFunction::Avg); });
}
int denox_hip_builder_concat(denox_hip_builder *b, int src0, int src1, int *out_tensor) {
  return guarded([&] { need(b, "builder"); need(out_tensor, "out_tensor"); *out_tensor = b->model.concat(src0, src1); });
}
int denox_hip_builder_pad(denox_hip_builder *b, int src, int64_t l, int64_t r, int64_t t, int64_t bo, int *out_tensor) {
  return guarded([&] { need(b, "builder"); need(out_tensor, "out_tensor"); *out_tensor = b->model.pad(src, symFromHandle(l), symFromHandle(r), symFromHandle(t), symFromHandle(bo), compiler::PaddingMode::Replicate); });
}
int denox_hip_builder_pad_mode(denox_hip_builder *b, int src, int64_t l, int64_t r, int64_t t, int64_t bo, int32_t mode, int *out_tensor) {
  return guarded([&] {
    need(b, "builder"); need(out_tensor, "out_tensor");
    if (mode != 0 && mode != 1) fail(Status::InvalidArgument, "pad mode must be 0 (replicate) or 1 (zero)");
    *out_tensor = b->model.pad(src, symFromHandle(l), symFromHandle(r), symFromHandle(t), symFromHandle(bo), mode ? compiler::PaddingMode::Zero : compiler::PaddingMode::Replicate);
  });
}
int denox_hip_builder_slice(denox_hip_builder *b, int src, int64_t l, int64_t r, int64_t t, int64_t bo, int *out_tensor) {
  return guarded([&] { need(b, "builder"); need(out_tensor, "out_tensor"); *out_tensor = b->model.slice(src, symFromHandle(l), symFromHandle(r), symFromHandle(t), symFromHandle(bo)); });
}
int denox_hip_builder_output(denox_hip_builder *b, int src, const char *name) {
  return guarded([&] { need(b, "builder"); need(name, "name"); b->model.output(src, name); });
}

int denox_hip_builder_import_onnx(denox_hip_builder *b, const void *onnx_bytes, size_t size) {
  return guarded([&] { need(b, "builder"); need(onnx_bytes, "onnx_bytes"); onnx::importModel(b->model, static_cast<const uint8_t *>(onnx_bytes), size); });
}
int denox_hip_builder_input_count(const denox_hip_builder *b, uint32_t *out) {
  return guarded([&] { need(b, "builder"); need(out, "out"); *out = static_cast<uint32_t>(b->model.inputs().size()); });
}
int denox_hip_builder_output_count(const denox_hip_builder *b, uint32_t *out) {
  return guarded([&] { need(b, "builder"); need(out, "out"); *out = static_cast<uint32_t>(b->model.outputs().size()); });
}
namespace {
void tensorInfo(const compiler::Model &m, const std::vector<compiler::TensorHandle> &list, uint32_t i, char *name, size_t capacity, uint32_t *channels) {
  if (i >= list.size()) fail(Status::InvalidArgument, "index out of range");
  const auto &t = m.tensors()[static_cast<size_t>(list[i])];
  if (name && capacity) {
    const size_t n = std::min(capacity - 1, t.name.size());
    std::memcpy(name, t.name.data(), n);
    name[n] = 0;
  }
  if (channels) *channels = t.channels;
}
} // namespace
int denox_hip_builder_input_info(const denox_hip_builder *b, uint32_t i, char *name, size_t capacity, uint32_t *out_channels) {
  return guarded([&] { need(b, "builder"); tensorInfo(b->model, b->model.inputs(), i, name, capacity, out_channels); });
}
int denox_hip_builder_output_info(const denox_hip_builder *b, uint32_t i, char *name, size_t capacity, uint32_t *out_channels) {
  return guarded([&] { need(b, "builder"); tensorInfo(b->model, b->model.outputs(), i, name, capacity, out_channels); });
}

// ---------------------------------------------------------------- compile
void denox_hip_compile_options_default(denox_hip_compile_options *o) {
  if (!o) return;
  std::memset(o, 0, sizeof(*o));
  o->enable_conv_relu_fusion = o->enable_concat_conv_fusion = o->enable_upsample_fusion = o->enable_pool_fusion = 1;
  o->enable_pad_fusion = o->enable_slice_fusion = 1;
  o->enable_alternating_traversal = 1;
  o->enable_upsample_fold = 1;
  o->enable_implicit_concat = 1;
  o->enable_conv_conv_fusion = 1;
  o->enable_blocked_layout = 1;
  o->layout_preference = 0;
  o->device = -1;
  o->populate_compile_kernels = 1;
  o->kernel_shard_index = 0;
  o->kernel_shard_count = 1;
}

int denox_hip_compile(const denox_hip_builder *b, const denox_hip_compile_options *o, const denox_hip_db *db, void **out_dnx, size_t *out_size) {
  return guarded([&] {
    need(b, "builder"); need(out_dnx, "out_dnx"); need(out_size, "out_size");
    const compiler::CompileOptions opt = toOptions(o);
    const hip::HipCompiler hipc = makeCompiler();
    compiler::CompileReport rep;
    const std::vector<uint8_t> blob = compiler::compile(b->model, hipc, db ? &db->db : nullptr, opt, &rep);
    std::ostringstream ss;
    ss << "edges=" << rep.superGraphEdges << " selected=" << rep.selectedEdges << " dispatches=" << rep.dispatches << " compiled=" << rep.kernelsCompiled
       << " cache_hits=" << rep.kernelCacheHits << " estimated_ms=" << rep.estimatedMs << "\n";
    for (const auto &s : rep.schedule) ss << s.shader << " " << s.config << " " << s.name << " " << s.costMs << (s.measured ? " measured" : " estimated") << "\n";
    for (const auto &w : rep.warnings) ss << "warning: " << w << "\n";
    g_lastReport = ss.str();
    void *p = std::malloc(blob.size());
    if (!p) fail(Status::Internal, "out of host memory");
    std::memcpy(p, blob.data(), blob.size());
    *out_dnx = p;
    *out_size = blob.size();
  });
}
const char *denox_hip_conv_config_names(void) {
  static const std::string names = [] {
    std::string s;
    for (const auto &n : compiler::conv_config_names()) s += (s.empty() ? "" : ",") + n;
    return s;
  }();
  return names.c_str();
}
const char *denox_hip_last_compile_report(void) { return g_lastReport.c_str(); }

int denox_hip_min_cost_subgraph(uint32_t node_count, const uint8_t *is_input, uint32_t edge_count, const uint32_t *edge_input_offsets,
                                 const int32_t *edge_inputs, const int32_t *edge_outputs, const double *edge_costs, uint32_t output_count,
                                 const int32_t *outputs, uint32_t *out_chosen, uint32_t *out_chosen_count, double *out_total) {
  return guarded([&] {
    need(is_input, "is_input"); need(edge_input_offsets, "edge_input_offsets"); need(edge_outputs, "edge_outputs"); need(edge_costs, "edge_costs");
    need(outputs, "outputs"); need(out_chosen, "out_chosen"); need(out_chosen_count, "out_chosen_count");
    std::vector<bool> isIn(node_count);
    for (uint32_t i = 0; i < node_count; ++i) isIn[i] = is_input[i] != 0;
    std::vector<compiler::HyperEdge> edges(edge_count);
    std::vector<double> costs(edge_costs, edge_costs + edge_count);
    for (uint32_t e = 0; e < edge_count; ++e) {
      if (edge_input_offsets[e + 1] < edge_input_offsets[e]) fail(Status::InvalidArgument, "edge_input_offsets must be non-decreasing");
      if (edge_input_offsets[e + 1] > edge_input_offsets[e]) need(edge_inputs, "edge_inputs");
      edges[e].inputs.assign(edge_inputs + edge_input_offsets[e], edge_inputs + edge_input_offsets[e + 1]);
      edges[e].output = edge_outputs[e];
    }
    double total = 0.0;
    const std::vector<size_t> chosen = compiler::minimum_cost_subgraph(isIn, edges, costs, std::vector<int>(outputs, outputs + output_count), &total);
    for (size_t i = 0; i < chosen.size(); ++i) out_chosen[i] = static_cast<uint32_t>(chosen[i]);
    *out_chosen_count = static_cast<uint32_t>(chosen.size());
    if (out_total) *out_total = total;
  });
}

static void jsonEscape(std::ostringstream &o, const std::string &s) {
  o << '"';
  for (char c : s) {
    if (c == '"' || c == '\\') o << '\\' << c;
    else if (static_cast<unsigned char>(c) < 0x20) o << ' ';
    else if (static_cast<unsigned char>(c) >= 0x80) { // names are ASCII; a damaged file must still yield valid JSON
      static const char *hex = "0123456789abcdef";
      o << "\\u00" << hex[(static_cast<unsigned char>(c) >> 4) & 15] << hex[c & 15];
    } else o << c;
  }
  o << '"';
}

int denox_hip_dnx_describe(const void *dnxbuf, size_t size, const char *const *names, const int64_t *values, uint32_t n, char **out_json) {
  return guarded([&] {
    need(dnxbuf, "dnx"); need(out_json, "out_json");
    const dnx::Model m = dnx::deserialize(dnxbuf, size);
    std::vector<int64_t> vars(m.sym_ir.varCount, 0);
    for (uint32_t i = 0; i < n; ++i) {
      need(names, "names"); need(values, "values");
      for (const auto &vn : m.value_names)
        if (vn.name == names[i] && vn.value.symbolic && static_cast<uint64_t>(vn.value.value) < vars.size()) vars[static_cast<size_t>(vn.value.value)] = values[i];
    }
    const std::vector<int64_t> dp = m.sym_ir.eval(vars);
    if (n > 0) m.checkRequirements(dp); // (without extents every variable reads as zero: a listing, not an evaluation)
    std::ostringstream o;
    o << "{\"producer\":"; jsonEscape(o, m.info.producer);
    o << ",\"var_count\":" << m.sym_ir.varCount << ",\"sym_ops\":" << m.sym_ir.ops.size();
    o << ",\"value_names\":[";
    for (size_t i = 0; i < m.value_names.size(); ++i) { if (i) o << ','; jsonEscape(o, m.value_names[i].name); }
    o << "],\"inputs\":[";
    for (size_t i = 0; i < m.inputs.size(); ++i) o << (i ? "," : "") << m.inputs[i];
    o << "],\"outputs\":[";
    for (size_t i = 0; i < m.outputs.size(); ++i) o << (i ? "," : "") << m.outputs[i];
    o << "],\"buffers\":[";
    for (size_t i = 0; i < m.buffers.size(); ++i) o << (i ? "," : "") << "{\"size\":" << m.buffers[i].size.eval(dp) << ",\"alignment\":" << m.buffers[i].alignment << "}";
    o << "],\"tensors\":[";
    std::vector<bool> isParam(m.tensors.size(), false);
    for (const auto &in : m.initializers) isParam[in.tensor] = true;
    for (size_t i = 0; i < m.tensors.size(); ++i) {
      const auto &t = m.tensors[i];
      o << (i ? "," : "") << "{\"buffer\":" << t.buffer << ",\"offset\":" << t.offset.eval(dp) << ",\"size\":" << t.size.eval(dp) << ",\"format\":" << static_cast<int>(t.info.format)
        << ",\"param\":" << (isParam[i] ? "true" : "false") << ",\"name\":";
      jsonEscape(o, t.info.name);
      if (t.info.has_extent) {
        o << ",\"width\":" << t.info.width.eval(dp) << ",\"height\":" << t.info.height.eval(dp) << ",\"channels\":" << t.info.channels.eval(dp);
        // the named extent an input's width / height is, when it is one (what `infer` sets from the image it is given)
        auto nameOf = [&](const dnx::ScalarSource &src) -> const std::string * {
          if (!src.symbolic) return nullptr;
          for (const auto &vn : m.value_names) if (vn.value.symbolic && vn.value.value == src.value) return &vn.name;
          return nullptr;
        };
        if (const std::string *nm = nameOf(t.info.width)) { o << ",\"width_name\":"; jsonEscape(o, *nm); }
        if (const std::string *nm = nameOf(t.info.height)) { o << ",\"height_name\":"; jsonEscape(o, *nm); }
      }
      o << "}";
    }
    o << "],\"binaries\":" << m.shader_binaries.size() << ",\"dispatches\":[";
    // SHA-256 of each code object: what ties a profile or a measurement to the exact kernel a dispatch runs
    std::vector<std::string> codeSha(m.shader_binaries.size());
    for (size_t i = 0; i < m.shader_binaries.size(); ++i) {
      Sha256 h;
      h.update(m.shader_binaries[i].code_object.data(), m.shader_binaries[i].code_object.size());
      codeSha[i] = Sha256::hex(h.digest());
    }
    for (size_t i = 0; i < m.dispatches.size(); ++i) {
      const auto &d = m.dispatches[i];
      o << (i ? "," : "") << "{\"name\":"; jsonEscape(o, d.info.name);
      o << ",\"entry_point\":"; jsonEscape(o, d.entry_point);
      o << ",\"src_path\":"; jsonEscape(o, d.info.src_path);
      o << ",\"debug_info\":"; jsonEscape(o, d.info.debug_info);
      o << ",\"code_sha256\":"; jsonEscape(o, d.binary_id < codeSha.size() ? codeSha[d.binary_id] : std::string());
      o << ",\"binary_id\":" << d.binary_id << ",\"workgroup_count\":[" << d.workgroup_count_x.eval(dp) << ',' << d.workgroup_count_y.eval(dp) << ',' << d.workgroup_count_z.eval(dp)
        << "],\"workgroup_size\":[" << d.workgroup_size[0] << ',' << d.workgroup_size[1] << ',' << d.workgroup_size[2] << "],\"bindings\":[";
      bool first = true;
      for (const auto &sb : d.bindings)
        for (const auto &b : sb.bindings) { o << (first ? "" : ",") << "{\"set\":" << sb.set << ",\"binding\":" << b.binding << ",\"access\":" << static_cast<int>(b.access) << ",\"tensor\":" << b.tensor << "}"; first = false; }
      o << "],\"push_constants\":[";
      for (size_t f = 0; f < d.push_constant.fields.size(); ++f) o << (f ? "," : "") << d.push_constant.fields[f].source.eval(dp);
      o << "],\"memory_reads\":" << (d.info.has_reads ? d.info.memory_reads.eval(dp) : 0) << ",\"memory_writes\":" << (d.info.has_writes ? d.info.memory_writes.eval(dp) : 0)
        << ",\"flops\":" << (d.info.has_flops ? d.info.flops.eval(dp) : 0) << "}";
    }
    o << "]}";
    const std::string s = o.str();
    char *p = static_cast<char *>(std::malloc(s.size() + 1));
    if (!p) fail(Status::Internal, "out of host memory");
    std::memcpy(p, s.c_str(), s.size() + 1);
    *out_json = p;
  });
}
void denox_hip_free(void *p) { std::free(p); }

// ---------------------------------------------------------------- database
int denox_hip_db_open(const char *path, denox_hip_db **out) {
  return guarded([&] { need(path, "path"); need(out, "out"); auto *d = new denox_hip_db(); try { d->db = Db::open(path); } catch (...) { delete d; throw; } *out = d; });
}
void denox_hip_db_close(denox_hip_db *db) { delete db; }
int denox_hip_db_row_count(const denox_hip_db *db, uint64_t *out) {
  return guarded([&] { need(db, "db"); need(out, "out"); *out = db->db.rows().size(); });
}
int denox_hip_db_populate(denox_hip_db *db, const denox_hip_builder *b, const denox_hip_compile_options *o, uint64_t *out_added) {
  return guarded([&] {
    need(db, "db"); need(b, "builder");
    const hip::HipCompiler hipc = makeCompiler();
    const size_t n = compiler::populate(db->db, b->model, hipc, toOptions(o), !o || o->populate_compile_kernels != 0, o ? o->kernel_shard_index : 0, o ? o->kernel_shard_count : 1);
    if (out_added) *out_added = n;
  });
}
void denox_hip_db_bench_options_default(denox_hip_db_bench_options *o) {
  if (!o) return;
  o->min_samples = 10; o->max_relative_error = 0.05; o->max_samples = 200; o->save_progress = 1; o->filter = nullptr;
}
int denox_hip_db_bench(denox_hip_db *db, denox_hip_context *ctx, const denox_hip_db_bench_options *o, denox_hip_db_bench_result *out) {
  return guarded([&] {
    need(db, "db"); need(ctx, "context");
    runtime::DbBenchOptions opt;
    if (o) {
      opt.minSamples = o->min_samples; opt.maxRelativeError = o->max_relative_error; opt.maxSamples = o->max_samples;
      opt.saveProgress = o->save_progress != 0;
      if (o->filter) opt.filter = o->filter;
    }
    const hip::HipCompiler hipc = makeCompiler();
    const runtime::DbBenchResult r = runtime::db_bench(db->db, ctx->ctx, hipc, opt);
    if (out) { out->benchmarked = r.benchmarked; out->converged = r.converged; out->skipped = r.skipped; out->failed = r.failed; }
  });
}
int denox_hip_db_add_sample(denox_hip_db *db, uint64_t row, double latency_ns) {
  return guarded([&] { need(db, "db"); db->db.add_dispatch_benchmark_result(row, latency_ns); });
}
int denox_hip_db_row_stats(const denox_hip_db *db, uint64_t row, uint64_t *samples, double *mean_ns, double *std_ns) {
  return guarded([&] {
    need(db, "db");
    if (row >= db->db.rows().size()) fail(Status::InvalidArgument, "row out of range");
    const DbDispatch &d = db->db.rows()[row];
    if (samples) *samples = d.samples;
    if (mean_ns) *mean_ns = d.meanNs;
    if (std_ns) *std_ns = d.stdNs();
  });
}
int denox_hip_db_writeback(const denox_hip_db *db) {
  return guarded([&] { need(db, "db"); db->db.atomic_writeback(); });
}
int denox_hip_db_dump_csv(const denox_hip_db *db, char **out_csv) {
  return guarded([&] {
    need(db, "db"); need(out_csv, "out_csv");
    const std::string s = db->db.to_csv();
    char *p = static_cast<char *>(std::malloc(s.size() + 1));
    if (!p) fail(Status::Internal, "out of host memory");
    std::memcpy(p, s.c_str(), s.size() + 1);
    *out_csv = p;
  });
}

// ---------------------------------------------------------------- runtime
int denox_hip_context_create(int device, denox_hip_context **out) {
  return guarded([&] { need(out, "out"); auto c = std::make_shared<runtime::Context>(device); *out = new denox_hip_context{std::move(c)}; });
}
void denox_hip_context_destroy(denox_hip_context *ctx) { delete ctx; }
int denox_hip_context_stream(const denox_hip_context *ctx, void **out_stream) {
  return guarded([&] { need(ctx, "context"); need(out_stream, "out_stream"); *out_stream = ctx->ctx->stream(); });
}

int denox_hip_model_create(denox_hip_context *ctx, const void *dnxbuf, size_t size, denox_hip_model **out) {
  return guarded([&] { need(ctx, "context"); need(dnxbuf, "dnx"); need(out, "out"); auto m = std::make_shared<runtime::Model>(ctx->ctx, dnxbuf, size); *out = new denox_hip_model{std::move(m)}; });
}
void denox_hip_model_destroy(denox_hip_model *m) { delete m; }
int denox_hip_model_dispatch_count(const denox_hip_model *m, uint32_t *out) {
  return guarded([&] { need(m, "model"); need(out, "out"); *out = static_cast<uint32_t>(m->model->dispatches().size()); });
}

int denox_hip_instance_create(denox_hip_model *m, const char *const *names, const int64_t *values, uint32_t n, denox_hip_instance **out) {
  return guarded([&] {
    need(m, "model"); need(out, "out");
    std::vector<runtime::ValueSpec> specs;
    for (uint32_t i = 0; i < n; ++i) { need(names, "names"); need(values, "values"); need(names[i], "name"); specs.push_back(runtime::ValueSpec{names[i], values[i]}); }
    auto inst = std::make_unique<runtime::Instance>(m->model, specs);
    *out = new denox_hip_instance{std::move(inst)};
  });
}
void denox_hip_instance_destroy(denox_hip_instance *inst) { delete inst; }
int denox_hip_instance_input_count(const denox_hip_instance *inst, uint32_t *out) {
  return guarded([&] { need(inst, "instance"); need(out, "out"); *out = static_cast<uint32_t>(inst->inst->inputCount()); });
}
int denox_hip_instance_output_count(const denox_hip_instance *inst, uint32_t *out) {
  return guarded([&] { need(inst, "instance"); need(out, "out"); *out = static_cast<uint32_t>(inst->inst->outputCount()); });
}
static void fillDesc(const runtime::TensorDesc &d, denox_hip_tensor_desc *out) {
  std::memset(out, 0, sizeof(*out));
  out->width = d.width; out->height = d.height; out->channels = d.channels;
  out->format = static_cast<int32_t>(d.format); out->dtype = static_cast<int32_t>(d.dtype); out->byte_size = d.byteSize;
  copyStr(out->name, sizeof(out->name), d.name);
}
int denox_hip_instance_input_desc(const denox_hip_instance *inst, uint32_t i, denox_hip_tensor_desc *out) {
  return guarded([&] { need(inst, "instance"); need(out, "out"); if (i >= inst->inst->inputCount()) fail(Status::InvalidArgument, "input index out of range"); fillDesc(inst->inst->inputDesc(i), out); });
}
int denox_hip_instance_output_desc(const denox_hip_instance *inst, uint32_t i, denox_hip_tensor_desc *out) {
  return guarded([&] { need(inst, "instance"); need(out, "out"); if (i >= inst->inst->outputCount()) fail(Status::InvalidArgument, "output index out of range"); fillDesc(inst->inst->outputDesc(i), out); });
}
int denox_hip_instance_infer(denox_hip_instance *inst, const void *const *in, void *const *out) {
  return guarded([&] { need(inst, "instance"); inst->inst->infer(in, out); });
}
int denox_hip_instance_infer_many(denox_hip_instance *inst, uint32_t frames, const void *const *in, void *const *out) {
  return guarded([&] { need(inst, "instance"); inst->inst->inferMany(frames, in, out); });
}
int denox_hip_host_alloc(size_t bytes, void **out) {
  return guarded([&] {
    need(out, "out");
    void *p = nullptr;
    runtime::hipCheck(hipHostMalloc(&p, bytes ? bytes : 1, hipHostMallocDefault), "hipHostMalloc");
    *out = p;
  });
}
void denox_hip_host_free(void *p) { if (p) (void)hipHostFree(p); }
int denox_hip_instance_infer_device(denox_hip_instance *inst, const void *const *in, void *const *out) {
  return guarded([&] { need(inst, "instance"); inst->inst->inferDevice(in, out); });
}
static_assert(DENOX_HIP_STATIC_SCRATCH_BYTES == runtime::kStaticScratchBytes, "header and library disagree on the static scratch size");
int denox_hip_instance_infer_device_static(denox_hip_instance *inst, const void *const *in, void *const *out) {
  return guarded([&] { need(inst, "instance"); inst->inst->inferDeviceStatic(in, out); });
}
int denox_hip_instance_synchronize(denox_hip_instance *inst) {
  return guarded([&] { need(inst, "instance"); inst->inst->synchronize(); });
}
int denox_hip_instance_input_device_ptr(const denox_hip_instance *inst, uint32_t i, void **out) {
  return guarded([&] { need(inst, "instance"); need(out, "out"); if (i >= inst->inst->inputCount()) fail(Status::InvalidArgument, "input index out of range"); *out = inst->inst->inputDevicePtr(i); });
}
int denox_hip_instance_output_device_ptr(const denox_hip_instance *inst, uint32_t i, void **out) {
  return guarded([&] { need(inst, "instance"); need(out, "out"); if (i >= inst->inst->outputCount()) fail(Status::InvalidArgument, "output index out of range"); *out = inst->inst->outputDevicePtr(i); });
}
int denox_hip_instance_bench(denox_hip_instance *inst, uint32_t warmup, denox_hip_timing *out, uint32_t capacity, uint32_t *out_count) {
  return guarded([&] {
    need(inst, "instance");
    const auto t = inst->inst->bench(static_cast<int>(warmup));
    if (out_count) *out_count = static_cast<uint32_t>(t.size());
    for (size_t i = 0; i < t.size() && i < capacity; ++i) {
      need(out, "out");
      std::memset(&out[i], 0, sizeof(out[i]));
      copyStr(out[i].name, sizeof(out[i].name), t[i].name);
      copyStr(out[i].input, sizeof(out[i].input), t[i].input);
      copyStr(out[i].output, sizeof(out[i].output), t[i].output);
      out[i].memory_reads = t[i].memoryReads; out[i].memory_writes = t[i].memoryWrites; out[i].flops = t[i].flops; out[i].latency_ms = t[i].latencyMs;
    }
  });
}
int denox_hip_instance_bench_in_frame(denox_hip_instance *inst, uint32_t dispatch, uint32_t frames, uint32_t warmup, float *out_ms) {
  return guarded([&] {
    need(inst, "instance"); need(out_ms, "out_ms");
    *out_ms = inst->inst->benchInFrame(dispatch, static_cast<int>(frames), static_cast<int>(warmup));
  });
}
int denox_hip_instance_device_bytes(const denox_hip_instance *inst, uint64_t *out) {
  return guarded([&] { need(inst, "instance"); need(out, "out"); *out = inst->inst->deviceBytes(); });
}

} // extern "C"
