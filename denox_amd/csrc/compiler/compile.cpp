#include "compile.hpp"
#include <algorithm>
#include <cstring>
#include <atomic>
#include <map>
#include <set>
#include <mutex>
#include <thread>

namespace denox::compiler {

std::vector<int64_t> assumed_symeval(const Model &model, const SymGraph &sym, const CompileOptions &opt) {
  std::vector<int64_t> vars;
  for (const std::string &n : sym.varNames()) {
    int64_t v = opt.defaultAssumedExtent;
    auto it = opt.assumptions.find(n);
    if (it != opt.assumptions.end()) v = it->second;
    else
      for (const auto &nv : model.valueNames()) // a variable may be known under several names
        if (nv.value.symbolic && sym.varNames().size() > static_cast<size_t>(nv.value.v) && sym.varNames()[nv.value.v] == n) {
          auto jt = opt.assumptions.find(nv.name);
          if (jt != opt.assumptions.end()) v = jt->second;
        }
    vars.push_back(v);
  }
  return sym.eval(vars);
}

std::vector<uint8_t> push_constant_bytes(const ComputeDispatch &d, const std::vector<int64_t> &dp, std::vector<uint16_t> *offsets) {
  // fields laid out in registration order at their natural alignment (serialize.cpp:379-398 of the reference)
  std::vector<uint8_t> bytes;
  if (offsets) offsets->clear();
  for (const auto &pc : d.pushConstants) {
    const size_t sz = dnx::scalarSize(pc.dtype);
    while (bytes.size() % sz) bytes.push_back(0);
    if (offsets) offsets->push_back(static_cast<uint16_t>(bytes.size()));
    const int64_t v = symValue(dp, pc.value);
    uint8_t tmp[8];
    std::memcpy(tmp, &v, 8); // little endian: the low bytes are the narrower value
    bytes.insert(bytes.end(), tmp, tmp + sz);
  }
  return bytes;
}

static double estimate_dispatch_ms(const ComputeDispatch &d, const std::vector<int64_t> &dp, const CompileOptions &opt) {
  const double bytes = (d.info.hasReads ? static_cast<double>(symValue(dp, d.info.memoryReads)) : 0.0) +
                       (d.info.hasWrites ? static_cast<double>(symValue(dp, d.info.memoryWrites)) : 0.0);
  const double flops = d.info.hasFlops ? static_cast<double>(symValue(dp, d.info.flops)) : 0.0;
  // conservative fractions of the published peaks plus a fixed launch cost
  const double tMem = bytes / (0.5 * opt.deviceInfo.hbmBytesPerSecond);
  const double tMath = flops / (0.3 * opt.deviceInfo.fp16MfmaFlops);
  return (std::max(tMem, tMath) + 3e-6) * 1e3;
}

// CompileOptions::layoutPreference: a positive value halves the cost of every candidate that touches a CHWC8 tensor
static double prefer(const SuperGraphEdge &e, const CompileOptions &opt, double cost) {
  if (opt.layoutPreference <= 0) return cost;
  const bool blocked = e.outputFormat != 0 || std::any_of(e.inputFormats.begin(), e.inputFormats.end(), [](int f) { return f != 0; });
  return blocked ? 0.5 * cost : cost;
}

double edge_cost_ms(const SuperGraphEdge &e, const std::vector<int64_t> &dp, const Db *db, const CompileOptions &opt, bool *measured) {
  double total = 0.0;
  bool all = db != nullptr;
  if (db) {
    for (const auto &d : e.dispatches) {
      const uint32_t wg[3] = {static_cast<uint32_t>(symValue(dp, d.workgroupCountX)), static_cast<uint32_t>(symValue(dp, d.workgroupCountY)),
                              static_cast<uint32_t>(symValue(dp, d.workgroupCountZ))};
      auto lat = db->query_dispatch_latency(d.kernel.sha256(), push_constant_bytes(d, dp), wg);
      if (!lat) { all = false; break; }
      total += *lat;
    }
  }
  if (measured) *measured = all;
  if (all) return prefer(e, opt, total);
  total = 0.0;
  for (const auto &d : e.dispatches) total += estimate_dispatch_ms(d, dp, opt);
  // estimates cannot tell configurations apart; the shader's prior breaks ties
  return prefer(e, opt, total / std::max(1e-3f, e.speedup));
}

namespace {
struct Selector {
  const std::vector<bool> &isInput;
  const std::vector<HyperEdge> &edges;
  const std::vector<double> &cost;
  std::vector<std::vector<size_t>> producers;
  std::map<std::vector<int>, std::pair<double, long>> memo; // needed set -> (cost, edge chosen for its largest member)

  std::vector<int> after(const std::vector<int> &needed, size_t e) const {
    std::vector<int> sub(needed.begin(), needed.end() - 1);
    for (int in : edges[e].inputs)
      if (!isInput[static_cast<size_t>(in)]) sub.push_back(in);
    std::sort(sub.begin(), sub.end());
    sub.erase(std::unique(sub.begin(), sub.end()), sub.end());
    return sub;
  }

  double solve(const std::vector<int> &needed) {
    if (needed.empty()) return 0.0;
    auto it = memo.find(needed);
    if (it != memo.end()) return it->second.first;
    // the largest node id: node ids are topologically ordered, so no other node
    // still needed can require it to be produced later
    const int t = needed.back();
    double best = kInfiniteCost;
    long bestEdge = -1;
    for (size_t e : producers[static_cast<size_t>(t)]) {
      const double c = cost[e] + solve(after(needed, e));
      if (c < best) { best = c; bestEdge = static_cast<long>(e); }
    }
    memo[needed] = {best, bestEdge};
    return best;
  }
};
} // namespace

std::vector<size_t> minimum_cost_subgraph(const std::vector<bool> &isInput, const std::vector<HyperEdge> &edges, const std::vector<double> &edgeCost,
                                          const std::vector<int> &outputs, double *totalCost) {
  if (edges.size() != edgeCost.size()) fail(Status::InvalidArgument, "one cost per edge expected");
  Selector s{isInput, edges, edgeCost, {}, {}};
  s.producers.resize(isInput.size());
  for (size_t e = 0; e < edges.size(); ++e) {
    const auto &edge = edges[e];
    if (edge.output < 0 || static_cast<size_t>(edge.output) >= isInput.size()) fail(Status::InvalidArgument, "edge output out of range");
    for (int in : edge.inputs)
      if (in < 0 || in >= edge.output) fail(Status::InvalidArgument, "hyper-graph nodes must be numbered in topological order");
    s.producers[static_cast<size_t>(edge.output)].push_back(e);
  }
  std::vector<int> needed;
  for (int o : outputs) {
    if (o < 0 || static_cast<size_t>(o) >= isInput.size()) fail(Status::InvalidArgument, "output out of range");
    if (!isInput[static_cast<size_t>(o)]) needed.push_back(o);
  }
  std::sort(needed.begin(), needed.end());
  needed.erase(std::unique(needed.begin(), needed.end()), needed.end());
  const double total = s.solve(needed);
  if (totalCost) *totalCost = total;
  std::vector<size_t> chosen;
  if (total >= kInfiniteCost) return chosen;
  std::vector<int> cur = needed;
  while (!cur.empty()) {
    const size_t e = static_cast<size_t>(s.memo.at(cur).second);
    chosen.push_back(e);
    cur = s.after(cur, e);
  }
  // producers come before consumers when sorted by output node
  std::sort(chosen.begin(), chosen.end(), [&](size_t a, size_t b) { return edges[a].output < edges[b].output; });
  return chosen;
}

std::vector<size_t> select_schedule(const Model &model, const SuperGraph &g, const std::vector<double> &edgeCost) {
  // Tensor t has four nodes, 4 t + 2 f + v: layout f (0 HWC, 1 CHWC8; SuperGraphEdge::outputFormat) and v = 1 for the tensor
  // as a channel range of its concat's output (SuperGraphEdge::outputVariant, HWC only).  Tensor handles are topologically
  // ordered, and so are these.  Model inputs and outputs are HWC tensors of their own.
  std::vector<bool> isInput(4 * model.tensors().size(), false);
  for (size_t i = 0; i < model.tensors().size(); ++i) isInput[4 * i] = model.tensors()[i].isInput;
  std::vector<HyperEdge> edges;
  for (const auto &e : g.edges) {
    HyperEdge h;
    for (size_t i = 0; i < e.inputs.size(); ++i)
      h.inputs.push_back(4 * e.inputs[i] + 2 * (e.inputFormats.empty() ? 0 : e.inputFormats[i]) + (e.inputVariants.empty() ? 0 : e.inputVariants[i]));
    h.output = 4 * e.output + 2 * e.outputFormat + e.outputVariant;
    edges.push_back(std::move(h));
  }
  std::vector<int> outputs;
  for (TensorHandle o : model.outputs()) outputs.push_back(4 * o);
  double total = 0.0;
  std::vector<size_t> chosen = minimum_cost_subgraph(isInput, edges, edgeCost, outputs, &total);
  if (total >= kInfiniteCost) fail(Status::Unsupported, "no kernel implements part of this graph (a layer has no matching shader)");
  return chosen;
}

static dnx::ScalarSource src(Sym s, dnx::ScalarType t = dnx::ScalarType::I64) { return dnx::ScalarSource::fromSym(s, t); }

std::vector<uint8_t> compile(const Model &modelIn, const hip::HipCompiler &hipc, const Db *db, const CompileOptions &opt, CompileReport *report) {
  if (modelIn.outputs().empty()) fail(Status::InvalidArgument, "model has no outputs");
  Model model = modelIn; // the symbol graph grows while dispatches are built
  SymGraph &sym = model.symGraph();
  const auto shaders = get_all_shaders(&hipc);
  SuperGraph g = implement(model, sym, shaders, opt);
  const std::vector<int64_t> dp = assumed_symeval(model, sym, opt);
  std::vector<double> cost(g.edges.size());
  std::vector<bool> measured(g.edges.size());
  for (size_t e = 0; e < g.edges.size(); ++e) {
    bool m = false;
    cost[e] = edge_cost_ms(g.edges[e], dp, db, opt, &m);
    measured[e] = m;
  }
  const std::vector<size_t> chosen = select_schedule(model, g, cost);

  dnx::Model out;
  out.version = 0;
  out.info.producer = "denox-hip";
  out.info.producer_version = "0.1";

  // ---- placement: one buffer per live tensor (placement.cpp:232-300 of the reference) ----
  std::map<uint32_t, uint32_t> tensorIndex; // super-graph tensor -> dnx tensor
  auto place = [&](uint32_t st) -> uint32_t {
    auto it = tensorIndex.find(st);
    if (it != tensorIndex.end()) return it->second;
    const SuperTensor &t = g.tensors[st];
    dnx::Buffer b;
    b.size = src(t.byteSize);
    b.alignment = t.alignment;
    out.buffers.push_back(b);
    dnx::Tensor dt;
    dt.buffer = static_cast<uint32_t>(out.buffers.size() - 1);
    dt.offset = src(Sym::Const(0));
    dt.size = src(t.byteSize);
    dt.info.format = t.format;
    dt.info.type = t.type;
    dt.info.name = t.name;
    if (t.modelTensor >= 0) {
      const TensorNode &n = model.tensors()[t.modelTensor];
      dt.info.has_extent = true;
      dt.info.width = src(n.width);
      dt.info.height = src(n.height);
      dt.info.channels = src(Sym::Const(n.channels));
    }
    out.tensors.push_back(std::move(dt));
    const uint32_t id = static_cast<uint32_t>(out.tensors.size() - 1);
    tensorIndex.emplace(st, id);
    return id;
  };

  // ---- kernels: distinct variants by hash (compile_shaders.cpp:35-48 of the reference) ----
  std::map<std::string, uint32_t> binaryIndex;
  auto binaryOf = [&](const hip::HipCompilerInstance &k) -> uint32_t {
    const std::string key = k.sha256();
    auto it = binaryIndex.find(key);
    if (it != binaryIndex.end()) return it->second;
    dnx::ShaderBinary sb;
    sb.code_object = k.compile();
    out.shader_binaries.push_back(std::move(sb));
    const uint32_t id = static_cast<uint32_t>(out.shader_binaries.size() - 1);
    binaryIndex.emplace(key, id);
    return id;
  };

  auto emitDispatch = [&](const ComputeDispatch &d) {
    dnx::ComputeDispatch o;
    o.binary_id = binaryOf(d.kernel);
    o.entry_point = d.entryPoint;
    o.workgroup_count_x = src(d.workgroupCountX);
    o.workgroup_count_y = src(d.workgroupCountY);
    o.workgroup_count_z = src(d.workgroupCountZ);
    for (int i = 0; i < 3; ++i) o.workgroup_size[i] = d.workgroupSize[i];
    dnx::DescriptorSetBinding set;
    set.set = 0;
    for (const auto &b : d.bindings) set.bindings.push_back(dnx::DescriptorBinding{b.binding, b.access, place(b.tensor.index)});
    o.bindings.push_back(std::move(set));
    uint16_t off = 0;
    for (const auto &pc : d.pushConstants) {
      const uint16_t sz = static_cast<uint16_t>(dnx::scalarSize(pc.dtype));
      off = static_cast<uint16_t>((off + sz - 1) / sz * sz);
      o.push_constant.fields.push_back(dnx::PushConstantField{pc.dtype, off, src(pc.value, pc.dtype)});
      off = static_cast<uint16_t>(off + sz);
    }
    o.push_constant.size = off;
    o.info.name = d.info.name;
    o.info.debug_info = d.info.config.empty() ? d.kernel.defineString() : d.info.config + " | " + d.kernel.defineString();
    o.info.src_path = d.info.srcPath;
    o.info.has_reads = d.info.hasReads; o.info.memory_reads = src(d.info.memoryReads);
    o.info.has_writes = d.info.hasWrites; o.info.memory_writes = src(d.info.memoryWrites);
    o.info.has_flops = d.info.hasFlops; o.info.flops = src(d.info.flops);
    out.dispatches.push_back(std::move(o));
  };

  // ---- interface tensors and layout conversion ----
  auto formatOf = [](const std::vector<InterfaceTensorDescriptor> &descs, const std::string &name, size_t index) {
    for (const auto &d : descs) if (d.name == name) return d.format;
    if (index < descs.size() && descs[index].name.empty()) return descs[index].format;
    return dnx::TensorFormat::SSBO_HWC;
  };
  auto layoutId = [](dnx::TensorFormat f) -> int {
    switch (f) {
    case dnx::TensorFormat::SSBO_HWC: return 0;
    case dnx::TensorFormat::SSBO_CHW: return 1;
    case dnx::TensorFormat::SSBO_CHWC8: return 2;
    default: fail(Status::Unsupported, "interface tensors must be SSBO_HWC, SSBO_CHW or SSBO_CHWC8");
    }
  };
  auto relayout = [&](TensorHandle t, dnx::TensorFormat from, dnx::TensorFormat to, bool external_is_source) -> uint32_t {
    // creates the externally visible tensor in its declared format plus the conversion dispatch
    const TensorNode &n = model.tensors()[t];
    if ((from == dnx::TensorFormat::SSBO_CHWC8 || to == dnx::TensorFormat::SSBO_CHWC8) && n.channels % 8) fail(Status::InvalidArgument, "CHWC8 needs a channel count divisible by 8");
    SuperTensor ext = g.tensors[t];
    ext.format = external_is_source ? from : to;
    ext.name = n.name;
    g.tensors.push_back(ext);
    const uint32_t extId = static_cast<uint32_t>(g.tensors.size() - 1);
    ComputeDispatch d;
    d.kernel = hipc.read("relayout.hip");
    d.kernel.define("CH", n.channels); d.kernel.define("SRC_LAYOUT", layoutId(from)); d.kernel.define("DST_LAYOUT", layoutId(to));
    d.entryPoint = "relayout_c" + std::to_string(n.channels) + "_" + std::to_string(layoutId(from)) + "to" + std::to_string(layoutId(to));
    d.kernel.define("KERNEL_NAME", d.entryPoint);
    // HWC <-> CHWC8 moves one 16-byte vector per thread, every other pair one pixel per thread (see relayout.hip)
    const bool blocky = from != dnx::TensorFormat::SSBO_CHW && to != dnx::TensorFormat::SSBO_CHW && n.channels % 8 == 0;
    d.workgroupCountX = sym.cdiv(sym.mul(sym.mul(n.width, n.height), blocky ? static_cast<int64_t>(n.channels / 8) : 1), 256);
    d.workgroupCountY = d.workgroupCountZ = Sym::Const(1);
    d.workgroupSize[0] = 256;
    TensorBinding in{0, 0, dnx::Access::ReadOnly, TensorId{external_is_source ? extId : static_cast<uint32_t>(t)}, BindingType::Input, false, Sym::Const(0)};
    TensorBinding ob{0, 1, dnx::Access::WriteOnly, TensorId{external_is_source ? static_cast<uint32_t>(t) : extId}, BindingType::Output, false, Sym::Const(0)};
    d.bindings = {in, ob};
    d.pushConstants = {PushConstantDesc{n.width, dnx::ScalarType::U32}, PushConstantDesc{n.height, dnx::ScalarType::U32}};
    d.info.name = "relayout"; d.info.operation = "relayout"; d.info.srcPath = "relayout.hip";
    d.info.hasReads = d.info.hasWrites = d.info.hasFlops = true;
    d.info.memoryReads = d.info.memoryWrites = g.tensors[t].byteSize;
    d.info.flops = Sym::Const(0);
    emitDispatch(d);
    return place(extId);
  };

  for (size_t i = 0; i < model.inputs().size(); ++i) {
    const TensorHandle t = model.inputs()[i];
    const dnx::TensorFormat f = formatOf(opt.inputDescriptors, model.tensors()[t].name, i);
    if (f == dnx::TensorFormat::SSBO_HWC) out.inputs.push_back(place(static_cast<uint32_t>(t)));
    else out.inputs.push_back(relayout(t, f, dnx::TensorFormat::SSBO_HWC, true));
  }

  // A tensor that lives inside another one (concat without a copy).  The tensor it lives in may itself be the source of a
  // later concat, so buffers and offsets are resolved once every selected edge has been seen, by following each chain to
  // the tensor that owns its memory (the reference unions the tensors with offsets, placement.cpp:232-255).
  struct Alias { uint32_t parent; Sym offset; };
  std::map<uint32_t, Alias> aliasOf;

  double total = 0.0;
  unsigned walk = 0; // alternates the tile walk of consecutive tiled dispatches
  for (size_t e : chosen) {
    SuperGraphEdge &edge = g.edges[e];
    if (opt.features.enableAlternatingTraversal)
      for (auto &d : edge.dispatches)
        if (d.traversalFlagIndex >= 0) d.pushConstants[static_cast<size_t>(d.traversalFlagIndex)].value = Sym::Const(walk++ & 1u);
    for (const auto &p : edge.parameters) {
      const uint32_t id = place(p.tensor.index);
      dnx::TensorInitializer init;
      init.tensor = id;
      init.data = p.lazyValue();
      if (init.data.size() != static_cast<size_t>(g.tensors[p.tensor.index].byteSize.v)) fail(Status::Internal, "parameter blob size mismatch");
      out.initializers.push_back(std::move(init));
    }
    for (const auto &d : edge.dispatches) emitDispatch(d);
    // implicit concat: src0 at offset 0, src1 behind it, dst aliases both (placement.cpp:253-255 of the reference)
    for (const auto &mc : edge.memoryConstrains) {
      const uint32_t a = place(mc.src0.index), b = place(mc.src1.index), dd = place(mc.dst.index);
      aliasOf[a] = Alias{dd, Sym::Const(0)};
      aliasOf[b] = Alias{dd, g.tensors[mc.src0.index].byteSize};
    }
    // pixel-major concat without a copy: the source is a channel range of the destination, from its first channel
    // to the end of the destination
    for (const auto &vc : edge.viewConstrains) {
      const uint32_t a = place(vc.src.index), dd = place(vc.dst.index);
      aliasOf[a] = Alias{dd, Sym::Const(static_cast<int64_t>(vc.byteOffset))};
      out.tensors[a].size = src(sym.sub(g.tensors[vc.dst.index].byteSize, static_cast<int64_t>(vc.byteOffset)));
    }
    total += cost[e];
    if (report) {
      report->schedule.push_back(ScheduleEntry{edge.shader, edge.config, edge.dispatches.empty() ? "" : edge.dispatches[0].info.name, cost[e], measured[e]});
      if (db && !measured[e]) report->warnings.push_back("no measured latency for " + edge.shader + " " + edge.config + "; used the roofline estimate");
    }
  }

  for (const auto &kv : aliasOf) {
    uint32_t root = kv.second.parent;
    Sym off = kv.second.offset;
    size_t hops = 0;
    for (auto it = aliasOf.find(root); it != aliasOf.end(); it = aliasOf.find(root)) {
      if (++hops > aliasOf.size()) fail(Status::Internal, "tensors placed inside each other form a cycle");
      off = sym.add(off, it->second.offset);
      root = it->second.parent;
    }
    out.tensors[kv.first].buffer = out.tensors[root].buffer;
    out.tensors[kv.first].offset = src(off);
  }

  for (size_t i = 0; i < model.outputs().size(); ++i) {
    const TensorHandle t = model.outputs()[i];
    const dnx::TensorFormat f = formatOf(opt.outputDescriptors, model.tensors()[t].name, i);
    if (f == dnx::TensorFormat::SSBO_HWC) out.outputs.push_back(place(static_cast<uint32_t>(t)));
    else out.outputs.push_back(relayout(t, dnx::TensorFormat::SSBO_HWC, f, false));
  }

  { // buffers whose tensor moved into another buffer are dropped
    std::vector<int> newIndex(out.buffers.size(), -1);
    std::vector<dnx::Buffer> kept;
    for (auto &t : out.tensors) {
      if (newIndex[t.buffer] < 0) { newIndex[t.buffer] = static_cast<int>(kept.size()); kept.push_back(out.buffers[t.buffer]); }
      t.buffer = static_cast<uint32_t>(newIndex[t.buffer]);
    }
    out.buffers = std::move(kept);
  }

  out.sym_ir = sym.compile();
  for (const auto &nv : model.valueNames()) out.value_names.push_back(dnx::ValueName{nv.name, src(nv.value)});
  for (const auto &q : model.requirements()) out.requirements.push_back(dnx::Requirement{src(q.lhs), src(q.rhs), static_cast<uint8_t>(q.relation), q.what});
  out.required_features = {1u}; // HipCodeObject: the binaries are gfx950 code objects, not SPIR-V
  dnx::validate(out);
  dnx::requireExecutable(out);
  if (report) {
    report->superGraphEdges = g.edges.size();
    report->selectedEdges = chosen.size();
    report->dispatches = out.dispatches.size();
    report->estimatedMs = total;
    report->kernelsCompiled = hipc.stats().compiled;
    report->kernelCacheHits = hipc.stats().cacheHits;
  }
  return dnx::serialize(out);
}

size_t populate(Db &db, const Model &modelIn, const hip::HipCompiler &hipc, const CompileOptions &opt, bool compileKernels, unsigned shardIndex, unsigned shardCount) {
  Model model = modelIn;
  SymGraph &sym = model.symGraph();
  const auto shaders = get_all_shaders(&hipc);
  const SuperGraph g = implement(model, sym, shaders, opt);
  const std::vector<int64_t> dp = assumed_symeval(model, sym, opt);
  size_t added = 0;
  for (const auto &edge : g.edges)
    for (const auto &d : edge.dispatches) {
      DbDispatch row;
      row.sha256 = d.kernel.sha256();
      row.pushConstants = push_constant_bytes(d, dp);
      row.wg[0] = static_cast<uint32_t>(symValue(dp, d.workgroupCountX));
      row.wg[1] = static_cast<uint32_t>(symValue(dp, d.workgroupCountY));
      row.wg[2] = static_cast<uint32_t>(symValue(dp, d.workgroupCountZ));
      row.srcPath = d.kernel.sourcePath();
      row.defines = d.kernel.defineString();
      row.entryPoint = d.entryPoint;
      for (int i = 0; i < 3; ++i) row.block[i] = d.workgroupSize[i];
      for (const auto &b : d.bindings) {
        const SuperTensor &t = g.tensors[b.tensor.index];
        row.bindings.push_back(DbBinding{static_cast<uint64_t>(symValue(dp, b.hasSpan ? b.span : t.byteSize)), t.alignment, t.isParam, static_cast<uint8_t>(b.access)});
      }
      row.operation = d.info.operation; row.shader = edge.shader; row.config = d.info.config;
      row.memoryReads = d.info.hasReads ? static_cast<uint64_t>(symValue(dp, d.info.memoryReads)) : 0;
      row.memoryWrites = d.info.hasWrites ? static_cast<uint64_t>(symValue(dp, d.info.memoryWrites)) : 0;
      row.flops = d.info.hasFlops ? static_cast<uint64_t>(symValue(dp, d.info.flops)) : 0;
      const size_t before = db.rows().size();
      db.insert_dispatch(row);
      if (db.rows().size() > before) ++added;
    }
  if (compileKernels) {
    // every distinct kernel variant, on all host threads (populate.cpp:70-99 of the reference);
    // the code objects land in the compiler's cache, where compile() and the benchmark find them
    std::map<std::string, const hip::HipCompilerInstance *> distinct;
    for (const auto &edge : g.edges)
      for (const auto &d : edge.dispatches) distinct.emplace(d.kernel.sha256(), &d.kernel);
    std::vector<const hip::HipCompilerInstance *> work;
    {
      // several processes can split the work: hiprtc serialises compilations inside one process
      size_t idx = 0;
      for (const auto &kv : distinct)
        if (shardCount <= 1 || idx++ % shardCount == shardIndex) work.push_back(kv.second);
    }
    std::atomic<size_t> next{0};
    std::mutex errMutex;
    std::string firstError;
    const unsigned nthreads = std::max(1u, std::min<unsigned>(std::thread::hardware_concurrency(), 16u));
    std::vector<std::thread> pool;
    for (unsigned t = 0; t < nthreads; ++t)
      pool.emplace_back([&] {
        for (size_t i = next++; i < work.size(); i = next++) {
          try {
            (void)work[i]->compile();
          } catch (const std::exception &e) {
            std::lock_guard<std::mutex> lock(errMutex);
            if (firstError.empty()) firstError = e.what();
          }
        }
      });
    for (auto &th : pool) th.join();
    if (!firstError.empty()) fail(Status::CompileError, firstError);
  }
  return added;
}

} // namespace denox::compiler
