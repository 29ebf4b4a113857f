// Compiler driver: graph -> super graph -> selected schedule -> placed tensors
// -> compiled kernels -> serialised model.
// Stages and their reference counterparts:
//   implement         compiler/src/denox/compiler/implement/implement.cpp:11-68
//   select_schedule   compiler/src/denox/compiler/selection/selection.cpp:23-266
//                     (+ common/src/denox/algorithm/minimum_const_subgraph.hpp:45-353)
//   placement         compiler/src/denox/compiler/placement/placement.cpp:18-326
//   compile_shaders   compiler/src/denox/compiler/compile_shaders/compile_shaders.cpp:35-83
//   serialize         compiler/src/denox/compiler/serialize/serialize.cpp:379-633
//   compile           compiler/src/denox/compiler/compile.cpp:21-61
//   populate          compiler/src/denox/compiler/populate.cpp:23-256
#pragma once
#include "../database/db.hpp"
#include "implement.hpp"
#include <string>
#include <vector>

namespace denox::compiler {

struct ScheduleEntry { std::string shader, config, name; double costMs; bool measured; };

struct CompileReport {
  size_t superGraphEdges = 0, selectedEdges = 0, dispatches = 0, kernelsCompiled = 0, kernelCacheHits = 0;
  double estimatedMs = 0.0;
  std::vector<ScheduleEntry> schedule;
  std::vector<std::string> warnings;
};

// Evaluated value table at the extents assumed for cost estimation.
std::vector<int64_t> assumed_symeval(const Model &model, const SymGraph &sym, const CompileOptions &opt);

// Cost of one super-graph edge in milliseconds: measured latencies from the
// database where every dispatch of the edge has one, else a roofline estimate.
double edge_cost_ms(const SuperGraphEdge &e, const std::vector<int64_t> &dp, const Db *db, const CompileOptions &opt, bool *measured);

// Minimum-cost sub-hypergraph (common/src/denox/algorithm/minimum_const_subgraph.hpp:45-49 of
// the reference): nodes are numbered in topological order, an edge produces its
// output node from all of its input nodes at a cost, every node is produced at
// most once.  Returns the edges of a cheapest set that derives every requested
// output from the input nodes, in execution order; empty with *totalCost >=
// kInfiniteCost when some output cannot be produced.  Exact: memoised search over
// the set of nodes still to be produced.
struct HyperEdge { std::vector<int> inputs; int output; };
constexpr double kInfiniteCost = 1e300;
std::vector<size_t> minimum_cost_subgraph(const std::vector<bool> &isInput, const std::vector<HyperEdge> &edges, const std::vector<double> &edgeCost,
                                          const std::vector<int> &outputs, double *totalCost);

// Minimum-cost set of super-graph edges producing every model output from the
// model inputs; returns edge indices in execution order.
std::vector<size_t> select_schedule(const Model &model, const SuperGraph &g, const std::vector<double> &edgeCost);

std::vector<uint8_t> compile(const Model &model, const hip::HipCompiler &hipc, const Db *db, const CompileOptions &opt, CompileReport *report);

// Insert one row per candidate dispatch (all matches, all configurations),
// evaluated at the assumed extents; returns the number of new rows.
size_t populate(Db &db, const Model &model, const hip::HipCompiler &hipc, const CompileOptions &opt, bool compileKernels = true,
                unsigned shardIndex = 0, unsigned shardCount = 1);

std::vector<uint8_t> push_constant_bytes(const ComputeDispatch &d, const std::vector<int64_t> &dp, std::vector<uint16_t> *offsets = nullptr);

} // namespace denox::compiler
