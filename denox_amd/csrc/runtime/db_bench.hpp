// Fills the timing table by running every unconverged dispatch on the GPU.
// Role of the reference's runtime::Db::bench (runtime/src/denox/runtime/db.hpp:9-37,
// db.cpp:665-868): hipEvent pairs instead of Vulkan timestamp queries, the same
// convergence rule (at least minSamples samples and standard error of the mean
// <= maxRelativeError * mean, db.cpp:626-649), all bindings of a dispatch placed
// at packed offsets of one scratch allocation with unspecified contents
// (db.cpp:337-384), results written back with temp-file + rename after every
// epoch when saveProgress is set (db.cpp:797-805).
#pragma once
#include "../database/db.hpp"
#include "../hip/hip_compiler.hpp"
#include "runtime.hpp"

namespace denox::runtime {

struct DbBenchOptions {
  uint32_t minSamples = 10;
  double maxRelativeError = 0.05;
  uint32_t maxSamples = 200;   // upper bound per dispatch and call
  uint32_t batch = 10;         // timed launches between convergence checks
  uint32_t warmup = 2;
  uint32_t epochSize = 500;    // dispatches per write-back
  bool saveProgress = true;
  std::string filter;          // only rows whose shader or operation contains this text
};

struct DbBenchResult { size_t benchmarked = 0, converged = 0, skipped = 0, failed = 0; };

DbBenchResult db_bench(Db &db, const ContextHandle &ctx, const hip::HipCompiler &hipc, const DbBenchOptions &opt);

} // namespace denox::runtime
