#include "db_bench.hpp"
#include <algorithm>
#include <chrono>
#include <cstring>
#include <sstream>
#include <vector>

namespace denox::runtime {

static bool converged(const DbDispatch &d, const DbBenchOptions &opt) {
  return d.samples >= opt.minSamples && d.relativeError() <= opt.maxRelativeError;
}

DbBenchResult db_bench(Db &db, const ContextHandle &ctx, const hip::HipCompiler &hipc, const DbBenchOptions &opt) {
  DbBenchResult res;
  ctx->makeCurrent();
  hipStream_t s = ctx->stream();
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipCheck(hipEventCreate(&e0), "hipEventCreate");
  hipCheck(hipEventCreate(&e1), "hipEventCreate");
  void *scratch = nullptr;
  uint64_t scratchBytes = 0;
  size_t sinceWriteback = 0;
  bool envRecorded = false;
  auto cleanup = [&]() {
    if (scratch) (void)hipFree(scratch);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
  };
  try {
    for (size_t r = 0; r < db.rows().size(); ++r) {
      DbDispatch &row = db.rows()[r];
      if (!opt.filter.empty() && row.shader.find(opt.filter) == std::string::npos && row.operation.find(opt.filter) == std::string::npos) { ++res.skipped; continue; }
      if (converged(row, opt)) { ++res.skipped; continue; }
      if (!envRecorded) { // one BenchEnv per session that measures anything (runtime/src/denox/runtime/db.cpp:694-698 of the reference)
        hipDeviceProp_t prop;
        hipCheck(hipGetDeviceProperties(&prop, ctx->device()), "hipGetDeviceProperties");
        int driver = 0;
        (void)hipDriverGetVersion(&driver);
        DbEnv env;
        env.device = std::string(prop.name) + " (" + prop.gcnArchName + ")";
        env.os = "Linux";
        env.driverVersion = "HIP " + std::to_string(driver);
        env.version = "denox-hip 0.1";
        env.startTimestamp = static_cast<uint64_t>(std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::system_clock::now().time_since_epoch()).count());
        env.jitWarmupIterations = static_cast<uint16_t>(std::min<uint32_t>(opt.warmup, 0xFFFF));
        env.measurementIterations = static_cast<uint16_t>(std::min<uint32_t>(opt.batch, 0xFFFF));
        db.create_bench_environment(std::move(env));
        envRecorded = true;
      }
      // rebuild the kernel variant from its source path and definitions
      hip::HipCompilerInstance k = hipc.read(row.srcPath);
      std::stringstream ss(row.defines);
      std::string kv;
      while (ss >> kv) {
        const size_t eq = kv.find('=');
        if (eq == std::string::npos) fail(Status::IoError, "db: malformed definition '" + kv + "'");
        k.define(kv.substr(0, eq), kv.substr(eq + 1));
      }
      if (k.sha256() != row.sha256) { ++res.failed; continue; } // kernel source changed since the row was made
      const std::vector<uint8_t> code = k.compile();
      hipModule_t mod = nullptr;
      hipCheck(hipModuleLoadData(&mod, code.data()), "hipModuleLoadData");
      try {
        hipFunction_t fn = nullptr;
        hipCheck(hipModuleGetFunction(&fn, mod, row.entryPoint.c_str()), "hipModuleGetFunction");
        // pack the bindings into one scratch allocation
        uint64_t need = 0;
        std::vector<uint64_t> offs;
        for (const auto &b : row.bindings) {
          const uint64_t al = std::max<uint64_t>(b.alignment, 256);
          need = (need + al - 1) / al * al;
          offs.push_back(need);
          need += b.byteSize + 256;
        }
        if (need > scratchBytes) {
          if (scratch) hipCheck(hipFree(scratch), "hipFree");
          scratch = nullptr;
          hipCheck(hipMalloc(&scratch, need), "hipMalloc(scratch)");
          scratchBytes = need;
          // Finite binary16 values of mixed sign and magnitude below 2: timings then include the
          // switching activity of real data (an all-zero buffer lets the chip clock higher than a
          // frame would) and no arithmetic meets NaN or infinity.
          std::vector<uint16_t> pattern(1u << 20);
          uint32_t lcg = 12345u;
          for (auto &h : pattern) {
            lcg = lcg * 1664525u + 1013904223u;
            h = static_cast<uint16_t>(((lcg >> 16) & 0x8000u) | (0x2C00u + ((lcg >> 8) % 0x1000u))); // |x| in [2^-4, 1)
          }
          for (uint64_t off = 0; off < need; off += pattern.size() * 2) {
            const uint64_t n = std::min<uint64_t>(pattern.size() * 2, need - off);
            hipCheck(hipMemcpyAsync(static_cast<uint8_t *>(scratch) + off, pattern.data(), n, hipMemcpyHostToDevice, s), "hipMemcpyAsync(scratch)");
          }
          hipCheck(hipStreamSynchronize(s), "hipStreamSynchronize");
        }
        std::vector<uint8_t> args(row.bindings.size() * sizeof(void *));
        for (size_t i = 0; i < offs.size(); ++i) {
          void *p = static_cast<uint8_t *>(scratch) + offs[i];
          std::memcpy(args.data() + i * sizeof(void *), &p, sizeof(void *));
        }
        const size_t pcAlign = 4; // every push constant emitted is 32 bit
        while (args.size() % pcAlign) args.push_back(0);
        args.insert(args.end(), row.pushConstants.begin(), row.pushConstants.end());
        size_t argSize = args.size();
        void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, args.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &argSize, HIP_LAUNCH_PARAM_END};
        auto launch = [&]() {
          hipCheck(hipModuleLaunchKernel(fn, row.wg[0], row.wg[1], row.wg[2], row.block[0], row.block[1], row.block[2], 0, s, nullptr, config), "hipModuleLaunchKernel");
        };
        if (row.wg[0] == 0 || row.wg[1] == 0 || row.wg[2] == 0) { ++res.skipped; (void)hipModuleUnload(mod); continue; }
        for (uint32_t i = 0; i < opt.warmup; ++i) launch();
        hipCheck(hipStreamSynchronize(s), "hipStreamSynchronize");
        uint32_t taken = 0;
        while (!converged(row, opt) && taken < opt.maxSamples) {
          for (uint32_t i = 0; i < opt.batch; ++i, ++taken) {
            hipCheck(hipEventRecord(e0, s), "hipEventRecord");
            launch();
            hipCheck(hipEventRecord(e1, s), "hipEventRecord");
            hipCheck(hipEventSynchronize(e1), "hipEventSynchronize");
            float ms = 0.0f;
            hipCheck(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
            db.add_dispatch_benchmark_result(r, static_cast<double>(ms) * 1e6);
          }
        }
        ++res.benchmarked;
        if (converged(row, opt)) ++res.converged;
      } catch (...) {
        (void)hipModuleUnload(mod);
        throw;
      }
      hipCheck(hipModuleUnload(mod), "hipModuleUnload");
      if (opt.saveProgress && ++sinceWriteback >= opt.epochSize) { db.atomic_writeback(); sinceWriteback = 0; }
    }
    if (opt.saveProgress && !db.path().empty()) db.atomic_writeback();
  } catch (...) {
    cleanup();
    throw;
  }
  cleanup();
  return res;
}

} // namespace denox::runtime
