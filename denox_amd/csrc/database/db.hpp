// Dispatch timing table -- the cost model behind schedule selection.
//
// Role of the reference's denox::Db (database/src/denox/db/Db.hpp:15-69,
// schema db.fbs:87-107): one row per distinct dispatch, keyed by the kernel's
// source hash, its push-constant bytes and its workgroup counts (bindings are
// deliberately not part of the key, db.fbs:93-102, Db.cpp:551-557); each row
// accumulates timing samples as a running mean / variance (Db.cpp:719-756) and
// is written back with temp-file + rename (Db.cpp:499-506).
//
// The file is a FlatBuffer of the reference's schema db.fbs:1-150 (identifier "dbdb", root table Db), written and read
// over common/flatbuf.hpp.  What a HIP backend keeps and the schema lacks is appended to the tables the way FlatBuffers
// schemas grow (new field ids at the end, skipped by readers of the original schema):
//   ShaderBinary    + src_path:string (2), defines:string (3)   the kernel is rebuilt from source + definitions; `spirv` stays empty
//   ComputeDispatch + entry_point:string (9), block_{x,y,z}:uint32 (10-12)
//   Timing          + sample_count:uint64 (3), mean_ns:double (4), m2:double (5)   the running statistics at full precision;
//                     mean_latency_ns / std_derivation_ns hold the same values rounded to whole nanoseconds, `samples` stays
//                     empty (individual samples are not kept)
// ComputeDispatch.hash is FNV-1a over the row's key; the reference's value comes from std::hash and is specific to its build.
#pragma once
#include <cmath>
#include <cstdint>
#include <map>
#include <optional>
#include <string>
#include <vector>

namespace denox {

struct DbBinding { uint64_t byteSize; uint16_t alignment; bool isParam; uint8_t access; };

struct DbDispatch {
  // key
  std::string sha256;           // of source + definitions (identifies the code object)
  std::vector<uint8_t> pushConstants;
  uint32_t wg[3] = {1, 1, 1};
  // what is needed to run it again
  std::string srcPath, defines, entryPoint;
  uint32_t block[3] = {1, 1, 1};
  std::vector<DbBinding> bindings;
  // info
  std::string operation, shader, config;
  uint64_t memoryReads = 0, memoryWrites = 0, flops = 0;
  // statistics over samples (nanoseconds): Welford running mean / M2
  uint64_t samples = 0;
  double meanNs = 0.0, m2 = 0.0;

  std::string key() const;
  double stdNs() const { return samples > 1 ? std::sqrt(m2 / static_cast<double>(samples)) : 0.0; }
  // standard error of the mean relative to the mean
  double relativeError() const;
};

// One benchmarking session (table BenchEnv, db.fbs:130-143; reference: DbEnv.hpp:14-27).
struct DbEnv {
  std::string device, os, driverVersion, commitHash, version;
  uint64_t startTimestamp = 0;
  uint16_t clockMode = 0; // ClockMode::Unavailable: clocks are not pinned by this backend
  uint16_t l2WarmupIterations = 0, jitWarmupIterations = 0, measurementIterations = 0;
};

class Db {
public:
  static Db open(const std::string &path); // missing file -> empty table bound to that path
  Db() = default;

  // insert if absent; returns the row index
  size_t insert_dispatch(const DbDispatch &d);
  std::optional<size_t> find(const std::string &key) const;
  // mean latency in milliseconds, nullopt when the dispatch has no samples
  std::optional<double> query_dispatch_latency(const std::string &sha256, const std::vector<uint8_t> &pc, const uint32_t wg[3]) const;
  void add_dispatch_benchmark_result(size_t row, double latencyNs);
  void atomic_writeback() const;
  std::string to_csv() const;
  // bytes of the file / a table from such bytes (Error(IoError) when they are not a timing database)
  std::vector<uint8_t> serialize() const;
  static Db deserialize(const void *data, size_t size, const std::string &path);
  uint32_t create_bench_environment(DbEnv env) { m_envs.push_back(std::move(env)); return static_cast<uint32_t>(m_envs.size() - 1); }
  const std::vector<DbEnv> &environments() const { return m_envs; }

  std::vector<DbDispatch> &rows() { return m_rows; }
  const std::vector<DbDispatch> &rows() const { return m_rows; }
  const std::string &path() const { return m_path; }

private:
  std::string m_path;
  std::vector<DbDispatch> m_rows;
  std::vector<DbEnv> m_envs;
  std::map<std::string, size_t> m_index;
};

} // namespace denox
