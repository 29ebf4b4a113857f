// Dispatch timing table -- the cost model behind schedule selection.
//
// Role of the reference's denox::Db (database/src/denox/db/Db.hpp:15-69,
// schema db.fbs:87-107): one row per distinct dispatch, keyed by the kernel's
// source hash, its push-constant bytes and its workgroup counts (bindings are
// deliberately not part of the key, db.fbs:93-102, Db.cpp:551-557); each row
// accumulates timing samples as a running mean / variance (Db.cpp:719-756) and
// is written back with temp-file + rename (Db.cpp:499-506).  FlatBuffers are
// not available, so the file is line-oriented text.
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

  std::vector<DbDispatch> &rows() { return m_rows; }
  const std::vector<DbDispatch> &rows() const { return m_rows; }
  const std::string &path() const { return m_path; }

private:
  std::string m_path;
  std::vector<DbDispatch> m_rows;
  std::map<std::string, size_t> m_index;
};

} // namespace denox
