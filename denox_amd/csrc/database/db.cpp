#include "db.hpp"
#include "../common/error.hpp"
#include "../common/flatbuf.hpp"
#include <algorithm>
#include <iterator>
#include <cmath>
#include <cstdio>
#include <fstream>
#include <sstream>
#include <unistd.h>

namespace denox {

static std::string hexOf(const std::vector<uint8_t> &b) {
  static const char *x = "0123456789abcdef";
  std::string s;
  for (uint8_t c : b) { s.push_back(x[c >> 4]); s.push_back(x[c & 15]); }
  return s.empty() ? "-" : s;
}

std::string DbDispatch::key() const {
  return sha256 + ":" + hexOf(pushConstants) + ":" + std::to_string(wg[0]) + "x" + std::to_string(wg[1]) + "x" + std::to_string(wg[2]);
}

double DbDispatch::relativeError() const {
  if (samples < 2 || meanNs <= 0.0) return 1e30;
  const double var = m2 / static_cast<double>(samples);
  return std::sqrt(var / static_cast<double>(samples)) / meanNs;
}

namespace {
// Field ids: declaration order of each table in db.fbs, then the additions listed in db.hpp.
namespace id {
enum { SB_src_sha256 = 0, SB_spirv = 1, SB_src_path = 2, SB_defines = 3 };                                              // db.fbs:8-12
enum { TBI_width = 0, TBI_height = 1, TBI_channels = 2, TBI_dtype = 3, TBI_is_param = 4 };                              // db.fbs:42-48
enum { TB_set = 0, TB_binding = 1, TB_access = 2, TB_format = 3, TB_storage = 4, TB_byte_size = 5, TB_min_align = 6, TB_info = 7 }; // db.fbs:50-59
enum { T_samples = 0, T_mean_latency_ns = 1, T_std_derivation_ns = 2, T_sample_count = 3, T_mean_ns = 4, T_m2 = 5 };    // db.fbs:68-72
enum { CDI_operation = 0, CDI_shader_name = 1, CDI_config = 2, CDI_memory_reads = 3, CDI_memory_writes = 4, CDI_flops = 5, CDI_coopmat = 6, CDI_inputs = 7, CDI_outputs = 8 }; // db.fbs:74-85
enum { CD_binary_id = 0, CD_wgx = 1, CD_wgy = 2, CD_wgz = 3, CD_push_constant = 4, CD_hash = 5, CD_bindings = 6, CD_time = 7, CD_info = 8, CD_entry_point = 9,
       CD_block_x = 10, CD_block_y = 11, CD_block_z = 12, CD_count = 13 };                                              // db.fbs:87-107
enum { BE_device = 0, BE_os = 1, BE_driver_version = 2, BE_commit_hash = 3, BE_version = 4, BE_start_timestamp = 5, BE_clock_mode = 6, BE_l2_warmup = 7,
       BE_jit_warmup = 8, BE_measurement = 9 };                                                                         // db.fbs:130-143
enum { Db_version = 0, Db_env = 1, Db_shader_binaries = 2, Db_dispatches = 3 };                                         // db.fbs:145-150
} // namespace id
constexpr char IDENTIFIER[4] = {'d', 'b', 'd', 'b'}; // db.fbs:4

uint64_t fnv1a(const std::string &s) {
  uint64_t h = 1469598103934665603ull;
  for (unsigned char c : s) { h ^= c; h *= 1099511628211ull; }
  return h;
}
// the digest as the eight 32-bit words of table ShaderBinary (DbShaderBinary.hpp of the reference keeps uint32_t h[8])
bool shaWords(const std::string &hex, uint32_t out[8]) {
  if (hex.size() != 64) return false;
  for (int w = 0; w < 8; ++w) {
    uint32_t v = 0;
    for (int k = 0; k < 8; ++k) {
      const char c = hex[static_cast<size_t>(w * 8 + k)];
      const int n = c >= '0' && c <= '9' ? c - '0' : c >= 'a' && c <= 'f' ? c - 'a' + 10 : -1;
      if (n < 0) return false;
      v = v << 4 | static_cast<uint32_t>(n);
    }
    out[w] = v;
  }
  return true;
}
std::string shaHex(const fb::Vector &words) {
  static const char *x = "0123456789abcdef";
  std::string s;
  for (uint32_t w = 0; w < 8; ++w) {
    const uint32_t v = words.get<uint32_t>(w);
    for (int k = 7; k >= 0; --k) s.push_back(x[(v >> (4 * k)) & 15]);
  }
  return s;
}
} // namespace

std::vector<uint8_t> Db::serialize() const {
  fb::Builder b(1u << 20);
  // one ShaderBinary per distinct kernel variant
  std::map<std::string, uint32_t> binaryOf;
  std::vector<const DbDispatch *> firstRow;
  for (const auto &d : m_rows)
    if (binaryOf.emplace(d.sha256, static_cast<uint32_t>(firstRow.size())).second) firstRow.push_back(&d);

  std::vector<fb::Off> rows(m_rows.size());
  for (size_t r = 0; r < m_rows.size(); ++r) {
    const DbDispatch &d = m_rows[r];
    std::vector<uint32_t> ins, outs;
    std::vector<fb::Off> bindings(d.bindings.size());
    for (size_t i = 0; i < d.bindings.size(); ++i) {
      const DbBinding &x = d.bindings[i];
      if (!x.isParam && x.access == 0) ins.push_back(static_cast<uint32_t>(i));
      if (x.access != 0) outs.push_back(static_cast<uint32_t>(i));
      b.startTable(5);
      b.addScalar<uint8_t>(id::TBI_is_param, x.isParam ? 1 : 0, 0);
      const fb::Off info = b.endTable();
      b.startTable(8);
      b.addScalar<uint32_t>(id::TB_binding, static_cast<uint32_t>(i), 0);
      b.addScalar<uint8_t>(id::TB_access, x.access, 0);
      b.addScalar<uint64_t>(id::TB_byte_size, x.byteSize, 0);
      b.addScalar<uint32_t>(id::TB_min_align, x.alignment, 0);
      b.addOffset(id::TB_info, info);
      bindings[i] = b.endTable();
    }
    const fb::Off bindingVec = b.createOffsetVector(bindings);
    const fb::Off inVec = b.createVector(ins.data(), 4, 4, ins.size()), outVec = b.createVector(outs.data(), 4, 4, outs.size());
    const fb::Off op = b.createString(d.operation), shader = b.createString(d.shader), config = b.createString(d.config);
    b.startTable(9);
    b.addOffset(id::CDI_operation, op);
    b.addOffset(id::CDI_shader_name, shader);
    b.addOffset(id::CDI_config, config);
    b.addScalar<uint64_t>(id::CDI_memory_reads, d.memoryReads, 0);
    b.addScalar<uint64_t>(id::CDI_memory_writes, d.memoryWrites, 0);
    b.addScalar<uint64_t>(id::CDI_flops, d.flops, 0);
    b.addScalar<uint8_t>(id::CDI_coopmat, d.flops != 0 ? 1 : 0, 0); // the matrix pipe is used by every kernel that counts flops
    b.addOffset(id::CDI_inputs, inVec);
    b.addOffset(id::CDI_outputs, outVec);
    const fb::Off info = b.endTable();
    fb::Off time = 0;
    if (d.samples) {
      const fb::Off samples = b.createOffsetVector({});
      b.startTable(6);
      b.addOffset(id::T_samples, samples);
      b.addScalar<uint64_t>(id::T_mean_latency_ns, static_cast<uint64_t>(std::llround(std::max(0.0, d.meanNs))), 0);
      b.addScalar<uint64_t>(id::T_std_derivation_ns, static_cast<uint64_t>(std::llround(d.stdNs())), 0);
      b.addScalar<uint64_t>(id::T_sample_count, d.samples, 0);
      b.addScalar<double>(id::T_mean_ns, d.meanNs, 0.0);
      b.addScalar<double>(id::T_m2, d.m2, 0.0);
      time = b.endTable();
    }
    const fb::Off pc = b.createVector(d.pushConstants.data(), 1, 1, d.pushConstants.size());
    const fb::Off entry = b.createString(d.entryPoint);
    b.startTable(id::CD_count);
    b.addScalar<uint32_t>(id::CD_binary_id, binaryOf.at(d.sha256), 0);
    b.addScalar<uint32_t>(id::CD_wgx, d.wg[0], 0);
    b.addScalar<uint32_t>(id::CD_wgy, d.wg[1], 0);
    b.addScalar<uint32_t>(id::CD_wgz, d.wg[2], 0);
    b.addOffset(id::CD_push_constant, pc);
    b.addScalar<uint64_t>(id::CD_hash, fnv1a(d.key()), 0);
    b.addOffset(id::CD_bindings, bindingVec);
    b.addOffset(id::CD_time, time);
    b.addOffset(id::CD_info, info);
    b.addOffset(id::CD_entry_point, entry);
    b.addScalar<uint32_t>(id::CD_block_x, d.block[0], 0);
    b.addScalar<uint32_t>(id::CD_block_y, d.block[1], 0);
    b.addScalar<uint32_t>(id::CD_block_z, d.block[2], 0);
    rows[r] = b.endTable();
  }
  const fb::Off dispatches = b.createOffsetVector(rows);

  std::vector<fb::Off> bins(firstRow.size());
  for (size_t i = 0; i < firstRow.size(); ++i) {
    uint32_t words[8];
    if (!shaWords(firstRow[i]->sha256, words)) fail(Status::Internal, "db: kernel hash is not a SHA-256 digest");
    const fb::Off sha = b.createVector(words, 4, 4, 8), spirv = b.createVector(nullptr, 4, 4, 0);
    const fb::Off src = b.createString(firstRow[i]->srcPath), defs = b.createString(firstRow[i]->defines);
    b.startTable(4);
    b.addOffset(id::SB_src_sha256, sha);
    b.addOffset(id::SB_spirv, spirv);
    b.addOffset(id::SB_src_path, src);
    b.addOffset(id::SB_defines, defs);
    bins[i] = b.endTable();
  }
  const fb::Off binaries = b.createOffsetVector(bins);

  std::vector<fb::Off> envs(m_envs.size());
  for (size_t i = 0; i < m_envs.size(); ++i) {
    const DbEnv &e = m_envs[i];
    const fb::Off device = b.createString(e.device), os = b.createString(e.os), driver = b.createString(e.driverVersion), commit = b.createString(e.commitHash),
                  version = b.createString(e.version);
    b.startTable(10);
    b.addOffset(id::BE_device, device);
    b.addOffset(id::BE_os, os);
    b.addOffset(id::BE_driver_version, driver);
    b.addOffset(id::BE_commit_hash, commit);
    b.addOffset(id::BE_version, version);
    b.addScalar<uint64_t>(id::BE_start_timestamp, e.startTimestamp, 0);
    b.addScalar<uint16_t>(id::BE_clock_mode, e.clockMode, 0);
    b.addScalar<uint16_t>(id::BE_l2_warmup, e.l2WarmupIterations, 0);
    b.addScalar<uint16_t>(id::BE_jit_warmup, e.jitWarmupIterations, 0);
    b.addScalar<uint16_t>(id::BE_measurement, e.measurementIterations, 0);
    envs[i] = b.endTable();
  }
  const fb::Off envVec = b.createOffsetVector(envs);

  b.startTable(4);
  b.addOffset(id::Db_env, envVec);
  b.addOffset(id::Db_shader_binaries, binaries);
  b.addOffset(id::Db_dispatches, dispatches);
  return b.finish(b.endTable(), IDENTIFIER); // version 0, as Db.cpp:484 of the reference writes
}

Db Db::deserialize(const void *data, size_t size, const std::string &path) {
  Db db;
  db.m_path = path;
  try {
    size_t spent = 0;
    const fb::Table root = fb::Table::root(data, size, IDENTIFIER, &spent);
    if (root.scalar<uint32_t>(id::Db_version, 0) != 0) fail(Status::IoError, "unknown version");
    const fb::Vector envs = root.vector(id::Db_env, 4, 4);
    for (uint32_t i = 0; i < envs.size(); ++i) {
      const fb::Table t = envs.table(i);
      DbEnv e;
      e.device = t.str(id::BE_device); e.os = t.str(id::BE_os); e.driverVersion = t.str(id::BE_driver_version);
      e.commitHash = t.str(id::BE_commit_hash); e.version = t.str(id::BE_version);
      e.startTimestamp = t.scalar<uint64_t>(id::BE_start_timestamp, 0);
      e.clockMode = t.scalar<uint16_t>(id::BE_clock_mode, 0);
      e.l2WarmupIterations = t.scalar<uint16_t>(id::BE_l2_warmup, 0);
      e.jitWarmupIterations = t.scalar<uint16_t>(id::BE_jit_warmup, 0);
      e.measurementIterations = t.scalar<uint16_t>(id::BE_measurement, 0);
      db.m_envs.push_back(std::move(e));
    }
    struct Binary { std::string sha, srcPath, defines; };
    std::vector<Binary> bins;
    const fb::Vector binaries = root.vector(id::Db_shader_binaries, 4, 4);
    for (uint32_t i = 0; i < binaries.size(); ++i) {
      const fb::Table t = binaries.table(i);
      const fb::Vector sha = t.vector(id::SB_src_sha256, 4, 4);
      if (sha.size() != 8) fail(Status::IoError, "kernel hash is not 8 words");
      bins.push_back(Binary{shaHex(sha), t.str(id::SB_src_path), t.str(id::SB_defines)});
    }
    const fb::Vector rows = root.vector(id::Db_dispatches, 4, 4);
    for (uint32_t r = 0; r < rows.size(); ++r) {
      const fb::Table t = rows.table(r);
      DbDispatch d;
      const uint32_t bin = t.scalar<uint32_t>(id::CD_binary_id, 0);
      if (bin >= bins.size()) fail(Status::IoError, "dispatch names a missing binary");
      d.sha256 = bins[bin].sha; d.srcPath = bins[bin].srcPath; d.defines = bins[bin].defines;
      d.wg[0] = t.scalar<uint32_t>(id::CD_wgx, 0); d.wg[1] = t.scalar<uint32_t>(id::CD_wgy, 0); d.wg[2] = t.scalar<uint32_t>(id::CD_wgz, 0);
      const fb::Vector pc = t.vector(id::CD_push_constant, 1, 1);
      if (pc.present()) d.pushConstants.assign(pc.data(), pc.data() + pc.size());
      d.entryPoint = t.str(id::CD_entry_point);
      d.block[0] = t.scalar<uint32_t>(id::CD_block_x, 0); d.block[1] = t.scalar<uint32_t>(id::CD_block_y, 0); d.block[2] = t.scalar<uint32_t>(id::CD_block_z, 0);
      const fb::Vector bindings = t.vector(id::CD_bindings, 4, 4);
      for (uint32_t i = 0; i < bindings.size(); ++i) {
        const fb::Table bt = bindings.table(i);
        DbBinding x;
        x.byteSize = bt.scalar<uint64_t>(id::TB_byte_size, 0);
        x.alignment = static_cast<uint16_t>(bt.scalar<uint32_t>(id::TB_min_align, 0));
        x.access = bt.scalar<uint8_t>(id::TB_access, 0);
        if (x.access > 2) fail(Status::IoError, "bad access");
        x.isParam = bt.table(id::TB_info).scalar<uint8_t>(id::TBI_is_param, 0) != 0;
        d.bindings.push_back(x);
      }
      const fb::Table info = t.table(id::CD_info);
      d.operation = info.str(id::CDI_operation); d.shader = info.str(id::CDI_shader_name); d.config = info.str(id::CDI_config);
      d.memoryReads = info.scalar<uint64_t>(id::CDI_memory_reads, 0);
      d.memoryWrites = info.scalar<uint64_t>(id::CDI_memory_writes, 0);
      d.flops = info.scalar<uint64_t>(id::CDI_flops, 0);
      const fb::Table time = t.table(id::CD_time);
      if (time.present()) {
        if (time.has(id::T_sample_count)) {
          d.samples = time.scalar<uint64_t>(id::T_sample_count, 0);
          d.meanNs = time.scalar<double>(id::T_mean_ns, 0.0);
          d.m2 = time.scalar<double>(id::T_m2, 0.0);
          if (!(d.meanNs >= 0.0) || !(d.m2 >= 0.0) || !std::isfinite(d.meanNs) || !std::isfinite(d.m2)) fail(Status::IoError, "bad statistics");
        } else { // a table in the reference's form: one Sample per measurement, whole-nanosecond mean and deviation
          d.samples = time.vector(id::T_samples, 4, 4).size();
          d.meanNs = static_cast<double>(time.scalar<uint64_t>(id::T_mean_latency_ns, 0));
          const double sd = static_cast<double>(time.scalar<uint64_t>(id::T_std_derivation_ns, 0));
          d.m2 = sd * sd * static_cast<double>(d.samples);
        }
      }
      db.insert_dispatch(d);
    }
  } catch (const Error &e) {
    fail(Status::IoError, "db: " + (path.empty() ? std::string("buffer") : path) + " is not a timing database (" + e.what() + ")");
  }
  return db;
}

Db Db::open(const std::string &path) {
  std::ifstream f(path, std::ios::binary);
  if (!f) {
    Db db;
    db.m_path = path;
    return db;
  }
  const std::vector<char> bytes((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
  return deserialize(bytes.data(), bytes.size(), path);
}

size_t Db::insert_dispatch(const DbDispatch &d) {
  const std::string k = d.key();
  auto it = m_index.find(k);
  if (it != m_index.end()) return it->second;
  m_rows.push_back(d);
  m_index.emplace(k, m_rows.size() - 1);
  return m_rows.size() - 1;
}

std::optional<size_t> Db::find(const std::string &key) const {
  auto it = m_index.find(key);
  if (it == m_index.end()) return std::nullopt;
  return it->second;
}

std::optional<double> Db::query_dispatch_latency(const std::string &sha256, const std::vector<uint8_t> &pc, const uint32_t wg[3]) const {
  DbDispatch probe;
  probe.sha256 = sha256; probe.pushConstants = pc;
  for (int i = 0; i < 3; ++i) probe.wg[i] = wg[i];
  auto r = find(probe.key());
  if (!r || m_rows[*r].samples == 0) return std::nullopt;
  return m_rows[*r].meanNs * 1e-6;
}

void Db::add_dispatch_benchmark_result(size_t row, double latencyNs) {
  if (row >= m_rows.size()) fail(Status::InvalidArgument, "db: row out of range");
  DbDispatch &d = m_rows[row];
  // Welford update
  d.samples += 1;
  const double delta = latencyNs - d.meanNs;
  d.meanNs += delta / static_cast<double>(d.samples);
  d.m2 += delta * (latencyNs - d.meanNs);
}

void Db::atomic_writeback() const {
  if (m_path.empty()) fail(Status::InvalidArgument, "db: no path to write to");
  const std::string tmp = m_path + ".tmp." + std::to_string(getpid());
  {
    const std::vector<uint8_t> bytes = serialize();
    std::ofstream f(tmp, std::ios::binary);
    if (!f) fail(Status::IoError, "db: cannot write " + tmp);
    f.write(reinterpret_cast<const char *>(bytes.data()), static_cast<std::streamsize>(bytes.size()));
    f.flush();
    if (!f) fail(Status::IoError, "db: write failed");
  }
  if (std::rename(tmp.c_str(), m_path.c_str()) != 0) { std::remove(tmp.c_str()); fail(Status::IoError, "db: rename failed"); }
}

std::string Db::to_csv() const {
  // column set of the reference's `dumpcsv` (cli/src/denox/cli/dumpcsv.cpp:15-46), minus host/driver fields
  std::ostringstream o;
  o << "operation,shader,config,src_path,defines,wg_x,wg_y,wg_z,flops,memory_reads,memory_writes,samples,latency_ms,std_ms\n";
  for (const auto &d : m_rows)
    o << '"' << d.operation << "\",\"" << d.shader << "\",\"" << d.config << "\",\"" << d.srcPath << "\",\"" << d.defines << "\"," << d.wg[0] << ',' << d.wg[1] << ',' << d.wg[2]
      << ',' << d.flops << ',' << d.memoryReads << ',' << d.memoryWrites << ',' << d.samples << ',' << d.meanNs * 1e-6 << ',' << d.stdNs() * 1e-6 << '\n';
  return o.str();
}

} // namespace denox
