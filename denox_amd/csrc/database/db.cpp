#include "db.hpp"
#include "../common/error.hpp"
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
static std::vector<uint8_t> unhex(const std::string &s) {
  std::vector<uint8_t> b;
  if (s == "-") return b;
  if (s.size() % 2) fail(Status::IoError, "db: odd hex string");
  auto nib = [](char c) -> int { if (c >= '0' && c <= '9') return c - '0'; if (c >= 'a' && c <= 'f') return c - 'a' + 10; fail(Status::IoError, "db: bad hex digit"); };
  for (size_t i = 0; i < s.size(); i += 2) b.push_back(static_cast<uint8_t>(nib(s[i]) * 16 + nib(s[i + 1])));
  return b;
}
// fields are tab separated; tabs/newlines never occur in the stored strings but are escaped defensively
static std::string esc(const std::string &s) { std::string o; for (char c : s) o += (c == '\t' || c == '\n') ? ' ' : c; return o.empty() ? "-" : o; }
static std::string unesc(const std::string &s) { return s == "-" ? "" : s; }

std::string DbDispatch::key() const {
  return sha256 + ":" + hexOf(pushConstants) + ":" + std::to_string(wg[0]) + "x" + std::to_string(wg[1]) + "x" + std::to_string(wg[2]);
}

double DbDispatch::relativeError() const {
  if (samples < 2 || meanNs <= 0.0) return 1e30;
  const double var = m2 / static_cast<double>(samples);
  return std::sqrt(var / static_cast<double>(samples)) / meanNs;
}

Db Db::open(const std::string &path) {
  Db db;
  db.m_path = path;
  std::ifstream f(path);
  if (!f) return db;
  std::string line;
  if (!std::getline(f, line) || line != "denox-hip-db 1") fail(Status::IoError, "db: unrecognised header in " + path);
  while (std::getline(f, line)) {
    if (line.empty()) continue;
    std::vector<std::string> c;
    std::stringstream ss(line);
    std::string cell;
    while (std::getline(ss, cell, '\t')) c.push_back(cell);
    if (c.size() != 21) fail(Status::IoError, "db: malformed row in " + path);
    DbDispatch d;
    size_t i = 0;
    d.sha256 = c[i++]; d.pushConstants = unhex(c[i++]);
    for (int k = 0; k < 3; ++k) d.wg[k] = static_cast<uint32_t>(std::stoul(c[i++]));
    d.srcPath = unesc(c[i++]); d.defines = unesc(c[i++]); d.entryPoint = unesc(c[i++]);
    for (int k = 0; k < 3; ++k) d.block[k] = static_cast<uint32_t>(std::stoul(c[i++]));
    { // bindings: size:align:param:access;...
      std::stringstream bs(c[i++]);
      std::string b;
      while (std::getline(bs, b, ';')) {
        if (b.empty() || b == "-") continue;
        DbBinding db_;
        unsigned long long sz; unsigned al, pr, ac;
        if (std::sscanf(b.c_str(), "%llu:%u:%u:%u", &sz, &al, &pr, &ac) != 4) fail(Status::IoError, "db: malformed binding");
        db_.byteSize = sz; db_.alignment = static_cast<uint16_t>(al); db_.isParam = pr != 0; db_.access = static_cast<uint8_t>(ac);
        d.bindings.push_back(db_);
      }
    }
    d.operation = unesc(c[i++]); d.shader = unesc(c[i++]); d.config = unesc(c[i++]);
    d.memoryReads = std::stoull(c[i++]); d.memoryWrites = std::stoull(c[i++]); d.flops = std::stoull(c[i++]);
    d.samples = std::stoull(c[i++]); d.meanNs = std::stod(c[i++]); d.m2 = std::stod(c[i++]);
    db.insert_dispatch(d);
  }
  return db;
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
    std::ofstream f(tmp);
    if (!f) fail(Status::IoError, "db: cannot write " + tmp);
    f << "denox-hip-db 1\n";
    f.precision(17);
    for (const auto &d : m_rows) {
      f << d.sha256 << '\t' << hexOf(d.pushConstants) << '\t' << d.wg[0] << '\t' << d.wg[1] << '\t' << d.wg[2] << '\t'
        << esc(d.srcPath) << '\t' << esc(d.defines) << '\t' << esc(d.entryPoint) << '\t' << d.block[0] << '\t' << d.block[1] << '\t' << d.block[2] << '\t';
      if (d.bindings.empty()) f << '-';
      for (const auto &b : d.bindings) f << b.byteSize << ':' << b.alignment << ':' << (b.isParam ? 1 : 0) << ':' << static_cast<unsigned>(b.access) << ';';
      f << '\t' << esc(d.operation) << '\t' << esc(d.shader) << '\t' << esc(d.config) << '\t' << d.memoryReads << '\t' << d.memoryWrites << '\t' << d.flops
        << '\t' << d.samples << '\t' << d.meanNs << '\t' << d.m2 << '\n';
    }
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
