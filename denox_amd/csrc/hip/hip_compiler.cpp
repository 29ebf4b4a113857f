#include "hip_compiler.hpp"
#include "../common/error.hpp"
#include "../common/sha256.hpp"
#include <cstdio>
#include <cstdlib>
#include <dirent.h>
#include <dlfcn.h>
#include <fcntl.h>
#include <fstream>
#include <hip/hiprtc.h>
#include <sstream>
#include <sys/stat.h>
#include <unistd.h>
#include <algorithm>

namespace denox::hip {

// Packed-fp32 instruction selection is switched off for every kernel.
static const char *const kFlags[] = {"-O3", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-ffp-contract=off"};

static std::string readFile(const std::string &path) {
  std::ifstream f(path, std::ios::binary);
  if (!f) fail(Status::IoError, "cannot read " + path);
  std::ostringstream ss;
  ss << f.rdbuf();
  return ss.str();
}

std::string libraryDirectory() {
  Dl_info info;
  if (dladdr(reinterpret_cast<void *>(&libraryDirectory), &info) && info.dli_fname) {
    std::string p = info.dli_fname;
    const size_t slash = p.rfind('/');
    return slash == std::string::npos ? "." : p.substr(0, slash);
  }
  return ".";
}

std::string defaultKernelDir() {
  if (const char *e = std::getenv("DENOX_HIP_KERNEL_DIR")) return e;
  return libraryDirectory() + "/../csrc/kernels";
}

std::string defaultCacheDir() {
  if (const char *e = std::getenv("DENOX_HIP_CACHE_DIR")) return e;
  return libraryDirectory() + "/../kernel_cache";
}

HipCompiler::HipCompiler(std::string kernelDir, std::string cacheDir, std::string arch)
    : m_kernelDir(std::move(kernelDir)), m_cacheDir(std::move(cacheDir)), m_arch(std::move(arch)) {
  std::vector<std::string> headers;
  if (DIR *d = opendir(m_kernelDir.c_str())) {
    while (dirent *e = readdir(d)) {
      std::string n = e->d_name;
      if (n.size() > 2 && n.substr(n.size() - 2) == ".h") headers.push_back(n);
    }
    closedir(d);
  } else {
    fail(Status::IoError, "kernel directory not found: " + m_kernelDir);
  }
  for (const auto &h : headers) m_headerText[h] = readFile(m_kernelDir + "/" + h);
  if (!m_cacheDir.empty()) mkdir(m_cacheDir.c_str(), 0755);
}

// Names of the headers of the kernel directory that `text` includes with #include "name".
static std::vector<std::string> includedHeaders(const std::string &text) {
  std::vector<std::string> out;
  size_t pos = 0;
  while ((pos = text.find("#include", pos)) != std::string::npos) {
    pos += 8;
    const size_t eol = text.find('\n', pos);
    const size_t q0 = text.find('"', pos);
    if (q0 == std::string::npos || (eol != std::string::npos && q0 > eol)) continue;
    const size_t q1 = text.find('"', q0 + 1);
    if (q1 == std::string::npos || (eol != std::string::npos && q1 > eol)) continue;
    out.push_back(text.substr(q0 + 1, q1 - q0 - 1));
  }
  return out;
}

HipCompilerInstance HipCompiler::read(const std::string &relPath) const {
  HipCompilerInstance inst;
  inst.m_compiler = this;
  inst.m_path = relPath;
  inst.m_source = readFile(m_kernelDir + "/" + relPath);
  // A kernel's identity covers the headers it can see, not every header of the directory: a change to the
  // convolution headers leaves the cached code objects of the bandwidth kernels valid.
  {
    std::vector<std::string> seen, todo = includedHeaders(inst.m_source);
    while (!todo.empty()) {
      const std::string h = todo.back();
      todo.pop_back();
      auto it = m_headerText.find(h);
      if (it == m_headerText.end() || std::find(seen.begin(), seen.end(), h) != seen.end()) continue;
      seen.push_back(h);
      for (const auto &n : includedHeaders(it->second)) todo.push_back(n);
    }
    std::sort(seen.begin(), seen.end());
    for (const auto &h : seen) inst.m_headers += "//" + h + "\n" + m_headerText.at(h);
  }
  // Experiment hook: extra "NAME=value NAME=value" definitions for every kernel (they take
  // part in the hash, so such code objects never mix with regular ones).
  if (const char *extra = std::getenv("DENOX_HIP_EXTRA_DEFINES")) {
    std::istringstream ss(extra);
    std::string kv;
    while (ss >> kv) {
      const size_t eq = kv.find('=');
      inst.define(eq == std::string::npos ? kv : kv.substr(0, eq), eq == std::string::npos ? std::string("1") : kv.substr(eq + 1));
    }
  }
  return inst;
}

std::string HipCompilerInstance::defineString() const {
  std::string s;
  for (const auto &[k, v] : m_defines) {
    if (!s.empty()) s += ' ';
    s += k + "=" + v;
  }
  return s;
}

std::string HipCompilerInstance::sha256() const {
  Sha256 h;
  h.update(m_source);
  h.update(std::string("\n//headers\n"));
  h.update(m_headers);
  h.update(std::string("\n//defines\n"));
  h.update(defineString());
  h.update(std::string("\n//flags\n"));
  for (const char *f : kFlags) h.update(std::string(f) + " ");
  h.update(m_compiler->m_arch);
  return Sha256::hex(h.digest());
}

std::vector<uint8_t> HipCompilerInstance::compile() const {
  const std::string key = sha256();
  const std::string cachePath = m_compiler->m_cacheDir.empty() ? "" : m_compiler->m_cacheDir + "/" + key + ".hsaco";
  if (!cachePath.empty()) {
    std::ifstream f(cachePath, std::ios::binary);
    if (f) {
      std::vector<uint8_t> code((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
      if (!code.empty()) {
        ++m_compiler->m_cacheHits;
        utimensat(AT_FDCWD, cachePath.c_str(), nullptr, 0); // modification time = last use: entries no source produces any more age out
        return code;
      }
    }
  }
  hiprtcProgram prog;
  if (hiprtcCreateProgram(&prog, m_source.c_str(), m_path.c_str(), 0, nullptr, nullptr) != HIPRTC_SUCCESS)
    fail(Status::HipError, "hiprtcCreateProgram failed for " + m_path);
  std::vector<std::string> opts;
  opts.push_back("--offload-arch=" + m_compiler->m_arch);
  for (const char *f : kFlags) opts.push_back(f);
  opts.push_back("-I" + m_compiler->m_kernelDir);
  for (const auto &[k, v] : m_defines) opts.push_back("-D" + k + "=" + v);
  std::vector<const char *> copts;
  for (const auto &o : opts) copts.push_back(o.c_str());
  const hiprtcResult rc = hiprtcCompileProgram(prog, static_cast<int>(copts.size()), copts.data());
  if (rc != HIPRTC_SUCCESS) {
    size_t n = 0;
    hiprtcGetProgramLogSize(prog, &n);
    std::string log(n, '\0');
    if (n) hiprtcGetProgramLog(prog, log.data());
    hiprtcDestroyProgram(&prog);
    fail(Status::CompileError, "hiprtc failed for " + m_path + " [" + defineString() + "]: " + hiprtcGetErrorString(rc) + "\n" + log);
  }
  size_t size = 0;
  hiprtcGetCodeSize(prog, &size);
  std::vector<uint8_t> code(size);
  hiprtcGetCode(prog, reinterpret_cast<char *>(code.data()));
  hiprtcDestroyProgram(&prog);
  ++m_compiler->m_compiled;
  if (!cachePath.empty()) { // temp file + rename: concurrent compilers never see a partial file
    const std::string tmp = cachePath + ".tmp." + std::to_string(getpid());
    std::ofstream f(tmp, std::ios::binary);
    if (f) {
      f.write(reinterpret_cast<const char *>(code.data()), static_cast<std::streamsize>(code.size()));
      f.close();
      if (f && std::rename(tmp.c_str(), cachePath.c_str()) != 0) std::remove(tmp.c_str());
    }
  }
  return code;
}

} // namespace denox::hip
