// Kernel-source compiler: HIP source + preprocessor definitions -> gfx950 code
// object, through hiprtc, with a content-addressed disk cache.
//
// Takes the place of the reference's GLSL front end
//   spirv/src/denox/glsl/GlslCompiler.hpp / GlslCompilerInstance.hpp:18-81
// (read(path) -> instance; define(name, value); compile(); fast_sha256()) and of
// the SPIR-V cache keyed by source hash in
//   compiler/src/denox/compiler/compile_shaders/compile_shaders.cpp:35-48,80-83.
#pragma once
#include <atomic>
#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <utility>
#include <vector>

namespace denox::hip {

class HipCompiler;

class HipCompilerInstance {
public:
  void define(const std::string &name, const std::string &value) { m_defines[name] = value; }
  void define(const std::string &name, long long value) { m_defines[name] = std::to_string(value); }
  const std::string &sourcePath() const { return m_path; }
  // SHA-256 over source, included headers, definitions and compiler flags:
  // identifies the code object (database key and cache file name).
  std::string sha256() const;
  // "NAME=value NAME=value": human-readable variant description
  std::string defineString() const;
  // Compile (or fetch from the cache).  Throws Error(CompileError) with the log.
  std::vector<uint8_t> compile() const;

private:
  friend class HipCompiler;
  const HipCompiler *m_compiler = nullptr;
  std::string m_path;   // path of the kernel source, relative to the kernel directory
  std::string m_source; // its text
  std::string m_headers; // names and text of the kernel-directory headers it includes, directly or through them
  std::map<std::string, std::string> m_defines;
};

class HipCompiler {
public:
  // kernelDir: directory holding the *.hip kernel sources and their headers.
  // cacheDir: where code objects are cached ("" disables the disk cache).
  HipCompiler(std::string kernelDir, std::string cacheDir, std::string arch = "gfx950");
  HipCompilerInstance read(const std::string &relPath) const;
  const std::string &kernelDir() const { return m_kernelDir; }
  const std::string &arch() const { return m_arch; }

  struct Stats { uint64_t compiled = 0, cacheHits = 0; };
  Stats stats() const { return Stats{m_compiled.load(), m_cacheHits.load()}; }

private:
  friend class HipCompilerInstance;
  std::string m_kernelDir, m_cacheDir, m_arch;
  std::map<std::string, std::string> m_headerText; // every *.h in the kernel directory
  mutable std::atomic<uint64_t> m_compiled{0}, m_cacheHits{0};
};

// Directory of the shared library this code is linked into (for default paths).
std::string libraryDirectory();
std::string defaultKernelDir();
std::string defaultCacheDir();

} // namespace denox::hip
