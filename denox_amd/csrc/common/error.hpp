// Error type of the host library.  Exceptions never cross the C ABI: the entry
// points in capi.cpp catch them and turn them into status codes plus a
// thread-local message (the reference throws std::runtime_error /
// diag::invalid_state straight at its callers, e.g. runtime/src/denox/runtime/context.hpp:79-82).
#pragma once
#include <stdexcept>
#include <string>

namespace denox {

enum class Status : int {
  Ok = 0,
  InvalidArgument = 1,
  InvalidModel = 2,   // corrupt / truncated / inconsistent IR
  HipError = 3,       // a HIP runtime or hiprtc call failed
  CompileError = 4,   // kernel source failed to compile
  Unsupported = 5,    // graph uses something no kernel implements
  IoError = 6,
  Internal = 7,
};

class Error : public std::runtime_error {
public:
  Error(Status s, const std::string &msg) : std::runtime_error(msg), status(s) {}
  Status status;
};

[[noreturn]] inline void fail(Status s, const std::string &msg) { throw Error(s, msg); }

} // namespace denox
