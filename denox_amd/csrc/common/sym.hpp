// Symbolic integers for dynamic image extents.
//
// The reference carries every extent, workgroup count, push constant and byte
// size as a `Sym` (constant or symbol) inside a `SymGraph`, simplifies with an
// affine/mod solver and finally lowers the live symbols to a straight-line
// int64 program, `SymIR` (common/src/denox/symbolic/SymIR.hpp:10-70,
// SymIR.cpp:5-95; wire form dnx.fbs:121-149).  Only SymIR crosses the
// compiler/runtime boundary, so this build keeps the builder small: a
// hash-consed expression DAG with constant folding and the obvious identities,
// which *is* already a straight-line program.
#pragma once
#include "error.hpp"
#include <cstdint>
#include <map>
#include <string>
#include <tuple>
#include <vector>

namespace denox {

// Wire opcodes (dnx.fbs:121-138).
enum SymOp : uint16_t {
  SYM_NOP = 0, SYM_ADD = 1, SYM_SUB = 2, SYM_MUL = 3, SYM_DIV = 4,
  SYM_MOD = 5, SYM_MIN = 6, SYM_MAX = 7,
  SYM_LHSC = 0x8000, SYM_RHSC = 0x4000,
};

struct Sym {
  bool symbolic = false;
  int64_t v = 0; // constant value, or index into the value table
  static Sym Const(int64_t c) { return Sym{false, c}; }
  static Sym Ref(int64_t id) { return Sym{true, id}; }
  bool isConst() const { return !symbolic; }
  bool operator==(const Sym &o) const { return symbolic == o.symbolic && v == o.v; }
  bool operator<(const Sym &o) const { return std::tie(symbolic, v) < std::tie(o.symbolic, o.v); }
};

struct SymIROp {
  uint16_t opcode; // base | LHSC | RHSC
  int64_t lhs, rhs;
};

struct SymIR {
  uint32_t varCount = 0;
  std::vector<SymIROp> ops;
  // Evaluate the whole table: dp[0..varCount) are the variables.
  std::vector<int64_t> eval(const std::vector<int64_t> &vars) const;
};

inline int64_t symValue(const std::vector<int64_t> &dp, Sym s) {
  if (!s.symbolic) return s.v;
  if (s.v < 0 || static_cast<size_t>(s.v) >= dp.size()) fail(Status::InvalidModel, "symbol index out of range");
  return dp[static_cast<size_t>(s.v)];
}

class SymGraph {
public:
  Sym var(const std::string &name);            // create or look up a free variable
  const std::vector<std::string> &varNames() const { return m_vars; }

  Sym add(Sym a, Sym b) { return op(SYM_ADD, a, b); }
  Sym sub(Sym a, Sym b) { return op(SYM_SUB, a, b); }
  Sym mul(Sym a, Sym b) { return op(SYM_MUL, a, b); }
  Sym div(Sym a, Sym b) { return op(SYM_DIV, a, b); }
  Sym mod(Sym a, Sym b) { return op(SYM_MOD, a, b); }
  Sym min(Sym a, Sym b) { return op(SYM_MIN, a, b); }
  Sym max(Sym a, Sym b) { return op(SYM_MAX, a, b); }
  Sym add(Sym a, int64_t b) { return add(a, Sym::Const(b)); }
  Sym sub(Sym a, int64_t b) { return sub(a, Sym::Const(b)); }
  Sym mul(Sym a, int64_t b) { return mul(a, Sym::Const(b)); }
  Sym div(Sym a, int64_t b) { return div(a, Sym::Const(b)); }
  Sym mod(Sym a, int64_t b) { return mod(a, Sym::Const(b)); }
  Sym cdiv(Sym a, int64_t b) { return div(add(a, b - 1), b); }
  // (a + align-1)/align*align
  Sym alignUp(Sym a, int64_t align) { return mul(cdiv(a, align), align); }
  // output extent of a sliding window: (x + 2p - d(k-1) - 1)/s + 1
  Sym pool(Sym x, int64_t k, int64_t p, int64_t s, int64_t d) {
    return add(div(add(x, 2 * p - d * (k - 1) - 1), s), 1);
  }
  Sym op(uint16_t base, Sym a, Sym b);

  // The value table reserves kMaxVars leading slots for variables so that a
  // variable may be declared after expressions exist; unused slots stay zero.
  static constexpr size_t kMaxVars = 8;
  SymIR compile() const;
  // value table for concrete variable values, for compile-time estimates
  std::vector<int64_t> eval(const std::vector<int64_t> &vars) const { return compile().eval(vars); }
  size_t varCount() const { return m_vars.size(); }

private:
  struct Node { uint16_t base; Sym a, b; };
  std::vector<std::string> m_vars;
  std::vector<Node> m_nodes;
  std::map<std::tuple<uint16_t, Sym, Sym>, int64_t> m_cse;
};

} // namespace denox
