#include "sym.hpp"
#include <algorithm>

namespace denox {

std::vector<int64_t> SymIR::eval(const std::vector<int64_t> &vars) const {
  // common/src/denox/symbolic/SymIR.cpp:5-95 with the wire decode of
  // runtime/src/denox/runtime/model.cpp:395-487 folded in.
  std::vector<int64_t> dp(varCount + ops.size(), 0);
  for (size_t i = 0; i < varCount && i < vars.size(); ++i) dp[i] = vars[i];
  for (size_t pc = 0; pc < ops.size(); ++pc) {
    const SymIROp &o = ops[pc];
    const bool lc = (o.opcode & SYM_LHSC) != 0, rc = (o.opcode & SYM_RHSC) != 0;
    const uint16_t base = o.opcode & 0x3FFF;
    const size_t limit = varCount + pc;
    if (lc && rc) fail(Status::InvalidModel, "SymIR op with two constant operands");
    if (!lc && (o.lhs < 0 || static_cast<size_t>(o.lhs) >= limit)) fail(Status::InvalidModel, "SymIR lhs out of range");
    if (!rc && (o.rhs < 0 || static_cast<size_t>(o.rhs) >= limit)) fail(Status::InvalidModel, "SymIR rhs out of range");
    const int64_t a = lc ? o.lhs : dp[static_cast<size_t>(o.lhs)];
    const int64_t b = rc ? o.rhs : dp[static_cast<size_t>(o.rhs)];
    int64_t v = 0;
    switch (base) {
    case SYM_ADD: v = a + b; break;
    case SYM_SUB: v = a - b; break;
    case SYM_MUL: v = a * b; break;
    case SYM_DIV:
      if (b == 0) fail(Status::InvalidArgument, "SymIR division by zero");
      v = a / b;
      break;
    case SYM_MOD:
      if (b == 0) fail(Status::InvalidArgument, "SymIR modulo by zero");
      v = a % b;
      if (v < 0) v += b;
      break;
    case SYM_MIN: v = std::min(a, b); break;
    case SYM_MAX: v = std::max(a, b); break;
    default: fail(Status::InvalidModel, "SymIR unknown opcode");
    }
    dp[limit] = v;
  }
  return dp;
}

Sym SymGraph::var(const std::string &name) {
  for (size_t i = 0; i < m_vars.size(); ++i)
    if (m_vars[i] == name) return Sym::Ref(static_cast<int64_t>(i));
  if (m_vars.size() >= kMaxVars) fail(Status::InvalidArgument, "too many symbolic variables (limit " + std::to_string(kMaxVars) + ")");
  m_vars.push_back(name);
  return Sym::Ref(static_cast<int64_t>(m_vars.size() - 1));
}

static int64_t fold(uint16_t base, int64_t a, int64_t b) {
  switch (base) {
  case SYM_ADD: return a + b;
  case SYM_SUB: return a - b;
  case SYM_MUL: return a * b;
  case SYM_DIV: if (b == 0) fail(Status::InvalidArgument, "division by zero"); return a / b;
  case SYM_MOD: { if (b == 0) fail(Status::InvalidArgument, "modulo by zero"); int64_t v = a % b; return v < 0 ? v + b : v; }
  case SYM_MIN: return std::min(a, b);
  case SYM_MAX: return std::max(a, b);
  default: fail(Status::Internal, "bad sym op");
  }
}

Sym SymGraph::op(uint16_t base, Sym a, Sym b) {
  if (a.isConst() && b.isConst()) return Sym::Const(fold(base, a.v, b.v));
  // identities that keep the program short
  if (base == SYM_ADD) { if (a.isConst() && a.v == 0) return b; if (b.isConst() && b.v == 0) return a; }
  if (base == SYM_SUB) { if (b.isConst() && b.v == 0) return a; if (a == b) return Sym::Const(0); }
  if (base == SYM_MUL) {
    if (a.isConst() && a.v == 1) return b;
    if (b.isConst() && b.v == 1) return a;
    if ((a.isConst() && a.v == 0) || (b.isConst() && b.v == 0)) return Sym::Const(0);
  }
  if (base == SYM_DIV && b.isConst() && b.v == 1) return a;
  if (base == SYM_MOD && b.isConst() && b.v == 1) return Sym::Const(0);
  if ((base == SYM_MIN || base == SYM_MAX) && a == b) return a;
  const bool commutative = base == SYM_ADD || base == SYM_MUL || base == SYM_MIN || base == SYM_MAX;
  if (commutative && b < a) std::swap(a, b); // canonical order: constants first
  auto key = std::make_tuple(base, a, b);
  auto it = m_cse.find(key);
  if (it != m_cse.end()) return Sym::Ref(it->second);
  m_nodes.push_back(Node{base, a, b});
  const int64_t id = static_cast<int64_t>(kMaxVars + m_nodes.size() - 1);
  m_cse.emplace(key, id);
  return Sym::Ref(id);
}

SymIR SymGraph::compile() const {
  SymIR ir;
  ir.varCount = static_cast<uint32_t>(kMaxVars);
  ir.ops.reserve(m_nodes.size());
  for (const Node &n : m_nodes) {
    uint16_t oc = n.base;
    if (n.a.isConst()) oc |= SYM_LHSC;
    if (n.b.isConst()) oc |= SYM_RHSC;
    ir.ops.push_back(SymIROp{oc, n.a.v, n.b.v});
  }
  return ir;
}

} // namespace denox
