#include "onnx_import.hpp"
#include "../common/error.hpp"
#include "../common/f16.hpp"
#include <algorithm>
#include <cmath>
#include <cstring>
#include <functional>
#include <limits>
#include <map>
#include <optional>
#include <string>
#include <vector>

namespace denox::onnx {
namespace {

using compiler::Model;
using compiler::TensorHandle;

[[noreturn]] void bad(const std::string &msg) { fail(Status::InvalidModel, "ONNX import: " + msg); }
[[noreturn]] void unsupported(const std::string &msg) { fail(Status::Unsupported, "ONNX import: " + msg); }

// ------------------------------------------------------------------ protobuf wire format
struct Pb {
  const uint8_t *p, *end;
  bool done() const { return p >= end; }
  uint64_t varint() {
    uint64_t r = 0;
    for (int shift = 0; shift < 64; shift += 7) {
      if (p >= end) bad("truncated varint");
      const uint8_t c = *p++;
      r |= static_cast<uint64_t>(c & 0x7F) << shift;
      if (!(c & 0x80)) return r;
    }
    bad("varint longer than 10 bytes");
  }
  // next field header; the payload is then read with one of the calls below
  void key(uint32_t &field, uint32_t &wire) {
    const uint64_t k = varint();
    field = static_cast<uint32_t>(k >> 3);
    wire = static_cast<uint32_t>(k & 7);
    if (field == 0) bad("field number 0");
  }
  Pb bytes() {
    const uint64_t n = varint();
    if (n > static_cast<uint64_t>(end - p)) bad("length-delimited field runs past the end");
    Pb sub{p, p + n};
    p += n;
    return sub;
  }
  std::string str() {
    Pb b = bytes();
    return std::string(reinterpret_cast<const char *>(b.p), static_cast<size_t>(b.end - b.p));
  }
  uint32_t fixed32() {
    if (end - p < 4) bad("truncated fixed32");
    uint32_t v;
    std::memcpy(&v, p, 4);
    p += 4;
    return v;
  }
  uint64_t fixed64() {
    if (end - p < 8) bad("truncated fixed64");
    uint64_t v;
    std::memcpy(&v, p, 8);
    p += 8;
    return v;
  }
  void skip(uint32_t wire) {
    switch (wire) {
    case 0: (void)varint(); break;
    case 1: (void)fixed64(); break;
    case 2: (void)bytes(); break;
    case 5: (void)fixed32(); break;
    default: bad("unsupported wire type " + std::to_string(wire));
    }
  }
};

float asFloat(uint32_t bits) { float f; std::memcpy(&f, &bits, 4); return f; }
double asDouble(uint64_t bits) { double d; std::memcpy(&d, &bits, 8); return d; }

// repeated scalar fields come packed (wire 2) or one by one
void readInts(Pb &pb, uint32_t wire, std::vector<int64_t> &out) {
  if (wire == 2) {
    Pb b = pb.bytes();
    while (!b.done()) out.push_back(static_cast<int64_t>(b.varint()));
  } else if (wire == 0) {
    out.push_back(static_cast<int64_t>(pb.varint()));
  } else {
    bad("integer field with wire type " + std::to_string(wire));
  }
}
void readFloats(Pb &pb, uint32_t wire, std::vector<float> &out) {
  if (wire == 2) {
    Pb b = pb.bytes();
    while (!b.done()) out.push_back(asFloat(b.fixed32()));
  } else if (wire == 5) {
    out.push_back(asFloat(pb.fixed32()));
  } else {
    bad("float field with wire type " + std::to_string(wire));
  }
}
void readDoubles(Pb &pb, uint32_t wire, std::vector<double> &out) {
  if (wire == 2) {
    Pb b = pb.bytes();
    while (!b.done()) out.push_back(asDouble(b.fixed64()));
  } else if (wire == 1) {
    out.push_back(asDouble(pb.fixed64()));
  } else {
    bad("double field with wire type " + std::to_string(wire));
  }
}

// ------------------------------------------------------------------ ONNX messages (the parts used)
enum DType { DT_FLOAT = 1, DT_UINT8 = 2, DT_INT8 = 3, DT_INT32 = 6, DT_INT64 = 7, DT_BOOL = 9, DT_FLOAT16 = 10, DT_DOUBLE = 11 };

struct TensorProto {
  std::vector<int64_t> dims;
  int dtype = 0;
  std::string name;
  const uint8_t *raw = nullptr;
  size_t rawSize = 0;
  std::vector<float> floatData;
  std::vector<int64_t> int32Data, int64Data;
  std::vector<double> doubleData;
  bool external = false;
};

TensorProto parseTensor(Pb pb) {
  TensorProto t;
  while (!pb.done()) {
    uint32_t f, w;
    pb.key(f, w);
    switch (f) {
    case 1: readInts(pb, w, t.dims); break;
    case 2: t.dtype = static_cast<int>(pb.varint()); break;
    case 4: readFloats(pb, w, t.floatData); break;
    case 5: readInts(pb, w, t.int32Data); break;
    case 7: readInts(pb, w, t.int64Data); break;
    case 8: t.name = pb.str(); break;
    case 9: { Pb b = pb.bytes(); t.raw = b.p; t.rawSize = static_cast<size_t>(b.end - b.p); break; }
    case 10: readDoubles(pb, w, t.doubleData); break;
    case 13: t.external = true; pb.skip(w); break;
    case 14: if (pb.varint() == 1) t.external = true; break;
    default: pb.skip(w);
    }
  }
  return t;
}

struct Attr {
  std::string name;
  int type = 0; // 1 FLOAT, 2 INT, 3 STRING, 4 TENSOR, 6 FLOATS, 7 INTS
  float f = 0;
  int64_t i = 0;
  std::string s;
  TensorProto t;
  bool hasT = false, hasF = false, hasI = false, hasS = false;
  std::vector<float> floats;
  std::vector<int64_t> ints;
};

Attr parseAttr(Pb pb) {
  Attr a;
  while (!pb.done()) {
    uint32_t f, w;
    pb.key(f, w);
    switch (f) {
    case 1: a.name = pb.str(); break;
    case 2: a.f = asFloat(pb.fixed32()); a.hasF = true; break;
    case 3: a.i = static_cast<int64_t>(pb.varint()); a.hasI = true; break;
    case 4: a.s = pb.str(); a.hasS = true; break;
    case 5: a.t = parseTensor(pb.bytes()); a.hasT = true; break;
    case 6: unsupported("graph-valued attribute '" + a.name + "'");
    case 7: readFloats(pb, w, a.floats); break;
    case 8: readInts(pb, w, a.ints); break;
    case 20: a.type = static_cast<int>(pb.varint()); break;
    default: pb.skip(w);
    }
  }
  return a;
}

struct Node {
  std::vector<std::string> in, out;
  std::string name, op, domain;
  std::vector<Attr> attrs;
  const Attr *attr(const char *n) const {
    for (const auto &a : attrs) if (a.name == n) return &a;
    return nullptr;
  }
  int64_t intAttr(const char *n, int64_t dflt) const { const Attr *a = attr(n); return a ? a->i : dflt; }
  float floatAttr(const char *n, float dflt) const { const Attr *a = attr(n); return a ? a->f : dflt; }
  std::string strAttr(const char *n, const char *dflt) const { const Attr *a = attr(n); return a ? a->s : std::string(dflt); }
  std::vector<int64_t> intsAttr(const char *n) const { const Attr *a = attr(n); return a ? a->ints : std::vector<int64_t>{}; }
};

Node parseNode(Pb pb) {
  Node n;
  while (!pb.done()) {
    uint32_t f, w;
    pb.key(f, w);
    switch (f) {
    case 1: n.in.push_back(pb.str()); break;
    case 2: n.out.push_back(pb.str()); break;
    case 3: n.name = pb.str(); break;
    case 4: n.op = pb.str(); break;
    case 5: n.attrs.push_back(parseAttr(pb.bytes())); break;
    case 7: n.domain = pb.str(); break;
    default: pb.skip(w);
    }
  }
  return n;
}

struct Dim { bool hasValue = false, hasParam = false; int64_t value = 0; std::string param; };
struct ValueInfo { std::string name; int elemType = 0; bool hasShape = false; std::vector<Dim> dims; };

ValueInfo parseValueInfo(Pb pb) {
  ValueInfo v;
  while (!pb.done()) {
    uint32_t f, w;
    pb.key(f, w);
    if (f == 1) { v.name = pb.str(); continue; }
    if (f != 2) { pb.skip(w); continue; }
    Pb type = pb.bytes();
    while (!type.done()) {
      uint32_t tf, tw;
      type.key(tf, tw);
      if (tf != 1) { type.skip(tw); continue; } // only tensor types
      Pb tt = type.bytes();
      while (!tt.done()) {
        uint32_t f3, w3;
        tt.key(f3, w3);
        if (f3 == 1) { v.elemType = static_cast<int>(tt.varint()); continue; }
        if (f3 != 2) { tt.skip(w3); continue; }
        v.hasShape = true;
        Pb shape = tt.bytes();
        while (!shape.done()) {
          uint32_t f4, w4;
          shape.key(f4, w4);
          if (f4 != 1) { shape.skip(w4); continue; }
          Pb dim = shape.bytes();
          Dim d;
          while (!dim.done()) {
            uint32_t f5, w5;
            dim.key(f5, w5);
            if (f5 == 1) { d.value = static_cast<int64_t>(dim.varint()); d.hasValue = true; }
            else if (f5 == 2) { d.param = dim.str(); d.hasParam = true; }
            else dim.skip(w5);
          }
          v.dims.push_back(d);
        }
      }
    }
  }
  return v;
}

// ------------------------------------------------------------------ values
// A host tensor: a small dense array evaluated at import time.  Integer elements are symbolic integers of the
// model (constants or expressions over the dynamic extents), floating elements are constants.
struct HostTensor {
  std::vector<int64_t> shape;
  bool isFloat = false;
  std::vector<Sym> iv;
  std::vector<double> fv;
  size_t count() const { size_t n = 1; for (auto d : shape) n *= static_cast<size_t>(d); return n; }
  size_t size() const { return isFloat ? fv.size() : iv.size(); }
};

struct Value {
  bool isDevice = false;
  TensorHandle dev = -1;
  // An image tensor may be a crop of `dev` that has not been turned into a layer yet: exporters slice one axis per
  // node, and consecutive crops become one Slice layer when something finally consumes them.
  bool cropped = false;
  Sym left, right, top, bottom; // half-open ranges in `dev`
  HostTensor host;
};

std::vector<size_t> stridesOf(const std::vector<int64_t> &shape) {
  std::vector<size_t> st(shape.size(), 1);
  for (int i = static_cast<int>(shape.size()) - 2; i >= 0; --i) st[i] = st[i + 1] * static_cast<size_t>(shape[i + 1]);
  return st;
}

constexpr int64_t kBig = int64_t(1) << 40; // ONNX uses INT64_MAX / INT32_MAX for "to the end"

struct Importer {
  Model &model;
  SymGraph &sg;
  std::map<std::string, Value> values;
  int64_t opset = 0;

  explicit Importer(Model &m) : model(m), sg(m.symGraph()) {}

  // ---------------------------------------------------------------- helpers
  static HostTensor fromTensorProto(const TensorProto &t) {
    if (t.external) unsupported("tensor '" + t.name + "' stores its data in an external file");
    HostTensor h;
    h.shape = t.dims;
    for (auto d : h.shape) if (d < 0 || d > (int64_t(1) << 31)) bad("tensor '" + t.name + "' has an invalid dimension");
    const size_t n = h.count();
    if (n > (size_t(1) << 28)) bad("tensor '" + t.name + "' is too large");
    auto rawAs = [&](size_t elem) {
      if (t.rawSize != n * elem) bad("tensor '" + t.name + "': raw_data holds " + std::to_string(t.rawSize) + " bytes, expected " + std::to_string(n * elem));
    };
    switch (t.dtype) {
    case DT_FLOAT:
      h.isFloat = true;
      if (t.raw) { rawAs(4); h.fv.resize(n); for (size_t i = 0; i < n; ++i) { float f; std::memcpy(&f, t.raw + 4 * i, 4); h.fv[i] = f; } }
      else { if (t.floatData.size() != n) bad("tensor '" + t.name + "': float_data count"); h.fv.assign(t.floatData.begin(), t.floatData.end()); }
      break;
    case DT_DOUBLE:
      h.isFloat = true;
      if (t.raw) { rawAs(8); h.fv.resize(n); for (size_t i = 0; i < n; ++i) std::memcpy(&h.fv[i], t.raw + 8 * i, 8); }
      else { if (t.doubleData.size() != n) bad("tensor '" + t.name + "': double_data count"); h.fv = t.doubleData; }
      break;
    case DT_FLOAT16:
      h.isFloat = true;
      h.fv.resize(n);
      if (t.raw) { rawAs(2); for (size_t i = 0; i < n; ++i) { uint16_t b; std::memcpy(&b, t.raw + 2 * i, 2); h.fv[i] = f16_to_f32(b); } }
      else { if (t.int32Data.size() != n) bad("tensor '" + t.name + "': int32_data count"); for (size_t i = 0; i < n; ++i) h.fv[i] = f16_to_f32(static_cast<uint16_t>(t.int32Data[i])); }
      break;
    case DT_INT64:
      h.iv.resize(n);
      if (t.raw) { rawAs(8); for (size_t i = 0; i < n; ++i) { int64_t v; std::memcpy(&v, t.raw + 8 * i, 8); h.iv[i] = Sym::Const(v); } }
      else { if (t.int64Data.size() != n) bad("tensor '" + t.name + "': int64_data count"); for (size_t i = 0; i < n; ++i) h.iv[i] = Sym::Const(t.int64Data[i]); }
      break;
    case DT_INT32:
      h.iv.resize(n);
      if (t.raw) { rawAs(4); for (size_t i = 0; i < n; ++i) { int32_t v; std::memcpy(&v, t.raw + 4 * i, 4); h.iv[i] = Sym::Const(v); } }
      else { if (t.int32Data.size() != n) bad("tensor '" + t.name + "': int32_data count"); for (size_t i = 0; i < n; ++i) h.iv[i] = Sym::Const(static_cast<int32_t>(t.int32Data[i])); }
      break;
    case DT_BOOL: case DT_UINT8: case DT_INT8:
      h.iv.resize(n);
      if (t.raw) { rawAs(1); for (size_t i = 0; i < n; ++i) h.iv[i] = Sym::Const(t.dtype == DT_INT8 ? static_cast<int8_t>(t.raw[i]) : t.raw[i]); }
      else { if (t.int32Data.size() != n) bad("tensor '" + t.name + "': int32_data count"); for (size_t i = 0; i < n; ++i) h.iv[i] = Sym::Const(t.int32Data[i]); }
      break;
    default:
      unsupported("tensor '" + t.name + "' has element type " + std::to_string(t.dtype));
    }
    return h;
  }

  static HostTensor intVector(const std::vector<Sym> &v) {
    HostTensor h;
    h.shape = {static_cast<int64_t>(v.size())};
    h.iv = v;
    return h;
  }

  const Value &get(const Node &n, size_t i) {
    if (i >= n.in.size() || n.in[i].empty()) bad(n.op + " '" + n.name + "' lacks input " + std::to_string(i));
    auto it = values.find(n.in[i]);
    if (it == values.end()) bad(n.op + " '" + n.name + "' reads '" + n.in[i] + "', which nothing produces");
    return it->second;
  }
  bool has(const Node &n, size_t i) const { return i < n.in.size() && !n.in[i].empty(); }
  const HostTensor &host(const Node &n, size_t i) {
    const Value &v = get(n, i);
    if (v.isDevice) unsupported(n.op + " '" + n.name + "': input " + std::to_string(i) + " must be known at import time (it is an image tensor)");
    return v.host;
  }
  TensorHandle materialize(Value &v) {
    if (v.cropped) {
      v.dev = model.slice(v.dev, v.left, v.right, v.top, v.bottom);
      v.cropped = false;
    }
    return v.dev;
  }
  TensorHandle device(const Node &n, size_t i) {
    (void)get(n, i);
    Value &v = values[n.in[i]];
    if (!v.isDevice) unsupported(n.op + " '" + n.name + "': input " + std::to_string(i) + " must be an image tensor");
    return materialize(v);
  }
  std::vector<int64_t> constInts(const Node &n, const HostTensor &h, const char *what) {
    if (h.isFloat) bad(n.op + " '" + n.name + "': " + what + " must be integers");
    std::vector<int64_t> out;
    for (const Sym &s : h.iv) {
      if (!s.isConst()) unsupported(n.op + " '" + n.name + "': " + what + " must be constant");
      out.push_back(s.v);
    }
    return out;
  }
  void setHost(const Node &n, HostTensor h, size_t o = 0) {
    if (h.size() != h.count()) fail(Status::Internal, "ONNX import: host tensor size mismatch in " + n.op);
    Value v;
    v.host = std::move(h);
    values[n.out.at(o)] = std::move(v);
  }
  void setDevice(const Node &n, TensorHandle t) {
    Value v;
    v.isDevice = true;
    v.dev = t;
    values[n.out.at(0)] = std::move(v);
  }
  // NCHW shape of an image tensor as symbolic integers
  std::vector<Sym> deviceShape(TensorHandle t) const {
    const auto &tn = model.tensors()[static_cast<size_t>(t)];
    return {Sym::Const(1), Sym::Const(tn.channels), tn.height, tn.width};
  }
  std::vector<Sym> deviceShape(const Value &v) {
    std::vector<Sym> d = deviceShape(v.dev);
    if (v.cropped) { d[2] = sg.sub(v.bottom, v.top); d[3] = sg.sub(v.right, v.left); }
    return d;
  }
  static int64_t normAxis(const Node &n, int64_t axis, int64_t rank) {
    if (axis < 0) axis += rank;
    if (axis < 0 || axis >= rank) bad(n.op + " '" + n.name + "': axis out of range");
    return axis;
  }

  // ---------------------------------------------------------------- host tensor operations
  // gather elements of `src` by a function output index -> source flat index
  static HostTensor remap(const HostTensor &src, std::vector<int64_t> shape, const std::function<size_t(const std::vector<int64_t> &)> &srcIndex) {
    HostTensor out;
    out.shape = std::move(shape);
    out.isFloat = src.isFloat;
    const size_t n = out.count();
    std::vector<int64_t> idx(out.shape.size(), 0);
    for (size_t k = 0; k < n; ++k) {
      const size_t s = srcIndex(idx);
      if (s >= src.size()) fail(Status::Internal, "ONNX import: host tensor index out of range");
      if (src.isFloat) out.fv.push_back(src.fv[s]); else out.iv.push_back(src.iv[s]);
      for (int d = static_cast<int>(idx.size()) - 1; d >= 0; --d) {
        if (++idx[d] < out.shape[d]) break;
        idx[d] = 0;
      }
    }
    return out;
  }

  Sym intBinary(const Node &n, Sym a, Sym b) {
    const std::string &op = n.op;
    if (op == "Add") return sg.add(a, b);
    if (op == "Sub") return sg.sub(a, b);
    if (op == "Mul") return sg.mul(a, b);
    if (op == "Div") {
      if (b.isConst() && b.v == 0) bad("Div '" + n.name + "': division by zero");
      return sg.div(a, b);
    }
    if (op == "Mod") {
      if (b.isConst() && b.v == 0) bad("Mod '" + n.name + "': division by zero");
      if (a.isConst() && b.isConst()) { // ONNX integer Mod with fmod = 0: the result takes the sign of the divisor
        int64_t r = a.v % b.v;
        if (r != 0 && ((r < 0) != (b.v < 0))) r += b.v;
        return Sym::Const(r);
      }
      return sg.mod(a, b); // extents are non-negative, divisors positive: plain remainder
    }
    if (op == "Min") return sg.min(a, b);
    if (op == "Max") return sg.max(a, b);
    unsupported("integer " + op);
  }
  static double floatBinary(const Node &n, double a, double b) {
    const std::string &op = n.op;
    if (op == "Add") return a + b;
    if (op == "Sub") return a - b;
    if (op == "Mul") return a * b;
    if (op == "Div") return a / b;
    if (op == "Mod") return std::fmod(a, b);
    if (op == "Min") return std::min(a, b);
    if (op == "Max") return std::max(a, b);
    if (op == "Pow") return std::pow(a, b);
    unsupported("floating-point " + op);
  }

  HostTensor toFloat(const Node &n, const HostTensor &h) {
    if (h.isFloat) return h;
    HostTensor f;
    f.shape = h.shape;
    f.isFloat = true;
    for (const Sym &s : h.iv) {
      if (!s.isConst()) unsupported(n.op + " '" + n.name + "': a symbolic integer cannot become a floating-point value");
      f.fv.push_back(static_cast<double>(s.v));
    }
    return f;
  }

  void binary(const Node &n) {
    if (n.in.size() < 2) bad(n.op + " '" + n.name + "' needs two inputs");
    HostTensor acc = host(n, 0);
    for (size_t k = 1; k < n.in.size(); ++k) { // Min / Max are variadic
      HostTensor b = host(n, k);
      if (acc.isFloat != b.isFloat) { acc = toFloat(n, acc); b = toFloat(n, b); }
      // numpy broadcasting
      const size_t rank = std::max(acc.shape.size(), b.shape.size());
      std::vector<int64_t> sa(rank, 1), sb(rank, 1), so(rank);
      std::copy(acc.shape.begin(), acc.shape.end(), sa.begin() + (rank - acc.shape.size()));
      std::copy(b.shape.begin(), b.shape.end(), sb.begin() + (rank - b.shape.size()));
      for (size_t d = 0; d < rank; ++d) {
        if (sa[d] != sb[d] && sa[d] != 1 && sb[d] != 1) bad(n.op + " '" + n.name + "': shapes do not broadcast");
        so[d] = std::max(sa[d], sb[d]);
      }
      const auto sta = stridesOf(sa), stb = stridesOf(sb);
      HostTensor out;
      out.shape = so;
      out.isFloat = acc.isFloat;
      const size_t cnt = out.count();
      std::vector<int64_t> idx(rank, 0);
      for (size_t e = 0; e < cnt; ++e) {
        size_t ia = 0, ib = 0;
        for (size_t d = 0; d < rank; ++d) {
          ia += (sa[d] == 1 ? 0 : static_cast<size_t>(idx[d])) * sta[d];
          ib += (sb[d] == 1 ? 0 : static_cast<size_t>(idx[d])) * stb[d];
        }
        if (out.isFloat) out.fv.push_back(floatBinary(n, acc.fv.at(ia), b.fv.at(ib)));
        else out.iv.push_back(intBinary(n, acc.iv.at(ia), b.iv.at(ib)));
        for (int d = static_cast<int>(rank) - 1; d >= 0; --d) {
          if (++idx[d] < so[d]) break;
          idx[d] = 0;
        }
      }
      acc = std::move(out);
    }
    setHost(n, std::move(acc));
  }

  void unary(const Node &n) {
    HostTensor h = host(n, 0);
    const std::string &op = n.op;
    if (h.isFloat) {
      for (double &v : h.fv) {
        if (op == "Neg") v = -v;
        else if (op == "Abs") v = std::fabs(v);
        else if (op == "Floor") v = std::floor(v);
        else if (op == "Ceil") v = std::ceil(v);
        else if (op == "Round") v = std::nearbyint(v); // ties to even
        else if (op == "Sqrt") v = std::sqrt(v);
        else if (op == "Reciprocal") v = 1.0 / v;
        else if (op == "Sign") v = (v > 0) - (v < 0);
        else unsupported(op);
      }
    } else {
      for (Sym &s : h.iv) {
        if (op == "Neg") s = sg.sub(Sym::Const(0), s);
        else if (op == "Abs") s = s.isConst() ? Sym::Const(std::llabs(s.v)) : sg.max(s, sg.sub(Sym::Const(0), s));
        else if (op == "Floor" || op == "Ceil" || op == "Round") {}
        else if (op == "Sign") { if (!s.isConst()) unsupported("Sign of a symbolic integer"); s = Sym::Const((s.v > 0) - (s.v < 0)); }
        else unsupported("integer " + op);
      }
    }
    setHost(n, std::move(h));
  }

  // Clip(X, [min], [max]) on a host tensor (details/ops/clip.cpp of the reference handles host tensors only, too);
  // before opset 11 the bounds are the attributes `min` / `max`.
  void opClip(const Node &n) {
    HostTensor h = host(n, 0);
    auto bound = [&](size_t input, const char *attr, bool &present) -> HostTensor {
      HostTensor b;
      present = false;
      if (has(n, input)) {
        b = host(n, input);
        if (b.count() != 1) bad("Clip '" + n.name + "': bounds must be scalars");
        present = true;
      } else if (const Attr *a = n.attr(attr)) {
        b.isFloat = true;
        b.fv = {static_cast<double>(a->f)};
        present = true;
      }
      return b;
    };
    bool hasLo = false, hasHi = false;
    HostTensor lo = bound(1, "min", hasLo), hi = bound(2, "max", hasHi);
    if (h.isFloat) {
      if (hasLo) lo = toFloat(n, lo);
      if (hasHi) hi = toFloat(n, hi);
      for (double &v : h.fv) {
        if (hasLo) v = std::max(v, lo.fv[0]);
        if (hasHi) v = std::min(v, hi.fv[0]);
      }
    } else {
      auto asInt = [&](const HostTensor &b) -> Sym {
        if (!b.isFloat) return b.iv[0];
        if (b.fv[0] != std::floor(b.fv[0]) || std::fabs(b.fv[0]) > 9e15) unsupported("Clip '" + n.name + "': fractional bound on an integer tensor");
        return Sym::Const(static_cast<int64_t>(b.fv[0]));
      };
      for (Sym &s : h.iv) {
        if (hasLo) s = sg.max(s, asInt(lo));
        if (hasHi) s = sg.min(s, asInt(hi));
      }
    }
    setHost(n, std::move(h));
  }

  void opConstant(const Node &n) {
    HostTensor h;
    if (const Attr *a = n.attr("value")) {
      if (!a->hasT) bad("Constant '" + n.name + "': attribute 'value' is no tensor");
      h = fromTensorProto(a->t);
    } else if (const Attr *a = n.attr("value_int")) {
      h.iv = {Sym::Const(a->i)};
    } else if (const Attr *a = n.attr("value_ints")) {
      h.shape = {static_cast<int64_t>(a->ints.size())};
      for (auto v : a->ints) h.iv.push_back(Sym::Const(v));
    } else if (const Attr *a = n.attr("value_float")) {
      h.isFloat = true;
      h.fv = {a->f};
    } else if (const Attr *a = n.attr("value_floats")) {
      h.isFloat = true;
      h.shape = {static_cast<int64_t>(a->floats.size())};
      h.fv.assign(a->floats.begin(), a->floats.end());
    } else {
      unsupported("Constant '" + n.name + "' without a value / value_int(s) / value_float(s) attribute");
    }
    setHost(n, std::move(h));
  }

  void opShape(const Node &n) {
    const Value &v = get(n, 0);
    std::vector<Sym> dims;
    if (v.isDevice) dims = deviceShape(v);
    else for (auto d : v.host.shape) dims.push_back(Sym::Const(d));
    const int64_t rank = static_cast<int64_t>(dims.size());
    int64_t start = n.intAttr("start", 0), end = n.attr("end") ? n.intAttr("end", rank) : rank;
    if (start < 0) start += rank;
    if (end < 0) end += rank;
    start = std::clamp<int64_t>(start, 0, rank);
    end = std::clamp<int64_t>(end, start, rank);
    setHost(n, intVector(std::vector<Sym>(dims.begin() + start, dims.begin() + end)));
  }

  void opGather(const Node &n) {
    const HostTensor &data = host(n, 0);
    const HostTensor &ind = host(n, 1);
    const int64_t rank = static_cast<int64_t>(data.shape.size());
    if (rank == 0) bad("Gather '" + n.name + "': data is a scalar");
    const int64_t axis = normAxis(n, n.intAttr("axis", 0), rank);
    const std::vector<int64_t> indices = constInts(n, ind, "indices");
    // out shape = data.shape[:axis] + indices.shape + data.shape[axis+1:]
    std::vector<int64_t> oshape(data.shape.begin(), data.shape.begin() + axis);
    oshape.insert(oshape.end(), ind.shape.begin(), ind.shape.end());
    oshape.insert(oshape.end(), data.shape.begin() + axis + 1, data.shape.end());
    const auto dst = stridesOf(data.shape);
    const auto ist = stridesOf(ind.shape);
    const size_t q = ind.shape.size();
    setHost(n, remap(data, oshape, [&](const std::vector<int64_t> &o) {
      size_t flatInd = 0;
      for (size_t d = 0; d < q; ++d) flatInd += static_cast<size_t>(o[axis + d]) * ist[d];
      int64_t sel = indices.at(flatInd);
      if (sel < 0) sel += data.shape[axis];
      if (sel < 0 || sel >= data.shape[axis]) bad("Gather '" + n.name + "': index out of range");
      size_t s = static_cast<size_t>(sel) * dst[axis];
      for (int64_t d = 0; d < axis; ++d) s += static_cast<size_t>(o[d]) * dst[d];
      for (int64_t d = axis + 1; d < rank; ++d) s += static_cast<size_t>(o[d - 1 + static_cast<int64_t>(q)]) * dst[d];
      return s;
    }));
  }

  std::vector<int64_t> axesOf(const Node &n, size_t inputIndex) {
    if (has(n, inputIndex)) return constInts(n, host(n, inputIndex), "axes");
    return n.intsAttr("axes");
  }

  void opUnsqueeze(const Node &n) {
    HostTensor h = host(n, 0);
    std::vector<int64_t> axes = axesOf(n, 1);
    const int64_t rank = static_cast<int64_t>(h.shape.size() + axes.size());
    for (auto &a : axes) a = normAxis(n, a, rank);
    std::sort(axes.begin(), axes.end());
    for (auto a : axes) h.shape.insert(h.shape.begin() + a, 1);
    setHost(n, std::move(h));
  }

  void opSqueeze(const Node &n) {
    HostTensor h = host(n, 0);
    std::vector<int64_t> axes = axesOf(n, 1);
    const int64_t rank = static_cast<int64_t>(h.shape.size());
    std::vector<int64_t> shape;
    for (int64_t d = 0; d < rank; ++d) {
      bool drop = axes.empty() ? h.shape[d] == 1 : false;
      for (auto a : axes) if (normAxis(n, a, rank) == d) { if (h.shape[d] != 1) bad("Squeeze '" + n.name + "': dimension is not 1"); drop = true; }
      if (!drop) shape.push_back(h.shape[d]);
    }
    h.shape = shape;
    setHost(n, std::move(h));
  }

  void opReshape(const Node &n) {
    HostTensor h = host(n, 0);
    std::vector<int64_t> shape = constInts(n, host(n, 1), "shape");
    const bool allowZero = n.intAttr("allowzero", 0) != 0;
    int64_t known = 1, infer = -1;
    for (size_t d = 0; d < shape.size(); ++d) {
      if (shape[d] == 0 && !allowZero) {
        if (d >= h.shape.size()) bad("Reshape '" + n.name + "': 0 refers to a missing dimension");
        shape[d] = h.shape[d];
      }
      if (shape[d] == -1) { if (infer >= 0) bad("Reshape '" + n.name + "': two -1 dimensions"); infer = static_cast<int64_t>(d); }
      else if (shape[d] < 0) bad("Reshape '" + n.name + "': negative dimension");
      else known *= shape[d];
    }
    const int64_t total = static_cast<int64_t>(h.count());
    if (infer >= 0) {
      if (known == 0 || total % known) bad("Reshape '" + n.name + "': element count does not divide");
      shape[static_cast<size_t>(infer)] = total / known;
    } else if (known != total) {
      bad("Reshape '" + n.name + "': element count changes");
    }
    h.shape = shape;
    setHost(n, std::move(h));
  }

  void opTranspose(const Node &n) {
    const HostTensor &h = host(n, 0);
    const size_t rank = h.shape.size();
    std::vector<int64_t> perm = n.intsAttr("perm");
    if (perm.empty()) for (size_t d = 0; d < rank; ++d) perm.push_back(static_cast<int64_t>(rank - 1 - d));
    if (perm.size() != rank) bad("Transpose '" + n.name + "': perm has the wrong length");
    std::vector<int64_t> oshape(rank);
    for (size_t d = 0; d < rank; ++d) oshape[d] = h.shape.at(static_cast<size_t>(normAxis(n, perm[d], static_cast<int64_t>(rank))));
    const auto st = stridesOf(h.shape);
    setHost(n, remap(h, oshape, [&](const std::vector<int64_t> &o) {
      size_t s = 0;
      for (size_t d = 0; d < rank; ++d) s += static_cast<size_t>(o[d]) * st[static_cast<size_t>(normAxis(n, perm[d], static_cast<int64_t>(rank)))];
      return s;
    }));
  }

  void opCast(const Node &n) {
    const Value &v = get(n, 0);
    const int64_t to = n.intAttr("to", 0);
    if (v.isDevice) { // image tensors are binary16 whatever the file says
      if (to != DT_FLOAT && to != DT_FLOAT16 && to != DT_DOUBLE) unsupported("Cast '" + n.name + "' of an image tensor to a non-floating type");
      values[n.out.at(0)] = v;
      return;
    }
    HostTensor h = v.host;
    const bool toFloatT = to == DT_FLOAT || to == DT_DOUBLE || to == DT_FLOAT16;
    const bool toInt = to == DT_INT64 || to == DT_INT32 || to == DT_UINT8 || to == DT_INT8 || to == DT_BOOL;
    if (!toFloatT && !toInt) unsupported("Cast '" + n.name + "' to element type " + std::to_string(to));
    if (toFloatT && !h.isFloat) h = toFloat(n, h);
    else if (toInt && h.isFloat) {
      HostTensor i;
      i.shape = h.shape;
      for (double d : h.fv) i.iv.push_back(Sym::Const(to == DT_BOOL ? (d != 0) : static_cast<int64_t>(d))); // truncation toward zero
      h = std::move(i);
    }
    setHost(n, std::move(h));
  }

  void opConstantOfShape(const Node &n) {
    const std::vector<int64_t> shape = constInts(n, host(n, 0), "shape");
    HostTensor fill;
    fill.isFloat = true;
    fill.fv = {0.0};
    if (const Attr *a = n.attr("value")) {
      fill = fromTensorProto(a->t);
      if (fill.size() != 1) bad("ConstantOfShape '" + n.name + "': value must hold one element");
    }
    HostTensor h;
    h.shape = shape;
    h.isFloat = fill.isFloat;
    for (auto d : shape) if (d < 0 || d > (1 << 20)) bad("ConstantOfShape '" + n.name + "': invalid shape");
    const size_t cnt = h.count();
    if (cnt > (size_t(1) << 22)) bad("ConstantOfShape '" + n.name + "': too large");
    if (h.isFloat) h.fv.assign(cnt, fill.fv[0]); else h.iv.assign(cnt, fill.iv[0]);
    setHost(n, std::move(h));
  }

  void opExpand(const Node &n) {
    const HostTensor &h = host(n, 0);
    const std::vector<int64_t> target = constInts(n, host(n, 1), "shape");
    const size_t rank = std::max(h.shape.size(), target.size());
    std::vector<int64_t> si(rank, 1), st(rank, 1), so(rank);
    std::copy(h.shape.begin(), h.shape.end(), si.begin() + (rank - h.shape.size()));
    std::copy(target.begin(), target.end(), st.begin() + (rank - target.size()));
    for (size_t d = 0; d < rank; ++d) {
      if (si[d] != st[d] && si[d] != 1 && st[d] != 1) bad("Expand '" + n.name + "': shapes do not broadcast");
      so[d] = std::max(si[d], st[d]);
    }
    const auto strides = stridesOf(si);
    setHost(n, remap(h, so, [&](const std::vector<int64_t> &o) {
      size_t s = 0;
      for (size_t d = 0; d < rank; ++d) s += (si[d] == 1 ? 0 : static_cast<size_t>(o[d])) * strides[d];
      return s;
    }));
  }

  // Slice parameters per axis; INT64_MAX-like ends mean "to the end"
  struct SliceArgs { std::vector<Sym> starts, ends; std::vector<int64_t> axes, steps; };
  SliceArgs sliceArgs(const Node &n, int64_t rank) {
    SliceArgs a;
    if (opset >= 10 || has(n, 1)) {
      const HostTensor &s = host(n, 1), &e = host(n, 2);
      if (s.isFloat || e.isFloat) bad("Slice '" + n.name + "': starts / ends must be integers");
      a.starts = s.iv;
      a.ends = e.iv;
      if (has(n, 3)) a.axes = constInts(n, host(n, 3), "axes");
      if (has(n, 4)) a.steps = constInts(n, host(n, 4), "steps");
    } else {
      for (auto v : n.intsAttr("starts")) a.starts.push_back(Sym::Const(v));
      for (auto v : n.intsAttr("ends")) a.ends.push_back(Sym::Const(v));
      a.axes = n.intsAttr("axes");
    }
    if (a.starts.size() != a.ends.size()) bad("Slice '" + n.name + "': starts and ends differ in length");
    if (a.axes.empty()) for (size_t i = 0; i < a.starts.size(); ++i) a.axes.push_back(static_cast<int64_t>(i));
    if (a.steps.empty()) a.steps.assign(a.starts.size(), 1);
    if (a.axes.size() != a.starts.size() || a.steps.size() != a.starts.size()) bad("Slice '" + n.name + "': axes / steps length");
    for (auto &ax : a.axes) ax = normAxis(n, ax, rank);
    return a;
  }

  void opSlice(const Node &n) {
    const Value &v = get(n, 0);
    if (v.isDevice) {
      const auto dims = deviceShape(v);
      const SliceArgs a = sliceArgs(n, 4);
      Sym lo[4] = {Sym::Const(0), Sym::Const(0), Sym::Const(0), Sym::Const(0)};
      Sym hi[4] = {dims[0], dims[1], dims[2], dims[3]};
      for (size_t k = 0; k < a.axes.size(); ++k) {
        const int64_t ax = a.axes[k];
        if (a.steps[k] != 1) unsupported("Slice '" + n.name + "': step " + std::to_string(a.steps[k]) + " on an image tensor");
        auto bound = [&](Sym s) { // negative constants count from the end, huge ones mean the end
          if (s.isConst()) {
            if (s.v < 0) return sg.add(dims[ax], s.v);
            if (s.v >= kBig) return dims[ax];
            if (dims[ax].isConst()) return Sym::Const(std::min(s.v, dims[ax].v));
          }
          return s;
        };
        lo[ax] = bound(a.starts[k]);
        hi[ax] = bound(a.ends[k]);
      }
      auto whole = [&](int ax) { return lo[ax] == Sym::Const(0) && hi[ax] == dims[ax]; };
      if (!whole(0) || !whole(1)) unsupported("Slice '" + n.name + "': only height and width of an image tensor can be sliced");
      Value out = v;
      if (!(whole(2) && whole(3))) { // compose with a crop that is still pending
        const Sym x0 = v.cropped ? v.left : Sym::Const(0), y0 = v.cropped ? v.top : Sym::Const(0);
        out.cropped = true;
        out.left = sg.add(x0, lo[3]);
        out.right = sg.add(x0, hi[3]);
        out.top = sg.add(y0, lo[2]);
        out.bottom = sg.add(y0, hi[2]);
      }
      values[n.out.at(0)] = std::move(out);
      return;
    }
    const HostTensor &h = v.host;
    const int64_t rank = static_cast<int64_t>(h.shape.size());
    const SliceArgs a = sliceArgs(n, rank);
    std::vector<int64_t> start(rank, 0), step(rank, 1), oshape = h.shape;
    for (size_t k = 0; k < a.axes.size(); ++k) {
      const int64_t ax = a.axes[k], dim = h.shape[ax], st = a.steps[k];
      if (!a.starts[k].isConst() || !a.ends[k].isConst()) unsupported("Slice '" + n.name + "': symbolic bounds on a host tensor");
      if (st == 0) bad("Slice '" + n.name + "': step 0");
      int64_t s = a.starts[k].v, e = a.ends[k].v;
      if (s < 0) s += dim;
      if (e < 0 && e > -kBig) e += dim;
      if (st > 0) { s = std::clamp<int64_t>(s, 0, dim); e = std::clamp<int64_t>(e, 0, dim); }
      else { s = std::clamp<int64_t>(s, 0, dim - 1); e = std::clamp<int64_t>(e, -1, dim - 1); }
      const int64_t cnt = st > 0 ? std::max<int64_t>(0, (e - s + st - 1) / st) : std::max<int64_t>(0, (s - e + (-st) - 1) / (-st));
      start[ax] = s;
      step[ax] = st;
      oshape[ax] = cnt;
    }
    const auto strides = stridesOf(h.shape);
    setHost(n, remap(h, oshape, [&](const std::vector<int64_t> &o) {
      size_t sidx = 0;
      for (int64_t d = 0; d < rank; ++d) sidx += static_cast<size_t>(start[d] + o[d] * step[d]) * strides[d];
      return sidx;
    }));
  }

  void opConcat(const Node &n) {
    if (n.in.empty()) bad("Concat '" + n.name + "' without inputs");
    const bool dev = get(n, 0).isDevice;
    for (size_t i = 0; i < n.in.size(); ++i) if (get(n, i).isDevice != dev) unsupported("Concat '" + n.name + "' mixes image tensors and host tensors");
    if (!n.attr("axis")) bad("Concat '" + n.name + "' lacks the axis attribute");
    if (dev) {
      if (normAxis(n, n.intAttr("axis", 1), 4) != 1) unsupported("Concat '" + n.name + "': image tensors concatenate along channels only");
      TensorHandle acc = device(n, 0);
      for (size_t i = 1; i < n.in.size(); ++i) acc = model.concat(acc, device(n, i));
      setDevice(n, acc);
      return;
    }
    const HostTensor &first = host(n, 0);
    const int64_t rank = static_cast<int64_t>(first.shape.size());
    if (rank == 0) bad("Concat '" + n.name + "' of scalars");
    const int64_t axis = normAxis(n, n.intAttr("axis", 0), rank);
    bool anyFloat = false;
    for (size_t i = 0; i < n.in.size(); ++i) anyFloat |= host(n, i).isFloat;
    std::vector<HostTensor> parts;
    std::vector<int64_t> oshape = first.shape;
    oshape[axis] = 0;
    for (size_t i = 0; i < n.in.size(); ++i) {
      HostTensor p = anyFloat ? toFloat(n, host(n, i)) : host(n, i);
      if (static_cast<int64_t>(p.shape.size()) != rank) bad("Concat '" + n.name + "': ranks differ");
      for (int64_t d = 0; d < rank; ++d) if (d != axis && p.shape[d] != first.shape[d]) bad("Concat '" + n.name + "': shapes differ off the axis");
      oshape[axis] += p.shape[axis];
      parts.push_back(std::move(p));
    }
    HostTensor out;
    out.shape = oshape;
    out.isFloat = anyFloat;
    size_t outer = 1, inner = 1;
    for (int64_t d = 0; d < axis; ++d) outer *= static_cast<size_t>(oshape[d]);
    for (int64_t d = axis + 1; d < rank; ++d) inner *= static_cast<size_t>(oshape[d]);
    for (size_t o = 0; o < outer; ++o)
      for (const HostTensor &p : parts) {
        const size_t len = static_cast<size_t>(p.shape[axis]) * inner;
        for (size_t e = 0; e < len; ++e) {
          if (anyFloat) out.fv.push_back(p.fv.at(o * len + e)); else out.iv.push_back(p.iv.at(o * len + e));
        }
      }
    setHost(n, std::move(out));
  }

  // ---------------------------------------------------------------- layers
  static std::vector<uint16_t> toHalf(const HostTensor &h) {
    std::vector<uint16_t> out(h.fv.size());
    for (size_t i = 0; i < h.fv.size(); ++i) out[i] = f32_to_f16(static_cast<float>(h.fv[i]));
    return out;
  }

  // symmetric [y, x] padding from ONNX pads [top, left, bottom, right] / auto_pad
  void spatialPads(const Node &n, int64_t ky, int64_t kx, int64_t dy, int64_t dx, int64_t sy, int64_t sx, unsigned &py, unsigned &px) {
    const std::string autoPad = n.strAttr("auto_pad", "NOTSET");
    std::vector<int64_t> pads = n.intsAttr("pads");
    if (autoPad == "SAME_UPPER" || autoPad == "SAME_LOWER") {
      if (sy != 1 || sx != 1) unsupported(n.op + " '" + n.name + "': auto_pad SAME with a stride");
      const int64_t ty = dy * (ky - 1), tx = dx * (kx - 1);
      if (ty % 2 || tx % 2) unsupported(n.op + " '" + n.name + "': auto_pad SAME needs an odd kernel extent");
      pads = {ty / 2, tx / 2, ty / 2, tx / 2};
    } else if (autoPad == "VALID") {
      pads = {0, 0, 0, 0};
    } else if (autoPad != "NOTSET") {
      bad(n.op + " '" + n.name + "': unknown auto_pad '" + autoPad + "'");
    }
    if (pads.empty()) pads = {0, 0, 0, 0};
    if (pads.size() != 4) unsupported(n.op + " '" + n.name + "': pads must have 4 entries (2-D)");
    if (pads[0] != pads[2] || pads[1] != pads[3]) unsupported(n.op + " '" + n.name + "': asymmetric padding");
    if (pads[0] < 0 || pads[1] < 0) bad(n.op + " '" + n.name + "': negative padding");
    py = static_cast<unsigned>(pads[0]);
    px = static_cast<unsigned>(pads[1]);
  }

  void opConv(const Node &n) {
    const TensorHandle x = device(n, 0);
    const HostTensor &w = host(n, 1);
    if (!w.isFloat || w.shape.size() != 4) unsupported("Conv '" + n.name + "': the weights must be a constant rank-4 floating-point tensor");
    if (n.intAttr("group", 1) != 1) unsupported("Conv '" + n.name + "': grouped convolution");
    const int64_t K = w.shape[0], C = w.shape[1], R = w.shape[2], S = w.shape[3];
    const auto ks = n.intsAttr("kernel_shape");
    if (!ks.empty() && (ks.size() != 2 || ks[0] != R || ks[1] != S)) bad("Conv '" + n.name + "': kernel_shape contradicts the weights");
    auto two = [&](const char *name) {
      std::vector<int64_t> v = n.intsAttr(name);
      if (v.empty()) v = {1, 1};
      if (v.size() != 2 || v[0] < 1 || v[1] < 1) bad("Conv '" + n.name + "': attribute '" + std::string(name) + "'");
      return v;
    };
    const auto strides = two("strides"), dil = two("dilations");
    unsigned py, px;
    spatialPads(n, R, S, dil[0], dil[1], strides[0], strides[1], py, px);
    if (static_cast<int64_t>(model.tensors()[static_cast<size_t>(x)].channels) != C)
      bad("Conv '" + n.name + "': the input has " + std::to_string(model.tensors()[static_cast<size_t>(x)].channels) + " channels, the weights expect " + std::to_string(C));
    const std::vector<uint16_t> wh = toHalf(w);
    std::vector<uint16_t> bh;
    if (has(n, 2)) {
      const HostTensor &b = host(n, 2);
      if (!b.isFloat || static_cast<int64_t>(b.size()) != K) bad("Conv '" + n.name + "': bias must hold one value per output channel");
      bh = toHalf(b);
    }
    setDevice(n, model.conv2d(x, static_cast<unsigned>(K), static_cast<unsigned>(C), static_cast<unsigned>(R), static_cast<unsigned>(S), wh.data(),
                              bh.empty() ? nullptr : bh.data(), static_cast<unsigned>(strides[1]), static_cast<unsigned>(strides[0]), px, py,
                              static_cast<unsigned>(dil[1]), static_cast<unsigned>(dil[0])));
  }

  // MaxPool and AveragePool (frontend/onnx/details/ops/max_pool.cpp:9-165, average_pool.cpp:9-156)
  void opPool(const Node &n, compiler::PoolFunction func) {
    const TensorHandle x = device(n, 0);
    const std::string what = n.op + " '" + n.name + "'";
    if (n.out.size() > 1 && !n.out[1].empty()) unsupported(what + ": the indices output");
    const auto ks = n.intsAttr("kernel_shape");
    if (ks.size() != 2) unsupported(what + ": kernel_shape must have 2 entries");
    std::vector<int64_t> strides = n.intsAttr("strides");
    if (strides.empty()) strides = {1, 1};
    if (strides.size() != 2) bad(what + ": strides");
    for (auto d : n.intsAttr("dilations")) if (d != 1) unsupported(what + ": dilation");
    if (n.intAttr("ceil_mode", 0) != 0) unsupported(what + ": ceil_mode");
    if (func == compiler::PoolFunction::Avg && n.intAttr("count_include_pad", 0) != 0) unsupported(what + ": count_include_pad");
    unsigned py, px;
    spatialPads(n, ks[0], ks[1], 1, 1, strides[0], strides[1], py, px);
    setDevice(n, model.pool(x, static_cast<unsigned>(ks[1]), static_cast<unsigned>(ks[0]), px, py, static_cast<unsigned>(strides[1]),
                            static_cast<unsigned>(strides[0]), func));
  }

  void opResize(const Node &n) {
    const TensorHandle x = device(n, 0);
    const std::string mode = n.strAttr("mode", "nearest");
    if (mode != "nearest") unsupported(n.op + " '" + n.name + "': mode '" + mode + "'");
    if (n.op == "Resize") {
      const std::string ctm = n.strAttr("coordinate_transformation_mode", "half_pixel");
      const std::string nm = n.strAttr("nearest_mode", "round_prefer_floor");
      // for an integer factor, floor(x / s) is what these combinations select
      const bool ok = (ctm == "asymmetric" && nm == "floor") || (ctm == "half_pixel" && nm == "round_prefer_floor") ||
                      (ctm == "pytorch_half_pixel" && nm == "round_prefer_floor");
      if (!ok) unsupported("Resize '" + n.name + "': coordinate_transformation_mode '" + ctm + "' with nearest_mode '" + nm + "'");
    }
    const auto dims = deviceShape(x);
    int64_t factor = 0;
    // scales: input 1 (Upsample, Resize-10) or input 2 (Resize-11+), or the attribute (Upsample-7); sizes: input 3
    const size_t scalesAt = (n.op == "Resize" && opset >= 11) ? 2 : 1;
    std::vector<double> scales;
    if (has(n, scalesAt) && host(n, scalesAt).size() > 0) {
      const HostTensor &s = host(n, scalesAt);
      if (!s.isFloat) bad(n.op + " '" + n.name + "': scales must be floating point");
      scales = s.fv;
    } else if (const Attr *a = n.attr("scales")) {
      scales.assign(a->floats.begin(), a->floats.end());
    }
    if (!scales.empty()) {
      if (scales.size() != 4 || scales[0] != 1.0 || scales[1] != 1.0 || scales[2] != scales[3]) unsupported(n.op + " '" + n.name + "': scales must be [1, 1, s, s]");
      factor = static_cast<int64_t>(scales[2]);
      if (static_cast<double>(factor) != scales[2] || factor < 1) unsupported(n.op + " '" + n.name + "': non-integer scale factor");
    } else if (n.op == "Resize" && has(n, 3)) {
      const HostTensor &sz = host(n, 3);
      if (sz.isFloat || sz.size() != 4) bad("Resize '" + n.name + "': sizes must be 4 integers");
      // accept sizes that are a common integer multiple of the input extents
      for (int64_t f = 1; f <= 8 && !factor; ++f)
        if (sz.iv[2] == sg.mul(dims[2], f) && sz.iv[3] == sg.mul(dims[3], f)) factor = f;
      if (!factor) unsupported("Resize '" + n.name + "': sizes are not an integer multiple of the input extents");
    } else {
      bad(n.op + " '" + n.name + "' has neither scales nor sizes");
    }
    setDevice(n, factor == 1 ? x : model.upsample(x, static_cast<unsigned>(factor), compiler::FilterMode::Nearest));
  }

  void opPad(const Node &n) {
    const Value &v = get(n, 0);
    if (!v.isDevice) unsupported("Pad '" + n.name + "' of a host tensor");
    const std::string mode = n.strAttr("mode", "constant");
    std::vector<Sym> pads;
    if (has(n, 1)) {
      const HostTensor &p = host(n, 1);
      if (p.isFloat || p.shape.size() != 1) bad("Pad '" + n.name + "': pads must be a 1-D integer tensor");
      pads = p.iv;
    } else {
      for (auto x : n.intsAttr("pads")) pads.push_back(Sym::Const(x));
    }
    std::vector<int64_t> axes = {0, 1, 2, 3};
    if (has(n, 3)) { axes = constInts(n, host(n, 3), "axes"); for (auto &a : axes) a = normAxis(n, a, 4); }
    if (pads.size() != 2 * axes.size()) bad("Pad '" + n.name + "': pads must hold " + std::to_string(2 * axes.size()) + " values");
    Sym before[4] = {Sym::Const(0), Sym::Const(0), Sym::Const(0), Sym::Const(0)}, after[4] = {Sym::Const(0), Sym::Const(0), Sym::Const(0), Sym::Const(0)};
    for (size_t k = 0; k < axes.size(); ++k) { before[axes[k]] = pads[k]; after[axes[k]] = pads[axes.size() + k]; }
    const Sym zero = Sym::Const(0);
    if (!(before[0] == zero) || !(after[0] == zero) || !(before[1] == zero) || !(after[1] == zero))
      unsupported("Pad '" + n.name + "': only height and width of an image tensor can be padded");
    const bool none = before[2] == zero && after[2] == zero && before[3] == zero && after[3] == zero;
    if (none) { values[n.out.at(0)] = v; return; }
    if (mode != "edge" && mode != "constant") unsupported("Pad '" + n.name + "': mode '" + mode + "' on an image tensor (only 'edge' and 'constant')");
    if (mode == "constant") { // the constant is input 2 (attribute `value` before opset 11); only 0 has a kernel
      double value = n.floatAttr("value", 0.0f);
      if (has(n, 2)) {
        const HostTensor c = toFloat(n, host(n, 2));
        if (c.count() != 1) bad("Pad '" + n.name + "': constant_value must be a scalar");
        value = c.fv[0];
      }
      if (value != 0.0) unsupported("Pad '" + n.name + "': constant padding with a value other than 0");
    }
    for (int ax = 2; ax < 4; ++ax)
      for (const Sym &s : {before[ax], after[ax]})
        if (s.isConst() && s.v < 0) unsupported("Pad '" + n.name + "': negative padding");
    setDevice(n, model.pad(device(n, 0), before[3], after[3], before[2], after[2], mode == "edge" ? compiler::PaddingMode::Replicate : compiler::PaddingMode::Zero));
  }

  // ---------------------------------------------------------------- graph
  void importInput(const ValueInfo &vi) {
    if (!vi.hasShape || vi.dims.size() != 4) unsupported("input '" + vi.name + "' must be a rank-4 NCHW tensor with a declared shape");
    if (vi.elemType != DT_FLOAT && vi.elemType != DT_FLOAT16) unsupported("input '" + vi.name + "' must be float or float16");
    const Dim &N = vi.dims[0], &C = vi.dims[1];
    if (!(N.hasValue && N.value == 1)) unsupported("input '" + vi.name + "': the batch dimension must be 1");
    if (!C.hasValue || C.value < 1 || C.value > 65535) unsupported("input '" + vi.name + "': the channel count must be static");
    auto extent = [&](const Dim &d, const char *suffix) {
      if (d.hasValue) { if (d.value < 1) bad("input '" + vi.name + "': non-positive extent"); return Sym::Const(d.value); }
      return model.requireValueOfName(d.hasParam && !d.param.empty() ? d.param : vi.name + "_" + suffix);
    };
    const Sym H = extent(vi.dims[2], "height"), W = extent(vi.dims[3], "width");
    Value v;
    v.isDevice = true;
    v.dev = model.input(vi.name, W, H, static_cast<unsigned>(C.value));
    values[vi.name] = std::move(v);
  }

  void importNode(const Node &n) {
    if (!n.domain.empty() && n.domain != "ai.onnx") unsupported("operator '" + n.op + "' of domain '" + n.domain + "'");
    if (n.out.empty()) bad(n.op + " '" + n.name + "' has no output");
    const std::string &op = n.op;
    if (op == "Constant") opConstant(n);
    else if (op == "Shape") opShape(n);
    else if (op == "Gather") opGather(n);
    else if (op == "Unsqueeze") opUnsqueeze(n);
    else if (op == "Squeeze") opSqueeze(n);
    else if (op == "Reshape") opReshape(n);
    else if (op == "Transpose") opTranspose(n);
    else if (op == "Cast") opCast(n);
    else if (op == "ConstantOfShape") opConstantOfShape(n);
    else if (op == "Expand") opExpand(n);
    else if (op == "Slice") opSlice(n);
    else if (op == "Concat") opConcat(n);
    else if (op == "Identity") values[n.out[0]] = get(n, 0);
    else if (op == "Add" || op == "Sub" || op == "Mul" || op == "Div" || op == "Mod" || op == "Min" || op == "Max" || op == "Pow") binary(n);
    else if (op == "Clip") opClip(n);
    else if (op == "Neg" || op == "Abs" || op == "Floor" || op == "Ceil" || op == "Round" || op == "Sqrt" || op == "Reciprocal" || op == "Sign") unary(n);
    else if (op == "Conv") opConv(n);
    else if (op == "Relu") setDevice(n, model.activation(device(n, 0), compiler::ActivationFunction::ReLU, 0.0f));
    else if (op == "LeakyRelu") setDevice(n, model.activation(device(n, 0), compiler::ActivationFunction::LeakyReLU, n.floatAttr("alpha", 0.01f)));
    else if (op == "MaxPool") opPool(n, compiler::PoolFunction::Max);
    else if (op == "AveragePool") opPool(n, compiler::PoolFunction::Avg);
    else if (op == "Resize" || op == "Upsample") opResize(n);
    else if (op == "Pad") opPad(n);
    else unsupported("operator '" + op + "' (node '" + n.name + "')");
  }

  void importGraph(Pb pb) {
    std::vector<Node> nodes;
    std::vector<TensorProto> inits;
    std::vector<ValueInfo> inputs, outputs;
    while (!pb.done()) {
      uint32_t f, w;
      pb.key(f, w);
      switch (f) {
      case 1: nodes.push_back(parseNode(pb.bytes())); break;
      case 5: inits.push_back(parseTensor(pb.bytes())); break;
      case 11: inputs.push_back(parseValueInfo(pb.bytes())); break;
      case 12: outputs.push_back(parseValueInfo(pb.bytes())); break;
      case 15: unsupported("sparse initializers");
      default: pb.skip(w);
      }
    }
    for (const TensorProto &t : inits) {
      Value v;
      v.host = fromTensorProto(t);
      values[t.name] = std::move(v);
    }
    for (const ValueInfo &vi : inputs)
      if (!values.count(vi.name)) importInput(vi); // (old files list initializers among the inputs)
    if (model.inputs().empty()) bad("the graph has no image input");
    for (const Node &n : nodes) importNode(n); // ONNX graphs are topologically sorted
    if (outputs.empty()) bad("the graph has no output");
    for (const ValueInfo &vi : outputs) {
      auto it = values.find(vi.name);
      if (it == values.end()) bad("graph output '" + vi.name + "' is never produced");
      if (!it->second.isDevice) unsupported("graph output '" + vi.name + "' is not an image tensor");
      model.output(materialize(it->second), vi.name);
    }
  }
};

} // namespace

void importModel(compiler::Model &model, const uint8_t *data, size_t size) {
  if (!data || size == 0) fail(Status::InvalidArgument, "ONNX import: empty buffer");
  if (!model.tensors().empty()) fail(Status::InvalidArgument, "ONNX import: the builder already holds a graph");
  Importer imp(model);
  Pb pb{data, data + size};
  const uint8_t *graphBegin = nullptr, *graphEnd = nullptr;
  bool functions = false;
  while (!pb.done()) {
    uint32_t f, w;
    pb.key(f, w);
    if (f == 7 && w == 2) {
      Pb g = pb.bytes();
      graphBegin = g.p;
      graphEnd = g.end;
    } else if (f == 8 && w == 2) {
      Pb o = pb.bytes();
      std::string domain;
      int64_t version = 0;
      while (!o.done()) {
        uint32_t f2, w2;
        o.key(f2, w2);
        if (f2 == 1) domain = o.str();
        else if (f2 == 2) version = static_cast<int64_t>(o.varint());
        else o.skip(w2);
      }
      if (domain.empty() || domain == "ai.onnx") imp.opset = std::max(imp.opset, version);
      else unsupported("operator set domain '" + domain + "'");
    } else if (f == 25) {
      functions = true;
      pb.skip(w);
    } else {
      pb.skip(w);
    }
  }
  if (functions) unsupported("model-local functions");
  if (imp.opset <= 0) bad("missing opset_import for the default domain");
  if (!graphBegin) bad("missing top-level graph");
  imp.importGraph(Pb{graphBegin, graphEnd});
}

} // namespace denox::onnx
