#include "model.hpp"

namespace denox::compiler {

const TensorNode &Model::get(TensorHandle h) const {
  if (h < 0 || static_cast<size_t>(h) >= m_tensors.size()) fail(Status::InvalidArgument, "invalid tensor handle");
  return m_tensors[static_cast<size_t>(h)];
}

TensorHandle Model::newTensor(Sym w, Sym h, unsigned c, int producer) {
  TensorNode t;
  t.width = w; t.height = h; t.channels = c; t.producer = producer;
  m_tensors.push_back(std::move(t));
  return static_cast<TensorHandle>(m_tensors.size() - 1);
}

TensorHandle Model::input(const std::string &name, Sym width, Sym height, unsigned channels) {
  if (channels == 0) fail(Status::InvalidArgument, "input with zero channels");
  TensorHandle t = newTensor(width, height, channels, -1);
  m_tensors[t].name = name;
  m_tensors[t].isInput = true;
  m_inputs.push_back(t);
  return t;
}

TensorHandle Model::conv2d(TensorHandle src, unsigned K, unsigned C, unsigned R, unsigned S, const uint16_t *w,
                           const uint16_t *bias, unsigned strideX, unsigned strideY, unsigned padX, unsigned padY,
                           unsigned dilX, unsigned dilY) {
  const TensorNode in = get(src);
  if (in.channels != C) fail(Status::InvalidArgument, "conv2d: filter expects " + std::to_string(C) + " input channels, tensor has " + std::to_string(in.channels));
  if (!w || K == 0 || R == 0 || S == 0 || strideX == 0 || strideY == 0 || dilX == 0 || dilY == 0) fail(Status::InvalidArgument, "conv2d: bad filter description");
  Op op;
  op.kind = OpKind::Conv;
  op.inputs = {src};
  op.K = K; op.C = C; op.R = R; op.S = S;
  op.weights.assign(w, w + static_cast<size_t>(K) * C * R * S);
  op.hasBias = bias != nullptr;
  if (bias) op.bias.assign(bias, bias + K);
  op.strideX = strideX; op.strideY = strideY; op.padX = padX; op.padY = padY; op.dilX = dilX; op.dilY = dilY;
  const Sym ow = m_sym.pool(in.width, S, padX, strideX, dilX);
  const Sym oh = m_sym.pool(in.height, R, padY, strideY, dilY);
  op.output = newTensor(ow, oh, K, static_cast<int>(m_ops.size()));
  m_tensors[src].consumers.push_back(static_cast<int>(m_ops.size()));
  m_ops.push_back(std::move(op));
  return m_ops.back().output;
}

TensorHandle Model::activation(TensorHandle src, ActivationFunction func, float alpha) {
  const TensorNode in = get(src);
  Op op;
  op.kind = OpKind::Activation;
  op.inputs = {src};
  op.func = func; op.alpha = alpha;
  op.output = newTensor(in.width, in.height, in.channels, static_cast<int>(m_ops.size()));
  m_tensors[src].consumers.push_back(static_cast<int>(m_ops.size()));
  m_ops.push_back(std::move(op));
  return m_ops.back().output;
}

TensorHandle Model::upsample(TensorHandle src, unsigned f, FilterMode) {
  const TensorNode in = get(src);
  if (f == 0) fail(Status::InvalidArgument, "upsample: zero scaling factor");
  Op op;
  op.kind = OpKind::Upsample;
  op.inputs = {src};
  op.scale = f;
  op.output = newTensor(m_sym.mul(in.width, f), m_sym.mul(in.height, f), in.channels, static_cast<int>(m_ops.size()));
  m_tensors[src].consumers.push_back(static_cast<int>(m_ops.size()));
  m_ops.push_back(std::move(op));
  return m_ops.back().output;
}

TensorHandle Model::pool(TensorHandle src, unsigned kx, unsigned ky, unsigned px, unsigned py, unsigned sx, unsigned sy, PoolFunction f) {
  const TensorNode in = get(src);
  if (kx == 0 || ky == 0 || sx == 0 || sy == 0) fail(Status::InvalidArgument, "pool: bad window");
  Op op;
  op.kind = OpKind::Pool;
  op.inputs = {src};
  op.kernelX = kx; op.kernelY = ky; op.poolPadX = px; op.poolPadY = py; op.poolStrideX = sx; op.poolStrideY = sy; op.poolFunc = f;
  op.output = newTensor(m_sym.pool(in.width, kx, px, sx, 1), m_sym.pool(in.height, ky, py, sy, 1), in.channels, static_cast<int>(m_ops.size()));
  m_tensors[src].consumers.push_back(static_cast<int>(m_ops.size()));
  m_ops.push_back(std::move(op));
  return m_ops.back().output;
}

// A relation that constants violate is an error now; one that involves a symbol is recorded and checked per instance.
void Model::require(Sym lhs, Sym rhs, int relation, const std::string &what) {
  if (lhs == rhs) return;
  if (lhs.isConst() && rhs.isConst()) {
    if (relation == 0 ? lhs.v != rhs.v : lhs.v > rhs.v)
      fail(Status::InvalidArgument, what + ": " + std::to_string(lhs.v) + (relation == 0 ? " != " : " > ") + std::to_string(rhs.v));
    return;
  }
  m_requirements.push_back(Requirement{lhs, rhs, relation, what});
}

TensorHandle Model::concat(TensorHandle src0, TensorHandle src1) {
  const TensorNode a = get(src0), b = get(src1);
  // extents must agree (the reference's importer leaves symbolic extents to the caller; here they are checked when an
  // instance is created: kernels index the sources with the result's extents)
  require(a.width, b.width, 0, "concat: widths of the sources differ");
  require(a.height, b.height, 0, "concat: heights of the sources differ");
  Op op;
  op.kind = OpKind::Concat;
  op.inputs = {src0, src1};
  op.output = newTensor(a.width, a.height, a.channels + b.channels, static_cast<int>(m_ops.size()));
  m_tensors[src0].consumers.push_back(static_cast<int>(m_ops.size()));
  m_tensors[src1].consumers.push_back(static_cast<int>(m_ops.size()));
  m_ops.push_back(std::move(op));
  return m_ops.back().output;
}

TensorHandle Model::pad(TensorHandle src, Sym left, Sym right, Sym top, Sym bottom, PaddingMode mode) {
  const TensorNode in = get(src);
  Op op;
  op.kind = OpKind::Pad;
  op.inputs = {src};
  op.left = left; op.right = right; op.top = top; op.bottom = bottom;
  op.padMode = mode;
  op.output = newTensor(m_sym.add(m_sym.add(in.width, left), right), m_sym.add(m_sym.add(in.height, top), bottom), in.channels, static_cast<int>(m_ops.size()));
  m_tensors[src].consumers.push_back(static_cast<int>(m_ops.size()));
  m_ops.push_back(std::move(op));
  return m_ops.back().output;
}

TensorHandle Model::slice(TensorHandle src, Sym left, Sym right, Sym top, Sym bottom) {
  const TensorNode in = get(src);
  Op op;
  op.kind = OpKind::Slice;
  op.inputs = {src};
  op.left = left; op.right = right; op.top = top; op.bottom = bottom;
  require(Sym::Const(0), left, 1, "slice: left bound below zero");
  require(Sym::Const(0), top, 1, "slice: top bound below zero");
  require(left, right, 1, "slice: left bound beyond the right one");
  require(top, bottom, 1, "slice: top bound beyond the bottom one");
  require(right, in.width, 1, "slice: right bound beyond the source's width");
  require(bottom, in.height, 1, "slice: bottom bound beyond the source's height");
  // [left, right) x [top, bottom) in source coordinates (frontend/model/Model.cpp:233-253 of the reference)
  op.output = newTensor(m_sym.sub(right, left), m_sym.sub(bottom, top), in.channels, static_cast<int>(m_ops.size()));
  m_tensors[src].consumers.push_back(static_cast<int>(m_ops.size()));
  m_ops.push_back(std::move(op));
  return m_ops.back().output;
}

void Model::output(TensorHandle src, const std::string &name) {
  (void)get(src);
  m_tensors[src].isOutput = true;
  if (m_tensors[src].name.empty()) m_tensors[src].name = name;
  m_outputs.push_back(src);
}

void Model::assignValueName(const std::string &name, Sym value) {
  for (auto &nv : m_valueNames)
    if (nv.name == name) { nv.value = value; return; }
  m_valueNames.push_back(NamedValue{name, value});
}

Sym Model::requireValueOfName(const std::string &name) {
  for (const auto &nv : m_valueNames) if (nv.name == name) return nv.value;
  Sym v = m_sym.var(name);
  m_valueNames.push_back(NamedValue{name, v});
  return v;
}

} // namespace denox::compiler
