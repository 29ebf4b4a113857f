// Front-end graph of a network: tensors with symbolic extents joined by layer
// operations.  Same builder surface as the reference's compiler::Model
//   compiler/src/denox/compiler/frontend/model/Model.hpp:33-62
//   (input / conv2d / activation / upsample / pool / concat / pad / slice / output,
//    assignValueName / requireValueOfName)
// which its ONNX importer drives (compiler/src/denox/compiler/frontend/onnx/onnx.cpp:70-158).
// Here the graph is built directly through the C ABI.
#pragma once
#include "../common/sym.hpp"
#include <cstdint>
#include <string>
#include <vector>

namespace denox::compiler {

enum class OpKind { Conv, Activation, Upsample, Pool, Concat, Pad, Slice };
enum class ActivationFunction { ReLU, LeakyReLU };
enum class PoolFunction { Max, Avg };
enum class FilterMode { Nearest };
enum class PaddingMode { Replicate, Zero }; // the reference's PaddingMode { Edge, Zero } (common/PaddingMode.hpp)

using TensorHandle = int; // index into Model::tensors

struct TensorNode {
  Sym width, height;
  unsigned channels = 0;
  std::string name;
  int producer = -1;            // op index, -1 for inputs
  std::vector<int> consumers;   // op indices
  bool isInput = false, isOutput = false;
};

struct Op {
  OpKind kind;
  std::vector<TensorHandle> inputs;
  TensorHandle output = -1;
  // Conv: weights in ONNX order [K][C][R][S], binary16 bit patterns
  unsigned K = 0, C = 0, R = 0, S = 0;
  std::vector<uint16_t> weights, bias;
  bool hasBias = false;
  unsigned strideX = 1, strideY = 1, padX = 0, padY = 0, dilX = 1, dilY = 1;
  // Activation
  ActivationFunction func = ActivationFunction::ReLU;
  float alpha = 0.0f;
  // Upsample
  unsigned scale = 2;
  // Pool
  unsigned kernelX = 2, kernelY = 2, poolStrideX = 2, poolStrideY = 2, poolPadX = 0, poolPadY = 0;
  PoolFunction poolFunc = PoolFunction::Max;
  // Pad: border widths.  Slice: the half-open source ranges [left, right) x [top, bottom)
  Sym left, right, top, bottom;
  PaddingMode padMode = PaddingMode::Replicate;
};

struct NamedValue { std::string name; Sym value; };

class Model {
public:
  SymGraph &symGraph() { return m_sym; }
  const SymGraph &symGraph() const { return m_sym; }

  TensorHandle input(const std::string &name, Sym width, Sym height, unsigned channels);
  TensorHandle conv2d(TensorHandle src, unsigned K, unsigned C, unsigned R, unsigned S, const uint16_t *weightsKCRS,
                      const uint16_t *bias, unsigned strideX, unsigned strideY, unsigned padX, unsigned padY,
                      unsigned dilX, unsigned dilY);
  TensorHandle activation(TensorHandle src, ActivationFunction func, float alpha);
  TensorHandle upsample(TensorHandle src, unsigned scalingFactor, FilterMode mode);
  TensorHandle pool(TensorHandle src, unsigned kx, unsigned ky, unsigned px, unsigned py, unsigned sx, unsigned sy, PoolFunction f);
  TensorHandle concat(TensorHandle src0, TensorHandle src1);
  TensorHandle pad(TensorHandle src, Sym left, Sym right, Sym top, Sym bottom, PaddingMode mode);
  TensorHandle slice(TensorHandle src, Sym left, Sym right, Sym top, Sym bottom);
  void output(TensorHandle src, const std::string &name);

  void assignValueName(const std::string &name, Sym value);
  Sym requireValueOfName(const std::string &name); // creates a free variable when unknown

  const std::vector<TensorNode> &tensors() const { return m_tensors; }
  const std::vector<Op> &ops() const { return m_ops; }
  const std::vector<TensorHandle> &inputs() const { return m_inputs; }
  const std::vector<TensorHandle> &outputs() const { return m_outputs; }
  const std::vector<NamedValue> &valueNames() const { return m_valueNames; }
  // relations between extents that a layer needs and that are not settled while the model is built (symbolic extents):
  // lhs == rhs (relation 0) or lhs <= rhs (1); checked when an instance is created
  struct Requirement { Sym lhs, rhs; int relation; std::string what; };
  const std::vector<Requirement> &requirements() const { return m_requirements; }

private:
  TensorHandle newTensor(Sym w, Sym h, unsigned c, int producer);
  const TensorNode &get(TensorHandle h) const;
  SymGraph m_sym;
  std::vector<TensorNode> m_tensors;
  std::vector<Op> m_ops;
  std::vector<TensorHandle> m_inputs, m_outputs;
  std::vector<NamedValue> m_valueNames;
  std::vector<Requirement> m_requirements;
  void require(Sym lhs, Sym rhs, int relation, const std::string &what);
};

} // namespace denox::compiler
