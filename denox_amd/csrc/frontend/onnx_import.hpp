// ONNX import: reads an ONNX ModelProto and drives the graph builder.
//
// Stands for the reference's importer
//   compiler/src/denox/compiler/frontend/onnx/onnx.cpp:70-158 (read)
//   compiler/src/denox/compiler/frontend/onnx/details/import_node.cpp, import_value_info.cpp, ops/*.cpp
// for the operators a denoising U-Net exported by PyTorch consists of: Conv, Relu, LeakyRelu, MaxPool,
// Resize / Upsample (nearest, integer factor), Concat, Pad (edge), Slice on image tensors, and the
// shape arithmetic PyTorch emits around them (Shape, Gather, Constant, ConstantOfShape, Unsqueeze, Squeeze,
// Concat, Reshape, Slice, Transpose, Cast, Expand, Identity, Add, Sub, Mul, Div, Mod, Min, Max, Neg, Abs, Floor,
// Ceil, Round, Sqrt, Reciprocal, Sign) evaluated at import time on small host tensors whose integer elements may be
// symbolic (functions of the dynamic image extents).
//
// The protobuf wire format is decoded directly (field numbers of onnx.proto, third_party/onnx/onnx.proto in the
// reference); no protobuf library is involved.
#pragma once
#include "../compiler/model.hpp"
#include <cstddef>
#include <cstdint>

namespace denox::onnx {

// Appends the network in `data` to `model` (inputs, layers, outputs).  Image tensors are NCHW with N = 1; dynamic
// height / width dimensions become the model's named extents (dim_param names).  Throws denox::Error.
void importModel(compiler::Model &model, const uint8_t *data, size_t size);

} // namespace denox::onnx
