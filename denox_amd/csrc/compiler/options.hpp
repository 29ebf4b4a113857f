// Compile options, after the reference's CompileOptions
// (compiler/src/denox/compiler/Options.hpp:13-72): feature switches,
// per-interface-tensor descriptors, assumed extents for cost estimates.
#pragma once
#include "../common/dnx.hpp"
#include "../device_info/device_info.hpp"
#include <map>
#include <string>
#include <vector>

namespace denox::compiler {

struct Features {
  bool enableConvReluFusion = true;   // conv + activation in one dispatch      (reference: Options.hpp:13-18)
  bool enableConcatConvFusion = true; // conv reads its two concat sources      (reference: ConcatConvCMShader)
  bool enableUpsampleFusion = true;   // conv reads a half-resolution source at (y/2, x/2)
  bool enablePoolFusion = true;       // conv stores the 2x2 max only
  bool enablePadFusion = true;        // conv reads an un-padded source through the replicate clamp
  bool enableSliceFusion = true;      // conv stores only the cropped window
  bool enableUpsampleFold = true;     // candidates that fold a fused 2x upsample into the conv weights (2x2 taps per output parity)
  bool enableAlternatingTraversal = true; // consecutive conv dispatches walk their tiles in opposite directions
  bool enableImplicitConcat = true;   // memory-aliasing concat where layouts allow it
  bool enableBlockedLayout = true;    // offer every internal tensor in CHWC8 beside HWC (reference: specialization.cpp:13-16)
  bool enableConvConvFusion = true;   // two consecutive 3x3 convolutions in one dispatch, the tensor between them kept in LDS
};

struct InterfaceTensorDescriptor {
  std::string name;
  dnx::TensorFormat format = dnx::TensorFormat::SSBO_HWC;
};

struct CompileOptions {
  Features features;
  std::vector<InterfaceTensorDescriptor> inputDescriptors, outputDescriptors;
  // extents assumed when a cost has to be estimated for a dynamic model
  // (reference: compiler/src/denox/compiler/assumed_symeval, cli/compile.cpp:20-21)
  std::map<std::string, int64_t> assumptions;
  int64_t defaultAssumedExtent = 1920;
  DeviceInfo deviceInfo;
  // restrict the conv configuration space to one named configuration ("" = all)
  std::string forceConvConfig;
  // > 0: candidates that read or write a CHWC8 tensor count half their cost, so that the blocked layout is taken wherever
  // it is offered (tests and measurements of that path); 0: cost alone decides
  int layoutPreference = 0;
  bool verbose = false;
};

} // namespace denox::compiler
