// Device limits the kernel configuration spaces are pruned with.
// Same role as the reference's DeviceInfo (device_info/src/denox/device_info/DeviceInfo.hpp:12-20,
// ResourceLimits.hpp:8-22, SubgroupProperties.hpp:7-15, CoopmatProperties.hpp:9-27), which it
// fills from Vulkan queries; here the table is CDNA4 (gfx950) and, when a device
// is present, refined from hipDeviceProp_t.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace denox {

struct MatrixShape { unsigned m, n, k; const char *atype, *acctype; };

struct DeviceInfo {
  std::string name = "gfx950";
  std::string arch = "gfx950";
  // subgroup
  unsigned subgroupSize = 64;
  // limits
  unsigned maxComputeWorkGroupInvocations = 1024;
  unsigned maxComputeWorkGroupSize[3] = {1024, 1024, 1024};
  unsigned maxComputeWorkGroupCount[3] = {0x7FFFFFFFu, 65535u, 65535u};
  unsigned maxComputeSharedMemory = 160 * 1024; // LDS bytes one workgroup may use
  unsigned maxPushConstantSize = 4096;          // kernel-argument bytes after the pointers
  unsigned vgprsPerLane = 512;                  // unified VGPR + AGPR file at one wave per SIMD
  // chip
  unsigned computeUnits = 256;
  unsigned xcdCount = 8;
  unsigned simdPerCu = 4;
  unsigned l2BytesPerXcd = 4u << 20;
  uint64_t infinityCacheBytes = 256ull << 20;
  uint64_t hbmBytes = 288ull << 30;
  // published peaks used by cost estimates and roofline reports
  double hbmBytesPerSecond = 8.0e12;
  double fp16MfmaFlops = 2.5e15;
  // matrix-core shapes with fp32 accumulation this backend emits
  std::vector<MatrixShape> matrixShapes = {{32, 32, 16, "f16", "f32"}, {16, 16, 32, "f16", "f32"}};
  bool fromDevice = false;
};

// Table values; no GPU needed.
DeviceInfo cdna4_device_info();
// Table refined by the HIP device's reported properties (name, CU count, LDS per block, memory).
DeviceInfo query_driver_device_info(int device);

} // namespace denox
