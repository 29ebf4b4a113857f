#include "device_info.hpp"
#include "../common/error.hpp"
#include <hip/hip_runtime_api.h>

namespace denox {

DeviceInfo cdna4_device_info() { return DeviceInfo{}; }

DeviceInfo query_driver_device_info(int device) {
  DeviceInfo info;
  hipDeviceProp_t p;
  hipError_t e = hipGetDeviceProperties(&p, device);
  if (e != hipSuccess) fail(Status::HipError, std::string("hipGetDeviceProperties: ") + hipGetErrorString(e));
  info.name = p.name;
  info.arch = p.gcnArchName;
  const size_t colon = info.arch.find(':');
  if (colon != std::string::npos) info.arch.resize(colon);
  info.subgroupSize = static_cast<unsigned>(p.warpSize);
  info.maxComputeWorkGroupInvocations = static_cast<unsigned>(p.maxThreadsPerBlock);
  for (int i = 0; i < 3; ++i) {
    info.maxComputeWorkGroupSize[i] = static_cast<unsigned>(p.maxThreadsDim[i]);
    info.maxComputeWorkGroupCount[i] = static_cast<unsigned>(p.maxGridSize[i]);
  }
  if (p.sharedMemPerBlock > 0) info.maxComputeSharedMemory = static_cast<unsigned>(p.sharedMemPerBlock);
  info.computeUnits = static_cast<unsigned>(p.multiProcessorCount);
  info.hbmBytes = p.totalGlobalMem;
  if (p.l2CacheSize > 0) info.l2BytesPerXcd = static_cast<unsigned>(p.l2CacheSize);
  info.fromDevice = true;
  return info;
}

} // namespace denox
