// The one device allocation the library owns without ever calling hipMalloc: a file-scope array that every GPU the
// library runs on holds from the moment this code object is loaded there until the process ends.  The allocation-free
// entry point (denox_hip_instance_infer_device_static) places an instance's intermediate tensors in it, so that it can
// run where hipMalloc is not allowed (under stream capture, in loops that must not allocate).
//
// In host code the array's name is only a stand-in for the device symbol; the address kernels can use comes from
// hipGetSymbolAddress, once per device, and is what the rest of the library passes around.
#include "runtime.hpp"
#include <hip/hip_runtime.h>
#include <mutex>

namespace denox::runtime {

static __device__ __attribute__((used)) __align__(256) unsigned char scratch[kStaticScratchBytes];

void *staticScratchAddress(int device) {
  constexpr int kMaxDevices = 64;
  static std::mutex mutex;
  static void *address[kMaxDevices] = {};
  if (device < 0 || device >= kMaxDevices) fail(Status::InvalidArgument, "device index out of range for the static scratch table");
  std::lock_guard<std::mutex> lock(mutex);
  if (!address[device]) {
    int current = -1;
    hipCheck(hipGetDevice(&current), "hipGetDevice");
    if (current != device) fail(Status::Internal, "staticScratchAddress: the device is not current");
    void *p = nullptr;
    hipCheck(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
    if (!p) fail(Status::HipError, "hipGetSymbolAddress(scratch) returned no address");
    address[device] = p;
  }
  return address[device];
}

} // namespace denox::runtime
