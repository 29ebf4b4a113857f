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

// All contexts of a GPU share the one array, and each context launches on a stream of its own: two calls from different
// contexts are not ordered by any stream.  The array therefore has a user per device: the context whose call used it last, with
// an event that context recorded behind that call's launches.  Another context may take the array only once that event has
// completed; while it has not, its call is refused instead of running into the other's intermediate tensors.
namespace {
struct ScratchUser {
  const void *context = nullptr;
  hipEvent_t done = nullptr;
};
std::mutex g_userMutex;
ScratchUser g_user[64];
} // namespace

void staticScratchAcquire(int device, const void *context) {
  std::lock_guard<std::mutex> lock(g_userMutex);
  ScratchUser &u = g_user[device];
  if (!u.context || u.context == context) return; // the same context's calls are ordered by its stream
  const hipError_t e = hipEventQuery(u.done);
  if (e == hipErrorNotReady)
    fail(Status::InvalidArgument, "the static scratch array of this GPU is still in use by a call made through another context; "
                                  "synchronize that context first (calls from different contexts are not ordered)");
  hipCheck(e, "hipEventQuery(static scratch)");
  u = ScratchUser{};
}

void staticScratchRecord(int device, const void *context, hipEvent_t done, hipStream_t stream) {
  hipCheck(hipEventRecord(done, stream), "hipEventRecord(static scratch)");
  std::lock_guard<std::mutex> lock(g_userMutex);
  g_user[device] = ScratchUser{context, done};
}

void staticScratchForget(int device, const void *context) {
  std::lock_guard<std::mutex> lock(g_userMutex);
  if (device >= 0 && device < 64 && g_user[device].context == context) g_user[device] = ScratchUser{};
}

} // namespace denox::runtime
