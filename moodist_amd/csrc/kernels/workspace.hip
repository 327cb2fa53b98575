// A fixed block of device memory for callers that may not allocate: the padded temporary of
// an allreduce whose element count the group size does not divide (the reference takes it
// from torch, core/processgroup.cc:1694-1697).  The block is a device array of this library,
// so each GPU the library runs on holds MDH_STATIC_WORKSPACE_BYTES of it from the moment its
// code is loaded there until the process ends; nothing is allocated or freed per call.
#include "device_common.h"

#include <mutex>

namespace {

// On the host this name stands for the array only as a handle for hipGetSymbolAddress: it is
// not a device address and is never passed to a kernel or a copy.
static __device__ __align__(256) unsigned char scratch[MDH_STATIC_WORKSPACE_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_lock;
void* g_address[kMaxDevices]; // per device: every GPU has its own copy of the array at its own address

} // namespace

extern "C" int mdh_static_workspace(void** address, size_t* bytes) {
  if (!address || !bytes) {
    mdh::set_error("mdh_static_workspace: null out pointer");
    return MDH_EINVAL;
  }
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess || device < 0 || device >= kMaxDevices) {
    mdh::set_error("mdh_static_workspace: no current device (%s)", hipGetErrorString(e));
    return MDH_ENODEVICE;
  }
  std::lock_guard<std::mutex> hold(g_lock);
  if (!g_address[device]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      mdh::set_error("mdh_static_workspace: hipGetSymbolAddress on device %d: %s", device, hipGetErrorString(e));
      return MDH_ENODEVICE;
    }
    g_address[device] = p;
  }
  *address = g_address[device];
  *bytes = (size_t)MDH_STATIC_WORKSPACE_BYTES;
  return MDH_OK;
}
