#include "hip_loader.h"

#include <dlfcn.h>

#include <atomic>
#include <mutex>
#include <stdexcept>
#include <string>

namespace moodist {

namespace {

template<typename F>
void resolve(void* lib, const char* libname, const char* sym, F& out) {
  void* p = dlsym(lib, sym);
  if (!p) {
    throw std::runtime_error(std::string("moodist: ") + libname + " has no symbol " + sym);
  }
  out = reinterpret_cast<F>(p);
}

std::string sibling_kernel_library() {
  // libmoodist_hip.so is installed beside this library
  Dl_info info;
  if (dladdr(reinterpret_cast<void*>(&sibling_kernel_library), &info) && info.dli_fname) {
    std::string path = info.dli_fname;
    size_t slash = path.rfind('/');
    if (slash != std::string::npos) {
      return path.substr(0, slash + 1) + "libmoodist_hip.so";
    }
  }
  return "libmoodist_hip.so";
}

HipRuntime load() {
  HipRuntime r{};
  void* rt = nullptr;
  const char* const names[] = {"libamdhip64.so.7", "libamdhip64.so.6", "libamdhip64.so", "/opt/rocm/lib/libamdhip64.so"};
  // a runtime the process has already mapped (torch's) is the one to use: a second copy would
  // have its own device state
  for (const char* name : names) {
    rt = dlopen(name, RTLD_NOW | RTLD_GLOBAL | RTLD_NOLOAD);
    if (rt) {
      break;
    }
  }
  for (const char* name : names) {
    if (rt) {
      break;
    }
    rt = dlopen(name, RTLD_NOW | RTLD_GLOBAL);
  }
  if (!rt) {
    throw std::runtime_error(std::string("moodist: cannot load the HIP runtime (libamdhip64.so): ") + dlerror());
  }
  const char* rn = "libamdhip64.so";
  resolve(rt, rn, "hipGetDeviceCount", r.GetDeviceCount);
  resolve(rt, rn, "hipSetDevice", r.SetDevice);
  resolve(rt, rn, "hipGetDevice", r.GetDevice);
  resolve(rt, rn, "hipMemcpyAsync", r.MemcpyAsync);
  resolve(rt, rn, "hipMemcpy2DAsync", r.Memcpy2DAsync);
  resolve(rt, rn, "hipStreamSynchronize", r.StreamSynchronize);
  resolve(rt, rn, "hipStreamIsCapturing", r.StreamIsCapturing);
  resolve(rt, rn, "hipGetLastError", r.GetLastError);
  resolve(rt, rn, "hipEventCreateWithFlags", r.EventCreateWithFlags);
  resolve(rt, rn, "hipEventDestroy", r.EventDestroy);
  resolve(rt, rn, "hipEventRecord", r.EventRecord);
  resolve(rt, rn, "hipStreamWaitEvent", r.StreamWaitEvent);
  resolve(rt, rn, "hipGetErrorString", r.GetErrorString);

  const std::string kpath = sibling_kernel_library();
  void* kl = dlopen(kpath.c_str(), RTLD_NOW | RTLD_LOCAL);
  if (!kl) {
    throw std::runtime_error("moodist: cannot load the gfx950 kernel library " + kpath + ": " + dlerror() +
                             " (there is no CPU fallback; build it with moodist_amd/csrc/build.sh)");
  }
  const char* kn = "libmoodist_hip.so";
  resolve(kl, kn, "mdh_abi_version", r.abi_version);
  resolve(kl, kn, "mdh_last_error", r.last_error);
  resolve(kl, kn, "mdh_error_string", r.error_string);
  resolve(kl, kn, "mdh_reduce", r.reduce);
  resolve(kl, kn, "mdh_reduce_many", r.reduce_many);
  resolve(kl, kn, "mdh_allreduce_many", r.allreduce_many);
  resolve(kl, kn, "mdh_gather", r.gather);
  resolve(kl, kn, "mdh_copy_boxes", r.copy_boxes);
  resolve(kl, kn, "mdh_copy_plan_create", r.copy_plan_create);
  resolve(kl, kn, "mdh_copy_plan_launch", r.copy_plan_launch);
  resolve(kl, kn, "mdh_copy_plan_destroy", r.copy_plan_destroy);
  resolve(kl, kn, "mdh_static_workspace", r.static_workspace);
  if (r.abi_version() != MDH_ABI_VERSION) {
    throw std::runtime_error("moodist: libmoodist_hip.so has ABI version " + std::to_string(r.abi_version()) +
                             ", this core expects " + std::to_string(MDH_ABI_VERSION));
  }
  return r;
}

std::atomic<bool> g_loaded{false};

} // namespace

const HipRuntime& hip() {
  static HipRuntime r = [] {
    HipRuntime loaded = load();
    g_loaded.store(true, std::memory_order_release);
    return loaded;
  }();
  return r;
}

bool hip_loaded() {
  return g_loaded.load(std::memory_order_acquire);
}

void refuse_capture(void* stream, const char* what) {
  const HipRuntime& h = hip();
  int status = 0; // hipStreamCaptureStatusNone
  const int rc = h.StreamIsCapturing(stream, &status);
  // the legacy default stream reports a capture going on elsewhere as an error of its own
  const bool capturing = rc == 0 ? status != 0 : rc == kHipErrorStreamCaptureImplicit;
  if (rc != 0) {
    h.GetLastError(); // anything else (no device, an unknown stream) is for the launch itself to report
  }
  if (capturing) {
    throw std::runtime_error(std::string("moodist: ") + what +
                             ": the stream is being captured into a graph; capture and replay of moodist collectives "
                             "is not supported (call on a stream that is not capturing)");
  }
}

void check_hip(int rc, const char* what) {
  if (rc != 0) {
    throw std::runtime_error(std::string("moodist: ") + what + ": " + hip().GetErrorString(rc));
  }
}

void check_mdh(int rc) {
  if (rc != 0) {
    const char* detail = hip().last_error();
    throw std::runtime_error(detail && *detail ? std::string(detail) : std::string(hip().error_string(rc)));
  }
}

} // namespace moodist
