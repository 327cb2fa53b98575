// HIP runtime loader: resolves libamdhip64.so and the kernel library
// libmoodist_hip.so with dlopen/dlsym on first GPU use, so that the host core
// links against neither and loads on a machine that has no ROCm at all.
//
// Takes the place of the reference's core/cuda_loader.cc (loadCuda :67-159
// for the driver API, loadNvml :170-191, loadNvrtc :201-222).  There is no
// NVML or run-time compiler counterpart: topology is not discovered (one GPU)
// and the kernels are compiled ahead of time for gfx950.
#pragma once

#include <cstddef>
#include <cstdint>

#include "moodist_hip.h"

namespace moodist {

// Own declarations of the few runtime entry points used, like the reference
// declares the CUDA driver API itself (core/cuda_loader.h) instead of
// including SDK headers.  hipError_t is an int-sized enum; 0 is success.
struct HipRuntime {
  int (*GetDeviceCount)(int* count);
  int (*SetDevice)(int device);
  int (*GetDevice)(int* device);
  int (*MemcpyAsync)(void* dst, const void* src, size_t bytes, int kind, void* stream);
  int (*Memcpy2DAsync)(void* dst, size_t dpitch, const void* src, size_t spitch, size_t width, size_t height, int kind,
      void* stream);
  int (*StreamSynchronize)(void* stream);
  int (*StreamIsCapturing)(void* stream, int* status);
  int (*GetLastError)();
  int (*EventCreateWithFlags)(void** event, unsigned flags);
  int (*EventDestroy)(void* event);
  int (*EventRecord)(void* event, void* stream);
  int (*StreamWaitEvent)(void* stream, void* event, unsigned flags);
  const char* (*GetErrorString)(int error);

  // thin C ABI of the kernel library (include/moodist_hip.h)
  decltype(&mdh_abi_version) abi_version;
  decltype(&mdh_last_error) last_error;
  decltype(&mdh_error_string) error_string;
  decltype(&mdh_reduce) reduce;
  decltype(&mdh_reduce_many) reduce_many;
  decltype(&mdh_allreduce_many) allreduce_many;
  decltype(&mdh_gather) gather;
  decltype(&mdh_copy_boxes) copy_boxes;
  decltype(&mdh_copy_plan_create) copy_plan_create;
  decltype(&mdh_copy_plan_launch) copy_plan_launch;
  decltype(&mdh_copy_plan_destroy) copy_plan_destroy;
  decltype(&mdh_static_workspace) static_workspace;
};

constexpr int kHipMemcpyDeviceToDevice = 3;
constexpr unsigned kHipEventDisableTiming = 2;
constexpr int kHipErrorInvalidValue = 1;
constexpr int kHipErrorStreamCaptureImplicit = 906;

// Loads on first call; throws std::runtime_error naming the missing library or
// symbol.  There is no CPU fallback: without the kernel library nothing runs.
const HipRuntime& hip();

// Whether hip() has loaded the runtime and the kernel library already (it does on first GPU use).
bool hip_loaded();

// Throws when `stream` is being captured into a graph: nothing of a collective may be recorded,
// because replaying a graph that holds these launches is not supported.  Loads the runtime.
void refuse_capture(void* stream, const char* what);

// Throws std::runtime_error("<what>: <hip error string>") when rc != 0.
void check_hip(int rc, const char* what);
// Throws std::runtime_error carrying the kernel library's message when rc != 0.
void check_mdh(int rc);

} // namespace moodist
