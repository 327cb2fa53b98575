// Error reporting, launch checking and tuning knobs shared by the C ABI.
#include "device_common.h"

#include <cstring>

namespace mdh {

namespace {
thread_local char g_error[512] = "";
}

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return MDH_ELAUNCH;
  }
  return MDH_OK;
}

Tuning& tuning() {
  static Tuning t;
  return t;
}

int refuse_capture(hipStream_t stream, const char* who) {
  if (tuning().allow_capture) {
    return MDH_OK;
  }
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  const hipError_t e = hipStreamIsCapturing(stream, &status);
  // the legacy default stream reports a capture going on elsewhere as an error of its own
  const bool capturing = e == hipSuccess ? status != hipStreamCaptureStatusNone : e == hipErrorStreamCaptureImplicit;
  if (e != hipSuccess) {
    (void)hipGetLastError(); // no device, or an unknown stream: the launch itself will say so
  }
  if (!capturing) {
    return MDH_OK;
  }
  set_error("%s: the stream is being captured into a graph; capture and replay of these launches is not supported "
            "(launch on a stream that is not capturing)", who);
  return MDH_ECAPTURE;
}

} // namespace mdh

extern "C" int mdh_abi_version(void) {
  return MDH_ABI_VERSION;
}

extern "C" const char* mdh_last_error(void) {
  return mdh::g_error;
}

extern "C" const char* mdh_error_string(int code) {
  switch (code) {
  case MDH_OK:
    return "success";
  case MDH_EINVAL:
    return "invalid argument";
  case MDH_EDTYPE:
    return "Unsupported dtype for reduce operation";
  case MDH_EOP:
    return "Unsupported reduce operation";
  case MDH_ELAUNCH:
    return "kernel launch failed";
  case MDH_ENODEVICE:
    return "no usable gfx950 device";
  case MDH_ECAPTURE:
    return "the stream is being captured into a graph, which these launches do not support";
  default:
    return "unknown error";
  }
}

namespace {
int* knob(const char* name) {
  mdh::Tuning& t = mdh::tuning();
  if (!name) {
    return nullptr;
  }
  if (!std::strcmp(name, "reduce_unroll")) {
    return &t.reduce_unroll;
  }
  if (!std::strcmp(name, "reduce_chunk")) {
    return &t.reduce_chunk;
  }
  if (!std::strcmp(name, "reduce_max_blocks")) {
    return &t.reduce_max_blocks;
  }
  if (!std::strcmp(name, "reduce_split_tiles")) {
    return &t.reduce_split_tiles;
  }
  if (!std::strcmp(name, "reduce_wg_per_cu")) {
    return &t.reduce_wg_per_cu;
  }
  if (!std::strcmp(name, "copy_unroll")) {
    return &t.copy_unroll;
  }
  if (!std::strcmp(name, "box_unroll")) {
    return &t.box_unroll;
  }
  if (!std::strcmp(name, "copy_wg_per_cu")) {
    return &t.copy_wg_per_cu;
  }
  if (!std::strcmp(name, "box_policy")) {
    return &t.box_policy;
  }
  if (!std::strcmp(name, "box_preload")) {
    return &t.box_preload;
  }
  if (!std::strcmp(name, "box_transpose_tile")) {
    return &t.box_transpose_tile;
  }
  if (!std::strcmp(name, "box_transpose")) {
    return &t.box_transpose;
  }
  if (!std::strcmp(name, "box_transpose_wgs")) {
    return &t.box_transpose_wgs;
  }
  if (!std::strcmp(name, "box_tile_cols")) {
    return &t.box_tile_cols;
  }
  if (!std::strcmp(name, "copy_max_blocks")) {
    return &t.copy_max_blocks;
  }
  if (!std::strcmp(name, "copy_xcd_run")) {
    return &t.copy_xcd_run;
  }
  if (!std::strcmp(name, "copy_grid_order")) {
    return &t.copy_grid_order;
  }
  if (!std::strcmp(name, "copy_tail_tiles")) {
    return &t.copy_tail_tiles;
  }
  if (!std::strcmp(name, "copy_lds")) {
    return &t.copy_lds;
  }
  if (!std::strcmp(name, "allow_capture")) {
    return &t.allow_capture;
  }
  return nullptr;
}
} // namespace

extern "C" int mdh_set_tuning(const char* name, int value) {
  int* k = knob(name);
  if (!k) {
    mdh::set_error("mdh_set_tuning: unknown knob");
    return MDH_EINVAL;
  }
  const bool unroll = std::strstr(name, "unroll") != nullptr || !std::strcmp(name, "reduce_chunk");
  if (unroll) {
    const bool sixteen = value == 16 && !std::strcmp(name, "reduce_unroll");
    if (!(value == 0 || value == 1 || value == 2 || value == 4 || value == 8 || sixteen)) {
      mdh::set_error("mdh_set_tuning: %s does not take %d", name, value);
      return MDH_EINVAL;
    }
  } else if (!std::strcmp(name, "box_tile_cols") || !std::strcmp(name, "copy_xcd_run")) {
    if (value < 0 || (value & (value - 1)) != 0 || value > 2048) {
      mdh::set_error("mdh_set_tuning: %s takes a power of two up to 2048, not %d", name, value);
      return MDH_EINVAL;
    }
  } else if (value < 0 || (std::strstr(name, "wg_per_cu") && value > 9) || (!std::strcmp(name, "box_policy") && value > 2) ||
             (!std::strcmp(name, "box_preload") && value > 1) || (!std::strcmp(name, "box_transpose") && value > 3) || (!std::strcmp(name, "box_transpose_tile") && value > 3) || (!std::strcmp(name, "allow_capture") && value > 1)) {
    mdh::set_error("mdh_set_tuning: %s does not take %d", name, value);
    return MDH_EINVAL;
  }
  *k = value;
  return MDH_OK;
}

extern "C" int mdh_get_tuning(const char* name, int* value) {
  int* k = knob(name);
  if (!k || !value) {
    mdh::set_error("mdh_get_tuning: unknown knob");
    return MDH_EINVAL;
  }
  *value = *k;
  return MDH_OK;
}
