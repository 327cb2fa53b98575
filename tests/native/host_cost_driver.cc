// Host cost of enqueuing one compiled redistribution, measured from a C++ loop: the general
// entry point (mdh_copy_boxes: checks, merges and tiles the boxes on every call) against a
// prepared plan (mdh_copy_plan_launch: patches addresses into kernel arguments made once).
// Also checks that both produce the same bytes.  Needs a GPU.
//   host_cost_driver.bin <path to libmoodist_hip.so>
// Built by __graft_entry__.build() with hipcc; run by tests/test_gpu_copy.py.
#include <hip/hip_runtime.h>

#include <dlfcn.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "moodist_hip.h"

#define CK(x)                                                                   \
  do {                                                                          \
    hipError_t e = (x);                                                         \
    if (e != hipSuccess) {                                                      \
      std::printf("HIP error %s at line %d\n", hipGetErrorString(e), __LINE__); \
      return 1;                                                                 \
    }                                                                           \
  } while (0)

struct Shape {
  const char* name;
  int itemsize;
  int ndim;
  int64_t global[3]; // whole tensor; sharded over dim 0 into 8 slabs, this rank takes block 0 of the last dim
};

int main(int argc, char** argv) {
  if (argc < 2) {
    std::printf("usage: %s libmoodist_hip.so\n", argv[0]);
    return 2;
  }
  void* lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  if (!lib) {
    std::printf("dlopen: %s\n", dlerror());
    return 2;
  }
  auto copy_boxes = (decltype(&mdh_copy_boxes))dlsym(lib, "mdh_copy_boxes");
  auto plan_create = (decltype(&mdh_copy_plan_create))dlsym(lib, "mdh_copy_plan_create");
  auto plan_launch = (decltype(&mdh_copy_plan_launch))dlsym(lib, "mdh_copy_plan_launch");
  auto plan_destroy = (decltype(&mdh_copy_plan_destroy))dlsym(lib, "mdh_copy_plan_destroy");
  auto last_error = (decltype(&mdh_last_error))dlsym(lib, "mdh_last_error");
  if (!copy_boxes || !plan_create || !plan_launch || !plan_destroy || !last_error) {
    std::printf("missing symbol\n");
    return 2;
  }
  const int P = 8;
  const Shape shapes[] = {{"fp32 8192x8192 row->column", 4, 2, {8192, 8192, 1}},
      {"bf16 8192x8192 row->column", 2, 2, {8192, 8192, 1}}, {"bf16 [64,512,1024] dim0->dim2", 2, 3, {64, 512, 1024}}};
  int failures = 0;
  for (const Shape& sh : shapes) {
    const int nd = sh.ndim;
    int64_t slab_shape[3], out_shape[3], box_shape[3];
    int64_t total = 1;
    for (int d = 0; d < nd; ++d) {
      slab_shape[d] = out_shape[d] = box_shape[d] = sh.global[d];
      total *= sh.global[d];
    }
    slab_shape[0] = sh.global[0] / P;
    out_shape[nd - 1] = sh.global[nd - 1] / P;
    box_shape[0] = slab_shape[0];
    box_shape[nd - 1] = out_shape[nd - 1];
    const size_t slab_bytes = (size_t)total / P * sh.itemsize, out_bytes = slab_bytes;
    char* slabs = nullptr;
    char *out_a = nullptr, *out_b = nullptr;
    CK(hipMalloc(&slabs, slab_bytes * P));
    CK(hipMalloc(&out_a, out_bytes));
    CK(hipMalloc(&out_b, out_bytes));
    std::vector<unsigned char> h(slab_bytes * P);
    unsigned s = 12345;
    for (auto& x : h) {
      s = s * 1664525u + 1013904223u;
      x = (unsigned char)(s >> 24);
    }
    CK(hipMemcpy(slabs, h.data(), h.size(), hipMemcpyHostToDevice));
    CK(hipMemset(out_a, 0, out_bytes));
    CK(hipMemset(out_b, 0xff, out_bytes));
    // element strides of the contiguous slab and output
    int64_t sstr[3], dstr[3];
    int64_t a = 1, b = 1;
    for (int d = nd; d-- > 0;) {
      sstr[d] = a, dstr[d] = b;
      a *= slab_shape[d], b *= out_shape[d];
    }
    std::vector<mdh_box> boxes(P), offsets(P);
    std::vector<int32_t> src_slots(P), dst_slots(P);
    std::vector<const void*> bases(P + 1);
    for (int r = 0; r < P; ++r) {
      mdh_box bx{};
      bx.ndim = nd;
      for (int d = 0; d < nd; ++d) {
        bx.shape[d] = box_shape[d], bx.src_strides[d] = sstr[d], bx.dst_strides[d] = dstr[d];
      }
      const size_t dst_off = (size_t)r * box_shape[0] * dstr[0] * sh.itemsize;
      offsets[r] = bx;
      offsets[r].src = (const void*)(uintptr_t)0; // this rank's block of the last dimension is block 0
      offsets[r].dst = (void*)(uintptr_t)dst_off;
      src_slots[r] = r, dst_slots[r] = P;
      bases[r] = slabs + (size_t)r * slab_bytes;
      bx.src = bases[r];
      bx.dst = out_a + dst_off;
      boxes[r] = bx;
    }
    bases[P] = out_b;
    mdh_copy_plan* plan = nullptr;
    if (plan_create(offsets.data(), src_slots.data(), dst_slots.data(), P, sh.itemsize, P + 1, &plan)) {
      std::printf("plan_create: %s\n", last_error());
      return 1;
    }
    // Bursts of 128 calls, each burst followed by an untimed synchronize: the queue never fills,
    // so the time measured is the host's alone, whatever the kernels take.
    const int kBurst = 128, kBursts = 100, N = kBurst * kBursts;
    auto time_loop = [&](auto&& call) {
      for (int i = 0; i < 200; ++i) {
        call();
      }
      (void)hipDeviceSynchronize();
      std::vector<double> per_call(kBursts);
      for (int b = 0; b < kBursts; ++b) {
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < kBurst; ++i) {
          call();
        }
        const auto t1 = std::chrono::steady_clock::now();
        (void)hipDeviceSynchronize();
        per_call[b] = std::chrono::duration<double, std::micro>(t1 - t0).count() / kBurst;
      }
      // the median burst: a burst during which the thread lost its core does not move it
      std::sort(per_call.begin(), per_call.end());
      return per_call[kBursts / 2];
    };
    int rc = 0;
    const double general = time_loop([&] { rc |= copy_boxes(boxes.data(), P, sh.itemsize, nullptr); });
    const double prepared = time_loop([&] { rc |= plan_launch(plan, bases.data(), P + 1, nullptr); });
    if (rc) {
      std::printf("launch failed: %s\n", last_error());
      return 1;
    }
    std::vector<unsigned char> ra(out_bytes), rb(out_bytes);
    CK(hipMemcpy(ra.data(), out_a, out_bytes, hipMemcpyDeviceToHost));
    CK(hipMemcpy(rb.data(), out_b, out_bytes, hipMemcpyDeviceToHost));
    const bool same = std::memcmp(ra.data(), rb.data(), out_bytes) == 0;
    failures += !same;
    std::printf("%-32s host us per call: general %.2f  prepared %.2f  (median of %d calls each in bursts of %d)  outputs %s\n", sh.name,
        general, prepared, N, kBurst, same ? "identical" : "DIFFER");
    plan_destroy(plan);
    CK(hipFree(slabs));
    CK(hipFree(out_a));
    CK(hipFree(out_b));
  }
  std::puts(failures ? "host cost driver: FAILED" : "host cost driver done");
  return failures ? 1 : 0;
}
