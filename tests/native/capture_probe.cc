// What a stream capture records of the copy kernels' launches, compared on the host with what
// an eager launch passes.  The launches of a prepared plan (the three compiled redistributions
// of the benchmark, a dense and a padded gather) are captured into a graph; the graph's kernel
// nodes are read back with hipGraphKernelNodeGetParams and their grid, block, LDS size and
// kernel-argument bytes are compared with mdh_copy_plan_step_arguments.  The graph is destroyed
// without being instantiated: NOTHING IS REPLAYED and no kernel of this program runs.
// The library refuses a capturing stream (MDH_ECAPTURE): that is checked first, on every case,
// and only then does the program set the knob "allow_capture", which exists for this comparison.
//   capture_probe.bin <path to libmoodist_hip.so>
// Built by __graft_entry__.build() with hipcc; run by tests/test_gpu_copy.py.
#include <hip/hip_runtime.h>

#include <dlfcn.h>

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

struct Case {
  const char* name;
  int itemsize;
  int ndim;
  int64_t global[3];  // sharded over dim 0 into 8 slabs; this rank takes block 0 of the last dim
  int64_t dst_pad;    // extra elements in the destination's innermost pitch
  bool gather;        // instead: every slab whole, one under the other
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
  auto plan_create = (decltype(&mdh_copy_plan_create))dlsym(lib, "mdh_copy_plan_create");
  auto plan_launch = (decltype(&mdh_copy_plan_launch))dlsym(lib, "mdh_copy_plan_launch");
  auto plan_launches = (decltype(&mdh_copy_plan_launches))dlsym(lib, "mdh_copy_plan_launches");
  auto plan_args = (decltype(&mdh_copy_plan_step_arguments))dlsym(lib, "mdh_copy_plan_step_arguments");
  auto plan_destroy = (decltype(&mdh_copy_plan_destroy))dlsym(lib, "mdh_copy_plan_destroy");
  auto last_error = (decltype(&mdh_last_error))dlsym(lib, "mdh_last_error");
  auto set_tuning = (decltype(&mdh_set_tuning))dlsym(lib, "mdh_set_tuning");
  if (!plan_create || !plan_launch || !plan_launches || !plan_args || !plan_destroy || !last_error || !set_tuning) {
    std::printf("missing symbol\n");
    return 2;
  }
  const int P = 8;
  const Case cases[] = {
      {"fp32 8192x8192 row->column", 4, 2, {8192, 8192, 1}, 0, false},
      {"bf16 8192x8192 row->column", 2, 2, {8192, 8192, 1}, 0, false},
      {"bf16 [64,512,1024] dim0->dim2", 2, 3, {64, 512, 1024}, 0, false},
      {"bf16 8 x [512,4096] gather, dense", 2, 2, {4096, 4096, 1}, 0, true},
      {"bf16 8 x [512,4096] gather, padded pitch", 2, 2, {4096, 4096, 1}, 64, true},
  };
  hipStream_t stream;
  CK(hipStreamCreate(&stream));
  int failures = 0;
  for (const Case& c : cases) {
    const int nd = c.ndim;
    int64_t slab_shape[3] = {1, 1, 1}, out_shape[3] = {1, 1, 1}, box_shape[3] = {1, 1, 1};
    int64_t total = 1;
    for (int d = 0; d < nd; ++d) {
      slab_shape[d] = out_shape[d] = box_shape[d] = c.global[d];
      total *= c.global[d];
    }
    slab_shape[0] = c.global[0] / P;
    box_shape[0] = slab_shape[0];
    if (!c.gather) {
      out_shape[nd - 1] = c.global[nd - 1] / P;
      box_shape[nd - 1] = out_shape[nd - 1];
    }
    int64_t out_pitch[3], slab_pitch[3];  // element strides, innermost first computed below
    {
      int64_t so = 1, ss = 1;
      for (int d = nd - 1; d >= 0; --d) {
        out_pitch[d] = so;
        slab_pitch[d] = ss;
        so *= out_shape[d] + (d == nd - 1 ? c.dst_pad : 0);
        ss *= slab_shape[d];
      }
    }
    int64_t out_elems = out_pitch[0] * out_shape[0];
    const size_t slab_bytes = (size_t)total / P * c.itemsize, out_bytes = (size_t)out_elems * c.itemsize;
    char *slabs = nullptr, *out = nullptr;
    CK(hipMalloc(&slabs, slab_bytes * P));
    CK(hipMalloc(&out, out_bytes));

    std::vector<mdh_box> boxes(P);
    std::vector<int32_t> src_slot(P), dst_slot(P, P);
    for (int r = 0; r < P; ++r) {
      mdh_box& b = boxes[r];
      std::memset(&b, 0, sizeof(b));
      b.ndim = nd;
      // offsets inside the bases (the plan's convention)
      b.src = (const void*)(uintptr_t)0;
      b.dst = (void*)(uintptr_t)((size_t)r * slab_shape[0] * out_pitch[0] * c.itemsize);
      for (int d = 0; d < nd; ++d) {
        b.shape[d] = box_shape[d];
        b.src_strides[d] = slab_pitch[d];
        b.dst_strides[d] = out_pitch[d];
      }
      src_slot[r] = r;
    }
    mdh_copy_plan* plan = nullptr;
    if (plan_create(boxes.data(), src_slot.data(), dst_slot.data(), P, c.itemsize, P + 1, &plan) != MDH_OK) {
      std::printf("%s: plan_create: %s\n", c.name, last_error());
      return 1;
    }
    std::vector<const void*> bases(P + 1);
    for (int r = 0; r < P; ++r) {
      bases[r] = slabs + (size_t)r * slab_bytes;
    }
    bases[P] = out;
    const int launches = plan_launches(plan);

    // what every caller gets: the launch is refused, the capture goes on undisturbed and ends
    // with an empty graph
    hipGraph_t graph = nullptr;
    if (set_tuning("allow_capture", 0) != MDH_OK) {
      std::printf("set_tuning: %s\n", last_error());
      return 1;
    }
    CK(hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed));
    const int refused = plan_launch(plan, bases.data(), P + 1, stream);
    CK(hipStreamEndCapture(stream, &graph));
    size_t refused_nodes = 0;
    CK(hipGraphGetNodes(graph, nullptr, &refused_nodes));
    CK(hipGraphDestroy(graph));
    graph = nullptr;
    if (refused != MDH_ECAPTURE || refused_nodes != 0 || !std::strstr(last_error(), "being captured")) {
      std::printf("%s: a launch on a capturing stream returned %d and recorded %zu node(s): %s\n", c.name, refused,
          refused_nodes, last_error());
      return 1;
    }
    std::printf("%-42s refused on a capturing stream, nothing recorded\n", c.name);
    if (set_tuning("allow_capture", 1) != MDH_OK) {
      std::printf("set_tuning: %s\n", last_error());
      return 1;
    }
    CK(hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed));
    const int rc = plan_launch(plan, bases.data(), P + 1, stream);
    CK(hipStreamEndCapture(stream, &graph));
    if (rc != MDH_OK) {
      std::printf("%s: plan_launch under capture: %s\n", c.name, last_error());
      return 1;
    }
    size_t nnodes = 0;
    CK(hipGraphGetNodes(graph, nullptr, &nnodes));
    std::vector<hipGraphNode_t> nodes(nnodes);
    CK(hipGraphGetNodes(graph, nodes.data(), &nnodes));
    // a stream capture gives a chain: order the kernel nodes by their dependencies' count
    std::vector<hipGraphNode_t> kernels;
    for (hipGraphNode_t n : nodes) {
      hipGraphNodeType type;
      CK(hipGraphNodeGetType(n, &type));
      if (type == hipGraphNodeTypeKernel) {
        kernels.push_back(n);
      }
    }
    bool ok = (int)kernels.size() == launches && nnodes == kernels.size();
    std::vector<int> position(kernels.size(), -1);
    for (size_t i = 0; i < kernels.size() && ok; ++i) {
      // the node's position in the chain = how many ancestors it has
      int depth = 0;
      hipGraphNode_t at = kernels[i];
      for (;;) {
        size_t ndeps = 0;
        CK(hipGraphNodeGetDependencies(at, nullptr, &ndeps));
        if (ndeps == 0) {
          break;
        }
        if (ndeps != 1) {
          ok = false;
          break;
        }
        hipGraphNode_t dep;
        CK(hipGraphNodeGetDependencies(at, &dep, &ndeps));
        at = dep;
        ++depth;
      }
      position[i] = depth;
    }
    size_t differing = 0, compared = 0;
    for (size_t i = 0; i < kernels.size() && ok; ++i) {
      hipKernelNodeParams kp;
      std::memset(&kp, 0, sizeof(kp));
      CK(hipGraphKernelNodeGetParams(kernels[i], &kp));
      std::vector<unsigned char> want(4096);
      size_t size = 0;
      uint32_t gx = 0, gy = 0, block = 0, lds = 0, leading = 0;
      if (plan_args(plan, bases.data(), P + 1, position[i], want.data(), want.size(), &size, &leading, &gx, &gy, &block,
              &lds) != MDH_OK) {
        std::printf("%s: step_arguments: %s\n", c.name, last_error());
        return 1;
      }
      const bool shape_ok = kp.gridDim.x == gx && kp.gridDim.y == gy && kp.gridDim.z == 1 && kp.blockDim.x == block &&
                            kp.blockDim.y == 1 && kp.blockDim.z == 1 && kp.sharedMemBytes == lds;
      if (!shape_ok) {
        std::printf("%s: launch %d recorded as grid %u x %u x %u, block %u, lds %u; passed %u x %u, block %u, lds %u\n",
            c.name, position[i], kp.gridDim.x, kp.gridDim.y, kp.gridDim.z, kp.blockDim.x, kp.sharedMemBytes, gx, gy,
            block, lds);
        ok = false;
      }
      if (!kp.kernelParams || !kp.kernelParams[0]) {
        std::printf("%s: launch %d: the node holds no argument array (extra = %p)\n", c.name, position[i],
            (void*)kp.extra);
        ok = false;
        continue;
      }
      // the passed block: `leading` 4-byte scalars, each a parameter of its own, then one struct
      std::vector<unsigned char> recorded(size);
      bool complete = true;
      for (uint32_t k = 0; k <= leading; ++k) {
        if (!kp.kernelParams[k]) {
          complete = false;
          break;
        }
        if (k < leading) {
          std::memcpy(recorded.data() + 4 * k, kp.kernelParams[k], 4);
        } else {
          std::memcpy(recorded.data() + 4 * leading, kp.kernelParams[k], size - 4 * leading);
        }
      }
      if (!complete) {
        std::printf("%s: launch %d: the node holds fewer than %u parameters\n", c.name, position[i], leading + 1);
        ok = false;
        continue;
      }
      const unsigned char* got = recorded.data();
      size_t first = size;
      for (size_t k = 0; k < size; ++k) {
        if (got[k] != want[k]) {
          if (first == size) {
            first = k;
          }
          ++differing;
        }
      }
      compared += size;
      if (first != size) {
        std::printf("%s: launch %d: recorded argument bytes differ from the passed ones, first at byte %zu of %zu\n",
            c.name, position[i], first, size);
        ok = false;
      }
    }
    std::printf("%-42s %d launch(es), %zu kernel node(s) of %zu, %zu argument bytes compared, %zu differ: %s\n", c.name,
        launches, kernels.size(), nnodes, compared, differing, ok ? "same" : "DIFFERENT");
    failures += ok ? 0 : 1;
    CK(hipGraphDestroy(graph));
    plan_destroy(plan);
    CK(hipFree(slabs));
    CK(hipFree(out));
  }
  CK(hipStreamDestroy(stream));
  std::printf(failures ? "FAILED\n" : "OK\n");
  return failures ? 1 : 0;
}
