// The library's fp32 -> bf16 narrowing (mdh::Traits<mdh::bf16_t>::narrow, which compiles to the
// hardware conversion of gfx950) against the rule it has to follow, for every one of the 2^32
// fp32 bit patterns: round to nearest, ties to even; a NaN keeps its sign and upper payload
// bits and gets the quiet bit.  Also widen(narrow(x)) == x for every bf16 pattern.
//   bf16_narrow_check.bin
// Built by __graft_entry__.build() with hipcc for gfx950; run by tests/test_gpu_reduce.py.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

#include "reduce_kernels.h"

#define CK(x)                                                                   \
  do {                                                                          \
    hipError_t e = (x);                                                         \
    if (e != hipSuccess) {                                                      \
      std::printf("HIP error %s at line %d\n", hipGetErrorString(e), __LINE__); \
      return 1;                                                                 \
    }                                                                           \
  } while (0)

// the rule, written out (what the CPU oracle's restatement does as well)
__device__ __forceinline__ uint16_t rule(uint32_t u) {
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    return (uint16_t)((u >> 16) | 0x0040u);
  }
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

struct Report {
  unsigned long long differing;
  unsigned long long slots;
  uint32_t first[16][3];
};

__global__ void check_all(Report* r) {
  const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint64_t n = (uint64_t)gridDim.x * blockDim.x;
  unsigned long long bad = 0;
  for (uint64_t u = tid; u < (1ull << 32); u += n) {
    const uint16_t want = rule((uint32_t)u);
    const uint16_t got = mdh::Traits<mdh::bf16_t>::narrow(__uint_as_float((uint32_t)u));
    if (want != got) {
      if (bad == 0) {
        const unsigned long long slot = atomicAdd(&r->slots, 1ull);
        if (slot < 16) {
          r->first[slot][0] = (uint32_t)u;
          r->first[slot][1] = want;
          r->first[slot][2] = got;
        }
      }
      ++bad;
    }
  }
  // every bf16 pattern survives widening and narrowing (NaNs come back quiet)
  if (tid < 65536) {
    const uint16_t h = (uint16_t)tid;
    const uint16_t back = mdh::Traits<mdh::bf16_t>::narrow(mdh::Traits<mdh::bf16_t>::widen(h));
    const bool nan = (h & 0x7fffu) > 0x7f80u;
    if (back != (nan ? (uint16_t)(h | 0x0040u) : h)) {
      ++bad;
    }
  }
  if (bad) {
    atomicAdd(&r->differing, bad);
  }
}

int main() {
  Report* dev = nullptr;
  CK(hipMalloc(&dev, sizeof(Report)));
  CK(hipMemset(dev, 0, sizeof(Report)));
  hipLaunchKernelGGL(check_all, dim3(4096), dim3(256), 0, 0, dev);
  CK(hipGetLastError());
  CK(hipDeviceSynchronize());
  Report host;
  CK(hipMemcpy(&host, dev, sizeof(Report), hipMemcpyDeviceToHost));
  std::printf("4294967296 fp32 patterns and 65536 bf16 patterns checked, %llu differ\n", host.differing);
  for (unsigned long long i = 0; i < host.slots && i < 16; ++i) {
    std::printf("  fp32 %08x: rule %04x, library %04x\n", host.first[i][0], host.first[i][1], host.first[i][2]);
  }
  CK(hipFree(dev));
  return host.differing ? 1 : 0;
}
