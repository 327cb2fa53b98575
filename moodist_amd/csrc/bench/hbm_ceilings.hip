// Measures what one MI355X delivers to plain streaming loops of the same shape
// as the library's kernels (256 lanes x U sub-tiles x 16 bytes per workgroup,
// buffer addressing): read only, write only, copy in one kernel, a read kernel
// followed by a write kernel, eight streams read only, and eight streams folded
// into one written stream under several cache policies, plus the period of
// back-to-back empty launches.  These are the ceilings the kernels' measured
// rates are judged against.
//
//   hbm_ceilings [MiB per stream, default 16]
//
// Every case rotates over six buffer sets (footprint well above twice the
// 256 MB Infinity Cache at the default size) and times 120 launches with HIP
// events after 10 warm-up launches.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define CHECK(x)                                                          \
  do {                                                                    \
    hipError_t e_ = (x);                                                  \
    if (e_ != hipSuccess) {                                               \
      std::printf("%s failed: %s\n", #x, hipGetErrorString(e_));          \
      std::exit(1);                                                       \
    }                                                                     \
  } while (0)

constexpr int kNt = 2, kSc1 = 16; // cache-policy bits of the buffer intrinsics' aux operand on gfx940+

__device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, (int)bytes, 0x00020000);
}

// K streams read and folded; one stream written unless WRITE is false.
template<int K, int U, int LAUX, int SAUX, bool WRITE>
__global__ __launch_bounds__(256) void fold_kernel(const char* src, size_t stride, char* dst, size_t ntiles) {
  constexpr uint32_t tile_bytes = 256 * U * 16;
  u32x4 keep = {0, 0, 0, 0};
  for (size_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
    u32x4 v[K][U];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const __amdgpu_buffer_rsrc_t rs = rsrc(src + (size_t)k * stride + tile * tile_bytes, tile_bytes);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        v[k][u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, threadIdx.x * 16 + u * 4096, 0, LAUX));
      }
    }
    const __amdgpu_buffer_rsrc_t rd = rsrc(dst + tile * tile_bytes, tile_bytes);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      f32x4 acc = __builtin_bit_cast(f32x4, v[0][u]);
#pragma unroll
      for (int k = 1; k < K; ++k) {
        acc += __builtin_bit_cast(f32x4, v[k][u]);
      }
      if (WRITE) {
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc), rd, threadIdx.x * 16 + u * 4096, 0, SAUX);
      } else {
        keep |= __builtin_bit_cast(u32x4, acc);
      }
    }
  }
  if (!WRITE && keep.x == 0x12345678u && keep.y == 0x9abcdef1u) { // never true: keeps the loads alive
    ((u32x4*)dst)[threadIdx.x] = keep;
  }
}

template<int U, int SAUX>
__global__ __launch_bounds__(256) void fill_kernel(char* dst, size_t ntiles) {
  constexpr uint32_t tile_bytes = 256 * U * 16;
  const u32x4 value = {1, 2, 3, threadIdx.x};
  for (size_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
    const __amdgpu_buffer_rsrc_t rd = rsrc(dst + tile * tile_bytes, tile_bytes);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      __builtin_amdgcn_raw_buffer_store_b128(value, rd, threadIdx.x * 16 + u * 4096, 0, SAUX);
    }
  }
}

__global__ __launch_bounds__(256) void empty_kernel(const char*, size_t, char*, size_t) {}

int main(int argc, char** argv) {
  const size_t mib = argc > 1 ? (size_t)std::atol(argv[1]) : 16;
  const size_t stream = mib << 20; // bytes per stream
  constexpr int K = 8, kSets = 6;
  const size_t set_bytes = stream * (K + 1);
  char* buf;
  CHECK(hipMalloc(&buf, set_bytes * kSets));
  CHECK(hipMemset(buf, 1, set_bytes * kSets));
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));

  auto run = [&](const char* name, double bytes, auto launch) {
    for (int i = 0; i < 10; ++i) {
      launch(i % kSets);
    }
    CHECK(hipDeviceSynchronize());
    const int iters = 120;
    CHECK(hipEventRecord(e0, 0));
    for (int i = 0; i < iters; ++i) {
      launch(i % kSets);
    }
    CHECK(hipEventRecord(e1, 0));
    CHECK(hipEventSynchronize(e1));
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    const double us = ms * 1e3 / iters;
    std::printf("%-58s %9.2f us %7.3f TB/s %5.1f %% of 8 TB/s\n", name, us, bytes / us / 1e6, bytes / us / 1e6 / 8 * 100);
    std::fflush(stdout);
  };
  auto set = [&](int s) { return buf + set_bytes * s; };

  std::printf("%zu MiB per stream, %d buffer sets of %zu MiB\n", mib, kSets, set_bytes >> 20);
  {
    // what a launch costs before it moves a byte: back-to-back empty kernels of the headline grid
    const int iters = 2000;
    for (int i = 0; i < 50; ++i) {
      hipLaunchKernelGGL(empty_kernel, dim3(1024), dim3(256), 0, 0, buf, 0, buf, 0);
    }
    CHECK(hipDeviceSynchronize());
    CHECK(hipEventRecord(e0, 0));
    for (int i = 0; i < iters; ++i) {
      hipLaunchKernelGGL(empty_kernel, dim3(1024), dim3(256), 0, 0, buf, 0, buf, 0);
    }
    CHECK(hipEventRecord(e1, 0));
    CHECK(hipEventSynchronize(e1));
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    std::printf("%-58s %9.2f us per launch\n", "empty kernel, 1024 workgroups, back to back", ms * 1e3 / iters);
  }
  const size_t whole = stream * 8;                 // the eight streams taken as one region
  const size_t t4 = 256 * 4 * 16, t1 = 256 * 16;
  run("read only, one stream of 8x, nt loads", (double)whole,
      [&](int s) { hipLaunchKernelGGL((fold_kernel<1, 4, kNt, 0, false>), dim3(whole / t4), dim3(256), 0, 0, set(s), 0, set(s), whole / t4); });
  run("read only, one stream of 8x, plain loads", (double)whole,
      [&](int s) { hipLaunchKernelGGL((fold_kernel<1, 4, 0, 0, false>), dim3(whole / t4), dim3(256), 0, 0, set(s), 0, set(s), whole / t4); });
  run("write only, 8x, one sub-tile, sc1 stores", (double)whole,
      [&](int s) { hipLaunchKernelGGL((fill_kernel<1, kSc1>), dim3(whole / t1), dim3(256), 0, 0, set(s), whole / t1); });
  run("write only, 8x, four sub-tiles, sc1 stores", (double)whole,
      [&](int s) { hipLaunchKernelGGL((fill_kernel<4, kSc1>), dim3(whole / t4), dim3(256), 0, 0, set(s), whole / t4); });
  const size_t half = whole / 2;
  run("copy 4x -> 4x in one kernel, nt loads, sc1 stores", (double)whole,
      [&](int s) { hipLaunchKernelGGL((fold_kernel<1, 4, kNt, kSc1, true>), dim3(half / t4), dim3(256), 0, 0, set(s), 0, set(s) + half, half / t4); });
  // an unused dynamic LDS allocation caps the workgroups resident on a CU: 40 KiB -> four, 64 KiB -> two
  run("copy 4x -> 4x, nt/sc1, two sub-tiles, four workgroups per CU", (double)whole,
      [&](int s) { hipLaunchKernelGGL((fold_kernel<1, 2, kNt, kSc1, true>), dim3(half / (t4 / 2)), dim3(256), 40960, 0, set(s), 0, set(s) + half, half / (t4 / 2)); });
  run("copy 4x -> 4x in one kernel, plain loads and stores", (double)whole,
      [&](int s) { hipLaunchKernelGGL((fold_kernel<1, 4, 0, 0, true>), dim3(half / t4), dim3(256), 0, 0, set(s), 0, set(s) + half, half / t4); });
  run("read kernel (4x) then write kernel (4x), same stream", (double)whole, [&](int s) {
    hipLaunchKernelGGL((fold_kernel<1, 4, kNt, 0, false>), dim3(half / t4), dim3(256), 0, 0, set(s), 0, set(s), half / t4);
    hipLaunchKernelGGL((fill_kernel<1, kSc1>), dim3(half / t1), dim3(256), 0, 0, set(s) + half, half / t1);
  });
  run("hipMemcpyAsync device to device, 4x -> 4x", (double)whole,
      [&](int s) { CHECK(hipMemcpyAsync(set(s) + half, set(s), half, hipMemcpyDeviceToDevice, 0)); });
  const double nine = (double)stream * 9;
  run("8 streams read only (no store), four sub-tiles", (double)stream * 8,
      [&](int s) { hipLaunchKernelGGL((fold_kernel<8, 4, kNt, 0, false>), dim3(stream / t4), dim3(256), 0, 0, set(s), stream, set(s) + stream * 8, stream / t4); });
  run("8 streams -> 1, nt loads, sc1 stores, four sub-tiles", nine,
      [&](int s) { hipLaunchKernelGGL((fold_kernel<8, 4, kNt, kSc1, true>), dim3(stream / t4), dim3(256), 0, 0, set(s), stream, set(s) + stream * 8, stream / t4); });
  run("8 streams -> 1, nt loads, nt stores, four sub-tiles", nine,
      [&](int s) { hipLaunchKernelGGL((fold_kernel<8, 4, kNt, kNt, true>), dim3(stream / t4), dim3(256), 0, 0, set(s), stream, set(s) + stream * 8, stream / t4); });
  run("8 streams -> 1, plain loads and stores, four sub-tiles", nine,
      [&](int s) { hipLaunchKernelGGL((fold_kernel<8, 4, 0, 0, true>), dim3(stream / t4), dim3(256), 0, 0, set(s), stream, set(s) + stream * 8, stream / t4); });
  run("8 streams -> 1, nt loads, sc1 stores, two sub-tiles", nine,
      [&](int s) { hipLaunchKernelGGL((fold_kernel<8, 2, kNt, kSc1, true>), dim3(stream / (t4 / 2)), dim3(256), 0, 0, set(s), stream, set(s) + stream * 8, stream / (t4 / 2)); });
  run("8 streams -> 1, nt loads, sc1 stores, one sub-tile", nine,
      [&](int s) { hipLaunchKernelGGL((fold_kernel<8, 1, kNt, kSc1, true>), dim3(stream / t1), dim3(256), 0, 0, set(s), stream, set(s) + stream * 8, stream / t1); });
  run("8 streams -> 1, nt/sc1, one sub-tile, two workgroups per CU", nine,
      [&](int s) { hipLaunchKernelGGL((fold_kernel<8, 1, kNt, kSc1, true>), dim3(stream / t1), dim3(256), 65536, 0, set(s), stream, set(s) + stream * 8, stream / t1); });
  run("8 streams -> 1, nt/sc1, four sub-tiles, persistent grid of 256", nine,
      [&](int s) { hipLaunchKernelGGL((fold_kernel<8, 4, kNt, kSc1, true>), dim3(256), dim3(256), 0, 0, set(s), stream, set(s) + stream * 8, stream / t4); });
  return 0;
}
