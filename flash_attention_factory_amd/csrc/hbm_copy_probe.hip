// Plain device-to-device copy of a known size, used only to calibrate HBM traffic
// counters: profile this program and the paged-attention bench with the same
// rocprofv3 --pmc FETCH_SIZE (or WRITE_SIZE) option; the ratio
// known_bytes / counter_reading of this copy is the scale applied to the counter
// readings of the attention kernels.
//
// usage: hbm_copy_probe [MiB per buffer = 1024] [launches = 5]
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(256) hbm_copy_kernel(u32x4 *__restrict__ dst,
                                                       const u32x4 *__restrict__ src, size_t n16) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n16; i += stride) dst[i] = src[i];
}

#define CHECK(x)                                                                   \
  do {                                                                             \
    hipError_t e_ = (x);                                                           \
    if (e_ != hipSuccess) {                                                        \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                      \
      return 1;                                                                    \
    }                                                                              \
  } while (0)

int main(int argc, char **argv) {
  const size_t mib = argc > 1 ? strtoull(argv[1], nullptr, 10) : 1024;
  const int launches = argc > 2 ? atoi(argv[2]) : 5;
  const size_t bytes = mib << 20, n16 = bytes / 16;
  u32x4 *src, *dst;
  CHECK(hipMalloc(&src, bytes));
  CHECK(hipMalloc(&dst, bytes));
  CHECK(hipMemset(src, 0x5a, bytes));
  CHECK(hipMemset(dst, 0, bytes));
  hipEvent_t a, b;
  CHECK(hipEventCreate(&a));
  CHECK(hipEventCreate(&b));
  for (int it = 0; it < launches; ++it) {
    CHECK(hipEventRecord(a, nullptr));
    hipLaunchKernelGGL(hbm_copy_kernel, dim3(256 * 32), dim3(256), 0, nullptr, dst, src, n16);
    CHECK(hipEventRecord(b, nullptr));
    CHECK(hipEventSynchronize(b));
    float ms = 0.f;
    CHECK(hipEventElapsedTime(&ms, a, b));
    printf("copy %zu MiB read + %zu MiB written: %.1f us, %.1f GB/s (read+write)\n", mib, mib,
           ms * 1e3, 2.0 * bytes / (ms * 1e-3) / 1e9);
  }
  CHECK(hipDeviceSynchronize());
  return 0;
}
