// Counter calibration for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE: launches a
// plain copy kernel that reads exactly N bytes and writes exactly N bytes, so
// that what the counters report for it fixes their scale on this device.
// It then times the runtime's own device-to-device copy of the same buffers
// (hipMemcpyAsync, 5 repetitions after a warm-up): the copy ceiling that the
// streaming pass's read rate is quoted next to.
//   usage: copy_probe [MiB = 1024] [launches = 3]
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>

typedef double v2d __attribute__((ext_vector_type(2)));

__global__ __launch_bounds__(256) void plain_copy(const v2d* __restrict__ src,
                                                  v2d* __restrict__ dst, size_t nvec) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < nvec; i += stride) dst[i] = src[i];
}

#define CK(x)                                                              \
  do {                                                                     \
    hipError_t e_ = (x);                                                   \
    if (e_ != hipSuccess) {                                                \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));              \
      return 1;                                                            \
    }                                                                      \
  } while (0)

int main(int argc, char** argv) {
  const size_t mib = argc > 1 ? (size_t)atol(argv[1]) : 1024;
  const int launches = argc > 2 ? atoi(argv[2]) : 3;
  const size_t bytes = mib << 20;
  v2d *src = nullptr, *dst = nullptr;
  CK(hipMalloc(&src, bytes));
  CK(hipMalloc(&dst, bytes));
  CK(hipMemset(src, 1, bytes));
  CK(hipMemset(dst, 0, bytes));
  CK(hipDeviceSynchronize());
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  float total = 0.f;
  for (int i = 0; i < launches; ++i) {
    CK(hipEventRecord(e0, 0));
    hipLaunchKernelGGL(plain_copy, dim3(256 * 8), dim3(256), 0, 0, src, dst, bytes / sizeof(v2d));
    CK(hipEventRecord(e1, 0));
    CK(hipDeviceSynchronize());
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    total += ms;
  }
  printf("plain_copy: %d launches, each reads %zu bytes and writes %zu bytes; %.3f ms avg, "
         "%.1f GB/s read+write\n", launches, bytes, bytes, total / launches,
         2.0 * bytes / (total / launches) * 1e-6);
  const int reps = 5;
  CK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, 0));
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0, 0));
  for (int i = 0; i < reps; ++i) CK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, 0));
  CK(hipEventRecord(e1, 0));
  CK(hipDeviceSynchronize());
  float ms = 0.f;
  CK(hipEventElapsedTime(&ms, e0, e1));
  printf("hipMemcpy device-to-device: %d copies of %zu bytes; %.3f ms avg, %.1f GB/s read+write "
         "(%.1f GB/s each way)\n", reps, bytes, ms / reps, 2.0 * bytes / (ms / reps) * 1e-6,
         1.0 * bytes / (ms / reps) * 1e-6);
  CK(hipFree(src));
  CK(hipFree(dst));
  return 0;
}
