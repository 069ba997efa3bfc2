// Measurement aid, built into its own small library that only the benchmark loads:
// a plain streaming copy of known size, against which a profiler's HBM byte counters
// (FETCH_SIZE, WRITE_SIZE) are calibrated.  Not part of the decode library or of its
// interface.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {
__global__ __launch_bounds__(256) void copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                   int64_t n_vec) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec;
       i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}
}  // namespace

// Copies n_bytes (a multiple of 16, both pointers 16-byte aligned) on `stream`, 16 bytes
// per lane.  Returns 0, -1 for arguments it refuses, or the HIP error code of the launch.
extern "C" int calibration_copy(const void* src, void* dst, int64_t n_bytes, void* stream) {
  if (!src || !dst || n_bytes <= 0 || (n_bytes & 15)) return -1;
  if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) return -1;
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(copy_kernel, dim3((unsigned)(cus * 8)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(src), static_cast<uint4*>(dst), n_bytes / 16);
  return (int)hipGetLastError();
}
