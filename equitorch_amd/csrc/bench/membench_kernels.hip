// Plain streaming kernels of known traffic, used by the benchmark script to calibrate hardware counters and to read
// the achievable HBM bandwidth of the device next to the tensor-product kernels.  Built into libcgtp_bench.so, which
// is not part of the product's C ABI.  copy: reads n_bytes and writes n_bytes; read: reads n_bytes; n_bytes must be a
// multiple of 16 and the pointers 16-byte aligned; status codes as in cgtp.h.
#include "cgtp_device.h"
#include "cgtp_host.h"

namespace cgtp {

__global__ void __launch_bounds__(256) copy_kernel(const f32x4* __restrict__ src, f32x4* __restrict__ dst, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

__global__ void __launch_bounds__(256) read_kernel(const f32x4* __restrict__ src, float* __restrict__ sink, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    acc += __builtin_nontemporal_load(src + i);
  const float s = acc.x + acc.y + acc.z + acc.w;
  if (s == 123456.789f) *sink = s;  // keeps the loads alive; practically never true
}


}  // namespace cgtp

using namespace cgtp;

extern "C" {

int cgtpbench_copy(void* dst, const void* src, int64_t n_bytes, void* stream) {
  if (!dst || !src) return CGTP_ERR_NULL;
  if (n_bytes < 0 || (n_bytes & 15)) return CGTP_ERR_SHAPE;
  if (((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u) != 0) return CGTP_ERR_ALIGN;
  if (n_bytes == 0) return CGTP_OK;
  hipLaunchKernelGGL(copy_kernel, dim3(256 * 16), dim3(256), 0, (hipStream_t)stream, (const f32x4*)src,
                     (f32x4*)dst, n_bytes / 16);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

int cgtpbench_read(const void* src, void* sink, int64_t n_bytes, void* stream) {
  if (!src || !sink) return CGTP_ERR_NULL;
  if (n_bytes < 0 || (n_bytes & 15)) return CGTP_ERR_SHAPE;
  if ((reinterpret_cast<uintptr_t>(src) & 15u) != 0) return CGTP_ERR_ALIGN;
  if (n_bytes == 0) return CGTP_OK;
  hipLaunchKernelGGL(read_kernel, dim3(256 * 16), dim3(256), 0, (hipStream_t)stream, (const f32x4*)src,
                     (float*)sink, n_bytes / 16);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

}  // extern "C"
