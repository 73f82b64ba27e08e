// Plain streaming kernels of known traffic, used by the benchmark script to calibrate hardware counters and to read
// the achievable HBM bandwidth of the device next to the tensor-product kernels.  Built into libcgtp_bench.so, which
// is not part of the product's C ABI.  copy: reads n_bytes and writes n_bytes; read: reads n_bytes; n_bytes must be a
// multiple of 16 and the pointers 16-byte aligned; status codes as in cgtp.h.
// lds_read: the rate at which wavefronts read LDS with ds_read_b128, ds_read_b64 or ds_read_b64_tr_b16 (the transpose
// read the bf16 weight-gradient kernel forms its matrix operands with), in the tile layouts that kernel can use.
// coissue: how much vector-ALU work (independent fp32 FMAs) hides behind matrix instructions on one SIMD, issued by
// the same wavefront (interleaved or in blocks) or by another wavefront of the SIMD.
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


// KIND 0: ds_read_b64_tr_b16, 1: ds_read_b64, 2: ds_read_b128.  Every wavefront issues eight reads, waits for them,
// and repeats.  Addresses (KIND 0 / 1): a tile of rows `pitch` bytes apart; lane group q = lane / 16 reads 32 bytes
// of each of four rows, rows 8q .. 8q+3 (row_mode 0) or 4q .. 4q+3 (row_mode 1); row_mode 2 and KIND 2: contiguous.
template <int KIND>
__global__ void __launch_bounds__(256) lds_read_kernel(int* __restrict__ out, int iters, int pitch, int row_mode) {
  extern __shared__ __align__(16) unsigned char smem[];
  typedef int i32x2 __attribute__((ext_vector_type(2)));
  typedef int i32x4 __attribute__((ext_vector_type(4)));
  const int lane = threadIdx.x & 63, ls = lane & 15, lq = lane >> 4;
  for (int i = threadIdx.x; i < 36000 / 4; i += 256) reinterpret_cast<int*>(smem)[i] = i;
  __syncthreads();
  const int row = (row_mode == 0 ? 8 : 4) * lq + (ls >> 2);
  const unsigned off = KIND == 2 ? lane * 16 : row_mode == 2 ? lane * 8 : row * pitch + (ls & 3) * 8;
  i32x4 acc = {0, 0, 0, 0};
  for (int it = 0; it < iters; ++it) {
    i32x2 v[8];
    i32x4 w[8];
    const unsigned a = off + (it & 1) * 16384;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (KIND == 0) asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v[u]) : "v"(a + u * 32));
      if (KIND == 1) asm volatile("ds_read_b64 %0, %1" : "=v"(v[u]) : "v"(a + (row_mode == 2 ? u * 512 : u * 32)));
      if (KIND == 2) asm volatile("ds_read_b128 %0, %1" : "=v"(w[u]) : "v"(a + u * 1024));
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (KIND == 2) acc += w[u];
      else { acc[0] += v[u][0]; acc[1] += v[u][1]; }
    }
  }
  out[blockIdx.x * 256 + threadIdx.x] = acc[0] + acc[1] + acc[2] + acc[3];
}

// MODE 0: matrix instructions only; 1: FMAs only; 2: one matrix instruction then R FMAs, eight times per iteration;
// 3: eight matrix instructions then 8 R FMAs; 4: wavefronts 0-3 of the workgroup matrix instructions only,
// wavefronts 4-7 FMAs only (512 threads: one of each per SIMD).  F32: v_mfma_f32_16x16x4_f32, else
// v_mfma_f32_16x16x32_bf16.  All operands in registers; 32 independent FMA chains.
template <int MODE, int R, bool F32>
__global__ void __launch_bounds__(512) coissue_kernel(float* __restrict__ out, int iters) {
  typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
  typedef float floatx4 __attribute__((ext_vector_type(4)));
  const int wave = threadIdx.x >> 6;
  floatx4 acc[8];
  float v[32];
  for (int i = 0; i < 8; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  for (int i = 0; i < 32; ++i) v[i] = threadIdx.x * 0.001f + i;
  bf16x8 a, b;
  for (int e = 0; e < 8; ++e) { a[e] = (__bf16)(float)(threadIdx.x & 7); b[e] = (__bf16)1.0f; }
  const float fa = (float)(threadIdx.x & 7), fb = 1.0f, m = 1.0001f, c = 0.5f;
  const bool do_m = MODE == 0 || MODE == 3 || (MODE == 4 && (wave & 4) == 0);
  const bool do_v = MODE == 1 || MODE == 3 || (MODE == 4 && (wave & 4) != 0);
  for (int it = 0; it < iters; ++it) {
    if (MODE == 2) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (F32) acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa, fb, acc[i], 0, 0, 0);
        else acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[i], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < R; ++j) v[(i * R + j) & 31] = __builtin_fmaf(v[(i * R + j) & 31], m, c);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
      if (do_m) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (F32) acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa, fb, acc[i], 0, 0, 0);
          else acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[i], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (do_v) {
#pragma unroll
        for (int j = 0; j < 8 * R; ++j) v[j & 31] = __builtin_fmaf(v[j & 31], m, c);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  float s = 0.f;
  for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  for (int i = 0; i < 32; ++i) s += v[i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

template <bool F32, int R>
static void (*coissue_fn(int mode))(float*, int) {
  switch (mode) {
    case 0: return coissue_kernel<0, R, F32>;
    case 1: return coissue_kernel<1, R, F32>;
    case 2: return coissue_kernel<2, R, F32>;
    case 3: return coissue_kernel<3, R, F32>;
    default: return coissue_kernel<4, R, F32>;
  }
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

// One launch of `workgroups` workgroups of four wavefronts, `lds_bytes` of LDS each (which sets how many share a
// compute unit), `iters` rounds of eight reads per wavefront; out: workgroups * 256 ints.  The caller times it.
int cgtpbench_lds_read(int kind, int row_mode, int pitch, int workgroups, int lds_bytes, int iters, void* out,
                       void* stream) {
  if (!out) return CGTP_ERR_NULL;
  if (kind < 0 || kind > 2 || row_mode < 0 || row_mode > 2 || workgroups <= 0 || iters <= 0) return CGTP_ERR_SHAPE;
  // the reads stay inside 36000 bytes: 28 rows of `pitch` bytes + 256 + the second buffer 16 KB further
  if (pitch < 256 || 28 * pitch + 256 + 16384 > 36000 || lds_bytes < 36000 || lds_bytes > 160 * 1024) return CGTP_ERR_SHAPE;
  void (*fn)(int*, int, int, int) = kind == 0 ? lds_read_kernel<0> : kind == 1 ? lds_read_kernel<1> : lds_read_kernel<2>;
  if (hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess)
    return CGTP_ERR_LDS;
  hipLaunchKernelGGL(fn, dim3((unsigned)workgroups), dim3(256), (size_t)lds_bytes, (hipStream_t)stream, (int*)out, iters,
                     pitch, row_mode);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

// One launch of one workgroup per compute unit (`workgroups`), 256 or 512 threads (one or two wavefronts per SIMD),
// `iters` iterations of 8 matrix instructions and / or 8 * fma_per_mfma FMAs per wavefront (fma_per_mfma 4 with the
// bf16 instruction, 8 with the fp32 one: the instruction's run time in issue slots); out: workgroups * threads floats.
int cgtpbench_coissue(int mode, int f32, int threads, int workgroups, int iters, void* out, void* stream) {
  if (!out) return CGTP_ERR_NULL;
  if (mode < 0 || mode > 4 || (threads != 256 && threads != 512) || workgroups <= 0 || iters <= 0) return CGTP_ERR_SHAPE;
  if (mode == 4 && threads != 512) return CGTP_ERR_SHAPE;
  void (*fn)(float*, int) = f32 ? coissue_fn<true, 8>(mode) : coissue_fn<false, 4>(mode);
  hipLaunchKernelGGL(fn, dim3((unsigned)workgroups), dim3((unsigned)threads), 0, (hipStream_t)stream, (float*)out, iters);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

}  // extern "C"
