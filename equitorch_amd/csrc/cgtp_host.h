// Host-side declarations shared by the translation units of libcgtp.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "cgtp.h"

namespace cgtp {

// The 160 KB of LDS of a gfx950 compute unit; a workgroup may claim all of it.
constexpr int64_t kLdsBytes = 160 * 1024;

inline int elem_size(int dtype) {
  switch (dtype) {
    case CGTP_F32: return 4;
    case CGTP_F64: return 8;
    case CGTP_BF16: return 2;
    case CGTP_F16: return 2;
    default: return 0;
  }
}

// out[i] = sum_k ws[k * n + i], accumulated in double in a fixed order (deterministic): 16 threads per column take
// every 16th partial each, their sums are added in thread order.
constexpr int kPartialSlices = 16, kPartialCols = 16;
template <typename T>
__global__ void __launch_bounds__(kPartialSlices * kPartialCols)
partial_sum_kernel(const T* __restrict__ ws, T* __restrict__ out, int64_t n_part, int64_t n) {
  __shared__ double part[kPartialSlices][kPartialCols];
  const int col = threadIdx.x % kPartialCols, slice = threadIdx.x / kPartialCols;
  const int64_t i = (int64_t)blockIdx.x * kPartialCols + col;
  double s = 0.0;
  if (i < n)
    for (int64_t k = slice; k < n_part; k += kPartialSlices) s += (double)ws[k * n + i];
  part[slice][col] = s;
  __syncthreads();
  if (slice == 0 && i < n) {
    double total = 0.0;
    for (int j = 0; j < kPartialSlices; ++j) total += part[j][col];
    out[i] = (T)total;
  }
}

template <typename T>
inline void launch_partial_sum(const T* ws, T* out, int64_t n_part, int64_t n, hipStream_t stream) {
  hipLaunchKernelGGL(partial_sum_kernel<T>, dim3((unsigned)((n + kPartialCols - 1) / kPartialCols)),
                     dim3(kPartialSlices * kPartialCols), 0, stream, ws, out, n_part, n);
}

// First pass of a sum over many rows: part[c * n + i] = sum of rows[r * n + i] over the rows r of chunk c
// (kSumRows rows); partial_sum_kernel then adds the chunks.  Fixed order, no atomics: four threads per column take
// every fourth row of the chunk each, four loads in flight, and their sums are added in thread order.
constexpr int kSumRows = 64;
constexpr int kSumSlices = 4, kSumCols = 64;
template <typename T>
__global__ void __launch_bounds__(kSumSlices * kSumCols) rows_sum_kernel(const T* __restrict__ rows, T* __restrict__ part,
                                                                         int64_t n_rows, int64_t n) {
  __shared__ T acc[kSumSlices][kSumCols];
  const int col = threadIdx.x % kSumCols, slice = threadIdx.x / kSumCols;
  const int64_t i = (int64_t)blockIdx.x * kSumCols + col;
  const int64_t r0 = (int64_t)blockIdx.y * kSumRows, r1 = r0 + kSumRows < n_rows ? r0 + kSumRows : n_rows;
  T s = T(0);
  if (i < n) {
    int64_t r = r0 + slice;
    for (; r + 3 * kSumSlices < r1; r += 4 * kSumSlices) {
      const T a = rows[r * n + i], b = rows[(r + kSumSlices) * n + i], c = rows[(r + 2 * kSumSlices) * n + i],
              d = rows[(r + 3 * kSumSlices) * n + i];
      s += a; s += b; s += c; s += d;
    }
    for (; r < r1; r += kSumSlices) s += rows[r * n + i];
  }
  acc[slice][col] = s;
  __syncthreads();
  if (slice == 0 && i < n) {
    T total = acc[0][col];
#pragma unroll
    for (int j = 1; j < kSumSlices; ++j) total += acc[j][col];
    part[blockIdx.y * n + i] = total;
  }
}

template <typename T>
inline void launch_rows_sum(const T* rows, T* part, int64_t n_rows, int64_t n, hipStream_t stream) {
  const int64_t chunks = (n_rows + kSumRows - 1) / kSumRows;
  hipLaunchKernelGGL(rows_sum_kernel<T>, dim3((unsigned)((n + kSumCols - 1) / kSumCols), (unsigned)chunks),
                     dim3(kSumSlices * kSumCols), 0, stream, rows, part, n_rows, n);
}

}  // namespace cgtp
