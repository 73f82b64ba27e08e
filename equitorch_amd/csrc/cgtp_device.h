// Device-side helpers shared by the cgtp kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cgtp {

constexpr int kWave = 64;

// ---- V-wide per-lane channel vectors held in registers ------------------------------------------------
template <typename T, int V>
__device__ __forceinline__ void mulv(T (&t)[V], T s, const T (&x)[V]) {
#pragma unroll
  for (int v = 0; v < V; ++v) t[v] = s * x[v];
}
template <typename T, int V>
__device__ __forceinline__ void fmav(T (&t)[V], T s, const T (&x)[V]) {
#pragma unroll
  for (int v = 0; v < V; ++v) t[v] = fma(s, x[v], t[v]);
}
template <typename T, int V>
__device__ __forceinline__ void mulvv(T (&t)[V], const T (&a)[V], const T (&b)[V]) {
#pragma unroll
  for (int v = 0; v < V; ++v) t[v] = a[v] * b[v];
}
template <typename T, int V>
__device__ __forceinline__ void fmavv(T (&o)[V], const T (&a)[V], const T (&b)[V]) {
#pragma unroll
  for (int v = 0; v < V; ++v) o[v] = fma(a[v], b[v], o[v]);
}
template <typename T, int V>
__device__ __forceinline__ T dotv(const T (&a)[V], const T (&b)[V]) {
  T r = a[0] * b[0];
#pragma unroll
  for (int v = 1; v < V; ++v) r = fma(a[v], b[v], r);
  return r;
}

// ---- vector global memory access: V consecutive elements of T as one transaction ------------------------
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));

template <typename T, int V>
struct VecOf;
template <> struct VecOf<float, 1> { using type = float; };
template <> struct VecOf<float, 2> { using type = f32x2; };
template <> struct VecOf<float, 4> { using type = f32x4; };
template <> struct VecOf<double, 1> { using type = double; };
template <> struct VecOf<double, 2> { using type = f64x2; };

template <typename T, int V>
__device__ __forceinline__ void load_vec(T (&dst)[V], const T* __restrict__ p) {
  using VT = typename VecOf<T, V>::type;
  VT v = *reinterpret_cast<const VT*>(p);
  const T* e = reinterpret_cast<const T*>(&v);
#pragma unroll
  for (int i = 0; i < V; ++i) dst[i] = e[i];
}
// Streaming load: data read once (per-edge weights) should not displace the gathered node rows in cache.
template <typename T, int V>
__device__ __forceinline__ void load_vec_stream(T (&dst)[V], const T* __restrict__ p) {
  using VT = typename VecOf<T, V>::type;
  VT v = __builtin_nontemporal_load(reinterpret_cast<const VT*>(p));
  const T* e = reinterpret_cast<const T*>(&v);
#pragma unroll
  for (int i = 0; i < V; ++i) dst[i] = e[i];
}
template <typename T, int V>
__device__ __forceinline__ void store_vec(T* __restrict__ p, const T (&src)[V]) {
  using VT = typename VecOf<T, V>::type;
  VT v;
  T* e = reinterpret_cast<T*>(&v);
#pragma unroll
  for (int i = 0; i < V; ++i) e[i] = src[i];
  *reinterpret_cast<VT*>(p) = v;
}
template <typename T, int V>
__device__ __forceinline__ void store_vec_stream(T* __restrict__ p, const T (&src)[V]) {
  using VT = typename VecOf<T, V>::type;
  VT v;
  T* e = reinterpret_cast<T*>(&v);
#pragma unroll
  for (int i = 0; i < V; ++i) e[i] = src[i];
  __builtin_nontemporal_store(v, reinterpret_cast<VT*>(p));
}

// ---- cross-lane -------------------------------------------------------------------------------------------
__device__ __forceinline__ float shfl_xor(float v, int mask) { return __shfl_xor(v, mask, kWave); }
__device__ __forceinline__ double shfl_xor(double v, int mask) { return __shfl_xor(v, mask, kWave); }

// Sum over groups of `width` consecutive lanes (width a power of two <= 64); every lane gets the group sum.
template <typename T>
__device__ __forceinline__ T group_sum(T v, int width) {
  for (int off = 1; off < width; off <<= 1) v += shfl_xor(v, off);
  return v;
}
// Sum across the 64/width groups (lanes with equal lane % width); every lane gets the sum.
template <typename T>
__device__ __forceinline__ T cross_group_sum(T v, int width) {
  for (int off = width; off < kWave; off <<= 1) v += shfl_xor(v, off);
  return v;
}

// The same sum for a block of registers, a stage at a time: all rows are exchanged before any is added, so a stage
// waits once for the cross-lane network instead of once per value (one value at a time, every exchange and its wait
// come one after the other: 72 round trips for 9 rows of 4 channels over 4 groups).  Same operands per addition as
// cross_group_sum, hence the same bits.
__device__ __forceinline__ float lane_exchange(float v, int byte_addr) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(byte_addr, __builtin_bit_cast(int, v)));
}
__device__ __forceinline__ double lane_exchange(double v, int byte_addr) {
  const long long b = __builtin_bit_cast(long long, v);
  const unsigned lo = (unsigned)__builtin_amdgcn_ds_bpermute(byte_addr, (int)(unsigned)b);
  const unsigned hi = (unsigned)__builtin_amdgcn_ds_bpermute(byte_addr, (int)(unsigned)(b >> 32));
  return __builtin_bit_cast(double, (long long)(((unsigned long long)hi << 32) | lo));
}
template <typename T, int D, int V>
__device__ __forceinline__ void cross_group_sum_rows(T (&acc)[D][V], int width) {
  const int lane = threadIdx.x & (kWave - 1);
  for (int off = width; off < kWave; off <<= 1) {
    const int addr = (lane ^ off) << 2;
    T t[D][V];
#pragma unroll
    for (int m = 0; m < D; ++m)
#pragma unroll
      for (int v = 0; v < V; ++v) t[m][v] = lane_exchange(acc[m][v], addr);
#pragma unroll
    for (int m = 0; m < D; ++m)
#pragma unroll
      for (int v = 0; v < V; ++v) acc[m][v] += t[m][v];
  }
}

// Sums of N values over groups of `width` consecutive lanes, left spread over the group's lanes: `done(s)` receives
// an array s with s[i] = the group's sum of val[i * width + cl] in the lane whose place in the group is cl (fewer
// entries the wider the group; entries past N are zero).  Stage b halves the values a lane still carries: the lane
// keeps those whose index has bit b equal to its own, hands the others to its partner cl ^ (1 << b) and adds what
// the partner hands over, so N values over 16 lanes take N/2 + N/4 + N/8 + N/16 exchanges in four dependent stages
// (11 for N = 9) where a butterfly sum of every value takes 4 N, and one lane-contiguous store can follow instead
// of N single-lane ones.  The first two stages stay inside quads (DPP), the others go through ds_bpermute, issued
// together per stage.  All lanes of a group must be active; the order of the additions is fixed.  In a kernel close to
// a register boundary the few extra live values can cost a wavefront per SIMD: check the resource usage of every
// instantiation that adopts it.
template <int B>
__device__ __forceinline__ float lane_xor_exchange(float v, int lane) {
  if constexpr (B == 0)
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
  else if constexpr (B == 1)
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
  else
    return lane_exchange(v, (lane ^ (1 << B)) << 2);
}
template <int B>
__device__ __forceinline__ double lane_xor_exchange(double v, int lane) {
  return lane_exchange(v, (lane ^ (1 << B)) << 2);
}
template <typename T, int N, int B = 0, typename Done>
__device__ __forceinline__ void group_sum_scatter(const T (&val)[N], int width, Done&& done) {
  if constexpr (B < 6) {
    if ((1 << B) < width) {   // the same for every lane
      constexpr int M = (N + 1) / 2;
      const int lane = threadIdx.x & (kWave - 1);
      const bool upper = (lane >> B) & 1;
      T keep[M], recv[M];
#pragma unroll
      for (int i = 0; i < M; ++i) {
        const T lo = val[2 * i];
        const T hi = 2 * i + 1 < N ? val[2 * i + 1] : T(0);
        keep[i] = upper ? hi : lo;
        recv[i] = lane_xor_exchange<B>(upper ? lo : hi, lane);
      }
#pragma unroll
      for (int i = 0; i < M; ++i) keep[i] += recv[i];
      group_sum_scatter<T, M, B + 1>(keep, width, done);
      return;
    }
  }
  done(val);
}
template <typename T, int N>
__device__ __forceinline__ constexpr int array_len(const T (&)[N]) { return N; }

}  // namespace cgtp
