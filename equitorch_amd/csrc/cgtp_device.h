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

}  // namespace cgtp
