// Radial basis and cutoff envelopes of the edge length, element-wise, one launch forward and one for the gradient.
//
//   bessel:     out[i, k] = (2 / r_max) * sin(freq[k] * r[i] / r_max) / r[i]
//   cutoffs:    u = clamp((r - r_min) / range, 0, 1)
//     polynomial  1 - (p+1)(p+2)/2 u^p + p(p+2) u^(p+1) - p(p+1)/2 u^(p+2)
//     cosine      (1 + cos(pi u)) / 2
//     mollifier   exp(1 - 1 / (1 - u^2 + eps))
//
// As tensor expressions these are six to ten launches each and as many again in the backward, every one over a tensor
// of a few MB: the launches, not the bytes, are what they cost.  The arithmetic follows the expressions operation by
// operation (same order, divisions where they divide), so that results agree with them to the last bits of the
// library functions involved.
#include "cgtp_device.h"
#include "cgtp_host.h"

namespace cgtp {

template <typename T>
__global__ void __launch_bounds__(256) bessel_fwd_kernel(const T* __restrict__ r, const T* __restrict__ freq,
                                                         T* __restrict__ out, int64_t n, int K, T prefactor, T r_max) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * K) return;
  const T x = r[i / K];
  out[i] = prefactor * (sin(freq[i % K] * x / r_max) / x);
}

// gr[i] = sum_k g[i, k] * d out[i, k] / d r[i];  gf_rows[i, k] = g[i, k] * d out[i, k] / d freq[k] (summed over i by
// the caller) when asked for.  One thread per row: the sum over k runs in index order.
template <typename T>
__global__ void __launch_bounds__(256) bessel_bwd_kernel(const T* __restrict__ r, const T* __restrict__ freq,
                                                         const T* __restrict__ g, T* __restrict__ gr,
                                                         T* __restrict__ gf_rows, int64_t n, int K, T prefactor, T r_max) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const T x = r[i];
  T acc = T(0);
  for (int k = 0; k < K; ++k) {
    const T f = freq[k], theta = f * x / r_max;
    const T s = sin(theta), c = cos(theta);
    const T gk = g[i * K + k] * prefactor;
    // d/dx [sin(f x / R) / x] = cos(theta) f / (R x) - sin(theta) / x^2
    acc += gk * (c * f / r_max / x - s / (x * x));
    if (gf_rows) gf_rows[i * K + k] = gk * (c / r_max);      // d/df [sin(f x / R) / x] = cos(theta) / R
  }
  if (gr) gr[i] = acc;
}

enum { kCutPolynomial = 0, kCutCosine = 1, kCutMollifier = 2 };

template <typename T>
__device__ __forceinline__ T cut_unit(T x, T r_min, T range, bool* inside) {
  if (r_min != T(0)) x = x - r_min;
  const T v = x / range;
  *inside = v >= T(0) && v <= T(1);      // where clamp passes the gradient on (both ends included)
  return v < T(0) ? T(0) : v > T(1) ? T(1) : v;
}

template <typename T, int KIND>
__global__ void __launch_bounds__(256) cutoff_kernel(const T* __restrict__ r, const T* __restrict__ g, T* __restrict__ out,
                                                     int64_t n, T r_min, T range, T param) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  bool inside;
  const T u = cut_unit(r[i], r_min, range, &inside);
  constexpr T pi = T(3.14159265358979323846);
  T val, der;      // envelope and its derivative with respect to u
  if (KIND == kCutPolynomial) {
    const T p = param, a = (p + T(1)) * (p + T(2)) / T(2), b = p * (p + T(2)), c = p * (p + T(1)) / T(2);
    val = T(1) - a * pow(u, p) + b * pow(u, p + T(1)) - c * pow(u, p + T(2));
    der = -a * (p * pow(u, p - T(1))) + b * ((p + T(1)) * pow(u, p)) - c * ((p + T(2)) * pow(u, p + T(1)));
  } else if (KIND == kCutCosine) {
    val = T(0.5) * (T(1) + cos(pi * u));
    der = T(0.5) * (-sin(pi * u) * pi);
  } else {
    const T q = T(1) - u * u + param, e = exp(T(1) - T(1) / q);
    val = e;
    der = e * (-(T(2) * u) / (q * q));     // d/du [-1/q] = q'/q^2 with q' = -2u
  }
  out[i] = g ? (inside ? g[i] * der / range : T(0)) : val;
}

template <typename T>
static int bessel_launch(const void* r, const void* freq, const void* g, void* out, void* gr, void* gf_rows, int64_t n,
                         int K, double r_max, hipStream_t stream) {
  const T pre = (T)(2.0 / r_max), rm = (T)r_max;
  if (!g) {
    const int64_t total = n * K;
    hipLaunchKernelGGL(bessel_fwd_kernel<T>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, (const T*)r,
                       (const T*)freq, (T*)out, n, K, pre, rm);
  } else {
    hipLaunchKernelGGL(bessel_bwd_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, (const T*)r,
                       (const T*)freq, (const T*)g, (T*)gr, (T*)gf_rows, n, K, pre, rm);
  }
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

template <typename T>
static int cutoff_launch(int kind, const void* r, const void* g, void* out, int64_t n, double r_min, double range,
                         double param, hipStream_t stream) {
  const dim3 grid((unsigned)((n + 255) / 256)), block(256);
  const T a = (T)r_min, b = (T)range, c = (T)param;
  if (kind == kCutPolynomial)
    hipLaunchKernelGGL((cutoff_kernel<T, kCutPolynomial>), grid, block, 0, stream, (const T*)r, (const T*)g, (T*)out, n, a, b, c);
  else if (kind == kCutCosine)
    hipLaunchKernelGGL((cutoff_kernel<T, kCutCosine>), grid, block, 0, stream, (const T*)r, (const T*)g, (T*)out, n, a, b, c);
  else
    hipLaunchKernelGGL((cutoff_kernel<T, kCutMollifier>), grid, block, 0, stream, (const T*)r, (const T*)g, (T*)out, n, a, b, c);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

static int radial_check(const void* r, const void* out, int64_t n, int dtype) {
  if (dtype != CGTP_F32 && dtype != CGTP_F64) return CGTP_ERR_DTYPE;
  if (n < 0 || n >= (int64_t)1 << 38) return CGTP_ERR_SHAPE;
  if (n > 0 && (!r || !out)) return CGTP_ERR_NULL;
  return CGTP_OK;
}

}  // namespace cgtp

using namespace cgtp;

extern "C" {

int cgtp_bessel(const void* r, const void* freq, void* out, int64_t n, int32_t num_basis, double r_max, int32_t dtype,
                void* stream) {
  const int st = radial_check(r, out, n, dtype);
  if (st != CGTP_OK) return st;
  if (num_basis <= 0 || num_basis > 4096 || !(r_max > 0)) return CGTP_ERR_SHAPE;
  if (n == 0) return CGTP_OK;
  if (!freq) return CGTP_ERR_NULL;
  return dtype == CGTP_F32 ? bessel_launch<float>(r, freq, nullptr, out, nullptr, nullptr, n, num_basis, r_max, (hipStream_t)stream)
                           : bessel_launch<double>(r, freq, nullptr, out, nullptr, nullptr, n, num_basis, r_max, (hipStream_t)stream);
}

int cgtp_bessel_grad(const void* r, const void* freq, const void* g, void* gr, void* gfreq_rows, int64_t n,
                     int32_t num_basis, double r_max, int32_t dtype, void* stream) {
  const int st = radial_check(r, g, n, dtype);
  if (st != CGTP_OK) return st;
  if (num_basis <= 0 || num_basis > 4096 || !(r_max > 0)) return CGTP_ERR_SHAPE;
  if (n == 0 || (!gr && !gfreq_rows)) return CGTP_OK;
  if (!freq) return CGTP_ERR_NULL;
  return dtype == CGTP_F32 ? bessel_launch<float>(r, freq, g, nullptr, gr, gfreq_rows, n, num_basis, r_max, (hipStream_t)stream)
                           : bessel_launch<double>(r, freq, g, nullptr, gr, gfreq_rows, n, num_basis, r_max, (hipStream_t)stream);
}

int cgtp_cutoff(int kind, const void* r, const void* g, void* out, int64_t n, double r_min, double range, double param,
                int32_t dtype, void* stream) {
  const int st = radial_check(r, out, n, dtype);
  if (st != CGTP_OK) return st;
  if (kind < 0 || kind > 2 || !(range > 0)) return CGTP_ERR_SHAPE;
  if (n == 0) return CGTP_OK;
  return dtype == CGTP_F32 ? cutoff_launch<float>(kind, r, g, out, n, r_min, range, param, (hipStream_t)stream)
                           : cutoff_launch<double>(kind, r, g, out, n, r_min, range, param, (hipStream_t)stream);
}

}  // extern "C"
