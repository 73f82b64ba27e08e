// Real spherical harmonics of one vector in registers, degree known at compile time: the in-kernel form of the
// recurrence that sh_kernels.hip runs with a run-time degree (see gen_sh.py for the factorisation and the
// coefficients).  Used by the fused edge kernels when they are handed edge vectors instead of harmonics.
#pragma once

#include <hip/hip_runtime.h>

#include "generated/sh_coef.inc"

namespace cgtp {

template <typename T> struct ShCoef;
template <> struct ShCoef<float> {
  __device__ static float step(int m) { return kShStepF[m]; }
  __device__ static float a(int l, int m) { return kShAF[l][m]; }
  __device__ static float b(int l, int m) { return kShBF[l][m]; }
};
template <> struct ShCoef<double> {
  __device__ static double step(int m) { return kShStepD[m]; }
  __device__ static double a(int l, int m) { return kShAD[l][m]; }
  __device__ static double b(int l, int m) { return kShBD[l][m]; }
};

constexpr double kShEps = 1e-12;    // torch.nn.functional.normalize: v / max(|v|, eps)

// What the second operand of a fused edge launch holds.
enum { kYHarmonics = 0, kYUnitVector = 1, kYRawVector = 2 };

// (x, y, z) = u / max(|u|, eps) when `normalize`, else u; inv = 1 / max(|u|, eps), len = |u| (both 1 otherwise).
template <typename T>
struct ShPoint {
  T x, y, z, inv, len;
  __device__ __forceinline__ ShPoint(T ux, T uy, T uz, bool normalize) : x(ux), y(uy), z(uz), inv(1), len(1) {
    if (normalize) {
      len = sqrt(ux * ux + uy * uy + uz * uz);
      inv = T(1) / (len > T(kShEps) ? len : T(kShEps));
      x = ux * inv; y = uy * inv; z = uz * inv;
    }
  }
  // gradient with respect to u from the gradient with respect to (x, y, z)
  __device__ __forceinline__ void pull_back(T& gx, T& gy, T& gz, bool normalize) const {
    if (!normalize) return;
    if (len > T(kShEps)) {
      const T dot = gx * x + gy * y + gz * z;
      gx = (gx - x * dot) * inv; gy = (gy - y * dot) * inv; gz = (gz - z * dot) * inv;
    } else {
      gx *= inv; gy *= inv; gz *= inv;
    }
  }
};

// Y[l^2 + l + m], l = 0..LMAX, of the point (x, y, z); homogeneous of degree l.
template <typename T, int LMAX>
__device__ __forceinline__ void sh_values(T x, T y, T z, T (&Y)[(LMAX + 1) * (LMAX + 1)]) {
  const T r2 = x * x + y * y + z * z;
  T C = 1, S = 0;
#pragma unroll
  for (int m = 0; m <= LMAX; ++m) {
    if (m > 0) {
      const T fm = ShCoef<T>::step(m), Cp = C, Sp = S;
      C = fm * (x * Cp - y * Sp);
      S = fm * (x * Sp + y * Cp);
    }
    T R1 = 0, R = 1;
#pragma unroll
    for (int l = m; l <= LMAX; ++l) {
      if (l > m) {
        const T R2 = R1;
        R1 = R;
        R = ShCoef<T>::a(l, m) * (z * R1 - ShCoef<T>::b(l, m) * (r2 * R2));
      }
      Y[l * l + l + m] = R * C;
      if (m) Y[l * l + l - m] = R * S;
    }
  }
}

// (gx, gy, gz) = sum_i g[i] dY[i]/d(x, y, z) at the point (x, y, z).
template <typename T, int LMAX>
__device__ __forceinline__ void sh_pull_back(T x, T y, T z, const T (&g)[(LMAX + 1) * (LMAX + 1)], T& gx, T& gy,
                                             T& gz) {
  const T r2 = x * x + y * y + z * z;
  gx = gy = gz = 0;
  T C = 1, S = 0, Cp = 0, Sp = 0;
#pragma unroll
  for (int m = 0; m <= LMAX; ++m) {
    T fm = 0;
    if (m > 0) {
      fm = ShCoef<T>::step(m);
      Cp = C; Sp = S;
      C = fm * (x * Cp - y * Sp);
      S = fm * (x * Sp + y * Cp);
    }
    const T dm = T(m) * fm;      // d(C_m, S_m)/d(x, y) = m f_m (C_{m-1}, S_{m-1}), rotated
    T R1 = 0, R = 1, Rz1 = 0, Rz = 0, Rr1 = 0, Rr = 0;   // R, dR/dz at fixed r^2, dR/d(r^2)
#pragma unroll
    for (int l = m; l <= LMAX; ++l) {
      if (l > m) {
        const T a = ShCoef<T>::a(l, m), b = ShCoef<T>::b(l, m);
        const T R2 = R1, Rz2 = Rz1, Rr2 = Rr1;
        R1 = R; Rz1 = Rz; Rr1 = Rr;
        R = a * (z * R1 - b * (r2 * R2));
        Rz = a * (R1 + z * Rz1 - b * (r2 * Rz2));
        Rr = a * (z * Rr1 - b * (R2 + r2 * Rr2));
      }
      const T gp = g[l * l + l + m], gm = m ? g[l * l + l - m] : T(0);
      const T q = gp * C + gm * S;
      gz += (Rz + T(2) * z * Rr) * q;
      gx += T(2) * Rr * x * q + R * dm * (gp * Cp + gm * Sp);
      gy += T(2) * Rr * y * q + R * dm * (gm * Cp - gp * Sp);
    }
  }
}

}  // namespace cgtp
