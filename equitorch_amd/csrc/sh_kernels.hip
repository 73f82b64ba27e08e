// Real spherical harmonics of edge vectors and their gradient (cgtp_sh_forward / cgtp_sh_backward).
//
// Replaces the explicit polynomials of equitorch/ops/spherical_harmonics.py:68-640 (a TorchScript function that
// materialises every intermediate as a tensor) by one kernel per direction.  One lane owns one vector and walks
//
//     Y_{l,+m} = R_l^m(z, r^2) C_m(x, y),   Y_{l,-m} = R_l^m S_m,      index l^2 + l +- m,
//
// order m outermost (C_m, S_m by one complex multiplication), degree l innermost (three-term recurrence in z and
// r^2 = x^2 + y^2 + z^2, see gen_sh.py).  The polynomials are homogeneous of degree l, as in the reference, so the
// result for an un-normalised vector is r^l times the harmonic of its direction.  The backward kernel carries the
// partial derivatives of R, C, S through the same recurrences and contracts them with grad_out on the fly.
//
// HBM-bound: 3 values in, (lmax+1)^2 out per vector.  Rows of 64 vectors are exchanged through a wavefront-private
// LDS tile so that global loads and stores are contiguous; when a tile would not fit (high degree), lanes address
// global memory directly.
#include <utility>

#include "cgtp_host.h"

#include "sh_device.h"

namespace cgtp {
namespace {

constexpr int kShBlock = 256;       // most vectors per workgroup, one per lane
constexpr int kShUnrolled = 8;      // degrees up to this one have kernels with the degree compiled in

// Row `lane` of a (64 x D) tile: in LDS at pitch `pitch`, or straight in global memory at pitch D.
template <typename T>
struct ShRow {
  T* p;
  __device__ T& operator[](int i) const { return p[i]; }
};

// Copies the wavefront's `cnt` rows of D values between the LDS tile and the contiguous global range, eight
// independent 256-byte row segments in flight per step (a global load per iteration would serialise on latency).
// Element j of the range is element j + (j / D) * (pitch - D) of the tile.  DC > 0: D is the compile-time constant
// DC; a full tile (64 rows) is then copied by straight-line code with constant offsets.
template <typename T, bool TO_GLOBAL, int DC>
__device__ __forceinline__ void sh_tile_copy(T* tile, int pitch, T* glob, int cnt, int D_arg, int lane) {
  constexpr int kBatch = 8;
  const int D = DC > 0 ? DC : D_arg;
  if (DC > 0 && cnt == 64) {
    const int pad = pitch - D;     // 0 or 1
#pragma unroll
    for (int t0 = 0; t0 < (DC > 0 ? DC : 1); t0 += kBatch) {
      T v[kBatch];
      int at[kBatch];
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        const int j = lane + 64 * (t0 + k);
        at[k] = j + (pad ? j / D : 0);
      }
      if (TO_GLOBAL) {
#pragma unroll
        for (int k = 0; k < kBatch; ++k)
          if (t0 + k < D) v[k] = tile[at[k]];
#pragma unroll
        for (int k = 0; k < kBatch; ++k)
          if (t0 + k < D) glob[lane + 64 * (t0 + k)] = v[k];
      } else {
#pragma unroll
        for (int k = 0; k < kBatch; ++k)
          if (t0 + k < D) v[k] = glob[lane + 64 * (t0 + k)];
#pragma unroll
        for (int k = 0; k < kBatch; ++k)
          if (t0 + k < D) tile[at[k]] = v[k];
      }
    }
    return;
  }
  const int total = cnt * D;
  const int dq = 64 / D, dr = 64 - dq * D;     // a step of 64 elements = dq rows and dr columns
  int r = lane / D, i = lane - r * D;
  for (int j0 = lane; j0 < total; j0 += 64 * kBatch) {
    T v[kBatch];
    int at[kBatch];
#pragma unroll
    for (int k = 0; k < kBatch; ++k) {
      at[k] = r * pitch + i;
      r += dq; i += dr;
      if (i >= D) { i -= D; ++r; }
    }
    if (TO_GLOBAL) {
#pragma unroll
      for (int k = 0; k < kBatch; ++k) v[k] = j0 + 64 * k < total ? tile[at[k]] : T(0);
#pragma unroll
      for (int k = 0; k < kBatch; ++k)
        if (j0 + 64 * k < total) glob[j0 + 64 * k] = v[k];
    } else {
#pragma unroll
      for (int k = 0; k < kBatch; ++k) v[k] = j0 + 64 * k < total ? glob[j0 + 64 * k] : T(0);
#pragma unroll
      for (int k = 0; k < kBatch; ++k)
        if (j0 + 64 * k < total) tile[at[k]] = v[k];
    }
  }
}

// LT >= 0: the degree is LT, known at compile time (both loops unroll, the coefficients become literals and the
// tile accesses independent); LT < 0: the degree is the run-time argument.
template <typename T, bool BWD, int LT>
__global__ void __launch_bounds__(kShBlock) sh_kernel(const T* __restrict__ xyz, const T* __restrict__ gout,
                                                      T* __restrict__ out, int64_t n, int lmax_arg, int normalize,
                                                      T scale, int pitch) {
  extern __shared__ __align__(16) unsigned char sh_smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lmax = LT >= 0 ? LT : lmax_arg;
  const int D = (lmax + 1) * (lmax + 1);
  constexpr int DC = LT >= 0 ? (LT + 1) * (LT + 1) : -1;
  const int64_t e0 = (int64_t)blockIdx.x * blockDim.x + wave * 64;   // first vector of this wavefront
  const int64_t e = e0 + lane;
  const bool live = e < n;
  const int cnt = e0 >= n ? 0 : (n - e0 < 64 ? (int)(n - e0) : 64);
  T* tile = pitch ? reinterpret_cast<T*>(sh_smem) + (size_t)wave * 64 * pitch : nullptr;

  T ux = 0, uy = 0, uz = 1;
  if (live) { ux = xyz[e * 3]; uy = xyz[e * 3 + 1]; uz = xyz[e * 3 + 2]; }
  T x = ux, y = uy, z = uz, inv = 1, len = 1;
  if (normalize) {
    len = sqrt(ux * ux + uy * uy + uz * uz);
    inv = T(1) / (len > T(kShEps) ? len : T(kShEps));
    x = ux * inv; y = uy * inv; z = uz * inv;
  }
  const T r2 = x * x + y * y + z * z;

  // the row this lane reads (backward: grad_out) or writes (forward: Y)
  T* base = BWD ? const_cast<T*>(gout) : out;
  if (BWD && tile) {
    sh_tile_copy<T, false, DC>(tile, pitch, base + e0 * D, cnt, D, lane);
    __syncthreads();
  }
  ShRow<T> row{tile ? tile + (size_t)lane * pitch : base + (live ? e : 0) * D};

  T gx = 0, gy = 0, gz = 0;
  T C = 1, S = 0;            // C_m, S_m
  T Cp = 0, Sp = 0;          // C_{m-1}, S_{m-1}
#pragma unroll
  for (int m = 0; m <= lmax; ++m) {
    T fm = 0;
    if (m > 0) {
      fm = ShCoef<T>::step(m);
      Cp = C; Sp = S;
      C = fm * (x * Cp - y * Sp);
      S = fm * (x * Sp + y * Cp);
    }
    // d(C_m, S_m)/d(x, y) = m f_m (C_{m-1}, S_{m-1}) rotated
    const T dm = T(m) * fm;
    T R1 = 0, R = 1;         // R_{l-1}, R_l (l = m)
    T Rz1 = 0, Rz = 0;       // dR/dz at fixed r^2
    T Rr1 = 0, Rr = 0;       // dR/d(r^2)
#pragma unroll
    for (int l = m; l <= lmax; ++l) {
      if (l > m) {
        const T a = ShCoef<T>::a(l, m), b = ShCoef<T>::b(l, m);
        const T R2 = R1, Rz2 = Rz1, Rr2 = Rr1;
        R1 = R; Rz1 = Rz; Rr1 = Rr;
        R = a * (z * R1 - b * (r2 * R2));
        if (BWD) {
          Rz = a * (R1 + z * Rz1 - b * (r2 * Rz2));
          Rr = a * (z * Rr1 - b * (R2 + r2 * Rr2));
        }
      }
      const int ip = l * l + l + m, im = l * l + l - m;
      if (!BWD) {
        if (live || tile) {
          row[ip] = scale * (R * C);
          if (m) row[im] = scale * (R * S);
        }
      } else {
        const T gp = (live || tile) ? row[ip] : T(0);
        const T gm = m && (live || tile) ? row[im] : T(0);
        const T q = gp * C + gm * S;                       // d/dR
        const T dz = Rz + T(2) * z * Rr, dr = T(2) * Rr;
        gz += dz * q;
        gx += dr * x * q + R * dm * (gp * Cp + gm * Sp);
        gy += dr * y * q + R * dm * (gm * Cp - gp * Sp);
      }
    }
  }

  if (!BWD) {
    if (tile) {
      __syncthreads();
      sh_tile_copy<T, true, DC>(tile, pitch, out + e0 * D, cnt, D, lane);
    }
  } else if (live) {
    gx *= scale; gy *= scale; gz *= scale;
    if (normalize) {
      if (len > T(kShEps)) {
        const T dot = gx * x + gy * y + gz * z;
        gx = (gx - x * dot) * inv; gy = (gy - y * dot) * inv; gz = (gz - z * dot) * inv;
      } else {
        gx *= inv; gy *= inv; gz *= inv;
      }
    }
    out[e * 3] = gx; out[e * 3 + 1] = gy; out[e * 3 + 2] = gz;
  }
}

// LDS pitch (elements) of the per-wavefront tile, odd so that lanes hit distinct banks, and the number of
// wavefronts per workgroup (4 or 2 within half of the LDS, else 1 within all of it); pitch 0 = no tile fits,
// lanes address global memory.
struct ShShape { int pitch, waves; };
ShShape sh_shape(int lmax, int dtype) {
  const int D = (lmax + 1) * (lmax + 1);
  const int pitch = D | 1;
  const int64_t per_wave = (int64_t)64 * pitch * elem_size(dtype);
  for (int waves = kShBlock / 64; waves >= 1; waves /= 2)
    if (per_wave * waves <= (waves > 1 ? kLdsBytes / 2 : kLdsBytes)) return {pitch, waves};
  return {0, kShBlock / 64};
}

int sh_check(const void* xyz, const void* a, const void* b, int64_t n, int lmax, int dtype) {
  if (dtype != CGTP_F32 && dtype != CGTP_F64) return CGTP_ERR_DTYPE;
  if (n < 0 || lmax < 0 || lmax > kShMaxDegree) return CGTP_ERR_SHAPE;
  if (n > 0 && (!xyz || !a || !b)) return CGTP_ERR_NULL;
  if (n >= ((int64_t)1 << 31) * 64) return CGTP_ERR_SHAPE;
  return CGTP_OK;
}

template <typename T, bool BWD>
using ShKernel = void (*)(const T*, const T*, T*, int64_t, int, int, T, int);

template <typename T, bool BWD, int... LS>
ShKernel<T, BWD> sh_pick(int lmax, std::integer_sequence<int, LS...>) {
  static const ShKernel<T, BWD> table[] = {sh_kernel<T, BWD, LS>...};
  return lmax <= kShUnrolled ? table[lmax] : sh_kernel<T, BWD, -1>;
}

template <typename T, bool BWD>
int sh_launch(const void* xyz, const void* gout, void* out, int64_t n, int lmax, int normalize, double scale,
              int dtype, hipStream_t stream) {
  if (n == 0) return CGTP_OK;
  const ShShape sh = sh_shape(lmax, dtype);
  const int block = sh.waves * 64;
  const size_t lds = (size_t)block * sh.pitch * sizeof(T);
  const unsigned grid = (unsigned)((n + block - 1) / block);
  const ShKernel<T, BWD> fn = sh_pick<T, BWD>(lmax, std::make_integer_sequence<int, kShUnrolled + 1>{});
  hipLaunchKernelGGL(fn, dim3(grid), dim3(block), lds, stream, (const T*)xyz, (const T*)gout, (T*)out, n, lmax,
                     normalize, (T)scale, sh.pitch);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

}  // namespace
}  // namespace cgtp

extern "C" {

int cgtp_sh_max_degree(void) { return kShMaxDegree; }

int cgtp_sh_forward(const void* xyz, void* out, int64_t n, int lmax, int normalize, double scale, int dtype,
                    void* stream) {
  using namespace cgtp;
  if (int rc = sh_check(xyz, out, out, n, lmax, dtype)) return rc;
  hipStream_t s = (hipStream_t)stream;
  return dtype == CGTP_F32 ? sh_launch<float, false>(xyz, nullptr, out, n, lmax, normalize, scale, dtype, s)
                           : sh_launch<double, false>(xyz, nullptr, out, n, lmax, normalize, scale, dtype, s);
}

int cgtp_sh_backward(const void* xyz, const void* grad_out, void* grad_xyz, int64_t n, int lmax, int normalize,
                     double scale, int dtype, void* stream) {
  using namespace cgtp;
  if (int rc = sh_check(xyz, grad_out, grad_xyz, n, lmax, dtype)) return rc;
  hipStream_t s = (hipStream_t)stream;
  return dtype == CGTP_F32 ? sh_launch<float, true>(xyz, grad_out, grad_xyz, n, lmax, normalize, scale, dtype, s)
                           : sh_launch<double, true>(xyz, grad_out, grad_xyz, n, lmax, normalize, scale, dtype, s);
}

}  // extern "C"
