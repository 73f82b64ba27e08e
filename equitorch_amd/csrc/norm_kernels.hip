// Layer RMS normalisation of equivariant features in one pass per direction (cgtp_layer_rms_forward /
// cgtp_layer_rms_backward):
//
//   ms[n, k]     = sum_{M in irrep k} sum_c x[n, M, c]^2 / C * (scaled ? 1 / dim_k : 1)
//   r[n, k]      = rsqrt(ms[n, k] + eps)
//   out[n, M, c] = x[n, M, c] * r[n, k(M)] * weight[k(M), c]
//
// The reference composes this from four operator launches (channel-mean squared norm, rsqrt, a per-irrep scaling
// and a gate with the weight, equitorch/nn/functional/normalization.py:111-157), each a pass over the feature
// tensor.  Here a row takes LPR = next_pow2(C / V) lanes with V channels each (16-byte accesses), a wavefront covers
// 64 / LPR rows, and the kernel walks the row irrep by irrep: the rows of one irrep are loaded into registers
// (at most kNormMaxDim = 13 of them, l <= 6), reduced across the row's lanes, scaled and written.  The backward
// recomputes nothing but the products it needs:
//
//   gy = grad_out * weight,   dot = sum_{M, c} gy * x / C * (scaled ? 1 / dim_k : 1),
//   grad_x = r * (gy - x * r^2 * dot),   grad_weight[k, c] = sum_n sum_M grad_out * x * r
//
// with the per-row terms of grad_weight written to a workspace and summed over rows in a fixed order afterwards.
// HBM-bound: x in and out once forward; x, grad_out in and grad_x out once backward.
#include "cgtp_device.h"
#include "cgtp_host.h"

namespace cgtp {
namespace {

constexpr int kNormMaxDim = 13;   // rows of the largest irrep held in registers (l = 6)
constexpr int kNormMaxIrreps = 64;

struct NormSeg {                  // irrep boundaries and 1 / dim as the caller's table holds it, passed by value
  int n_irreps;
  short first[kNormMaxIrreps + 1];
  float rdim[kNormMaxIrreps];
};

template <typename T, int V>
struct NormLane {
  int64_t row;     // this lane's row, clamped into range
  int c;           // first of its V channels, clamped into range
  int sub, lpr;
  bool ok;
};

template <typename T, int V>
__device__ __forceinline__ NormLane<T, V> norm_lane(int64_t n_rows, int C, int lpr_log2) {
  NormLane<T, V> L;
  const int lane = threadIdx.x & (kWave - 1);
  L.lpr = 1 << lpr_log2;
  L.sub = lane & (L.lpr - 1);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int64_t r = wave * (kWave >> lpr_log2) + (lane >> lpr_log2);
  const int c = L.sub * V;
  L.ok = r < n_rows && c < C;
  L.row = r < n_rows ? r : 0;
  L.c = c < C ? c : 0;
  return L;
}

template <typename T, int V>
__global__ void __launch_bounds__(256) layer_rms_fwd_kernel(const T* __restrict__ x, const T* __restrict__ weight,
                                                            T* __restrict__ out, T* __restrict__ rsigma, NormSeg seg,
                                                            int64_t n_rows, int D, int C, int scaled, T eps,
                                                            int lpr_log2) {
  const NormLane<T, V> L = norm_lane<T, V>(n_rows, C, lpr_log2);
  const T* xr = x + (L.row * D) * C + L.c;
  T* orow = out + (L.row * D) * C + L.c;
  for (int k = 0; k < seg.n_irreps; ++k) {
    const int m0 = seg.first[k], dim = seg.first[k + 1] - m0;   // the same for every lane: scalar branches below
    T v[kNormMaxDim][V];
#pragma unroll
    for (int j = 0; j < kNormMaxDim; ++j)
      if (j < dim) load_vec<T, V>(v[j], xr + (int64_t)(m0 + j) * C);
    T ss = T(0);
#pragma unroll
    for (int j = 0; j < kNormMaxDim; ++j)
      if (j < dim) {
#pragma unroll
        for (int e = 0; e < V; ++e) ss += v[j][e] * v[j][e];
      }
    ss = group_sum(L.ok ? ss : T(0), L.lpr);
    const T ms = scaled ? ss / T(C) * T(seg.rdim[k]) : ss / T(C);
    const T r = T(1) / sqrt(ms + eps);
    if (L.ok && L.sub == 0 && rsigma) rsigma[L.row * seg.n_irreps + k] = r;
    T w[V];
#pragma unroll
    for (int e = 0; e < V; ++e) w[e] = r;
    if (weight) {
      T g[V];
      load_vec<T, V>(g, weight + (int64_t)k * C + L.c);
#pragma unroll
      for (int e = 0; e < V; ++e) w[e] *= g[e];
    }
    if (L.ok) {
#pragma unroll
      for (int j = 0; j < kNormMaxDim; ++j)
        if (j < dim) {
          T o[V];
#pragma unroll
          for (int e = 0; e < V; ++e) o[e] = v[j][e] * w[e];
          store_vec<T, V>(orow + (int64_t)(m0 + j) * C, o);
        }
    }
  }
}

// gw_rows: (n_rows, n_irreps, C) per-row terms of grad_weight, or nullptr.
template <typename T, int V>
__global__ void __launch_bounds__(256) layer_rms_bwd_kernel(const T* __restrict__ x, const T* __restrict__ weight,
                                                            const T* __restrict__ rsigma, const T* __restrict__ gout,
                                                            T* __restrict__ gx, T* __restrict__ gw_rows, NormSeg seg,
                                                            int64_t n_rows, int D, int C, int scaled, int lpr_log2) {
  const NormLane<T, V> L = norm_lane<T, V>(n_rows, C, lpr_log2);
  const T* xr = x + (L.row * D) * C + L.c;
  const T* gr = gout + (L.row * D) * C + L.c;
  T* gxr = gx ? gx + (L.row * D) * C + L.c : nullptr;
  for (int k = 0; k < seg.n_irreps; ++k) {
    const int m0 = seg.first[k], dim = seg.first[k + 1] - m0;
    T v[kNormMaxDim][V], g[kNormMaxDim][V];
#pragma unroll
    for (int j = 0; j < kNormMaxDim; ++j)
      if (j < dim) {
        load_vec<T, V>(v[j], xr + (int64_t)(m0 + j) * C);
        load_vec<T, V>(g[j], gr + (int64_t)(m0 + j) * C);
      }
    const T r = rsigma[L.row * seg.n_irreps + k];
    T w[V];
#pragma unroll
    for (int e = 0; e < V; ++e) w[e] = T(1);
    if (weight) load_vec<T, V>(w, weight + (int64_t)k * C + L.c);
    // per-row term of grad_weight and the block's dot product <grad_out * weight, x>
    T gw[V], dot = T(0);
#pragma unroll
    for (int e = 0; e < V; ++e) gw[e] = T(0);
#pragma unroll
    for (int j = 0; j < kNormMaxDim; ++j)
      if (j < dim) {
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const T p = g[j][e] * v[j][e];
          gw[e] += p;
          dot += p * w[e];
        }
      }
    if (gw_rows && L.ok) {
#pragma unroll
      for (int e = 0; e < V; ++e) gw[e] *= r;
      store_vec<T, V>(gw_rows + (L.row * seg.n_irreps + k) * C + L.c, gw);
    }
    if (gxr) {
      dot = group_sum(L.ok ? dot : T(0), L.lpr) / T(C);
      if (scaled) dot *= T(seg.rdim[k]);
      const T back = r * r * dot;
      if (L.ok) {
#pragma unroll
        for (int j = 0; j < kNormMaxDim; ++j)
          if (j < dim) {
            T o[V];
#pragma unroll
            for (int e = 0; e < V; ++e) o[e] = r * (g[j][e] * w[e] - v[j][e] * back);
            store_vec<T, V>(gxr + (int64_t)(m0 + j) * C, o);
          }
      }
    }
  }
}

// Shape of a launch: vector width (16 bytes when C and the pointers allow it), lanes per row; 0 = unsupported.
struct NormShape { int v, lpr_log2; };

template <typename T>
NormShape norm_shape(int C, const void* const* ptrs, int n_ptrs) {
  constexpr int VW = 16 / sizeof(T);
  bool aligned = C % VW == 0;
  for (int i = 0; i < n_ptrs; ++i)
    if (ptrs[i] && (reinterpret_cast<uintptr_t>(ptrs[i]) & 15u)) aligned = false;
  const int v = aligned ? VW : 1;
  const int lanes = (C + v - 1) / v;
  if (lanes > kWave) return {0, 0};
  int lg = 0;
  while ((1 << lg) < lanes) ++lg;
  return {v, lg};
}

int norm_check(const void* x, const int32_t* irrep_seg, const float* irrep_rdims, int n_irreps, int64_t n_rows, int D,
               int C, int dtype, NormSeg* seg) {
  if (dtype != CGTP_F32 && dtype != CGTP_F64) return CGTP_ERR_DTYPE;
  if (n_rows < 0 || D <= 0 || C <= 0 || n_irreps <= 0 || n_irreps > kNormMaxIrreps) return CGTP_ERR_SHAPE;
  if (!irrep_seg || (n_rows > 0 && !x)) return CGTP_ERR_NULL;
  if (irrep_seg[0] != 0 || irrep_seg[n_irreps] != D) return CGTP_ERR_SHAPE;
  seg->n_irreps = n_irreps;
  for (int k = 0; k <= n_irreps; ++k) {
    if (k && (irrep_seg[k] <= irrep_seg[k - 1] || irrep_seg[k] - irrep_seg[k - 1] > kNormMaxDim)) return CGTP_ERR_SHAPE;
    seg->first[k] = (short)irrep_seg[k];
    if (k) seg->rdim[k - 1] = irrep_rdims ? irrep_rdims[k - 1] : 1.0f / (float)(irrep_seg[k] - irrep_seg[k - 1]);
  }
  return CGTP_OK;
}

unsigned norm_grid(int64_t n_rows, int lpr_log2) {
  const int64_t rows_per_block = (int64_t)4 * (kWave >> lpr_log2);
  return (unsigned)((n_rows + rows_per_block - 1) / rows_per_block);
}

template <typename T>
int fwd_launch(const void* x, const void* weight, void* out, void* rsigma, const NormSeg& seg, int64_t n_rows, int D,
               int C, int scaled, double eps, hipStream_t stream) {
  const void* ptrs[3] = {x, weight, out};
  const NormShape s = norm_shape<T>(C, ptrs, 3);
  if (!s.v) return CGTP_ERR_SHAPE;
  auto kern = s.v == 1 ? layer_rms_fwd_kernel<T, 1> : layer_rms_fwd_kernel<T, 16 / sizeof(T)>;
  hipLaunchKernelGGL(kern, dim3(norm_grid(n_rows, s.lpr_log2)), dim3(256), 0, stream, (const T*)x, (const T*)weight,
                     (T*)out, (T*)rsigma, seg, n_rows, D, C, scaled, (T)eps, s.lpr_log2);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

template <typename T>
int bwd_launch(const void* x, const void* weight, const void* rsigma, const void* gout, void* gx, void* gweight,
               void* workspace, const NormSeg& seg, int64_t n_rows, int D, int C, int scaled, hipStream_t stream) {
  const void* ptrs[5] = {x, weight, gout, gx, gweight ? workspace : nullptr};
  const NormShape s = norm_shape<T>(C, ptrs, 5);
  if (!s.v) return CGTP_ERR_SHAPE;
  auto kern = s.v == 1 ? layer_rms_bwd_kernel<T, 1> : layer_rms_bwd_kernel<T, 16 / sizeof(T)>;
  hipLaunchKernelGGL(kern, dim3(norm_grid(n_rows, s.lpr_log2)), dim3(256), 0, stream, (const T*)x, (const T*)weight,
                     (const T*)rsigma, (const T*)gout, (T*)gx, gweight ? (T*)workspace : (T*)nullptr, seg, n_rows, D, C,
                     scaled, s.lpr_log2);
  if (hipGetLastError() != hipSuccess) return CGTP_ERR_LAUNCH;
  if (gweight) {
    const int64_t per_row = (int64_t)seg.n_irreps * C;
    const int64_t chunks = (n_rows + kSumRows - 1) / kSumRows;
    T* part = (T*)workspace + n_rows * per_row;
    launch_rows_sum<T>((const T*)workspace, part, n_rows, per_row, stream);
    launch_partial_sum<T>((const T*)part, (T*)gweight, chunks, per_row, stream);
    if (hipGetLastError() != hipSuccess) return CGTP_ERR_LAUNCH;
  }
  return CGTP_OK;
}

}  // namespace
}  // namespace cgtp

extern "C" {

int cgtp_layer_rms_supported(const int32_t* irrep_seg, int n_irreps, int C, int dtype) {
  using namespace cgtp;
  if (!irrep_seg || n_irreps <= 0 || n_irreps > kNormMaxIrreps || C <= 0) return 0;
  if (dtype != CGTP_F32 && dtype != CGTP_F64) return 0;
  for (int k = 1; k <= n_irreps; ++k) {
    const int dim = irrep_seg[k] - irrep_seg[k - 1];
    if (dim <= 0 || dim > kNormMaxDim) return 0;
  }
  return C <= kWave || (C % (16 / (int)elem_size(dtype)) == 0 && C / (16 / (int)elem_size(dtype)) <= kWave);
}

int64_t cgtp_layer_rms_workspace_bytes(int64_t n_rows, int n_irreps, int C, int dtype) {
  using namespace cgtp;
  if (n_rows <= 0 || n_irreps <= 0 || C <= 0) return 0;
  const int64_t per_row = (int64_t)n_irreps * C;
  return (n_rows + (n_rows + kSumRows - 1) / kSumRows) * per_row * elem_size(dtype);
}

int cgtp_layer_rms_forward(const void* x, const void* weight, void* out, void* rsigma, const int32_t* irrep_seg,
                           const float* irrep_rdims, int n_irreps, int64_t n_rows, int D, int C, int scaled,
                           double eps, int dtype, void* stream) {
  using namespace cgtp;
  NormSeg seg;
  if (int rc = norm_check(x, irrep_seg, irrep_rdims, n_irreps, n_rows, D, C, dtype, &seg)) return rc;
  if (n_rows == 0) return CGTP_OK;
  if (!out) return CGTP_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  return dtype == CGTP_F32 ? fwd_launch<float>(x, weight, out, rsigma, seg, n_rows, D, C, scaled, eps, s)
                           : fwd_launch<double>(x, weight, out, rsigma, seg, n_rows, D, C, scaled, eps, s);
}

int cgtp_layer_rms_backward(const void* x, const void* weight, const void* rsigma, const void* grad_out,
                            void* grad_x, void* grad_weight, void* workspace, const int32_t* irrep_seg,
                            const float* irrep_rdims, int n_irreps, int64_t n_rows, int D, int C, int scaled,
                            int dtype, void* stream) {
  using namespace cgtp;
  NormSeg seg;
  if (int rc = norm_check(x, irrep_seg, irrep_rdims, n_irreps, n_rows, D, C, dtype, &seg)) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (n_rows == 0) {   // no rows (the operands may be null): the sum over them is zero, written by the summation
                       // kernel over zero partials
    if (grad_weight) {
      if (dtype == CGTP_F32) launch_partial_sum<float>(nullptr, (float*)grad_weight, 0, (int64_t)n_irreps * C, s);
      else launch_partial_sum<double>(nullptr, (double*)grad_weight, 0, (int64_t)n_irreps * C, s);
    }
    return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
  }
  if (!rsigma || !grad_out) return CGTP_ERR_NULL;
  if (grad_weight && !workspace) return CGTP_ERR_WORKSPACE;
  return dtype == CGTP_F32
             ? bwd_launch<float>(x, weight, rsigma, grad_out, grad_x, grad_weight, workspace, seg, n_rows, D, C, scaled, s)
             : bwd_launch<double>(x, weight, rsigma, grad_out, grad_x, grad_weight, workspace, seg, n_rows, D, C, scaled, s);
}

}  // extern "C"
