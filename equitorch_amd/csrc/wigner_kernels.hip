// Rotation of equivariant features by Euler angles in one pass (cgtp_wigner_rotate):
//
//   out[n] = Z(alpha_n) J Z(beta_n) J Z(gamma_n) x[n]          (transposed: Z(gamma)^T J^T Z(beta)^T J^T Z(alpha)^T)
//
// The reference applies the five factors as five operator launches (sparse_vecsca for the rotations about z,
// sparse_scale for the constant matrix J, equitorch/nn/functional/wigner_d.py:14-56), each a pass over the feature
// tensor.  The rotation is block diagonal over the irreps, so here a row is walked irrep by irrep: the 2l+1
// components of one irrep (l <= 6) are loaded into registers, the factors are applied there, and the result is
// written.  A row takes LPR = next_pow2(C / V) lanes with V channels each (16-byte accesses); a wavefront covers
// 64 / LPR rows.
//
//   Z(phi):  y[m] = cs[2|m|] x[m] - sign(m) cs[2|m| - 1] x[-m],  y[0] = cs[0] x[0],   cs = (1, sin phi, cos phi, sin 2 phi, ...)
//            (equitorch/utils/_structs.py:460-521), one (N, 1 + 2 max_m) tensor per angle, NULL = factor skipped
//            (with beta skipped both J factors go too, as in the reference);
//   J:       dense (2l+1) x (2l+1) block per irrep, passed by the caller (the values of its sparse table), staged in
//            LDS and read with wave-uniform addresses.
//
// Products and sums are formed in the order of the table-driven composition (multiply, multiply, add for Z; fused
// multiply-adds over the columns in rising order for J), so results agree with it to the last bit wherever J's
// dropped entries are zeros.  HBM-bound: the feature tensor in and out once.
#include "cgtp_device.h"
#include "cgtp_host.h"

namespace cgtp {
namespace {

constexpr int kRotMaxL = 6;
constexpr int kRotMaxIrreps = 64;

struct RotIrreps {                 // passed by value: first component, degree and offset of the J block of every irrep
  int n_irreps;
  short first[kRotMaxIrreps];
  unsigned char degree[kRotMaxIrreps];
  short j_offset[kRotMaxIrreps];
};

// y = Z(cs) v in place; `flip`: the transposed factor (sines negated).
template <typename T, int L, int V>
__device__ __forceinline__ void rot_z(T (&v)[2 * L + 1][V], const T* __restrict__ cs, bool flip) {
  const T c0 = cs[0];
#pragma unroll
  for (int e = 0; e < V; ++e) v[L][e] = v[L][e] * c0;
#pragma unroll
  for (int m = 1; m <= L; ++m) {
    const T c = cs[2 * m];
    const T s = flip ? -cs[2 * m - 1] : cs[2 * m - 1];
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const T p = v[L + m][e], q = v[L - m][e];
      // table order: the cosine term first, then the sine term with its sign
      v[L + m][e] = p * c + (-(q * s));
      v[L - m][e] = q * c + p * s;
    }
  }
}

// v <- J v (`flip`: J^T v) with the dense block `jb` (row-major, in LDS).
template <typename T, int L, int V>
__device__ __forceinline__ void rot_j(T (&v)[2 * L + 1][V], const T* jb, bool flip) {
  constexpr int DIM = 2 * L + 1;
  T y[DIM][V];
#pragma unroll
  for (int r = 0; r < DIM; ++r) {
#pragma unroll
    for (int e = 0; e < V; ++e) y[r][e] = T(0);
#pragma unroll
    for (int c = 0; c < DIM; ++c) {
      const T j = flip ? jb[c * DIM + r] : jb[r * DIM + c];
#pragma unroll
      for (int e = 0; e < V; ++e) y[r][e] = fma(j, v[c][e], y[r][e]);
    }
  }
#pragma unroll
  for (int r = 0; r < DIM; ++r)
#pragma unroll
    for (int e = 0; e < V; ++e) v[r][e] = y[r][e];
}

template <typename T, int L, int V>
__device__ __forceinline__ void rot_irrep(const T* __restrict__ xr, T* __restrict__ orow, int C, bool ok,
                                          const T* first, const T* middle, const T* last, const T* jb, bool flip) {
  constexpr int DIM = 2 * L + 1;
  T v[DIM][V];
#pragma unroll
  for (int j = 0; j < DIM; ++j) load_vec<T, V>(v[j], xr + (int64_t)j * C);
  if (first) rot_z<T, L, V>(v, first, flip);
  if (middle) {
    rot_j<T, L, V>(v, jb, flip);
    rot_z<T, L, V>(v, middle, flip);
    rot_j<T, L, V>(v, jb, flip);
  }
  if (last) rot_z<T, L, V>(v, last, flip);
  if (ok) {
#pragma unroll
    for (int j = 0; j < DIM; ++j) store_vec<T, V>(orow + (int64_t)j * C, v[j]);
  }
}

// first / middle / last: the sincos tensors of the factors in the order they are applied (gamma, beta, alpha for
// the rotation; alpha, beta, gamma with flip for its transpose), each (n_rows, cs_dim) or nullptr.
// MAXL: the largest degree the launch has to handle (2, 4 or 6): the register allotment follows the largest block.
template <typename T, int V, int MAXL>
__global__ void __launch_bounds__(256) wigner_rotate_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                            const T* __restrict__ first, const T* __restrict__ middle,
                                                            const T* __restrict__ last, const T* __restrict__ jblocks,
                                                            int j_elems, RotIrreps irr, int64_t n_rows, int D, int C,
                                                            int cs_dim, int flip, int lpr_log2) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* sj = reinterpret_cast<T*>(smem);
  for (int t = threadIdx.x; t < j_elems; t += blockDim.x) sj[t] = jblocks[t];
  __syncthreads();
  const int lane = threadIdx.x & (kWave - 1);
  const int lpr = 1 << lpr_log2, sub = lane & (lpr - 1);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int64_t r = wave * (kWave >> lpr_log2) + (lane >> lpr_log2);
  const int c = sub * V;
  const bool ok = r < n_rows && c < C;
  const int64_t row = r < n_rows ? r : 0;
  const int cc = c < C ? c : 0;
  const T* xrow = x + (row * D) * C + cc;
  T* orow = out + (row * D) * C + cc;
  const T* f = first ? first + row * cs_dim : nullptr;
  const T* m = middle ? middle + row * cs_dim : nullptr;
  const T* l = last ? last + row * cs_dim : nullptr;
  for (int k = 0; k < irr.n_irreps; ++k) {
    const int m0 = irr.first[k];
    const T* jb = sj + irr.j_offset[k];
    const T* xi = xrow + (int64_t)m0 * C;
    T* oi = orow + (int64_t)m0 * C;
    switch (irr.degree[k]) {     // the same for every lane: a scalar branch
      case 0: rot_irrep<T, 0, V>(xi, oi, C, ok, f, m, l, jb, flip); break;
      case 1: rot_irrep<T, 1, V>(xi, oi, C, ok, f, m, l, jb, flip); break;
      case 2: rot_irrep<T, 2, V>(xi, oi, C, ok, f, m, l, jb, flip); break;
      case 3: if constexpr (MAXL >= 3) rot_irrep<T, 3, V>(xi, oi, C, ok, f, m, l, jb, flip); break;
      case 4: if constexpr (MAXL >= 4) rot_irrep<T, 4, V>(xi, oi, C, ok, f, m, l, jb, flip); break;
      case 5: if constexpr (MAXL >= 5) rot_irrep<T, 5, V>(xi, oi, C, ok, f, m, l, jb, flip); break;
      case 6: if constexpr (MAXL >= 6) rot_irrep<T, 6, V>(xi, oi, C, ok, f, m, l, jb, flip); break;
      default: break;
    }
  }
}

// ---- gradients of the rotation with respect to the features and the sincos tensors ------------------------------
// With u0 = x, u2 = J Z(gamma) u0, u4 = J Z(beta) u2 (the inputs of the three rotations about z) recomputed in
// registers and h the gradient flowing back from the output,
//   d cs[2m]   += sum_c h[+m] u[+m] + h[-m] u[-m],   d cs[2m-1] += sum_c -h[+m] u[-m] + h[-m] u[+m],   d cs[0] += sum_c h[0] u[0]
// at each rotation (h taken before that rotation's transpose is applied to it), summed over the irreps and the
// channels of the row.
template <typename T, int L, int V, int NACC>
__device__ __forceinline__ void rot_z_grad(T (&acc)[NACC], const T (&h)[2 * L + 1][V], const T (&u)[2 * L + 1][V]) {
#pragma unroll
  for (int e = 0; e < V; ++e) acc[0] += h[L][e] * u[L][e];
#pragma unroll
  for (int m = 1; m <= L; ++m) {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      acc[2 * m] += h[L + m][e] * u[L + m][e] + h[L - m][e] * u[L - m][e];
      acc[2 * m - 1] += h[L - m][e] * u[L + m][e] - h[L + m][e] * u[L - m][e];
    }
  }
}

template <typename T, int L, int V>
__device__ __forceinline__ void rot_copy(T (&dst)[2 * L + 1][V], const T (&src)[2 * L + 1][V]) {
#pragma unroll
  for (int j = 0; j < 2 * L + 1; ++j)
#pragma unroll
    for (int e = 0; e < V; ++e) dst[j][e] = src[j][e];
}

template <typename T, int L, int V, int NACC>
__device__ __forceinline__ void rot_irrep_bwd(const T* __restrict__ xr, const T* __restrict__ gr, T* __restrict__ gxr,
                                              int C, bool ok, const T* ca, const T* cb, const T* cg, const T* jb,
                                              T (&acc_a)[NACC], T (&acc_b)[NACC], T (&acc_g)[NACC]) {
  constexpr int DIM = 2 * L + 1;
  T u0[DIM][V], u2[DIM][V], u[DIM][V], h[DIM][V];
#pragma unroll
  for (int j = 0; j < DIM; ++j) {
    load_vec<T, V>(u0[j], xr + (int64_t)j * C);
    load_vec<T, V>(h[j], gr + (int64_t)j * C);
  }
  rot_copy<T, L, V>(u, u0);
  if (cg) rot_z<T, L, V>(u, cg, false);
  if (cb) {
    rot_j<T, L, V>(u, jb, false);
    rot_copy<T, L, V>(u2, u);
    rot_z<T, L, V>(u, cb, false);
    rot_j<T, L, V>(u, jb, false);
  }
  // u is now the input of the last rotation about z
  if (ca) {
    rot_z_grad<T, L, V, NACC>(acc_a, h, u);
    rot_z<T, L, V>(h, ca, true);
  }
  if (cb) {
    rot_j<T, L, V>(h, jb, true);
    rot_z_grad<T, L, V, NACC>(acc_b, h, u2);
    rot_z<T, L, V>(h, cb, true);
    rot_j<T, L, V>(h, jb, true);
  }
  if (cg) {
    rot_z_grad<T, L, V, NACC>(acc_g, h, u0);
    rot_z<T, L, V>(h, cg, true);
  }
  if (gxr && ok) {
#pragma unroll
    for (int j = 0; j < DIM; ++j) store_vec<T, V>(gxr + (int64_t)j * C, h[j]);
  }
}

template <typename T, int V, int MAXL>
__global__ void __launch_bounds__(256) wigner_rotate_bwd_kernel(
    const T* __restrict__ x, const T* __restrict__ gout, const T* __restrict__ cs_a, const T* __restrict__ cs_b,
    const T* __restrict__ cs_g, const T* __restrict__ jblocks, int j_elems, RotIrreps irr, int64_t n_rows, int D, int C,
    int cs_dim, T* __restrict__ gx, T* __restrict__ g_a, T* __restrict__ g_b, T* __restrict__ g_g, int lpr_log2) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int NACC = 2 * MAXL + 1;
  T* sj = reinterpret_cast<T*>(smem);
  for (int t = threadIdx.x; t < j_elems; t += blockDim.x) sj[t] = jblocks[t];
  __syncthreads();
  const int lane = threadIdx.x & (kWave - 1);
  const int lpr = 1 << lpr_log2, sub = lane & (lpr - 1);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int64_t r = wave * (kWave >> lpr_log2) + (lane >> lpr_log2);
  const int c = sub * V;
  const bool ok = r < n_rows && c < C;
  const int64_t row = r < n_rows ? r : 0;
  const int cc = c < C ? c : 0;
  const T* xrow = x + (row * D) * C + cc;
  const T* grow = gout + (row * D) * C + cc;
  T* gxrow = gx ? gx + (row * D) * C + cc : nullptr;
  const T* ca = cs_a ? cs_a + row * cs_dim : nullptr;
  const T* cb = cs_b ? cs_b + row * cs_dim : nullptr;
  const T* cg = cs_g ? cs_g + row * cs_dim : nullptr;
  T acc_a[NACC], acc_b[NACC], acc_g[NACC];
#pragma unroll
  for (int i = 0; i < NACC; ++i) acc_a[i] = acc_b[i] = acc_g[i] = T(0);
  for (int k = 0; k < irr.n_irreps; ++k) {
    const int m0 = irr.first[k];
    const T* jb = sj + irr.j_offset[k];
    const T* xi = xrow + (int64_t)m0 * C;
    const T* gi = grow + (int64_t)m0 * C;
    T* oi = gxrow ? gxrow + (int64_t)m0 * C : nullptr;
#define CGTP_ROT_BWD(LL) rot_irrep_bwd<T, LL, V, NACC>(xi, gi, oi, C, ok, ca, cb, cg, jb, acc_a, acc_b, acc_g)
    switch (irr.degree[k]) {     // the same for every lane: a scalar branch
      case 0: CGTP_ROT_BWD(0); break;
      case 1: CGTP_ROT_BWD(1); break;
      case 2: CGTP_ROT_BWD(2); break;
      case 3: if constexpr (MAXL >= 3) CGTP_ROT_BWD(3); break;
      case 4: if constexpr (MAXL >= 4) CGTP_ROT_BWD(4); break;
      case 5: if constexpr (MAXL >= 5) CGTP_ROT_BWD(5); break;
      case 6: if constexpr (MAXL >= 6) CGTP_ROT_BWD(6); break;
      default: break;
    }
#undef CGTP_ROT_BWD
  }
  // sums over the channels of the row; columns of the sincos tensors beyond the largest degree get zero
  T* outs[3] = {g_a, g_b, g_g};
  T* accs[3] = {acc_a, acc_b, acc_g};
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    if (!outs[a]) continue;
#pragma unroll
    for (int i = 0; i < NACC; ++i) {
      const T total = group_sum(ok ? accs[a][i] : T(0), lpr);
      if (r < n_rows && sub == 0 && i < cs_dim) outs[a][r * cs_dim + i] = total;
    }
    if (r < n_rows && sub == 0)
      for (int i = NACC; i < cs_dim; ++i) outs[a][r * cs_dim + i] = T(0);
  }
}

template <typename T, int V>
int rotate_bwd_launch_v(const void* x, const void* gout, const void* ca, const void* cb, const void* cg,
                        const void* jblocks, int j_elems, const RotIrreps& irr, int max_l, int64_t n_rows, int D, int C,
                        int cs_dim, void* gx, void* ga, void* gb, void* gg, hipStream_t stream) {
  const int lanes = (C + V - 1) / V;
  if (lanes > kWave) return CGTP_ERR_SHAPE;
  int lg = 0;
  while ((1 << lg) < lanes) ++lg;
  const int64_t rows_per_block = (int64_t)4 * (kWave >> lg);
  const int64_t blocks = (n_rows + rows_per_block - 1) / rows_per_block;
  if (blocks > 0x7fffffff) return CGTP_ERR_SHAPE;
  auto kern = max_l <= 2 ? wigner_rotate_bwd_kernel<T, V, 2>
                         : max_l <= 4 ? wigner_rotate_bwd_kernel<T, V, 4> : wigner_rotate_bwd_kernel<T, V, 6>;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), (size_t)j_elems * sizeof(T), stream, (const T*)x,
                     (const T*)gout, (const T*)ca, (const T*)cb, (const T*)cg, (const T*)jblocks, j_elems, irr, n_rows, D,
                     C, cs_dim, (T*)gx, (T*)ga, (T*)gb, (T*)gg, lg);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

// Five sets of 2l+1 rows live at once: the channels per lane shrink with the largest degree so that they fit.
template <typename T>
int rotate_bwd_launch(const void* x, const void* gout, const void* ca, const void* cb, const void* cg,
                      const void* jblocks, int j_elems, const RotIrreps& irr, int max_l, int64_t n_rows, int D, int C,
                      int cs_dim, void* gx, void* ga, void* gb, void* gg, hipStream_t stream) {
  constexpr int VW = 16 / sizeof(T);            // 4 (fp32) or 2 (fp64)
  constexpr int VH = VW / 2;                    // 2 or 1
  const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gout) | reinterpret_cast<uintptr_t>(gx);
  const int want = max_l <= 4 ? VW : VH;
  int v = 1;
  if (want == VW && C % VW == 0 && (bits & 15u) == 0 && C / VW <= kWave) v = VW;
  else if (VH > 1 && C % VH == 0 && (bits & (VH * sizeof(T) - 1)) == 0 && C / VH <= kWave) v = VH;
  if (v == VW)
    return rotate_bwd_launch_v<T, VW>(x, gout, ca, cb, cg, jblocks, j_elems, irr, max_l, n_rows, D, C, cs_dim, gx, ga, gb, gg, stream);
  if (VH > 1 && v == VH)
    return rotate_bwd_launch_v<T, (VH > 1 ? VH : 1)>(x, gout, ca, cb, cg, jblocks, j_elems, irr, max_l, n_rows, D, C, cs_dim, gx, ga, gb, gg, stream);
  return rotate_bwd_launch_v<T, 1>(x, gout, ca, cb, cg, jblocks, j_elems, irr, max_l, n_rows, D, C, cs_dim, gx, ga, gb, gg, stream);
}

template <typename T>
int rotate_launch(const void* x, void* out, const void* first, const void* middle, const void* last,
                  const void* jblocks, int j_elems, const RotIrreps& irr, int max_l, int64_t n_rows, int D, int C,
                  int cs_dim, int flip, hipStream_t stream) {
  constexpr int VW = 16 / sizeof(T);
  const bool aligned = C % VW == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  const int v = aligned ? VW : 1;
  const int lanes = (C + v - 1) / v;
  if (lanes > kWave) return CGTP_ERR_SHAPE;
  int lg = 0;
  while ((1 << lg) < lanes) ++lg;
  const int64_t rows_per_block = (int64_t)4 * (kWave >> lg);
  const int64_t blocks = (n_rows + rows_per_block - 1) / rows_per_block;
  if (blocks > 0x7fffffff) return CGTP_ERR_SHAPE;
  auto kern = v == 1 ? (max_l <= 2 ? wigner_rotate_kernel<T, 1, 2> : max_l <= 4 ? wigner_rotate_kernel<T, 1, 4>
                                                                               : wigner_rotate_kernel<T, 1, 6>)
                     : (max_l <= 2 ? wigner_rotate_kernel<T, VW, 2> : max_l <= 4 ? wigner_rotate_kernel<T, VW, 4>
                                                                                : wigner_rotate_kernel<T, VW, 6>);
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), (size_t)j_elems * sizeof(T), stream, (const T*)x, (T*)out,
                     (const T*)first, (const T*)middle, (const T*)last, (const T*)jblocks, j_elems, irr, n_rows, D, C,
                     cs_dim, flip, lg);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

}  // namespace
}  // namespace cgtp

extern "C" {

int cgtp_wigner_rotate_supported(const int32_t* irrep_first, const int32_t* irrep_degree, int n_irreps, int C,
                                 int dtype) {
  using namespace cgtp;
  if (!irrep_first || !irrep_degree || n_irreps <= 0 || n_irreps > kRotMaxIrreps || C <= 0) return 0;
  if (dtype != CGTP_F32 && dtype != CGTP_F64) return 0;
  int at = 0;
  for (int k = 0; k < n_irreps; ++k) {
    if (irrep_degree[k] < 0 || irrep_degree[k] > kRotMaxL || irrep_first[k] != at) return 0;
    at += 2 * irrep_degree[k] + 1;
  }
  const int vw = 16 / (int)elem_size(dtype);
  return C <= kWave || (C % vw == 0 && C / vw <= kWave);
}

static int rot_setup(const int32_t* irrep_first, const int32_t* irrep_degree, int n_irreps, int C, int cs_dim,
                     int dtype, cgtp::RotIrreps* irr, int* D, int* j_elems, int* max_l) {
  using namespace cgtp;
  if (!cgtp_wigner_rotate_supported(irrep_first, irrep_degree, n_irreps, C, dtype)) return CGTP_ERR_SHAPE;
  irr->n_irreps = n_irreps;
  *D = *j_elems = *max_l = 0;
  for (int k = 0; k < n_irreps; ++k) {
    const int dim = 2 * irrep_degree[k] + 1;
    irr->first[k] = (short)irrep_first[k];
    irr->degree[k] = (unsigned char)irrep_degree[k];
    irr->j_offset[k] = (short)*j_elems;
    *j_elems += dim * dim;
    *D += dim;
    if (irrep_degree[k] > *max_l) *max_l = irrep_degree[k];
  }
  if (cs_dim < 1 + 2 * *max_l || *j_elems > 0x7fff) return CGTP_ERR_SHAPE;
  return CGTP_OK;
}

int cgtp_wigner_rotate(const void* x, void* out, const void* sincos_alpha, const void* sincos_beta,
                       const void* sincos_gamma, const void* j_blocks, const int32_t* irrep_first,
                       const int32_t* irrep_degree, int n_irreps, int64_t n_rows, int C, int cs_dim, int transposed,
                       int dtype, void* stream) {
  using namespace cgtp;
  RotIrreps irr;
  int D = 0, j_elems = 0, max_l = 0;
  if (n_rows < 0 || cs_dim <= 0) return CGTP_ERR_SHAPE;
  if (int rc = rot_setup(irrep_first, irrep_degree, n_irreps, C, cs_dim, dtype, &irr, &D, &j_elems, &max_l)) return rc;
  if (n_rows == 0) return CGTP_OK;
  if (!x || !out || !j_blocks) return CGTP_ERR_NULL;
  // factors in the order they act on x: gamma, (J beta J), alpha; the transpose runs them backwards
  const void* first = transposed ? sincos_alpha : sincos_gamma;
  const void* last = transposed ? sincos_gamma : sincos_alpha;
  hipStream_t s = (hipStream_t)stream;
  return dtype == CGTP_F32
             ? rotate_launch<float>(x, out, first, sincos_beta, last, j_blocks, j_elems, irr, max_l, n_rows, D, C, cs_dim,
                                    transposed, s)
             : rotate_launch<double>(x, out, first, sincos_beta, last, j_blocks, j_elems, irr, max_l, n_rows, D, C, cs_dim,
                                     transposed, s);
}

int cgtp_wigner_rotate_backward(const void* x, const void* grad_out, const void* sincos_alpha, const void* sincos_beta,
                                const void* sincos_gamma, const void* j_blocks, const int32_t* irrep_first,
                                const int32_t* irrep_degree, int n_irreps, int64_t n_rows, int C, int cs_dim,
                                void* grad_x, void* grad_alpha, void* grad_beta, void* grad_gamma, int dtype,
                                void* stream) {
  using namespace cgtp;
  RotIrreps irr;
  int D = 0, j_elems = 0, max_l = 0;
  if (n_rows < 0 || cs_dim <= 0) return CGTP_ERR_SHAPE;
  if (int rc = rot_setup(irrep_first, irrep_degree, n_irreps, C, cs_dim, dtype, &irr, &D, &j_elems, &max_l)) return rc;
  if (n_rows == 0) return CGTP_OK;
  if (!x || !grad_out || !j_blocks) return CGTP_ERR_NULL;
  if ((grad_alpha && !sincos_alpha) || (grad_beta && !sincos_beta) || (grad_gamma && !sincos_gamma)) return CGTP_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  return dtype == CGTP_F32
             ? rotate_bwd_launch<float>(x, grad_out, sincos_alpha, sincos_beta, sincos_gamma, j_blocks, j_elems, irr,
                                        max_l, n_rows, D, C, cs_dim, grad_x, grad_alpha, grad_beta, grad_gamma, s)
             : rotate_bwd_launch<double>(x, grad_out, sincos_alpha, sincos_beta, sincos_gamma, j_blocks, j_elems, irr,
                                         max_l, n_rows, D, C, cs_dim, grad_x, grad_alpha, grad_beta, grad_gamma, s);
}

}  // extern "C"
