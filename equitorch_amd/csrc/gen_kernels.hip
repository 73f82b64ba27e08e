// General table-driven contraction over two channel axes (u, w):
//
//   out[r, o, (u), (w)] = sum_{t in seg[o]} coef[t] * sum_{axes not in out} A[r, ia_t, ..] * B[r, ib_t, ..] * W[r, iw_t, ..]
//
// Each operand carries any subset of the two channel axes; an axis that the output carries is element-wise,
// an axis it does not carry is summed.  This covers the matrix members of the reference's operator family
// (vecmat, outer, mat_t_vec), the fully connected tensor products built from them and all their gradients.
// It is the any-shape, any-table path: one thread per output element, table in LDS, no tiling.
#include "cgtp_device.h"
#include "cgtp_host.h"

namespace cgtp {

template <typename T>
struct GenOp {
  const T* data;
  int64_t row_stride, idx_stride, u_stride, w_stride;  // strides are 0 for an axis the operand lacks
  int present;
};

template <typename T>
struct GenDev {
  GenOp<T> a, b, w;
  const T* coef;
  const uint32_t* idx;
  const int32_t* seg;
  int n_out, nnz;
  T* out;
  int64_t n_rows;
  int U, Wd, out_u, out_w, reduce_rows;
};

template <typename T>
__device__ __forceinline__ T gen_term(const GenDev<T>& a, int64_t r, uint32_t pk, int u, int w) {
  T v = T(1);
  if (a.a.present) v *= a.a.data[r * a.a.row_stride + (int64_t)(pk & 1023u) * a.a.idx_stride + u * a.a.u_stride + w * a.a.w_stride];
  if (a.b.present) v *= a.b.data[r * a.b.row_stride + (int64_t)((pk >> 10) & 1023u) * a.b.idx_stride + u * a.b.u_stride + w * a.b.w_stride];
  if (a.w.present) v *= a.w.data[r * a.w.row_stride + (int64_t)(pk >> 20) * a.w.idx_stride + u * a.w.u_stride + w * a.w.w_stride];
  return v;
}

// grid.x = output rows (1 if rows are reduced) * n_out; threads stride over the output's channel elements.
template <typename T>
__global__ void __launch_bounds__(256) gen_kernel(const GenDev<T> a) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* s_coef = reinterpret_cast<T*>(smem);
  uint32_t* s_idx = reinterpret_cast<uint32_t*>(s_coef + a.nnz);
  int32_t* s_seg = reinterpret_cast<int32_t*>(s_idx + a.nnz);
  for (int t = threadIdx.x; t < a.nnz; t += blockDim.x) {
    s_coef[t] = a.coef ? a.coef[t] : T(1);
    s_idx[t] = a.idx[t];
  }
  for (int t = threadIdx.x; t <= a.n_out; t += blockDim.x) s_seg[t] = a.seg[t];
  __syncthreads();

  const int64_t orow = blockIdx.x / a.n_out;
  const int o = (int)(blockIdx.x % a.n_out);
  const int nu = a.out_u ? a.U : 1, nw = a.out_w ? a.Wd : 1;  // extent of the output's channel axes
  const int cu = a.out_u ? 1 : a.U, cw = a.out_w ? 1 : a.Wd;  // extent of the summed axes
  const int64_t r0 = a.reduce_rows ? 0 : orow, r1 = a.reduce_rows ? a.n_rows : orow + 1;
  const int tb = s_seg[o], te = s_seg[o + 1];
  for (int e = threadIdx.x; e < nu * nw; e += blockDim.x) {
    const int eu = a.out_u ? e / nw : 0, ew = a.out_w ? e % nw : 0;
    T acc = T(0);
    for (int64_t r = r0; r < r1; ++r)
      for (int t = tb; t < te; ++t) {
        const uint32_t pk = s_idx[t];
        T inner = T(0);
        for (int su = 0; su < cu; ++su)
          for (int sw = 0; sw < cw; ++sw) inner += gen_term(a, r, pk, eu + su, ew + sw);
        acc = fma(s_coef[t], inner, acc);
      }
    a.out[((int64_t)orow * a.n_out + o) * nu * nw + e] = acc;
  }
}

// The same contraction with one workgroup per output row: the table is staged once per row instead of once per
// (row, output index), and the threads run over all (output index, channel element) pairs of the row, so that outputs
// with few channel elements (an axis summed away) still fill the workgroup.  Consecutive threads take consecutive
// elements of the innermost output axis: stores, and the loads of operands that carry that axis, are contiguous.
template <typename T>
__global__ void __launch_bounds__(256) gen_row_kernel(const GenDev<T> a) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* s_coef = reinterpret_cast<T*>(smem);
  uint32_t* s_idx = reinterpret_cast<uint32_t*>(s_coef + a.nnz);
  int32_t* s_seg = reinterpret_cast<int32_t*>(s_idx + a.nnz);
  for (int t = threadIdx.x; t < a.nnz; t += blockDim.x) {
    s_coef[t] = a.coef ? a.coef[t] : T(1);
    s_idx[t] = a.idx[t];
  }
  for (int t = threadIdx.x; t <= a.n_out; t += blockDim.x) s_seg[t] = a.seg[t];
  __syncthreads();

  const int64_t r = blockIdx.x;
  const int nu = a.out_u ? a.U : 1, nw = a.out_w ? a.Wd : 1;  // extent of the output's channel axes
  const int cu = a.out_u ? 1 : a.U, cw = a.out_w ? 1 : a.Wd;  // extent of the summed axes
  const int per_out = nu * nw, total = a.n_out * per_out;
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    const int o = i / per_out, e = i - o * per_out;
    const int eu = a.out_u ? e / nw : 0, ew = a.out_w ? e % nw : 0;
    const int tb = s_seg[o], te = s_seg[o + 1];
    T acc = T(0);
    for (int t = tb; t < te; ++t) {
      const uint32_t pk = s_idx[t];
      T inner = T(0);
      for (int su = 0; su < cu; ++su)
        for (int sw = 0; sw < cw; ++sw) inner += gen_term(a, r, pk, eu + su, ew + sw);
      acc = fma(s_coef[t], inner, acc);
    }
    a.out[r * total + i] = acc;
  }
}

// ---- two-operand fast paths: the stages of the fully connected ("uvw") tensor product and their gradients -------
// One operand X carries one or both channel axes with the w axis contiguous, the other (Y) one axis, contiguous; the
// third slot is empty.  One workgroup per row; a thread owns V consecutive w (one 16-byte access) of one u.
//   outer:       out[r, o, u, w] = sum_t c_t X[r, ix_t, u] Y[r, iy_t, w]
//   contract w:  out[r, o, u]    = sum_t c_t sum_w X[r, ix_t, u, w] Y[r, iy_t, w]     (reduced over the lanes of one u)
//   contract u:  out[r, o, w]    = sum_t c_t sum_u X[r, ix_t, u, w] Y[r, iy_t, u]     (reduced through LDS)
template <typename T>
struct PairDev {
  const T* x; const T* y;
  int64_t x_row, x_idx, y_row, y_idx;   // strides in elements (x_idx: between sparse indices; u stride of X is W)
  int x_shift, y_shift;                 // bit position of the operand's index in the packed table entry
  uint32_t x_mask, y_mask;              // 10 bits for the first two slots, 12 for the third
  const T* coef; const uint32_t* idx; const int32_t* seg;
  int n_out, nnz;
  T* out;
  int64_t n_rows;
  int U, W;
};

enum { kPairOuter = 0, kPairContractW = 1, kPairContractU = 2 };

template <typename T, int V, int MODE>
__global__ void __launch_bounds__(256) gen_pair_kernel(const PairDev<T> a) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* s_coef = reinterpret_cast<T*>(smem);
  uint32_t* s_idx = reinterpret_cast<uint32_t*>(s_coef + a.nnz);
  int32_t* s_seg = reinterpret_cast<int32_t*>(s_idx + a.nnz);
  // contract u: [U tile][W] partial sums, behind the table at the next 16-byte boundary
  const size_t table_bytes = (size_t)a.nnz * (sizeof(T) + 4) + (size_t)(a.n_out + 1) * 4;
  T* s_red = reinterpret_cast<T*>(smem + ((table_bytes + 15) & ~(size_t)15));
  for (int t = threadIdx.x; t < a.nnz; t += blockDim.x) {
    s_coef[t] = a.coef ? a.coef[t] : T(1);
    s_idx[t] = a.idx[t];
  }
  for (int t = threadIdx.x; t <= a.n_out; t += blockDim.x) s_seg[t] = a.seg[t];
  __syncthreads();

  const int64_t r = blockIdx.x;
  const int wv = a.W / V;                         // lanes per u (a power of two for the contracting modes)
  const int u_tile = blockDim.x / wv;             // rows of u the workgroup covers at once
  const int w0 = (threadIdx.x % wv) * V, ut = threadIdx.x / wv;
  const T* xr = a.x + r * a.x_row;
  const T* yr = a.y + r * a.y_row;
  for (int o = 0; o < a.n_out; ++o) {
    const int tb = s_seg[o], te = s_seg[o + 1];
    for (int u0 = 0; u0 < a.U; u0 += u_tile) {
      const int u = u0 + ut;
      const bool live = u < a.U;
      const int uu = live ? u : 0;
      T acc[V];
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = T(0);
      for (int t = tb; t < te; ++t) {
        const uint32_t pk = s_idx[t];
        const T c = s_coef[t];
        const int64_t ix = (pk >> a.x_shift) & a.x_mask, iy = (pk >> a.y_shift) & a.y_mask;
        if (MODE == kPairOuter) {
          const T xv = xr[ix * a.x_idx + uu];
          T yv[V];
          load_vec<T, V>(yv, yr + iy * a.y_idx + w0);
#pragma unroll
          for (int e = 0; e < V; ++e) acc[e] = fma(c * xv, yv[e], acc[e]);
        } else {
          T xv[V];
          load_vec<T, V>(xv, xr + ix * a.x_idx + (int64_t)uu * a.W + w0);
          if (MODE == kPairContractW) {
            T yv[V];
            load_vec<T, V>(yv, yr + iy * a.y_idx + w0);
#pragma unroll
            for (int e = 0; e < V; ++e) acc[e] = fma(c * xv[e], yv[e], acc[e]);
          } else {
            const T yv = c * yr[iy * a.y_idx + uu];
#pragma unroll
            for (int e = 0; e < V; ++e) acc[e] = fma(xv[e], yv, acc[e]);
          }
        }
      }
      if (MODE == kPairOuter) {
        if (live) store_vec<T, V>(a.out + ((r * a.n_out + o) * a.U + u) * a.W + w0, acc);
      } else if (MODE == kPairContractW) {
        T sum = acc[0];
#pragma unroll
        for (int e = 1; e < V; ++e) sum += acc[e];
        sum = group_sum(sum, wv);
        if (live && w0 == 0) a.out[(r * a.n_out + o) * a.U + u] = sum;
      } else {
        // partial sums of this tile of u into LDS, then one thread per w adds them in a fixed order
        __syncthreads();
#pragma unroll
        for (int e = 0; e < V; ++e) s_red[ut * a.W + w0 + e] = live ? acc[e] : T(0);
        __syncthreads();
        for (int w = threadIdx.x; w < a.W; w += blockDim.x) {
          T sum = T(0);
          for (int j = 0; j < u_tile; ++j) sum += s_red[j * a.W + w];
          T* dst = a.out + (r * a.n_out + o) * a.W + w;
          *dst = u0 == 0 ? sum : *dst + sum;
        }
      }
    }
  }
}

static int gen_check(const cgtp_gen_args* a, int64_t* lds) {
  if (!a) return CGTP_ERR_NULL;
  if (a->dtype != CGTP_F32 && a->dtype != CGTP_F64) return CGTP_ERR_DTYPE;
  if (a->n_out < 0 || a->nnz < 0 || a->n_rows < 0 || a->U <= 0 || a->W <= 0) return CGTP_ERR_SHAPE;
  if (!a->idx || !a->seg || !a->out) return CGTP_ERR_NULL;
  const cgtp_gen_operand* ops[3] = {&a->a, &a->b, &a->w};
  for (const cgtp_gen_operand* o : ops) {
    if (o->present && !o->data) return CGTP_ERR_NULL;
    if (o->row_stride < 0 || o->idx_stride < 0 || o->u_stride < 0 || o->w_stride < 0) return CGTP_ERR_SHAPE;
  }
  *lds = (int64_t)a->nnz * (elem_size(a->dtype) + 4) + ((int64_t)a->n_out + 1) * 4;
  if (*lds > kLdsBytes) return CGTP_ERR_LDS;
  const int64_t blocks = (a->reduce_rows ? 1 : a->n_rows) * a->n_out;
  if (blocks >= (int64_t)1 << 31) return CGTP_ERR_SHAPE;
  return CGTP_OK;
}

template <typename T>
static GenOp<T> gen_op(const cgtp_gen_operand& o) {
  return GenOp<T>{(const T*)o.data, o.row_stride, o.idx_stride, o.u_stride, o.w_stride, o.present};
}

// Recognises the three two-operand shapes above (operands in any two of the three slots) and launches the fast
// kernel; kNotPair when the call has another shape.
constexpr int kNotPair = -1;

template <typename T>
static int gen_pair_launch(const cgtp_gen_args* a, int64_t table_lds, hipStream_t stream) {
  constexpr int V = 16 / sizeof(T);
  if (a->reduce_rows || a->n_rows < 256 || a->n_out == 0 || a->W % V || a->W / V > 256) return kNotPair;
  const cgtp_gen_operand* ops[3] = {&a->a, &a->b, &a->w};
  const int shifts[3] = {0, 10, 20};
  int present[3], n_present = 0;
  for (int k = 0; k < 3; ++k)
    if (ops[k]->present) present[n_present++] = k;
  if (n_present != 2) return kNotPair;
  auto has_u = [&](int k) { return ops[k]->u_stride != 0; };
  auto has_w = [&](int k) { return ops[k]->w_stride != 0; };
  int mode = -1, xk = -1, yk = -1;
  for (int swap = 0; swap < 2 && mode < 0; ++swap) {
    const int p = present[swap], q = present[1 - swap];
    if (a->out_has_u && a->out_has_w && has_u(p) && !has_w(p) && !has_u(q) && has_w(q) && ops[p]->u_stride == 1 &&
        ops[q]->w_stride == 1) {
      mode = kPairOuter; xk = p; yk = q;
    } else if (has_u(p) && has_w(p) && ops[p]->w_stride == 1 && ops[p]->u_stride == a->W) {
      if (a->out_has_u && !a->out_has_w && has_w(q) && !has_u(q) && ops[q]->w_stride == 1) {
        mode = kPairContractW; xk = p; yk = q;
      } else if (!a->out_has_u && a->out_has_w && has_u(q) && !has_w(q) && ops[q]->u_stride == 1) {
        mode = kPairContractU; xk = p; yk = q;
      }
    }
  }
  if (mode < 0) return kNotPair;
  const int wv = a->W / V;
  if (mode != kPairOuter && (wv & (wv - 1))) return kNotPair;        // lanes of one u are reduced by shuffles
  if (mode == kPairContractW && wv > kWave) return kNotPair;
  const uintptr_t bits = reinterpret_cast<uintptr_t>(ops[xk]->data) | reinterpret_cast<uintptr_t>(ops[yk]->data) |
                         reinterpret_cast<uintptr_t>(a->out);
  if ((bits & 15u) || ops[xk]->row_stride % V || ops[xk]->idx_stride % V || ops[yk]->row_stride % V ||
      ops[yk]->idx_stride % V)
    return kNotPair;
  PairDev<T> d;
  d.x = (const T*)ops[xk]->data; d.y = (const T*)ops[yk]->data;
  d.x_row = ops[xk]->row_stride; d.x_idx = ops[xk]->idx_stride;
  d.y_row = ops[yk]->row_stride; d.y_idx = ops[yk]->idx_stride;
  d.x_shift = shifts[xk]; d.y_shift = shifts[yk];
  d.x_mask = xk == 2 ? 4095u : 1023u; d.y_mask = yk == 2 ? 4095u : 1023u;
  d.coef = (const T*)a->coef; d.idx = a->idx; d.seg = a->seg; d.n_out = a->n_out; d.nnz = a->nnz;
  d.out = (T*)a->out; d.n_rows = a->n_rows; d.U = a->U; d.W = a->W;
  const int u_tile = 256 / wv;
  int64_t lds = (table_lds + 15) / 16 * 16;
  if (mode == kPairContractU) lds += (int64_t)u_tile * a->W * sizeof(T);
  if (lds > 48 * 1024 || 256 % wv) return kNotPair;
  auto kern = mode == kPairOuter ? gen_pair_kernel<T, V, kPairOuter>
                                 : mode == kPairContractW ? gen_pair_kernel<T, V, kPairContractW>
                                                          : gen_pair_kernel<T, V, kPairContractU>;
  hipLaunchKernelGGL(kern, dim3((unsigned)a->n_rows), dim3(256), (size_t)lds, stream, d);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

template <typename T>
static int gen_launch(const cgtp_gen_args* a, int64_t lds, hipStream_t stream) {
  const int64_t out_rows = a->reduce_rows ? 1 : a->n_rows;
  const int64_t blocks = out_rows * a->n_out;
  if (blocks == 0) return CGTP_OK;
  GenDev<T> d;
  d.a = gen_op<T>(a->a); d.b = gen_op<T>(a->b); d.w = gen_op<T>(a->w);
  d.coef = (const T*)a->coef; d.idx = a->idx; d.seg = a->seg; d.n_out = a->n_out; d.nnz = a->nnz;
  d.out = (T*)a->out; d.n_rows = a->n_rows; d.U = a->U; d.Wd = a->W;
  d.out_u = a->out_has_u; d.out_w = a->out_has_w; d.reduce_rows = a->reduce_rows;
  if (const int rc = gen_pair_launch<T>(a, lds, stream); rc != kNotPair) return rc;
  // enough rows to fill the chip: one workgroup per row; else (and for sums over rows) one per (row, output index)
  const bool by_row = !a->reduce_rows && a->n_rows >= 1024;
  auto kern = by_row ? gen_row_kernel<T> : gen_kernel<T>;
  if (lds > 48 * 1024 &&
      hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return CGTP_ERR_LDS;
  hipLaunchKernelGGL(kern, dim3((unsigned)(by_row ? a->n_rows : blocks)), dim3(256), (size_t)lds, stream, d);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

}  // namespace cgtp

using namespace cgtp;

extern "C" {

int cgtp_gen_validate(const cgtp_gen_args* args) {
  int64_t lds = 0;
  return gen_check(args, &lds);
}

int cgtp_gen_contract(const cgtp_gen_args* a, void* stream) {
  int64_t lds = 0;
  const int st = gen_check(a, &lds);
  if (st != CGTP_OK) return st;
  return a->dtype == CGTP_F32 ? gen_launch<float>(a, lds, (hipStream_t)stream)
                              : gen_launch<double>(a, lds, (hipStream_t)stream);
}

}  // extern "C"
