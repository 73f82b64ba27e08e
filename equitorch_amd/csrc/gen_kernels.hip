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
  auto kern = gen_kernel<T>;
  if (lds > 48 * 1024 &&
      hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return CGTP_ERR_LDS;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), (size_t)lds, stream, d);
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
