// Generic sparse trilinear contraction with the coefficient / index table staged in LDS, and the indexed
// scale-segment reduction.  These kernels take the tables at run time, so they serve every irreps
// configuration (and the reference's table-driven operator API); configurations with a compiled-in table
// use the kernels of uvu_kernels.hip instead.
#include <atomic>
#include <cstddef>
#include "cgtp_device.h"
#include "cgtp_host.h"

namespace cgtp {

template <typename T>
struct OperandDev {
  const T* data;
  const int64_t* rows;
  int64_t row_stride, idx_stride;
  int kind, size;
};

template <typename T>
struct TriDev {
  OperandDev<T> a, b, w;
  const T* coef;
  const uint32_t* idx;
  const int32_t* seg;
  int n_out, nnz;
  T* out;  // or the workspace when rows are reduced
  int64_t n_rows;
  int C, reduce_rows;
};

template <typename T>
__device__ __forceinline__ const T* row_ptr(const OperandDev<T>& o, int64_t r) {
  const int64_t rr = o.rows ? o.rows[r] : r;
  return o.data + rr * o.row_stride;
}

// One wavefront per row (or per contiguous share of the rows when they are reduced); lanes run over
// channels.  The table is read from LDS with wave-uniform addresses (broadcast reads).
template <typename T, bool REDUCE_C>
__global__ void __launch_bounds__(256) tri_kernel(const TriDev<T> a, int64_t n_waves) {
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

  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (wave >= n_waves) return;

  const int64_t per = a.reduce_rows ? (a.n_rows + n_waves - 1) / n_waves : 1;
  const int64_t stride = a.reduce_rows ? n_waves * per : n_waves;  // reduce_rows: a single pass
  // a wavefront of a row sum whose share is empty (wave * per >= n_rows) still writes its partial row, as zeros:
  // the second pass adds all n_waves partial rows
  for (int64_t r0 = wave * per; a.reduce_rows || r0 < a.n_rows; r0 += stride) {
    const int64_t r1 = (r0 + per < a.n_rows) ? r0 + per : a.n_rows;
    const int64_t orow = a.reduce_rows ? wave : r0;
    for (int o = 0; o < a.n_out; ++o) {
      const int tb = s_seg[o], te = s_seg[o + 1];
      T total = T(0);
      for (int cb = 0; cb < a.C; cb += kWave) {
        const int c = cb + lane;
        const bool ok = c < a.C;
        T acc = T(0);
        if (ok) {
          for (int64_t r = r0; r < r1; ++r) {
            const T* pa = a.a.kind ? row_ptr(a.a, r) + (a.a.kind == CGTP_OPERAND_VEC ? c : 0) : nullptr;
            const T* pb = a.b.kind ? row_ptr(a.b, r) + (a.b.kind == CGTP_OPERAND_VEC ? c : 0) : nullptr;
            const T* pw = a.w.kind ? row_ptr(a.w, r) + (a.w.kind == CGTP_OPERAND_VEC ? c : 0) : nullptr;
            for (int t = tb; t < te; ++t) {
              const uint32_t u = s_idx[t];
              T v = s_coef[t];
              if (pa) v *= pa[(int64_t)(u & 1023u) * a.a.idx_stride];
              if (pb) v *= pb[(int64_t)((u >> 10) & 1023u) * a.b.idx_stride];
              if (pw) v *= pw[(int64_t)(u >> 20) * a.w.idx_stride];
              acc += v;
            }
          }
        }
        if constexpr (REDUCE_C) {
          total += acc;
        } else {
          if (ok) a.out[(orow * a.n_out + o) * a.C + c] = acc;
        }
      }
      if constexpr (REDUCE_C) {
        total = group_sum(total, kWave);
        if (lane == 0) a.out[orow * a.n_out + o] = total;
      }
    }
    if (a.reduce_rows) break;
  }
}

// The same contraction with the operands of a row staged in LDS first (the caller states the extent of every
// operand's index axis): a wavefront copies the 64-channel slice of its row's operands into its own LDS region with
// coalesced loads, then walks the table reading operands from LDS at wave-uniform row offsets — no global loads,
// 64-bit address arithmetic or operand-kind branches per coefficient.  A per-channel operand occupies size x 64
// elements, a channel-less one size elements, an absent one a single 1.  Writes one result per row (a sum over rows
// is taken afterwards by the launcher).
template <typename T>
struct StagedOperand {
  int offset;   // first element of the operand inside the wavefront's region
  int stride;   // elements between sparse indices: 64 | 1 | 0
};

template <typename T, bool REDUCE_C>
__global__ void __launch_bounds__(256) tri_staged_kernel(const TriDev<T> a, int64_t n_waves, int region_elems) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* s_coef = reinterpret_cast<T*>(smem);
  uint32_t* s_idx = reinterpret_cast<uint32_t*>(s_coef + a.nnz);
  int32_t* s_seg = reinterpret_cast<int32_t*>(s_idx + a.nnz);
  const int table_elems = ((int)((a.nnz * (sizeof(T) + 4) + (a.n_out + 1) * 4 + 15) / 16)) * (16 / (int)sizeof(T));
  for (int t = threadIdx.x; t < a.nnz; t += blockDim.x) {
    s_coef[t] = a.coef ? a.coef[t] : T(1);
    s_idx[t] = a.idx[t];
  }
  for (int t = threadIdx.x; t <= a.n_out; t += blockDim.x) s_seg[t] = a.seg[t];
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (wave >= n_waves) return;
  T* region = reinterpret_cast<T*>(smem) + table_elems + (threadIdx.x / kWave) * region_elems;
  const OperandDev<T>* ops[3] = {&a.a, &a.b, &a.w};
  StagedOperand<T> so[3];
  int off = 0;
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    const int kind = ops[k]->kind;
    so[k].offset = off;
    so[k].stride = kind == CGTP_OPERAND_VEC ? kWave : (kind == CGTP_OPERAND_SCALAR ? 1 : 0);
    off += kind == CGTP_OPERAND_VEC ? ops[k]->size * kWave : (kind == CGTP_OPERAND_SCALAR ? ops[k]->size : 1);
  }
  // this lane's element of every operand: per-channel operands are read at [index * 64 + lane], the others at [index]
  const T* la = region + so[0].offset + (so[0].stride == kWave ? lane : 0);
  const T* lb = region + so[1].offset + (so[1].stride == kWave ? lane : 0);
  const T* lw = region + so[2].offset + (so[2].stride == kWave ? lane : 0);

  for (int64_t r = wave; r < a.n_rows; r += n_waves) {
    for (int cb = 0; cb < a.C; cb += kWave) {
      const int c = cb + lane;
      const bool ok = c < a.C;
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        const OperandDev<T>& o = *ops[k];
        T* dst = region + so[k].offset;
        if (o.kind == CGTP_OPERAND_VEC) {
          const T* src = row_ptr(o, r) + (ok ? c : 0);
          for (int i = 0; i < o.size; ++i) dst[i * kWave + lane] = ok ? src[(int64_t)i * o.idx_stride] : T(0);
        } else if (o.kind == CGTP_OPERAND_SCALAR) {
          if (cb == 0) {
            const T* src = row_ptr(o, r);
            for (int i = lane; i < o.size; i += kWave) dst[i] = src[(int64_t)i * o.idx_stride];
          }
        } else if (cb == 0 && lane == 0) {
          dst[0] = T(1);
        }
      }
      // LDS operations of one wavefront complete in order: the reads below see the writes above
      for (int o = 0; o < a.n_out; ++o) {
        const int tb = __builtin_amdgcn_readfirstlane(s_seg[o]), te = __builtin_amdgcn_readfirstlane(s_seg[o + 1]);
        T acc = T(0);
#pragma unroll 4
        for (int t = tb; t < te; ++t) {
          const uint32_t u = __builtin_amdgcn_readfirstlane(s_idx[t]);
          const int ia = (u & 1023u) * so[0].stride, ib = ((u >> 10) & 1023u) * so[1].stride, iw = (u >> 20) * so[2].stride;
          acc += s_coef[t] * la[ia] * lb[ib] * lw[iw];
        }
        if constexpr (REDUCE_C) {
          const T sum = group_sum(ok ? acc : T(0), kWave);
          // channel blocks of one output row are accumulated by lane 0 in the output itself
          if (lane == 0) {
            T* dst = a.out + r * a.n_out + o;
            *dst = cb == 0 ? sum : *dst + sum;
          }
        } else {
          if (ok) a.out[(r * a.n_out + o) * a.C + c] = acc;
        }
      }
    }
  }
}

// The same contraction for light tables (about one coefficient per operand row: gates, per-irrep scalings and
// block sums, rotations about z), where staging cannot pay and the row-by-row kernel above is bound by latency.
// A row takes LPR = next_pow2(C / V) lanes with V channels each (16-byte accesses), so a wavefront covers 64 / LPR
// rows at once; the coefficients are walked in table order four at a time, all operand loads of the four issued
// before any arithmetic, and a result row is stored when the output index changes (the indices are the same for
// every lane: scalar branches).  No reduction over rows; C / V <= 64.
template <typename T>
struct LightOperand {
  const T* p;        // this lane's row (+ channel for per-channel operands), or nullptr
  int64_t stride;    // elements between sparse indices
  bool vec;
};

template <typename T, int V>
__device__ __forceinline__ void light_fetch(const LightOperand<T>& o, uint32_t i, T (&dst)[V]) {
  if (!o.p) {
#pragma unroll
    for (int v = 0; v < V; ++v) dst[v] = T(1);
  } else if (o.vec) {
    load_vec<T, V>(dst, o.p + (int64_t)i * o.stride);
  } else {
    const T x = o.p[(int64_t)i * o.stride];
#pragma unroll
    for (int v = 0; v < V; ++v) dst[v] = x;
  }
}

template <typename T, int V, bool REDUCE_C>
__global__ void __launch_bounds__(256) tri_light_kernel(const TriDev<T> a, int lpr_log2) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int U = 2;   // coefficients in flight per lane: two measured best (65536 rows x 9 x 64 fp32: Gate forward 0.081 ms at four, 0.074 at two; eight halves the occupancy, one doubles the backward time)
  T* s_coef = reinterpret_cast<T*>(smem);
  uint32_t* s_idx = reinterpret_cast<uint32_t*>(s_coef + a.nnz);
  int32_t* s_out = reinterpret_cast<int32_t*>(s_idx + a.nnz);      // output index of every coefficient
  for (int t = threadIdx.x; t < a.nnz; t += blockDim.x) {
    s_coef[t] = a.coef ? a.coef[t] : T(1);
    s_idx[t] = a.idx[t];
  }
  for (int o = threadIdx.x; o < a.n_out; o += blockDim.x)
    for (int t = a.seg[o]; t < a.seg[o + 1]; ++t) s_out[t] = o;
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1);
  const int lpr = 1 << lpr_log2, slot = lane >> lpr_log2, sub = lane & (lpr - 1);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int64_t r = wave * (kWave >> lpr_log2) + slot;
  const int c = sub * V;
  const bool ok = r < a.n_rows && c < a.C;
  const int64_t rr = r < a.n_rows ? r : 0;       // idle lanes read row 0 and store nothing
  const int cc = c < a.C ? c : 0;
  LightOperand<T> ops[3];
  const OperandDev<T>* src[3] = {&a.a, &a.b, &a.w};
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    ops[k].vec = src[k]->kind == CGTP_OPERAND_VEC;
    ops[k].stride = src[k]->idx_stride;
    ops[k].p = src[k]->kind ? row_ptr(*src[k], rr) + (ops[k].vec ? cc : 0) : nullptr;
  }
  auto emit = [&](int o, const T (&acc)[V]) __attribute__((always_inline)) {
    if constexpr (REDUCE_C) {
      T sum = T(0);
#pragma unroll
      for (int v = 0; v < V; ++v) sum += acc[v];
      sum = group_sum(ok ? sum : T(0), lpr);
      if (ok && sub == 0) a.out[r * a.n_out + o] = sum;
    } else {
      if (ok) store_vec<T, V>(a.out + (r * a.n_out + o) * a.C + c, acc);
    }
  };
  T acc[V];
#pragma unroll
  for (int v = 0; v < V; ++v) acc[v] = T(0);
  int cur = 0;      // outputs before `cur` are written; rows without coefficients are written as zeros
  for (int t0 = 0; t0 < a.nnz; t0 += U) {
    T xa[U][V], xb[U][V], xw[U][V], cf[U];
    int oi[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const int t = min(t0 + k, a.nnz - 1);
      const uint32_t u = __builtin_amdgcn_readfirstlane(s_idx[t]);
      oi[k] = __builtin_amdgcn_readfirstlane(s_out[t]);
      cf[k] = s_coef[t];
      light_fetch<T, V>(ops[0], u & 1023u, xa[k]);
      light_fetch<T, V>(ops[1], (u >> 10) & 1023u, xb[k]);
      light_fetch<T, V>(ops[2], u >> 20, xw[k]);
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
      if (t0 + k < a.nnz) {
        while (cur < oi[k]) {
          emit(cur, acc);
#pragma unroll
          for (int v = 0; v < V; ++v) acc[v] = T(0);
          ++cur;
        }
#pragma unroll
        for (int v = 0; v < V; ++v) acc[v] += cf[k] * xa[k][v] * xb[k][v] * xw[k][v];
      }
    }
  }
  while (cur < a.n_out) {
    emit(cur, acc);
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = T(0);
    ++cur;
  }
}

// out[n, m, c] = sum_{t in [seg[m], seg[m+1])} scale[t] * in[n, index[t], c].  One wavefront per (n, m, chunk of
// 64 * V channels): wide rows are spread over several wavefronts, and the terms of a segment are fetched four at
// a time (indices and scales first, then the four rows; the last one to three singly) and added in position
// order, so the sum is the same whatever the launch shape.
template <typename T, int V>
__global__ void __launch_bounds__(256) segment_sum_kernel(const T* __restrict__ in, const T* __restrict__ scale,
                                                          const int64_t* __restrict__ index,
                                                          const int64_t* __restrict__ seg, T* __restrict__ out,
                                                          int64_t n_batch, int64_t in_size, int64_t out_size,
                                                          int64_t C, int chunks) {
  constexpr int U = 4;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (wave >= n_batch * out_size * chunks) return;
  const int64_t row = wave / chunks;
  const int64_t c = ((wave % chunks) * kWave + lane) * V;
  const int64_t n = row / out_size, m = row % out_size;
  const int64_t tb = seg ? seg[m] : m, te = seg ? seg[m + 1] : m + 1;
  const T* base = in + n * in_size * C + (c < C ? c : 0);
  const bool ok = c < C;
  T acc[V];
#pragma unroll
  for (int v = 0; v < V; ++v) acc[v] = T(0);
  // Terms four at a time.  The positions and scales of the next four are requested while the rows of these four are
  // on their way (a group then costs one round trip to memory, not two), and a last group of one to three terms
  // takes the same path with its missing terms pointed at the last one and left out of the sum.  Additions in
  // position order, whatever the launch shape.
  auto fetch = [&](int64_t t0, int64_t (&idx)[U], T (&sc)[U]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t t = t0 + u < te ? t0 + u : te - 1;
      idx[u] = index ? index[t] : t;
      sc[u] = scale ? scale[t] : T(1);
    }
  };
  int64_t idx[U];
  T sc[U];
  if (tb < te) fetch(tb, idx, sc);
  for (int64_t t0 = tb; t0 < te; t0 += U) {
    T x[U][V];
#pragma unroll
    for (int u = 0; u < U; ++u) load_vec<T, V>(x[u], base + idx[u] * C);
    T scn[U];
#pragma unroll
    for (int u = 0; u < U; ++u) scn[u] = sc[u];
    if (t0 + U < te) fetch(t0 + U, idx, sc);
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (t0 + u < te) fmav<T, V>(acc, scn[u], x[u]);     // the same in every lane
  }
  if (ok) store_vec<T, V>(out + (n * out_size + m) * C + c, acc);
}

static int64_t tri_table_bytes(const cgtp_tri_args* a) {
  return (int64_t)a->nnz * (elem_size(a->dtype) + 4) + ((int64_t)a->n_out + 1) * 4;
}

// LDS bytes of the staged kernel (table + four operand regions) and elements per region, or 0 if the operands'
// extents are unknown, the regions do not fit, or staging would not pay.
constexpr int64_t kLightReuse = 8;

static int64_t tri_staged_lds(const cgtp_tri_args* a, int64_t table_bytes, int64_t* region_elems) {
  const cgtp_operand* ops[3] = {&a->a, &a->b, &a->w};
  int64_t region = 0, vec_rows = 0;
  for (const cgtp_operand* o : ops) {
    if (o->kind != CGTP_OPERAND_NONE && o->size <= 0) return 0;
    region += o->kind == CGTP_OPERAND_VEC ? (int64_t)o->size * kWave : (o->kind == CGTP_OPERAND_SCALAR ? o->size : 1);
    if (o->kind == CGTP_OPERAND_VEC) vec_rows += o->size;
  }
  // staging pays when operand rows are read many times; with up to kLightReuse coefficients per staged row
  // (gates, block sums, rotations, SO(2) maps, the second stage of the reference's two-launch products) reading the
  // operands through the caches is faster
  if (a->nnz <= kLightReuse * vec_rows) return 0;
  region = (region + 3) / 4 * 4;
  const int64_t lds = (table_bytes + 15) / 16 * 16 + 4 * region * elem_size(a->dtype);
  if (lds > kLdsBytes) return 0;
  *region_elems = region;
  return lds;
}

static int tri_check(const cgtp_tri_args* a, int64_t* lds_bytes, int64_t* n_waves) {
  if (!a) return CGTP_ERR_NULL;
  if (a->dtype != CGTP_F32 && a->dtype != CGTP_F64) return CGTP_ERR_DTYPE;
  if (a->n_out < 0 || a->nnz < 0 || a->n_rows < 0 || a->C <= 0) return CGTP_ERR_SHAPE;
  if (!a->idx || !a->seg || !a->out) return CGTP_ERR_NULL;
  const cgtp_operand* ops[3] = {&a->a, &a->b, &a->w};
  for (const cgtp_operand* o : ops) {
    if (o->kind < CGTP_OPERAND_NONE || o->kind > CGTP_OPERAND_SCALAR) return CGTP_ERR_SHAPE;
    if (o->kind != CGTP_OPERAND_NONE && !o->data) return CGTP_ERR_NULL;
    if (o->kind != CGTP_OPERAND_NONE && (o->row_stride < 0 || o->idx_stride < 0)) return CGTP_ERR_SHAPE;
  }
  *lds_bytes = tri_table_bytes(a);
  if (*lds_bytes > kLdsBytes) return CGTP_ERR_LDS;
  if (a->reduce_rows) {
    int64_t nw = a->n_rows < 1024 ? a->n_rows : 1024;
    *n_waves = nw;
    if (nw > 0 && !a->workspace) return CGTP_ERR_WORKSPACE;
  } else {
    *n_waves = a->n_rows < 16384 ? a->n_rows : 16384;
  }
  return CGTP_OK;
}

template <typename T>
static OperandDev<T> op_dev(const cgtp_operand& o) {
  return OperandDev<T>{(const T*)o.data, o.rows, o.row_stride, o.idx_stride, o.kind, o.size};
}

// tri_light_kernel serves a launch when the shapes allow it: V channels per lane (16 bytes) if every per-channel
// operand and the output keep 16-byte alignment from row to row and index to index, else one; at most 64 lanes per
// row; table within the default LDS limit.  Returns V, or 0 when the kernel does not apply.
template <typename T, int V>
static bool light_aligned(const cgtp_tri_args* a, const void* out) {
  if (V == 1) return true;
  if (a->C % V) return false;
  const cgtp_operand* ops[3] = {&a->a, &a->b, &a->w};
  for (const cgtp_operand* o : ops)
    if (o->kind == CGTP_OPERAND_VEC &&
        ((reinterpret_cast<uintptr_t>(o->data) & (V * sizeof(T) - 1)) || o->row_stride % V || o->idx_stride % V))
      return false;
  return (reinterpret_cast<uintptr_t>(out) & (V * sizeof(T) - 1)) == 0;
}

template <typename T>
static int light_width(const cgtp_tri_args* a) {
  constexpr int VW = 16 / sizeof(T);
  if (a->n_out == 0 || a->n_rows == 0) return 0;
  if ((int64_t)a->nnz * (sizeof(T) + 8) > 48 * 1024) return 0;
  // rows summed afterwards go through the workspace (allocated 256-byte aligned by the caller's allocator; checked)
  const void* out = a->reduce_rows ? a->workspace : a->out;
  if (light_aligned<T, VW>(a, out) && a->C / VW <= kWave) return VW;
  return a->C <= kWave ? 1 : 0;
}

template <typename T, int V>
static int tri_light_launch_v(const cgtp_tri_args* a, const TriDev<T>& d, hipStream_t stream) {
  const int lanes = (a->C + V - 1) / V;
  int lpr_log2 = 0;
  while ((1 << lpr_log2) < lanes) ++lpr_log2;
  const int64_t lds = (int64_t)a->nnz * (sizeof(T) + 8);
  const int64_t rows_per_block = (int64_t)4 * (kWave >> lpr_log2);
  const int64_t blocks = (a->n_rows + rows_per_block - 1) / rows_per_block;
  if (blocks > 0x7fffffff) return CGTP_ERR_SHAPE;
  auto kern = a->reduce_c ? tri_light_kernel<T, V, true> : tri_light_kernel<T, V, false>;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), (size_t)lds, stream, d, lpr_log2);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

// Sum over rows of per-row results in the workspace: chunks of kSumRows rows, then the chunks, both in a fixed order.
template <typename T>
static int tri_sum_rows(const cgtp_tri_args* a, int64_t per_row, hipStream_t stream) {
  const int64_t chunks = (a->n_rows + kSumRows - 1) / kSumRows;
  T* part = (T*)a->workspace + a->n_rows * per_row;
  launch_rows_sum<T>((const T*)a->workspace, part, a->n_rows, per_row, stream);
  launch_partial_sum<T>((const T*)part, (T*)a->out, chunks, per_row, stream);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

template <typename T>
static int tri_launch(const cgtp_tri_args* a, int64_t lds, int64_t n_waves, hipStream_t stream) {
  const int64_t per_row = (int64_t)a->n_out * (a->reduce_c ? 1 : a->C);
  if (n_waves == 0) {
    if (a->reduce_rows && per_row > 0) launch_partial_sum<T>(nullptr, (T*)a->out, 0, per_row, stream);  // writes 0
    return CGTP_OK;
  }
  TriDev<T> d;
  d.a = op_dev<T>(a->a); d.b = op_dev<T>(a->b); d.w = op_dev<T>(a->w);
  d.coef = (const T*)a->coef; d.idx = a->idx; d.seg = a->seg;
  d.n_out = a->n_out; d.nnz = a->nnz;
  d.out = a->reduce_rows ? (T*)a->workspace : (T*)a->out;
  d.n_rows = a->n_rows; d.C = a->C; d.reduce_rows = a->reduce_rows;
  // operands staged in LDS when their extents are known and four regions fit next to the table; a sum over rows
  // then goes through per-row results in the workspace and two fixed-order passes
  int64_t region = 0;
  const int64_t staged_lds = tri_staged_lds(a, lds, &region);
  if (staged_lds > 0) {
    auto skern = a->reduce_c ? tri_staged_kernel<T, true> : tri_staged_kernel<T, false>;
    if (staged_lds > 48 * 1024 &&
        hipFuncSetAttribute((const void*)skern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)staged_lds) != hipSuccess)
      return CGTP_ERR_LDS;
    const int64_t nw = a->n_rows < 16384 ? a->n_rows : 16384;
    hipLaunchKernelGGL(skern, dim3((unsigned)((nw + 3) / 4)), dim3(256), (size_t)staged_lds, stream, d, nw, (int)region);
    if (hipGetLastError() != hipSuccess) return CGTP_ERR_LAUNCH;
    return a->reduce_rows ? tri_sum_rows<T>(a, per_row, stream) : CGTP_OK;
  }
  if (const int v = light_width<T>(a)) {
    constexpr int VW = 16 / sizeof(T);
    const int rc = v == 1 ? tri_light_launch_v<T, 1>(a, d, stream) : tri_light_launch_v<T, VW>(a, d, stream);
    if (rc != CGTP_OK) return rc;
    return a->reduce_rows ? tri_sum_rows<T>(a, per_row, stream) : CGTP_OK;
  }
  auto kern = a->reduce_c ? tri_kernel<T, true> : tri_kernel<T, false>;
  if (lds > 48 * 1024) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return CGTP_ERR_LDS;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)((n_waves + 3) / 4)), dim3(256), (size_t)lds, stream, d, n_waves);
  if (hipGetLastError() != hipSuccess) return CGTP_ERR_LAUNCH;
  if (a->reduce_rows) {
    launch_partial_sum<T>((const T*)a->workspace, (T*)a->out, n_waves, per_row, stream);
    if (hipGetLastError() != hipSuccess) return CGTP_ERR_LAUNCH;
  }
  return CGTP_OK;
}

template <typename T, int VW>
static int segsum_launch(const void* in, const void* scale, const int64_t* index, const int64_t* seg, void* out,
                         int64_t n_batch, int64_t in_size, int64_t out_size, int64_t C, hipStream_t stream) {
  if (n_batch * out_size == 0) return CGTP_OK;
  const bool vec = (C % VW) == 0 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  const int v = vec ? VW : 1;
  const int chunks = (int)((C + (int64_t)kWave * v - 1) / ((int64_t)kWave * v));
  const int64_t waves = n_batch * out_size * chunks;
  dim3 grid((unsigned)((waves + 3) / 4));
  if (vec)
    hipLaunchKernelGGL((segment_sum_kernel<T, VW>), grid, dim3(256), 0, stream, (const T*)in, (const T*)scale,
                       index, seg, (T*)out, n_batch, in_size, out_size, C, chunks);
  else
    hipLaunchKernelGGL((segment_sum_kernel<T, 1>), grid, dim3(256), 0, stream, (const T*)in, (const T*)scale,
                       index, seg, (T*)out, n_batch, in_size, out_size, C, chunks);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

}  // namespace cgtp

using namespace cgtp;

extern "C" {

const char* cgtp_status_string(int status) {
  switch (status) {
    case CGTP_OK: return "ok";
    case CGTP_ERR_NULL: return "required pointer is NULL";
    case CGTP_ERR_SHAPE: return "invalid or inconsistent extent";
    case CGTP_ERR_ALIGN: return "pointer or stride misaligned";
    case CGTP_ERR_DTYPE: return "unsupported element type";
    case CGTP_ERR_CONFIG: return "unknown specialised-table id";
    case CGTP_ERR_LDS: return "table does not fit in LDS";
    case CGTP_ERR_LAUNCH: return "kernel launch failed";
    case CGTP_ERR_WORKSPACE: return "workspace missing or too small";
    case CGTP_ERR_SCRATCH_LIMIT: return "partial results exceed the library's fixed scratch array";
    default: return "unknown status";
  }
}

int cgtp_version(void) { return 3; }

int cgtp_abi_layout(int which, int64_t* out, int capacity) {
#define CGTP_OFF(S, f) (int64_t) offsetof(S, f)
  static const int64_t operand[] = {sizeof(cgtp_operand), CGTP_OFF(cgtp_operand, data), CGTP_OFF(cgtp_operand, rows),
                                    CGTP_OFF(cgtp_operand, row_stride), CGTP_OFF(cgtp_operand, idx_stride),
                                    CGTP_OFF(cgtp_operand, kind), CGTP_OFF(cgtp_operand, size)};
  static const int64_t tri[] = {sizeof(cgtp_tri_args), CGTP_OFF(cgtp_tri_args, a), CGTP_OFF(cgtp_tri_args, b),
                                CGTP_OFF(cgtp_tri_args, w), CGTP_OFF(cgtp_tri_args, coef), CGTP_OFF(cgtp_tri_args, idx),
                                CGTP_OFF(cgtp_tri_args, seg), CGTP_OFF(cgtp_tri_args, n_out), CGTP_OFF(cgtp_tri_args, nnz),
                                CGTP_OFF(cgtp_tri_args, out), CGTP_OFF(cgtp_tri_args, workspace),
                                CGTP_OFF(cgtp_tri_args, n_rows), CGTP_OFF(cgtp_tri_args, C), CGTP_OFF(cgtp_tri_args, dtype),
                                CGTP_OFF(cgtp_tri_args, reduce_c), CGTP_OFF(cgtp_tri_args, reduce_rows)};
  static const int64_t gen_operand[] = {sizeof(cgtp_gen_operand), CGTP_OFF(cgtp_gen_operand, data),
                                        CGTP_OFF(cgtp_gen_operand, row_stride), CGTP_OFF(cgtp_gen_operand, idx_stride),
                                        CGTP_OFF(cgtp_gen_operand, u_stride), CGTP_OFF(cgtp_gen_operand, w_stride),
                                        CGTP_OFF(cgtp_gen_operand, present), CGTP_OFF(cgtp_gen_operand, _pad)};
  static const int64_t gen[] = {sizeof(cgtp_gen_args), CGTP_OFF(cgtp_gen_args, a), CGTP_OFF(cgtp_gen_args, b),
                                CGTP_OFF(cgtp_gen_args, w), CGTP_OFF(cgtp_gen_args, coef), CGTP_OFF(cgtp_gen_args, idx),
                                CGTP_OFF(cgtp_gen_args, seg), CGTP_OFF(cgtp_gen_args, n_out), CGTP_OFF(cgtp_gen_args, nnz),
                                CGTP_OFF(cgtp_gen_args, out), CGTP_OFF(cgtp_gen_args, n_rows), CGTP_OFF(cgtp_gen_args, U),
                                CGTP_OFF(cgtp_gen_args, W), CGTP_OFF(cgtp_gen_args, out_has_u),
                                CGTP_OFF(cgtp_gen_args, out_has_w), CGTP_OFF(cgtp_gen_args, reduce_rows),
                                CGTP_OFF(cgtp_gen_args, dtype)};
  static const int64_t uvu[] = {sizeof(cgtp_uvu_args), CGTP_OFF(cgtp_uvu_args, cfg), CGTP_OFF(cgtp_uvu_args, dtype),
                                CGTP_OFF(cgtp_uvu_args, C), CGTP_OFF(cgtp_uvu_args, w_shared),
                                CGTP_OFF(cgtp_uvu_args, n_rows), CGTP_OFF(cgtp_uvu_args, n_x_rows),
                                CGTP_OFF(cgtp_uvu_args, n_seg), CGTP_OFF(cgtp_uvu_args, ptr), CGTP_OFF(cgtp_uvu_args, perm),
                                CGTP_OFF(cgtp_uvu_args, seg_ids), CGTP_OFF(cgtp_uvu_args, gather),
                                CGTP_OFF(cgtp_uvu_args, pos_per_wave), CGTP_OFF(cgtp_uvu_args, y_vec),
                                CGTP_OFF(cgtp_uvu_args, wave_seg), CGTP_OFF(cgtp_uvu_args, n_waves),
                                CGTP_OFF(cgtp_uvu_args, x), CGTP_OFF(cgtp_uvu_args, y), CGTP_OFF(cgtp_uvu_args, w),
                                CGTP_OFF(cgtp_uvu_args, out), CGTP_OFF(cgtp_uvu_args, grad_out),
                                CGTP_OFF(cgtp_uvu_args, grad_x), CGTP_OFF(cgtp_uvu_args, grad_y),
                                CGTP_OFF(cgtp_uvu_args, grad_w), CGTP_OFF(cgtp_uvu_args, workspace),
                                CGTP_OFF(cgtp_uvu_args, x_gather), CGTP_OFF(cgtp_uvu_args, y_channels),
                                CGTP_OFF(cgtp_uvu_args, reserved_), CGTP_OFF(cgtp_uvu_args, path_scale),
                                CGTP_OFF(cgtp_uvu_args, radial_h), CGTP_OFF(cgtp_uvu_args, radial_w),
                                CGTP_OFF(cgtp_uvu_args, radial_r), CGTP_OFF(cgtp_uvu_args, reserved2_),
                                CGTP_OFF(cgtp_uvu_args, wave_pos)};
  static const int64_t uvt_item[] = {sizeof(cgtp_uvt_item), CGTP_OFF(cgtp_uvt_item, p), CGTP_OFF(cgtp_uvt_item, kb0),
                                     CGTP_OFF(cgtp_uvt_item, nkb), CGTP_OFF(cgtp_uvt_item, t0), CGTP_OFF(cgtp_uvt_item, t1),
                                     CGTP_OFF(cgtp_uvt_item, out_row), CGTP_OFF(cgtp_uvt_item, flags),
                                     CGTP_OFF(cgtp_uvt_item, reserved_)};
  static const int64_t uvt[] = {sizeof(cgtp_uvt_args), CGTP_OFF(cgtp_uvt_args, x), CGTP_OFF(cgtp_uvt_args, y),
                                CGTP_OFF(cgtp_uvt_args, wp), CGTP_OFF(cgtp_uvt_args, out), CGTP_OFF(cgtp_uvt_args, items),
                                CGTP_OFF(cgtp_uvt_args, term_a), CGTP_OFF(cgtp_uvt_args, term_b),
                                CGTP_OFF(cgtp_uvt_args, term_c), CGTP_OFF(cgtp_uvt_args, n_rows),
                                CGTP_OFF(cgtp_uvt_args, n_items), CGTP_OFF(cgtp_uvt_args, dx), CGTP_OFF(cgtp_uvt_args, dy),
                                CGTP_OFF(cgtp_uvt_args, dout), CGTP_OFF(cgtp_uvt_args, cx), CGTP_OFF(cgtp_uvt_args, cy),
                                CGTP_OFF(cgtp_uvt_args, cout), CGTP_OFF(cgtp_uvt_args, kbi), CGTP_OFF(cgtp_uvt_args, dtype),
                                CGTP_OFF(cgtp_uvt_args, n_terms), CGTP_OFF(cgtp_uvt_args, n_groups),
                                CGTP_OFF(cgtp_uvt_args, group_ptr)};
  static const int64_t uvt_gw[] = {sizeof(cgtp_uvt_gw_args), CGTP_OFF(cgtp_uvt_gw_args, x), CGTP_OFF(cgtp_uvt_gw_args, y),
                                   CGTP_OFF(cgtp_uvt_gw_args, g), CGTP_OFF(cgtp_uvt_gw_args, gw),
                                   CGTP_OFF(cgtp_uvt_gw_args, workspace), CGTP_OFF(cgtp_uvt_gw_args, items),
                                   CGTP_OFF(cgtp_uvt_gw_args, path_ptr), CGTP_OFF(cgtp_uvt_gw_args, term_a),
                                   CGTP_OFF(cgtp_uvt_gw_args, term_b), CGTP_OFF(cgtp_uvt_gw_args, term_c),
                                   CGTP_OFF(cgtp_uvt_gw_args, n_rows), CGTP_OFF(cgtp_uvt_gw_args, n_items),
                                   CGTP_OFF(cgtp_uvt_gw_args, n_terms), CGTP_OFF(cgtp_uvt_gw_args, n_paths),
                                   CGTP_OFF(cgtp_uvt_gw_args, dx), CGTP_OFF(cgtp_uvt_gw_args, dy),
                                   CGTP_OFF(cgtp_uvt_gw_args, dg), CGTP_OFF(cgtp_uvt_gw_args, cx),
                                   CGTP_OFF(cgtp_uvt_gw_args, cy), CGTP_OFF(cgtp_uvt_gw_args, cout),
                                   CGTP_OFF(cgtp_uvt_gw_args, dtype), CGTP_OFF(cgtp_uvt_gw_args, reserved_)};
  static const int64_t uvt_gy[] = {sizeof(cgtp_uvt_gy_args), CGTP_OFF(cgtp_uvt_gy_args, x), CGTP_OFF(cgtp_uvt_gy_args, g),
                                   CGTP_OFF(cgtp_uvt_gy_args, wp), CGTP_OFF(cgtp_uvt_gy_args, gy),
                                   CGTP_OFF(cgtp_uvt_gy_args, items), CGTP_OFF(cgtp_uvt_gy_args, term_m),
                                   CGTP_OFF(cgtp_uvt_gy_args, term_b), CGTP_OFF(cgtp_uvt_gy_args, term_c),
                                   CGTP_OFF(cgtp_uvt_gy_args, n_rows), CGTP_OFF(cgtp_uvt_gy_args, n_items),
                                   CGTP_OFF(cgtp_uvt_gy_args, n_terms), CGTP_OFF(cgtp_uvt_gy_args, dx),
                                   CGTP_OFF(cgtp_uvt_gy_args, dy), CGTP_OFF(cgtp_uvt_gy_args, dg),
                                   CGTP_OFF(cgtp_uvt_gy_args, cx), CGTP_OFF(cgtp_uvt_gy_args, cout),
                                   CGTP_OFF(cgtp_uvt_gy_args, dtype)};
  static const int64_t uvu_tab[] = {sizeof(cgtp_uvu_tab), CGTP_OFF(cgtp_uvu_tab, coef), CGTP_OFF(cgtp_uvu_tab, idx),
                                    CGTP_OFF(cgtp_uvu_tab, paths),
                                    CGTP_OFF(cgtp_uvu_tab, nnz), CGTP_OFF(cgtp_uvu_tab, n_segments),
                                    CGTP_OFF(cgtp_uvu_tab, D1), CGTP_OFF(cgtp_uvu_tab, D2),
                                    CGTP_OFF(cgtp_uvu_tab, DO), CGTP_OFF(cgtp_uvu_tab, P)};
  static const int64_t psw_table[] = {sizeof(cgtp_psw_table), CGTP_OFF(cgtp_psw_table, entries),
                                      CGTP_OFF(cgtp_psw_table, coef), CGTP_OFF(cgtp_psw_table, slots),
                                      CGTP_OFF(cgtp_psw_table, blocks), CGTP_OFF(cgtp_psw_table, n_entries),
                                      CGTP_OFF(cgtp_psw_table, n_slots), CGTP_OFF(cgtp_psw_table, n_blocks),
                                      CGTP_OFF(cgtp_psw_table, max_rows), CGTP_OFF(cgtp_psw_table, D1),
                                      CGTP_OFF(cgtp_psw_table, D2), CGTP_OFF(cgtp_psw_table, DO),
                                      CGTP_OFF(cgtp_psw_table, P)};
  static const int64_t psw_args[] = {sizeof(cgtp_psw_args), CGTP_OFF(cgtp_psw_args, x), CGTP_OFF(cgtp_psw_args, y),
                                     CGTP_OFF(cgtp_psw_args, w), CGTP_OFF(cgtp_psw_args, out),
                                     CGTP_OFF(cgtp_psw_args, g), CGTP_OFF(cgtp_psw_args, gx),
                                     CGTP_OFF(cgtp_psw_args, gy), CGTP_OFF(cgtp_psw_args, gw),
                                     CGTP_OFF(cgtp_psw_args, n_rows), CGTP_OFF(cgtp_psw_args, cx),
                                     CGTP_OFF(cgtp_psw_args, cy), CGTP_OFF(cgtp_psw_args, cout),
                                     CGTP_OFF(cgtp_psw_args, dtype)};
#undef CGTP_OFF
  const int64_t* tabs[] = {operand, tri, gen_operand, gen, uvu, uvt_item, uvt, uvt_gw, uvt_gy, uvu_tab, psw_table,
                           psw_args};
  const int counts[] = {(int)(sizeof(operand) / 8), (int)(sizeof(tri) / 8), (int)(sizeof(gen_operand) / 8),
                        (int)(sizeof(gen) / 8), (int)(sizeof(uvu) / 8), (int)(sizeof(uvt_item) / 8),
                        (int)(sizeof(uvt) / 8), (int)(sizeof(uvt_gw) / 8), (int)(sizeof(uvt_gy) / 8),
                        (int)(sizeof(uvu_tab) / 8), (int)(sizeof(psw_table) / 8), (int)(sizeof(psw_args) / 8)};
  if (which < 0 || which >= 12) return -1;
  for (int i = 0; out && i < counts[which] && i < capacity; ++i) out[i] = tabs[which][i];
  return counts[which];
}

int cgtp_tri_validate(const cgtp_tri_args* args) {
  int64_t lds = 0, nw = 0;
  cgtp_tri_args tmp;
  if (args) {
    tmp = *args;
    if (tmp.reduce_rows && !tmp.workspace) tmp.workspace = (void*)&tmp;  // size query / dry run
    return tri_check(&tmp, &lds, &nw);
  }
  return CGTP_ERR_NULL;
}

int64_t cgtp_tri_workspace_bytes(const cgtp_tri_args* a) {
  if (!a || !a->reduce_rows) return 0;
  const int64_t per_row = (int64_t)a->n_out * (a->reduce_c ? 1 : a->C);
  int64_t region = 0;
  // per-row results + first-pass partials when the staged or the light kernel serves the launch (the light kernel's
  // choice of vector width does not change the size; judge it with a workspace that is aligned)
  cgtp_tri_args probe = *a;
  probe.workspace = nullptr;
  const bool light = a->dtype == CGTP_F32 ? light_width<float>(&probe) > 0 : light_width<double>(&probe) > 0;
  if (tri_staged_lds(a, tri_table_bytes(a), &region) > 0 || light)
    return (a->n_rows + (a->n_rows + kSumRows - 1) / kSumRows) * per_row * elem_size(a->dtype);
  const int64_t nw = a->n_rows < 1024 ? a->n_rows : 1024;
  return nw * per_row * elem_size(a->dtype);
}

int cgtp_tri_contract(const cgtp_tri_args* a, void* stream) {
  int64_t lds = 0, nw = 0;
  const int st = tri_check(a, &lds, &nw);
  if (st != CGTP_OK) return st;
  return a->dtype == CGTP_F32 ? tri_launch<float>(a, lds, nw, (hipStream_t)stream)
                              : tri_launch<double>(a, lds, nw, (hipStream_t)stream);
}

// ---- the row-summing contraction for callers that cannot allocate ---------------------------------------------
// The partial rows of a sum over rows live in a fixed device array instead of a caller-provided workspace.  Every
// device that loads the library holds its own copy of the array at its own address; host code never uses the
// array's name as a pointer, only the address hipGetSymbolAddress reports for the current device.
constexpr int64_t kStaticScratchBytes = 16ll << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static std::atomic<void*> g_scratch_of_device[kMaxDevices];

static int static_scratch(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return CGTP_ERR_LAUNCH;
  void* p = g_scratch_of_device[dev].load(std::memory_order_acquire);
  if (!p) {
    // first call on this device: ask the runtime where this device's copy of the array lives (no allocation: the
    // array is part of the loaded code object).  Racing first calls obtain the same address.
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return CGTP_ERR_LAUNCH;
    g_scratch_of_device[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return CGTP_OK;
}

int64_t cgtp_tri_static_scratch_bytes(void) { return kStaticScratchBytes; }

int cgtp_tri_contract_static(const cgtp_tri_args* a, void* stream) {
  if (!a) return CGTP_ERR_NULL;
  cgtp_tri_args b = *a;
  b.workspace = nullptr;
  if (b.reduce_rows) {
    // validate with a placeholder first so that shape / dtype errors are reported as such
    cgtp_tri_args probe = b;
    probe.workspace = (void*)&probe;
    int64_t lds = 0, nw = 0;
    const int st = tri_check(&probe, &lds, &nw);
    if (st != CGTP_OK) return st;
    if (cgtp_tri_workspace_bytes(&b) > kStaticScratchBytes) return CGTP_ERR_SCRATCH_LIMIT;
    void* p = nullptr;
    const int rc = static_scratch(&p);
    if (rc != CGTP_OK) return rc;
    b.workspace = p;      // every partial row the second pass reads is written by the first: nothing to clear
  }
  return cgtp_tri_contract(&b, stream);
}

int cgtp_segment_sum(const void* in, const void* scale, const int64_t* index, const int64_t* seg, void* out,
                     int64_t n_batch, int64_t in_size, int64_t out_size, int64_t C, int32_t dtype, void* stream) {
  if (!in || !out) return CGTP_ERR_NULL;
  if (n_batch < 0 || in_size < 0 || out_size < 0 || C <= 0) return CGTP_ERR_SHAPE;
  if (dtype == CGTP_F32)
    return segsum_launch<float, 4>(in, scale, index, seg, out, n_batch, in_size, out_size, C, (hipStream_t)stream);
  if (dtype == CGTP_F64)
    return segsum_launch<double, 2>(in, scale, index, seg, out, n_batch, in_size, out_size, C, (hipStream_t)stream);
  return CGTP_ERR_DTYPE;
}

}  // extern "C"
