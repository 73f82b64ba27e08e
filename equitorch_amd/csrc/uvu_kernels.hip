// Channel-wise ("uvu") sparse Clebsch-Gordan tensor product with the table compiled into the kernel.
//
// Work decomposition (wave64): a wavefront is split into 64/LPE "slots" of LPE lanes; a lane owns V
// consecutive channels, so one slot covers LPE*V >= C channels of one row (edge) with V*sizeof(T)-byte
// coalesced accesses.  In row mode every slot owns one batch row.  In segment mode a wavefront owns one
// segment (destination node in the forward, source node in the backward) of a sorted edge list; its slots
// walk the segment's edges round-robin, accumulate in registers, and the slots are summed with cross-lane
// shuffles before a single store, so the edge -> node reduction needs no atomics and is deterministic.
#include "cgtp_device.h"
#include "cgtp_host.h"

namespace cgtp {
#include "generated/uvu_configs.inc"

template <typename T>
struct UvuDev {
  const T* x;
  const T* y;
  const T* w;
  T* out;
  const T* g;
  T* gx;
  T* gy;
  T* gw;
  T* ws;
  const int64_t* ptr;
  const int64_t* perm;
  const int64_t* gather;
  int64_t n_rows, n_seg;
  int C, lpe_log2, w_shared;
};

template <class TP, typename T, int V, bool SEG>
__global__ void __launch_bounds__(256) uvu_fwd_kernel(const UvuDev<T> a) {
  constexpr int D1 = TP::D1, D2 = TP::D2, DO = TP::DO, P = TP::P;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int lpe = 1 << a.lpe_log2, slots = kWave >> a.lpe_log2;
  const int slot = lane >> a.lpe_log2, cl = lane & (lpe - 1);
  const int c0 = (blockIdx.y * lpe + cl) * V;
  const bool cok = c0 < a.C;
  const int64_t C = a.C;

  T w[P][V];
  if (a.w_shared && cok) {
#pragma unroll
    for (int p = 0; p < P; ++p) load_vec<T, V>(w[p], a.w + p * C + c0);
  }
  T acc[DO][V];
#pragma unroll
  for (int m = 0; m < DO; ++m)
#pragma unroll
    for (int v = 0; v < V; ++v) acc[m][v] = T(0);

  auto one_row = [&](int64_t e, int64_t xr) {
    T x[D1][V], y[D2];
#pragma unroll
    for (int j = 0; j < D2; ++j) y[j] = a.y[e * D2 + j];
    if (cok) {
#pragma unroll
      for (int i = 0; i < D1; ++i) load_vec<T, V>(x[i], a.x + (xr * D1 + i) * C + c0);
      if (!a.w_shared) {
#pragma unroll
        for (int p = 0; p < P; ++p) load_vec_stream<T, V>(w[p], a.w + (e * P + p) * C + c0);
      }
      TP::template fwd<T, V>(x, y, w, acc);
    }
  };

  if constexpr (SEG) {
    if (wave >= a.n_seg) return;
    const int64_t beg = a.ptr[wave], end = a.ptr[wave + 1];
    for (int64_t pos = beg + slot; pos < end; pos += slots) {
      const int64_t e = a.perm ? a.perm[pos] : pos;
      one_row(e, a.gather ? a.gather[e] : e);
    }
#pragma unroll
    for (int m = 0; m < DO; ++m)
#pragma unroll
      for (int v = 0; v < V; ++v) acc[m][v] = cross_group_sum(acc[m][v], lpe);
    if (slot == 0 && cok) {
#pragma unroll
      for (int m = 0; m < DO; ++m) store_vec<T, V>(a.out + (wave * DO + m) * C + c0, acc[m]);
    }
  } else {
    const int64_t r = wave * slots + slot;
    if (r < a.n_rows) {
      one_row(r, a.gather ? a.gather[r] : r);
      if (cok) {
#pragma unroll
        for (int m = 0; m < DO; ++m) store_vec_stream<T, V>(a.out + (r * DO + m) * C + c0, acc[m]);
      }
    }
  }
}

// Backward.  WRED: the weight is shared over rows, so its gradient is summed over every row a wavefront
// visits and written as one partial per wavefront into the workspace (partial_sum_kernel finishes the sum).
template <class TP, typename T, int V, bool SEG, bool WRED>
__global__ void __launch_bounds__(256) uvu_bwd_kernel(const UvuDev<T> a, int64_t n_waves) {
  constexpr int D1 = TP::D1, D2 = TP::D2, DO = TP::DO, P = TP::P;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int lpe = 1 << a.lpe_log2, slots = kWave >> a.lpe_log2;
  const int slot = lane >> a.lpe_log2, cl = lane & (lpe - 1);
  const int c0 = cl * V;
  const bool cok = c0 < a.C;
  const int64_t C = a.C;
  if (wave >= n_waves) return;

  T w[P][V], x[D1][V], gx[D1][V], gw[P][V];
  if (a.w_shared && cok) {
#pragma unroll
    for (int p = 0; p < P; ++p) load_vec<T, V>(w[p], a.w + p * C + c0);
  }
  auto zero_gx = [&]() {
#pragma unroll
    for (int i = 0; i < D1; ++i)
#pragma unroll
      for (int v = 0; v < V; ++v) gx[i][v] = T(0);
  };
  auto zero_gw = [&]() {
#pragma unroll
    for (int p = 0; p < P; ++p)
#pragma unroll
      for (int v = 0; v < V; ++v) gw[p][v] = T(0);
  };
  zero_gx();
  zero_gw();

  // one edge / row: e = row of y, w, gy, gw; gr = row of grad_out; x already in registers
  auto one_row = [&](int64_t e, int64_t gr) {
    T g[DO][V], y[D2], gy[D2];
#pragma unroll
    for (int j = 0; j < D2; ++j) {
      y[j] = a.y[e * D2 + j];
      gy[j] = T(0);
    }
    if (cok) {
#pragma unroll
      for (int m = 0; m < DO; ++m) load_vec<T, V>(g[m], a.g + (gr * DO + m) * C + c0);
      if (!a.w_shared) {
#pragma unroll
        for (int p = 0; p < P; ++p) load_vec_stream<T, V>(w[p], a.w + (e * P + p) * C + c0);
      }
      if constexpr (!WRED) zero_gw();
      TP::template bwd<T, V>(x, y, w, g, gx, gy, gw);
      if constexpr (!WRED) {
        if (a.gw) {
#pragma unroll
          for (int p = 0; p < P; ++p) store_vec_stream<T, V>(a.gw + (e * P + p) * C + c0, gw[p]);
        }
      }
    }
    if (a.gy) {
#pragma unroll
      for (int j = 0; j < D2; ++j) {
        const T s = group_sum(gy[j], lpe);
        if (cl == (j & (lpe - 1))) a.gy[e * D2 + j] = s;
      }
    }
  };

  if constexpr (SEG) {
    if (cok) {
#pragma unroll
      for (int i = 0; i < D1; ++i) load_vec<T, V>(x[i], a.x + (wave * D1 + i) * C + c0);
    }
    const int64_t beg = a.ptr[wave], end = a.ptr[wave + 1];
    for (int64_t pos = beg + slot; pos < end; pos += slots) {
      const int64_t e = a.perm ? a.perm[pos] : pos;
      one_row(e, a.gather ? a.gather[e] : e);
    }
    if (a.gx) {
#pragma unroll
      for (int i = 0; i < D1; ++i)
#pragma unroll
        for (int v = 0; v < V; ++v) gx[i][v] = cross_group_sum(gx[i][v], lpe);
      if (slot == 0 && cok) {
#pragma unroll
        for (int i = 0; i < D1; ++i) store_vec<T, V>(a.gx + (wave * D1 + i) * C + c0, gx[i]);
      }
    }
  } else {
    for (int64_t r = wave * slots + slot; r < a.n_rows; r += n_waves * slots) {
      if (cok) {
#pragma unroll
        for (int i = 0; i < D1; ++i) load_vec<T, V>(x[i], a.x + (r * D1 + i) * C + c0);
      }
      zero_gx();
      one_row(r, a.gather ? a.gather[r] : r);
      if (a.gx && cok) {
#pragma unroll
        for (int i = 0; i < D1; ++i) store_vec_stream<T, V>(a.gx + (r * D1 + i) * C + c0, gx[i]);
      }
    }
  }
  if constexpr (WRED) {
#pragma unroll
    for (int p = 0; p < P; ++p)
#pragma unroll
      for (int v = 0; v < V; ++v) gw[p][v] = cross_group_sum(gw[p][v], lpe);
    if (slot == 0 && cok) {
#pragma unroll
      for (int p = 0; p < P; ++p) store_vec<T, V>(a.ws + (wave * P + p) * C + c0, gw[p]);
    }
  }
}

// ---- host side ----------------------------------------------------------------------------------------------
struct UvuPlan {
  int V, lpe_log2;
  int64_t n_waves;  // backward: wavefronts launched (== partial count when the weight gradient is reduced)
};

template <typename T>
using FwdFn = void (*)(const UvuDev<T>);
template <typename T>
using BwdFn = void (*)(const UvuDev<T>, int64_t);

template <typename T>
struct UvuEntry {
  uint64_t fingerprint;
  int dims[5];
  const char* name;
  FwdFn<T> fwd[2][2];     // [vector path][SEG]
  BwdFn<T> bwd[2][2][2];  // [vector path][SEG][WRED]
};

template <typename T>
struct VecWidth;
template <> struct VecWidth<float> { static constexpr int value = 4; };
template <> struct VecWidth<double> { static constexpr int value = 2; };

template <class TP, typename T>
static UvuEntry<T> make_entry() {
  constexpr int VW = VecWidth<T>::value;
  UvuEntry<T> e;
  e.fingerprint = TP::FINGERPRINT;
  e.dims[0] = TP::D1; e.dims[1] = TP::D2; e.dims[2] = TP::DO; e.dims[3] = TP::P; e.dims[4] = TP::NNZ;
  e.name = TP::NAME;
  e.fwd[0][0] = uvu_fwd_kernel<TP, T, 1, false>;
  e.fwd[0][1] = uvu_fwd_kernel<TP, T, 1, true>;
  e.fwd[1][0] = uvu_fwd_kernel<TP, T, VW, false>;
  e.fwd[1][1] = uvu_fwd_kernel<TP, T, VW, true>;
  e.bwd[0][0][0] = uvu_bwd_kernel<TP, T, 1, false, false>;
  e.bwd[0][0][1] = uvu_bwd_kernel<TP, T, 1, false, true>;
  e.bwd[0][1][0] = uvu_bwd_kernel<TP, T, 1, true, false>;
  e.bwd[0][1][1] = uvu_bwd_kernel<TP, T, 1, true, true>;
  e.bwd[1][0][0] = uvu_bwd_kernel<TP, T, VW, false, false>;
  e.bwd[1][0][1] = uvu_bwd_kernel<TP, T, VW, false, true>;
  e.bwd[1][1][0] = uvu_bwd_kernel<TP, T, VW, true, false>;
  e.bwd[1][1][1] = uvu_bwd_kernel<TP, T, VW, true, true>;
  return e;
}

template <typename T>
static const UvuEntry<T>* entries(int* count) {
#define CGTP_X(TP) make_entry<TP, T>(),
  static const UvuEntry<T> table[] = {CGTP_FOREACH_UVU_CONFIG(CGTP_X)};
#undef CGTP_X
  *count = (int)(sizeof(table) / sizeof(table[0]));
  return table;
}

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static constexpr int64_t kMaxRowWaves = 2048;

static int uvu_plan(const cgtp_uvu_args* a, int backward, UvuPlan* plan) {
  if (!a) return CGTP_ERR_NULL;
  int n_cfg = 0;
  entries<float>(&n_cfg);
  if (a->cfg < 0 || a->cfg >= n_cfg) return CGTP_ERR_CONFIG;
  if (a->dtype != CGTP_F32 && a->dtype != CGTP_F64) return CGTP_ERR_DTYPE;
  if (a->C <= 0 || a->n_rows < 0 || a->n_seg < 0 || a->n_x_rows < 0) return CGTP_ERR_SHAPE;
  if (!a->x || !a->y || !a->w) return CGTP_ERR_NULL;
  if (a->n_seg > 0 && !a->ptr) return CGTP_ERR_NULL;
  if (a->n_seg == 0 && (a->ptr || a->perm)) return CGTP_ERR_SHAPE;
  if (backward) {
    if (!a->grad_out) return CGTP_ERR_NULL;
    if (a->n_seg > 0 && a->n_x_rows != a->n_seg) return CGTP_ERR_SHAPE;
    if (a->n_seg == 0 && a->n_x_rows != a->n_rows) return CGTP_ERR_SHAPE;
  } else {
    if (!a->out) return CGTP_ERR_NULL;
    if (!a->gather && a->n_x_rows != a->n_rows) return CGTP_ERR_SHAPE;
  }
  const int vw = a->dtype == CGTP_F32 ? 4 : 2;
  bool vec = (a->C % vw) == 0 && aligned16(a->x) && aligned16(a->w);
  if (backward) {
    vec = vec && aligned16(a->grad_out) && (!a->grad_x || aligned16(a->grad_x)) &&
          (!a->grad_w || aligned16(a->grad_w)) && (!a->workspace || aligned16(a->workspace));
  } else {
    vec = vec && aligned16(a->out);
  }
  plan->V = vec ? vw : 1;
  const int lanes = (a->C + plan->V - 1) / plan->V;
  int lg = 0;
  while ((1 << lg) < lanes && lg < 6) ++lg;
  plan->lpe_log2 = lg;
  if (backward && lanes > kWave) return CGTP_ERR_SHAPE;  // channel reduction of grad_y stays inside one slot
  const int slots = kWave >> lg;
  if (a->n_seg > 0) {
    plan->n_waves = a->n_seg;
  } else {
    int64_t nw = (a->n_rows + slots - 1) / slots;
    if (backward && a->w_shared && a->grad_w && nw > kMaxRowWaves) nw = kMaxRowWaves;
    plan->n_waves = nw;
  }
  if (backward && a->w_shared && a->grad_w && !a->workspace && plan->n_waves > 0) return CGTP_ERR_WORKSPACE;
  return CGTP_OK;
}

template <typename T>
static UvuDev<T> to_dev(const cgtp_uvu_args* a, const UvuPlan& plan) {
  UvuDev<T> d;
  d.x = (const T*)a->x; d.y = (const T*)a->y; d.w = (const T*)a->w; d.out = (T*)a->out;
  d.g = (const T*)a->grad_out; d.gx = (T*)a->grad_x; d.gy = (T*)a->grad_y; d.gw = (T*)a->grad_w;
  d.ws = (T*)a->workspace;
  d.ptr = a->ptr; d.perm = a->perm; d.gather = a->gather;
  d.n_rows = a->n_rows; d.n_seg = a->n_seg;
  d.C = a->C; d.lpe_log2 = plan.lpe_log2; d.w_shared = a->w_shared;
  return d;
}

template <typename T>
static int launch_fwd(const cgtp_uvu_args* a, const UvuPlan& plan, hipStream_t stream) {
  int n = 0;
  const UvuEntry<T>& e = entries<T>(&n)[a->cfg];
  const bool seg = a->n_seg > 0;
  const int slots = kWave >> plan.lpe_log2;
  const int64_t waves = seg ? a->n_seg : (a->n_rows + slots - 1) / slots;
  if (waves == 0) return CGTP_OK;
  const int chunk = (1 << plan.lpe_log2) * plan.V;
  dim3 grid((unsigned)((waves + 3) / 4), (unsigned)((a->C + chunk - 1) / chunk));
  hipLaunchKernelGGL(e.fwd[plan.V > 1][seg], grid, dim3(256), 0, stream, to_dev<T>(a, plan));
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

template <typename T>
static int launch_bwd(const cgtp_uvu_args* a, const UvuPlan& plan, hipStream_t stream) {
  int n = 0;
  const UvuEntry<T>& e = entries<T>(&n)[a->cfg];
  const bool seg = a->n_seg > 0;
  const bool wred = a->w_shared && a->grad_w;
  if (plan.n_waves == 0) {
    if (wred) (void)hipMemsetAsync(a->grad_w, 0, sizeof(T) * e.dims[3] * a->C, stream);
    return CGTP_OK;
  }
  dim3 grid((unsigned)((plan.n_waves + 3) / 4));
  hipLaunchKernelGGL(e.bwd[plan.V > 1][seg][wred], grid, dim3(256), 0, stream, to_dev<T>(a, plan),
                     plan.n_waves);
  if (hipGetLastError() != hipSuccess) return CGTP_ERR_LAUNCH;
  if (wred) {
    const int64_t nel = (int64_t)e.dims[3] * a->C;
    hipLaunchKernelGGL(partial_sum_kernel<T>, dim3((unsigned)((nel + 255) / 256)), dim3(256), 0, stream,
                       (const T*)a->workspace, (T*)a->grad_w, plan.n_waves, nel);
    if (hipGetLastError() != hipSuccess) return CGTP_ERR_LAUNCH;
  }
  return CGTP_OK;
}

}  // namespace cgtp

using namespace cgtp;

extern "C" {

int cgtp_uvu_num_configs(void) {
  int n = 0;
  entries<float>(&n);
  return n;
}

int cgtp_uvu_find(uint64_t fingerprint) {
  int n = 0;
  const UvuEntry<float>* t = entries<float>(&n);
  for (int i = 0; i < n; ++i)
    if (t[i].fingerprint == fingerprint) return i;
  return -1;
}

uint64_t cgtp_uvu_describe(int cfg, int32_t* dims) {
  int n = 0;
  const UvuEntry<float>* t = entries<float>(&n);
  if (cfg < 0 || cfg >= n) return 0;
  if (dims)
    for (int i = 0; i < 5; ++i) dims[i] = t[cfg].dims[i];
  return t[cfg].fingerprint;
}

int cgtp_uvu_validate(const cgtp_uvu_args* args, int backward) {
  UvuPlan plan;
  return uvu_plan(args, backward, &plan);
}

int64_t cgtp_uvu_bwd_workspace_bytes(const cgtp_uvu_args* a) {
  if (!a || !(a->w_shared && a->grad_w)) return 0;
  cgtp_uvu_args tmp = *a;
  static char dummy[16] __attribute__((aligned(16)));
  if (!tmp.workspace) tmp.workspace = dummy;
  UvuPlan plan;
  if (uvu_plan(&tmp, 1, &plan) != CGTP_OK) return 0;
  int32_t dims[5];
  cgtp_uvu_describe(a->cfg, dims);
  const int64_t esz = a->dtype == CGTP_F32 ? 4 : 8;
  return plan.n_waves * dims[3] * (int64_t)a->C * esz;
}

int cgtp_uvu_fwd(const cgtp_uvu_args* a, void* stream) {
  UvuPlan plan;
  const int st = uvu_plan(a, 0, &plan);
  if (st != CGTP_OK) return st;
  return a->dtype == CGTP_F32 ? launch_fwd<float>(a, plan, (hipStream_t)stream)
                              : launch_fwd<double>(a, plan, (hipStream_t)stream);
}

int cgtp_uvu_bwd(const cgtp_uvu_args* a, void* stream) {
  UvuPlan plan;
  const int st = uvu_plan(a, 1, &plan);
  if (st != CGTP_OK) return st;
  return a->dtype == CGTP_F32 ? launch_bwd<float>(a, plan, (hipStream_t)stream)
                              : launch_bwd<double>(a, plan, (hipStream_t)stream);
}

}  // extern "C"
