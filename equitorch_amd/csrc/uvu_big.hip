// Channel-wise ("uvu") tensor product for configurations with very large tables (lmax = 6: 106 weight paths, 6460
// coefficients): fp32, one batch row per group of lanes, one channel per lane.  The arithmetic (about two vector
// instructions per coefficient and channel) dominates the memory traffic here, so the kernels keep only what the
// generated bodies need in registers: the input rows x and y, a ring of weight values fetched a few paths ahead,
// and the 2l+1 output (or output-gradient) rows of the irrep being worked on.
#include "uvu_common.h"

namespace cgtp {
#include "generated/uvu_big_configs.inc"

// Lanes past the batch or the channel count re-read the last valid element and store nothing, so that every lane
// runs the same code and the channel sum of grad_y can use full-width shuffles.
// YC: the second operand carries channels, y (n_rows, D2, C); one value per lane like x.
template <class TP, bool PS, bool YC = false>
__global__ void __launch_bounds__(256, 2) uvu_big_fwd_kernel(const UvuDev<float> a) {
  constexpr int D1 = TP::D1, D2 = TP::D2, DO = TP::DO, P = TP::P;
  const Lanes L(a.lpe_log2);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int64_t C = a.C;
  const int c_raw = blockIdx.y * L.lpe + L.cl;
  const int64_t r_raw = wave * L.slots + L.slot;
  const bool live = r_raw < a.n_rows && c_raw < a.C;
  const int64_t r = min(r_raw, a.n_rows - 1);
  const int c = min(c_raw, a.C - 1);
  const int64_t xr = a.gather ? a.gather[r] : r;
  float x[D1], y[D2];
#pragma unroll
  for (int j = 0; j < D2; ++j) y[j] = YC ? a.y[(r * D2 + j) * C + c] : a.y[r * D2 + j];
#pragma unroll
  for (int i = 0; i < D1; ++i) x[i] = a.x[(xr * D1 + i) * C + c];
  const float* wrow = a.w + (a.w_shared ? 0 : r) * P * C + c;
  float* orow = a.out + r * DO * C + c;
  const float* __restrict__ ps = a.ps;
  TP::fwd(
      x, y,
      [&](int p) __attribute__((always_inline)) {
        const float w = __builtin_nontemporal_load(wrow + p * C);
        if constexpr (PS) return w * ps[p]; else return w;
      },
      [&](int m, float v) __attribute__((always_inline)) {
        if (live) __builtin_nontemporal_store(v, orow + m * C);
      });
}

template <class TP, int GW, bool PS, bool YC = false>
__global__ void __launch_bounds__(256, 2) uvu_big_bwd_kernel(const UvuDev<float> a, int64_t n_waves) {
  constexpr int D1 = TP::D1, D2 = TP::D2, DO = TP::DO, P = TP::P;
  const Lanes L(a.lpe_log2);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (wave >= n_waves) return;
  const int64_t C = a.C;
  const int64_t r_raw = wave * L.slots + L.slot;
  const int c_raw = blockIdx.y * L.lpe + L.cl;  // rows wider than one wavefront: one channel chunk per blockIdx.y
  const bool row_ok = r_raw < a.n_rows, live = row_ok && c_raw < a.C;
  const int64_t r = min(r_raw, a.n_rows - 1);
  const int c = min(c_raw, a.C - 1);
  const int64_t gr = a.gather ? a.gather[r] : r;
  const int64_t xr = a.x_gather ? a.x_gather[r] : r;
  float y[D2], gy[D2], g[DO];
#pragma unroll
  for (int j = 0; j < D2; ++j) {
    y[j] = YC ? a.y[(r * D2 + j) * C + c] : a.y[r * D2 + j];
    gy[j] = 0.f;
  }
  const float* grow = a.g + gr * DO * C + c;
#pragma unroll
  for (int m = 0; m < DO; ++m) g[m] = grow[m * C];
  const float* xrow = a.x + xr * D1 * C + c;
  const float* wrow = a.w + (a.w_shared ? 0 : r) * P * C + c;
  float* gwrow = a.gw + r * P * C + c;
  float* gxrow = a.gx + r * D1 * C + c;
  const bool gx_live = a.gx && live;
  const float* __restrict__ ps = a.ps;
  TP::bwd(
      [&](int i) __attribute__((always_inline)) { return xrow[i * C]; }, y,
      [&](int p) __attribute__((always_inline)) {
        const float w = __builtin_nontemporal_load(wrow + p * C);
        if constexpr (PS) return w * ps[p]; else return w;
      },
      g,
      [&](int i, float v) __attribute__((always_inline)) {
        if (gx_live) __builtin_nontemporal_store(v, gxrow + i * C);
      },
      gy,
      [&](int p, float v) __attribute__((always_inline)) {
        if constexpr (GW == kGwStore) {
          if (live) __builtin_nontemporal_store(PS ? v * ps[p] : v, gwrow + p * C);
        }
      });
  if (YC) {
    if (a.gy && live) {
#pragma unroll
      for (int j = 0; j < D2; ++j) __builtin_nontemporal_store(gy[j], a.gy + (r * D2 + j) * C + c);
    }
  } else if (a.gy) {
    const float keep = c_raw < a.C ? 1.f : 0.f;  // duplicate channels of the padding lanes do not count
    // several channel chunks: each writes its partial sums to the workspace, the host sums them in chunk order
    float* gyrow = (gridDim.y > 1 ? a.ws + (int64_t)blockIdx.y * a.n_rows * D2 : a.gy) + r * D2;
#pragma unroll
    for (int j = 0; j < D2; ++j) {
      const float s = group_sum(gy[j] * keep, L.lpe);
      if (row_ok && L.cl == (j & (L.lpe - 1))) gyrow[j] = s;
    }
  }
}

template <class TP, bool PS>
static UvuBigEntry make_big_entry() {
  UvuBigEntry e;
  e.fingerprint = TP::FINGERPRINT;
  e.fingerprint_rounded[0] = TP::FINGERPRINT_BF16; e.fingerprint_rounded[1] = TP::FINGERPRINT_F16;
  e.dims[0] = TP::D1; e.dims[1] = TP::D2; e.dims[2] = TP::DO; e.dims[3] = TP::P; e.dims[4] = TP::NNZ;
  e.name = TP::NAME;
  e.coef = TP::COEF; e.idx = TP::IDX;
  e.fwd = uvu_big_fwd_kernel<TP, PS>;
  e.bwd[kGwNone] = uvu_big_bwd_kernel<TP, kGwNone, PS>;
  e.bwd[kGwStore] = uvu_big_bwd_kernel<TP, kGwStore, PS>;
  e.fwd_yc = uvu_big_fwd_kernel<TP, PS, true>;
  e.bwd_yc[kGwNone] = uvu_big_bwd_kernel<TP, kGwNone, PS, true>;
  e.bwd_yc[kGwStore] = uvu_big_bwd_kernel<TP, kGwStore, PS, true>;
  return e;
}

// Two sets, as for the register-resident kernels: uvu_big_ps.hip includes this file with CGTP_UVU_PS_UNIT defined and
// provides the set that applies one factor per weight path.
#ifdef CGTP_UVU_PS_UNIT
const UvuBigEntry* uvu_big_entries_scaled(int* count) {
#define CGTP_X(TP) make_big_entry<TP, true>(),
#else
const UvuBigEntry* uvu_big_entries(int* count) {
#define CGTP_X(TP) make_big_entry<TP, false>(),
#endif
  static const UvuBigEntry table[] = {CGTP_FOREACH_UVU_BIG_CONFIG(CGTP_X)};
#undef CGTP_X
  *count = (int)(sizeof(table) / sizeof(table[0]));
  return table;
}

}  // namespace cgtp
