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
    for (int j = 0; j < D2; ++j) gy[j] *= keep;
    group_sum_scatter<float, D2>(gy, L.lpe, [&](const auto& s) {   // lane cl ends up with components cl, cl + lpe, ...
#pragma unroll
      for (int i = 0; i < array_len(s); ++i) {
        const int j = i * L.lpe + L.cl;
        if (row_ok && j < D2) gyrow[j] = s[i];
      }
    });
  }
}

// ---- segment mode: gather, product and segment sum in one launch ------------------------------------------------
// The sorted edge list is cut into ranges of `per_range` consecutive positions, one range per slot (group of lanes
// that handles one edge).  A slot walks its range one position at a time and adds the finished rows of every edge to
// an accumulator row in LDS (rows x 64 floats per wavefront, lane-private columns: no conflicts; plain read-add-write,
// which measured 15 % faster per launch than ds_add_f32); when the
// segment id changes it stores the row and clears it.  A segment that lies inside the range goes to its row of the
// result; the (at most two) segments that continue in a neighbouring range go to the range's partial rows
// ws[range][0 | 1], which uvu_fixup_kernel adds in range order.  Per-edge messages never reach memory.
struct BigSegRange {   // positions and ranges fit 32 bits (the host checks n_rows < 2^31)
  int p0, p1;
  bool first_complete, last_complete;
  __device__ __forceinline__ BigSegRange(const int64_t* __restrict__ seg_ids, int range, int per_range, int n_rows) {
    const int64_t b = (int64_t)range * per_range;
    p0 = b < n_rows ? (int)b : n_rows;
    p1 = b + per_range < n_rows ? (int)(b + per_range) : n_rows;
    first_complete = p0 >= p1 || p0 == 0 || seg_ids[p0 - 1] != seg_ids[p0];
    last_complete = p0 >= p1 || p1 == n_rows || seg_ids[p1 - 1] != seg_ids[p1];
  }
};

// The channel count as a value the compiler cannot follow from one loop iteration to the next.  The generated bodies
// address row p of an operand at p * C; with C invariant over the loop, all of these products (one per weight path
// and row: more than a hundred) are computed once in front of the loop and kept, which takes more scalar registers
// than there are: they end up parked in vector registers, and those in scratch.  Used in the backward (lmax = 6: 3.19
// -> 2.87 ms per launch); the forward, with fewer rows to address, is faster without (1.68 against 1.72 ms).
__device__ __forceinline__ int opaque_copy(int v) {
  asm volatile("" : "+s"(v));
  return v;
}

// Segment id, edge and gathered row of the k-th position of a range; past the end of the range, those of its last
// position (of position 0 for an empty range), so that every slot runs the same loads.
struct BigSegIndex {
  int sid, edge, other;
  __device__ __forceinline__ BigSegIndex(const UvuDev<float>& a, const BigSegRange& R, int k) {
    const int q = R.p0 + k;
    const int qq = q < R.p1 ? q : (R.p1 > R.p0 ? R.p1 - 1 : 0);
    sid = (int)a.seg_ids[qq];
    edge = a.perm ? (int)a.perm[qq] : qq;
    other = (int)a.gather[qq];
  }
};

// Store the slot's accumulator row (D rows of one channel per lane) as the row of segment `seg` and clear it.
template <int D>
__device__ __forceinline__ void big_seg_flush(float* __restrict__ acc, float* __restrict__ rows, float* __restrict__ ws,
                                              int seg, int range, bool first, bool complete, int64_t C, int c,
                                              bool c_ok) {
  float* dst = (complete ? rows + (int64_t)seg * D * C : ws + ((int64_t)range * 2 + (first ? 0 : 1)) * D * C) + c;
#pragma unroll
  for (int m = 0; m < D; ++m) {
    const float v = acc[m * kWave];
    acc[m * kWave] = 0.f;
    if (c_ok) dst[m * C] = v;
  }
}

template <class TP, bool PS>
__global__ void __launch_bounds__(256, 2) uvu_big_seg_fwd_kernel(const UvuDev<float> a, int64_t n_waves) {
  constexpr int D1 = TP::D1, D2 = TP::D2, DO = TP::DO, P = TP::P;
  extern __shared__ float big_seg_lds[];
  const Lanes L(a.lpe_log2);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (wave >= n_waves) return;
  float* acc = big_seg_lds + (threadIdx.x / kWave) * DO * kWave + L.lane;
#pragma unroll
  for (int m = 0; m < DO; ++m) acc[m * kWave] = 0.f;
  const int64_t C = a.C;
  const int c_raw = blockIdx.y * L.lpe + L.cl;
  const bool c_ok = c_raw < a.C;
  const int c = min(c_raw, a.C - 1);
  const int range = (int)wave * L.slots + L.slot;
  const BigSegRange R(a.seg_ids, range, a.pos_per_wave, (int)a.n_rows);
  const float* __restrict__ ps = a.ps;
  int cur = -1;
  bool first = true;
  BigSegIndex I(a, R, 0);
  for (int k = 0; k < a.pos_per_wave; ++k) {       // the same trip count in every slot; `live` masks the tail
    const bool live = R.p0 + k < R.p1;
    const int sid = I.sid;
    const int64_t e = I.edge, xr = I.other;
    if (k + 1 < a.pos_per_wave) I = BigSegIndex(a, R, k + 1);   // in flight during this position's arithmetic
    if (live && sid != cur) {
      if (cur >= 0) {
        big_seg_flush<DO>(acc, a.out, a.ws, cur, range, first, first ? R.first_complete : true, C, c, c_ok);
        first = false;
      }
      cur = sid;
    }
    float x[D1], y[D2];
#pragma unroll
    for (int j = 0; j < D2; ++j) y[j] = a.y[e * D2 + j];
#pragma unroll
    for (int i = 0; i < D1; ++i) x[i] = a.x[(xr * D1 + i) * C + c];
    const float* wrow = a.w + (a.w_shared ? 0 : e) * P * C + c;
    TP::fwd(
        x, y,
        [&](int p) __attribute__((always_inline)) {
          const float w = __builtin_nontemporal_load(wrow + p * C);
          if constexpr (PS) return w * ps[p]; else return w;
        },
        [&](int m, float v) __attribute__((always_inline)) {
          acc[m * kWave] += live ? v : 0.f;   // no branch: the reads can be issued early
        });
  }
  if (cur >= 0)
    big_seg_flush<DO>(acc, a.out, a.ws, cur, range, first, (first ? R.first_complete : true) && R.last_complete, C, c,
                      c_ok);
}

// Backward of the above over the list sorted by the other end: a segment is a row of x, its gradient is summed in
// LDS; grad_out rows are gathered, grad_y and the weight gradient are written per edge.
//
// The body needs all 256 registers, so nothing may stay in a register from one position to the next: whatever the
// compiler carries across the body it spills to scratch, and a reload from scratch waits on the counter that also
// counts the 106 weight-gradient stores of the position before (they would otherwise drain in the background).
// Therefore
//  * everything that follows from the thread index and the kernel arguments (lane roles, range, channel, pointers)
//    is derived again in every iteration from a copy of the thread index the compiler cannot follow (opaque_lane);
//  * the two values that do change (open segment, "nothing flushed yet") live in LDS (kBigSegStateInts per lane);
//  * the indices of the next positions are staged in LDS a chunk at a time: every `lanes per edge` iterations the
//    lanes of a slot load segment id, edge and gathered row of that many positions with one coalesced load each
//    (kBigSegIndexInts per wavefront), and an iteration reads its three values from there.
constexpr int kBigSegIndexInts = kWave * 3;
constexpr int kBigSegStateInts = 2;
__device__ __forceinline__ int opaque_lane() {
  int v = threadIdx.x;
  asm volatile("" : "+v"(v));
  return v;
}

template <class TP, int GW, bool PS>
__global__ void __launch_bounds__(256, 2) uvu_big_seg_bwd_kernel(const UvuDev<float> a, int64_t n_waves) {
  constexpr int D1 = TP::D1, D2 = TP::D2, DO = TP::DO, P = TP::P;
  extern __shared__ float big_seg_lds[];
  if ((int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave >= n_waves) return;
  int* const idx_all = reinterpret_cast<int*>(big_seg_lds + 4 * D1 * kWave);
  volatile int* const state = reinterpret_cast<volatile int*>(idx_all + 4 * kBigSegIndexInts) + threadIdx.x;
  {
    float* acc = big_seg_lds + (threadIdx.x / kWave) * D1 * kWave + (threadIdx.x & (kWave - 1));
#pragma unroll
    for (int i = 0; i < D1; ++i) acc[i * kWave] = 0.f;
    state[0] = -1;    // open segment
    state[256] = 1;   // no segment of the range flushed yet
  }
  const float* __restrict__ ps = a.ps;
  const int per = a.pos_per_wave, n_rows = (int)a.n_rows;
  for (int k = 0; k <= per; ++k) {      // iteration `per` only closes the range
    const int tid = opaque_lane();
    const int lane = tid & (kWave - 1), wv = tid >> 6;
    const int lpe = 1 << a.lpe_log2, slot = lane >> a.lpe_log2, cl = lane & (lpe - 1);
    const int64_t C = opaque_copy(a.C);
    const int c_raw = blockIdx.y * lpe + cl;
    const bool c_ok = c_raw < a.C;
    const int c = min(c_raw, a.C - 1);
    const int range = ((int)blockIdx.x * 4 + wv) * (kWave >> a.lpe_log2) + slot;
    const int64_t b0 = (int64_t)range * per;
    const int p0 = b0 < n_rows ? (int)b0 : n_rows;
    const int p1 = b0 + per < n_rows ? (int)(b0 + per) : n_rows;
    float* acc = big_seg_lds + wv * D1 * kWave + lane;
    int* idx = idx_all + wv * kBigSegIndexInts;
    const int cur = state[0];
    const bool first = state[256] != 0;
    if (k == per) {
      if (cur >= 0 && a.gx) {
        const bool first_complete = p0 == 0 || a.seg_ids[p0 - 1] != a.seg_ids[p0];
        const bool last_complete = p1 == n_rows || a.seg_ids[p1 - 1] != a.seg_ids[p1];
        big_seg_flush<D1>(acc, a.gx, a.ws, cur, range, first, (first ? first_complete : true) && last_complete, C, c,
                          c_ok);
      }
      break;
    }
    const int kk = k & (lpe - 1);
    if (kk == 0) {   // the same in every lane: stage the indices of the next lpe positions of every slot
      const int q = p0 + k + cl;
      const int qq = q < p1 ? q : (p1 > p0 ? p1 - 1 : 0);
      idx[lane * 3 + 0] = (int)a.seg_ids[qq];
      idx[lane * 3 + 1] = a.perm ? (int)a.perm[qq] : qq;
      idx[lane * 3 + 2] = (int)a.gather[qq];
      __builtin_amdgcn_wave_barrier();
    }
    const int ent = (slot * lpe + kk) * 3;
    const int sid = idx[ent];
    const int64_t e = idx[ent + 1], gr = idx[ent + 2];
    const bool live = p0 + k < p1;
    if (live && sid != cur) {
      if (cur >= 0) {
        if (a.gx) {
          const bool first_complete = p0 == 0 || a.seg_ids[p0 - 1] != a.seg_ids[p0];
          big_seg_flush<D1>(acc, a.gx, a.ws, cur, range, first, first ? first_complete : true, C, c, c_ok);
        }
        state[256] = 0;
      }
      state[0] = sid;
    }
    float y[D2], gy[D2], g[DO];
#pragma unroll
    for (int j = 0; j < D2; ++j) {
      y[j] = a.y[e * D2 + j];
      gy[j] = 0.f;
    }
    const float* grow = a.g + gr * DO * C + c;
#pragma unroll
    for (int m = 0; m < DO; ++m) g[m] = grow[m * C];
    const float* xrow = a.x + (int64_t)sid * D1 * C + c;
    const float* wrow = a.w + (a.w_shared ? 0 : e) * P * C + c;
    float* gwrow = a.gw + e * P * C + c;
    const bool store = live && c_ok;
    TP::bwd(
        [&](int i) __attribute__((always_inline)) { return xrow[i * C]; }, y,
        [&](int p) __attribute__((always_inline)) {
          const float w = __builtin_nontemporal_load(wrow + p * C);
          if constexpr (PS) return w * ps[p]; else return w;
        },
        g,
        [&](int i, float v) __attribute__((always_inline)) {
          if (live) acc[i * kWave] += v;   // under a branch on purpose: hoisted reads would not fit the registers here
        },
        gy,
        [&](int p, float v) __attribute__((always_inline)) {
          if constexpr (GW == kGwStore) {
            if (store) __builtin_nontemporal_store(PS ? v * ps[p] : v, gwrow + p * C);
          }
        });
    if (a.gy) {
      const float keep = c_ok ? 1.f : 0.f;  // duplicate channels of the padding lanes do not count
      float* gyrow = a.gy + e * D2;
#pragma unroll
      for (int j = 0; j < D2; ++j) gy[j] *= keep;
      group_sum_scatter<float, D2>(gy, lpe, [&](const auto& s) {   // lane cl ends up with components cl, cl + lpe, ...
#pragma unroll
        for (int i = 0; i < array_len(s); ++i) {
          const int j = i * lpe + cl;
          if (live && j < D2) gyrow[j] = s[i];
        }
      });
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
  e.seg_fwd = uvu_big_seg_fwd_kernel<TP, PS>;
  e.seg_bwd[kGwNone] = uvu_big_seg_bwd_kernel<TP, kGwNone, PS>;
  e.seg_bwd[kGwStore] = uvu_big_seg_bwd_kernel<TP, kGwStore, PS>;
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
