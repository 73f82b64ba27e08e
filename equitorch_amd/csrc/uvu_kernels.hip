// Channel-wise ("uvu") sparse Clebsch-Gordan tensor product with the table compiled into the kernel.
//
// Work decomposition (wave64): a wavefront is split into 64/LPE "slots" of LPE lanes; a lane owns V
// consecutive channels, so one slot covers LPE*V >= C channels of one row (edge) with V*sizeof(T)-byte
// coalesced accesses.  In row mode every slot owns one batch row.
//
// In segment mode (fused gather + tensor product + scatter-sum over an edge list sorted by segment id:
// destination node in the forward, source node in the backward) every wavefront owns the same number of
// consecutive sorted positions, so the load is balanced whatever the degree distribution.  In every step its
// slots take the next consecutive positions that belong to one segment (a step never straddles a segment
// boundary; slots past the boundary idle and the next step starts at the boundary), the per-edge result is
// accumulated in registers, and when the segment id changes the accumulator is summed over the slots with
// cross-lane shuffles and stored once.  A segment that lies entirely inside the wavefront's range is written to the
// output directly; the (at most two) segments cut by the range boundary are written as partial rows to a
// workspace and summed in a fixed order by uvu_fixup_kernel.  No atomics: results are deterministic.
#include "uvu_common.h"
#include "sh_device.h"

namespace cgtp {
#include "generated/uvu_configs.inc"

template <typename T, int D, int V>
__device__ __forceinline__ void zero_rows(T (&a)[D][V]) {
#pragma unroll
  for (int m = 0; m < D; ++m)
#pragma unroll
    for (int v = 0; v < V; ++v) a[m][v] = T(0);
}

// ---- row mode ------------------------------------------------------------------------------------------------
template <class TP, typename T, int V, bool PS>
__global__ void __launch_bounds__(256) uvu_fwd_kernel(const UvuDev<T> a) {
  constexpr int D1 = TP::D1, D2 = TP::D2, DO = TP::DO, P = TP::P;
  const Lanes L(a.lpe_log2);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int c0 = (blockIdx.y * L.lpe + L.cl) * V;
  const int64_t C = a.C;
  const int64_t r = wave * L.slots + L.slot;
  if (r >= a.n_rows || c0 >= a.C) return;
  const int64_t xr = a.gather ? a.gather[r] : r;
  const int64_t wr = a.w_shared ? 0 : r;
  T x[D1][V], y[D2], acc[DO][V];
#pragma unroll
  for (int j = 0; j < D2; ++j) y[j] = a.y[r * D2 + j];
#pragma unroll
  for (int i = 0; i < D1; ++i) load_vec<T, V>(x[i], a.x + (xr * D1 + i) * C + c0);
  const T* wrow = a.w + wr * P * C + c0;
  T w[P][V];  // every weight row is requested before the arithmetic starts: maximal memory-level parallelism
#pragma unroll
  for (int p = 0; p < P; ++p) load_vec_stream<T, V>(w[p], wrow + p * C);
  if constexpr (PS) {  // this instantiation applies one factor per weight path
#pragma unroll
    for (int p = 0; p < P; ++p) {
      const T f = a.ps[p];
#pragma unroll
      for (int v = 0; v < V; ++v) w[p][v] *= f;
    }
  }
  zero_rows(acc);
  TP::template fwd<T, V>(x, y, [&](int p, T (&wp)[V]) {
#pragma unroll
          for (int v = 0; v < V; ++v) wp[v] = w[p][v];
        }, acc);
#pragma unroll
  for (int m = 0; m < DO; ++m) store_vec_stream<T, V>(a.out + (r * DO + m) * C + c0, acc[m]);
}


template <class TP, typename T, int V, int GW, bool PS>
__global__ void __launch_bounds__(256, 2) uvu_bwd_kernel(const UvuDev<T> a, int64_t n_waves) {
  constexpr int D1 = TP::D1, D2 = TP::D2, DO = TP::DO, P = TP::P;
  const Lanes L(a.lpe_log2);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int c0 = L.cl * V;
  const bool cok = c0 < a.C;
  const int64_t C = a.C;
  if (wave >= n_waves) return;

  T gwacc[GW == kGwReduce ? P : 1][V], gx[D1][V];
  zero_rows(gwacc);
  zero_rows(gx);
#pragma unroll 1
  for (int64_t r = wave * L.slots + L.slot; r < a.n_rows; r += n_waves * L.slots) {
    const int64_t gr = a.gather ? a.gather[r] : r;
    const int64_t xr = a.x_gather ? a.x_gather[r] : r;
    T x[D1][V], g[DO][V], y[D2], gy[D2];
#pragma unroll
    for (int j = 0; j < D2; ++j) {
      y[j] = a.y[r * D2 + j];
      gy[j] = T(0);
    }
    if (cok) {
#pragma unroll
      for (int i = 0; i < D1; ++i) load_vec<T, V>(x[i], a.x + (xr * D1 + i) * C + c0);
#pragma unroll
      for (int m = 0; m < DO; ++m) load_vec<T, V>(g[m], a.g + (gr * DO + m) * C + c0);
      const T* wrow = a.w + (a.w_shared ? 0 : r) * P * C + c0;
      T w[P][V];  // every weight row is requested before the arithmetic starts: maximal memory-level parallelism
#pragma unroll
      for (int p = 0; p < P; ++p) load_vec_stream<T, V>(w[p], wrow + p * C);
      if constexpr (PS) {  // this instantiation applies one factor per weight path
#pragma unroll
        for (int p = 0; p < P; ++p) {
          const T f = a.ps[p];
#pragma unroll
          for (int v = 0; v < V; ++v) w[p][v] *= f;
        }
      }
      T* gwrow = a.gw + r * P * C + c0;
      TP::template bwd<T, V>(
          x, y, [&](int p, T (&wp)[V]) {
#pragma unroll
          for (int v = 0; v < V; ++v) wp[v] = w[p][v];
        }, g, gx, gy,
          [&](int p, const T (&gwp)[V]) {
            if constexpr (GW == kGwReduce) {
#pragma unroll
              for (int v = 0; v < V; ++v) gwacc[p][v] += gwp[v];
            } else if constexpr (GW == kGwStore) {
              if constexpr (PS) {
                const T f = a.ps[p];
                T sc[V];
#pragma unroll
                for (int v = 0; v < V; ++v) sc[v] = gwp[v] * f;
                store_vec_stream<T, V>(gwrow + p * C, sc);
              } else {
                store_vec_stream<T, V>(gwrow + p * C, gwp);
              }
            }
          });
      if (a.gx) {
#pragma unroll
        for (int i = 0; i < D1; ++i) store_vec_stream<T, V>(a.gx + (r * D1 + i) * C + c0, gx[i]);
      }
      zero_rows(gx);
    }
    if (a.gy) {
#pragma unroll
      for (int j = 0; j < D2; ++j) {
        const T s = group_sum(gy[j], L.lpe);
        if (L.cl == (j & (L.lpe - 1))) a.gy[r * D2 + j] = s;
      }
    }
  }
  if constexpr (GW == kGwReduce) {
#pragma unroll
    for (int p = 0; p < P; ++p)
#pragma unroll
      for (int v = 0; v < V; ++v) {
        gwacc[p][v] = cross_group_sum(gwacc[p][v], L.lpe);
        if constexpr (PS) gwacc[p][v] *= a.ps[p];
      }
    if (L.slot == 0 && cok) {
#pragma unroll
      for (int p = 0; p < P; ++p) store_vec<T, V>(a.wsw + (wave * P + p) * C + c0, gwacc[p]);
    }
  }
}

// ---- segment mode ----------------------------------------------------------------------------------------------
// Range [p0, p1) of sorted positions owned by one wavefront.  Three ways to cut the edge list:
//  * aligned (wave_seg given): the wavefront owns the whole segments [s0, s1); every row it produces is final,
//    and it also zero-fills the rows of empty segments in [s0, s1);
//  * at given positions (wave_pos given): range k is [wave_pos[k], wave_pos[k + 1]) — the caller cuts where it
//    likes, e.g. so that every wavefront has the same number of steps;
//  * by position (neither): exactly per_wave positions each.
// In the last two the first / last segment of a range may continue in a neighbouring wavefront and then goes
// through a partial row (see uvu_fixup_kernel).
struct SegRange {
  int64_t p0, p1;
  int s0, s1;                          // aligned mode: owned segments; else -1
  bool first_complete, last_complete;  // does the first / last segment of the range begin / end inside it?
  __device__ __forceinline__ SegRange(const int64_t* __restrict__ seg_ids, const int64_t* __restrict__ ptr,
                                      const int32_t* __restrict__ wave_seg, const int64_t* __restrict__ wave_pos,
                                      int64_t wave, int per_wave, int64_t n_rows) {
    if (wave_seg) {
      s0 = wave_seg[wave];
      s1 = wave_seg[wave + 1];
      p0 = ptr[s0];
      p1 = ptr[s1];
      first_complete = last_complete = true;
    } else {
      s0 = s1 = -1;
      if (wave_pos) {
        p0 = wave_pos[wave];
        p1 = wave_pos[wave + 1];
      } else {
        p0 = wave * per_wave;
        p1 = p0 + per_wave < n_rows ? p0 + per_wave : n_rows;
      }
      first_complete = p0 == 0 || seg_ids[p0 - 1] != seg_ids[p0];
      last_complete = p1 == n_rows || seg_ids[p1 - 1] != seg_ids[p1];
    }
  }
};

// Progress of a wavefront through its range.
struct SegStep {
  int cur = -1;       // segment being accumulated (-1: none yet)
  bool first = true;  // no segment of this range has been flushed yet
  int next_row;       // aligned mode: lowest owned segment whose row has not been written yet
};

// Rows [from, to) := 0, all lanes of the wavefront cooperating.
template <typename T>
__device__ __forceinline__ void zero_fill_rows(T* __restrict__ rows, int from, int to, int64_t row_len, int lane) {
  if (!rows || from >= to) return;
  T* p = rows + (int64_t)from * row_len;
  const int64_t n = (int64_t)(to - from) * row_len;
  for (int64_t i = lane; i < n; i += kWave) p[i] = T(0);
}

// Sum `acc` over the slots and store it as the row of segment `st.cur`: to `final_rows` if the segment is
// complete in this wavefront's range, else to the wavefront's partial row 0 (range's first segment) or 1 (last).
template <typename T, int D, int V>
__device__ __forceinline__ void flush_segment(SegStep& st, T (&acc)[D][V], T* __restrict__ final_rows,
                                              T* __restrict__ ws, int64_t wave, bool complete, const SegRange& R,
                                              const Lanes& L, bool cok, int64_t C, int c0) {
  cross_group_sum_rows<T, D, V>(acc, L.lpe);
  T* dst = complete ? final_rows + (int64_t)st.cur * D * C : ws + (wave * 2 + (st.first ? 0 : 1)) * D * C;
  if (L.slot == 0 && cok && final_rows) {  // final_rows == nullptr: this result was not requested
#pragma unroll
    for (int m = 0; m < D; ++m) store_vec<T, V>(dst + m * C + c0, acc[m]);
  }
  if (R.s0 >= 0) {
    zero_fill_rows(final_rows, st.next_row, st.cur, D * C, L.lane);
    st.next_row = st.cur + 1;
  }
  st.first = false;
  zero_rows(acc);
}

// Index data of up to 64 consecutive sorted positions [c0, c1), fetched with one coalesced load per array (lane i
// holds position c0 + i) and handed to the slots with cross-lane shuffles, so that no step waits on a chain of
// dependent index loads.
struct SegIndexRegs {
  int sid, edge, other;  // segment id, edge id, row of the gathered operand
  int npos;
  __device__ __forceinline__ SegIndexRegs(const int64_t* __restrict__ seg_ids, const int64_t* __restrict__ perm,
                                          const int64_t* __restrict__ gather, int64_t c0, int64_t c1, int lane) {
    npos = (int)(c1 - c0);
    const int64_t p = c0 + (lane < npos ? lane : 0);
    sid = (int)seg_ids[p];
    edge = (int)(perm ? perm[p] : p);
    other = (int)gather[p];
    // The step loop reads these registers through the cross-lane unit in every step.  While the loads are still
    // pending when the loop is entered, the compiler's wait for them sits inside the loop, where the counter it
    // waits on also counts the stores of the step before: every step then begins by draining them.  Passing the
    // values through an (empty) instruction here puts the wait in front of the loop.
    asm volatile("" : "+v"(sid), "+v"(edge), "+v"(other));
  }
};

// One step of a wavefront's walk over its sorted positions: slot s looks at offset off0 + s of the current index
// chunk; the step covers the leading slots whose segment id equals that of off0.  Flushes the accumulator when
// the segment changes.
template <typename T, int D, int V>
__device__ __forceinline__ bool seg_step_begin(SegStep& st, T (&acc)[D][V], T* __restrict__ final_rows,
                                               T* __restrict__ ws, const SegIndexRegs& I, int& off0, int& edge,
                                               int& other, int64_t wave, const SegRange& R, const Lanes& L,
                                               int lpe_log2, bool cok, int64_t C, int c0) {
  const int off = off0 + L.slot;
  const int src = off < I.npos ? off : off0;
  const int sid = __shfl(I.sid, src, kWave);
  edge = __shfl(I.edge, src, kWave);
  other = __shfl(I.other, src, kWave);
  const int lead = __builtin_amdgcn_readlane(I.sid, off0);   // off0 is the same in every lane: a scalar read, no wait
  if (lead != st.cur) {
    if (st.cur >= 0)
      flush_segment<T, D, V>(st, acc, final_rows, ws, wave, st.first ? R.first_complete : true, R, L, cok, C, c0);
    st.cur = lead;
  }
  const bool valid = off < I.npos && sid == lead;
  off0 += __popcll(__ballot(valid)) >> lpe_log2;
  return valid;
}

// End of a wavefront's range: flush the open segment and zero-fill the remaining owned empty segments.
template <typename T, int D, int V>
__device__ __forceinline__ void seg_finish(SegStep& st, T (&acc)[D][V], T* __restrict__ final_rows,
                                           T* __restrict__ ws, int64_t wave, const SegRange& R, const Lanes& L,
                                           bool cok, int64_t C, int c0) {
  if (st.cur >= 0)
    flush_segment<T, D, V>(st, acc, final_rows, ws, wave, (st.first ? R.first_complete : true) && R.last_complete, R,
                           L, cok, C, c0);
  if (R.s0 >= 0) zero_fill_rows(final_rows, st.next_row, R.s1, (int64_t)D * C, L.lane);
}

// YV: the second operand is an edge vector; its harmonics are evaluated here (sh_device.h).
template <class TP, typename T, int V, bool PS, bool YV = false>
__global__ void __launch_bounds__(256) uvu_seg_fwd_kernel(const UvuDev<T> a, int64_t n_waves) {
  constexpr int D1 = TP::D1, D2 = TP::D2, DO = TP::DO, P = TP::P;
  const Lanes L(a.lpe_log2);
  const int64_t wave = seg_wave_index(n_waves);
  if (wave < 0) return;
  const int c0 = L.cl * V;
  const bool cok = c0 < a.C;
  const int64_t C = a.C;
  const SegRange R(a.seg_ids, a.ptr, a.wave_seg, a.wave_pos, wave, a.pos_per_wave, a.n_rows);

  T acc[DO][V];
  zero_rows(acc);
  SegStep st;
  st.next_row = R.s0;
  for (int64_t cb = R.p0; cb < R.p1; cb += kWave) {
  const SegIndexRegs I(a.seg_ids, a.perm, a.gather, cb, cb + kWave < R.p1 ? cb + kWave : R.p1, L.lane);
  for (int off0 = 0; off0 < I.npos;) {
    int ei, oi;
    if (seg_step_begin<T, DO, V>(st, acc, a.out, a.ws, I, off0, ei, oi, wave, R, L, a.lpe_log2, cok, C, c0)) {
      const int64_t e = ei, xr = oi;
      T x[D1][V], y[D2];
      if constexpr (YV) {
        const ShPoint<T> pt(a.y[e * 3], a.y[e * 3 + 1], a.y[e * 3 + 2], a.y_vec == kYUnitVector);
        sh_values<T, TP::SH_LMAX>(pt.x, pt.y, pt.z, y);
      } else {
#pragma unroll
        for (int j = 0; j < D2; ++j) y[j] = a.y[e * D2 + j];
      }
      if (cok) {
#pragma unroll
        for (int i = 0; i < D1; ++i) load_vec<T, V>(x[i], a.x + (xr * D1 + i) * C + c0);
        const T* wrow = a.w + (a.w_shared ? 0 : e) * P * C + c0;
        T w[P][V];  // every weight row is requested before the arithmetic starts: maximal memory-level parallelism
#pragma unroll
        for (int p = 0; p < P; ++p) load_vec_stream<T, V>(w[p], wrow + p * C);
        if constexpr (PS) {  // this instantiation applies one factor per weight path
#pragma unroll
          for (int p = 0; p < P; ++p) {
            const T f = a.ps[p];
#pragma unroll
            for (int v = 0; v < V; ++v) w[p][v] *= f;
          }
        }
        TP::template fwd<T, V>(x, y, [&](int p, T (&wp)[V]) {
#pragma unroll
          for (int v = 0; v < V; ++v) wp[v] = w[p][v];
        }, acc);
      }
    }
  }
  }
  seg_finish<T, DO, V>(st, acc, a.out, a.ws, wave, R, L, cok, C, c0);
}

template <class TP, typename T, int V, int GW, bool PS, bool YV = false>
__global__ void __launch_bounds__(256, 2) uvu_seg_bwd_kernel(const UvuDev<T> a, int64_t n_waves) {
  constexpr int D1 = TP::D1, D2 = TP::D2, DO = TP::DO, P = TP::P;
  const Lanes L(a.lpe_log2);
  const int64_t wave = seg_wave_index(n_waves);
  if (wave < 0) return;
  const int c0 = L.cl * V;
  const bool cok = c0 < a.C;
  const int64_t C = a.C;
  const SegRange R(a.seg_ids, a.ptr, a.wave_seg, a.wave_pos, wave, a.pos_per_wave, a.n_rows);

  T gwacc[GW == kGwReduce ? P : 1][V], acc[D1][V];
  zero_rows(gwacc);
  zero_rows(acc);
  SegStep st;
  st.next_row = R.s0;
  // The rows of x belong to the segment, not to the edge: they stay in registers over the steps of a segment (every
  // load instruction costs delivery bandwidth, whether or not it hits in cache).
  T x[D1][V];
  zero_rows(x);
  int x_seg = -1;
  for (int64_t cb = R.p0; cb < R.p1; cb += kWave) {
  const SegIndexRegs I(a.seg_ids, a.perm, a.gather, cb, cb + kWave < R.p1 ? cb + kWave : R.p1, L.lane);
  for (int off0 = 0; off0 < I.npos;) {
    int ei, oi;
    const bool valid = seg_step_begin<T, D1, V>(st, acc, a.gx, a.ws, I, off0, ei, oi, wave, R, L, a.lpe_log2, cok, C, c0);
    if (st.cur != x_seg) {   // the same for all lanes of the wavefront
      x_seg = st.cur;
      if (cok) {
#pragma unroll
        for (int i = 0; i < D1; ++i) load_vec<T, V>(x[i], a.x + ((int64_t)x_seg * D1 + i) * C + c0);
      }
    }
    if (valid) {
      const int64_t e = ei, gr = oi;
      T g[DO][V], y[D2], gy[D2];
      T ux = 0, uy = 0, uz = 0;
      if constexpr (YV) {
        ux = a.y[e * 3]; uy = a.y[e * 3 + 1]; uz = a.y[e * 3 + 2];
        const ShPoint<T> pt(ux, uy, uz, a.y_vec == kYUnitVector);
        sh_values<T, TP::SH_LMAX>(pt.x, pt.y, pt.z, y);
      } else {
#pragma unroll
        for (int j = 0; j < D2; ++j) y[j] = a.y[e * D2 + j];
      }
#pragma unroll
      for (int j = 0; j < D2; ++j) gy[j] = T(0);
      if (cok) {
#pragma unroll
        for (int m = 0; m < DO; ++m) load_vec<T, V>(g[m], a.g + (gr * DO + m) * C + c0);
        const T* wrow = a.w + (a.w_shared ? 0 : e) * P * C + c0;
        T w[P][V];  // every weight row is requested before the arithmetic starts: maximal memory-level parallelism
#pragma unroll
        for (int p = 0; p < P; ++p) load_vec_stream<T, V>(w[p], wrow + p * C);
        if constexpr (PS) {  // this instantiation applies one factor per weight path
#pragma unroll
          for (int p = 0; p < P; ++p) {
            const T f = a.ps[p];
#pragma unroll
            for (int v = 0; v < V; ++v) w[p][v] *= f;
          }
        }
        T* gwrow = a.gw + e * P * C + c0;
        TP::template bwd<T, V>(
            x, y, [&](int p, T (&wp)[V]) {
#pragma unroll
          for (int v = 0; v < V; ++v) wp[v] = w[p][v];
        }, g, acc, gy,
            [&](int p, const T (&gwp)[V]) {
              if constexpr (GW == kGwReduce) {
#pragma unroll
                for (int v = 0; v < V; ++v) gwacc[p][v] += gwp[v];
              } else if constexpr (GW == kGwStore) {
                if constexpr (PS) {
                  const T f = a.ps[p];
                  T sc[V];
#pragma unroll
                  for (int v = 0; v < V; ++v) sc[v] = gwp[v] * f;
                  store_vec_stream<T, V>(gwrow + p * C, sc);
                } else {
                  store_vec_stream<T, V>(gwrow + p * C, gwp);
                }
              }
            });
      }
      if (a.gy) {
        // Sums over the channels of an edge.  kSpread: the halving exchange (group_sum_scatter) — a quarter of the
        // cross-lane moves, issued together, one store.  It keeps a few more values live at once; in the
        // instantiations named by kSpread that costs nothing, in most others it costs a wavefront per SIMD or
        // scratch, and those sum one component at a time as before.
        constexpr bool kSpread = sizeof(T) == 4 && V == 4 && GW != kGwReduce && D2 >= 9;
        if constexpr (YV && kSpread) {
          // chain rule through the harmonics (and the normalisation): linear in grad_y, so every lane applies it
          // to its own channels' share first and three values per edge are summed over the channels instead of D2
          const ShPoint<T> pt(ux, uy, uz, a.y_vec == kYUnitVector);
          T v3[3];
          sh_pull_back<T, TP::SH_LMAX>(pt.x, pt.y, pt.z, gy, v3[0], v3[1], v3[2]);
          pt.pull_back(v3[0], v3[1], v3[2], a.y_vec == kYUnitVector);
          group_sum_scatter<T, 3>(v3, L.lpe, [&](const auto& s) {
#pragma unroll
            for (int i = 0; i < array_len(s); ++i) {
              const int j = i * L.lpe + L.cl;
              if (j < 3) a.gy[e * 3 + j] = s[i];
            }
          });
        } else if constexpr (YV) {
#pragma unroll
          for (int j = 0; j < D2; ++j) gy[j] = group_sum(gy[j], L.lpe);
          const ShPoint<T> pt(ux, uy, uz, a.y_vec == kYUnitVector);
          T vx, vy, vz;
          sh_pull_back<T, TP::SH_LMAX>(pt.x, pt.y, pt.z, gy, vx, vy, vz);
          pt.pull_back(vx, vy, vz, a.y_vec == kYUnitVector);
          if (L.cl == 0) { a.gy[e * 3] = vx; a.gy[e * 3 + 1] = vy; a.gy[e * 3 + 2] = vz; }
        } else if constexpr (kSpread) {
          group_sum_scatter<T, D2>(gy, L.lpe, [&](const auto& s) {   // lane cl ends up with components cl, cl + lpe, ...
#pragma unroll
            for (int i = 0; i < array_len(s); ++i) {
              const int j = i * L.lpe + L.cl;
              if (j < D2) a.gy[e * D2 + j] = s[i];
            }
          });
        } else {
#pragma unroll
          for (int j = 0; j < D2; ++j) {
            const T s = group_sum(gy[j], L.lpe);
            if (L.cl == (j & (L.lpe - 1))) a.gy[e * D2 + j] = s;
          }
        }
      }
    }
  }
  }
  seg_finish<T, D1, V>(st, acc, a.gx, a.ws, wave, R, L, cok, C, c0);
  if constexpr (GW == kGwReduce) {
#pragma unroll
    for (int p = 0; p < P; ++p)
#pragma unroll
      for (int v = 0; v < V; ++v) {
        gwacc[p][v] = cross_group_sum(gwacc[p][v], L.lpe);
        if constexpr (PS) gwacc[p][v] *= a.ps[p];
      }
    if (L.slot == 0 && cok) {
#pragma unroll
      for (int p = 0; p < P; ++p) store_vec<T, V>(a.wsw + (wave * P + p) * C + c0, gwacc[p]);
    }
  }
}

// Rows of segments cut by a wavefront boundary: rows[v] = sum of the partial rows of the wavefronts that
// touch v, in ascending wavefront order; rows of empty segments are zeroed.  One wavefront per segment.
// wave_pos (n_waves + 1 ascending positions) when the ranges were cut at given positions, else per_wave each.
// Called by all lanes of a wavefront with the same q.  Ranges cut at given positions are about equally long, so the
// answer lies near q * n_waves / n_rows: the wavefront looks at 64 consecutive entries around that guess with one
// coalesced load (a binary search is eleven dependent loads at 2048 ranges, and this kernel does little else) and
// falls back to the search when the window misses.
// `first` receives the first position of the range found (from the window, not from another load).
__device__ __forceinline__ int64_t range_of_position(const int64_t* __restrict__ wave_pos, int64_t n_waves, int per_wave,
                                                     int64_t n_rows, int64_t q, int lane, int64_t* first) {
  if (!wave_pos) {
    const int64_t k = q / per_wave;
    *first = k * per_wave;
    return k;
  }
  int64_t base = q * n_waves / n_rows - 32;
  if (base > n_waves - 63) base = n_waves - 63;
  if (base < 0) base = 0;
  const int64_t idx = base + lane;
  const int64_t pos = idx <= n_waves ? wave_pos[idx] : INT64_MAX;
  const bool le = pos <= q;                                   // entries are ascending: a prefix of the lanes
  const int cnt = __popcll(__ballot(le));
  if (cnt > 0 && (cnt < kWave || base + kWave > n_waves)) {
    // positions fit 32 bits in segment mode
    *first = (int64_t)(unsigned)__shfl((int)pos, cnt - 1, kWave);
    return base + cnt - 1;
  }
  int64_t lo = 0, hi = n_waves - 1;   // largest k with wave_pos[k] <= q
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) >> 1;
    if (wave_pos[mid] <= q) lo = mid; else hi = mid - 1;
  }
  *first = wave_pos[lo];
  return lo;
}

template <typename T>
__global__ void __launch_bounds__(256) uvu_fixup_kernel(T* __restrict__ rows, const T* __restrict__ ws,
                                                        const int64_t* __restrict__ ptr, int64_t n_seg,
                                                        int64_t row_len, int per_wave,
                                                        const int64_t* __restrict__ wave_pos, int64_t n_waves,
                                                        int64_t n_rows) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t v = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (v >= n_seg) return;
  const int64_t b = ptr[v], e = ptr[v + 1];
  T* dst = rows + v * row_len;
  if (e == b) {
    for (int64_t i = lane; i < row_len; i += kWave) dst[i] = T(0);
    return;
  }
  int64_t first_a, first_b;
  const int64_t ka = range_of_position(wave_pos, n_waves, per_wave, n_rows, b, lane, &first_a);
  const int64_t kb = range_of_position(wave_pos, n_waves, per_wave, n_rows, e - 1, lane, &first_b);
  if (ka == kb) return;  // written in full by wavefront ka
  const int slot_a = (b == first_a) ? 0 : 1;
  // 16 bytes per lane and three groups of lanes' worth in flight: a row of 9 x 64 floats is one round trip
  constexpr int N = 16 / sizeof(T);
  const bool wide = row_len % N == 0 && ((reinterpret_cast<uintptr_t>(rows) | reinterpret_cast<uintptr_t>(ws)) & 15) == 0;
  if (wide) {
    constexpr int U = 3;
    for (int64_t i0 = (int64_t)lane * N; i0 < row_len; i0 += (int64_t)U * kWave * N) {
      T s[U][N];
      const T* src = ws + (ka * 2 + slot_a) * row_len;
      for (int64_t k = ka;;) {           // all loads of a partial row are issued before any is added
        T t[U][N];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int64_t i = i0 + (int64_t)u * kWave * N;
          load_vec<T, N>(t[u], src + (i < row_len ? i : i0));
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int n = 0; n < N; ++n) s[u][n] = k == ka ? t[u][n] : s[u][n] + t[u][n];
        if (++k > kb) break;
        src = ws + (k * 2) * row_len;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t i = i0 + (int64_t)u * kWave * N;
        if (i < row_len) store_vec<T, N>(dst + i, s[u]);
      }
    }
    return;
  }
  for (int64_t i = lane; i < row_len; i += kWave) {
    T s = ws[(ka * 2 + slot_a) * row_len + i];
    for (int64_t k = ka + 1; k <= kb; ++k) s += ws[(k * 2) * row_len + i];
    dst[i] = s;
  }
}

// ---- host side ----------------------------------------------------------------------------------------------
struct UvuPlan {
  int V, lpe_log2, pos_per_wave;
  int big_idx;        // >= 0: entry of the block-wise kernels that runs this launch
  int64_t n_waves;    // wavefronts of the main kernel
  int64_t ws_elems;   // segment mode: elements of partial rows at the start of the workspace
  int64_t wsw_elems;  // elements of shared-weight-gradient partials after them
};

template <typename T>
using FwdFn = void (*)(const UvuDev<T>);
template <typename T>
using WaveFn = void (*)(const UvuDev<T>, int64_t);

template <typename T>
struct UvuEntry {
  uint64_t fingerprint;
  uint64_t fingerprint_rounded[2];  // of the table rounded to bf16 / fp16 (a module converted to that type)
  int dims[5];
  const char* name;
  const float* coef;               // the compiled table, table order
  const unsigned char (*idx)[4];   // (M, M1, M2, p) per entry
  int v_fwd, v_bwd;         // channels per lane of the vector paths
  FwdFn<T> fwd[2];          // [vector path]
  WaveFn<T> bwd[2][3];      // [vector path][weight-gradient mode]
  WaveFn<T> seg_fwd[2];     // [vector path]
  WaveFn<T> seg_bwd[2][3];  // [vector path][weight-gradient mode]
  int sh_lmax;              // >= 0: the second operand is laid out like harmonics of degrees 0..sh_lmax, and
  WaveFn<T> seg_fwd_vec[2]; // the segment kernels exist in a form that evaluates them from edge vectors
  WaveFn<T> seg_bwd_vec[2][3];
};

// Channels per lane of the vector path: the widest 16-byte-or-narrower vector whose per-lane register arrays
// (inputs, weights, accumulators; two registers per double) leave room for at least two wavefronts per SIMD.
template <typename T>
constexpr int pick_v(int rows, int scalars, int budget) {
  const int regs = sizeof(T) / 4;
  for (int v = 16 / (int)sizeof(T); v > 1; v /= 2)
    if ((rows * v + scalars) * regs <= budget) return v;
  return 1;
}
template <class TP, typename T>
constexpr int v_fwd() { return pick_v<T>(TP::D1 + TP::P + TP::DO, TP::D2, 150); }
template <class TP, typename T>
constexpr int v_bwd() { return pick_v<T>(2 * TP::D1 + TP::DO + 2 * TP::P, 2 * TP::D2, 236); }

template <class TP, typename T, bool PS>
static UvuEntry<T> make_entry() {
  constexpr int VF = v_fwd<TP, T>(), VB = v_bwd<TP, T>();
  UvuEntry<T> e;
  e.fingerprint = TP::FINGERPRINT;
  e.fingerprint_rounded[0] = TP::FINGERPRINT_BF16; e.fingerprint_rounded[1] = TP::FINGERPRINT_F16;
  e.dims[0] = TP::D1; e.dims[1] = TP::D2; e.dims[2] = TP::DO; e.dims[3] = TP::P; e.dims[4] = TP::NNZ;
  e.name = TP::NAME;
  e.coef = TP::COEF; e.idx = TP::IDX;
  e.v_fwd = VF; e.v_bwd = VB;
  e.fwd[0] = uvu_fwd_kernel<TP, T, 1, PS>;
  e.fwd[1] = uvu_fwd_kernel<TP, T, VF, PS>;
  e.bwd[0][0] = uvu_bwd_kernel<TP, T, 1, kGwNone, PS>;
  e.bwd[0][1] = uvu_bwd_kernel<TP, T, 1, kGwStore, PS>;
  e.bwd[0][2] = uvu_bwd_kernel<TP, T, 1, kGwReduce, PS>;
  e.bwd[1][0] = uvu_bwd_kernel<TP, T, VB, kGwNone, PS>;
  e.bwd[1][1] = uvu_bwd_kernel<TP, T, VB, kGwStore, PS>;
  e.bwd[1][2] = uvu_bwd_kernel<TP, T, VB, kGwReduce, PS>;
  e.seg_fwd[0] = uvu_seg_fwd_kernel<TP, T, 1, PS>;
  e.seg_fwd[1] = uvu_seg_fwd_kernel<TP, T, VF, PS>;
  e.seg_bwd[0][0] = uvu_seg_bwd_kernel<TP, T, 1, kGwNone, PS>;
  e.seg_bwd[0][1] = uvu_seg_bwd_kernel<TP, T, 1, kGwStore, PS>;
  e.seg_bwd[0][2] = uvu_seg_bwd_kernel<TP, T, 1, kGwReduce, PS>;
  e.seg_bwd[1][0] = uvu_seg_bwd_kernel<TP, T, VB, kGwNone, PS>;
  e.seg_bwd[1][1] = uvu_seg_bwd_kernel<TP, T, VB, kGwStore, PS>;
  e.seg_bwd[1][2] = uvu_seg_bwd_kernel<TP, T, VB, kGwReduce, PS>;
  e.sh_lmax = TP::SH_LMAX;
  if constexpr (TP::SH_LMAX >= 0) {
    static_assert((TP::SH_LMAX + 1) * (TP::SH_LMAX + 1) == TP::D2, "harmonics layout");
    e.seg_fwd_vec[0] = uvu_seg_fwd_kernel<TP, T, 1, PS, true>;
    e.seg_fwd_vec[1] = uvu_seg_fwd_kernel<TP, T, VF, PS, true>;
    e.seg_bwd_vec[0][0] = uvu_seg_bwd_kernel<TP, T, 1, kGwNone, PS, true>;
    e.seg_bwd_vec[0][1] = uvu_seg_bwd_kernel<TP, T, 1, kGwStore, PS, true>;
    e.seg_bwd_vec[0][2] = uvu_seg_bwd_kernel<TP, T, 1, kGwReduce, PS, true>;
    e.seg_bwd_vec[1][0] = uvu_seg_bwd_kernel<TP, T, VB, kGwNone, PS, true>;
    e.seg_bwd_vec[1][1] = uvu_seg_bwd_kernel<TP, T, VB, kGwStore, PS, true>;
    e.seg_bwd_vec[1][2] = uvu_seg_bwd_kernel<TP, T, VB, kGwReduce, PS, true>;
  } else {
    for (auto& f : e.seg_fwd_vec) f = nullptr;
    for (auto& r : e.seg_bwd_vec)
      for (auto& f : r) f = nullptr;
  }
  return e;
}

// The kernels exist twice: as they are for a table equal to the compiled one, and with one factor per weight path
// applied to the weights and their gradient (PS).  The second set is instantiated in its own translation unit
// (uvu_kernels_ps.hip includes this file with CGTP_UVU_PS_UNIT defined) so that both compile side by side.
template <typename T, bool PS>
static const UvuEntry<T>* make_entries(int* count) {
#define CGTP_X(TP) make_entry<TP, T, PS>(),
  static const UvuEntry<T> table[] = {CGTP_FOREACH_UVU_CONFIG(CGTP_X)};
#undef CGTP_X
  *count = (int)(sizeof(table) / sizeof(table[0]));
  return table;
}
const UvuEntry<float>* uvu_entries_scaled_f32(int* count);
const UvuEntry<double>* uvu_entries_scaled_f64(int* count);

#if defined(CGTP_UVU_PS_UNIT)
const UvuEntry<float>* uvu_entries_scaled_f32(int* count) { return make_entries<float, true>(count); }
const UvuEntry<double>* uvu_entries_scaled_f64(int* count) { return make_entries<double, true>(count); }
}  // namespace cgtp
#elif defined(CGTP_UVU_RADIAL_UNIT)
}  // namespace cgtp
#else
template <typename T>
static const UvuEntry<T>* entries(int* count) { return make_entries<T, false>(count); }
template <typename T>
static const UvuEntry<T>* entries_scaled(int* count);
template <>
const UvuEntry<float>* entries_scaled<float>(int* count) { return uvu_entries_scaled_f32(count); }
template <>
const UvuEntry<double>* entries_scaled<double>(int* count) { return uvu_entries_scaled_f64(count); }

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static constexpr int64_t kMaxRowWaves = 2048;
static constexpr int kDefaultPosPerWave = 32;

static int uvu_plan(const cgtp_uvu_args* a, int backward, bool need_ws, UvuPlan* plan) {
  if (!a) return CGTP_ERR_NULL;
  int n_cfg = 0, n_big = 0;
  const UvuEntry<float>* tab = entries<float>(&n_cfg);
  const UvuBigEntry* big_tab = uvu_big_entries(&n_big);
  if (a->cfg < 0 || a->cfg >= n_cfg + n_big) return CGTP_ERR_CONFIG;
  const bool seg_mode = a->n_seg > 0;
  // The block-wise kernels (one channel per lane) serve the configurations that have no register-resident body
  // (indices n_cfg and up) and, because they are faster there, every fp32 row-mode launch of the others.
  int big_idx = a->cfg >= n_cfg ? a->cfg - n_cfg : -1;
  if (big_idx < 0 && a->dtype == CGTP_F32 && !seg_mode) {
    for (int i = 0; i < n_big; ++i)
      if (big_tab[i].fingerprint == tab[a->cfg].fingerprint) big_idx = i;
  }
  if (a->y_channels) {  // channelled second operand: block-wise kernels only (fp32, row mode, one wavefront wide)
    if (seg_mode || a->y_vec) return CGTP_ERR_SHAPE;
    if (a->dtype != CGTP_F32) return CGTP_ERR_DTYPE;
    if (a->cfg < n_cfg) {
      big_idx = -1;
      for (int i = 0; i < n_big; ++i)
        if (big_tab[i].fingerprint == tab[a->cfg].fingerprint) big_idx = i;
    }
    if (big_idx < 0) return CGTP_ERR_CONFIG;
  }
  const bool big = big_idx >= 0;
  plan->big_idx = big_idx;
  const int* dims = big ? big_tab[big_idx].dims : tab[a->cfg].dims;
  if (a->dtype != CGTP_F32 && a->dtype != CGTP_F64) return CGTP_ERR_DTYPE;
  if (a->cfg >= n_cfg && a->dtype != CGTP_F32) return CGTP_ERR_DTYPE;
  if (a->C <= 0 || a->n_rows < 0 || a->n_seg < 0 || a->n_x_rows < 0 || a->pos_per_wave < 0) return CGTP_ERR_SHAPE;
  if (!a->x || !a->y || (!a->w && !a->radial_h)) return CGTP_ERR_NULL;
  const bool seg = a->n_seg > 0;
  if (a->radial_h) {   // weights produced in the kernel
    int n_rad = 0;
    const UvuRadialEntry* rad = uvu_radial_entries(&n_rad);
    if (big || a->cfg >= n_rad || !rad[a->cfg].fwd[0]) return CGTP_ERR_CONFIG;
    if (a->y_vec && !rad[a->cfg].fwd[1]) return CGTP_ERR_CONFIG;
    if (a->dtype != CGTP_F32) return CGTP_ERR_DTYPE;
    if (!seg || a->w_shared || a->path_scale || a->C != kRadialC) return CGTP_ERR_SHAPE;
    if (a->radial_r < 4 || a->radial_r > kRadialMaxR || a->radial_r % 4) return CGTP_ERR_SHAPE;
    if (!a->radial_w) return CGTP_ERR_NULL;
    if ((int64_t)rad[a->cfg].lds_floats_per_r * a->radial_r * 4 > kLdsBytes) return CGTP_ERR_LDS;
    if (!aligned16(a->radial_h) || !aligned16(a->radial_w)) return CGTP_ERR_ALIGN;
  }
  if (big && seg) {
    // block-wise kernels in segment mode: ranges by position only, harmonics given, per-edge weights (or no weight
    // gradient), rows no wider than one wavefront
    if (a->wave_seg || a->wave_pos || a->y_vec || a->y_channels) return CGTP_ERR_SHAPE;
    if (backward && a->w_shared && a->grad_w) return CGTP_ERR_SHAPE;
    if (a->C > kWave) return CGTP_ERR_SHAPE;
  }
  if (seg && (!a->ptr || !a->seg_ids || !a->gather)) return CGTP_ERR_NULL;
  if (!seg && (a->ptr || a->perm || a->seg_ids)) return CGTP_ERR_SHAPE;
  if (seg && (a->n_seg >= (int64_t)1 << 31 || a->n_rows >= (int64_t)1 << 31 || a->n_x_rows >= (int64_t)1 << 31))
    return CGTP_ERR_SHAPE;  // segment mode keeps ids and rows in 32-bit registers
  if (seg && (a->wave_seg || a->wave_pos) && a->n_waves <= 0) return CGTP_ERR_SHAPE;
  if (seg && a->wave_seg && a->wave_pos) return CGTP_ERR_SHAPE;
  if (a->y_vec) {  // harmonics evaluated in the kernel: fused segment kernels of a config laid out for them
    if (a->y_vec != kYUnitVector && a->y_vec != kYRawVector) return CGTP_ERR_SHAPE;
    if (!seg) return CGTP_ERR_SHAPE;
    if (tab[a->cfg].sh_lmax < 0) return CGTP_ERR_CONFIG;
  }
  if (backward) {
    if (!a->grad_out) return CGTP_ERR_NULL;
    if (seg && a->n_x_rows != a->n_seg) return CGTP_ERR_SHAPE;
    if (!seg && !a->x_gather && a->n_x_rows != a->n_rows) return CGTP_ERR_SHAPE;
    if (seg && a->x_gather) return CGTP_ERR_SHAPE;
  } else {
    if (!a->out) return CGTP_ERR_NULL;
    if (!seg && !a->gather && a->n_x_rows != a->n_rows) return CGTP_ERR_SHAPE;
  }
  int vw;
  if (big) {
    vw = 1;
  } else if (a->dtype == CGTP_F32) {
    vw = backward ? tab[a->cfg].v_bwd : tab[a->cfg].v_fwd;
  } else {
    int n64 = 0;
    const UvuEntry<double>* tab64 = entries<double>(&n64);
    vw = backward ? tab64[a->cfg].v_bwd : tab64[a->cfg].v_fwd;
  }
  bool vec = vw > 1 && (a->C % vw) == 0 && aligned16(a->x) && (aligned16(a->w) || a->radial_h);
  if (backward) {
    vec = vec && aligned16(a->grad_out) && (!a->grad_x || aligned16(a->grad_x)) &&
          (!a->grad_w || aligned16(a->grad_w));
  } else {
    vec = vec && aligned16(a->out);
  }
  if (a->workspace) vec = vec && aligned16(a->workspace);
  if (a->radial_h && !(vec && vw == 4)) return CGTP_ERR_ALIGN;   // these kernels exist for four channels per lane only
  plan->V = vec ? vw : 1;
  const int lanes = (a->C + plan->V - 1) / plan->V;
  int lg = 0;
  while ((1 << lg) < lanes && lg < 6) ++lg;
  plan->lpe_log2 = lg;
  // channel reduction of grad_y and the segment accumulators stay inside one slot
  // (the block-wise kernels cut wider rows into chunks of one wavefront and sum grad_y over the chunks afterwards)
  if (!big && (backward || seg) && lanes > kWave) return CGTP_ERR_SHAPE;
  const int slots = kWave >> lg;
  const int64_t row_d = backward ? dims[0] : dims[2];
  const bool wred = backward && a->w_shared && a->grad_w;
  plan->ws_elems = plan->wsw_elems = 0;
  plan->pos_per_wave = 0;
  if (seg && a->wave_seg) {
    plan->n_waves = a->n_waves;  // segment-aligned ranges: every row is final, no partial rows
  } else if (seg && a->wave_pos) {
    plan->n_waves = a->n_waves;  // ranges cut at given positions: partial rows as for ranges by position
    if (!backward || a->grad_x) plan->ws_elems = plan->n_waves * 2 * row_d * a->C;
  } else if (seg && big) {
    // one range per slot; by default as many ranges as fill the resident wavefronts once (two per SIMD), but no
    // fewer than 4 positions each.  pos_per_wave here counts the positions of a range.
    int64_t per = a->pos_per_wave > 0 ? a->pos_per_wave : (a->n_rows + kMaxRowWaves * slots - 1) / (kMaxRowWaves * slots);
    if (a->pos_per_wave <= 0 && per < 4) per = 4;
    if (per >= (int64_t)1 << 30) return CGTP_ERR_SHAPE;
    plan->pos_per_wave = (int)per;
    const int64_t n_ranges = (a->n_rows + per - 1) / per;
    plan->n_waves = (n_ranges + slots - 1) / slots;
    if (!backward || a->grad_x) plan->ws_elems = plan->n_waves * slots * 2 * row_d * a->C;
  } else if (seg) {
    int ppw = a->pos_per_wave > 0 ? a->pos_per_wave : kDefaultPosPerWave;
    ppw = ((ppw + slots - 1) / slots) * slots;
    plan->pos_per_wave = ppw;
    plan->n_waves = (a->n_rows + ppw - 1) / ppw;
    if (!backward || a->grad_x) plan->ws_elems = plan->n_waves * 2 * row_d * a->C;
  } else {
    int64_t nw = (a->n_rows + slots - 1) / slots;
    if (wred && !big && nw > kMaxRowWaves) nw = kMaxRowWaves;  // the block-wise kernels take one pass per wavefront
    plan->n_waves = nw;
    // block-wise backward wider than one wavefront: grad_y partials of every channel chunk, summed afterwards
    if (big && backward && a->grad_y && !a->y_channels && a->C > kWave)
      plan->ws_elems = (int64_t)((a->C + kWave - 1) / kWave) * a->n_rows * dims[1];
  }
  if (wred && big) {
    // block-wise kernels write the weight gradient of every row; two summation passes follow (kSumRows rows
    // each, then the partials)
    const int64_t chunks = (a->n_rows + kSumRows - 1) / kSumRows;
    plan->wsw_elems = (a->n_rows + chunks) * dims[3] * a->C;
  } else if (wred) {
    plan->wsw_elems = plan->n_waves * dims[3] * a->C;
  }
  if (need_ws && plan->ws_elems + plan->wsw_elems > 0 && !a->workspace) return CGTP_ERR_WORKSPACE;
  return CGTP_OK;
}

template <typename T>
static UvuDev<T> to_dev(const cgtp_uvu_args* a, const UvuPlan& plan) {
  UvuDev<T> d;
  d.x = (const T*)a->x; d.y = (const T*)a->y; d.w = (const T*)a->w; d.out = (T*)a->out;
  d.g = (const T*)a->grad_out; d.gx = (T*)a->grad_x; d.gy = (T*)a->grad_y; d.gw = (T*)a->grad_w;
  d.ws = (T*)a->workspace;
  d.wsw = d.ws ? d.ws + plan.ws_elems : nullptr;
  d.ptr = a->ptr; d.perm = a->perm; d.gather = a->gather; d.x_gather = a->x_gather; d.seg_ids = a->seg_ids; d.wave_seg = a->wave_seg;
  d.wave_pos = a->wave_pos; d.n_waves = plan.n_waves;
  d.n_rows = a->n_rows; d.n_seg = a->n_seg;
  d.C = a->C; d.lpe_log2 = plan.lpe_log2; d.w_shared = a->w_shared; d.pos_per_wave = plan.pos_per_wave;
  d.y_vec = a->y_vec;
  d.ps = (const T*)a->path_scale;
  d.rh = (const T*)a->radial_h; d.rw = (const T*)a->radial_w; d.R = a->radial_r;
  return d;
}

// Workgroups of a segment-mode launch: 4 wavefronts each, rounded up to whole eighths (see seg_wave_index).
static inline unsigned seg_grid(int64_t n_waves) {
  const int64_t blocks = (n_waves + 3) / 4;
  return (unsigned)(((blocks + 7) / 8) * 8);
}

static inline int launched() { return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH; }

template <typename T>
static int launch_fixup(T* rows, const UvuDev<T>& d, int64_t row_len, hipStream_t stream) {
  hipLaunchKernelGGL(uvu_fixup_kernel<T>, dim3((unsigned)((d.n_seg + 3) / 4)), dim3(256), 0, stream, rows,
                     (const T*)d.ws, d.ptr, d.n_seg, row_len, d.pos_per_wave, d.wave_pos, d.n_waves, d.n_rows);
  return launched();
}

int uvu_fixup_rows_f32(float* rows, const float* ws, const int64_t* ptr, int64_t n_seg, int64_t row_len, int per_range,
                       int64_t n_ranges, int64_t n_rows, hipStream_t stream) {
  hipLaunchKernelGGL(uvu_fixup_kernel<float>, dim3((unsigned)((n_seg + 3) / 4)), dim3(256), 0, stream, rows, ws, ptr,
                     n_seg, row_len, per_range, (const int64_t*)nullptr, n_ranges, n_rows);
  return launched();
}

static int launch_big(const cgtp_uvu_args* a, const UvuPlan& plan, int backward, hipStream_t stream) {
  int n_big = 0;
  const UvuBigEntry& e = (a->path_scale ? uvu_big_entries_scaled(&n_big) : uvu_big_entries(&n_big))[plan.big_idx];
  const bool wred = backward && a->w_shared && a->grad_w;
  const int64_t w_elems = (int64_t)e.dims[3] * a->C;
  if (a->n_seg > 0) {   // fused gather / product / segment sum; the fix-up sees one range per slot
    UvuDev<float> d = to_dev<float>(a, plan);
    const int rows = backward ? e.dims[0] : e.dims[2];
    if (plan.n_waves > 0) {
      void (*fn)(const UvuDev<float>, int64_t) = backward ? e.seg_bwd[a->grad_w ? kGwStore : kGwNone] : e.seg_fwd;
      // accumulator rows of the four wavefronts; the backward also stages indices (64 x 3 ints per wavefront) and
      // keeps two ints of state per lane there
      const size_t lds = (size_t)4 * rows * kWave * sizeof(float) + (backward ? (4 * kWave * 3 + 256 * 2) * sizeof(int) : 0);
      if (lds > (size_t)kLdsBytes) return CGTP_ERR_LDS;
      if (lds > 48 * 1024 &&
          hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return CGTP_ERR_LDS;
      hipLaunchKernelGGL(fn, dim3((unsigned)((plan.n_waves + 3) / 4)), dim3(256), lds, stream, d, plan.n_waves);
      if (launched() != CGTP_OK) return CGTP_ERR_LAUNCH;
    }
    float* out_rows = backward ? d.gx : d.out;
    if (!out_rows) return CGTP_OK;
    d.n_waves = plan.n_waves * (kWave >> plan.lpe_log2);
    return launch_fixup<float>(out_rows, d, (int64_t)rows * a->C, stream);   // also zeroes the rows of empty segments
  }
  if (plan.n_waves == 0) {
    if (wred) launch_partial_sum<float>(nullptr, (float*)a->grad_w, 0, w_elems, stream);   // zero partials: writes 0
    return CGTP_OK;
  }
  UvuDev<float> d = to_dev<float>(a, plan);
  if (backward) {
    if (wred) d.gw = d.wsw;  // per-row gradients into the workspace, summed below
    const int chunk = 1 << plan.lpe_log2;
    const int64_t c_chunks = (a->C + chunk - 1) / chunk;
    hipLaunchKernelGGL((a->y_channels ? e.bwd_yc : e.bwd)[a->grad_w ? kGwStore : kGwNone],
                       dim3((unsigned)((plan.n_waves + 3) / 4), (unsigned)c_chunks), dim3(256), 0, stream, d,
                       plan.n_waves);
    if (plan.ws_elems > 0) {  // grad_y: fixed-order sum of the channel chunks' partials
      if (launched() != CGTP_OK) return CGTP_ERR_LAUNCH;
      launch_partial_sum<float>((const float*)d.ws, (float*)a->grad_y, c_chunks, a->n_rows * e.dims[1], stream);
    }
    if (wred) {
      if (launched() != CGTP_OK) return CGTP_ERR_LAUNCH;
      const int64_t chunks = (a->n_rows + kSumRows - 1) / kSumRows;
      float* part = d.wsw + a->n_rows * w_elems;
      launch_rows_sum<float>((const float*)d.wsw, part, a->n_rows, w_elems, stream);
      if (launched() != CGTP_OK) return CGTP_ERR_LAUNCH;
      launch_partial_sum<float>((const float*)part, (float*)a->grad_w, chunks, w_elems, stream);
    }
  } else {
    const int chunk = 1 << plan.lpe_log2;
    dim3 grid((unsigned)((plan.n_waves + 3) / 4), (unsigned)((a->C + chunk - 1) / chunk));
    hipLaunchKernelGGL(a->y_channels ? e.fwd_yc : e.fwd, grid, dim3(256), 0, stream, d);
  }
  return launched();
}

// Segment kernels that produce the weights themselves: the shared matrix lives in LDS.
static int launch_radial(const cgtp_uvu_args* a, const UvuDev<float>& d, const UvuPlan& plan, int backward,
                         hipStream_t stream) {
  int n = 0;
  const UvuRadialEntry& e = uvu_radial_entries(&n)[a->cfg];
  void (*fn)(const UvuDev<float>, int64_t) = backward ? e.bwd[a->y_vec ? 1 : 0][a->grad_w ? 1 : 0] : e.fwd[a->y_vec ? 1 : 0];
  const size_t lds = (size_t)e.lds_floats_per_r * a->radial_r * sizeof(float);
  if (lds > 48 * 1024 &&
      hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return CGTP_ERR_LDS;
  hipLaunchKernelGGL(fn, dim3(seg_grid(plan.n_waves)), dim3(256), lds, stream, d, plan.n_waves);
  return CGTP_OK;
}

template <typename T>
static int launch_fwd(const cgtp_uvu_args* a, const UvuPlan& plan, hipStream_t stream) {
  int n = 0;
  const UvuEntry<T>& e = (a->path_scale ? entries_scaled<T>(&n) : entries<T>(&n))[a->cfg];
  const UvuDev<T> d = to_dev<T>(a, plan);
  const int vi = plan.V > 1;
  if (a->n_seg > 0) {
    if (plan.n_waves > 0) {
      if constexpr (sizeof(T) == 4) {
        if (a->radial_h) {
          const int st = launch_radial(a, d, plan, 0, stream);
          if (st != CGTP_OK) return st;
        } else {
          hipLaunchKernelGGL(a->y_vec ? e.seg_fwd_vec[vi] : e.seg_fwd[vi], dim3(seg_grid(plan.n_waves)), dim3(256), 0,
                             stream, d, plan.n_waves);
        }
      } else {
        hipLaunchKernelGGL(a->y_vec ? e.seg_fwd_vec[vi] : e.seg_fwd[vi], dim3(seg_grid(plan.n_waves)), dim3(256), 0,
                           stream, d, plan.n_waves);
      }
      if (launched() != CGTP_OK) return CGTP_ERR_LAUNCH;
    }
    return a->wave_seg ? CGTP_OK : launch_fixup<T>(d.out, d, (int64_t)e.dims[2] * a->C, stream);
  }
  if (plan.n_waves == 0) return CGTP_OK;
  const int chunk = (1 << plan.lpe_log2) * plan.V;
  dim3 grid((unsigned)((plan.n_waves + 3) / 4), (unsigned)((a->C + chunk - 1) / chunk));
  hipLaunchKernelGGL(e.fwd[vi], grid, dim3(256), 0, stream, d);
  return launched();
}

template <typename T>
static int launch_bwd(const cgtp_uvu_args* a, const UvuPlan& plan, hipStream_t stream) {
  int n = 0;
  const UvuEntry<T>& e = (a->path_scale ? entries_scaled<T>(&n) : entries<T>(&n))[a->cfg];
  const UvuDev<T> d = to_dev<T>(a, plan);
  const int vi = plan.V > 1;
  const bool seg = a->n_seg > 0;
  const bool wred = a->w_shared && a->grad_w;
  const int64_t w_elems = (int64_t)e.dims[3] * a->C;
  if (plan.n_waves == 0) {
    if (wred) launch_partial_sum<T>(nullptr, (T*)a->grad_w, 0, w_elems, stream);   // zero partials: writes 0
  } else {
    const int gwm = !a->grad_w ? kGwNone : (wred ? kGwReduce : kGwStore);
    bool done = false;
    if constexpr (sizeof(T) == 4) {
      if (a->radial_h) {
        const int st = launch_radial(a, d, plan, 1, stream);
        if (st != CGTP_OK) return st;
        done = true;
      }
    }
    if (!done)
      hipLaunchKernelGGL(seg ? (a->y_vec ? e.seg_bwd_vec[vi][gwm] : e.seg_bwd[vi][gwm]) : e.bwd[vi][gwm],
                         dim3(seg ? seg_grid(plan.n_waves) : (unsigned)((plan.n_waves + 3) / 4)), dim3(256), 0, stream, d,
                         plan.n_waves);
    if (launched() != CGTP_OK) return CGTP_ERR_LAUNCH;
    if (wred) {
      launch_partial_sum<T>((const T*)d.wsw, (T*)a->grad_w, plan.n_waves, w_elems, stream);
      if (launched() != CGTP_OK) return CGTP_ERR_LAUNCH;
    }
  }
  if (seg && a->grad_x && !a->wave_seg) return launch_fixup<T>(d.gx, d, (int64_t)e.dims[0] * a->C, stream);
  return CGTP_OK;
}

}  // namespace cgtp

using namespace cgtp;

extern "C" {

int cgtp_uvu_num_configs(void) {
  int n = 0, n_big = 0;
  entries<float>(&n);
  uvu_big_entries(&n_big);
  return n + n_big;
}

int cgtp_uvu_find(uint64_t fingerprint) {
  int n = 0, n_big = 0;
  const UvuEntry<float>* t = entries<float>(&n);
  const UvuBigEntry* b = uvu_big_entries(&n_big);
  for (int i = 0; i < n; ++i)
    if (t[i].fingerprint == fingerprint) return i;
  for (int i = 0; i < n_big; ++i)
    if (b[i].fingerprint == fingerprint) return n + i;
  return -1;
}

int cgtp_uvu_find_rounded(uint64_t fingerprint, int dtype) {
  if (dtype != CGTP_BF16 && dtype != CGTP_F16) return -1;
  const int k = dtype == CGTP_F16;
  int n = 0, n_big = 0;
  const UvuEntry<float>* t = entries<float>(&n);
  const UvuBigEntry* b = uvu_big_entries(&n_big);
  for (int i = 0; i < n; ++i)
    if (t[i].fingerprint_rounded[k] == fingerprint) return i;
  for (int i = 0; i < n_big; ++i)
    if (b[i].fingerprint_rounded[k] == fingerprint) return n + i;
  return -1;
}

uint64_t cgtp_uvu_describe(int cfg, int32_t* dims) {
  int n = 0, n_big = 0;
  const UvuEntry<float>* t = entries<float>(&n);
  const UvuBigEntry* b = uvu_big_entries(&n_big);
  if (cfg < 0 || cfg >= n + n_big) return 0;
  const int* d = cfg < n ? t[cfg].dims : b[cfg - n].dims;
  if (dims)
    for (int i = 0; i < 5; ++i) dims[i] = d[i];
  return cfg < n ? t[cfg].fingerprint : b[cfg - n].fingerprint;
}

int cgtp_uvu_table(int cfg, float* coef, int32_t* idx) {
  int n = 0, n_big = 0;
  const UvuEntry<float>* t = entries<float>(&n);
  const UvuBigEntry* b = uvu_big_entries(&n_big);
  if (cfg < 0 || cfg >= n + n_big) return -1;
  const int nnz = cfg < n ? t[cfg].dims[4] : b[cfg - n].dims[4];
  const float* c = cfg < n ? t[cfg].coef : b[cfg - n].coef;
  const unsigned char (*ix)[4] = cfg < n ? t[cfg].idx : b[cfg - n].idx;
  for (int k = 0; k < nnz; ++k) {
    if (coef) coef[k] = c[k];
    for (int j = 0; idx && j < 4; ++j) idx[4 * k + j] = ix[k][j];
  }
  return nnz;
}

int cgtp_uvu_sh_degree(int cfg) {
  int n = 0;
  const UvuEntry<float>* t = entries<float>(&n);
  return cfg >= 0 && cfg < n ? t[cfg].sh_lmax : -1;
}

int cgtp_uvu_radial_supported(int cfg) {
  int n = 0;
  const UvuRadialEntry* t = uvu_radial_entries(&n);
  return cfg >= 0 && cfg < n && t[cfg].fwd[0] != nullptr;
}

int cgtp_uvu_slots(int cfg, int dtype, int C, int backward) {
  int n = 0, n64 = 0;
  const UvuEntry<float>* t = entries<float>(&n);
  const UvuEntry<double>* t64 = entries<double>(&n64);
  if (cfg < 0 || cfg >= n || C <= 0 || (dtype != CGTP_F32 && dtype != CGTP_F64)) return 0;
  int vw = dtype == CGTP_F32 ? (backward ? t[cfg].v_bwd : t[cfg].v_fwd) : (backward ? t64[cfg].v_bwd : t64[cfg].v_fwd);
  if (C % vw) vw = 1;
  const int lanes = (C + vw - 1) / vw;
  if (lanes > kWave) return 0;
  int lg = 0;
  while ((1 << lg) < lanes) ++lg;
  return kWave >> lg;
}

int cgtp_uvu_blockwise_only(int cfg) {
  int n = 0, n_big = 0;
  entries<float>(&n);
  uvu_big_entries(&n_big);
  return cfg >= n && cfg < n + n_big;
}

int cgtp_uvu_validate(const cgtp_uvu_args* args, int backward) {
  UvuPlan plan;
  return uvu_plan(args, backward, false, &plan);
}

int64_t cgtp_uvu_workspace_bytes(const cgtp_uvu_args* a, int backward) {
  UvuPlan plan;
  if (uvu_plan(a, backward, false, &plan) != CGTP_OK) return 0;
  return (plan.ws_elems + plan.wsw_elems) * (a->dtype == CGTP_F32 ? 4 : 8);
}

int cgtp_uvu_fwd(const cgtp_uvu_args* a, void* stream) {
  UvuPlan plan;
  const int st = uvu_plan(a, 0, true, &plan);
  if (st != CGTP_OK) return st;
  if (plan.big_idx >= 0) return launch_big(a, plan, 0, (hipStream_t)stream);
  return a->dtype == CGTP_F32 ? launch_fwd<float>(a, plan, (hipStream_t)stream)
                              : launch_fwd<double>(a, plan, (hipStream_t)stream);
}

int cgtp_uvu_bwd(const cgtp_uvu_args* a, void* stream) {
  UvuPlan plan;
  const int st = uvu_plan(a, 1, true, &plan);
  if (st != CGTP_OK) return st;
  if (plan.big_idx >= 0) return launch_big(a, plan, 1, (hipStream_t)stream);
  return a->dtype == CGTP_F32 ? launch_bwd<float>(a, plan, (hipStream_t)stream)
                              : launch_bwd<double>(a, plan, (hipStream_t)stream);
}

}  // extern "C"
#endif  // CGTP_UVU_PS_UNIT / CGTP_UVU_RADIAL_UNIT
