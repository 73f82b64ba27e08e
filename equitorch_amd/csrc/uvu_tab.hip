// Channel-wise ("uvu") tensor product over an edge list for ANY table, handed over as data: gather at one end,
// product, and segment sum at the other end in one launch, fp32.
//
//   out[v, M, c] = sum_{e in segment v} sum_t coef_t * x[other(e), a_t, c] * y[e, b_t] * w[e, p_t, c]
//
// The table (per entry the rows a, b and flags that close a (path, output row) segment or a path; per segment its
// output row and path) is walked by every wavefront in the same order, four entries at a time, so everything that
// depends on the table alone lives in scalar registers and is read through the scalar cache; what depends on the
// edge lives in LDS, per slot (the group of lanes that handles one edge, V channels per lane):
//   xs  [D1][CP]  the gathered rows of the edge's other end          (CP = lanes per edge x V)
//   ys  [D2]      the edge's second operand
//   cy  [nnz]     coef_t * y[b_t] of every entry, formed 64 entries at a time with lanes over entries
//   acc [DO][CP]  the sums of the open segment
// and per (path, output row) the product accumulates in registers before it is multiplied by the path's weight and
// added to the segment's row (an LDS addition that returns nothing: no round trip on the critical path).  The LDS
// reads of the next four entries and the weight of the next path are requested before the current ones are used.  The sorted edge list is cut into ranges of consecutive positions, one per slot;
// segments that continue in a neighbouring range go through partial rows and the fix-up pass of the compiled-table
// kernels (same layout), so there are no atomics and results do not depend on the launch shape.
//
// The backward walks the list sorted by the other end: a segment is a row of x, its gradient is summed in LDS
// (gxa [D1][CP]); the rows of grad_out are gathered (gs [DO][CP]); grad_y is summed over the channels through
// per-lane partials (gyp [D2][lanes + 1]) and written per edge, the weight gradient per edge and path.
#include "uvu_common.h"

namespace cgtp {

struct TabDev {
  const float* coef;        // (NZ64 + 64) coefficients in walk order (by path, then output row), padding entries 0
  const uint32_t* idx;      // (NZ64 + 64) entry words (see kTabEndSeg), padding entries 0
  const uint32_t* paths;   // (paths in walk order + 2) the weight path of every run of entries, then 0xffff twice
  int nnz, nseg, D1, D2, DO, P;   // NZ64 = nnz rounded up to a multiple of 64
};

// The table is read-only for the whole launch and indexed by values every lane agrees on: through the constant
// address space such reads are scalar loads (one per wavefront, scalar cache) and their results scalar registers.
#define CGTP_CONSTANT __attribute__((address_space(4)))
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
template <typename T>
__device__ __forceinline__ const T CGTP_CONSTANT* as_constant(const T* p) {
  return reinterpret_cast<const T CGTP_CONSTANT*>(reinterpret_cast<uintptr_t>(p));
}
// what one wavefront writes to LDS is visible to its later reads (LDS operations of a wavefront complete in order);
// this only keeps the compiler from moving memory operations across the point
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// Per-slot LDS regions, in floats; every region starts on a 16-byte boundary.
struct TabLayout {
  int CP, D2P, NZP, GYP;      // channels per slot (padded), D2 and nnz rounded up to 4, pitch of a grad_y partial row
  int acc, xs, gs, ys, cy, gyp, slot_floats;
  __host__ __device__ TabLayout(int lpe, int V, int D1, int D2, int DO, int nnz, bool backward) {
    CP = lpe * V;
    D2P = (D2 + 3) & ~3;
    NZP = (nnz + 3) & ~3;
    GYP = lpe + 1;
    const auto up4 = [](int n) { return (n + 3) & ~3; };
    int at = 0;
    acc = at; at += up4((backward ? D1 : DO) * CP);
    xs = at; at += up4(D1 * CP);
    gs = at; at += backward ? up4(DO * CP) : 0;
    ys = at; at += D2P;
    cy = at; at += NZP;
    gyp = at; at += backward ? up4(D2 * GYP) : 0;
    slot_floats = at;
  }
};

template <int V>
__device__ __forceinline__ void lds_load(float (&v)[V], const float* p) {
  if constexpr (V == 4) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  } else {
#pragma unroll
    for (int i = 0; i < V; ++i) v[i] = p[i];
  }
}
template <int V>
__device__ __forceinline__ void lds_store(float* p, const float (&v)[V]) {
  if constexpr (V == 4) {
    *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
  } else {
#pragma unroll
    for (int i = 0; i < V; ++i) p[i] = v[i];
  }
}

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// Range of sorted positions of one slot, and whether its first / last segment lie wholly inside it.
struct TabRange {
  int p0, p1;
  bool first_complete, last_complete;
  __device__ __forceinline__ TabRange(const int64_t* __restrict__ seg_ids, int range, int per_range, int n_rows) {
    const int64_t b = (int64_t)range * per_range;
    p0 = b < n_rows ? (int)b : n_rows;
    p1 = b + per_range < n_rows ? (int)(b + per_range) : n_rows;
    first_complete = p0 >= p1 || p0 == 0 || seg_ids[p0 - 1] != seg_ids[p0];
    last_complete = p0 >= p1 || p1 == n_rows || seg_ids[p1 - 1] != seg_ids[p1];
  }
};
// Segment id, edge and gathered row of the k-th position of a range (past its end: of its last position).
struct TabIndex {
  int sid, edge, other;
  __device__ __forceinline__ TabIndex(const UvuDev<float>& a, const TabRange& R, int k) {
    const int q = R.p0 + k;
    const int qq = q < R.p1 ? q : (R.p1 > R.p0 ? R.p1 - 1 : 0);
    sid = (int)a.seg_ids[qq];
    edge = a.perm ? (int)a.perm[qq] : qq;
    other = (int)a.gather[qq];
  }
};

// Store the slot's D accumulator rows as the row of segment `seg` (or as a partial row of the range) and clear them.
template <int V>
__device__ __forceinline__ void tab_flush(float* __restrict__ acc, int CP, int D, float* __restrict__ rows,
                                          float* __restrict__ ws, int seg, int range, bool first, bool complete,
                                          int64_t C, int c0, bool c_ok) {
  float* dst = (complete ? rows + (int64_t)seg * D * C : ws + ((int64_t)range * 2 + (first ? 0 : 1)) * D * C) + c0;
  const float zero[V] = {};
  for (int m = 0; m < D; ++m) {
    float v[V];
    lds_load<V>(v, acc + m * CP);
    lds_store<V>(acc + m * CP, zero);
    if (c_ok) store_vec<float, V>(dst + m * C, v);
  }
}

// cy[t] = coef_t * y[b_t] for every entry and slot: lanes over entries (the padding entries have coefficient 0).
__device__ __forceinline__ void tab_scale_entries(const TabDev& t, const TabLayout& Y, float* __restrict__ wave_lds,
                                                  int slots, int lane) {
  for (int t0 = lane; t0 < Y.NZP; t0 += 4 * kWave) {     // four entries per lane in flight (the tables are padded)
    float c[4];
    int b[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int tt = min(t0 + u * kWave, Y.NZP - 1);
      c[u] = t.coef[tt];
      b[u] = (t.idx[tt] >> 8) & 255;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int tt = t0 + u * kWave;
      if (tt < Y.NZP) {
        for (int s = 0; s < slots; ++s) {
          float* base = wave_lds + s * Y.slot_floats;
          base[Y.cy + tt] = c[u] * base[Y.ys + b[u]];
        }
      }
    }
  }
}

// p[0..V) += v: read, add, write.  (LDS floating-point additions that return nothing — ds_add_f32 — would spare the
// round trip, but measured three to four times slower per launch here: 1.45 against 0.48 ms forward, 6.3 against 1.4 ms
// backward at 206 coefficients, 65536 edges, 64 channels.)
template <int V>
__device__ __forceinline__ void lds_add(float* p, const float (&v)[V]) {
  float o[V];
  lds_load<V>(o, p);
#pragma unroll
  for (int i = 0; i < V; ++i) o[i] += v[i];
  lds_store<V>(p, o);
}

// Rows of an operand into LDS, sixteen at a time: all loads of a batch are requested before the first is stored (a
// loop of load - store pairs would wait for memory once per row).
template <int V>
__device__ __forceinline__ void tab_stage_rows(float* __restrict__ dst, int CP, const float* __restrict__ src, int64_t C,
                                               int rows, bool zero) {
  constexpr int B = 16;
  for (int i0 = 0; i0 < rows; i0 += B) {
    float v[B][V];
#pragma unroll
    for (int u = 0; u < B; ++u) load_vec<float, V>(v[u], src + (int64_t)min(i0 + u, rows - 1) * C);
#pragma unroll
    for (int u = 0; u < B; ++u) {
      if (zero) {
#pragma unroll
        for (int q = 0; q < V; ++q) v[u][q] = 0.f;
      }
      if (i0 + u < rows) lds_store<V>(dst + (i0 + u) * CP, v[u]);
    }
  }
}

// Entry word: row of x | row of y << 8 | kTabEndSeg | kTabEndPath | output row << 18.
constexpr unsigned kTabEndSeg = 1u << 16, kTabEndPath = 1u << 17;
constexpr int kTabRowShift = 18;

// The entry words of the table, 64 at a time: lane j of the wavefront holds entry 64 * chunk + j (one coalesced load,
// the next chunk requested while this one is walked), and the walk reads an entry with v_readlane into a scalar
// register.  No scalar memory loads in the walk: they share their wait counter with LDS and return out of order, so
// waiting for one means draining every LDS operation in flight.
struct TabWords {
  const uint32_t* words;
  int lane;
  unsigned cur, next;
  __device__ __forceinline__ TabWords(const uint32_t* w, int lane_) : words(w), lane(lane_) {
    cur = words[lane];
    next = words[kWave + lane];
  }
  // entry `i` (>= the first entry of the current chunk, < the end of the next one)
  __device__ __forceinline__ unsigned at(int i) const {
    return (unsigned)__builtin_amdgcn_readlane((int)cur, i & (kWave - 1));
  }
  // call when the walk moves on to entry `i`, a multiple of 64
  __device__ __forceinline__ void turn(int i) {
    cur = next;
    next = words[i + kWave + lane];
  }
};

// The paths in walk order, read one path ahead at the (few) path ends.
struct TabPaths {
  const uint32_t CGTP_CONSTANT* seq;
  int pi;
  int cur, after;
  __device__ __forceinline__ explicit TabPaths(const uint32_t* p) : seq(as_constant(p)), pi(0) {
    cur = uniform((int)seq[0]);
    after = uniform((int)seq[1]);
  }
  __device__ __forceinline__ void advance() {
    ++pi;
    cur = after;
    after = uniform((int)seq[pi + 1]);
  }
};

template <int V>
__global__ void __launch_bounds__(256) uvu_tab_seg_fwd_kernel(const UvuDev<float> a, const TabDev t, int64_t n_waves) {
  extern __shared__ __align__(16) float tab_lds[];
  const Lanes L(a.lpe_log2);
  const int wv = threadIdx.x / kWave;
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + wv;
  if (wave >= n_waves) return;
  const TabLayout Y(L.lpe, V, t.D1, t.D2, t.DO, t.nnz, false);
  float* wave_lds = tab_lds + (int64_t)wv * L.slots * Y.slot_floats;
  float* mine = wave_lds + L.slot * Y.slot_floats;
  float* acc = mine + Y.acc + L.cl * V;
  const float* xs = mine + Y.xs + L.cl * V;
  const float* cy = mine + Y.cy;
  const int CP = Y.CP;
  const float zero[V] = {};
  for (int m = 0; m < t.DO; ++m) lds_store<V>(acc + m * CP, zero);
  const int64_t C = a.C;
  const int c0 = L.cl * V;
  const bool c_ok = c0 < a.C;
  const int cc = c_ok ? c0 : 0;
  const int range = (int)wave * L.slots + L.slot;
  const TabRange R(a.seg_ids, range, a.pos_per_wave, (int)a.n_rows);
  const int nq = Y.NZP >> 2;
  int cur = -1;
  bool first = true;
  TabIndex I(a, R, 0);
  for (int k = 0; k < a.pos_per_wave; ++k) {       // the same trip count in every slot; `live` masks the tail
    const bool live = R.p0 + k < R.p1;
    const int sid = I.sid;
    const int64_t e = I.edge, xr = I.other;
    if (k + 1 < a.pos_per_wave) I = TabIndex(a, R, k + 1);
    if (live && sid != cur) {
      if (cur >= 0) {
        tab_flush<V>(acc, CP, t.DO, a.out, a.ws, cur, range, first, first ? R.first_complete : true, C, c0, c_ok);
        first = false;
      }
      cur = sid;
    }
    // stage the edge's operands
    {
      tab_stage_rows<V>(mine + Y.xs + L.cl * V, CP, a.x + xr * t.D1 * C + cc, C, t.D1, false);
      for (int j = L.cl; j < t.D2; j += L.lpe) mine[Y.ys + j] = a.y[e * t.D2 + j];
    }
    wave_sync();
    tab_scale_entries(t, Y, wave_lds, L.slots, L.lane);
    wave_sync();
    // walk the table four entries at a time; the operands of the next four are requested before these are used
    const float* wrow = a.w + (a.w_shared ? 0 : e) * t.P * C + cc;
    const float keep = live ? 1.f : 0.f;
    TabPaths W(t.paths);
    TabWords T(t.idx, L.lane);
    float w[V], w_after[V], inter[V];
    load_vec<float, V>(w, wrow + W.cur * C);
    load_vec<float, V>(w_after, wrow + min(W.after, t.P - 1) * C);
#pragma unroll
    for (int v = 0; v < V; ++v) inter[v] = 0.f;
    // two sets of registers for the four entries in flight, used in turn (no copies between them)
    unsigned eA[4], eB[4];
    float xA[4][V], xB[4][V];
    f32x4 sA, sB;
#pragma unroll
    for (int j = 0; j < 4; ++j) eA[j] = T.at(j);
    sA = *reinterpret_cast<const f32x4*>(cy);
#pragma unroll
    for (int j = 0; j < 4; ++j) lds_load<V>(xA[j], xs + (int)(eA[j] & 255) * CP);
    auto quad = [&](int q, const unsigned (&ee)[4], const float (&xv)[4][V], const f32x4& s4, unsigned (&en)[4],
                    float (&xn)[4][V], f32x4& sn) __attribute__((always_inline)) {
      const int nx = 4 * (q + 1);               // first entry of the next four (padding past the table)
      if ((nx & (kWave - 1)) == 0) T.turn(nx);
#pragma unroll
      for (int j = 0; j < 4; ++j) en[j] = T.at(nx + j);
      sn = *reinterpret_cast<const f32x4*>(cy + (q + 1 < nq ? nx : 4 * q));
#pragma unroll
      for (int j = 0; j < 4; ++j) lds_load<V>(xn[j], xs + (int)(en[j] & 255) * CP);
      const float ss[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int v = 0; v < V; ++v) inter[v] = fmaf(ss[j], xv[j][v], inter[v]);
        if (ee[j] & kTabEndSeg) {               // the same in every lane: a scalar branch
          float o[V];
#pragma unroll
          for (int v = 0; v < V; ++v) {
            o[v] = w[v] * keep * inter[v];
            inter[v] = 0.f;
          }
          lds_add<V>(acc + (int)((ee[j] >> kTabRowShift) & 255) * CP, o);
          if (ee[j] & kTabEndPath) {
#pragma unroll
            for (int v = 0; v < V; ++v) w[v] = w_after[v];
            W.advance();
            load_vec<float, V>(w_after, wrow + min(W.after, t.P - 1) * C);
          }
        }
      }
    };
    for (int q = 0; q < nq; q += 2) {
      quad(q, eA, xA, sA, eB, xB, sB);
      if (q + 1 < nq) quad(q + 1, eB, xB, sB, eA, xA, sA);
    }
    wave_sync();
  }
  if (cur >= 0)
    tab_flush<V>(acc, CP, t.DO, a.out, a.ws, cur, range, first, (first ? R.first_complete : true) && R.last_complete, C,
                 c0, c_ok);
}

template <int V>
__global__ void __launch_bounds__(256) uvu_tab_seg_bwd_kernel(const UvuDev<float> a, const TabDev t, int64_t n_waves) {
  extern __shared__ __align__(16) float tab_lds[];
  const Lanes L(a.lpe_log2);
  const int wv = threadIdx.x / kWave;
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + wv;
  if (wave >= n_waves) return;
  const TabLayout Y(L.lpe, V, t.D1, t.D2, t.DO, t.nnz, true);
  float* wave_lds = tab_lds + (int64_t)wv * L.slots * Y.slot_floats;
  float* mine = wave_lds + L.slot * Y.slot_floats;
  float* gxa = mine + Y.acc + L.cl * V;
  const float* xs = mine + Y.xs + L.cl * V;
  const float* gs = mine + Y.gs + L.cl * V;
  const float* cy = mine + Y.cy;
  float* gyp = mine + Y.gyp + L.cl;
  const int CP = Y.CP, GYP = Y.GYP;
  const float zero[V] = {};
  for (int i = 0; i < t.D1; ++i) lds_store<V>(gxa + i * CP, zero);
  const int64_t C = a.C;
  const int c0 = L.cl * V;
  const bool c_ok = c0 < a.C;
  const int cc = c_ok ? c0 : 0;
  const int range = (int)wave * L.slots + L.slot;
  const TabRange R(a.seg_ids, range, a.pos_per_wave, (int)a.n_rows);
  const bool want_gx = a.gx != nullptr, want_gy = a.gy != nullptr, want_gw = a.gw != nullptr;
  const int nq = Y.NZP >> 2;
  int cur = -1;
  bool first = true;
  TabIndex I(a, R, 0);
  for (int k = 0; k < a.pos_per_wave; ++k) {
    const bool live = R.p0 + k < R.p1;
    const int sid = I.sid;
    const int64_t e = I.edge, gr = I.other;
    if (k + 1 < a.pos_per_wave) I = TabIndex(a, R, k + 1);
    if (live && sid != cur) {
      if (cur >= 0) {
        if (want_gx)
          tab_flush<V>(gxa, CP, t.D1, a.gx, a.ws, cur, range, first, first ? R.first_complete : true, C, c0, c_ok);
        first = false;
      }
      cur = sid;
    }
    {
      tab_stage_rows<V>(mine + Y.xs + L.cl * V, CP, a.x + (int64_t)sid * t.D1 * C + cc, C, t.D1, false);
      // padding lanes must not count in the channel sums: their rows of grad_out are zero
      tab_stage_rows<V>(mine + Y.gs + L.cl * V, CP, a.g + gr * t.DO * C + cc, C, t.DO, !c_ok);
      for (int j = L.cl; j < t.D2; j += L.lpe) mine[Y.ys + j] = a.y[e * t.D2 + j];
      for (int j = 0; j < t.D2; ++j) gyp[j * GYP] = 0.f;
    }
    wave_sync();
    tab_scale_entries(t, Y, wave_lds, L.slots, L.lane);
    wave_sync();
    const float* wrow = a.w + (a.w_shared ? 0 : e) * t.P * C + cc;
    float* gwrow = a.gw + e * t.P * C + c0;
    const float keep = live ? 1.f : 0.f;
    TabPaths W(t.paths);
    TabWords T(t.idx, L.lane);
    TabWords K(reinterpret_cast<const uint32_t*>(t.coef), L.lane);
    float w[V], w_after[V], gm[V], wg[V], inter[V], gwp[V];
    load_vec<float, V>(w, wrow + W.cur * C);
    load_vec<float, V>(w_after, wrow + min(W.after, t.P - 1) * C);
    unsigned eA[4], eB[4];
    float xA[4][V], xB[4][V];
    f32x4 sA, sB;
#pragma unroll
    for (int j = 0; j < 4; ++j) eA[j] = T.at(j);
    // the output row of the first segment: every entry carries its segment's row
    lds_load<V>(gm, gs + (int)((eA[0] >> kTabRowShift) & 255) * CP);
#pragma unroll
    for (int v = 0; v < V; ++v) {
      wg[v] = w[v] * gm[v];
      inter[v] = 0.f;
      gwp[v] = 0.f;
    }
    sA = *reinterpret_cast<const f32x4*>(cy);
#pragma unroll
    for (int j = 0; j < 4; ++j) lds_load<V>(xA[j], xs + (int)(eA[j] & 255) * CP);
    auto quad = [&](int q, const unsigned (&ee)[4], const float (&xv)[4][V], const f32x4& s4, unsigned (&en)[4],
                    float (&xn)[4][V], f32x4& sn) __attribute__((always_inline)) {
      float cs[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) cs[j] = __builtin_bit_cast(float, K.at(4 * q + j));
      const int nx = 4 * (q + 1);
      if ((nx & (kWave - 1)) == 0) {
        T.turn(nx);
        K.turn(nx);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) en[j] = T.at(nx + j);
      sn = *reinterpret_cast<const f32x4*>(cy + (q + 1 < nq ? nx : 4 * q));
#pragma unroll
      for (int j = 0; j < 4; ++j) lds_load<V>(xn[j], xs + (int)(en[j] & 255) * CP);
      const float ss[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int arow = ee[j] & 255, brow = (ee[j] >> 8) & 255;
#pragma unroll
        for (int v = 0; v < V; ++v) inter[v] = fmaf(ss[j], xv[j][v], inter[v]);
        float gxo[V], gyo = 0.f;
        if (want_gx) lds_load<V>(gxo, gxa + arow * CP);       // both rows requested before either is updated
        if (want_gy) gyo = gyp[brow * GYP];
        if (want_gx) {
          const float sk = ss[j] * keep;
#pragma unroll
          for (int v = 0; v < V; ++v) gxo[v] = fmaf(sk, wg[v], gxo[v]);
          lds_store<V>(gxa + arow * CP, gxo);
        }
        if (want_gy) {
          float d = xv[j][0] * wg[0];
#pragma unroll
          for (int v = 1; v < V; ++v) d = fmaf(xv[j][v], wg[v], d);
          gyp[brow * GYP] = fmaf(cs[j], d, gyo);
        }
        if (ee[j] & kTabEndSeg) {
#pragma unroll
          for (int v = 0; v < V; ++v) {
            gwp[v] = fmaf(inter[v], gm[v], gwp[v]);
            inter[v] = 0.f;
          }
          if (ee[j] & kTabEndPath) {         // this path's weight gradient is complete
            if (want_gw && live && c_ok) store_vec_stream<float, V>(gwrow + W.cur * C, gwp);
#pragma unroll
            for (int v = 0; v < V; ++v) {
              gwp[v] = 0.f;
              w[v] = w_after[v];
            }
            W.advance();
            load_vec<float, V>(w_after, wrow + min(W.after, t.P - 1) * C);
          }
          // the entry after this one opens the next segment (in the padding: row 0)
          const unsigned nxt = j < 3 ? ee[j < 3 ? j + 1 : 3] : en[0];
          lds_load<V>(gm, gs + (int)((nxt >> kTabRowShift) & 255) * CP);
#pragma unroll
          for (int v = 0; v < V; ++v) wg[v] = w[v] * gm[v];
        }
      }
    };
    for (int q = 0; q < nq; q += 2) {
      quad(q, eA, xA, sA, eB, xB, sB);
      if (q + 1 < nq) quad(q + 1, eB, xB, sB, eA, xA, sA);
    }
    wave_sync();
    if (want_gy) {     // lane cl sums the lanes' partials of rows cl, cl + lanes, ...
      for (int j = L.cl; j < t.D2; j += L.lpe) {
        const float* row = mine + Y.gyp + j * GYP;
        float s = row[0];
        for (int q = 1; q < L.lpe; ++q) s += row[q];
        if (live) a.gy[e * t.D2 + j] = s;
      }
    }
    wave_sync();
  }
  if (cur >= 0 && want_gx)
    tab_flush<V>(gxa, CP, t.D1, a.gx, a.ws, cur, range, first, (first ? R.first_complete : true) && R.last_complete, C,
                 c0, c_ok);
}

// ---- host side ------------------------------------------------------------------------------------------------
static inline bool tab_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

struct TabPlan {
  int V, lpe_log2, slots, per, waves_per_group;
  int64_t n_ranges, n_waves, ws_elems;
  size_t lds_bytes;
};

static constexpr int64_t kTabResidentWaves = 2048;
static constexpr int kTabMaxEntries = 8192;
static constexpr int64_t kTabGroupLds = 64 * 1024;     // LDS a workgroup aims to stay under (two or more per CU)

static int tab_plan(const cgtp_uvu_args* a, const cgtp_uvu_tab* t, int backward, TabPlan* plan) {
  if (!a || !t) return CGTP_ERR_NULL;
  if (a->dtype != CGTP_F32) return CGTP_ERR_DTYPE;
  if (!t->coef || !t->idx || !t->paths) return CGTP_ERR_NULL;
  if (t->nnz <= 0 || t->nnz > kTabMaxEntries || t->n_segments <= 0 || t->n_segments > t->nnz) return CGTP_ERR_SHAPE;
  if (t->D1 <= 0 || t->D2 <= 0 || t->DO <= 0 || t->P <= 0 || t->D1 > 255 || t->D2 > 255 || t->DO > 255 || t->P > 65534)
    return CGTP_ERR_SHAPE;
  if (a->C <= 0 || a->n_rows < 0 || a->n_seg <= 0 || a->n_x_rows < 0 || a->pos_per_wave < 0) return CGTP_ERR_SHAPE;
  if (a->n_seg >= (int64_t)1 << 31 || a->n_rows >= (int64_t)1 << 31 || a->n_x_rows >= (int64_t)1 << 31) return CGTP_ERR_SHAPE;
  if (!a->x || !a->y || !a->w || !a->ptr || !a->seg_ids || !a->gather) return CGTP_ERR_NULL;
  if (a->wave_seg || a->wave_pos || a->y_vec || a->y_channels || a->radial_h || a->path_scale || a->x_gather)
    return CGTP_ERR_SHAPE;
  if (backward) {
    if (!a->grad_out) return CGTP_ERR_NULL;
    if (a->n_x_rows != a->n_seg) return CGTP_ERR_SHAPE;
    if (a->w_shared && a->grad_w) return CGTP_ERR_SHAPE;      // a shared weight's gradient is a sum over all edges
  } else if (!a->out) {
    return CGTP_ERR_NULL;
  }
  bool vec = a->C % 4 == 0 && tab_aligned16(a->x) && tab_aligned16(a->w) && (!a->workspace || tab_aligned16(a->workspace));
  if (backward)
    vec = vec && tab_aligned16(a->grad_out) && (!a->grad_x || tab_aligned16(a->grad_x)) &&
          (!a->grad_w || tab_aligned16(a->grad_w));
  else
    vec = vec && tab_aligned16(a->out);
  plan->V = vec ? 4 : 1;
  const int lanes = (a->C + plan->V - 1) / plan->V;
  if (lanes > kWave) return CGTP_ERR_SHAPE;
  int lg = 0;
  while ((1 << lg) < lanes) ++lg;
  plan->lpe_log2 = lg;
  plan->slots = kWave >> lg;
  int64_t per = a->pos_per_wave > 0 ? a->pos_per_wave
                                    : (a->n_rows + kTabResidentWaves * plan->slots - 1) / (kTabResidentWaves * plan->slots);
  if (a->pos_per_wave <= 0 && per < 4) per = 4;
  if (per >= (int64_t)1 << 30) return CGTP_ERR_SHAPE;
  plan->per = (int)per;
  plan->n_ranges = (a->n_rows + per - 1) / per;
  plan->n_waves = (plan->n_ranges + plan->slots - 1) / plan->slots;
  const int64_t row_d = backward ? t->D1 : t->DO;
  plan->ws_elems = (!backward || a->grad_x) ? plan->n_waves * plan->slots * 2 * row_d * a->C : 0;
  const TabLayout Y(1 << lg, plan->V, t->D1, t->D2, t->DO, t->nnz, backward != 0);
  const int64_t wave_bytes = (int64_t)plan->slots * Y.slot_floats * sizeof(float);
  if (wave_bytes > kLdsBytes) return CGTP_ERR_LDS;
  int g = 4;
  while (g > 1 && g * wave_bytes > kTabGroupLds) g >>= 1;
  plan->waves_per_group = g;
  plan->lds_bytes = (size_t)(g * wave_bytes);
  return CGTP_OK;
}

static UvuDev<float> tab_dev(const cgtp_uvu_args* a, const TabPlan& plan) {
  UvuDev<float> d = {};
  d.x = (const float*)a->x; d.y = (const float*)a->y; d.w = (const float*)a->w; d.out = (float*)a->out;
  d.g = (const float*)a->grad_out; d.gx = (float*)a->grad_x; d.gy = (float*)a->grad_y; d.gw = (float*)a->grad_w;
  d.ws = (float*)a->workspace;
  d.ptr = a->ptr; d.perm = a->perm; d.gather = a->gather; d.seg_ids = a->seg_ids;
  d.n_rows = a->n_rows; d.n_seg = a->n_seg; d.n_waves = plan.n_waves;
  d.C = a->C; d.lpe_log2 = plan.lpe_log2; d.w_shared = a->w_shared; d.pos_per_wave = plan.per;
  return d;
}

static int tab_launch(const cgtp_uvu_args* a, const cgtp_uvu_tab* t, int backward, hipStream_t stream) {
  TabPlan plan;
  const int rc = tab_plan(a, t, backward, &plan);
  if (rc != CGTP_OK) return rc;
  if (plan.ws_elems > 0 && !a->workspace) return CGTP_ERR_WORKSPACE;
  const UvuDev<float> d = tab_dev(a, plan);
  const TabDev td = {t->coef, t->idx, t->paths, t->nnz, t->n_segments, t->D1, t->D2, t->DO, t->P};
  if (plan.n_waves > 0) {
    void (*fn)(const UvuDev<float>, const TabDev, int64_t) =
        backward ? (plan.V == 4 ? uvu_tab_seg_bwd_kernel<4> : uvu_tab_seg_bwd_kernel<1>)
                 : (plan.V == 4 ? uvu_tab_seg_fwd_kernel<4> : uvu_tab_seg_fwd_kernel<1>);
    if (plan.lds_bytes > 48 * 1024 &&
        hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)plan.lds_bytes) != hipSuccess)
      return CGTP_ERR_LDS;
    const int64_t groups = (plan.n_waves + plan.waves_per_group - 1) / plan.waves_per_group;
    hipLaunchKernelGGL(fn, dim3((unsigned)groups), dim3((unsigned)(plan.waves_per_group * kWave)), plan.lds_bytes, stream,
                       d, td, plan.n_waves);
    if (hipGetLastError() != hipSuccess) return CGTP_ERR_LAUNCH;
  }
  float* rows = backward ? d.gx : d.out;
  if (!rows) return CGTP_OK;
  // every range is one "wavefront" of the fix-up pass; it also writes the zero rows of empty segments
  return uvu_fixup_rows_f32(rows, d.ws, d.ptr, d.n_seg, (backward ? t->D1 : t->DO) * (int64_t)a->C, plan.per,
                            plan.n_waves * plan.slots, d.n_rows, stream);
}

}  // namespace cgtp

using namespace cgtp;

extern "C" {

int64_t cgtp_uvu_tab_workspace_bytes(const cgtp_uvu_args* a, const cgtp_uvu_tab* t, int backward) {
  TabPlan plan;
  if (tab_plan(a, t, backward, &plan) != CGTP_OK) return -1;
  return plan.ws_elems * (int64_t)sizeof(float);
}

int cgtp_uvu_tab_validate(const cgtp_uvu_args* a, const cgtp_uvu_tab* t, int backward) {
  TabPlan plan;
  return tab_plan(a, t, backward, &plan);
}

int cgtp_uvu_tab_fwd(const cgtp_uvu_args* a, const cgtp_uvu_tab* t, void* stream) {
  return tab_launch(a, t, 0, (hipStream_t)stream);
}

int cgtp_uvu_tab_bwd(const cgtp_uvu_args* a, const cgtp_uvu_tab* t, void* stream) {
  return tab_launch(a, t, 1, (hipStream_t)stream);
}

}  // extern "C"
