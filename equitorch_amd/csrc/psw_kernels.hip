// Fully connected products with a weight PER SAMPLE, any table (handed over as data), fp32 / fp64:
//
//   out[n, M, w] = sum_t coef_t * sum_{u, v} x[n, a_t, u] * y[n, b_t, v] * W[n, p_t, u * V + v, w]
//
// (V = 1 and y (N, D2) for the u1v / 1vu products, y absent for channel mixing between irreps).  Each weight element
// is used once, so the product is a stream over W: the kernels are bound by the HBM rate as long as enough loads are
// in flight, and everything else is arranged around that.
//
// One wavefront handles S samples (S a power of two <= 64 / lanes a weight row needs), all output irreps, all
// paths.  A lane is (sample s, row slice ks, channel group wl): it owns V output channels w of its sample and takes
// every KS-th row k of a weight matrix, so one load instruction of the wavefront reads KS consecutive rows (KS * C_out
// elements, contiguous) of S weight matrices.  The paths are walked output irrep by output irrep ("block": L = 2l+1
// consecutive output rows); per path and chunk of TK rows k the coupled operand
//   t[k][j] = sum_{t in path, M_t = m0 + j} coef_t * x[a_t, u(k)] * y[b_t, v(k)]            (j < L)
// is formed in LDS by all lanes of the sample (table entries read through the scalar cache), then the lanes stream
// their rows of W and accumulate acc[j][w] += t[k][j] * W[k, w] in registers for all L rows of the block at once
// (the row count is a template parameter: 1, 3, 5, 8 or 16 rows per pass).  At the end of a block the KS slices are
// added across lanes and the rows written.  `inter` of the reference's two-launch form never exists in memory.
//
// The backward walks the same way with grad_out[m0 + j][w] of the block in registers:
//   grad_W[k, w] = sum_j t[k][j] * g[j][w]                                  (stored as W is read: streaming)
//   gt[k][j]     = sum_w W[k, w] * g[j][w]                                  (summed over the lanes of a row, to LDS)
// and gt is carried back through the table entries into grad_x / grad_y, which accumulate in LDS over the whole walk
// (lanes own distinct u resp. v, so nothing is added atomically; grad_y of an operand without channels goes through
// per-lane partial rows) and are written once at the end.
#include "cgtp_device.h"
#include "cgtp_host.h"

namespace cgtp {

#define CGTP_CONSTANT __attribute__((address_space(4)))
template <typename T>
__device__ __forceinline__ const T CGTP_CONSTANT* psw_constant(const T* p) {
  return reinterpret_cast<const T CGTP_CONSTANT*>(reinterpret_cast<uintptr_t>(p));
}
// LDS operations of one wavefront complete in order; this only keeps the compiler from moving them across
__device__ __forceinline__ void psw_wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

constexpr unsigned kPswEndRow = 1u << 24;   // entry word: last entry of its (path, output row) run
constexpr unsigned kPswNoTerm = 1u << 25;   // entry word: the path has no term for this row (the row of t is zero)

template <typename T>
struct PswDev {
  const T* x; const T* y; const T* w; T* out;
  const T* g; T* gx; T* gy; T* gw;
  const uint32_t* entries;   // j | a << 8 | b << 16 | kPswEndRow | kPswNoTerm
  const T* coef;
  const int32_t* slots;      // (path, e0, e1) per walked path
  const int32_t* blocks;     // (m0, L, q0, q1) per output irrep
  int64_t N;
  int n_blocks, D1, D2, U, Vy, Wc, P, DO, K;
  int s_log2, lps_log2, TK, JP;
};

// Per-sample LDS regions in elements; every region starts on a 16-byte boundary.
struct PswLayout {
  int xs, ys, t, gt, gxl, gyl, D2P, region;
  __host__ __device__ PswLayout(int D1, int D2, int U, int Vy, int TK, int JP, int LS, bool backward) {
    const auto up4 = [](int n) { return (n + 3) & ~3; };
    D2P = D2 | 1;
    int at = 0;
    xs = at; at += up4(D1 * U);
    ys = at; at += up4(D2 * Vy);
    t = at; at += TK * JP + 16;
    gt = at; at += backward ? TK * JP + 16 : 0;
    gxl = at; at += backward ? up4(D1 * U) : 0;
    gyl = at; at += backward ? up4(Vy == 1 ? LS * D2P : D2 * Vy) : 0;
    region = at;
  }
};

template <typename T, int JB>
__device__ __forceinline__ void psw_read_row(T (&r)[JB], const T* p) {
  constexpr int W = 16 / sizeof(T);
  if constexpr (JB == 1) {
    r[0] = p[0];
  } else {
    using VT = typename VecOf<T, W>::type;
    constexpr int NV = (JB + W - 1) / W;
    VT v[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] = reinterpret_cast<const VT*>(p)[i];
    const T* e = reinterpret_cast<const T*>(v);
#pragma unroll
    for (int j = 0; j < JB; ++j) r[j] = e[j];
  }
}

struct PswLane {
  int lane, LS, li, s, LPS, wl, ks, KS;
  __device__ __forceinline__ PswLane(int s_log2, int lps_log2) {
    lane = threadIdx.x & (kWave - 1);
    LS = kWave >> s_log2;
    li = lane & (LS - 1);
    s = lane >> (6 - s_log2);
    LPS = 1 << lps_log2;
    wl = li & (LPS - 1);
    ks = li >> lps_log2;
    KS = LS >> lps_log2;
  }
};

// t[kc][j] for the TKc rows k0 .. of path entries e0 .. e1; lanes of the sample over kc.
template <typename T>
__device__ __forceinline__ void psw_form_t(const PswDev<T>& a, T* t, const T* xs, const T* ys, int e0, int e1, int k0,
                                           int TKc, const PswLane& L) {
  const auto ent = psw_constant(a.entries);
  const auto cf = psw_constant(a.coef);
  for (int kc = L.li; kc < TKc; kc += L.LS) {
    const int k = k0 + kc;
    const int u = k / a.Vy, v = k - u * a.Vy;
    const T* xu = xs + u;
    const T* yv = ys + v;
    T* row = t + kc * a.JP;
    T val = T(0);
    for (int e = e0; e < e1; ++e) {
      const unsigned wd = ent[e];
      const T c = cf[e];
      if (!(wd & kPswNoTerm)) val = fma(c * xu[(int)((wd >> 8) & 255u) * a.U], yv[(int)((wd >> 16) & 255u) * a.Vy], val);
      if (wd & kPswEndRow) {
        row[wd & 255u] = val;
        val = T(0);
      }
    }
  }
}

// ---- forward --------------------------------------------------------------------------------------------
template <typename T, int V, int JB, int NB>
__device__ __forceinline__ void psw_fwd_block(const PswDev<T>& a, const PswLayout& lay, T* lds, const PswLane& L,
                                              int64_t n, bool sample_ok, int m0, int rows, int j0, int q0, int q1) {
  const auto slots = psw_constant(a.slots);
  const bool lane_ok = sample_ok && L.wl * V < a.Wc;
  const T* xs = lds + lay.xs;
  const T* ys = lds + lay.ys;
  T* t = lds + lay.t;
  T acc[JB][V];
#pragma unroll
  for (int j = 0; j < JB; ++j)
#pragma unroll
    for (int v = 0; v < V; ++v) acc[j][v] = T(0);
  // The walk over (path, chunk of rows, batch of NB rows a lane) is flat: the rows of the next batch are requested
  // before the current ones are used, across chunk and path boundaries, so forming a chunk's t overlaps the loads.
  const auto load_batch = [&](T (&wv)[NB][V], int q, int k0, int kk0) {
    const int p = slots[3 * q];
    const int TKc = a.K - k0 < a.TK ? a.K - k0 : a.TK;
    const T* wrow = a.w + ((n * a.P + p) * (int64_t)a.K + k0) * a.Wc + L.wl * V;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int kk = kk0 + i * L.KS + L.ks;
      if (lane_ok && kk < TKc) {
        load_vec_stream<T, V>(wv[i], wrow + (int64_t)kk * a.Wc);
      } else {
#pragma unroll
        for (int v = 0; v < V; ++v) wv[i][v] = T(0);
      }
    }
  };
  int q = q0, k0 = 0, kk0 = 0;
  T cur[NB][V];
  if (q < q1) load_batch(cur, q, k0, kk0);
  while (q < q1) {
    const int TKc = a.K - k0 < a.TK ? a.K - k0 : a.TK;
    if (kk0 == 0) {
      psw_wave_sync();   // the previous chunk's rows have been read
      psw_form_t(a, t, xs, ys, slots[3 * q + 1], slots[3 * q + 2], k0, TKc, L);
      psw_wave_sync();
    }
    int nq = q, nk0 = k0, nkk0 = kk0 + NB * L.KS;
    if (nkk0 >= TKc) {
      nkk0 = 0;
      nk0 = k0 + a.TK;
      if (nk0 >= a.K) { nk0 = 0; ++nq; }
    }
    T nxt[NB][V];
    if (nq < q1) {
      load_batch(nxt, nq, nk0, nkk0);
    } else {
#pragma unroll
      for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int v = 0; v < V; ++v) nxt[i][v] = T(0);
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int kk = kk0 + i * L.KS + L.ks;
      T tj[JB];
      psw_read_row<T, JB>(tj, t + (kk < TKc ? kk : TKc - 1) * a.JP + j0);
#pragma unroll
      for (int j = 0; j < JB; ++j) fmav<T, V>(acc[j], tj[j], cur[i]);
    }
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int v = 0; v < V; ++v) cur[i][v] = nxt[i][v];
    q = nq; k0 = nk0; kk0 = nkk0;
  }
  // add the row slices: lanes that differ in ks
  for (int off = L.LPS; off < L.LS; off <<= 1) {
    const int addr = (L.lane ^ off) << 2;
    T r[JB][V];
#pragma unroll
    for (int j = 0; j < JB; ++j)
#pragma unroll
      for (int v = 0; v < V; ++v) r[j][v] = lane_exchange(acc[j][v], addr);
#pragma unroll
    for (int j = 0; j < JB; ++j)
#pragma unroll
      for (int v = 0; v < V; ++v) acc[j][v] += r[j][v];
  }
  if (lane_ok && L.ks == 0) {
    T* o = a.out + (n * a.DO + m0 + j0) * (int64_t)a.Wc + L.wl * V;
#pragma unroll
    for (int j = 0; j < JB; ++j)
      if (j < rows) store_vec<T, V>(o + (int64_t)j * a.Wc, acc[j]);
  }
}

template <typename T>
__device__ __forceinline__ void psw_stage(const PswDev<T>& a, const PswLayout& lay, T* lds, const PswLane& L, int64_t n,
                                          bool sample_ok) {
  const int nx = a.D1 * a.U, ny = a.D2 * a.Vy;
  for (int i = L.li; i < nx; i += L.LS) lds[lay.xs + i] = sample_ok ? a.x[n * nx + i] : T(0);
  for (int i = L.li; i < ny; i += L.LS) lds[lay.ys + i] = a.y == nullptr ? T(1) : (sample_ok ? a.y[n * ny + i] : T(0));
}

template <typename T, int V, bool BIG, int NB>
__global__ void __launch_bounds__(kWave) psw_fwd_kernel(const PswDev<T> a) {
  extern __shared__ __align__(16) unsigned char psw_lds_raw[];
  const PswLane L(a.s_log2, a.lps_log2);
  const PswLayout lay(a.D1, a.D2, a.U, a.Vy, a.TK, a.JP, L.LS, false);
  T* lds = reinterpret_cast<T*>(psw_lds_raw) + L.s * lay.region;
  const int64_t n = ((int64_t)blockIdx.x << a.s_log2) + L.s;
  const bool sample_ok = n < a.N;
  psw_stage(a, lay, lds, L, n, sample_ok);
  const auto blocks = psw_constant(a.blocks);
  for (int b = 0; b < a.n_blocks; ++b) {
    const int m0 = blocks[4 * b], rows_all = blocks[4 * b + 1], q0 = blocks[4 * b + 2], q1 = blocks[4 * b + 3];
    for (int j0 = 0; j0 < rows_all;) {
      const int rows = rows_all - j0;
      if (rows <= 1) { psw_fwd_block<T, V, 1, NB>(a, lay, lds, L, n, sample_ok, m0, rows, j0, q0, q1); j0 += 1; }
      else if (rows <= 3) { psw_fwd_block<T, V, 3, NB>(a, lay, lds, L, n, sample_ok, m0, rows, j0, q0, q1); j0 += 3; }
      else if (rows <= 5) { psw_fwd_block<T, V, 5, NB>(a, lay, lds, L, n, sample_ok, m0, rows, j0, q0, q1); j0 += 5; }
      else if (!BIG || rows <= 8) { psw_fwd_block<T, V, 8, NB>(a, lay, lds, L, n, sample_ok, m0, rows, j0, q0, q1); j0 += 8; }
      else if constexpr (BIG) { psw_fwd_block<T, V, 16, NB>(a, lay, lds, L, n, sample_ok, m0, rows, j0, q0, q1); j0 += 16; }
    }
  }
}

// ---- backward -------------------------------------------------------------------------------------------
// gt of the rows j0 .. j0 + JB of one chunk carried back through the entries of the path.
template <typename T>
__device__ __forceinline__ void psw_carry_back(const PswDev<T>& a, const PswLayout& lay, T* lds, const PswLane& L,
                                               int e0, int e1, int k0, int TKc, int j0, int jb) {
  const auto ent = psw_constant(a.entries);
  const auto cf = psw_constant(a.coef);
  const T* xs = lds + lay.xs;
  const T* ys = lds + lay.ys;
  const T* gt = lds + lay.gt;
  T* gxl = lds + lay.gxl;
  T* gyl = lds + lay.gyl;
  const bool want_x = a.gx != nullptr, want_y = a.gy != nullptr;
  if (a.Vy == 1) {
    T* mine = gyl + L.li * lay.D2P;
    for (int kc = L.li; kc < TKc; kc += L.LS) {
      const int u = k0 + kc;
      const T* gr = gt + kc * a.JP;
      for (int e = e0; e < e1; ++e) {
        const unsigned wd = ent[e];
        const int j = (int)(wd & 255u) - j0;
        if (j < 0 || j >= jb || (wd & kPswNoTerm)) continue;
        const int ia = (int)((wd >> 8) & 255u) * a.U + u, ib = (int)((wd >> 16) & 255u);
        const T cg = cf[e] * gr[j + j0];
        if (want_x) gxl[ia] = fma(cg, ys[ib], gxl[ia]);
        if (want_y) mine[ib] = fma(cg, xs[ia], mine[ib]);
      }
    }
    return;
  }
  const int uc = TKc / a.Vy, u0 = k0 / a.Vy;
  if (want_x) {
    for (int ul = L.li; ul < uc; ul += L.LS) {
      const T* gr = gt + (int64_t)ul * a.Vy * a.JP;
      for (int e = e0; e < e1; ++e) {
        const unsigned wd = ent[e];
        const int j = (int)(wd & 255u);
        if (j < j0 || j >= j0 + jb || (wd & kPswNoTerm)) continue;
        const T* yb = ys + (int)((wd >> 16) & 255u) * a.Vy;
        T sum = T(0);
        for (int v = 0; v < a.Vy; ++v) sum = fma(yb[v], gr[v * a.JP + j], sum);
        const int ia = (int)((wd >> 8) & 255u) * a.U + u0 + ul;
        gxl[ia] = fma(cf[e], sum, gxl[ia]);
      }
    }
  }
  if (want_y) {
    for (int v = L.li; v < a.Vy; v += L.LS) {
      const T* gr = gt + v * a.JP;
      for (int e = e0; e < e1; ++e) {
        const unsigned wd = ent[e];
        const int j = (int)(wd & 255u);
        if (j < j0 || j >= j0 + jb || (wd & kPswNoTerm)) continue;
        const T* xa = xs + (int)((wd >> 8) & 255u) * a.U + u0;
        T sum = T(0);
        for (int ul = 0; ul < uc; ++ul) sum = fma(xa[ul], gr[(int64_t)ul * a.Vy * a.JP + j], sum);
        const int ib = (int)((wd >> 16) & 255u) * a.Vy + v;
        gyl[ib] = fma(cf[e], sum, gyl[ib]);
      }
    }
  }
}

template <typename T, int V, int JB, int NB>
__device__ __forceinline__ void psw_bwd_block(const PswDev<T>& a, const PswLayout& lay, T* lds, const PswLane& L,
                                              int64_t n, bool sample_ok, int m0, int rows, int j0, int q0, int q1) {
  const auto slots = psw_constant(a.slots);
  const bool lane_ok = sample_ok && L.wl * V < a.Wc;
  const T* xs = lds + lay.xs;
  const T* ys = lds + lay.ys;
  T* t = lds + lay.t;
  T* gt = lds + lay.gt;
  const bool want_w = a.gw != nullptr, want_t = a.gx != nullptr || a.gy != nullptr;
  const int jb = rows < JB ? rows : JB;
  T gr[JB][V];
  {
    const T* gp = a.g + (n * a.DO + m0 + j0) * (int64_t)a.Wc + L.wl * V;
#pragma unroll
    for (int j = 0; j < JB; ++j) {
      if (lane_ok && j < rows) {
        load_vec<T, V>(gr[j], gp + (int64_t)j * a.Wc);
      } else {
#pragma unroll
        for (int v = 0; v < V; ++v) gr[j][v] = T(0);
      }
    }
  }
  // flat walk as in the forward, NB rows a lane per batch
  const auto load_batch = [&](T (&wv)[NB][V], int q, int k0, int kk0) {
    const int p = slots[3 * q];
    const int TKc = a.K - k0 < a.TK ? a.K - k0 : a.TK;
    const T* wrow = a.w + ((n * a.P + p) * (int64_t)a.K + k0) * a.Wc + L.wl * V;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int kk = kk0 + i * L.KS + L.ks;
      if (want_t && lane_ok && kk < TKc) {
        load_vec_stream<T, V>(wv[i], wrow + (int64_t)kk * a.Wc);
      } else {
#pragma unroll
        for (int v = 0; v < V; ++v) wv[i][v] = T(0);
      }
    }
  };
  int q = q0, k0 = 0, kk0 = 0;
  T cur[NB][V];
  if (q < q1) load_batch(cur, q, k0, kk0);
  while (q < q1) {
    const int p = slots[3 * q], e0 = slots[3 * q + 1], e1 = slots[3 * q + 2];
    const int TKc = a.K - k0 < a.TK ? a.K - k0 : a.TK;
    if (kk0 == 0) {
      psw_wave_sync();   // the previous chunk's t and gt have been read
      if (want_w) psw_form_t(a, t, xs, ys, e0, e1, k0, TKc, L);
      psw_wave_sync();
    }
    int nq = q, nk0 = k0, nkk0 = kk0 + NB * L.KS;
    if (nkk0 >= TKc) {
      nkk0 = 0;
      nk0 = k0 + a.TK;
      if (nk0 >= a.K) { nk0 = 0; ++nq; }
    }
    T nxt[NB][V];
    if (nq < q1) {
      load_batch(nxt, nq, nk0, nkk0);
    } else {
#pragma unroll
      for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int v = 0; v < V; ++v) nxt[i][v] = T(0);
    }
    T* gwrow = want_w ? a.gw + ((n * a.P + p) * (int64_t)a.K + k0) * a.Wc + L.wl * V : nullptr;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int kk = kk0 + i * L.KS + L.ks;
      const bool active = kk < TKc;
      const int row = active ? kk : TKc - 1;
      if (want_w) {
        T tj[JB], o[V];
        psw_read_row<T, JB>(tj, t + row * a.JP + j0);
        mulv<T, V>(o, tj[0], gr[0]);
        // rows past the block's own (a pass holds JB >= rows) were never written in t: whatever the LDS holds there
        // must not reach the sum, not even multiplied by the zero rows of grad_out (it may be NaN)
#pragma unroll
        for (int j = 1; j < JB; ++j) fmav<T, V>(o, j < jb ? tj[j] : T(0), gr[j]);
        if (lane_ok && active) {
          T* dst = gwrow + (int64_t)kk * a.Wc;
          if (j0 > 0) {   // a block wider than one pass: the earlier rows' part is there already
            T old[V];
            load_vec<T, V>(old, dst);
#pragma unroll
            for (int v = 0; v < V; ++v) o[v] += old[v];
          }
          store_vec_stream<T, V>(dst, o);
        }
      }
      if (want_t) {
        T d[JB];
#pragma unroll
        for (int j = 0; j < JB; ++j) d[j] = dotv<T, V>(cur[i], gr[j]);
        T* grow = gt + row * a.JP + j0;
        group_sum_scatter<T, JB>(d, L.LPS, [&](const auto& sums) {
#pragma unroll
          for (int i2 = 0; i2 < array_len(sums); ++i2) {
            const int j = i2 * L.LPS + L.wl;
            if (active && j < jb) grow[j] = sums[i2];
          }
        });
      }
    }
    if (want_t && nkk0 == 0) {   // the chunk's last batch
      psw_wave_sync();
      psw_carry_back(a, lay, lds, L, e0, e1, k0, TKc, j0, jb);
    }
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int v = 0; v < V; ++v) cur[i][v] = nxt[i][v];
    q = nq; k0 = nk0; kk0 = nkk0;
  }
}

template <typename T, int V, bool BIG, int NB>
__global__ void __launch_bounds__(kWave) psw_bwd_kernel(const PswDev<T> a) {
  extern __shared__ __align__(16) unsigned char psw_lds_raw[];
  const PswLane L(a.s_log2, a.lps_log2);
  const PswLayout lay(a.D1, a.D2, a.U, a.Vy, a.TK, a.JP, L.LS, true);
  T* lds = reinterpret_cast<T*>(psw_lds_raw) + L.s * lay.region;
  const int64_t n = ((int64_t)blockIdx.x << a.s_log2) + L.s;
  const bool sample_ok = n < a.N;
  psw_stage(a, lay, lds, L, n, sample_ok);
  const int nx = a.D1 * a.U, ny = a.D2 * a.Vy;
  const int ngy = a.Vy == 1 ? L.LS * lay.D2P : ny;
  for (int i = L.li; i < nx; i += L.LS) lds[lay.gxl + i] = T(0);
  for (int i = L.li; i < ngy; i += L.LS) lds[lay.gyl + i] = T(0);
  const auto blocks = psw_constant(a.blocks);
  for (int b = 0; b < a.n_blocks; ++b) {
    const int m0 = blocks[4 * b], rows_all = blocks[4 * b + 1], q0 = blocks[4 * b + 2], q1 = blocks[4 * b + 3];
    for (int j0 = 0; j0 < rows_all;) {
      const int rows = rows_all - j0;
      if (rows <= 1) { psw_bwd_block<T, V, 1, NB>(a, lay, lds, L, n, sample_ok, m0, rows, j0, q0, q1); j0 += 1; }
      else if (rows <= 3) { psw_bwd_block<T, V, 3, NB>(a, lay, lds, L, n, sample_ok, m0, rows, j0, q0, q1); j0 += 3; }
      else if (rows <= 5) { psw_bwd_block<T, V, 5, NB>(a, lay, lds, L, n, sample_ok, m0, rows, j0, q0, q1); j0 += 5; }
      else if (!BIG || rows <= 8) { psw_bwd_block<T, V, 8, NB>(a, lay, lds, L, n, sample_ok, m0, rows, j0, q0, q1); j0 += 8; }
      else if constexpr (BIG) { psw_bwd_block<T, V, 16, NB>(a, lay, lds, L, n, sample_ok, m0, rows, j0, q0, q1); j0 += 16; }
    }
  }
  psw_wave_sync();
  if (!sample_ok) return;
  if (a.gx != nullptr)
    for (int i = L.li; i < nx; i += L.LS) a.gx[n * nx + i] = lds[lay.gxl + i];
  if (a.gy != nullptr) {
    if (a.Vy == 1) {
      for (int b = L.li; b < a.D2; b += L.LS) {
        T sum = T(0);
        for (int l = 0; l < L.LS; ++l) sum += lds[lay.gyl + l * lay.D2P + b];
        a.gy[n * ny + b] = sum;
      }
    } else {
      for (int i = L.li; i < ny; i += L.LS) a.gy[n * ny + i] = lds[lay.gyl + i];
    }
  }
}

// ---- host -----------------------------------------------------------------------------------------------
struct PswPlan {
  int V, s_log2, lps_log2, TK, JP;
  int64_t lds_bytes, groups;
};

constexpr int64_t kPswMaxLds = 64 * 1024, kPswLdsPerWave = 20 * 1024;

int psw_plan(const cgtp_psw_args* a, const cgtp_psw_table* tab, bool backward, PswPlan* plan) {
  if (a == nullptr || tab == nullptr) return CGTP_ERR_NULL;
  if (a->dtype != CGTP_F32 && a->dtype != CGTP_F64) return CGTP_ERR_DTYPE;
  if (a->n_rows < 0 || a->cx <= 0 || a->cy <= 0 || a->cout <= 0) return CGTP_ERR_SHAPE;
  if (tab->D1 <= 0 || tab->D2 <= 0 || tab->DO <= 0 || tab->D1 > 255 || tab->D2 > 255 || tab->P <= 0 ||
      tab->n_blocks <= 0 || tab->n_slots <= 0 || tab->n_entries <= 0 || tab->max_rows <= 0 || tab->max_rows > 255)
    return CGTP_ERR_SHAPE;
  if (a->y == nullptr && (a->cy != 1 || tab->D2 != 1)) return CGTP_ERR_SHAPE;
  if (a->x == nullptr || a->w == nullptr || tab->entries == nullptr || tab->coef == nullptr || tab->slots == nullptr ||
      tab->blocks == nullptr)
    return CGTP_ERR_NULL;
  if (backward ? a->g == nullptr : a->out == nullptr) return CGTP_ERR_NULL;
  const int es = elem_size(a->dtype), vec = 16 / es;
  const auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const bool wide = a->cout % vec == 0 && aligned(a->w) && (backward ? aligned(a->g) && (a->gw == nullptr || aligned(a->gw))
                                                                      : aligned(a->out));
  plan->V = wide ? vec : 1;
  const int lanes = (a->cout + plan->V - 1) / plan->V;
  if (lanes > kWave) return CGTP_ERR_SHAPE;
  plan->lps_log2 = 0;
  while ((1 << plan->lps_log2) < lanes) ++plan->lps_log2;
  // as many samples per wavefront as leave the GPU sixteen thousand wavefronts or more
  const int s_max_log2 = 6 - plan->lps_log2;
  plan->s_log2 = 0;
  // a batch is four rows a lane: with fewer than 4 x row slices rows in a weight matrix most of its loads would be
  // idle, so short matrices get more samples per wavefront instead of more slices
  const int64_t rows_k = (int64_t)a->cx * a->cy;
  while (plan->s_log2 < s_max_log2 && 4 * (kWave >> (plan->s_log2 + plan->lps_log2)) > (rows_k > 4 ? rows_k : 4))
    ++plan->s_log2;
  while (plan->s_log2 < s_max_log2 && (a->n_rows >> (plan->s_log2 + 1)) >= 16384) ++plan->s_log2;
  const int64_t K = (int64_t)a->cx * a->cy;
  if (K > (1 << 24)) return CGTP_ERR_SHAPE;
  plan->JP = (tab->max_rows + 3) & ~3;
  for (;; --plan->s_log2) {
    const int LS = kWave >> plan->s_log2;
    const int want = LS > 32 ? LS : 32;   // rows of a chunk: every lane of the sample forms at least one
    if (a->cy == 1) {
      plan->TK = want;
    } else {   // whole u: the gradients of the operands are summed per u resp. per v
      const int uc = want / a->cy > 1 ? want / a->cy : 1;
      plan->TK = uc * a->cy;
    }
    if (plan->TK > K) plan->TK = (int)K;
    const PswLayout lay(tab->D1, tab->D2, a->cx, a->cy, plan->TK, plan->JP, LS, backward);
    plan->lds_bytes = (int64_t)lay.region * es << plan->s_log2;
    // fewer samples per wavefront while its LDS share would keep the wavefronts per CU below about eight
    if (plan->s_log2 == 0 || plan->lds_bytes <= kPswLdsPerWave) break;
  }
  if (plan->lds_bytes > kPswMaxLds) return CGTP_ERR_LDS;
  plan->groups = (a->n_rows + (1 << plan->s_log2) - 1) >> plan->s_log2;
  if (plan->groups > 0x7fffffffLL) return CGTP_ERR_SHAPE;
  return CGTP_OK;
}

template <typename T>
int psw_launch_t(const cgtp_psw_args* a, const cgtp_psw_table* tab, bool backward, const PswPlan& plan,
                 hipStream_t stream) {
  PswDev<T> d;
  d.x = (const T*)a->x; d.y = (const T*)a->y; d.w = (const T*)a->w; d.out = (T*)a->out;
  d.g = (const T*)a->g; d.gx = (T*)a->gx; d.gy = (T*)a->gy; d.gw = (T*)a->gw;
  d.entries = tab->entries; d.coef = (const T*)tab->coef; d.slots = tab->slots; d.blocks = tab->blocks;
  d.N = a->n_rows;
  d.n_blocks = tab->n_blocks; d.D1 = tab->D1; d.D2 = tab->D2; d.U = a->cx; d.Vy = a->cy; d.Wc = a->cout;
  d.P = tab->P; d.DO = tab->DO; d.K = a->cx * a->cy;
  d.s_log2 = plan.s_log2; d.lps_log2 = plan.lps_log2; d.TK = plan.TK; d.JP = plan.JP;
  const dim3 grid((unsigned)plan.groups), block(kWave);
  constexpr int VEC = 16 / sizeof(T);
  // blocks of at most 8 rows (l <= 3): kernels without the 16-row pass, which would set their register count
  const bool big = tab->max_rows > 8;
  const auto go = [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, block, plan.lds_bytes, stream, d); };
  if (!backward) {
    // rows of W a lane has in flight per batch: eight when a weight matrix has that many rows per row slice (142
    // registers, three wavefronts per SIMD, 24 rows in flight per SIMD: 0.158 -> 0.137 ms at lmax = 3, 64 -> 64
    // channels), four otherwise (a batch of eight would be half idle) and in the kernels with the 16-row pass
    const bool deep = !big && d.K >= 8 * (kWave >> (plan.s_log2 + plan.lps_log2));
    if (plan.V == 1) big ? go(psw_fwd_kernel<T, 1, true, 4>) : deep ? go(psw_fwd_kernel<T, 1, false, 8>) : go(psw_fwd_kernel<T, 1, false, 4>);
    else big ? go(psw_fwd_kernel<T, VEC, true, 4>) : deep ? go(psw_fwd_kernel<T, VEC, false, 8>) : go(psw_fwd_kernel<T, VEC, false, 4>);
  } else {
    // rows of W a lane has in flight per batch: four when the weights come from HBM (bytes in flight are what the
    // rate follows: 0.50 -> 0.42 ms at 738 MB), two when they fit the 256 MB last-level cache (loads return sooner
    // and the fourth wavefront per SIMD that the smaller batch leaves room for counts more: 0.10 against 0.14 ms at
    // 185 MB) and in the kernels with the 16-row pass (registers)
    const int64_t w_bytes = a->n_rows * (int64_t)tab->P * d.K * d.Wc * (int64_t)sizeof(T);
    const bool deep = !big && w_bytes > (256LL << 20);
    if (plan.V == 1) big ? go(psw_bwd_kernel<T, 1, true, 2>) : deep ? go(psw_bwd_kernel<T, 1, false, 4>) : go(psw_bwd_kernel<T, 1, false, 2>);
    else big ? go(psw_bwd_kernel<T, VEC, true, 2>) : deep ? go(psw_bwd_kernel<T, VEC, false, 4>) : go(psw_bwd_kernel<T, VEC, false, 2>);
  }
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

int psw_launch(const cgtp_psw_args* a, const cgtp_psw_table* tab, bool backward, hipStream_t stream) {
  PswPlan plan;
  const int st = psw_plan(a, tab, backward, &plan);
  if (st != CGTP_OK) return st;
  if (a->n_rows == 0) return CGTP_OK;
  if (backward && a->gx == nullptr && a->gy == nullptr && a->gw == nullptr) return CGTP_OK;
  return a->dtype == CGTP_F32 ? psw_launch_t<float>(a, tab, backward, plan, stream)
                              : psw_launch_t<double>(a, tab, backward, plan, stream);
}

}  // namespace cgtp

extern "C" {

int cgtp_psw_validate(const cgtp_psw_args* a, const cgtp_psw_table* t, int backward) {
  cgtp::PswPlan plan;
  return cgtp::psw_plan(a, t, backward != 0, &plan);
}

int cgtp_psw_fwd(const cgtp_psw_args* a, const cgtp_psw_table* t, void* stream) {
  return cgtp::psw_launch(a, t, false, (hipStream_t)stream);
}

int cgtp_psw_bwd(const cgtp_psw_args* a, const cgtp_psw_table* t, void* stream) {
  return cgtp::psw_launch(a, t, true, (hipStream_t)stream);
}

}  // extern "C"
