// Segment-mode channel-wise tensor product whose per-edge weights are produced inside the kernel:
//   w[e, p, c] = sum_r h[e, r] * W_last[r, p, c]          (R <= 16 features per edge, e.g. a radial embedding)
// instead of being read from a (E, P, C) tensor that another kernel wrote (for the lmax = 2, C = 64 edge workload that
// tensor is 2816 of the 3157 bytes an edge moves in the forward).  fp32, C = 64: a wavefront works on four edges per
// step, 16 lanes x 4 channels each.
//
// The product runs on the matrix cores as 16 independent 4x4 outer products per instruction
// (v_mfma_f32_4x4x1_16b_f32): block b = channels 4 b .. 4 b + 3, row i = channel 4 b + i (operand A: lane 4 b + i
// holds W_last[r, p, lane] — one conflict-free LDS read per (r, p), W_last is staged once per workgroup), column j =
// edge j of the step (operand B: lane 4 b + j holds h[e_j, r]); R instructions accumulate one path's weights of all
// four edges.  The result lane 4 b + j holds channels 4 b .. 4 b + 3 of edge j — exactly what lane 16 j + b of the
// tensor-product code needs, so one cross-lane move per register hands them over.
// The backward forms the weights the same way and writes the weight gradient per edge as before; the gradients of h
// and W_last are contractions of that tensor (over the channels and paths, and over the edges) which one further
// kernel, uvu_radial_grad_kernel below, takes in a single pass over it.
//
// Matrix instructions need every lane: the weights are formed for all four slots of a step before the slots past a
// segment boundary are masked off for the tensor-product body.
#define CGTP_UVU_RADIAL_UNIT
#include "uvu_kernels.hip"

namespace cgtp {

typedef float floatx4 __attribute__((ext_vector_type(4)));

// smallest stride >= pc that is 1 modulo the 32 LDS banks
constexpr int radial_stride(int pc) { return (pc + 30) / 32 * 32 + 1; }

template <class TP>
__device__ __forceinline__ void radial_stage(float* lds, const float* __restrict__ rw, int R) {
  constexpr int PC = TP::P * kRadialC, S = radial_stride(PC);
  for (int i = threadIdx.x; i < R * PC; i += blockDim.x) {
    const int r = i / PC;
    lds[r * S + (i - r * PC)] = rw[i];
  }
}

// Weights of this lane's edge and channels (lane 16 s + cl: edge of slot s, channels 4 cl .. 4 cl + 3) for all paths.
// ej: edge of slot (lane & 3), the column this lane supplies to the matrix instructions.  Every lane of the wavefront
// must call this (matrix instructions and cross-lane moves).
template <class TP>
__device__ __forceinline__ void radial_weights(const float* lds, const float* __restrict__ rh, int R, int64_t ej, int lane,
                                               float (&w)[TP::P][4]) {
  constexpr int P = TP::P, S = radial_stride(P * kRadialC);
  const float* hrow = rh + ej * R;
  floatx4 hq[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) hq[q] = *reinterpret_cast<const floatx4*>(hrow + (4 * q < R ? 4 * q : 0));
  // all paths side by side: P independent chains of matrix instructions keep the pipeline full
  floatx4 acc[P];
#pragma unroll
  for (int p = 0; p < P; ++p) acc[p] = floatx4{0.f, 0.f, 0.f, 0.f};
  const float* col = lds + lane;
  for (int q = 0; 4 * q < R; ++q) {
    const floatx4 hv = q == 0 ? hq[0] : q == 1 ? hq[1] : q == 2 ? hq[2] : hq[3];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int p = 0; p < P; ++p)
        acc[p] = __builtin_amdgcn_mfma_f32_4x4x1f32(col[(4 * q + i) * S + p * kRadialC], hv[i], acc[p], 0, 0, 0);
  }
  const int src = 4 * (lane & 15) + (lane >> 4);   // result lane 4 b + j holds channels 4 b .. 4 b + 3 of edge j
#pragma unroll
  for (int p = 0; p < P; ++p)
#pragma unroll
    for (int v = 0; v < 4; ++v) w[p][v] = __shfl(acc[p][v], src, kWave);
}

template <class TP, bool YV>
__global__ void __launch_bounds__(256) uvu_seg_fwd_radial_kernel(const UvuDev<float> a, int64_t n_waves) {
  using T = float;
  constexpr int V = 4, D1 = TP::D1, D2 = TP::D2, DO = TP::DO, P = TP::P;
  extern __shared__ __align__(16) float rw_lds[];
  radial_stage<TP>(rw_lds, a.rw, a.R);
  __syncthreads();
  const Lanes L(4);
  const int64_t wave = seg_wave_index(n_waves);
  if (wave < 0) return;
  const int c0 = L.cl * V;
  constexpr int64_t C = kRadialC;
  const SegRange R(a.seg_ids, a.ptr, a.wave_seg, a.wave_pos, wave, a.pos_per_wave, a.n_rows);

  T acc[DO][V];
  zero_rows(acc);
  SegStep st;
  st.next_row = R.s0;
  for (int64_t cb = R.p0; cb < R.p1; cb += kWave) {
  const SegIndexRegs I(a.seg_ids, a.perm, a.gather, cb, cb + kWave < R.p1 ? cb + kWave : R.p1, L.lane);
  for (int off0 = 0; off0 < I.npos;) {
    int ei, oi;
    const bool valid = seg_step_begin<T, DO, V>(st, acc, a.out, a.ws, I, off0, ei, oi, wave, R, L, 4, true, C, c0);
    // the edge's operands are requested first: the gathers are in flight while the weights are formed
    T x[D1][V], y[D2], yv[3];
    if (valid) {
      const int64_t e = ei, xr = oi;
      if constexpr (YV) {
#pragma unroll
        for (int j = 0; j < 3; ++j) yv[j] = a.y[e * 3 + j];
      } else {
#pragma unroll
        for (int j = 0; j < D2; ++j) y[j] = a.y[e * D2 + j];
      }
#pragma unroll
      for (int i = 0; i < D1; ++i) load_vec<T, V>(x[i], a.x + (xr * D1 + i) * C + c0);
    }
    // slots past the segment boundary carry the position the step started at: their weights are formed and dropped
    T w[P][V];
    radial_weights<TP>(rw_lds, a.rh, a.R, __shfl(ei, (L.lane & 3) << 4, kWave), L.lane, w);
    if (valid) {
      if constexpr (YV) {
        const ShPoint<T> pt(yv[0], yv[1], yv[2], a.y_vec == kYUnitVector);
        sh_values<T, TP::SH_LMAX>(pt.x, pt.y, pt.z, y);
      }
      TP::template fwd<T, V>(x, y, [&](int p, T (&wp)[V]) {
#pragma unroll
        for (int v = 0; v < V; ++v) wp[v] = w[p][v];
      }, acc);
    }
  }
  }
  seg_finish<T, DO, V>(st, acc, a.out, a.ws, wave, R, L, true, C, c0);
}

template <class TP, bool YV, int GW>
__global__ void __launch_bounds__(256, 2) uvu_seg_bwd_radial_kernel(const UvuDev<float> a, int64_t n_waves) {
  using T = float;
  constexpr int V = 4, D1 = TP::D1, D2 = TP::D2, DO = TP::DO, P = TP::P;
  extern __shared__ __align__(16) float rw_lds[];
  radial_stage<TP>(rw_lds, a.rw, a.R);
  __syncthreads();
  const Lanes L(4);
  const int64_t wave = seg_wave_index(n_waves);
  if (wave < 0) return;
  const int c0 = L.cl * V;
  constexpr int64_t C = kRadialC;
  const SegRange R(a.seg_ids, a.ptr, a.wave_seg, a.wave_pos, wave, a.pos_per_wave, a.n_rows);

  T acc[D1][V];
  zero_rows(acc);
  SegStep st;
  st.next_row = R.s0;
  for (int64_t cb = R.p0; cb < R.p1; cb += kWave) {
  const SegIndexRegs I(a.seg_ids, a.perm, a.gather, cb, cb + kWave < R.p1 ? cb + kWave : R.p1, L.lane);
  for (int off0 = 0; off0 < I.npos;) {
    int ei, oi;
    const bool valid = seg_step_begin<T, D1, V>(st, acc, a.gx, a.ws, I, off0, ei, oi, wave, R, L, 4, true, C, c0);
    T w[P][V];
    radial_weights<TP>(rw_lds, a.rh, a.R, __shfl(ei, (L.lane & 3) << 4, kWave), L.lane, w);
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
#pragma unroll
      for (int m = 0; m < DO; ++m) load_vec<T, V>(g[m], a.g + (gr * DO + m) * C + c0);
      // the segment's rows of x are read again in every step (the plain kernel keeps them in registers over a
      // segment; here the registers go to the weights' production, and the rows hit in the first-level cache)
      T x[D1][V];
#pragma unroll
      for (int i = 0; i < D1; ++i) load_vec<T, V>(x[i], a.x + ((int64_t)st.cur * D1 + i) * C + c0);
      T* gwrow = a.gw + e * P * C + c0;
      TP::template bwd<T, V>(
          x, y, [&](int p, T (&wp)[V]) {
#pragma unroll
        for (int v = 0; v < V; ++v) wp[v] = w[p][v];
      }, g, acc, gy,
          [&](int p, const T (&gwp)[V]) {
            if constexpr (GW == kGwStore) store_vec_stream<T, V>(gwrow + p * C, gwp);
          });
      if (a.gy) {
        if constexpr (YV) {
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
        } else {
          // one component at a time: the halving exchange of the plain kernels needs registers this kernel does not
          // have (its scratch grows from 136 to 396 bytes per lane and the launch from 0.20 to 0.26 ms)
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
  seg_finish<T, D1, V>(st, acc, a.gx, a.ws, wave, R, L, true, C, c0);
}

// ---- gradients of the features and of the shared matrix --------------------------------------------------------
//   grad_h[e, r]    = sum_{p, c} grad_w[e, p, c] * W_last[r, p, c]
//   grad_W[r, p, c] = sum_e h[e, r] * grad_w[e, p, c]
// in one pass over grad_w (E, P, 64), the tensor the backward above wrote.  A workgroup walks tiles of 16 edges, staged
// in LDS (the next tile is requested into registers before this one is multiplied; three workgroups share a compute
// unit and cover each other's waits); wavefront p owns the 64 columns of path p.  Both products run on v_mfma_f32_16x16x4_f32:
//   grad_W^T tile: A = h^T (16 features x 4 edges), B = grad_w (4 edges x 16 columns): one LDS word per lane and step;
//   grad_h tile:   A = W_last (16 features x 4 columns, held in registers for the whole kernel), B = grad_w^T
//                  (4 columns x 16 edges): a lane's four columns of four steps are one 16-byte LDS read.
// The row pitch of the staged tile (P * 64 + 16 words) makes both read patterns conflict-free.  The wavefronts'
// partial grad_h tiles are added through LDS in wavefront order; the workgroups' partial grad_W go to a workspace and
// are added in workgroup order by radial_reduce_kernel.  No atomics.
constexpr int kRgTile = 16;

__global__ void __launch_bounds__(1024) uvu_radial_grad_kernel(const float* __restrict__ gw, const float* __restrict__ h,
                                                              const float* __restrict__ wl, float* __restrict__ gh,
                                                              float* __restrict__ part, int64_t n_rows, int R, int P,
                                                              int tiles_per_group) {
  extern __shared__ __align__(16) float rg_lds[];
  const int PC = P * kRadialC, pitch = PC + 16;
  float* tile = rg_lds;                                     // [16 edges][pitch]
  float* hs = rg_lds + kRgTile * pitch;                     // [16 edges][16 features]
  float* ghs = hs + kRgTile * 16;                           // [P][16 features][16 edges + 1]
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1), r = lane & 15, q = lane >> 4;
  const int nthreads = blockDim.x;
  const int64_t t_begin = (int64_t)blockIdx.x * tiles_per_group;
  const int64_t n_tiles = (n_rows + kRgTile - 1) / kRgTile;
  const int64_t t_end = t_begin + tiles_per_group < n_tiles ? t_begin + tiles_per_group : n_tiles;

  // W_last of this wavefront's path as operand A of the grad_h product: lane (feature r, q) holds columns
  // 16 g + 4 q .. + 3 of the path for g < 4 (rows past R are zero)
  floatx4 wa[4];
#pragma unroll
  for (int g = 0; g < 4; ++g)
    wa[g] = r < R ? *reinterpret_cast<const floatx4*>(wl + (int64_t)r * PC + wave * kRadialC + 16 * g + 4 * q)
                  : floatx4{0.f, 0.f, 0.f, 0.f};
  floatx4 acc[4];   // grad_W^T of this path: tile g = columns 16 g .. + 15; lane (column r, q) holds features 4 q .. + 3
#pragma unroll
  for (int g = 0; g < 4; ++g) acc[g] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int pc4 = PC / 4;
  floatx4 stage[4];
  float hstage = 0.f;
  auto request = [&](int64_t t) __attribute__((always_inline)) {
    const int64_t e0 = t * kRgTile;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int idx = threadIdx.x + k * nthreads, e = idx / pc4, c4 = idx - e * pc4;
      stage[k] = e0 + e < n_rows ? *reinterpret_cast<const floatx4*>(gw + (e0 + e) * PC + c4 * 4) : floatx4{0.f, 0.f, 0.f, 0.f};
    }
    if (threadIdx.x < kRgTile * 16) {
      const int e = threadIdx.x >> 4, f = threadIdx.x & 15;
      hstage = (e0 + e < n_rows && f < R) ? h[(e0 + e) * R + f] : 0.f;
    }
  };
  auto commit = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int idx = threadIdx.x + k * nthreads, e = idx / pc4, c4 = idx - e * pc4;
      *reinterpret_cast<floatx4*>(tile + e * pitch + c4 * 4) = stage[k];
    }
    if (threadIdx.x < kRgTile * 16) hs[threadIdx.x] = hstage;
  };

  if (t_begin < t_end) {
    request(t_begin);
    commit();
  }
  __syncthreads();
  for (int64_t t = t_begin; t < t_end; ++t) {
    if (t + 1 < t_end) request(t + 1);
    const float* tl = tile + wave * kRadialC;
    const float* hl = hs;
    // grad_W^T += grad_w^T h: contraction over the 16 edges, four per step
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const float hv = hl[(4 * ks + q) * 16 + r];            // A: feature r, edge 4 ks + q
#pragma unroll
      for (int g = 0; g < 4; ++g)
        acc[g] = __builtin_amdgcn_mfma_f32_16x16x4f32(hv, tl[(4 * ks + q) * pitch + 16 * g + r], acc[g], 0, 0, 0);
    }
    // grad_h^T (features x edges) of this path's columns: contraction over 64 columns, 16 per group of four steps
    floatx4 gacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const floatx4 b = *reinterpret_cast<const floatx4*>(tl + r * pitch + 16 * g + 4 * q);   // edge r, columns 16 g + 4 q ..
#pragma unroll
      for (int i = 0; i < 4; ++i) gacc = __builtin_amdgcn_mfma_f32_16x16x4f32(wa[g][i], b[i], gacc, 0, 0, 0);
    }
    // lane (edge r, q) holds features 4 q .. + 3 of edge r
#pragma unroll
    for (int i = 0; i < 4; ++i) ghs[(wave * 16 + 4 * q + i) * 17 + r] = gacc[i];
    __syncthreads();
    if (threadIdx.x < kRgTile * 16) {
      const int e = threadIdx.x >> 4, f = threadIdx.x & 15;
      float sum = 0.f;
      for (int w = 0; w < P; ++w) sum += ghs[(w * 16 + f) * 17 + e];
      const int64_t row = t * kRgTile + e;
      if (row < n_rows && f < R) gh[row * R + f] = sum;
    }
    if (t + 1 < t_end) commit();   // every wavefront is past its reads of the tile (barrier above)
    __syncthreads();
  }
  // this workgroup's partial grad_W: part[group][feature][column]
  float* out = part + (int64_t)blockIdx.x * R * PC + wave * kRadialC;
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int f = 4 * q + i;
      if (f < R) out[(int64_t)f * PC + 16 * g + r] = acc[g][i];
    }
}

// out[i] = sum over the groups of part[g][i]: 64 outputs per workgroup, 16 threads per output that each add every
// 16th group in ascending order, then one thread adds the 16 sums in order (a fixed order whatever the launch).
__global__ void __launch_bounds__(1024) radial_reduce_kernel(const float* __restrict__ part, float* __restrict__ out,
                                                             int64_t n_groups, int64_t n) {
  __shared__ float sums[16][64];
  const int o = threadIdx.x & 63, gl = threadIdx.x >> 6;
  const int64_t i = (int64_t)blockIdx.x * 64 + o;
  float s = 0.f;
  if (i < n)
    for (int64_t g = gl; g < n_groups; g += 16) s += part[g * n + i];
  sums[gl][o] = s;
  __syncthreads();
  if (gl == 0 && i < n) {
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < 16; ++k) t += sums[k][o];
    out[i] = t;
  }
}

static int64_t radial_groups(int64_t n_rows) {
  const int64_t n_tiles = (n_rows + kRgTile - 1) / kRgTile;
  return n_tiles < 512 ? (n_tiles > 0 ? n_tiles : 1) : 512;
}

template <class TP>
static UvuRadialEntry make_radial_entry() {
  UvuRadialEntry e;
  e.lds_floats_per_r = radial_stride(TP::P * kRadialC);
  e.fwd[0] = e.fwd[1] = nullptr;
  e.bwd[0][0] = e.bwd[0][1] = e.bwd[1][0] = e.bwd[1][1] = nullptr;
  // only where the plain kernels also keep four channels per lane (the register budget of larger tables does not)
  if constexpr (v_fwd<TP, float>() == 4 && v_bwd<TP, float>() == 4) {
    e.fwd[0] = uvu_seg_fwd_radial_kernel<TP, false>;
    e.bwd[0][0] = uvu_seg_bwd_radial_kernel<TP, false, kGwNone>;
    e.bwd[0][1] = uvu_seg_bwd_radial_kernel<TP, false, kGwStore>;
    if constexpr (TP::SH_LMAX >= 0) {
      e.fwd[1] = uvu_seg_fwd_radial_kernel<TP, true>;
      e.bwd[1][0] = uvu_seg_bwd_radial_kernel<TP, true, kGwNone>;
      e.bwd[1][1] = uvu_seg_bwd_radial_kernel<TP, true, kGwStore>;
    }
  }
  return e;
}

const UvuRadialEntry* uvu_radial_entries(int* count) {
#define CGTP_X(TP) make_radial_entry<TP>(),
  static const UvuRadialEntry table[] = {CGTP_FOREACH_UVU_CONFIG(CGTP_X)};
#undef CGTP_X
  *count = (int)(sizeof(table) / sizeof(table[0]));
  return table;
}

}  // namespace cgtp

using namespace cgtp;

extern "C" {

int64_t cgtp_uvu_radial_grad_workspace_bytes(int64_t n_rows, int32_t radial_r, int32_t n_paths) {
  if (n_rows <= 0 || radial_r <= 0 || n_paths <= 0) return 0;
  return radial_groups(n_rows) * radial_r * n_paths * kRadialC * (int64_t)sizeof(float);
}

int cgtp_uvu_radial_grad(const void* grad_w, const void* radial_h, const void* radial_w, void* grad_radial_h,
                         void* grad_radial_w, void* workspace, int64_t n_rows, int32_t radial_r, int32_t n_paths,
                         int32_t dtype, void* stream) {
  if (dtype != CGTP_F32) return CGTP_ERR_DTYPE;
  if (n_rows < 0 || radial_r <= 0 || radial_r > kRadialMaxR || n_paths < 4 || n_paths > 16) return CGTP_ERR_SHAPE;
  if (!radial_w || !grad_radial_h || !grad_radial_w || (n_rows && (!grad_w || !radial_h))) return CGTP_ERR_NULL;
  if ((reinterpret_cast<uintptr_t>(grad_w) | reinterpret_cast<uintptr_t>(radial_w)) & 15u) return CGTP_ERR_ALIGN;
  const int PC = n_paths * kRadialC;
  const int64_t n_out = (int64_t)radial_r * PC;
  hipStream_t st = (hipStream_t)stream;
  if (n_rows == 0) {
    hipLaunchKernelGGL(radial_reduce_kernel, dim3((unsigned)((n_out + 63) / 64)), dim3(1024), 0, st,
                       (const float*)nullptr, (float*)grad_radial_w, (int64_t)0, n_out);
    return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
  }
  if (!workspace) return CGTP_ERR_WORKSPACE;
  const int64_t groups = radial_groups(n_rows);
  const int64_t n_tiles = (n_rows + kRgTile - 1) / kRgTile;
  const int tiles_per_group = (int)((n_tiles + groups - 1) / groups);
  const size_t lds = ((size_t)kRgTile * (PC + 16) + kRgTile * 16 + (size_t)n_paths * 16 * 17) * sizeof(float);
  if (lds > (size_t)kLdsBytes) return CGTP_ERR_LDS;
  if (lds > 48 * 1024 && hipFuncSetAttribute((const void*)uvu_radial_grad_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                             (int)lds) != hipSuccess)
    return CGTP_ERR_LDS;
  hipLaunchKernelGGL(uvu_radial_grad_kernel, dim3((unsigned)groups), dim3((unsigned)(n_paths * kWave)), lds, st,
                     (const float*)grad_w, (const float*)radial_h, (const float*)radial_w, (float*)grad_radial_h,
                     (float*)workspace, n_rows, (int)radial_r, (int)n_paths, tiles_per_group);
  if (hipGetLastError() != hipSuccess) return CGTP_ERR_LAUNCH;
  hipLaunchKernelGGL(radial_reduce_kernel, dim3((unsigned)((n_out + 63) / 64)), dim3(1024), 0, st,
                     (const float*)workspace, (float*)grad_radial_w, groups, n_out);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

}  // extern "C"
