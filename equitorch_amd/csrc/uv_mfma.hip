// Fully connected ("uv") Clebsch-Gordan tensor product on the matrix cores, bf16 in / fp32 accumulate / bf16 out:
//
//   out[n, m, w] = sum_t coef_t * y[n, b_t] * sum_u x[n, a_t, u] * W[p_t, u, w]
//
// A workgroup owns 16 samples and stages their whole input rows (DIN x C_in bf16 per sample) in LDS once; each
// of its four wavefronts owns a 32-wide block of output channels.  Per weight path and input row the wavefront
// forms two 16(channels) x 16(samples) accumulator tiles with 2 * C_in/32 MFMAs (v_mfma_f32_16x16x32_bf16: A =
// 16-byte weight fragments held in registers for the whole path, B = 16-byte fragments of the staged input read
// from LDS and shared by both tiles), and then applies the Clebsch-Gordan coefficients as fp32 FMAs between
// accumulator tiles: in the accumulator layout a lane belongs to exactly one sample, so coef * y[n, b] is a
// per-lane scalar.  Output rows are finished one output irrep at a time, which keeps the live accumulators to
// (2l+1) * 8 registers; the whole wavefront fits 256 registers, so two workgroups share a compute unit and one
// stages its input while the other computes.  The staged rows are padded by 16 bytes per sample so that the 16
// lanes of one LDS phase hit distinct banks.
#include "cgtp_device.h"
#include "cgtp_host.h"

// accumulator-tile updates are written as o += s * z; let them contract to FMAs in this file
#pragma clang fp contract(fast)

namespace cgtp {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

// this lane's 8 consecutive k of every K step of one staged input row
template <int KS>
__device__ __forceinline__ void load_b(bf16x8 (&b)[KS], const unsigned char* xs) {
#pragma unroll
  for (int k = 0; k < KS; ++k) {
    b[k] = *reinterpret_cast<const bf16x8*>(xs + k * 64);
  }
}

// Z_t[w, n] = sum_k A_t[w, k] * B[k, n] for the two channel tiles t over KS steps of 32
template <int KS>
__device__ __forceinline__ void mfma_chain(const bf16x8 (&a)[2][KS], const bf16x8 (&b)[KS], floatx4& z0, floatx4& z1) {
  z0 = floatx4{0.f, 0.f, 0.f, 0.f};
  z1 = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int k = 0; k < KS; ++k) {
    z0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[0][k], b[k], z0, 0, 0, 0);
    z1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[1][k], b[k], z1, 0, 0, 0);
  }
}

__device__ __forceinline__ float dot8(const floatx4& g0, const floatx4& g1, const floatx4& z0, const floatx4& z1) {
  float s = g0[0] * z0[0];
  s += g0[1] * z0[1]; s += g0[2] * z0[2]; s += g0[3] * z0[3];
  s += g1[0] * z1[0]; s += g1[1] * z1[1]; s += g1[2] * z1[2]; s += g1[3] * z1[3];
  return s;
}

#include "generated/uv_configs.inc"

constexpr int kUvSamples = 16;


// Stage the 16 samples' rows of one workgroup: 16-byte pieces, coalesced in global memory; every load is issued
// before the first LDS write.  Rows past the end of the batch re-read the last row (their results are never stored).
template <int ROW_BYTES>
__device__ __forceinline__ void uv_stage(const __bf16* __restrict__ x, int64_t n0, int64_t n_rows, unsigned char* smem) {
  constexpr int ROW_PITCH = ROW_BYTES + 16;
  constexpr int PIECES = ROW_BYTES / 16, TOTAL = kUvSamples * PIECES, PER_THREAD = (TOTAL + 255) / 256;
  constexpr int UNROLL = PER_THREAD < 16 ? PER_THREAD : 16;
  for (int base = 0; base < TOTAL; base += 256 * UNROLL) {
    f32x4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int i = min(base + u * 256 + (int)threadIdx.x, TOTAL - 1), s = i / PIECES, c = i % PIECES;
      const int64_t row = min(n0 + s, n_rows - 1);
      v[u] = *reinterpret_cast<const f32x4*>(reinterpret_cast<const unsigned char*>(x) + row * ROW_BYTES + c * 16);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int i = min(base + u * 256 + (int)threadIdx.x, TOTAL - 1), s = i / PIECES, c = i % PIECES;
      *reinterpret_cast<f32x4*>(smem + s * ROW_PITCH + c * 16) = v[u];
    }
  }
}

// Weight fragments of one 32-channel block.  Row r = 4*g + i of channel tile t is output channel blk*32 + 8*g + 4*t
// + i, so that in the accumulator layout (lane (n, q) holds rows 4*q .. 4*q+3 of column n) a lane ends up with 8
// consecutive channels of its sample.  The weights arrive packed in fragment order (uv_pack_kernel): per (path,
// channel block) 2 * KS chunks of 1 KB, chunk t * KS + k holding the 16 bytes of every lane, so that a wavefront's
// load is one contiguous KB.
template <int CIN>
struct UvWeights {
  const __bf16* base;
  int64_t path_stride;
  __device__ __forceinline__ UvWeights(const __bf16* wp, int wblk, int lane, int cout)
      : base(wp + (int64_t)wblk * (2 * (CIN / 32) * 512) + lane * 8), path_stride((int64_t)cout * CIN) {}
  __device__ __forceinline__ void operator()(int p, bf16x8 (&frag)[2][CIN / 32]) const {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int k = 0; k < CIN / 32; ++k)
        frag[t][k] = *reinterpret_cast<const bf16x8*>(base + p * path_stride + (t * (CIN / 32) + k) * 512);
  }
};

template <class CFG, int CIN>
__global__ void __launch_bounds__(256, 2) uv_kernel(const __bf16* __restrict__ x, const __bf16* __restrict__ y,
                                                    const __bf16* __restrict__ wp, __bf16* __restrict__ out,
                                                    int64_t n_rows, int cout) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int DIN = CFG::DIN, DOUT = CFG::DOUT, D2 = CFG::D2;
  constexpr int ROW_BYTES = DIN * CIN * 2;      // one sample's input rows
  constexpr int ROW_PITCH = ROW_BYTES + 16;     // + pad: consecutive samples start 16 B further in the banks
  const int64_t n0 = (int64_t)blockIdx.x * kUvSamples;
  uv_stage<ROW_BYTES>(x, n0, n_rows, smem);
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int n = lane & 15, q = lane >> 4;
  const bool valid = n0 + n < n_rows;
  float yv[D2];
#pragma unroll
  for (int j = 0; j < D2; ++j) yv[j] = (float)y[min(n0 + n, n_rows - 1) * D2 + j];
  const unsigned char* xs = smem + n * ROW_PITCH + q * 16;

  // one 32-channel block per wavefront, blockIdx.y tiles wider outputs
  const int wblk = blockIdx.y * (blockDim.x / kWave) + wave;
  if (wblk * 32 >= cout) return;
  __bf16* orow = out + (n0 + n) * DOUT * cout + wblk * 32 + 8 * q;
  CFG::template run<CIN>(
      xs, UvWeights<CIN>(wp, wblk, lane, cout), yv,
      [&](int row, const floatx4& o0, const floatx4& o1) __attribute__((always_inline)) {
        if (valid) {
          bf16x8 v;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            v[i] = (__bf16)o0[i];
            v[4 + i] = (__bf16)o1[i];
          }
          // written once and not read again by this launch: keep it out of the way of the weights in L2
          __builtin_nontemporal_store(__builtin_bit_cast(f32x4, v), reinterpret_cast<f32x4*>(orow + row * cout));
        }
      });
}

// Gradient w.r.t. the harmonics: gy[n, b] = sum_t coef_t * sum_w g[n, m_t, w] * Z[p_t, a_t][w, n] with the same
// tiles Z as the forward.  Every lane sums over its 8 channels, the four lanes of a sample and the four wavefronts
// (channel blocks) are then added through LDS in a fixed order.  cout <= 128: one workgroup sees all channels.
template <class CFG, int CIN>
__global__ void __launch_bounds__(256, 2) uv_gy_kernel(const __bf16* __restrict__ x, const __bf16* __restrict__ g,
                                                       const __bf16* __restrict__ wp, __bf16* __restrict__ gy,
                                                       int64_t n_rows, int cout) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int DIN = CFG::DIN, DOUT = CFG::DOUT, D2 = CFG::D2;
  constexpr int ROW_BYTES = DIN * CIN * 2, ROW_PITCH = ROW_BYTES + 16;
  const int64_t n0 = (int64_t)blockIdx.x * kUvSamples;
  uv_stage<ROW_BYTES>(x, n0, n_rows, smem);
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int n = lane & 15, q = lane >> 4;
  const unsigned char* xs = smem + n * ROW_PITCH + q * 16;
  const int n_blk = cout / 32;
  float part[D2];
#pragma unroll
  for (int j = 0; j < D2; ++j) part[j] = 0.f;
  if (wave < n_blk) {
    const __bf16* grow = g + min(n0 + n, n_rows - 1) * DOUT * cout + wave * 32 + 8 * q;
    CFG::template run<CIN>(
        xs, UvWeights<CIN>(wp, wave, lane, cout), part,
        [&](int row, floatx4& g0, floatx4& g1) __attribute__((always_inline)) {
          const bf16x8 v = *reinterpret_cast<const bf16x8*>(grow + row * cout);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            g0[i] = (float)v[i];
            g1[i] = (float)v[4 + i];
          }
        });
    // the four lanes of a sample: all values of a stage are exchanged before any is added (one wait per stage
    // instead of one per value); same operands per addition as value-by-value
#pragma unroll
    for (int off = 16; off < kWave; off <<= 1) {
      float t[D2];
#pragma unroll
      for (int j = 0; j < D2; ++j) t[j] = lane_exchange(part[j], (lane ^ off) << 2);
#pragma unroll
      for (int j = 0; j < D2; ++j) part[j] += t[j];
    }
  }
  __syncthreads();  // every wavefront is done with the staged rows; reuse the front of LDS for the partial sums
  float* red = reinterpret_cast<float*>(smem);
  if (wave < n_blk && q == 0) {
#pragma unroll
    for (int j = 0; j < D2; ++j) red[(wave * kUvSamples + n) * D2 + j] = part[j];
  }
  __syncthreads();
  for (int i = threadIdx.x; i < kUvSamples * D2; i += blockDim.x) {
    float s = 0.f;
    for (int w = 0; w < n_blk; ++w) s += red[w * kUvSamples * D2 + i];
    if (n0 + i / D2 < n_rows) gy[n0 * D2 + i] = (__bf16)s;
  }
}

// ---- weight gradient ---------------------------------------------------------------------------------------
//   gW[p, u, w] = sum_n sum_a x[n, a, u] * G[n, p, a, w],   G[n, p, a, w] = sum_(m, b) coef * y[n, b] * g[n, m, w]
// A workgroup owns one path and one chunk of samples and keeps the whole (C_in x C_out) fp32 accumulator in
// registers (four wavefronts, 64 x 64 each).  Per step of 32 samples it stages the path's rows of x in LDS as they
// lie in memory ([sample][channel]), forms the mixed rows G on the vector ALUs into LDS in the same layout, and then
// contracts over the samples on the matrix cores: both MFMA operands need 8 consecutive samples of one channel per
// lane, which ds_read_b64_tr_b16 delivers from the [sample][channel] tiles (within 16 lanes, lane L receives the
// four 16-bit elements that lanes L/4, L/4 + 4, L/4 + 8, L/4 + 12 addressed at position L % 4).  Chunk partials go
// to a workspace and are summed in a fixed order by uv_gw_reduce_kernel.
constexpr int kGwStep = 32;    // samples per MFMA step (K of v_mfma_f32_16x16x32_bf16)
constexpr int kGwChunk = 512;  // samples per workgroup
constexpr int kGwPad = 32;     // bytes added to a tile row: the four rows a 16-lane transpose read touches land in
                               // distinct banks

struct UvGwMeta {              // per configuration, passed by value: workgroup -> path; x rows and g rows of a path
  unsigned char order[64], a0[64], na[64], m0[64], nm[64];
};

__device__ __forceinline__ bf16x8 lds_read_tr(const unsigned char* p0, const unsigned char* p1) {
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0));
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p1));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  const s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(bf16x8, v);
}

template <class CFG>
__global__ void __launch_bounds__(256, 1) uv_gw_kernel(const __bf16* __restrict__ x, const __bf16* __restrict__ y,
                                                       const __bf16* __restrict__ g, float* __restrict__ part,
                                                       int64_t n_rows, int cin, int cout, UvGwMeta meta) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int D1 = CFG::D1, DO = CFG::DO, D2 = CFG::D2, P = CFG::P;
  // the same for every lane: keep them in scalar registers so that the switch over paths is a scalar branch
  // Workgroups are dealt to the 8 XCDs round-robin by index.  The P workgroups of one chunk of samples read the same
  // rows of x and g, so they are given indices that land on one XCD (one L2): index = 8 * slot + xcd, chunk =
  // 8 * (slot / P) + xcd, path = order[slot % P].
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int p = __builtin_amdgcn_readfirstlane(meta.order[slot % P]);
  const int64_t c = (int64_t)(slot / P) * 8 + xcd;
  if (c * kGwChunk >= n_rows) return;
  const int a0 = __builtin_amdgcn_readfirstlane(meta.a0[p]), na = __builtin_amdgcn_readfirstlane(meta.na[p]);
  const int pu = cin * 2 + kGwPad, pw = cout * 2 + kGwPad;   // tile row pitches
  unsigned char* xt = smem;                           // [na][32][pu]  rows of x
  unsigned char* gt = smem + CFG::MAX_ROWS * kGwStep * pu;  // [na][32][pw]  mixed rows
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int vu = wave >> 1, vw = wave & 1;            // this wavefront's 64 x 64 block of the accumulator
  floatx4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int64_t n_begin = c * kGwChunk, n_end = min(n_begin + (int64_t)kGwChunk, n_rows);
  const int sn = tid >> 3, cg = tid & 7;              // mixing: sample of the step and 8-channel group (two passes)
  const int ls = lane & 15, lq = lane >> 4;           // fragment reads
  // Operands of a step are fetched into registers one step ahead, row by row between the matrix work of the step
  // before, so that neither their issue nor their latency is exposed.  x: per input row 32 samples x cin/8 16-byte
  // pieces, thread = (sample, piece) in at most two passes; g: this thread's sample, two 8-channel groups of every
  // row of the path's output irrep.  Row counts are the same for every lane: the guards are scalar branches.
  constexpr int MR = CFG::MAX_ROWS;
  const int m0 = __builtin_amdgcn_readfirstlane(meta.m0[p]), nm = __builtin_amdgcn_readfirstlane(meta.nm[p]);
  const int lp = 31 - __builtin_clz(cin / 8);          // log2 of the pieces per row and sample
  const int xpiece = tid & ((1 << lp) - 1), xs0 = tid >> lp, xstride = 256 >> lp;   // samples per pass
  f32x4 xpre[MR][2];
  bf16x8 gpre[2][MR];
  float ypre[D2];
  const __bf16 *xsrc[2], *gsrc[2];
  auto prefetch_begin = [&](int64_t nb) __attribute__((always_inline)) {
#pragma unroll
    for (int v = 0; v < 2; ++v)
      xsrc[v] = x + (min(nb + min(xs0 + v * xstride, kGwStep - 1), n_rows - 1) * D1 + a0) * cin + xpiece * 8;
    const int64_t row = min(nb + sn, n_rows - 1);
#pragma unroll
    for (int h = 0; h < 2; ++h) gsrc[h] = g + (row * DO + m0) * cout + min((cg + 8 * h) * 8, cout - 8);
    if constexpr (D2 % 8 == 0) {
#pragma unroll
      for (int j = 0; j < D2; j += 8) {
        const bf16x8 v = *reinterpret_cast<const bf16x8*>(y + row * D2 + j);
#pragma unroll
        for (int e = 0; e < 8; ++e) ypre[j + e] = (float)v[e];
      }
    } else {
#pragma unroll
      for (int j = 0; j < D2; ++j) ypre[j] = (float)y[row * D2 + j];
    }
  };
  auto prefetch_row = [&](int r) __attribute__((always_inline)) {
    if (r < na) {
#pragma unroll
      for (int v = 0; v < 2; ++v) xpre[r][v] = *reinterpret_cast<const f32x4*>(xsrc[v] + r * cin);
    }
    if (r < nm) {
#pragma unroll
      for (int h = 0; h < 2; ++h) gpre[h][r] = *reinterpret_cast<const bf16x8*>(gsrc[h] + r * cout);
    }
  };
  prefetch_begin(n_begin);
#pragma unroll
  for (int r = 0; r < MR; ++r) prefetch_row(r);
  // The 32 samples of a step are contracted in the order the transpose reads like best: k-slots 8q..8q+3 of lane
  // group q are samples 4q..4q+3, slots 8q+4..8q+7 samples 16+4q..16+4q+3 (the same for both operands, so the sum
  // is unchanged): the four groups of one read then touch 16 consecutive tile rows, which the row pitch spreads
  // over all banks (groups 8 rows apart share theirs).
  const unsigned char* xa = xt + (4 * lq + (ls >> 2)) * pu + (ls & 3) * 8;
  const unsigned char* gb = gt + (4 * lq + (ls >> 2)) * pw + (ls & 3) * 8;
  for (int64_t nb = n_begin; nb < n_end; nb += kGwStep) {
    __syncthreads();  // the previous step's fragment reads are done
#pragma unroll
    for (int v = 0; v < 2; ++v) {
      const int s_ = min(xs0 + v * xstride, kGwStep - 1);
#pragma unroll
      for (int r = 0; r < MR; ++r)
        if (r < na) *reinterpret_cast<f32x4*>(xt + (r * kGwStep + s_) * pu + xpiece * 16) = xpre[r][v];
    }
    // mixed rows; samples past the end get y = 0 and so contribute nothing
    {
      float yv[D2];
      const float live = nb + sn < n_end ? 1.f : 0.f;
#pragma unroll
      for (int j = 0; j < D2; ++j) yv[j] = ypre[j] * live;
      unsigned char* drow = gt + sn * pw;
      CFG::mix(
          p, yv,
          [&](int h, int j) __attribute__((always_inline)) {
            floatx8 f;
#pragma unroll
            for (int e = 0; e < 8; ++e) f[e] = (float)gpre[h][j][e];
            return f;
          },
          [&](int h, int r, const floatx8& v) __attribute__((always_inline)) {
            const int ch = (cg + 8 * h) * 8;
            bf16x8 o;
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (__bf16)v[e];
            if (ch < cout) *reinterpret_cast<bf16x8*>(drow + r * kGwStep * pw + ch * 2) = o;
          });
    }
    __syncthreads();
    // contract over the 32 samples of the step, row by row, fetching the next step's rows in between
    const bool more = nb + kGwStep < n_end;
    if (more) prefetch_begin(nb + kGwStep);
#pragma unroll
    for (int r = 0; r < MR; ++r) {
      if (more) prefetch_row(r);
      if (r < na) {
        const unsigned char* xr = xa + r * kGwStep * pu;
        const unsigned char* gr = gb + r * kGwStep * pw;
        bf16x8 fa[4], fb[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // tiles past the channel count repeat the last one; their products are never stored.  No branches
          // here: a branch per read would make every read wait for the one before.
          const int ut = min(vu * 4 + i, cin / 16 - 1), wt = min(vw * 4 + i, cout / 16 - 1);
          fa[i] = lds_read_tr(xr + ut * 32, xr + ut * 32 + 16 * pu);
          fb[i] = lds_read_tr(gr + wt * 32, gr + wt * 32 + 16 * pw);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
      }
    }
  }
  // accumulator element e of lane (col = lane & 15, q) is row 4*q + e of the tile
  float* out = part + (c * P + p) * (int64_t)cin * cout;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int u0 = (vu * 4 + i) * 16 + 4 * lq, w_ = (vw * 4 + j) * 16 + ls;
      if (u0 < cin && w_ < cout) {
#pragma unroll
        for (int e = 0; e < 4; ++e) out[(int64_t)(u0 + e) * cout + w_] = acc[i][j][e];
      }
    }
}

// path_scale (one factor per weight path, or nullptr): the module's table is the compiled one with every path's
// coefficients multiplied by that factor; per_path = elements of one path's weight matrix.
__global__ void uv_gw_reduce_kernel(const float* __restrict__ part, __bf16* __restrict__ gw, int64_t n_chunks, int64_t n,
                                    const float* __restrict__ path_scale, int64_t per_path) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float s = 0.f;
  for (int64_t k = 0; k < n_chunks; ++k) s += part[k * n + i];
  if (path_scale) s *= path_scale[i / per_path];
  gw[i] = (__bf16)s;
}

// packed[p][blk][t][k][lane = 16*q + r][e] = Wt[p][blk*32 + 8*(r/4) + 4*t + r%4][k*32 + 8*q + e], where
// Wt[p][row][col] = w[p * rows * cols + row * row_stride + col * col_stride]; one thread per 16-byte piece.
__global__ void uv_pack_kernel(const __bf16* __restrict__ w, __bf16* __restrict__ packed, int64_t n_pieces, int rows,
                               int cols, int64_t row_stride, int64_t col_stride, const float* __restrict__ path_scale) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_pieces) return;
  const int ks = cols / 32, nblk = rows / 32;
  const int lane = (int)(i & 63);
  int64_t c = i >> 6;
  const int k = (int)(c % ks); c /= ks;
  const int t = (int)(c & 1); c >>= 1;
  const int blk = (int)(c % nblk);
  const int64_t p = c / nblk;
  const int r = lane & 15, q = lane >> 4;
  const int64_t row = blk * 32 + 8 * (r >> 2) + 4 * t + (r & 3), col = k * 32 + 8 * q;
  const __bf16* src = w + p * rows * cols + row * row_stride + col * col_stride;
  bf16x8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = src[e * col_stride];
  if (path_scale) {      // folded in fp32, rounded to bf16 once
    const float f = path_scale[p];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (__bf16)((float)v[e] * f);
  }
  *reinterpret_cast<bf16x8*>(packed + i * 8) = v;
}

using UvFn = void (*)(const __bf16*, const __bf16*, const __bf16*, __bf16*, int64_t, int);
using UvGwFn = void (*)(const __bf16*, const __bf16*, const __bf16*, float*, int64_t, int, int, UvGwMeta);

struct UvEntry {
  uint64_t fingerprint;
  uint64_t fingerprint_rounded[2];  // of the table rounded to bf16 / fp16 (a module converted to that type)
  const char* name;
  int din[2], dout[2], d2, p;
  UvFn fn[3][3];  // [direction 0, direction 1, grad y][C_in = 32, 64, 128]
  UvGwFn gw_fn;
  int gw_max_rows;
  UvGwMeta gw_meta;  // order: paths with the most rows first, so that long workgroups start first
  int dims[5];       // D1, D2, DO, P, NNZ
  const float* coef;                 // the compiled table, table order
  const unsigned char (*idx)[4];     // (M, M1, M2, p) per entry
};

template <class D0, class D1, class GY, class GW, class TAB>
static UvEntry make_uv_entry(uint64_t fp, uint64_t fp_bf16, uint64_t fp_f16, const char* name) {
  UvEntry e;
  e.dims[0] = TAB::D1; e.dims[1] = TAB::D2; e.dims[2] = TAB::DO; e.dims[3] = TAB::P; e.dims[4] = TAB::NNZ;
  e.coef = TAB::COEF; e.idx = TAB::IDX;
  e.fingerprint = fp; e.fingerprint_rounded[0] = fp_bf16; e.fingerprint_rounded[1] = fp_f16; e.name = name;
  e.din[0] = D0::DIN; e.dout[0] = D0::DOUT; e.din[1] = D1::DIN; e.dout[1] = D1::DOUT;
  e.d2 = D0::D2; e.p = D0::P;
  e.fn[0][0] = uv_kernel<D0, 32>; e.fn[0][1] = uv_kernel<D0, 64>; e.fn[0][2] = uv_kernel<D0, 128>;
  e.fn[1][0] = uv_kernel<D1, 32>; e.fn[1][1] = uv_kernel<D1, 64>; e.fn[1][2] = uv_kernel<D1, 128>;
  e.fn[2][0] = uv_gy_kernel<GY, 32>; e.fn[2][1] = uv_gy_kernel<GY, 64>; e.fn[2][2] = uv_gy_kernel<GY, 128>;
  static_assert(GW::P <= 64, "path order table too small");
  e.gw_fn = uv_gw_kernel<GW>;
  e.gw_max_rows = GW::MAX_ROWS;
  int k = 0;
  for (int rows = GW::MAX_ROWS; rows >= 1; --rows)
    for (int p = 0; p < GW::P; ++p)
      if (GW::NA[p] == rows) e.gw_meta.order[k++] = (unsigned char)p;
  for (int p = 0; p < GW::P; ++p) {
    e.gw_meta.a0[p] = GW::A0[p];
    e.gw_meta.na[p] = GW::NA[p];
    e.gw_meta.m0[p] = GW::M0[p];
    e.gw_meta.nm[p] = GW::NM[p];
  }
  return e;
}

static const UvEntry* uv_entries(int* count) {
#define CGTP_X(D0, D1, GY, GW, TAB, FP, FP_BF16, FP_F16, NAME) \
  make_uv_entry<D0, D1, GY, GW, TAB>(FP, FP_BF16, FP_F16, NAME),
  static const UvEntry table[] = {CGTP_FOREACH_UV_CONFIG(CGTP_X)};
#undef CGTP_X
  *count = (int)(sizeof(table) / sizeof(table[0]));
  return table;
}

static int uv_check(int cfg, int direction, const void* x, const void* y, const void* wp, const void* out,
                    int64_t n_rows, int cin, int cout, int dtype, int* ci, int64_t* lds) {
  int n = 0;
  const UvEntry* t = uv_entries(&n);
  if (cfg < 0 || cfg >= n) return CGTP_ERR_CONFIG;
  if (direction != 0 && direction != 1) return CGTP_ERR_SHAPE;
  if (dtype != CGTP_BF16) return CGTP_ERR_DTYPE;
  if (!x || !y || !wp || !out) return CGTP_ERR_NULL;
  if (n_rows < 0 || cout <= 0 || cout % 32 != 0) return CGTP_ERR_SHAPE;
  *ci = cin == 32 ? 0 : cin == 64 ? 1 : cin == 128 ? 2 : -1;
  if (*ci < 0) return CGTP_ERR_SHAPE;
  const uintptr_t al = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(wp) | reinterpret_cast<uintptr_t>(out);
  if (al & 15u) return CGTP_ERR_ALIGN;
  *lds = (int64_t)kUvSamples * ((int64_t)t[cfg].din[direction] * cin * 2 + 16);
  if (*lds > kLdsBytes) return CGTP_ERR_LDS;
  return CGTP_OK;
}

}  // namespace cgtp

using namespace cgtp;

extern "C" {

int cgtp_uv_num_configs(void) {
  int n = 0;
  uv_entries(&n);
  return n;
}

int cgtp_uv_find(uint64_t fingerprint) {
  int n = 0;
  const UvEntry* t = uv_entries(&n);
  for (int i = 0; i < n; ++i)
    if (t[i].fingerprint == fingerprint) return i;
  return -1;
}

int cgtp_uv_find_rounded(uint64_t fingerprint, int dtype) {
  if (dtype != CGTP_BF16 && dtype != CGTP_F16) return -1;
  int n = 0;
  const UvEntry* t = uv_entries(&n);
  for (int i = 0; i < n; ++i)
    if (t[i].fingerprint_rounded[dtype == CGTP_F16] == fingerprint) return i;
  return -1;
}

int cgtp_uv_table(int cfg, int32_t* dims, float* coef, int32_t* idx) {
  int n = 0;
  const UvEntry* t = uv_entries(&n);
  if (cfg < 0 || cfg >= n) return -1;
  const UvEntry& e = t[cfg];
  for (int i = 0; dims && i < 5; ++i) dims[i] = e.dims[i];
  for (int k = 0; k < e.dims[4]; ++k) {
    if (coef) coef[k] = e.coef[k];
    for (int j = 0; idx && j < 4; ++j) idx[4 * k + j] = e.idx[k][j];
  }
  return e.dims[4];
}

int cgtp_uv_pack_weights(int direction, const void* w, void* packed, int32_t n_paths, int32_t cin, int32_t cout,
                         int32_t dtype, const float* path_scale, void* stream) {
  if (direction != 0 && direction != 1) return CGTP_ERR_SHAPE;
  if (dtype != CGTP_BF16) return CGTP_ERR_DTYPE;
  if (!w || !packed) return CGTP_ERR_NULL;
  if (n_paths < 0 || cin <= 0 || cout <= 0 || cin % 32 != 0 || cout % 32 != 0) return CGTP_ERR_SHAPE;
  if ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(packed)) & 15u) return CGTP_ERR_ALIGN;
  if (n_paths == 0) return CGTP_OK;
  // rows = result channels, cols = contracted channels; direction 0 reads W (P, cin, cout) transposed, direction 1
  // reads W (P, cout, cin) as stored
  const int64_t n_pieces = (int64_t)n_paths * cin * cout / 8;
  const int64_t row_stride = direction == 0 ? 1 : cin, col_stride = direction == 0 ? cout : 1;
  hipLaunchKernelGGL(uv_pack_kernel, dim3((unsigned)((n_pieces + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const __bf16*)w, (__bf16*)packed, n_pieces, (int)cout, (int)cin, row_stride, col_stride,
                     path_scale);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

int cgtp_uv_validate(int cfg, int direction, const void* x, const void* y, const void* wp, const void* out,
                     int64_t n_rows, int32_t cin, int32_t cout, int32_t dtype) {
  int ci = 0;
  int64_t lds = 0;
  return uv_check(cfg, direction, x, y, wp, out, n_rows, cin, cout, dtype, &ci, &lds);
}

int cgtp_uv_apply(int cfg, int direction, const void* x, const void* y, const void* wp, void* out, int64_t n_rows,
                  int32_t cin, int32_t cout, int32_t dtype, void* stream) {
  int ci = 0;
  int64_t lds = 0;
  const int st = uv_check(cfg, direction, x, y, wp, out, n_rows, cin, cout, dtype, &ci, &lds);
  if (st != CGTP_OK) return st;
  if (n_rows == 0) return CGTP_OK;
  int n = 0;
  UvFn fn = uv_entries(&n)[cfg].fn[direction][ci];
  if (hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return CGTP_ERR_LDS;
  hipLaunchKernelGGL(fn, dim3((unsigned)((n_rows + kUvSamples - 1) / kUvSamples), (unsigned)((cout + 127) / 128)),
                     dim3(256), (size_t)lds,
                     (hipStream_t)stream, (const __bf16*)x, (const __bf16*)y, (const __bf16*)wp, (__bf16*)out, n_rows,
                     (int)cout);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

int cgtp_uv_grad_y(int cfg, const void* x, const void* g, const void* wp, void* gy, int64_t n_rows, int32_t cin,
                   int32_t cout, int32_t dtype, void* stream) {
  int ci = 0;
  int64_t lds = 0;
  const int st = uv_check(cfg, 0, x, g, wp, gy, n_rows, cin, cout, dtype, &ci, &lds);
  if (st != CGTP_OK) return st;
  if (cout > 128) return CGTP_ERR_SHAPE;
  if (reinterpret_cast<uintptr_t>(g) & 15u) return CGTP_ERR_ALIGN;
  if (n_rows == 0) return CGTP_OK;
  int n = 0;
  UvFn fn = uv_entries(&n)[cfg].fn[2][ci];
  if (hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return CGTP_ERR_LDS;
  hipLaunchKernelGGL(fn, dim3((unsigned)((n_rows + kUvSamples - 1) / kUvSamples)), dim3(256), (size_t)lds,
                     (hipStream_t)stream, (const __bf16*)x, (const __bf16*)g, (const __bf16*)wp, (__bf16*)gy, n_rows,
                     (int)cout);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

int64_t cgtp_uv_grad_w_workspace_bytes(int cfg, int64_t n_rows, int32_t cin, int32_t cout) {
  int n = 0;
  const UvEntry* t = uv_entries(&n);
  if (cfg < 0 || cfg >= n || n_rows <= 0 || cin <= 0 || cout <= 0) return 0;
  const int64_t n_chunks = (n_rows + kGwChunk - 1) / kGwChunk;
  return n_chunks * t[cfg].p * (int64_t)cin * cout * (int64_t)sizeof(float);
}

int cgtp_uv_grad_w(int cfg, const void* x, const void* y, const void* g, void* gw, void* workspace, int64_t n_rows,
                   int32_t cin, int32_t cout, int32_t dtype, const float* path_scale, void* stream) {
  int n = 0;
  const UvEntry* t = uv_entries(&n);
  if (cfg < 0 || cfg >= n) return CGTP_ERR_CONFIG;
  if (dtype != CGTP_BF16) return CGTP_ERR_DTYPE;
  if (!x || !y || !g || !gw) return CGTP_ERR_NULL;
  if (n_rows < 0 || cin <= 0 || cout <= 0 || cin % 32 != 0 || cout % 32 != 0 || cin > 128 || cout > 128)
    return CGTP_ERR_SHAPE;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(workspace)) & 15u)
    return CGTP_ERR_ALIGN;
  const UvEntry& e = t[cfg];
  const int64_t n_out = (int64_t)e.p * cin * cout;
  hipStream_t st = (hipStream_t)stream;
  if (n_rows == 0) {  // no samples: the gradient is zero (the summation kernel over zero chunks writes it; a fill
                      // kernel rather than a memset, so that the call can be captured into a graph)
    hipLaunchKernelGGL(uv_gw_reduce_kernel, dim3((unsigned)((n_out + 255) / 256)), dim3(256), 0, st,
                       (const float*)nullptr, (__bf16*)gw, (int64_t)0, n_out, (const float*)nullptr,
                       (int64_t)cin * cout);
    return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
  }
  if (!workspace) return CGTP_ERR_WORKSPACE;
  const int64_t lds = (int64_t)e.gw_max_rows * kGwStep * ((int64_t)cin * 2 + cout * 2 + 2 * kGwPad);
  if (lds > kLdsBytes) return CGTP_ERR_LDS;
  if (hipFuncSetAttribute((const void*)e.gw_fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return CGTP_ERR_LDS;
  const int64_t n_chunks = (n_rows + kGwChunk - 1) / kGwChunk;
  const int64_t n_chunks8 = (n_chunks + 7) / 8 * 8;  // whole rounds over the XCDs; the surplus workgroups exit
  hipLaunchKernelGGL(e.gw_fn, dim3((unsigned)(n_chunks8 * e.p)), dim3(256), (size_t)lds, st, (const __bf16*)x,
                     (const __bf16*)y, (const __bf16*)g, (float*)workspace, n_rows, (int)cin, (int)cout, e.gw_meta);
  hipLaunchKernelGGL(uv_gw_reduce_kernel, dim3((unsigned)((n_out + 255) / 256)), dim3(256), 0, st,
                     (const float*)workspace, (__bf16*)gw, n_chunks, n_out, path_scale, (int64_t)cin * cout);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

}  // extern "C"
