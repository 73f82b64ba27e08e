// Fully connected Clebsch-Gordan tensor products ("uv" / "uvw" families) in fp32 on the matrix cores, driven by
// run-time tables (any irreps, any normalisation):
//
//   out[n, M, w] = sum_{segments s = (p, M)} sum_k inter_s[n, k] * W[p, k, w]
//   inter_s[n, k] = sum_{t in s} coef_t * x[n, a_t, k] * y[n, b_t]                 (y without channels, k = u)
//   inter_s[n, k] = sum_{t in s} coef_t * x[n, a_t, u] * y[n, b_t, v],  k = u * CY + v   (y with channels: "uvw")
//
// Order: coupling first.  The mixed operand inter_s (the reference's stage-1 intermediate, which it writes to memory
// for the whole batch) is formed on the vector ALUs directly in the layout of an MFMA B operand — lane (n, g) holds
// k = 16 kb + 4 g + i of sample n — from the rows of x and y staged once per workgroup in LDS, and is contracted
// with the weights by v_mfma_f32_16x16x4_f32 into a 16 (w) x 16 (n) accumulator tile per block of output channels.
// The walk is a flat list of items (one per segment) ordered by output row, so a wavefront keeps only the
// accumulators of the row it is working on.  A workgroup's wavefronts share the staged rows of its samples and split
// the output rows (groups of items) and the output channels between them.  Weight fragments come from a copy of W
// repacked in fragment order (one contiguous KB per wavefront load) and are requested four blocks of 16 k ahead.
// The gradient with respect to the channelled operand is the same kernel with the roles of the rows exchanged and
// the weight packed transposed; the other two gradients have kernels of their own below.
//
// The file compiles twice: as it is for fp32 (v_mfma_f32_16x16x4_f32), and from uvt_kernels_f64.hip with CGTP_UVT_F64
// defined for fp64 (v_mfma_f64_16x16x4_f64, same lane layouts); each set lives in its own namespace.
#include "cgtp_device.h"
#include "cgtp_host.h"

#ifdef CGTP_UVT_F64
#define UVT_NS uvt_f64
typedef double real;
#else
#define UVT_NS uvt_f32
typedef float real;
#endif

#pragma clang fp contract(fast)

namespace cgtp {
namespace UVT_NS {

typedef real realx4 __attribute__((ext_vector_type(4)));
typedef real realx2 __attribute__((ext_vector_type(2)));
#ifdef CGTP_UVT_F64
constexpr int kDtype = CGTP_F64;
#else
constexpr int kDtype = CGTP_F32;
#endif
constexpr int kTermBytes = 8 + (int)sizeof(real);   // LDS bytes of one term: two row indices and a coefficient

// D = A (16 x 4) * B (4 x 16) + C in the operands' own precision.  Operand layouts are the same for both instructions
// (A: lane holds row lane % 16, k = lane / 16; B: column lane % 16, k = lane / 16); the accumulator's are not: lane
// (column lane % 16, group g = lane / 16) holds in element e row 4 g + e in single and row g + 4 e in double precision.
__host__ __device__ constexpr int acc_row(int g, int e) { return sizeof(real) == 8 ? g + 4 * e : 4 * g + e; }
// Row of operand A that has to carry item c of 16 so that element e of group g ends up holding item 4 g + e (the
// weight fragments are packed in this order: consumers then read four consecutive output channels per lane).
__host__ __device__ constexpr int a_row_of(int c) { return sizeof(real) == 8 ? (c % 4) * 4 + c / 4 : c; }
__device__ __forceinline__ realx4 mfma16(real a, real b, realx4 c, int, int, int) {
#ifdef CGTP_UVT_F64
  return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
#else
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
#endif
}


constexpr int kUvtFirst = 1, kUvtLast = 2;   // item flags: first / last item of its output row
constexpr int kUvtMaxGroups = 8;             // = wavefronts per workgroup
constexpr int64_t kUvtTableRoom = 24 * 1024;  // LDS kept free for the walk tables when the launch shape is chosen

struct UvtDev {
  const real* x;
  const real* y;
  const real* wp;
  real* out;
  const cgtp_uvt_item* items;
  const int32_t* ta;
  const int32_t* tb;
  const real* tc;
  int64_t n_rows;
  int n_items, n_terms, dx, dy, dout, cx, cy, cout;
  int kx;        // y without channels: cx rounded up to 16 (row length of the staged x); with: cx
  int px, py;    // LDS pitch per sample of the x and y tiles, in elements
  int kblocks;   // K / 16 (K padded to 16)
  int wbp;       // blocks of 16 output channels, rounded up to a multiple of 4 (as packed)
  int sb_log2;   // log2 of the 16-sample blocks per workgroup
  int ns;        // sets of 16 samples per wavefront (1 or 2)
  int wgroups;   // wavefronts of a sample block that split the output channels (power of two)
  int igroups;   // groups of items (whole output rows) the remaining wavefronts of a sample block split
  int zero_floats;  // zeros in LDS that the unused term slots of an item read
  int group_ptr[kUvtMaxGroups + 1];   // items of group i: group_ptr[i] .. group_ptr[i + 1]
};

// Rows of the workgroup's samples into LDS: x as [sample][row][kx] (zero-padded channels), y as [sample][row] or
// [sample][row][cy].  Samples past the end of the batch are staged as zeros.
template <bool YC>
__device__ __forceinline__ void uvt_stage(const UvtDev& a, real* xs, real* ys, int64_t nb0, int n_samples) {
  const int kx4 = a.kx / 4, per_sample = a.dx * kx4;
  for (int i = threadIdx.x; i < n_samples * per_sample; i += blockDim.x) {
    const int s = i / per_sample, rem = i - s * per_sample, row = rem / kx4, c4 = rem - row * kx4;
    const int64_t n = nb0 + s;
    realx4 v = {0.f, 0.f, 0.f, 0.f};
    if (n < a.n_rows && c4 * 4 < a.cx) v = *reinterpret_cast<const realx4*>(a.x + (n * a.dx + row) * a.cx + c4 * 4);
    *reinterpret_cast<realx4*>(xs + (size_t)s * a.px + row * a.kx + c4 * 4) = v;
  }
  if constexpr (YC) {
    const int cy4 = a.cy / 4, per_y = a.dy * cy4;
    for (int i = threadIdx.x; i < n_samples * per_y; i += blockDim.x) {
      const int s = i / per_y, rem = i - s * per_y;
      const int64_t n = nb0 + s;
      realx4 v = {0.f, 0.f, 0.f, 0.f};
      if (n < a.n_rows) v = *reinterpret_cast<const realx4*>(a.y + n * a.dy * a.cy + rem * 4);
      *reinterpret_cast<realx4*>(ys + (size_t)s * a.py + rem * 4) = v;
    }
  } else {
    for (int i = threadIdx.x; i < n_samples * a.dy; i += blockDim.x) {
      const int s = i / a.dy, b = i - s * a.dy;
      const int64_t n = nb0 + s;
      ys[(size_t)s * a.py + b] = n < a.n_rows ? a.y[n * a.dy + b] : 0.f;
    }
  }
}

// The walk tables of a launch, copied to LDS by every workgroup (a few KB): reading them from memory with scalar loads
// would put a memory round trip in front of every item, and a workgroup that fills the LDS with its samples' rows has
// a single wavefront per SIMD to hide it behind.
struct UvtTables {
  const cgtp_uvt_item* items;
  const int32_t* ta;
  const int32_t* tb;
  const real* tc;
};

template <class Dev>
__device__ __forceinline__ UvtTables uvt_stage_tables(const Dev& a, unsigned char* at) {
  int32_t* dst = reinterpret_cast<int32_t*>(at);
  const int32_t* src = reinterpret_cast<const int32_t*>(a.items);
  for (int i = threadIdx.x; i < a.n_items * 8; i += blockDim.x) dst[i] = src[i];
  real* tc = reinterpret_cast<real*>(dst + a.n_items * 8);   // first: items are 32 bytes, so this is aligned for doubles
  int32_t* ta = reinterpret_cast<int32_t*>(tc + a.n_terms);
  int32_t* tb = ta + a.n_terms;
  for (int i = threadIdx.x; i < a.n_terms; i += blockDim.x) {
    ta[i] = a.ta[i];
    tb[i] = a.tb[i];
    tc[i] = a.tc[i];
  }
  return UvtTables{reinterpret_cast<const cgtp_uvt_item*>(dst), ta, tb, tc};
}

__device__ __forceinline__ cgtp_uvt_item uvt_item_at(const UvtTables& tab, int j) {
  const int32_t* p = reinterpret_cast<const int32_t*>(tab.items + j);
  cgtp_uvt_item it;
  it.p = __builtin_amdgcn_readfirstlane(p[0]); it.kb0 = __builtin_amdgcn_readfirstlane(p[1]);
  it.nkb = __builtin_amdgcn_readfirstlane(p[2]); it.t0 = __builtin_amdgcn_readfirstlane(p[3]);
  it.t1 = __builtin_amdgcn_readfirstlane(p[4]); it.out_row = __builtin_amdgcn_readfirstlane(p[5]);
  it.flags = __builtin_amdgcn_readfirstlane(p[6]); it.reserved_ = 0;
  return it;
}

// The first kUvtTerms terms of an item's segment in registers, read once per item: per lane the LDS address of the
// term's row of x at the item's first block of k (so that block j is an immediate offset away: no address arithmetic
// per read) and the factor coef * y[n, b]; with a channelled y the addresses of both rows and the coefficient.  Slots
// past the end of the segment point at row 0 with a zero factor, so that the code has no branches around register
// arrays (a conditional assignment to an array element costs the compiler a copy of the array).
constexpr int kUvtTerms = 8;
// Blocks of 16 k in the ring of weight fragments; k is padded to whole turns of it (zero weights, zero rows of the
// staged tiles).  Four blocks cover the round trip to L2 by themselves, which the large products need (their rows fill
// the LDS: one workgroup per compute unit).  Up to 64 contracted channels the ring is two blocks: with at most 32 a
// ring of four would be half padding (twice the LDS per sample, twice the matrix instructions), and at 64 the 32
// registers it saves let a second workgroup onto the compute unit, which covers the latency better than the deeper
// ring did (64 -> 64 channels, lmax = 3, 32768 samples: forward 415 -> 355 us, grad y 734 -> 561 us).
// Past 64 channels the ring is also two where four would pad k by two or three blocks (80, 96, 144, 160 ... channels:
// 96 -> 96, lmax = 2, 32768 samples: forward 475 -> 348 us, grad y 586 -> 346 us).
__host__ __device__ constexpr int uvt_kbi(int64_t K) {
  const int64_t kb = (K + 15) / 16;
  return K <= 64 || kb % 4 == 1 || kb % 4 == 2 ? 2 : 4;
}
template <bool YC>
struct UvtTerms {
  const real* xr[kUvtTerms];
  const real* yr[kUvtTerms];   // YC only
  real s[kUvtTerms];
  int n;
};

template <bool YC>
__device__ __forceinline__ void uvt_terms(const UvtDev& a, const UvtTables& tab, const cgtp_uvt_item& it, const real* xl,
                                          const real* yl, const real* zeros, int g, UvtTerms<YC>& T) {
  T.n = min(it.t1 - it.t0, kUvtTerms);
#pragma unroll
  for (int k = 0; k < kUvtTerms; ++k) {
    const bool live = k < T.n;
    // a slot past the end of the segment reads a block of zeros in LDS (not a row of the input: 0 * inf would leak)
    const int t = live ? it.t0 + k : it.t0;
    const int ia = __builtin_amdgcn_readfirstlane(tab.ta[t]);
    const int ib = __builtin_amdgcn_readfirstlane(tab.tb[t]);
    const real c = live ? tab.tc[t] : 0.f;
    if constexpr (YC) {
      T.xr[k] = live ? xl + ia * a.cx : zeros;
      T.yr[k] = live ? yl + ib * a.cy : zeros;
      T.s[k] = c;
    } else {
      T.xr[k] = live ? xl + ia * a.kx + 4 * g : zeros;
      T.s[k] = live ? c * yl[ib] : 0.f;
    }
  }
}

// This lane's part of block j of 16 k of the mixed operand of an item: inter_s[n, 16 j + 4 g + i], i < 4.
// With a channelled y, lut[j * 4 + g] holds the offsets (u, v) of k = 16 j + 4 g = u * cy + v.
template <bool YC>
__device__ __forceinline__ realx4 uvt_mix_block(const UvtTerms<YC>& T, int j, const int2* lut) {
  realx4 bf = {0.f, 0.f, 0.f, 0.f};
  int2 o = make_int2(0, 0);
  if constexpr (YC) o = lut[j * 4];
#pragma unroll
  for (int half = 0; half < kUvtTerms; half += 2) {
    if (half == 0 || T.n > half) {      // wave-uniform; guards accumulation into one local only.  Pairs of slots: most
                                        // segments of the tables up to lmax = 3 have one or two terms
#pragma unroll
      for (int k = half; k < half + 2; ++k) {
        if constexpr (YC) {
          bf += (T.s[k] * T.xr[k][o.x]) * *reinterpret_cast<const realx4*>(T.yr[k] + o.y);
        } else {
          bf += T.s[k] * *reinterpret_cast<const realx4*>(T.xr[k] + j * 16);
        }
      }
    }
  }
  return bf;
}

// Terms beyond the first kUvtTerms of a segment (large irreps only): straight from the tables.
template <bool YC>
__device__ __forceinline__ realx4 uvt_mix_tail(const UvtDev& a, const UvtTables& tab, const cgtp_uvt_item& it, int j,
                                                const real* xl, const real* yl, int g, const int2* lut) {
  realx4 bf = {0.f, 0.f, 0.f, 0.f};
  for (int t = it.t0 + kUvtTerms; t < it.t1; ++t) {
    const int ia = tab.ta[t], ib = tab.tb[t];
    const real c = tab.tc[t];
    if constexpr (YC) {
      const int2 o = lut[j * 4];
      bf += (c * xl[ia * a.cx + o.x]) * *reinterpret_cast<const realx4*>(yl + ib * a.cy + o.y);
    } else {
      bf += (c * yl[ib]) * *reinterpret_cast<const realx4*>(xl + ia * a.kx + (it.kb0 + j) * 16 + 4 * g);
    }
  }
  return bf;
}

// WB: blocks of 16 output channels per wavefront.  k is padded to whole multiples of KBI blocks of 16 (zero
// weights, zero rows), so the ring of weight fragments turns in straight-line code.
// While the matrix instructions of block j run, the vector ALUs mix block j + 1; the weight fragments of block j + 4
// (of the next item past the end of this one) are requested as soon as block j's are consumed.  Everything an item
// needs besides its operands is wave-uniform (scalar registers).  A wavefront issues one instruction every four
// cycles, a matrix instruction keeps its pipeline busy for 32: with 4 WB matrix instructions per block next to
// about 50 vector and LDS instructions, two wavefronts per SIMD keep the matrix pipeline fed when WB >= 2.
// NS = 2 (y without channels, WB = KBI = 4 only): the wavefront multiplies each weight fragment with the mixed rows
// of two sets of 16 samples (two accumulator sets), which halves the requests to the L2 per matrix instruction —
// at 128 channels the rate of those requests bounds the kernel, not the matrix pipeline.  Taken where the rows of
// 32 samples fit the LDS.
template <bool YC, int WB, int KBI, int NS = 1>
__global__ void __launch_bounds__(kUvtMaxGroups* kWave) uvt_apply_kernel(const UvtDev a) {
  static_assert(NS == 1 || (NS == 2 && !YC), "two sample sets: y without channels");
  extern __shared__ __align__(16) unsigned char smem[];
  const int sb_count = (1 << a.sb_log2) * NS;
  real* xs = reinterpret_cast<real*>(smem);
  real* ys = xs + (size_t)(16 * sb_count) * a.px;
  const int64_t nb0 = (int64_t)blockIdx.x * (16 * sb_count);
  uvt_stage<YC>(a, xs, ys, nb0, 16 * sb_count);
  unsigned char* after = reinterpret_cast<unsigned char*>(ys + (size_t)(16 * sb_count) * a.py);
  const UvtTables tab = uvt_stage_tables(a, after);
  // (u, v) of k = 16 kb + 4 g for a channelled y; (0, 0) in the zero-padded tail of k
  int2* lut_all = reinterpret_cast<int2*>(after + ((size_t)a.n_items * 32 + (size_t)a.n_terms * kTermBytes + 15) / 16 * 16);
  if constexpr (YC) {
    for (int i = threadIdx.x; i < a.kblocks * 4; i += blockDim.x) {
      const int k0 = i * 4, u = k0 / a.cy;
      lut_all[i] = k0 < a.cx * a.cy ? make_int2(u, k0 - u * a.cy) : make_int2(0, 0);
    }
  }
  real* zeros = reinterpret_cast<real*>(lut_all + (YC ? a.kblocks * 4 : 0));
  for (int i = threadIdx.x; i < a.zero_floats; i += blockDim.x) zeros[i] = 0.f;
  __syncthreads();

  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1), r = lane & 15, g = lane >> 4;
  const int sb = (wave & ((1 << a.sb_log2) - 1)) * NS, rest = wave >> a.sb_log2;   // first set of this wavefront
  const int wg = rest & (a.wgroups - 1), ig = rest / a.wgroups;
  const int wb0 = (blockIdx.y * a.wgroups + wg) * WB;
  if (wb0 * 16 >= a.cout) return;
  int j = a.group_ptr[ig];
  const int j_end = a.group_ptr[ig + 1];
  if (j >= j_end) return;
  const int64_t n = nb0 + sb * 16 + r;
  const real* xl = xs + (size_t)(sb * 16 + r) * a.px;
  const real* yl = ys + (size_t)(sb * 16 + r) * a.py;
  const int2* lut_g = lut_all + g;

  const int64_t kstride = (int64_t)a.wbp * 256;
  auto wbase_of = [&](const cgtp_uvt_item& it) __attribute__((always_inline)) {
    // wave-uniform base of the item's fragments; a lane adds 16 bytes times its index
    return a.wp + ((int64_t)it.p * a.kblocks * a.wbp + wb0) * 256 + lane * 4;
  };
  realx4 acc[WB], A[KBI][WB];
  // second set of samples (NS = 2): rows 16 further in the staged tiles
  realx4 acc2[NS == 2 ? WB : 1];
  const int x2 = 16 * a.px;
  const real* yl2 = yl + (size_t)16 * a.py;
  auto load_a = [&](const real* base, int kb, realx4 (&Aj)[WB]) __attribute__((always_inline)) {
#pragma unroll
    for (int wb = 0; wb < WB; ++wb) Aj[wb] = *reinterpret_cast<const realx4*>(base + kb * kstride + wb * 256);
  };
#pragma unroll
  for (int wb = 0; wb < WB; ++wb) acc[wb] = realx4{0.f, 0.f, 0.f, 0.f};
  if constexpr (NS == 2) {
#pragma unroll
    for (int wb = 0; wb < WB; ++wb) acc2[wb] = realx4{0.f, 0.f, 0.f, 0.f};
  }

  cgtp_uvt_item it = uvt_item_at(tab, j);
  const real* base = wbase_of(it);
#pragma unroll
  for (int jj = 0; jj < KBI; ++jj) load_a(base, jj, A[jj]);
  while (j < j_end) {
    const bool more = j + 1 < j_end;
    const cgtp_uvt_item it2 = uvt_item_at(tab, more ? j + 1 : j);
    const real* base2 = wbase_of(it2);
    UvtTerms<YC> T;
    uvt_terms<YC>(a, tab, it, xl, yl, zeros, g, T);
    const bool tail = it.t1 - it.t0 > kUvtTerms;
    auto mix = [&](int kb) __attribute__((always_inline)) {
      realx4 b = uvt_mix_block<YC>(T, kb, lut_g);
      if (tail) b += uvt_mix_tail<YC>(a, tab, it, kb, xl, yl, g, lut_g);
      return b;
    };
    // second set: its factors coef * y[n + 16, b]; the rows of x are those of the first set x2 further (slots past
    // the end stay on the block of zeros)
    real s2[NS == 2 ? kUvtTerms : 1];
    int xo[NS == 2 ? kUvtTerms : 1];
    if constexpr (NS == 2) {
#pragma unroll
      for (int k = 0; k < kUvtTerms; ++k) {
        const bool live = k < T.n;
        const int t = live ? it.t0 + k : it.t0;
        const int ib = __builtin_amdgcn_readfirstlane(tab.tb[t]);
        s2[k] = live ? tab.tc[t] * yl2[ib] : 0.f;
        xo[k] = live ? x2 : 0;
      }
    }
    auto mix2 = [&](int kb) __attribute__((always_inline)) {
      realx4 b = {0.f, 0.f, 0.f, 0.f};
      if constexpr (NS == 2) {
#pragma unroll
        for (int half = 0; half < kUvtTerms; half += 2) {
          if (half == 0 || T.n > half) {
#pragma unroll
            for (int k = half; k < half + 2; ++k) b += s2[k] * *reinterpret_cast<const realx4*>(T.xr[k] + xo[k] + kb * 16);
          }
        }
        if (tail) b += uvt_mix_tail<YC>(a, tab, it, kb, xl + x2, yl2, g, lut_g);
      }
      return b;
    };
    const bool first = it.flags & kUvtFirst;
#pragma unroll
    for (int wb = 0; wb < WB; ++wb) acc[wb] = first ? realx4{0.f, 0.f, 0.f, 0.f} : acc[wb];
    if constexpr (NS == 2) {
#pragma unroll
      for (int wb = 0; wb < WB; ++wb) acc2[wb] = first ? realx4{0.f, 0.f, 0.f, 0.f} : acc2[wb];
    }
    realx4 Bc = mix(0);
    realx4 Bc2 = mix2(0);
    for (int kb = 0; kb < a.kblocks; kb += KBI) {
      const bool wrap = kb + KBI >= a.kblocks;        // the fragments requested now belong to the next item
      const real* wnext = wrap ? base2 : base;
      const int kbn = wrap ? 0 : kb + KBI;
#pragma unroll
      for (int jj = 0; jj < KBI; ++jj) {
        const int kb_next = (jj + 1 < KBI || !wrap) ? kb + jj + 1 : kb + jj;
        const realx4 Bn = mix(kb_next);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int wb = 0; wb < WB; ++wb) {
            acc[wb] = mfma16(A[jj][wb][i], Bc[i], acc[wb], 0, 0, 0);
            if constexpr (NS == 2) acc2[wb] = mfma16(A[jj][wb][i], Bc2[i], acc2[wb], 0, 0, 0);
          }
        if constexpr (NS == 2) Bc2 = mix2(kb_next);
        load_a(wnext, kbn + jj, A[jj]);
        Bc = Bn;
      }
    }
    if (it.flags & kUvtLast) {
      // accumulator layout: lane (n = r, g) holds output channels 16 wb + 4 g .. + 3 of sample n
      if (n < a.n_rows) {
        real* orow = a.out + (n * a.dout + it.out_row) * a.cout;
#pragma unroll
        for (int wb = 0; wb < WB; ++wb) {
          const int w = (wb0 + wb) * 16 + 4 * g;
          if (w < a.cout) *reinterpret_cast<realx4*>(orow + w) = acc[wb];
        }
      }
      if constexpr (NS == 2) {
        if (n + 16 < a.n_rows) {
          real* orow = a.out + ((n + 16) * a.dout + it.out_row) * a.cout;
#pragma unroll
          for (int wb = 0; wb < WB; ++wb) {
            const int w = (wb0 + wb) * 16 + 4 * g;
            if (w < a.cout) *reinterpret_cast<realx4*>(orow + w) = acc2[wb];
          }
        }
      }
    }
    ++j;
    it = it2;
    base = base2;
  }
}

// packed[((p * kblocks + kb) * wbp + wb) * 256 + lane * 4 + i] = W[p][16 kb + 4 (lane / 16) + i][16 wb + lane % 16]
// (zero outside K x cout), W addressed with element strides so that the transposed weight of the backward needs no
// copy of its own.
__global__ void uvt_pack_kernel(const real* __restrict__ w, real* __restrict__ packed, int64_t n_vec, int K, int cout,
                                int kblocks, int wbp, int64_t stride_p, int64_t stride_k, int64_t stride_c) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_vec) return;
  const int lane = (int)(i & 63);
  int64_t c = i >> 6;
  const int wb = (int)(c % wbp); c /= wbp;
  const int kb = (int)(c % kblocks);
  const int64_t p = c / kblocks;
  // row i of the fragment carries the output channel c with a_row_of(c) == i (the permutation is its own inverse)
  const int col = wb * 16 + a_row_of(lane & 15);
  realx4 v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int k = kb * 16 + 4 * (lane >> 4) + e;
    if (k < K && col < cout) v[e] = w[p * stride_p + k * stride_k + col * stride_c];
  }
  *reinterpret_cast<realx4*>(packed + i * 4) = v;
}


// ---- gradient of a shared weight ---------------------------------------------------------------------------------
//   gW[p, k, w] = sum_n sum_{segments s = (p, M)} inter_s[n, k] * g[n, M, w]
// The contraction runs over the samples: four per matrix instruction (A: lane (k = lane % 16, sample = lane / 16)
// holds inter_s[n, k]; B: lane (w = lane % 16, sample) holds g[n, M, w]).  A workgroup owns one weight path, one chunk
// of samples and a 128 (k) x 128 (w) block of the path's gradient, which its four wavefronts split 2 x 2 into parts of
// 4 x 4 accumulator tiles.  Two wavefronts need the same inter values and two the same g values, and the vector
// memory path of a compute unit delivers about 64 bytes a cycle — loading every operand in the wavefront that uses it
// took twice the time of the matrix instructions.  So the wavefronts load disjoint quarters of a step of eight
// samples (sample pair = wavefront, four consecutive channels = lane), mix the terms, and exchange the results
// through a double-buffered LDS stage; the loads of step i + 2 are in flight while step i is multiplied.
// The chunks' partial results go to a workspace and are summed in chunk order by uvt_gw_reduce_kernel (no atomics:
// the result does not depend on the launch).
struct UvtGwDev {
  const real* x;
  const real* y;
  const real* g;
  real* part;                 // (n_chunks, n_paths, K, cout)
  const cgtp_uvt_item* items;  // segments sorted by path: p, out_row = M, t0, t1
  const int32_t* path_ptr;     // [n_paths + 1] into items
  const int32_t* ta;
  const int32_t* tb;
  const real* tc;
  int64_t n_rows;
  int n_paths, dx, dy, dg, cx, cy, cout, K, chunk;
};

constexpr int kGwT = 4;        // accumulator tiles per wavefront and axis
constexpr int kGwStep = 8;     // samples per step (two matrix instructions deep)

// Tile rows and columns are interleaved with the channels — row r of k-tile i is channel 4 r + i of the wavefront's
// 64, column r of w-tile j is output channel 4 r + j — so that a lane's operands of the four tiles are four
// consecutive channels: one 16-byte LDS read per operand and step.
// NARROW (few output channels): the block is 256 (k) x 64 (w), the four wavefronts split k four ways and share the
// w columns, a thread loads and mixes two samples of its four k channels per step; with 128 columns for 32 or 64
// output channels most of the matrix instructions would multiply zeros.  NARROW = 2 (at most 32 output channels):
// 256 (k) x 32 (w), two w tiles per wavefront, column r of tile j is output channel 2 r + j.
template <bool YC, int NARROW>
__global__ void __launch_bounds__(256, sizeof(real) == 8 ? 1 : NARROW ? 2 : 3) uvt_grad_w_kernel(const UvtGwDev a) {
  constexpr int KT = NARROW ? 256 : 128, WT = NARROW == 2 ? 32 : NARROW ? 64 : 128, NA = NARROW ? 2 : 1;
  constexpr int TW = NARROW == 2 ? 2 : kGwT;      // w tiles per wavefront
  __shared__ __attribute__((aligned(16))) real lds_a[2][kGwStep][KT + 4];   // rows 4 banks apart
  __shared__ __attribute__((aligned(16))) real lds_b[2][kGwStep][WT + 4];
  const int tid = threadIdx.x;
  const int wave = tid / kWave, lane = tid & (kWave - 1), r = lane & 15, g4 = lane >> 4;
  const int p = blockIdx.y;
  const int kgroups = (a.K + KT - 1) / KT;
  const int kgrp = blockIdx.z % kgroups, wgrp = blockIdx.z / kgroups;
  const int64_t n_begin = (int64_t)blockIdx.x * a.chunk;
  const int64_t n_end = n_begin + a.chunk < a.n_rows ? n_begin + a.chunk : a.n_rows;

  // loading role: channels lq .. lq + 3 of the block's k range for sample ls (and ls + 4 if NARROW), channels
  // lqb .. lqb + 3 of its w range for sample lsb (NARROW: the first 128 threads only)
  const int ls = NARROW ? tid >> 6 : 2 * wave + (lane >> 5), lq = NARROW ? 4 * (tid & 63) : 4 * (lane & 31);
  const int lsb = NARROW == 2 ? (tid >> 3) & 7 : NARROW ? (tid >> 4) & 7 : ls;
  const int lqb = NARROW == 2 ? 4 * (tid & 7) : NARROW ? 4 * (tid & 15) : lq;
  const bool b_thread = !NARROW || tid < (NARROW == 2 ? 64 : 128);
  // K and cout are multiples of 4 (checked by the launcher), so a lane's four channels are all inside or all outside
  const bool kok = kgrp * KT + lq < a.K, wok = b_thread && wgrp * WT + lqb < a.cout;
  const int kc = kok ? kgrp * KT + lq : 0, wc = wok ? wgrp * WT + lqb : 0;
  int xo = kc, yo = 0;
  if constexpr (YC) {
    xo = kc / a.cy;
    yo = kc - xo * a.cy;
  }
  // multiplying role: channels kh * 64 .. + 63 by output channels wh * 64 .. + 63
  const int kh = NARROW ? wave : wave & 1, wh = NARROW ? 0 : wave >> 1;

  realx4 acc[kGwT][TW];
#pragma unroll
  for (int i = 0; i < kGwT; ++i)
#pragma unroll
    for (int j = 0; j < TW; ++j) acc[i][j] = realx4{0.f, 0.f, 0.f, 0.f};

  const int s_begin = a.path_ptr[p], s_end = a.path_ptr[p + 1];
  const int steps = (int)((n_end - n_begin + kGwStep - 1) / kGwStep);
  const int total = (s_end - s_begin) * steps;

  // state of the loads in flight: the segment's terms in scalar registers (at most kUvtTerms per item: the caller
  // splits longer segments; slots past the end repeat the first term's rows with coefficient zero)
  int ld_item = s_begin - 1, ld_step = steps;
  int n_slots = 0;              // the item's term count rounded up to a pair: pairs of slots past it are skipped
  int xrow[kUvtTerms], yrow[kUvtTerms], grow = 0;
  real c[kUvtTerms];
  realx4 v4[NA][kUvtTerms];     // y without channels: four channels of x; with: four channels of y
  real v1[NA][kUvtTerms];       // y without channels: y[n, b]; with: x[n, a, u]
  realx4 bv4;
  bool ld_live[NA] = {}, ldb_live = false;

  auto issue = [&]() __attribute__((always_inline)) {
    if (ld_step == steps) {
      ld_step = 0;
      ++ld_item;
      const cgtp_uvt_item it = a.items[ld_item];
      const int n_t = it.t1 - it.t0;
      n_slots = __builtin_amdgcn_readfirstlane((n_t + 1) & ~1);
#pragma unroll
      for (int k = 0; k < kUvtTerms; ++k) {
        const int t = k < n_t ? it.t0 + k : it.t0;
        xrow[k] = a.ta[t] * a.cx;
        yrow[k] = a.tb[t] * (YC ? a.cy : 1);
        c[k] = k < n_t ? a.tc[t] : 0.f;
      }
      grow = it.out_row * a.cout;
    }
    const int64_t n0 = n_begin + (int64_t)ld_step * kGwStep;
    {
      const int64_t n = n0 + lsb;
      ldb_live = n < n_end;
      bv4 = *reinterpret_cast<const realx4*>(a.g + (ldb_live ? n : n_end - 1) * a.dg * a.cout + grow + wc);
    }
#pragma unroll
    for (int j = 0; j < NA; ++j) {
      const int64_t n = n0 + ls + 4 * j;
      ld_live[j] = n < n_end;
      const int64_t nc = ld_live[j] ? n : n_end - 1;
      const real* xn = a.x + nc * a.dx * a.cx + xo;
      const real* yn = a.y + nc * a.dy * (YC ? a.cy : 1) + yo;
#pragma unroll
      for (int h = 0; h < kUvtTerms; h += 2) {
        if (h < n_slots) {            // the same in every lane: a scalar branch
#pragma unroll
          for (int k = h; k < h + 2; ++k) {
            if constexpr (YC) {
              v1[j][k] = xn[xrow[k]];
              v4[j][k] = *reinterpret_cast<const realx4*>(yn + yrow[k]);
            } else {
              v4[j][k] = *reinterpret_cast<const realx4*>(xn + xrow[k]);
              v1[j][k] = yn[yrow[k]];
            }
          }
        }
      }
    }
    ++ld_step;
  };
  // mixes the terms of the loads in flight and puts both operands into stage buf
  auto commit = [&](int buf) __attribute__((always_inline)) {
    const realx4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < NA; ++j) {
      realx4 av = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int h = 0; h < kUvtTerms; h += 2) {
        if (h < n_slots) {            // slots of the loads in flight: commit runs before the next issue
          av += (c[h] * v1[j][h]) * v4[j][h];
          av += (c[h + 1] * v1[j][h + 1]) * v4[j][h + 1];
        }
      }
      *reinterpret_cast<realx4*>(&lds_a[buf][ls + 4 * j][lq]) = (ld_live[j] && kok) ? av : zero;
    }
    if (b_thread) *reinterpret_cast<realx4*>(&lds_b[buf][lsb][lqb]) = (ldb_live && wok) ? bv4 : zero;
  };

  if (total > 0) {
    issue();
    commit(0);
    if (total > 1) issue();
    __syncthreads();
    for (int i = 0; i < total; ++i) {
      const int buf = i & 1;
      realx4 af[2];
      real bf[2][TW];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        af[ks] = *reinterpret_cast<const realx4*>(&lds_a[buf][4 * ks + g4][kh * 64 + 4 * r]);
        if constexpr (TW == 4) {
          const realx4 b = *reinterpret_cast<const realx4*>(&lds_b[buf][4 * ks + g4][wh * 64 + 4 * r]);
          bf[ks][0] = b[0]; bf[ks][1] = b[1]; bf[ks][2] = b[2]; bf[ks][3] = b[3];
        } else {
          const realx2 b = *reinterpret_cast<const realx2*>(&lds_b[buf][4 * ks + g4][2 * r]);
          bf[ks][0] = b[0]; bf[ks][1] = b[1];
        }
      }
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int ti = 0; ti < kGwT; ++ti)
#pragma unroll
          for (int tj = 0; tj < TW; ++tj)
            acc[ti][tj] = mfma16(af[ks][ti], bf[ks][tj], acc[ti][tj], 0, 0, 0);
      if (i + 1 < total) commit(buf ^ 1);
      if (i + 2 < total) issue();
      __syncthreads();
    }
  }
  // accumulator layout: lane (column r, g4) holds rows 4 g4 .. + 3 of a tile; tile (i, j) row q is channel
  // 4 q + i of the wavefront's 64, column r is output channel 4 r + j
  real* out = a.part + ((int64_t)blockIdx.x * a.n_paths + p) * a.K * a.cout;
  const int kbase = kgrp * KT + kh * 64;
  const int w0 = wgrp * WT + wh * 64 + TW * r;
  if (w0 < a.cout) {
#pragma unroll
    for (int i = 0; i < kGwT; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int k = kbase + 4 * acc_row(g4, e) + i;
        if (k < a.K) {
          if constexpr (TW == 4) {
            realx4 v;
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = acc[i][j][e];
            *reinterpret_cast<realx4*>(out + (int64_t)k * a.cout + w0) = v;
          } else {
            const realx2 v = {acc[i][0][e], acc[i][1][e]};
            *reinterpret_cast<realx2*>(out + (int64_t)k * a.cout + w0) = v;
          }
        }
      }
  }
}

// Weights of at most 64 x 64 (K <= 64 and at most 64 output channels — the channel mixing of 64-channel models): one
// block, and the block of the kernel above would be three quarters zeros.  Here a wavefront owns the whole block and a
// chunk of samples by itself: the operands' layout in memory is the matrix instructions' own (lane (r, g) holds the
// four channels 4 r .. 4 r + 3 of sample g of four: one 16-byte load, element i = tile i), so nothing is exchanged
// through LDS and there is no barrier; two steps of eight samples are loaded before the first is multiplied, and
// several wavefronts per SIMD cover each other's load latency.  An axis of at most 32 channels takes two channels a
// lane and two tiles (32 x 32 weights, lmax = 3, 32768 samples: 461 -> 226 us).
template <int N> struct UvtVec;
template <> struct UvtVec<2> { typedef realx2 type; };
template <> struct UvtVec<4> { typedef realx4 type; };

// TI / TJ: channels a lane holds of the contracted and of the output axis = accumulator tiles along each (4: up to 64
// channels, 2: up to 32 — a 32 x 32 weight in 4 x 4 tiles would multiply three quarters zeros).
template <bool YC, int TI, int TJ>
__global__ void __launch_bounds__(kWave) uvt_grad_w_small_kernel(const UvtGwDev a) {
  typedef typename UvtVec<TI>::type VI;
  typedef typename UvtVec<TJ>::type VJ;
  const int lane = threadIdx.x, r = lane & 15, g4 = lane >> 4;
  const int p = blockIdx.y;
  const int64_t n_begin = (int64_t)blockIdx.x * a.chunk;
  const int64_t n_end = n_begin + a.chunk < a.n_rows ? n_begin + a.chunk : a.n_rows;
  const bool kok = TI * r < a.K, wok = TJ * r < a.cout;
  const int kc = kok ? TI * r : 0, wc = wok ? TJ * r : 0;
  int xo = kc, yo = 0;
  if constexpr (YC) {
    xo = kc / a.cy;
    yo = kc - xo * a.cy;
  }
  realx4 acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j) acc[i][j] = realx4{0.f, 0.f, 0.f, 0.f};
  constexpr int NS = 4;          // groups of four samples in flight: two steps of eight
  VI zi;
  VJ zj;
#pragma unroll
  for (int i = 0; i < TI; ++i) zi[i] = 0.f;
#pragma unroll
  for (int j = 0; j < TJ; ++j) zj[j] = 0.f;
  for (int s = a.path_ptr[p]; s < a.path_ptr[p + 1]; ++s) {
    const cgtp_uvt_item it = a.items[s];
    const int n_t = __builtin_amdgcn_readfirstlane(it.t1 - it.t0);
    const int grow = __builtin_amdgcn_readfirstlane(it.out_row) * a.cout;
    for (int64_t n0 = n_begin; n0 < n_end; n0 += 4 * NS) {
      VI av[NS];
      VJ bv[NS];
      const real* xn[NS];
      const real* yn[NS];
      bool live[NS];
#pragma unroll
      for (int q = 0; q < NS; ++q) {
        const int64_t n = n0 + 4 * q + g4;
        live[q] = n < n_end;
        const int64_t nc = live[q] ? n : n_end - 1;
        xn[q] = a.x + nc * a.dx * a.cx + xo;
        yn[q] = a.y + nc * a.dy * (YC ? a.cy : 1) + yo;
        bv[q] = *reinterpret_cast<const VJ*>(a.g + nc * a.dg * a.cout + grow + wc);
        av[q] = zi;
      }
      for (int t0 = 0; t0 < n_t; t0 += 2) {          // the segment's terms, two at a time (most have one or two)
        const bool two = t0 + 1 < n_t;
        const int ta0 = a.ta[it.t0 + t0] * a.cx, tb0 = a.tb[it.t0 + t0] * (YC ? a.cy : 1);
        const int ta1 = a.ta[it.t0 + (two ? t0 + 1 : t0)] * a.cx, tb1 = a.tb[it.t0 + (two ? t0 + 1 : t0)] * (YC ? a.cy : 1);
        const real c0 = a.tc[it.t0 + t0], c1 = two ? a.tc[it.t0 + t0 + 1] : real(0);
        VI v4[NS][2];
        real v1[NS][2];
#pragma unroll
        for (int q = 0; q < NS; ++q) {
          if constexpr (YC) {
            v1[q][0] = xn[q][ta0]; v4[q][0] = *reinterpret_cast<const VI*>(yn[q] + tb0);
            v1[q][1] = xn[q][ta1]; v4[q][1] = *reinterpret_cast<const VI*>(yn[q] + tb1);
          } else {
            v4[q][0] = *reinterpret_cast<const VI*>(xn[q] + ta0); v1[q][0] = yn[q][tb0];
            v4[q][1] = *reinterpret_cast<const VI*>(xn[q] + ta1); v1[q][1] = yn[q][tb1];
          }
        }
#pragma unroll
        for (int q = 0; q < NS; ++q) {
          av[q] += (c0 * v1[q][0]) * v4[q][0];
          av[q] += (c1 * v1[q][1]) * v4[q][1];
        }
      }
#pragma unroll
      for (int q = 0; q < NS; ++q) {
        const VI af = (live[q] && kok) ? av[q] : zi;
        const VJ bf = (live[q] && wok) ? bv[q] : zj;
#pragma unroll
        for (int ti = 0; ti < TI; ++ti)
#pragma unroll
          for (int tj = 0; tj < TJ; ++tj) acc[ti][tj] = mfma16(af[ti], bf[tj], acc[ti][tj], 0, 0, 0);
      }
    }
  }
  real* out = a.part + ((int64_t)blockIdx.x * a.n_paths + p) * a.K * a.cout;
  if (wok) {
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int k = TI * acc_row(g4, e) + i;
        if (k < a.K) {
          VJ v;
#pragma unroll
          for (int j = 0; j < TJ; ++j) v[j] = acc[i][j][e];
          *reinterpret_cast<VJ*>(out + (int64_t)k * a.cout + TJ * r) = v;
        }
      }
  }
}

// gw[i] = sum over the chunks c of part[c * n + i], in a fixed order: a thread owns four consecutive elements (n is a
// multiple of 4) and every fourth chunk, four loads in flight; the four slices of a column are added in slice order.
// (One thread per element walking all chunks one after the other took 33 us for 128 chunks of 12 288 elements: 128
// dependent round trips.)
constexpr int kGwReduceCols = 64, kGwReduceSlices = 4;
__global__ void __launch_bounds__(kGwReduceCols * kGwReduceSlices)
uvt_gw_reduce_kernel(const real* __restrict__ part, real* __restrict__ gw, int64_t n_chunks, int64_t n4) {
  __shared__ realx4 acc[kGwReduceSlices][kGwReduceCols];
  const int col = threadIdx.x % kGwReduceCols, slice = threadIdx.x / kGwReduceCols;
  const int64_t i = (int64_t)blockIdx.x * kGwReduceCols + col;
  realx4 s = {0.f, 0.f, 0.f, 0.f};
  if (i < n4) {
    const realx4* p = reinterpret_cast<const realx4*>(part) + i;
    int64_t c = slice;
    for (; c + 3 * kGwReduceSlices < n_chunks; c += 4 * kGwReduceSlices) {
      const realx4 a0 = p[c * n4], a1 = p[(c + kGwReduceSlices) * n4], a2 = p[(c + 2 * kGwReduceSlices) * n4],
                   a3 = p[(c + 3 * kGwReduceSlices) * n4];
      s += a0; s += a1; s += a2; s += a3;
    }
    for (; c < n_chunks; c += kGwReduceSlices) s += p[c * n4];
  }
  acc[slice][col] = s;
  __syncthreads();
  if (slice == 0 && i < n4) {
    realx4 total = acc[0][col];
#pragma unroll
    for (int j = 1; j < kGwReduceSlices; ++j) total += acc[j][col];
    reinterpret_cast<realx4*>(gw)[i] = total;
  }
}

// few output channels and a long contracted axis: 256 x 64 blocks (single precision; in double precision the second
// set of operands in flight does not fit the registers)
static int uvt_gw_narrow(int64_t K, int32_t cout) {
  return sizeof(real) == 4 && cout <= 64 && K >= 256 ? (cout <= 32 ? 2 : 1) : 0;
}

static int64_t uvt_gw_blocks(int64_t K, int32_t cout) {
  const int narrow = uvt_gw_narrow(K, cout);
  const int64_t kt = narrow ? 256 : 128, wt = narrow == 2 ? 32 : narrow ? 64 : 128;
  return ((K + kt - 1) / kt) * ((cout + wt - 1) / wt);
}

// one wavefront per (path, chunk of samples) with the whole weight block in its registers
static bool uvt_gw_small(int64_t K, int32_t cout) { return sizeof(real) == 4 && K <= 64 && cout <= 64; }   // doubles: 312 registers

static int64_t uvt_gw_chunk(int64_t n_rows, int32_t n_paths, int64_t K, int32_t cout) {
  if (uvt_gw_small(K, cout)) {
    // wavefronts, not workgroups of four: chunks of 32 samples or more, at most 8192 wavefronts and 512 partial
    // results (three paths over 65 536 samples: 641 us for the layer's step with at most 128, 442 with 512, 492 with
    // 2048 — the partial results are 16 KB each and the reduction reads them all)
    int64_t chunk = 32;
    while ((n_rows + chunk - 1) / chunk > 512 || ((n_rows + chunk - 1) / chunk) * n_paths > 8192) chunk *= 2;
    return chunk;
  }
  // samples per workgroup: at most 128 partial results; 256 samples, fewer (down to 32: four steps) while the launch
  // would have less than three workgroups per compute unit — a node-level layer has a few thousand samples and a
  // handful of paths, and with 256 samples per workgroup its 48 workgroups took 100 us for 0.3 GFLOP
  const int64_t per_chunk = n_paths * uvt_gw_blocks(K, cout);
  int64_t chunk = 256;
  while (chunk > 32 && ((n_rows + chunk - 1) / chunk) * per_chunk < 768 && (n_rows + chunk / 2 - 1) / (chunk / 2) <= 128)
    chunk /= 2;
  while ((n_rows + chunk - 1) / chunk > 128) chunk *= 2;
  return chunk;
}

// ---- gradient of a second operand without channels ("u1v") --------------------------------------------------------
//   gy[n, b] = sum_{segments s = (p, a)} sum_{t in s} coef_t * sum_w g[n, M_t, w] * Z_s[n, w],
//   Z_s[n, w] = sum_k x[n, a, k] * W[p, k, w]
// The second operand is what is asked for, so nothing can be coupled before the channel contraction: a wavefront
// forms Z_s for 16 samples and 32 output channels on the matrix cores (operands: the packed weight of the forward
// and the plain row a of x staged in LDS), then takes the scalar products with the rows of g its segment's terms
// name.  The accumulator lane (sample r, group q) holds four consecutive channels of its sample, so a term costs two
// 16-byte loads of g (requested before the matrix instructions start), eight multiply-adds, a sum over the four
// groups and one LDS add into the wavefront's own (sample, b) array — no atomics between wavefronts; the arrays are
// added in wavefront order at the end.  Eight wavefronts share a workgroup's 16 samples: the segments are dealt round
// robin to groups of wavefronts, the blocks of 32 output channels within a group.
struct UvtGyDev {
  const real* x;
  const real* g;
  const real* wp;
  real* gy;
  const cgtp_uvt_item* items;   // segments: p, out_row = a, t0, t1
  const int32_t* ta;            // row M of g
  const int32_t* tb;            // row b of gy
  const real* tc;
  int64_t n_rows;
  int n_items, n_terms, dx, dy, dg, cx, cout;
  int kx, px, kblocks, wbp;
  int wchunks, wgroups;         // blocks of 32 output channels; wavefronts of a group that share a segment (1, 2, 4)
};

constexpr int kGyWB = sizeof(real) == 8 ? 1 : 2;   // blocks of 16 output channels per pass (registers: doubles take two)
constexpr int kGyWaves = 8;
// kGyRing (template argument): blocks of 16 k in flight = uvt_kbi(K), the packing pads k to whole multiples

// kGyHalves: sets of 16 samples per workgroup (1 or 2).  With two, a wavefront multiplies every weight fragment with
// the rows of both sets (two accumulator sets), which halves the requests to the L2 per matrix instruction — the
// rate of those requests, not the matrix pipeline, is what bounds this kernel.  Taken where the rows of 32 samples
// fit the LDS and the batch still fills the chip.
template <int kGyRing, int kGyHalves>
__global__ void __launch_bounds__(kGyWaves* kWave) uvt_grad_y_kernel(const UvtGyDev a) {
  constexpr int SW = 16 * kGyHalves;
  extern __shared__ __align__(16) unsigned char smem[];
  real* xs = reinterpret_cast<real*>(smem);
  real* part = xs + (size_t)SW * a.px;                       // [wavefront][sample][b]
  const int64_t nb0 = (int64_t)blockIdx.x * SW;
  {
    const int kx4 = a.kx / 4, per_sample = a.dx * kx4;
    for (int i = threadIdx.x; i < SW * per_sample; i += blockDim.x) {
      const int s = i / per_sample, rem = i - s * per_sample, row = rem / kx4, c4 = rem - row * kx4;
      const int64_t n = nb0 + s;
      realx4 v = {0.f, 0.f, 0.f, 0.f};
      if (n < a.n_rows && c4 * 4 < a.cx) v = *reinterpret_cast<const realx4*>(a.x + (n * a.dx + row) * a.cx + c4 * 4);
      *reinterpret_cast<realx4*>(xs + (size_t)s * a.px + row * a.kx + c4 * 4) = v;
    }
  }
  for (int i = threadIdx.x; i < kGyWaves * SW * a.dy; i += blockDim.x) part[i] = 0.f;
  const UvtTables tab = uvt_stage_tables(a, reinterpret_cast<unsigned char*>(part + kGyWaves * SW * a.dy));
  __syncthreads();

  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1), r = lane & 15, q = lane >> 4;
  const int wg = wave & (a.wgroups - 1), sg = wave / a.wgroups, sgroups = kGyWaves / a.wgroups;
  // samples past the end are staged as zeros (Z = 0); their rows of g are read from the last sample
  const real* gn[kGyHalves];
  real* mine[kGyHalves];
#pragma unroll
  for (int h = 0; h < kGyHalves; ++h) {
    const int64_t n = nb0 + 16 * h + r;
    gn[h] = a.g + (n < a.n_rows ? n : a.n_rows - 1) * a.dg * a.cout;
    mine[h] = part + (size_t)(wave * SW + 16 * h + r) * a.dy;
  }
  const real* xl = xs + (size_t)r * a.px + 4 * q;    // set h: 16 h px further
  const size_t xhalf = (size_t)16 * a.px;
  const realx4 zero = {0.f, 0.f, 0.f, 0.f};

  // The passes of this wavefront — (segment, block of 32 output channels) — form one sequence; the weight fragments
  // and the rows of x run kGyRing blocks of 16 k ahead of the matrix instructions, across the ends of the passes
  // (a weight fragment comes from the L2 in more cycles than one block's eight matrix instructions take).
  const int64_t kstride = (int64_t)a.wbp * 256;
  realx4 A[kGyRing][kGyWB], B[kGyRing][kGyHalves];
  auto load = [&](const real* wbase, const real* xrow, int kb, realx4 (&Aj)[kGyWB], realx4 (&Bj)[kGyHalves]) __attribute__((always_inline)) {
#pragma unroll
    for (int wb = 0; wb < kGyWB; ++wb) Aj[wb] = *reinterpret_cast<const realx4*>(wbase + kb * kstride + wb * 256);
#pragma unroll
    for (int h = 0; h < kGyHalves; ++h) Bj[h] = *reinterpret_cast<const realx4*>(xrow + h * xhalf + kb * 16);
  };
  auto wbase_of = [&](const cgtp_uvt_item& it, int wc) __attribute__((always_inline)) {
    return a.wp + ((int64_t)it.p * a.kblocks * a.wbp + wc * kGyWB) * 256 + lane * 4;
  };
  int s = sg, wc = wg;
  cgtp_uvt_item it = uvt_item_at(tab, s < a.n_items ? s : 0);
  const real* wbase = wbase_of(it, wc);
  const real* xrow = xl + it.out_row * a.kx;
  if (s < a.n_items) {
#pragma unroll
    for (int j = 0; j < kGyRing; ++j) load(wbase, xrow, j, A[j], B[j]);   // kblocks is a multiple of kGyRing
  }
  while (s < a.n_items) {
    // the pass after this one
    int s2 = s, wc2 = wc + a.wgroups;
    if (wc2 >= a.wchunks) {
      wc2 = wg;
      s2 = s + sgroups;
    }
    const bool more = s2 < a.n_items;
    const cgtp_uvt_item it2 = uvt_item_at(tab, more ? s2 : s);
    const real* wbase2 = more ? wbase_of(it2, wc2) : wbase;
    const real* xrow2 = more ? xl + it2.out_row * a.kx : xrow;

    const int n_t = it.t1 - it.t0;
    // the segment's first kUvtTerms terms in scalar registers (slots past the end: the first term again, never used)
    int mrow[kUvtTerms], brow[kUvtTerms];
    real c[kUvtTerms];
#pragma unroll
    for (int k = 0; k < kUvtTerms; ++k) {
      const int t = k < n_t ? it.t0 + k : it.t0;
      mrow[k] = n_t > 0 ? __builtin_amdgcn_readfirstlane(tab.ta[t]) * a.cout : 0;
      brow[k] = __builtin_amdgcn_readfirstlane(tab.tb[t]);
      c[k] = tab.tc[t];
    }
    const int wb0 = wc * kGyWB;
    int wcol[kGyWB];
    bool wok[kGyWB];
#pragma unroll
    for (int wb = 0; wb < kGyWB; ++wb) {
      const int w = (wb0 + wb) * 16 + 4 * q;       // cout is a multiple of 4: all four channels inside or outside
      wok[wb] = w < a.cout;
      wcol[wb] = wok[wb] ? w : 0;
    }
    // rows of g of the terms, requested before the matrix instructions: slots in pairs up to the segment's term count
    realx4 gv[kGyHalves][kUvtTerms][kGyWB];
#pragma unroll
    for (int h = 0; h < kUvtTerms; h += 2) {
      if (h == 0 || n_t > h) {
#pragma unroll
        for (int k = h; k < h + 2; ++k)
#pragma unroll
          for (int hs = 0; hs < kGyHalves; ++hs)
#pragma unroll
            for (int wb = 0; wb < kGyWB; ++wb)
              gv[hs][k][wb] = *reinterpret_cast<const realx4*>(gn[hs] + mrow[k] + wcol[wb]);
      }
    }

    realx4 acc[kGyHalves][kGyWB];
#pragma unroll
    for (int hs = 0; hs < kGyHalves; ++hs)
#pragma unroll
      for (int wb = 0; wb < kGyWB; ++wb) acc[hs][wb] = zero;
    for (int kb = 0; kb < a.kblocks; kb += kGyRing) {
      const bool wrap = kb + kGyRing >= a.kblocks;   // the blocks requested now belong to the next pass
      const real* wnext = wrap ? wbase2 : wbase;
      const real* xnext = wrap ? xrow2 : xrow;
      const int kbn = wrap ? 0 : kb + kGyRing;
#pragma unroll
      for (int j = 0; j < kGyRing; ++j) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int hs = 0; hs < kGyHalves; ++hs)
#pragma unroll
            for (int wb = 0; wb < kGyWB; ++wb)
              acc[hs][wb] = mfma16(A[j][wb][i], B[j][hs][i], acc[hs][wb], 0, 0, 0);
        load(wnext, xnext, kbn + j, A[j], B[j]);
      }
    }
    // accumulator: lane (sample r, q) holds Z[n, 16 (wb0 + wb) + 4 q + e]
    auto add_term = [&](const realx4 (&gt)[kGyWB], const realx4 (&z)[kGyWB], real* to, real coef, int b) __attribute__((always_inline)) {
      real d = 0.f;
#pragma unroll
      for (int wb = 0; wb < kGyWB; ++wb) {
        const realx4 gg = wok[wb] ? gt[wb] : zero;
#pragma unroll
        for (int e = 0; e < 4; ++e) d += gg[e] * z[wb][e];
      }
      d += __shfl_xor(d, 16);
      d += __shfl_xor(d, 32);
      if (q == 0) atomicAdd(to + b, coef * d);   // LDS, this wavefront's own array: in program order
    };
#pragma unroll
    for (int k = 0; k < kUvtTerms; ++k)
      if (k < n_t) {
#pragma unroll
        for (int hs = 0; hs < kGyHalves; ++hs) add_term(gv[hs][k], acc[hs], mine[hs], c[k], brow[k]);
      }
    for (int t = it.t0 + kUvtTerms; t < it.t1; ++t) {   // longer segments (large irreps only)
      const int m = __builtin_amdgcn_readfirstlane(tab.ta[t]) * a.cout;
      const int b = __builtin_amdgcn_readfirstlane(tab.tb[t]);
      const real coef = tab.tc[t];
#pragma unroll
      for (int hs = 0; hs < kGyHalves; ++hs) {
        realx4 gt[kGyWB];
#pragma unroll
        for (int wb = 0; wb < kGyWB; ++wb) gt[wb] = *reinterpret_cast<const realx4*>(gn[hs] + m + wcol[wb]);
        add_term(gt, acc[hs], mine[hs], coef, b);
      }
    }
    s = s2; wc = wc2; it = it2; wbase = wbase2; xrow = xrow2;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < SW * a.dy; i += blockDim.x) {
    const int64_t ni = nb0 + i / a.dy;
    if (ni < a.n_rows) {
      real sum = 0.f;
#pragma unroll
      for (int w = 0; w < kGyWaves; ++w) sum += part[w * SW * a.dy + i];
      a.gy[nb0 * a.dy + i] = sum;
    }
  }
}

struct UvtPlan {
  int wb, kbi, yc;
  bool two_sets_ok;
  int64_t per_block, fixed;
  int64_t lds;
  dim3 grid;
  unsigned threads;
  UvtDev dev;
};

static inline int round_up(int v, int m) { return (v + m - 1) / m * m; }
static inline int pow2_floor(int v) { int p = 1; while (p * 2 <= v) p *= 2; return p; }
static inline int pow2_ceil(int v) { int p = 1; while (p < v) p *= 2; return p; }

// Launch shape from the extents alone: LDS pitches, channel blocks per wavefront, and how a workgroup's (up to) eight
// wavefronts are spent: on groups of output rows first (they share everything staged and repeat no arithmetic), on
// blocks of output channels (they repeat the mixing), on further blocks of 16 samples when LDS and batch allow.
static int uvt_shape(int64_t n_rows, int dx, int dy, int dout, int cx, int cy, int cout, UvtPlan* plan) {
  if (n_rows < 0 || dx <= 0 || dy <= 0 || dout <= 0 || cx <= 0 || cy < 0 || cout <= 0) return CGTP_ERR_SHAPE;
  if (cx % 4 || cout % 4 || cy % 4) return CGTP_ERR_SHAPE;
  const bool yc = cy > 0;
  if (yc && ((int64_t)cx * cy) % 16) return CGTP_ERR_SHAPE;
  UvtDev& d = plan->dev;
  d.n_rows = n_rows; d.dx = dx; d.dy = dy; d.dout = dout; d.cx = cx; d.cy = cy; d.cout = cout;
  const int64_t K = yc ? (int64_t)cx * cy : cx;
  if (K > (1 << 24)) return CGTP_ERR_SHAPE;
  const int kbi = uvt_kbi(K);
  d.kblocks = round_up((int)((K + 15) / 16), kbi);   // whole turns of the fragment ring: the tail is zero weights
  d.kx = yc ? cx : d.kblocks * 16;
  d.px = dx * d.kx + 4;
  d.py = yc ? dy * cy + 4 : (dy | 1);
  const int wblocks = (cout + 15) / 16;
  d.wbp = round_up(wblocks, 4);
  // blocks of 16 output channels per wavefront; in double precision four blocks do not fit the registers
  const int wb = (wblocks >= 4 && sizeof(real) == 4) ? 4 : wblocks >= 2 ? 2 : 1;
  const int need = (wblocks + wb - 1) / wb;             // wavefronts (or workgroups) that cover the output channels
  int wgroups = need >= 2 ? 2 : 1;
  int igroups = pow2_floor(dout < kUvtMaxGroups / wgroups ? dout : kUvtMaxGroups / wgroups);
  while (wgroups < pow2_ceil(need) && wgroups * 2 * igroups <= kUvtMaxGroups) wgroups *= 2;
  d.zero_floats = yc ? round_up((cx > cy + 4 ? cx : cy + 4) + 4, 4) : d.kblocks * 16 + 16;
  const int64_t per_block = (int64_t)16 * (d.px + d.py) * (int64_t)sizeof(real);   // LDS bytes of one 16-sample block
  const int64_t fixed = (yc ? (int64_t)d.kblocks * 32 : 0) + (int64_t)d.zero_floats * (int64_t)sizeof(real) + 32;
  if (per_block + fixed > kLdsBytes - kUvtTableRoom) return CGTP_ERR_LDS;
  // further sample blocks: while wavefronts are left, two workgroups still fit a compute unit, and the batch is large
  // enough to fill the chip with such workgroups
  int sb_log2 = 0;
  const int64_t blocks16 = (n_rows + 15) / 16;
  while ((wgroups * igroups) << (sb_log2 + 1) <= kUvtMaxGroups &&
         (per_block << (sb_log2 + 1)) + fixed <= kLdsBytes / 2 - kUvtTableRoom && (blocks16 >> (sb_log2 + 1)) >= 512)
    ++sb_log2;
  // Two sets of samples per wavefront: the widest form of the kernel only (single precision, y without channels, 64
  // output channels per wavefront, a ring of four: one workgroup per compute unit anyway), where two workgroups per
  // compute unit remain in the batch; uvt_plan() takes it if the rows of 32 samples fit the LDS beside the tables.
  plan->two_sets_ok = sizeof(real) == 4 && !yc && wb == 4 && kbi == 4 && sb_log2 == 0 && blocks16 / 2 >= 512;
  plan->per_block = per_block; plan->fixed = fixed;
  d.sb_log2 = sb_log2; d.ns = 1; d.wgroups = wgroups; d.igroups = igroups;
  plan->wb = wb; plan->kbi = kbi; plan->yc = yc;
  plan->lds = (per_block << sb_log2) + fixed;
  plan->threads = (unsigned)((wgroups * igroups) << sb_log2) * kWave;
  plan->grid = dim3((unsigned)((blocks16 + (1 << sb_log2) - 1) >> sb_log2), (unsigned)((need + wgroups - 1) / wgroups));
  return CGTP_OK;
}

static int uvt_plan(const cgtp_uvt_args* a, UvtPlan* plan) {
  if (!a) return CGTP_ERR_NULL;
  if (a->dtype != kDtype) return CGTP_ERR_DTYPE;
  if (a->n_items < 0 || a->n_terms < 0) return CGTP_ERR_SHAPE;
  const int st = uvt_shape(a->n_rows, a->dx, a->dy, a->dout, a->cx, a->cy, a->cout, plan);
  if (st != CGTP_OK) return st;
  UvtDev& d = plan->dev;
  // the item list must be cut for this launch shape: cgtp_uvt_chunk(), cgtp_uvt_item_groups()
  if (a->kbi != plan->kbi || a->n_groups != d.igroups) return CGTP_ERR_SHAPE;
  if (a->group_ptr[0] != 0 || a->group_ptr[d.igroups] != a->n_items) return CGTP_ERR_SHAPE;
  for (int i = 0; i < d.igroups; ++i)
    if (a->group_ptr[i] > a->group_ptr[i + 1]) return CGTP_ERR_SHAPE;
  if (!a->x || !a->y || !a->wp || !a->out || (a->n_items && (!a->items || !a->term_a || !a->term_b || !a->term_c)))
    return CGTP_ERR_NULL;
  const uintptr_t al = reinterpret_cast<uintptr_t>(a->x) | reinterpret_cast<uintptr_t>(a->wp) |
                       reinterpret_cast<uintptr_t>(a->out) | (a->cy > 0 ? reinterpret_cast<uintptr_t>(a->y) : 0);
  if (al & 15u) return CGTP_ERR_ALIGN;
  d.x = (const real*)a->x; d.y = (const real*)a->y; d.wp = (const real*)a->wp; d.out = (real*)a->out;
  d.items = a->items; d.ta = a->term_a; d.tb = a->term_b; d.tc = (const real*)a->term_c;
  d.n_items = a->n_items; d.n_terms = a->n_terms;
  for (int i = 0; i <= kUvtMaxGroups; ++i) d.group_ptr[i] = i <= d.igroups ? a->group_ptr[i] : a->n_items;
  const int64_t tables = ((int64_t)a->n_items * 32 + (int64_t)a->n_terms * kTermBytes + 15) / 16 * 16;
  if (plan->two_sets_ok && 2 * plan->per_block + plan->fixed + tables <= kLdsBytes) {
    d.ns = 2;
    plan->lds = 2 * plan->per_block + plan->fixed;
    plan->grid.x = (unsigned)(((a->n_rows + 15) / 16 + 1) / 2);
  }
  plan->lds += tables;
  if (plan->lds > kLdsBytes) return CGTP_ERR_LDS;
  return CGTP_OK;
}

// ---- entry points of this precision (the C entry points below dispatch on dtype) ------------------------------

int64_t packed_elems(int32_t n_paths, int64_t K, int32_t cout) {
  if (n_paths < 0 || K <= 0 || cout <= 0) return 0;
  return (int64_t)n_paths * round_up((int)((K + 15) / 16), uvt_kbi(K)) * round_up((cout + 15) / 16, 4) * 256;
}

int pack_weights(const void* w, void* packed, int32_t n_paths, int64_t K, int32_t cout, int64_t stride_p,
                          int64_t stride_k, int64_t stride_c, int32_t dtype, void* stream) {
  if (dtype != kDtype) return CGTP_ERR_DTYPE;
  if (!w || !packed) return CGTP_ERR_NULL;
  if (n_paths < 0 || K <= 0 || cout <= 0 || K > (1 << 24)) return CGTP_ERR_SHAPE;
  if (reinterpret_cast<uintptr_t>(packed) & 15u) return CGTP_ERR_ALIGN;
  const int64_t n_vec = packed_elems(n_paths, K, cout) / 4;
  if (n_vec == 0) return CGTP_OK;
  hipLaunchKernelGGL(uvt_pack_kernel, dim3((unsigned)((n_vec + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const real*)w, (real*)packed, n_vec, (int)K, (int)cout,
                     round_up((int)((K + 15) / 16), uvt_kbi(K)), round_up((cout + 15) / 16, 4), stride_p, stride_k, stride_c);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

int chunk(int64_t n_rows, int32_t dx, int32_t dy, int32_t dout, int32_t cx, int32_t cy, int32_t cout) {
  UvtPlan plan;
  const int st = uvt_shape(n_rows, dx, dy, dout, cx, cy, cout, &plan);
  return st == CGTP_OK ? plan.kbi : -st;
}

int item_groups(int64_t n_rows, int32_t dx, int32_t dy, int32_t dout, int32_t cx, int32_t cy, int32_t cout) {
  UvtPlan plan;
  const int st = uvt_shape(n_rows, dx, dy, dout, cx, cy, cout, &plan);
  return st == CGTP_OK ? plan.dev.igroups : -st;
}

int validate(const cgtp_uvt_args* a) {
  UvtPlan plan;
  return uvt_plan(a, &plan);
}

int apply(const cgtp_uvt_args* a, void* stream) {
  UvtPlan plan;
  const int st = uvt_plan(a, &plan);
  if (st != CGTP_OK) return st;
  if (a->n_rows == 0 || a->n_items == 0) return CGTP_OK;
  void (*fn)(const UvtDev) = nullptr;
  if (plan.kbi == 4) {
    if (plan.yc) {
      fn = plan.wb == 2 ? uvt_apply_kernel<true, 2, 4> : uvt_apply_kernel<true, 1, 4>;
    } else {
      fn = plan.wb == 2 ? uvt_apply_kernel<false, 2, 4> : uvt_apply_kernel<false, 1, 4>;
    }
#ifndef CGTP_UVT_F64
    if (plan.wb == 4) fn = plan.yc ? uvt_apply_kernel<true, 4, 4> : plan.dev.ns == 2 ? uvt_apply_kernel<false, 4, 4, 2> : uvt_apply_kernel<false, 4, 4>;
#endif
  } else {
    if (plan.yc) {
      fn = plan.wb == 2 ? uvt_apply_kernel<true, 2, 2> : uvt_apply_kernel<true, 1, 2>;
    } else {
      fn = plan.wb == 2 ? uvt_apply_kernel<false, 2, 2> : uvt_apply_kernel<false, 1, 2>;
    }
#ifndef CGTP_UVT_F64
    if (plan.wb == 4) fn = plan.yc ? uvt_apply_kernel<true, 4, 2> : uvt_apply_kernel<false, 4, 2>;
#endif
  }
  if (plan.lds > 48 * 1024 &&
      hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)plan.lds) != hipSuccess)
    return CGTP_ERR_LDS;
  hipLaunchKernelGGL(fn, plan.grid, dim3(plan.threads), (size_t)plan.lds, (hipStream_t)stream, plan.dev);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

int64_t grad_w_workspace_bytes(int64_t n_rows, int32_t n_paths, int64_t K, int32_t cout) {
  if (n_rows <= 0 || n_paths <= 0 || K <= 0 || cout <= 0) return 0;
  const int64_t chunk = uvt_gw_chunk(n_rows, n_paths, K, cout);
  return ((n_rows + chunk - 1) / chunk) * n_paths * K * cout * (int64_t)sizeof(real);
}

int grad_w(const cgtp_uvt_gw_args* a, void* stream) {
  if (!a) return CGTP_ERR_NULL;
  if (a->dtype != kDtype) return CGTP_ERR_DTYPE;
  if (a->n_rows < 0 || a->n_paths <= 0 || a->n_items < 0 || a->dx <= 0 || a->dy <= 0 || a->dg <= 0 || a->cx <= 0 ||
      a->cy < 0 || a->cout <= 0)
    return CGTP_ERR_SHAPE;
  if (!a->x || !a->y || !a->g || !a->gw || !a->path_ptr || (a->n_items && (!a->items || !a->term_a || !a->term_b || !a->term_c)))
    return CGTP_ERR_NULL;
  const int64_t K = a->cy > 0 ? (int64_t)a->cx * a->cy : a->cx;
  if (K > (1 << 24)) return CGTP_ERR_SHAPE;
  if (K % 4 || a->cout % 4 || a->cy % 4) return CGTP_ERR_SHAPE;   // 16-byte operand loads
  if ((reinterpret_cast<uintptr_t>(a->x) | reinterpret_cast<uintptr_t>(a->g) | (a->cy > 0 ? reinterpret_cast<uintptr_t>(a->y) : 0)) & 15u)
    return CGTP_ERR_ALIGN;
  // the partial results and the gradient are summed four elements at a time
  if ((reinterpret_cast<uintptr_t>(a->gw) | reinterpret_cast<uintptr_t>(a->workspace)) & (sizeof(realx4) - 1)) return CGTP_ERR_ALIGN;
  const int64_t n_out = (int64_t)a->n_paths * K * a->cout;
  hipStream_t st = (hipStream_t)stream;
  if (a->n_rows == 0) {   // no samples: the gradient is zero (written by the summation kernel over zero chunks)
    hipLaunchKernelGGL(uvt_gw_reduce_kernel, dim3((unsigned)((n_out / 4 + kGwReduceCols - 1) / kGwReduceCols)),
                       dim3(kGwReduceCols * kGwReduceSlices), 0, st, (const real*)nullptr, (real*)a->gw, (int64_t)0,
                       n_out / 4);
    return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
  }
  if (!a->workspace) return CGTP_ERR_WORKSPACE;
  UvtGwDev d;
  d.x = (const real*)a->x; d.y = (const real*)a->y; d.g = (const real*)a->g; d.part = (real*)a->workspace;
  d.items = a->items; d.path_ptr = a->path_ptr; d.ta = a->term_a; d.tb = a->term_b; d.tc = (const real*)a->term_c;
  d.n_rows = a->n_rows; d.n_paths = a->n_paths; d.dx = a->dx; d.dy = a->dy; d.dg = a->dg; d.cx = a->cx; d.cy = a->cy;
  d.cout = a->cout; d.K = (int)K;
  d.chunk = (int)uvt_gw_chunk(a->n_rows, a->n_paths, K, a->cout);
  const int64_t n_chunks = (a->n_rows + d.chunk - 1) / d.chunk;
  const int narrow = uvt_gw_narrow(K, a->cout);
  const int64_t zblocks = uvt_gw_blocks(K, a->cout);
  if (zblocks > 65535 || a->n_paths > 65535) return CGTP_ERR_SHAPE;
  dim3 grid((unsigned)n_chunks, (unsigned)a->n_paths, (unsigned)zblocks);
  if (uvt_gw_small(K, a->cout)) {
    const bool yc = a->cy > 0, ki = K <= 32, wj = a->cout <= 32;      // two channels a lane where 32 cover the axis
    void (*small)(const UvtGwDev) =
        ki ? (wj ? (yc ? uvt_grad_w_small_kernel<true, 2, 2> : uvt_grad_w_small_kernel<false, 2, 2>)
                 : (yc ? uvt_grad_w_small_kernel<true, 2, 4> : uvt_grad_w_small_kernel<false, 2, 4>))
           : (wj ? (yc ? uvt_grad_w_small_kernel<true, 4, 2> : uvt_grad_w_small_kernel<false, 4, 2>)
                 : (yc ? uvt_grad_w_small_kernel<true, 4, 4> : uvt_grad_w_small_kernel<false, 4, 4>));
    hipLaunchKernelGGL(small, dim3((unsigned)n_chunks, (unsigned)a->n_paths), dim3(kWave), 0, st, d);
    if (hipGetLastError() != hipSuccess) return CGTP_ERR_LAUNCH;
    hipLaunchKernelGGL(uvt_gw_reduce_kernel, dim3((unsigned)((n_out / 4 + kGwReduceCols - 1) / kGwReduceCols)),
                       dim3(kGwReduceCols * kGwReduceSlices), 0, st, (const real*)a->workspace, (real*)a->gw, n_chunks,
                       n_out / 4);
    return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
  }
  void (*fn)(const UvtGwDev) = a->cy > 0 ? uvt_grad_w_kernel<true, 0> : uvt_grad_w_kernel<false, 0>;
#ifndef CGTP_UVT_F64
  if (narrow == 1) fn = a->cy > 0 ? uvt_grad_w_kernel<true, 1> : uvt_grad_w_kernel<false, 1>;
  if (narrow == 2) fn = a->cy > 0 ? uvt_grad_w_kernel<true, 2> : uvt_grad_w_kernel<false, 2>;
#endif
  hipLaunchKernelGGL(fn, grid, dim3(256), 0, st, d);
  if (hipGetLastError() != hipSuccess) return CGTP_ERR_LAUNCH;
  hipLaunchKernelGGL(uvt_gw_reduce_kernel, dim3((unsigned)((n_out / 4 + kGwReduceCols - 1) / kGwReduceCols)),
                     dim3(kGwReduceCols * kGwReduceSlices), 0, st, (const real*)a->workspace, (real*)a->gw, n_chunks,
                     n_out / 4);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

int grad_y(const cgtp_uvt_gy_args* a, void* stream) {
  if (!a) return CGTP_ERR_NULL;
  if (a->dtype != kDtype) return CGTP_ERR_DTYPE;
  if (a->n_rows < 0 || a->n_items < 0 || a->n_terms < 0 || a->dx <= 0 || a->dy <= 0 || a->dg <= 0 || a->cx <= 0 ||
      a->cout <= 0)
    return CGTP_ERR_SHAPE;
  if (a->cx % 4 || a->cout % 4) return CGTP_ERR_SHAPE;
  if (!a->x || !a->g || !a->wp || !a->gy || (a->n_items && (!a->items || !a->term_m || !a->term_b || !a->term_c)))
    return CGTP_ERR_NULL;
  if ((reinterpret_cast<uintptr_t>(a->x) | reinterpret_cast<uintptr_t>(a->g) | reinterpret_cast<uintptr_t>(a->wp)) & 15u)
    return CGTP_ERR_ALIGN;
  UvtGyDev d;
  d.x = (const real*)a->x; d.g = (const real*)a->g; d.wp = (const real*)a->wp; d.gy = (real*)a->gy;
  d.items = a->items; d.ta = a->term_m; d.tb = a->term_b; d.tc = (const real*)a->term_c;
  d.n_rows = a->n_rows; d.n_items = a->n_items; d.n_terms = a->n_terms;
  d.dx = a->dx; d.dy = a->dy; d.dg = a->dg; d.cx = a->cx; d.cout = a->cout;
  const int ring = uvt_kbi(a->cx);
  d.kblocks = round_up((a->cx + 15) / 16, ring);
  d.kx = d.kblocks * 16;
  d.px = a->dx * d.kx + 4;
  d.wbp = round_up((a->cout + 15) / 16, 4);
  d.wchunks = (a->cout + 16 * kGyWB - 1) / (16 * kGyWB);
  d.wgroups = d.wchunks >= 4 ? 4 : d.wchunks >= 2 ? 2 : 1;
  auto lds_of = [&](int halves) {
    return ((int64_t)16 * halves * d.px + (int64_t)kGyWaves * 16 * halves * a->dy) * (int64_t)sizeof(real) +
           (int64_t)a->n_items * 32 + (int64_t)a->n_terms * kTermBytes + 16;
  };
  // Two sets of 16 samples per workgroup: single precision (the doubles' registers do not take a second set of g
  // rows), the rows of 32 samples fit the LDS, at least two workgroups per compute unit remain — and the kernel with
  // one set would not have two workgroups on a compute unit to gain from: a ring of four (151 registers), or walk
  // tables, which every workgroup copies, a third as large as its rows of x.  lmax = 2, 32768 samples, 128 -> 128
  // channels: 590 -> 518 us; lmax = 4, 16384 samples, 32 -> 32: 463 -> 372 us; where two workgroups of the one-set
  // kernel fit, they are faster (64 -> 64, lmax = 3: 563 against 616 us).
  const int64_t table_bytes = (int64_t)a->n_items * 32 + (int64_t)a->n_terms * kTermBytes;
  const bool one_wg_anyway = ring == 4 || 3 * table_bytes >= (int64_t)16 * d.px * (int64_t)sizeof(real);
  const int halves = sizeof(real) == 4 && one_wg_anyway && lds_of(2) <= kLdsBytes && a->n_rows >= 32 * 512 ? 2 : 1;
  const int64_t lds = lds_of(halves);
  if (lds > kLdsBytes) return CGTP_ERR_LDS;
  if (a->n_rows == 0) return CGTP_OK;
  void (*fn)(const UvtGyDev) = halves == 2 ? (ring == 4 ? uvt_grad_y_kernel<4, 2> : uvt_grad_y_kernel<2, 2>)
                                           : (ring == 4 ? uvt_grad_y_kernel<4, 1> : uvt_grad_y_kernel<2, 1>);
  if (lds > 48 * 1024 && hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return CGTP_ERR_LDS;
  const int64_t per_wg = 16 * halves;
  hipLaunchKernelGGL(fn, dim3((unsigned)((a->n_rows + per_wg - 1) / per_wg)), dim3(kGyWaves * kWave), (size_t)lds, (hipStream_t)stream, d);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}


}  // namespace UVT_NS
}  // namespace cgtp

#ifndef CGTP_UVT_F64
// The double-precision set of the same kernels and entry points: uvt_kernels_f64.hip compiles this file with
// CGTP_UVT_F64 defined.
namespace cgtp {
namespace uvt_f64 {
int pack_weights(const void* w, void* packed, int32_t n_paths, int64_t K, int32_t cout, int64_t stride_p, int64_t stride_k,
                 int64_t stride_c, int32_t dtype, void* stream);
int chunk(int64_t n_rows, int32_t dx, int32_t dy, int32_t dout, int32_t cx, int32_t cy, int32_t cout);
int item_groups(int64_t n_rows, int32_t dx, int32_t dy, int32_t dout, int32_t cx, int32_t cy, int32_t cout);
int validate(const cgtp_uvt_args* a);
int apply(const cgtp_uvt_args* a, void* stream);
int64_t grad_w_workspace_bytes(int64_t n_rows, int32_t n_paths, int64_t K, int32_t cout);
int grad_w(const cgtp_uvt_gw_args* a, void* stream);
int grad_y(const cgtp_uvt_gy_args* a, void* stream);
}  // namespace uvt_f64
}  // namespace cgtp

using namespace cgtp;

extern "C" {

int64_t cgtp_uvt_packed_elems(int32_t n_paths, int64_t K, int32_t cout) { return uvt_f32::packed_elems(n_paths, K, cout); }

int cgtp_uvt_pack_weights(const void* w, void* packed, int32_t n_paths, int64_t K, int32_t cout, int64_t stride_p,
                          int64_t stride_k, int64_t stride_c, int32_t dtype, void* stream) {
  return dtype == CGTP_F64 ? uvt_f64::pack_weights(w, packed, n_paths, K, cout, stride_p, stride_k, stride_c, dtype, stream)
                           : uvt_f32::pack_weights(w, packed, n_paths, K, cout, stride_p, stride_k, stride_c, dtype, stream);
}

int cgtp_uvt_chunk(int64_t n_rows, int32_t dx, int32_t dy, int32_t dout, int32_t cx, int32_t cy, int32_t cout,
                   int32_t dtype) {
  if (dtype != CGTP_F32 && dtype != CGTP_F64) return -CGTP_ERR_DTYPE;
  return dtype == CGTP_F64 ? uvt_f64::chunk(n_rows, dx, dy, dout, cx, cy, cout) : uvt_f32::chunk(n_rows, dx, dy, dout, cx, cy, cout);
}

int cgtp_uvt_item_groups(int64_t n_rows, int32_t dx, int32_t dy, int32_t dout, int32_t cx, int32_t cy, int32_t cout,
                         int32_t dtype) {
  if (dtype != CGTP_F32 && dtype != CGTP_F64) return -CGTP_ERR_DTYPE;
  return dtype == CGTP_F64 ? uvt_f64::item_groups(n_rows, dx, dy, dout, cx, cy, cout)
                           : uvt_f32::item_groups(n_rows, dx, dy, dout, cx, cy, cout);
}

int cgtp_uvt_validate(const cgtp_uvt_args* a) {
  return a && a->dtype == CGTP_F64 ? uvt_f64::validate(a) : uvt_f32::validate(a);
}

int cgtp_uvt_apply(const cgtp_uvt_args* a, void* stream) {
  return a && a->dtype == CGTP_F64 ? uvt_f64::apply(a, stream) : uvt_f32::apply(a, stream);
}

int64_t cgtp_uvt_grad_w_workspace_bytes(int64_t n_rows, int32_t n_paths, int64_t K, int32_t cout, int32_t dtype) {
  return dtype == CGTP_F64 ? uvt_f64::grad_w_workspace_bytes(n_rows, n_paths, K, cout)
                           : uvt_f32::grad_w_workspace_bytes(n_rows, n_paths, K, cout);
}

int cgtp_uvt_grad_w(const cgtp_uvt_gw_args* a, void* stream) {
  return a && a->dtype == CGTP_F64 ? uvt_f64::grad_w(a, stream) : uvt_f32::grad_w(a, stream);
}

int cgtp_uvt_grad_y(const cgtp_uvt_gy_args* a, void* stream) {
  return a && a->dtype == CGTP_F64 ? uvt_f64::grad_y(a, stream) : uvt_f32::grad_y(a, stream);
}

}  // extern "C"
#endif  // CGTP_UVT_F64
