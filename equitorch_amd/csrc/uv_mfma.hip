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

// Z_t[w, n] = sum_k A_t[w, k] * B[k, n] for the two channel tiles t over KS steps of 32; xs points at this lane's
// 8 consecutive k of step 0.
template <int KS>
__device__ __forceinline__ void mfma_chain(const bf16x8 (&a)[2][KS], const unsigned char* xs, floatx4& z0,
                                           floatx4& z1) {
  z0 = floatx4{0.f, 0.f, 0.f, 0.f};
  z1 = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int k = 0; k < KS; ++k) {
    const bf16x8 b = *reinterpret_cast<const bf16x8*>(xs + k * 64);
    z0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[0][k], b, z0, 0, 0, 0);
    z1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[1][k], b, z1, 0, 0, 0);
  }
}

#include "generated/uv_configs.inc"

constexpr int kUvSamples = 16;

template <class CFG, int CIN>
__global__ void __launch_bounds__(256, 2) uv_kernel(const __bf16* __restrict__ x, const __bf16* __restrict__ y,
                                                    const __bf16* __restrict__ wt, __bf16* __restrict__ out,
                                                    int64_t n_rows, int cout) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int DIN = CFG::DIN, DOUT = CFG::DOUT, D2 = CFG::D2;
  constexpr int ROW_BYTES = DIN * CIN * 2;      // one sample's input rows
  constexpr int ROW_PITCH = ROW_BYTES + 16;     // + pad: consecutive samples start 16 B further in the banks
  const int64_t n0 = (int64_t)blockIdx.x * kUvSamples;

  // stage the 16 samples' rows: 16-byte pieces, coalesced in global memory
  constexpr int PIECES = ROW_BYTES / 16;
  for (int i = threadIdx.x; i < kUvSamples * PIECES; i += blockDim.x) {
    const int s = i / PIECES, c = i % PIECES;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (n0 + s < n_rows)
      v = *reinterpret_cast<const f32x4*>(reinterpret_cast<const unsigned char*>(x) + (n0 + s) * ROW_BYTES + c * 16);
    *reinterpret_cast<f32x4*>(smem + s * ROW_PITCH + c * 16) = v;
  }
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int n = lane & 15, q = lane >> 4;
  const bool valid = n0 + n < n_rows;
  float yv[D2];
#pragma unroll
  for (int j = 0; j < D2; ++j) yv[j] = valid ? (float)y[(n0 + n) * D2 + j] : 0.f;
  const unsigned char* xs = smem + n * ROW_PITCH + q * 16;

  // one 32-channel block per wavefront, blockIdx.y tiles wider outputs
  const int wblk = blockIdx.y * (blockDim.x / kWave) + wave;
  if (wblk * 32 >= cout) return;
  // Row r = 4*g + i of channel tile t is output channel wblk*32 + 8*g + 4*t + i, so that in the accumulator layout
  // (lane (n, q) holds rows 4*q .. 4*q+3 of column n) a lane ends up with 8 consecutive channels of its sample.
  // A fragment: lane (r = lane & 15, q) holds Wt[p][channel(t, r)][k*32 + q*8 .. +8]
  const __bf16* wrow = wt + (int64_t)(wblk * 32 + 8 * (n >> 2) + (n & 3)) * CIN + q * 8;
  const int64_t path_stride = (int64_t)cout * CIN;
  __bf16* orow = out + (n0 + n) * DOUT * cout + wblk * 32 + 8 * q;
  CFG::template run<CIN>(
      xs,
      [&](int p, bf16x8(&frag)[2][CIN / 32]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int k = 0; k < CIN / 32; ++k)
            frag[t][k] = *reinterpret_cast<const bf16x8*>(wrow + p * path_stride + t * 4 * CIN + k * 32);
      },
      yv,
      [&](int row, const floatx4& o0, const floatx4& o1) __attribute__((always_inline)) {
        if (valid) {
          bf16x8 v;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            v[i] = (__bf16)o0[i];
            v[4 + i] = (__bf16)o1[i];
          }
          *reinterpret_cast<bf16x8*>(orow + row * cout) = v;
        }
      });
}

using UvFn = void (*)(const __bf16*, const __bf16*, const __bf16*, __bf16*, int64_t, int);

struct UvEntry {
  uint64_t fingerprint;
  const char* name;
  int din[2], dout[2], d2, p;
  UvFn fn[2][3];  // [direction][C_in = 32, 64, 128]
};

template <class D0, class D1>
static UvEntry make_uv_entry(uint64_t fp, const char* name) {
  UvEntry e;
  e.fingerprint = fp; e.name = name;
  e.din[0] = D0::DIN; e.dout[0] = D0::DOUT; e.din[1] = D1::DIN; e.dout[1] = D1::DOUT;
  e.d2 = D0::D2; e.p = D0::P;
  e.fn[0][0] = uv_kernel<D0, 32>; e.fn[0][1] = uv_kernel<D0, 64>; e.fn[0][2] = uv_kernel<D0, 128>;
  e.fn[1][0] = uv_kernel<D1, 32>; e.fn[1][1] = uv_kernel<D1, 64>; e.fn[1][2] = uv_kernel<D1, 128>;
  return e;
}

static const UvEntry* uv_entries(int* count) {
#define CGTP_X(D0, D1, FP, NAME) make_uv_entry<D0, D1>(FP, NAME),
  static const UvEntry table[] = {CGTP_FOREACH_UV_CONFIG(CGTP_X)};
#undef CGTP_X
  *count = (int)(sizeof(table) / sizeof(table[0]));
  return table;
}

static int uv_check(int cfg, int direction, const void* x, const void* y, const void* wt, const void* out,
                    int64_t n_rows, int cin, int cout, int dtype, int* ci, int64_t* lds) {
  int n = 0;
  const UvEntry* t = uv_entries(&n);
  if (cfg < 0 || cfg >= n) return CGTP_ERR_CONFIG;
  if (direction != 0 && direction != 1) return CGTP_ERR_SHAPE;
  if (dtype != CGTP_BF16) return CGTP_ERR_DTYPE;
  if (!x || !y || !wt || !out) return CGTP_ERR_NULL;
  if (n_rows < 0 || cout <= 0 || cout % 32 != 0) return CGTP_ERR_SHAPE;
  *ci = cin == 32 ? 0 : cin == 64 ? 1 : cin == 128 ? 2 : -1;
  if (*ci < 0) return CGTP_ERR_SHAPE;
  const uintptr_t al = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(wt) | reinterpret_cast<uintptr_t>(out);
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

int cgtp_uv_validate(int cfg, int direction, const void* x, const void* y, const void* wt, const void* out,
                     int64_t n_rows, int32_t cin, int32_t cout, int32_t dtype) {
  int ci = 0;
  int64_t lds = 0;
  return uv_check(cfg, direction, x, y, wt, out, n_rows, cin, cout, dtype, &ci, &lds);
}

int cgtp_uv_apply(int cfg, int direction, const void* x, const void* y, const void* wt, void* out, int64_t n_rows,
                  int32_t cin, int32_t cout, int32_t dtype, void* stream) {
  int ci = 0;
  int64_t lds = 0;
  const int st = uv_check(cfg, direction, x, y, wt, out, n_rows, cin, cout, dtype, &ci, &lds);
  if (st != CGTP_OK) return st;
  if (n_rows == 0) return CGTP_OK;
  int n = 0;
  UvFn fn = uv_entries(&n)[cfg].fn[direction][ci];
  if (hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return CGTP_ERR_LDS;
  hipLaunchKernelGGL(fn, dim3((unsigned)((n_rows + kUvSamples - 1) / kUvSamples), (unsigned)((cout + 127) / 128)),
                     dim3(256), (size_t)lds,
                     (hipStream_t)stream, (const __bf16*)x, (const __bf16*)y, (const __bf16*)wt, (__bf16*)out, n_rows,
                     (int)cout);
  return hipGetLastError() == hipSuccess ? CGTP_OK : CGTP_ERR_LAUNCH;
}

}  // extern "C"
