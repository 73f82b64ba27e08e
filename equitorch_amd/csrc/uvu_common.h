// Kernel-side argument block and lane decomposition shared by the channel-wise ("uvu") tensor-product kernels.
#pragma once

#include "cgtp_device.h"
#include "cgtp_host.h"

namespace cgtp {

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
  T* ws;   // segment mode: partial rows (n_waves, 2, D, C)
  T* wsw;  // per-wavefront partial sums of a shared weight's gradient (n_waves, P, C)
  const int64_t* ptr;
  const int64_t* perm;
  const int64_t* gather;
  const int64_t* x_gather;  // row mode backward: optional row of x per batch row
  const int64_t* seg_ids;
  const int32_t* wave_seg;  // segment mode: optional wavefront -> first segment table (segment-aligned ranges)
  const int64_t* wave_pos;  // segment mode: optional wavefront -> first sorted position table (ranges cut anywhere)
  int64_t n_rows, n_seg, n_waves;
  int C, lpe_log2, w_shared, pos_per_wave;
  int y_vec;  // segment mode: y holds edge vectors (kYUnitVector / kYRawVector) instead of harmonics
  const T* ps;  // optional factor of every weight path (the caller's table = compiled table x ps[p]); nullptr = ones
  // weights produced in the kernel: w[e, p, c] = sum_r rh[e, r] * rw[r, p, c] (segment mode, fp32, C = 64)
  const T* rh;   // (n_rows, R)
  const T* rw;   // (R, P, C)
  int R;
};

// Segment mode: which range of the sorted edge list a wavefront takes.  Workgroups are dispatched to the 8 XCDs
// round-robin (workgroup b runs on XCD b % 8); handing XCD k the k-th contiguous eighth of the ranges keeps the rows
// gathered by one XCD's wavefronts — rows near its own segments when edges connect nearby nodes — inside that
// XCD's L2.  Returns -1 for the padding workgroups of the last eighth.
__device__ __forceinline__ int64_t seg_wave_index(int64_t n_waves) {
  const int waves_per_block = blockDim.x / kWave;
  const int64_t blocks = (n_waves + waves_per_block - 1) / waves_per_block;
  const int64_t per_xcd = (blocks + 7) / 8;
  const int64_t block = (int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if ((int64_t)(blockIdx.x >> 3) >= per_xcd || block >= blocks) return -1;
  // the wavefront's number within the workgroup as a scalar: everything derived from it (range, segment ids,
  // flags) then lives in scalar registers
  const int64_t wave = block * waves_per_block + __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
  return wave < n_waves ? wave : -1;
}

struct Lanes {
  int lane, lpe, slots, slot, cl;
  __device__ __forceinline__ explicit Lanes(int lpe_log2) {
    lane = threadIdx.x & (kWave - 1);
    lpe = 1 << lpe_log2;
    slots = kWave >> lpe_log2;
    slot = lane >> lpe_log2;
    cl = lane & (lpe - 1);
  }
};

// What the backward does with the weight gradient.  kGwReduce: the weight is shared over rows, so its gradient
// is summed over every row a wavefront visits and written as one partial per wavefront into the workspace
// (partial_sum_kernel finishes the sum).  A compile-time choice keeps the generated body free of branches.
enum { kGwNone = 0, kGwStore = 1, kGwReduce = 2 };

// Block-wise kernels (uvu_big.hip): fp32, row mode, one channel per lane.  They write the weight gradient per row;
// for a shared weight the caller sums the rows.
struct UvuBigEntry {
  uint64_t fingerprint;
  uint64_t fingerprint_rounded[2];  // of the table rounded to bf16 / fp16
  int dims[5];
  const char* name;
  const float* coef;                // the compiled table, table order
  const unsigned char (*idx)[4];    // (M, M1, M2, p) per entry
  void (*fwd)(const UvuDev<float>);
  void (*bwd[2])(const UvuDev<float>, int64_t);  // [kGwNone, kGwStore]
  // the same with a channelled second operand, y (n_rows, D2, C) ("uuu"): grad_y is then per channel as well
  void (*fwd_yc)(const UvuDev<float>);
  void (*bwd_yc[2])(const UvuDev<float>, int64_t);
  // segment mode (gather, product and segment sum fused); dynamic LDS: 4 x rows x 64 floats per workgroup, the
  // backward 5120 bytes more (staged indices and per-lane state)
  void (*seg_fwd)(const UvuDev<float>, int64_t);
  void (*seg_bwd[2])(const UvuDev<float>, int64_t);
};
// Segment-mode kernels that form the per-edge weights from per-edge features and a shared matrix (uvu_radial.hip);
// [0]: second operand given as harmonics, [1]: as edge vectors (nullptr where the config has no such form).
struct UvuRadialEntry {
  void (*fwd[2])(const UvuDev<float>, int64_t);
  void (*bwd[2][2])(const UvuDev<float>, int64_t);   // [.][weight gradient written per edge]
  int lds_floats_per_r;   // LDS floats per row of the shared matrix
};
const UvuRadialEntry* uvu_radial_entries(int* count);
constexpr int kRadialMaxR = 16;
constexpr int kRadialC = 64;

// The fix-up pass of the segment kernels for callers outside their translation unit: adds the partial rows
// ws[(range, 2, row_len)] of the segments that span several ranges (ranges of `per_range` sorted positions each) in
// range order, and writes zero rows for empty segments.  Status code.
int uvu_fixup_rows_f32(float* rows, const float* ws, const int64_t* ptr, int64_t n_seg, int64_t row_len, int per_range,
                       int64_t n_ranges, int64_t n_rows, hipStream_t stream);

const UvuBigEntry* uvu_big_entries(int* count);
const UvuBigEntry* uvu_big_entries_scaled(int* count);  // the same kernels applying UvuDev::ps

}  // namespace cgtp
