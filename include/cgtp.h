/*
 * cgtp — sparse Clebsch-Gordan tensor-product kernels for AMD gfx950 (MI355X), C ABI.
 *
 * Every entry point takes raw device pointers, extents and a HIP stream (passed as void*; NULL = the null
 * stream), enqueues its kernels on that stream and returns immediately with a status code.  Nothing here
 * allocates, frees or synchronises; buffers (including workspaces) are owned by the caller.  Tensors use
 * the Equitorch layout (batch, irreps_dim, channels), channel-last and contiguous unless a stride is given.
 *
 * The reference (GTML-LAB/Equitorch) has no FFI: its boundary is the Python signature of the Triton launch
 * wrappers.  Each declaration below names the wrapper it stands in for.
 */
#ifndef CGTP_H
#define CGTP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status codes ---------------------------------------------------------------------------------- */
enum {
  CGTP_OK = 0,
  CGTP_ERR_NULL = 1,        /* a required pointer is NULL                                   */
  CGTP_ERR_SHAPE = 2,       /* negative / zero / inconsistent extent                        */
  CGTP_ERR_ALIGN = 3,       /* pointer or stride not aligned for the requested vector width */
  CGTP_ERR_DTYPE = 4,       /* unsupported element type                                     */
  CGTP_ERR_CONFIG = 5,      /* unknown specialised-table id                                 */
  CGTP_ERR_LDS = 6,         /* table does not fit the 160 KB LDS of a CU                    */
  CGTP_ERR_LAUNCH = 7,      /* hipLaunchKernel reported an error                            */
  CGTP_ERR_WORKSPACE = 8,   /* workspace missing or too small                               */
  CGTP_ERR_SCRATCH_LIMIT = 9 /* cgtp_tri_contract_static: partial results beyond the fixed scratch array */
};

enum { CGTP_F32 = 0, CGTP_F64 = 1, CGTP_BF16 = 2, CGTP_F16 = 3 };

const char* cgtp_status_string(int status);
/* ABI version; bumped on any signature change. */
int cgtp_version(void);
/* Layout of the argument structs as this library was compiled, so that a binding that mirrors them by hand (ctypes,
 * cgo, JNI) can check itself: which = CGTP_LAYOUT_*; writes sizeof(struct) followed by the byte offset of every field
 * in declaration order to out[0 .. capacity) and returns how many numbers the full description has (-1: bad id). */
enum { CGTP_LAYOUT_OPERAND = 0, CGTP_LAYOUT_TRI_ARGS = 1, CGTP_LAYOUT_GEN_OPERAND = 2, CGTP_LAYOUT_GEN_ARGS = 3,
       CGTP_LAYOUT_UVU_ARGS = 4, CGTP_LAYOUT_UVT_ITEM = 5, CGTP_LAYOUT_UVT_ARGS = 6, CGTP_LAYOUT_UVT_GW_ARGS = 7,
       CGTP_LAYOUT_UVT_GY_ARGS = 8, CGTP_LAYOUT_UVU_TABLE = 9, CGTP_LAYOUT_PSW_TABLE = 10, CGTP_LAYOUT_PSW_ARGS = 11 };
int cgtp_abi_layout(int which, int64_t* out, int capacity);

/* ---- generic sparse trilinear contraction -------------------------------------------------------------
 *
 *   out[r, o, c] = sum_{t in [seg[o], seg[o+1])} coef[t] * A[ra(r), ia[t], c] * B[rb(r), ib[t], (c)]
 *                                                        * W[rw(r), iw[t], c]
 *
 * with each operand optional, per-channel ("vec") or channel-less ("scalar"), per-row or shared, and
 * optionally row-gathered.  Covers, with the reference's own tables, indexed_mul / vecsca / scavec / inner
 * _scale_gather (equitorch/ops/batched_sparse_dense_op.py:156-232, 1665-1750, 994-1035, 713-788) and both
 * stages of the u1u / 1uu / uu1 / uuu tensor products (equitorch/nn/functional/linears.py:16-252,
 * equitorch/nn/functional/tensor_products.py:9-90) in one launch.  The table (coef, packed indices, seg)
 * is staged into LDS by every workgroup.
 */
enum { CGTP_OPERAND_NONE = 0, CGTP_OPERAND_VEC = 1, CGTP_OPERAND_SCALAR = 2 };

typedef struct cgtp_operand {
  const void* data;        /* element type = args.dtype                                         */
  const int64_t* rows;     /* optional: row r reads data row rows[r]; NULL = identity           */
  int64_t row_stride;      /* elements between rows; 0 = one row shared by every r              */
  int64_t idx_stride;      /* elements between consecutive sparse indices (C for vec, 1 scalar) */
  int32_t kind;            /* CGTP_OPERAND_*                                                    */
  int32_t size;            /* extent of the sparse index axis, or 0 if unknown (known extents let the kernel
                              stage the operand in LDS)                                            */
} cgtp_operand;

typedef struct cgtp_tri_args {
  cgtp_operand a, b, w;
  /* table, all device pointers */
  const void* coef;        /* [nnz] element type = dtype (f32 or f64); NULL = all ones           */
  const uint32_t* idx;     /* [nnz] packed ia | ib << 10 | iw << 20 (each < 1024, iw < 4096)     */
  const int32_t* seg;      /* [n_out + 1]                                                        */
  int32_t n_out, nnz;
  /* output */
  void* out;               /* (n_rows, n_out, C), (n_rows, n_out) if reduce_c, row axis dropped if reduce_rows */
  void* workspace;         /* reduce_rows only: cgtp_tri_workspace_bytes() bytes                   */
  int64_t n_rows;
  int32_t C;
  int32_t dtype;           /* CGTP_F32 | CGTP_F64                                                  */
  int32_t reduce_c;        /* sum over channels (inner-product family)                             */
  int32_t reduce_rows;     /* sum over rows (gradient of an operand shared across the batch)      */
} cgtp_tri_args;

int64_t cgtp_tri_workspace_bytes(const cgtp_tri_args* args);
/* Host-only validation of the same conditions the launch checks; needs no device. */
int cgtp_tri_validate(const cgtp_tri_args* args);
int cgtp_tri_contract(const cgtp_tri_args* args, void* stream);

/* cgtp_tri_contract for callers that cannot allocate device memory or pass a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  args->workspace
 * is ignored; when reduce_rows != 0 the partial rows of the sum over rows live in a fixed device array inside the
 * library (cgtp_tri_static_scratch_bytes() = 16 MiB per device, held until the process ends).  A launch whose
 * cgtp_tri_workspace_bytes() exceeds that returns CGTP_ERR_SCRATCH_LIMIT without launching.  Calls nothing that
 * allocates.  Results are bit-identical to cgtp_tri_contract.  All calls on one device share the array: two calls
 * that overlap in time on one device (different streams or threads) race; calls on one stream do not.  The first call
 * on a device looks the array's address up (hipGetSymbolAddress); make it outside graph capture. */
int64_t cgtp_tri_static_scratch_bytes(void);
int cgtp_tri_contract_static(const cgtp_tri_args* args, void* stream);

/* ---- general contraction over two channel axes (u, w) ----------------------------------------------------
 *
 *   out[r, o, (u), (w)] = sum_{t in seg[o]} coef[t] * sum_{axes not in out} A[r, ia_t, ..] * B[r, ib_t, ..] * W[r, iw_t, ..]
 *
 * Each operand carries any subset of {u, w} (stride 0 for an axis it lacks); an axis the output carries is
 * element-wise, the others are summed.  Any-shape path for the matrix members of the reference's operator
 * family — indexed_vecmat / outer / mat_t_vec _scale_gather (equitorch/ops/batched_sparse_dense_op.py:1383-1459,
 * 436-512, 1200-1238) — for the fully connected products built from them (TensorProductU1VDummy and siblings,
 * equitorch/nn/functional/linears.py:254-492; TensorProductUVWDummy, nn/functional/tensor_products.py:92-172)
 * and for all their gradients.  Same packed table as cgtp_tri_contract.  reduce_rows sums over rows.
 */
typedef struct cgtp_gen_operand {
  const void* data;
  int64_t row_stride;      /* 0: shared over rows */
  int64_t idx_stride;      /* elements between sparse indices */
  int64_t u_stride;        /* 0: operand has no u axis */
  int64_t w_stride;        /* 0: operand has no w axis */
  int32_t present;
  int32_t _pad;
} cgtp_gen_operand;

typedef struct cgtp_gen_args {
  cgtp_gen_operand a, b, w;
  const void* coef;        /* [nnz] dtype; NULL = ones */
  const uint32_t* idx;     /* [nnz] ia | ib << 10 | iw << 20 */
  const int32_t* seg;      /* [n_out + 1] */
  int32_t n_out, nnz;
  void* out;               /* (n_rows | 1, n_out, [U], [W]) contiguous */
  int64_t n_rows;
  int32_t U, W;            /* extents of the two channel axes */
  int32_t out_has_u, out_has_w;
  int32_t reduce_rows;
  int32_t dtype;           /* CGTP_F32 | CGTP_F64 */
} cgtp_gen_args;

int cgtp_gen_validate(const cgtp_gen_args* args);
int cgtp_gen_contract(const cgtp_gen_args* args, void* stream);

/* ---- indexed scale-segment: out[n, m, c] = sum_{t in seg m} scale[t] * in[n, index[t], c] --------------
 * Stands in for indexed_scale_segment_gpu (equitorch/ops/indexed_scale_segment_op.py:110-141), including the
 * seg == NULL mode (pure scaled gather, one term per output) and optional scale / index.  With N == 1,
 * in = messages viewed as (1, E, D*C), index = dst-sorted edge permutation, seg = dst CSR pointer, this is
 * the edge -> node scatter-sum.  index / seg are int64 as in the reference's tables.
 */
int cgtp_segment_sum(const void* in, const void* scale, const int64_t* index, const int64_t* seg, void* out,
                     int64_t n_batch, int64_t in_size, int64_t out_size, int64_t C, int32_t dtype,
                     void* stream);

/* ---- specialised channel-wise ("uvu") tensor product -----------------------------------------------------
 *
 *   out[n, M, c] = sum_t coef_t * x[xr(n), M1_t, c] * y[n, M2_t] * W[(n), p_t, c]
 *
 * Fused replacement for the two launches of TensorProductU1UDummy.forward
 * (equitorch/nn/functional/linears.py:18-42: indexed_vecsca_scale_gather then indexed_mul_scale_gather) and,
 * in the backward entry, for the seven launches of its backward (:44-83).  The Clebsch-Gordan table is
 * compiled into the kernel; cgtp_uvu_find() maps a table fingerprint to a config id (or -1).
 *
 * Segment mode (n_seg > 0) additionally fuses a gather of the node operand and the scatter-sum over an edge
 * list sorted by segment id (destination node in the forward, source node in the backward).  All per-edge
 * index arrays are then indexed by SORTED POSITION q: the edge is e = perm ? perm[q] : q (rows of y, W, grad_y,
 * grad_w), seg_ids[q] is its (ascending) segment id, gather[q] the row of the gathered operand (forward: row
 * of x; backward: row of grad_out; in the backward x is read at row seg_ids[q]).  ptr is the CSR pointer of
 * seg_ids.  The sorted list is cut into one range per wavefront in one of two ways.  With wave_seg (n_waves + 1
 * ascending segment indices, first 0, last n_seg) wavefront k owns the whole segments [wave_seg[k],
 * wave_seg[k+1]) and writes their rows directly (zero rows for empty segments); the caller balances the ranges
 * (about 32 positions each works well).  Without it every wavefront owns pos_per_wave consecutive positions, or the
 * positions between two entries of wave_pos, and segments cut by a range boundary go through partial rows in the
 * workspace and a fix-up kernel.  Either way
 * there are no atomics and results are deterministic.
 *
 * Configs whose tables are too large for a register-resident body (cgtp_uvu_blockwise_only(): e.g. lmax = 6, 6460
 * coefficients) run segment mode on their block-wise kernels: fp32, C <= 64, harmonics given, per-edge weights (or
 * no weight gradient), ranges by position only (wave_seg and wave_pos must be NULL); one range per group of lanes
 * that handles an edge, pos_per_wave then counts the positions of such a range (0 = as many ranges as fill the GPU
 * once), and the sums over a segment are kept in LDS.
 */
int cgtp_uvu_num_configs(void);
int cgtp_uvu_find(uint64_t fingerprint);
/* The same for the table of a module converted to reduced precision (reference: TensorProductInfo._apply moves
 * the coefficient tensors with the module, equitorch/structs/__init__.py:7-102): `fingerprint` is taken over the
 * coefficients as they read in `dtype` (CGTP_BF16 | CGTP_F16); matches the config whose fp32 table rounds to them. */
int cgtp_uvu_find_rounded(uint64_t fingerprint, int dtype);
/* Describes config `cfg`: dims (D1, D2, DO, P, NNZ) written to dims[5]; returns its fingerprint (0 if bad). */
uint64_t cgtp_uvu_describe(int cfg, int32_t* dims);
/* The compiled table of config `cfg` (dims from cgtp_uvu_describe): coef[NNZ] fp32 values, idx[4 * NNZ] = (M, M1, M2,
 * p) per entry in table order; either may be NULL.  Returns NNZ, -1 for a bad id.  Host only.  See
 * cgtp_uvu_args.path_scale. */
int cgtp_uvu_table(int cfg, float* coef, int32_t* idx);
/* Degree L if the second operand of config `cfg` is laid out like harmonics of degrees 0..L and the fused
 * kernels can evaluate them from edge vectors (cgtp_uvu_args.y_vec); -1 otherwise. */
int cgtp_uvu_sh_degree(int cfg);

typedef struct cgtp_uvu_args {
  int32_t cfg;             /* from cgtp_uvu_find                                                   */
  int32_t dtype;           /* CGTP_F32 | CGTP_F64                                                  */
  int32_t C;               /* channels                                                             */
  int32_t w_shared;        /* 1: W is (P, C); 0: W is (n_rows, P, C)                               */
  int64_t n_rows;          /* batch rows / edges                                                   */
  int64_t n_x_rows;        /* rows of x (== n_rows unless gathered / segment-owned)                */
  int64_t n_seg;           /* number of segments (nodes); 0 = row mode                             */
  const int64_t* ptr;      /* segment mode: [n_seg + 1] CSR pointer over sorted positions          */
  const int64_t* perm;     /* segment mode: [n_rows] sorted position -> edge id, NULL = identity   */
  const int64_t* seg_ids;  /* segment mode: [n_rows] sorted position -> segment id, ascending      */
  const int64_t* gather;   /* [n_rows] row of the gathered operand (fwd: x, bwd: grad_out); row mode: per
                              row, optional; segment mode: per sorted position, required           */
  int32_t pos_per_wave;    /* segment mode without wave_seg: positions per wavefront; 0 = 32 (block-wise-only configs: see above) */
  int32_t y_vec;           /* segment mode: 0 = y holds harmonics (n_rows, D2); 1 / 2 = y holds edge vectors
                              (n_rows, 3) and the kernel evaluates the harmonics of degrees 0..sqrt(D2)-1 itself,
                              of y / max(|y|, 1e-12) (1) or of y as it is (2); grad_y is then (n_rows, 3).  Needs a
                              config whose second operand is laid out like harmonics (cgtp_uvu_sh_degree >= 0).
                              Fuses SphericalHarmonics.forward (equitorch/nn/sphericals.py:31-35) into the edge
                              kernel; no counterpart as one call in the reference                             */
  const int32_t* wave_seg; /* segment mode, optional: [n_waves + 1] first segment of every wavefront */
  int64_t n_waves;         /* number of ranges in wave_seg                                         */
  const void* x;           /* (n_x_rows, D1, C); bwd segment mode: n_x_rows == n_seg               */
  const void* y;           /* (n_rows, D2); (n_rows, 3) if y_vec                                   */
  const void* w;           /* (n_rows | 1, P, C)                                                   */
  /* forward */
  void* out;               /* (n_seg ? n_seg : n_rows, DO, C)                                      */
  /* backward */
  const void* grad_out;    /* (rows addressed by gather / row id, DO, C)                           */
  void* grad_x;            /* (n_seg ? n_seg : n_rows, D1, C) or NULL                              */
  void* grad_y;            /* (n_rows, D2), (n_rows, 3) if y_vec, or NULL                          */
  void* grad_w;            /* (n_rows | 1, P, C) or NULL                                           */
  void* workspace;         /* cgtp_uvu_workspace_bytes() bytes (segment mode, bwd of a shared W, fp32 row-mode
                              bwd with grad_y and C > 64)                                          */
  const int64_t* x_gather; /* row mode backward, optional: [n_rows] row of x of every batch row (x then has
                              n_x_rows rows; grad_x stays per batch row, (n_rows, D1, C))              */
  int32_t y_channels;      /* row mode, fp32: 1 = y and grad_y carry channels, (n_rows, D2, C): the "uuu" product
                              TensorProductUUUDummy (equitorch/nn/functional/tensor_products.py:9-90), on the
                              block-wise kernels                                                     */
  int32_t reserved_;
  const void* path_scale;  /* optional, device, P values of dtype: the caller's table is the compiled one with the
                              coefficients of weight path p multiplied by path_scale[p] (other path_norm / channel_norm
                              than the compiled default, equitorch/utils/_structs.py:177-206); NULL = all ones        */
  /* Weights produced inside the segment kernels (w may then be NULL):
   *   W[e, p, c] = sum_r radial_h[e, r] * radial_w[r, p, c]
   * the last linear layer of the network that maps per-edge radial features (BesselBasis and cutoffs,
   * equitorch/nn/radials.py:10-58, nn/cutoffs.py:7-131, then the user's MLP) to tensor-product weights — in the
   * reference a separate linear whose (E, P, C) output the product then reads.  fp32, C = 64, segment mode, configs
   * whose kernels keep four channels per lane (cgtp_uvu_radial_supported), radial_r in {4, 8, 12, 16}, no path_scale
   * (fold it into radial_w), 16-byte aligned pointers.  Backward: grad_w (n_rows, P, C) is written when given;
   * cgtp_uvu_radial_grad turns it into the gradients of radial_h and radial_w. */
  const void* radial_h;    /* (n_rows, radial_r) or NULL                                          */
  const void* radial_w;    /* (radial_r, P, C)                                                    */
  int32_t radial_r;
  int32_t reserved2_;
  const int64_t* wave_pos; /* segment mode, optional (not together with wave_seg): [n_waves + 1] ascending sorted
                              positions, first 0, last n_rows, strictly increasing: wavefront k walks positions
                              wave_pos[k] .. wave_pos[k + 1].  Cuts may fall inside segments (partial rows in the
                              workspace, as without any table); cutting after equal numbers of steps —
                              cgtp_uvu_slots() positions of one segment per step — keeps the wavefronts equally long */
} cgtp_uvu_args;

/* 1 if config `cfg` has segment kernels that produce the weights themselves (cgtp_uvu_args.radial_h). */
int cgtp_uvu_radial_supported(int cfg);
/* The other two gradients of that mode, from the per-edge weight gradient grad_w (n_rows, n_paths, 64) the backward
 * wrote, in one pass over it:
 *   grad_radial_h[e, r]    = sum_{p, c} grad_w[e, p, c] * radial_w[r, p, c]
 *   grad_radial_w[r, p, c] = sum_e radial_h[e, r] * grad_w[e, p, c]
 * (in the reference: autograd through the linear layer that produced the weights).  fp32; 4 <= n_paths <= 16,
 * radial_r <= 16; grad_w and radial_w 16-byte aligned.  The workgroups' partial sums over the edges live in `workspace`
 * (cgtp_uvu_radial_grad_workspace_bytes) and are added in a fixed order. */
int64_t cgtp_uvu_radial_grad_workspace_bytes(int64_t n_rows, int32_t radial_r, int32_t n_paths);
int cgtp_uvu_radial_grad(const void* grad_w, const void* radial_h, const void* radial_w, void* grad_radial_h,
                         void* grad_radial_w, void* workspace, int64_t n_rows, int32_t radial_r, int32_t n_paths,
                         int32_t dtype, void* stream);

/* ---- channel-wise product over an edge list for a table that is not compiled in ---------------------------
 *
 * The same fused launch as cgtp_uvu_fwd / cgtp_uvu_bwd in segment mode — gather at one end of the edge, product,
 * segment sum at the other, no per-edge messages in memory, no atomics — for ANY table, handed over as data and
 * read by the kernels through the scalar cache, with the per-edge operands and the segment sums in LDS.  Replaces,
 * for irreps without a compiled table, the reference's composition of index_select, the table-driven product
 * kernels (equitorch/ops/batched_sparse_dense_op.py:63-152, 1578-1662 behind equitorch/nn/functional/linears.py:16-93)
 * and indexed_scale_segment (equitorch/ops/indexed_scale_segment_op.py:7-108).
 *
 * `a` is read as in segment mode with ranges by position: dtype CGTP_F32, n_seg > 0, ptr / seg_ids / gather (and
 * perm) given, C <= 256 (<= 64 unless C is a multiple of 4 and the operands are 16-byte aligned), harmonics given
 * (y_vec, y_channels, radial_*, path_scale, wave_seg, wave_pos, x_gather unused and zero); cfg is ignored.  Per-edge
 * or shared weights; a shared weight's gradient is not formed here (CGTP_ERR_SHAPE with w_shared and grad_w).
 * pos_per_wave counts the sorted positions of one range (one range per group of lanes that handles an edge); 0 = as
 * many ranges as fill the GPU once.  workspace: cgtp_uvu_tab_workspace_bytes() bytes (partial rows of the segments a
 * range boundary cuts). */
typedef struct cgtp_uvu_tab {
  const float* coef;        /* [nnz64 + 128] device, nnz64 = nnz rounded up to a multiple of 64: coefficients, entries
                               sorted by (path, output row); zeros past nnz                                     */
  const uint32_t* idx;      /* [nnz64 + 128] device, one word per entry: row of x | row of y << 8 | 1 << 16 on the last
                               entry of a (path, output row) segment | 1 << 17 on the last entry of a path | output row
                               << 18 (rows < 256); zeros past nnz                                              */
  const uint32_t* paths;    /* [n_paths_walked + 2] device: the weight path of every run of entries in walk order, then
                               0xffff twice                                                                    */
  int32_t nnz, n_segments;  /* nnz <= 8192; n_segments = number of (path, output row) runs                      */
  int32_t D1, D2, DO, P;    /* rows of x, y, out (each < 256) and number of weight paths                        */
} cgtp_uvu_tab;
int64_t cgtp_uvu_tab_workspace_bytes(const cgtp_uvu_args* a, const cgtp_uvu_tab* t, int backward);
/* Status the launch would return for these arguments (pointers are only tested for NULL and alignment). Host only. */
int cgtp_uvu_tab_validate(const cgtp_uvu_args* a, const cgtp_uvu_tab* t, int backward);
int cgtp_uvu_tab_fwd(const cgtp_uvu_args* a, const cgtp_uvu_tab* t, void* stream);
int cgtp_uvu_tab_bwd(const cgtp_uvu_args* a, const cgtp_uvu_tab* t, void* stream);

/* Positions of one segment a wavefront takes per step (64 / lanes per edge) in a segment-mode launch of config
 * `cfg` with C channels and aligned operands; 0 if there is no such launch.  Host only. */
int cgtp_uvu_slots(int cfg, int dtype, int C, int backward);
/* 1 if config `cfg` exists only as block-wise kernels (one channel per lane, fp32), else 0. */
int cgtp_uvu_blockwise_only(int cfg);
int cgtp_uvu_validate(const cgtp_uvu_args* args, int backward);
/* Bytes of workspace the forward (backward = 0) or backward (1) launch of `args` needs; 0 if none. */
int64_t cgtp_uvu_workspace_bytes(const cgtp_uvu_args* args, int backward);
int cgtp_uvu_fwd(const cgtp_uvu_args* args, void* stream);
int cgtp_uvu_bwd(const cgtp_uvu_args* args, void* stream);

/* ---- fully connected ("uv") tensor product on the matrix cores --------------------------------------------
 *
 *   out[n, m, w] = sum_t coef_t * y[n, b_t] * sum_u x[n, a_t, u] * Wt[p_t, w, u]        bf16 in, fp32 accumulate
 *
 * Fused replacement for TensorProductU1VDummy.forward (equitorch/nn/functional/linears.py:257-280:
 * indexed_vecsca_scale_gather then indexed_vecmat_scale_gather, with the (N, segments, C_in) intermediate in
 * memory) and, with direction = 1, for the grad-input1 product of its backward (:290-293).  The table is compiled
 * in; cgtp_uv_find() maps the fingerprint of the forward table to a config id (or -1).
 *   direction 0: x = input1 (n_rows, D1, cin), out (n_rows, DO, cout), W stored (P, cin, cout);
 *   direction 1: x = grad_out (n_rows, DO, cin), out = grad_input1 (n_rows, D1, cout), W stored (P, cout, cin)
 *                (here cin = C_out of the module and cout = its C_in).
 * y is (n_rows, D2).  cin in {32, 64, 128}, cout a multiple of 32, dtype CGTP_BF16, 16-byte aligned pointers.
 *
 * The kernel reads the weight in matrix-core fragment order, wp: cgtp_uv_pack_weights() rewrites W as stored by the
 * module (same element count, one small launch per weight update and direction) so that every wavefront load of
 * weight fragments is one contiguous KB; strided 64-byte pieces reach a third of that rate from L2.
 */
int cgtp_uv_num_configs(void);
int cgtp_uv_find(uint64_t fingerprint);
/* As cgtp_uvu_find_rounded, for the fully connected product. */
int cgtp_uv_find_rounded(uint64_t fingerprint, int dtype);
/* path_scale (device, n_paths floats, or NULL): factor of every weight path, folded into the packed copy — for a
 * table that equals the compiled one up to one factor per path (other path / channel normalisation, see
 * cgtp_uv_table). */
int cgtp_uv_pack_weights(int direction, const void* w, void* packed, int32_t n_paths, int32_t cin, int32_t cout,
                         int32_t dtype, const float* path_scale, void* stream);
/* The compiled table of config `cfg`: dims[5] = (D1, D2, DO, P, NNZ), coef[NNZ] (fp32 values), idx[4 * NNZ] =
 * (M, M1, M2, p) per entry, in table order; each output may be NULL.  Returns NNZ, -1 for a bad id.  Host only.  A
 * caller whose table has the same entries with every path's coefficients multiplied by one factor per path (the
 * reference's path_norm / channel_norm options, equitorch/utils/_structs.py:177-206) passes those factors as
 * path_scale and runs on the same kernels. */
int cgtp_uv_table(int cfg, int32_t* dims, float* coef, int32_t* idx);
int cgtp_uv_validate(int cfg, int direction, const void* x, const void* y, const void* wp, const void* out,
                     int64_t n_rows, int32_t cin, int32_t cout, int32_t dtype);
int cgtp_uv_apply(int cfg, int direction, const void* x, const void* y, const void* wp, void* out, int64_t n_rows,
                  int32_t cin, int32_t cout, int32_t dtype, void* stream);
/* Gradient w.r.t. the harmonics of direction 0 (the uu1/vu1 product of the reference's backward,
 * equitorch/nn/functional/linears.py:294-300, without its (N, segments, C) intermediates):
 *   gy[n, b] = sum_t [b_t = b] coef_t * sum_w g[n, m_t, w] * sum_u x[n, a_t, u] * W[p_t, u, w]
 * x (n_rows, D1, cin), g = grad_out (n_rows, DO, cout), wp = direction-0 packed weights, gy (n_rows, D2);
 * cout <= 128.  Sums run in a fixed order (no atomics). */
int cgtp_uv_grad_y(int cfg, const void* x, const void* g, const void* wp, void* gy, int64_t n_rows, int32_t cin,
                   int32_t cout, int32_t dtype, void* stream);
/* Gradient w.r.t. the shared weight (the reference accumulates batch outer products with atomics,
 * indexed_outer_scale_gather with out_accumulated, equitorch/nn/functional/linears.py:301-307):
 *   gw[p, u, w] = sum_n sum_t [p_t = p] coef_t * y[n, b_t] * x[n, a_t, u] * g[n, m_t, w]
 * x (n_rows, D1, cin), y (n_rows, D2), g = grad_out (n_rows, DO, cout), gw (P, cin, cout) as the module stores W;
 * cin, cout multiples of 32 up to 128.  The samples are contracted on the matrix cores in chunks; the fp32 chunk
 * partials live in `workspace` (cgtp_uv_grad_w_workspace_bytes bytes) and are added in a fixed order. */
int64_t cgtp_uv_grad_w_workspace_bytes(int cfg, int64_t n_rows, int32_t cin, int32_t cout);
int cgtp_uv_grad_w(int cfg, const void* x, const void* y, const void* g, void* gw, void* workspace, int64_t n_rows,
                   int32_t cin, int32_t cout, int32_t dtype, const float* path_scale, void* stream);

/* ---- radial basis and cutoff envelopes ---------------------------------------------------------------------------
 *
 * Element-wise functions of the edge length r (n values), fp32 / fp64, one launch forward and one for the gradient.
 * The reference writes them as tensor expressions: BesselBasis.forward (equitorch/nn/radials.py:46-58) and
 * radial_standarize / polynomial_cutoff / cosine_cutoff / mollifier_cutoff (equitorch/nn/functional/cutoffs.py:4-25,
 * :30-49, :52-64, :67-80) behind the cutoff modules (equitorch/nn/cutoffs.py:7-131).
 *
 *   cgtp_bessel:       out[i, k] = (2 / r_max) * sin(freq[k] * r[i] / r_max) / r[i]          out (n, num_basis)
 *   cgtp_bessel_grad:  gr[i] = sum_k g[i, k] * d out[i, k] / d r[i]                             (NULL: not wanted)
 *                      gfreq_rows[i, k] = g[i, k] * d out[i, k] / d freq[k]                     (NULL: not wanted;
 *                      the caller sums it over i: the gradient of trainable frequencies)
 *   cgtp_cutoff:       u = clamp((r - r_min) / range, 0, 1);  kind 0: polynomial envelope of order param,
 *                      1: cosine, 2: mollifier with eps = param.  g == NULL: out[i] = envelope(u);
 *                      else out[i] = g[i] * d envelope / d r[i] (zero where the clamp is active). */
int cgtp_bessel(const void* r, const void* freq, void* out, int64_t n, int32_t num_basis, double r_max, int32_t dtype,
                void* stream);
int cgtp_bessel_grad(const void* r, const void* freq, const void* g, void* gr, void* gfreq_rows, int64_t n,
                     int32_t num_basis, double r_max, int32_t dtype, void* stream);
int cgtp_cutoff(int kind, const void* r, const void* g, void* out, int64_t n, double r_min, double range, double param,
                int32_t dtype, void* stream);

/* ---- fully connected products in fp32 / fp64 on the matrix cores, any table --------------------------------------
 *
 *   out[n, M, w] = sum_{segments s = (p, M)} sum_k inter_s[n, k] * W[p, k, w]
 *   inter_s[n, k] = sum_{t in s} coef_t * x[n, a_t, k] * y[n, b_t]                       (cy == 0, K = cx)
 *   inter_s[n, k] = sum_{t in s} coef_t * x[n, a_t, u] * y[n, b_t, v],  k = u * cy + v   (cy > 0, K = cx * cy)
 *
 * One fused launch for TensorProductU1VDummy.forward (equitorch/nn/functional/linears.py:257-280: vecsca, then vecmat
 * with the (N, segments, C_in) intermediate in memory), for TensorProductUVWDummy.forward
 * (equitorch/nn/functional/tensor_products.py:95-101: outer, then vecmat over the flattened (u, v) axis) and, with
 * the rows' roles exchanged and the weight packed transposed, for the grad-input products of their backward passes
 * (tensor_product_1vu / tensor_product_uvw with permuted weights, linears.py:290-293, tensor_products.py:126-150).
 * Shared weights only.  The caller supplies the walk as a flat list of items, one per segment, with the segment's
 * terms t0..t1 in (term_a = row of x, term_b = row of y, term_c = coefficient); flags: 1 = first item of its output
 * row, 2 = last (kb0, nkb: 0, unused).  The items of an output row are consecutive, and every output row needs at
 * least one item (t0 = t1 for a row without terms: it is written as zeros).  The wavefronts of a workgroup split the
 * output rows: the list is ordered in cgtp_uvt_item_groups() groups of whole rows, group i being items group_ptr[i] ..
 * group_ptr[i + 1] (groups of about equal length keep the wavefronts equally busy; empty groups are allowed).
 * cgtp_uvt_chunk() (blocks of 16 k the kernels pad K to with zero weights) must be passed as `kbi`.
 * x (n_rows, dx, cx), y (n_rows, dy) or (n_rows, dy, cy), out (n_rows, dout, cout), all of one dtype (CGTP_F32 |
 * CGTP_F64) and contiguous; cx, cy,
 * cout multiples of 4, cx * cy a multiple of 16 when cy > 0; 16-byte aligned pointers; the rows of 16 samples must
 * fit the LDS (CGTP_ERR_LDS otherwise).  wp = cgtp_uvt_pack_weights(W): W (n_paths, K, cout) read through element
 * strides (so that a transposed or flattened view needs no copy), rewritten in matrix-core fragment order, zero-padded;
 * cgtp_uvt_packed_elems() elements.
 */
typedef struct cgtp_uvt_item {
  int32_t p, kb0, nkb, t0, t1, out_row, flags, reserved_;
} cgtp_uvt_item;

typedef struct cgtp_uvt_args {
  const void* x;
  const void* y;
  const void* wp;
  void* out;
  const cgtp_uvt_item* items;   /* device */
  const int32_t* term_a;        /* device */
  const int32_t* term_b;        /* device */
  const void* term_c;           /* device, dtype */
  int64_t n_rows;
  int32_t n_items;
  int32_t dx, dy, dout;
  int32_t cx, cy, cout;
  int32_t kbi;                  /* chunk length the items were cut for: cgtp_uvt_chunk() */
  int32_t dtype;                /* CGTP_F32 | CGTP_F64 */
  int32_t n_terms;              /* entries of term_a / term_b / term_c (the tables are copied to LDS: 32 B per item +
                                   12 B per term must fit next to the samples' rows, CGTP_ERR_LDS otherwise) */
  int32_t n_groups;             /* cgtp_uvt_item_groups() */
  int32_t group_ptr[9];         /* n_groups + 1 item offsets, group_ptr[0] = 0, group_ptr[n_groups] = n_items */
} cgtp_uvt_args;

int64_t cgtp_uvt_packed_elems(int32_t n_paths, int64_t K, int32_t cout);
int cgtp_uvt_pack_weights(const void* w, void* packed, int32_t n_paths, int64_t K, int32_t cout, int64_t stride_p,
                          int64_t stride_k, int64_t stride_c, int32_t dtype, void* stream);
/* Launch shape for these extents, or -status when the kernels do not take them: blocks of 16 k that K is padded to
 * a multiple of; groups of output rows the item list has to come in.  Host only. */
int cgtp_uvt_chunk(int64_t n_rows, int32_t dx, int32_t dy, int32_t dout, int32_t cx, int32_t cy, int32_t cout,
                   int32_t dtype);
int cgtp_uvt_item_groups(int64_t n_rows, int32_t dx, int32_t dy, int32_t dout, int32_t cx, int32_t cy, int32_t cout,
                         int32_t dtype);
int cgtp_uvt_validate(const cgtp_uvt_args* args);
int cgtp_uvt_apply(const cgtp_uvt_args* args, void* stream);

/* Gradient of the shared weight of the products above (the reference accumulates batch outer products with atomics:
 * indexed_outer_scale_gather with out_accumulated, equitorch/nn/functional/linears.py:301-307,
 * tensor_products.py:152-158):
 *   gw[p, k, w] = sum_n sum_{segments s = (p, M)} inter_s[n, k] * g[n, M, w]
 * with inter_s as in cgtp_uvt_apply (never written to memory).  items: the segments sorted by weight path (fields p,
 * out_row = M, t0, t1 are read; at most 8 terms per item — a longer segment is given as several items),
 * path_ptr[n_paths + 1] their ranges per path; x (n_rows, dx, cx), y (n_rows, dy) or
 * (n_rows, dy, cy), g = grad_out (n_rows, dg, cout), gw (n_paths, K, cout) contiguous as the module stores the
 * weight.  The samples are contracted on the matrix cores in chunks; the chunks' partial results live in `workspace`
 * (cgtp_uvt_grad_w_workspace_bytes) and are added in a fixed order.  Channel counts multiples of 4, 16-byte aligned
 * pointers; gw and workspace aligned to four elements (16 bytes fp32, 32 bytes fp64). */
typedef struct cgtp_uvt_gw_args {
  const void* x;
  const void* y;
  const void* g;
  void* gw;
  void* workspace;
  const cgtp_uvt_item* items;   /* device */
  const int32_t* path_ptr;      /* device */
  const int32_t* term_a;        /* device */
  const int32_t* term_b;        /* device */
  const void* term_c;           /* device, dtype */
  int64_t n_rows;
  int32_t n_items, n_terms, n_paths;
  int32_t dx, dy, dg;
  int32_t cx, cy, cout;
  int32_t dtype;                /* CGTP_F32 | CGTP_F64 */
  int32_t reserved_;
} cgtp_uvt_gw_args;

int64_t cgtp_uvt_grad_w_workspace_bytes(int64_t n_rows, int32_t n_paths, int64_t K, int32_t cout, int32_t dtype);
int cgtp_uvt_grad_w(const cgtp_uvt_gw_args* args, void* stream);

/* ---- fully connected products with a weight per sample ---------------------------------------------------
 *
 *   out[n, M, w] = sum_t coef_t * sum_{u, v} x[n, a_t, u] * y[n, b_t, v] * W[n, p_t, u * cy + v, w]
 *
 * One streaming launch over the per-sample weight W (n_rows, n_paths, cx * cy, cout), each element read once, for
 * the products the reference runs as two launches with the (N, segments, C_in) intermediate in memory when the
 * weight has a batch axis (per-sample detection: equitorch/nn/tensor_products.py:152-155; u1v / 1vu:
 * equitorch/nn/functional/linears.py:254-412; uvw: equitorch/nn/functional/tensor_products.py:95-158; channel mixing
 * between irreps with y = NULL: linears.py:494-571; kernel ops/batched_sparse_dense_op.py:1289-1381).  The backward
 * writes grad_W in the same stream (read W, write grad_W) and sums grad_x / grad_y per sample in LDS; any of gx / gy
 * / gw may be NULL.  The table is data: the paths are walked output irrep by output irrep.
 *   blocks  [n_blocks][4]  (first output row, rows L, first slot, one past the last slot); the rows of different
 *                          blocks do not overlap; output rows outside every block are not written
 *   slots   [n_slots][3]   (weight path p, first entry, one past the last entry) of a walked path; the rows of gw
 *                          that belong to a path without a slot are not written (the caller zeroes them)
 *   entries [n_entries]    j | a << 8 | b << 16 | 1 << 24 on the last entry of a run of equal j; j = output row - the
 *                          block's first row; sorted by j inside a slot; every j < L occurs in every slot of the
 *                          block (where the path has no term for it: one entry j | 1 << 24 | 1 << 25, no operand is
 *                          read for it)
 *   coef    [n_entries]    dtype
 * x (n_rows, D1, cx), y (n_rows, D2, cy) or NULL (then cy = 1, D2 = 1 and y = 1), out / g (n_rows, DO, cout), all
 * contiguous, dtype CGTP_F32 | CGTP_F64.  cout <= 64 vector lanes: cout <= 256 (fp32) / 128 (fp64) when it is a
 * multiple of 4 / 2 and W, out, g, gw are 16-byte aligned, cout <= 64 otherwise (CGTP_ERR_SHAPE beyond); D1, D2,
 * max_rows < 256; one sample's rows must fit 64 KB of LDS (CGTP_ERR_LDS otherwise). */
typedef struct cgtp_psw_table {
  const uint32_t* entries;  /* device */
  const void* coef;         /* device, dtype */
  const int32_t* slots;     /* device */
  const int32_t* blocks;    /* device */
  int32_t n_entries, n_slots, n_blocks;
  int32_t max_rows;         /* largest L of a block */
  int32_t D1, D2, DO, P;
} cgtp_psw_table;

typedef struct cgtp_psw_args {
  const void* x;
  const void* y;
  const void* w;
  void* out;       /* forward */
  const void* g;   /* backward: grad_out */
  void* gx;
  void* gy;
  void* gw;
  int64_t n_rows;
  int32_t cx, cy, cout;
  int32_t dtype;
} cgtp_psw_args;

/* Status the launch would return for these arguments. Host only. */
int cgtp_psw_validate(const cgtp_psw_args* a, const cgtp_psw_table* t, int backward);
int cgtp_psw_fwd(const cgtp_psw_args* a, const cgtp_psw_table* t, void* stream);
int cgtp_psw_bwd(const cgtp_psw_args* a, const cgtp_psw_table* t, void* stream);

/* Gradient of a second operand without channels (u1v):
 *   gy[n, b] = sum_t coef_t * sum_w grad_out[n, M_t, w] * (sum_k x[n, a_t, k] * W[p_t, k, w])
 * (the reference obtains it from autograd through sparse_mul and the batched matmul,
 * equitorch/nn/functional/linears.py:283-336).  wp: the weight as packed for the forward by cgtp_uvt_pack_weights.
 * items: one per segment (p, a = out_row) with its terms t0 .. t1 (nkb, kb0, flags unused); term_m / term_b: rows of
 * grad_out and of gy.  x (n_rows, dx, cx), grad_out (n_rows, dg, cout), gy (n_rows, dy); cx and cout multiples of 4,
 * 16-byte aligned pointers.  The 16 staged samples of a workgroup must fit the LDS (CGTP_ERR_LDS otherwise). */
typedef struct cgtp_uvt_gy_args {
  const void* x;
  const void* g;
  const void* wp;
  void* gy;
  const cgtp_uvt_item* items;   /* device */
  const int32_t* term_m;        /* device */
  const int32_t* term_b;        /* device */
  const void* term_c;           /* device, dtype */
  int64_t n_rows;
  int32_t n_items, n_terms;
  int32_t dx, dy, dg;
  int32_t cx, cout;
  int32_t dtype;                /* CGTP_F32 | CGTP_F64 */
} cgtp_uvt_gy_args;

int cgtp_uvt_grad_y(const cgtp_uvt_gy_args* args, void* stream);

/* ---- real spherical harmonics of vectors -----------------------------------------------------------------
 * Stands in for spherical_harmonics (equitorch/ops/spherical_harmonics.py:68-640: explicit polynomials per
 * degree, TorchScript, differentiated by autograd) together with its callers' pre- and post-processing:
 * torch.nn.functional.normalize(input, dim=-1) of SphericalHarmonics.forward (equitorch/nn/sphericals.py:31-35)
 * when normalize != 0, and the 1/sqrt(4 pi) factor of integral_normalize
 * (equitorch/nn/functional/sphericals.py:9-14) passed as scale (1.0 otherwise).
 * xyz: (n, 3); out / grad_out: (n, (lmax+1)^2), index l^2 + l + m; grad_xyz: (n, 3).  Component order and
 * normalisation as in the reference: Y_1 = sqrt(3) (y, z, x), |Y_l|^2 = 2l+1 on the unit sphere, homogeneous
 * of degree l when normalize == 0.  lmax <= cgtp_sh_max_degree() (17, the reference's limit).
 * dtype: CGTP_F32 | CGTP_F64.  n == 0 returns CGTP_OK without a launch.
 */
int cgtp_sh_max_degree(void);
int cgtp_sh_forward(const void* xyz, void* out, int64_t n, int lmax, int normalize, double scale, int dtype,
                    void* stream);
int cgtp_sh_backward(const void* xyz, const void* grad_out, void* grad_xyz, int64_t n, int lmax, int normalize,
                     double scale, int dtype, void* stream);

/* ---- layer RMS normalisation of equivariant features ------------------------------------------------------
 * Stands in for layer_rms_norm (equitorch/nn/functional/normalization.py:111-157: channel_mean_squared_norm,
 * rsqrt, sparse_vecsca with the per-sample factors and sparse_mul with the weight; four launches and their
 * autograd backward) with one launch per direction:
 *   ms[n,k] = sum_{M in irrep k, c} x[n,M,c]^2 / (C * (scaled ? dim_k : 1)),  r = rsqrt(ms + eps),
 *   out[n,M,c] = x[n,M,c] * r[n,k(M)] * weight[k(M),c]          (weight NULL = no scaling)
 * x, out, grad_out, grad_x: (n_rows, D, C) contiguous; weight, grad_weight: (n_irreps, C); rsigma: (n_rows,
 * n_irreps), written by the forward (NULL = not wanted) and read by the backward.  irrep_seg: HOST array of
 * n_irreps + 1 block boundaries, irrep_seg[0] = 0, irrep_seg[n_irreps] = D (IrrepsInfo.irrep_seg); irrep_rdims:
 * HOST array of the n_irreps factors 1 / dim_k as the table holds them (IrrepsInfo.rdims, fp32; NULL = computed
 * here), read when scaled != 0; blocks of at most 13 components (l <= 6), at most 64 irreps, C <= 64 or C/4 (fp32) resp. C/2 (fp64) <= 64 with 16-byte
 * aligned pointers: cgtp_layer_rms_supported tells.  grad_x and grad_weight may each be NULL; grad_weight needs a
 * workspace of cgtp_layer_rms_workspace_bytes (per-row terms, summed over rows in a fixed order).
 * dtype: CGTP_F32 | CGTP_F64.
 */
int cgtp_layer_rms_supported(const int32_t* irrep_seg, int n_irreps, int C, int dtype);
int64_t cgtp_layer_rms_workspace_bytes(int64_t n_rows, int n_irreps, int C, int dtype);
int cgtp_layer_rms_forward(const void* x, const void* weight, void* out, void* rsigma, const int32_t* irrep_seg,
                           const float* irrep_rdims, int n_irreps, int64_t n_rows, int D, int C, int scaled,
                           double eps, int dtype, void* stream);
int cgtp_layer_rms_backward(const void* x, const void* weight, const void* rsigma, const void* grad_out,
                            void* grad_x, void* grad_weight, void* workspace, const int32_t* irrep_seg,
                            const float* irrep_rdims, int n_irreps, int64_t n_rows, int D, int C, int scaled,
                            int dtype, void* stream);

/* ---- rotation of equivariant features by Euler angles -------------------------------------------------------
 * Stands in for sparse_wigner_rotation (equitorch/nn/functional/wigner_d.py:14-56: three sparse_vecsca launches
 * for the rotations about z and two sparse_scale launches for the constant matrix J) with one launch:
 *   out[n] = Z(alpha_n) J Z(beta_n) J Z(gamma_n) x[n],   transposed != 0: the transpose of that matrix (the
 * gradient with respect to x), Z(phi): y[m] = cs[2|m|] x[m] - sign(m) cs[2|m|-1] x[-m], y[0] = cs[0] x[0].
 * x, out: (n_rows, D, C) contiguous; sincos_*: (n_rows, cs_dim) with cs = (1, sin phi, cos phi, sin 2 phi, ...),
 * cs_dim >= 1 + 2 max l, NULL = that factor is skipped (a NULL beta skips both J as well); j_blocks: DEVICE array,
 * the dense (2l+1) x (2l+1) row-major block of J for every irrep one after the other; irrep_first / irrep_degree:
 * HOST arrays, first component and degree l of every irrep (consecutive blocks covering 0 .. D-1, l <= 6, at most 64
 * irreps).  C <= 64, or C/4 (fp32) resp. C/2 (fp64) <= 64 with 16-byte aligned pointers:
 * cgtp_wigner_rotate_supported tells.  dtype: CGTP_F32 | CGTP_F64.
 * cgtp_wigner_rotate_backward: from x and grad_out (n_rows, D, C), the gradient of the features (grad_x, NULL = not
 * wanted) and of the sincos tensors (grad_alpha / grad_beta / grad_gamma, each (n_rows, cs_dim) or NULL; columns
 * beyond 1 + 2 max l are written as zeros) in one launch that recomputes the intermediate features in registers
 * (the reference's autograd keeps them in memory).
 */
int cgtp_wigner_rotate_supported(const int32_t* irrep_first, const int32_t* irrep_degree, int n_irreps, int C,
                                 int dtype);
int cgtp_wigner_rotate(const void* x, void* out, const void* sincos_alpha, const void* sincos_beta,
                       const void* sincos_gamma, const void* j_blocks, const int32_t* irrep_first,
                       const int32_t* irrep_degree, int n_irreps, int64_t n_rows, int C, int cs_dim, int transposed,
                       int dtype, void* stream);
int cgtp_wigner_rotate_backward(const void* x, const void* grad_out, const void* sincos_alpha, const void* sincos_beta,
                                const void* sincos_gamma, const void* j_blocks, const int32_t* irrep_first,
                                const int32_t* irrep_degree, int n_irreps, int64_t n_rows, int C, int cs_dim,
                                void* grad_x, void* grad_alpha, void* grad_beta, void* grad_gamma, int dtype,
                                void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CGTP_H */
