// Internal interface between the HBM-bound kernels and the C-ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/archscale_muon.h"

namespace archscale {

enum { DT_BF16 = MUON_DTYPE_BF16, DT_F32 = MUON_DTYPE_F32 };
enum { EPS_ADD = MUON_EPS_ADD, EPS_CLAMP = MUON_EPS_CLAMP };

typedef muon_pre_item PreItem;
typedef muon_post_item PostItem;
typedef muon_scalar_item ScalarItem;

enum { ALGO_ADAMW = MUON_ALGO_ADAMW, ALGO_LION = MUON_ALGO_LION };

// hyper-parameters of the scalar updates, precomputed on the host
// (the layout of muon_hyper in the C ABI: the *_dev entry points hand the kernels a device pointer to one)
typedef muon_hyper ScalarHyper;

struct MomentumCoef {
  float mm, mg, um, ug, l2;
};

hipError_t launch_momentum(const PreItem* items, const int32_t* prefix, int n_items, int total_chunks,
                           MomentumCoef c, hipStream_t stream);

// per-matrix Frobenius norms of in[batch][rows][cols] -> scale[b] = 1/(|X|+eps) or 1/max(|X|,eps); with pow2 that
// factor is split into pow2[b] (a power of two) times scale[b] (between 0.7 and 1.5)
hipError_t launch_norm_scale(const void* in, int in_dtype, int cast_first, long in_bstride, int ld, int batch,
                             int rows, int cols, float eps, int eps_mode, float* partial, float* scale,
                             hipStream_t stream, float* pow2 = nullptr);

// D = bf16(scale*in) in the input's orientation and T = its transpose (either may be null), both zero-padded to
// d_rows x d_cols / d_cols x d_rows (multiples of 64); scale may be null (= 1).  tile_sumsq (optional): the sum of
// squares of the values written, one float per 64x64 tile: [batch][d_rows / 64][d_cols / 64].
hipError_t launch_layout(const void* in, int in_dtype, int cast_first, long in_bstride, int ld, int batch, int rows,
                         int cols, const float* scale, void* D, long d_bstride, int ldd, int d_rows, int d_cols,
                         void* T, long t_bstride, int ldt, hipStream_t stream, int out_f16 = 0, int out_shift = 0,
                         float* tile_sumsq = nullptr);

// the same pass over up to LAYOUT_PTRS_MAX matrices of one shape that are separate allocations (pointers by value, as
// they are: no scale, bf16 output), one launch: matrix i goes to D + i * d_bstride / T + i * t_bstride and its tile sums
// to tile_sumsq + i * (d_rows / 64) * (d_cols / 64)
constexpr int LAYOUT_PTRS_MAX = 64;
struct LayoutPtrs {
  const void* p[LAYOUT_PTRS_MAX];
};
hipError_t launch_layout_ptrs(const LayoutPtrs& ptrs, int n_mats, int in_dtype, int ld, int rows, int cols, void* D,
                              long d_bstride, int ldd, int d_rows, int d_cols, void* T, long t_bstride, int ldt,
                              hipStream_t stream, float* tile_sumsq);

// momentum fused with the layout pass of the Newton-Schulz operand (see momentum_layout_kernel): one launch covers up
// to MOMG_MAX_MATS matrices (separate allocations: pointers by value) of up to MOMG_MAX_CLS shape classes, either all by
// the transposing / padding tile pass or all by the linear pass (the operand image is the matrix itself)
constexpr int MOMG_MAX_MATS = 96;
constexpr int MOMG_MAX_CLS = 6;
constexpr int MOMLAY_TILE = 128;   // rows and columns of the tile of one block of the tile pass; one partial sum per tile
struct MomClass {
  int rows, cols;                // every matrix of the class is rows x cols, contiguous
  int transpose;                 // dst holds the transpose of the matrix (d_cols x d_rows) instead of the matrix
  int d_rows, d_cols;            // tile pass: extents of the matrix padded to multiples of MOMLAY_TILE
  int ldd;                       // tile pass: leading dimension of dst
  int blocks_per_mat;            // tiles (tile pass) or chunks of MUON_CHUNK_ELEMS (linear pass) of one matrix
  int tiles_x;                   // tile pass: tiles along the source columns
  long d_bstride;                // elements between consecutive matrices in dst
  uint16_t* dst;                 // bf16 image of matrix 0 of the class
  float* partial;                // [matrices of the class][blocks_per_mat] sums of squares of the values written
};
struct MomGroupParams {
  int n_mats, n_cls, linear;
  int g_dtype, m_dtype, w_dtype;
  MomentumCoef c;
  MomClass cls[MOMG_MAX_CLS];
  int32_t blk_start[MOMG_MAX_MATS + 1];   // first block of matrix i of the launch
  int32_t idx_in_cls[MOMG_MAX_MATS];      // index of matrix i within its class (selects its slot in dst and partial)
  uint8_t cls_of[MOMG_MAX_MATS];
  const void* g[MOMG_MAX_MATS];
  void* m[MOMG_MAX_MATS];
  const void* w[MOMG_MAX_MATS];           // read only when c.l2 != 0
};
static_assert(sizeof(MomGroupParams) <= 4096, "kernel arguments are limited to 4 KiB");
int momentum_class_blocks(const MomClass& k, int linear);
hipError_t launch_momentum_group(const MomGroupParams& p, hipStream_t stream);
hipError_t launch_norm_scale_from_partials(const float* partial, int partials_per_mat, int batch, float eps, int eps_mode,
                                           float* scale, hipStream_t stream);
// the same for several batches in one launch: block b serves matrix b - mat_start[i] of batch i
constexpr int NORMG_MAX = 16;
struct NormGroup {
  const float* partial;   // [batch][per_mat]
  float* scale;           // [batch]
  int per_mat;
};
struct NormGroupParams {
  int n;
  int32_t mat_start[NORMG_MAX + 1];
  NormGroup g[NORMG_MAX];
};
hipError_t launch_norm_scale_groups(const NormGroupParams& p, float eps, int eps_mode, hipStream_t stream);

// p[0 .. n) <- 0 with a plain kernel (a launch that a graph capture records like any other)
hipError_t launch_zero_i32(int* p, long n, hipStream_t stream);

hipError_t launch_unpad_copy(const void* src, long s_bstride, int lds_, void* dst, long d_bstride, int ldd,
                             int batch, int rows, int cols, hipStream_t stream);

// hdev (nullable, device memory): when given, the kernels take the hyper-parameters from it instead of the by-value
// arguments, so a captured launch follows a schedule
hipError_t launch_post_plain(const PostItem* items, const int32_t* prefix, int n_items, int total_chunks,
                             float lr, float lrwd, int cautious, hipStream_t stream, const ScalarHyper* hdev = nullptr);

hipError_t launch_post_muonh(const PostItem* items, const int32_t* prefix, int n_items, int total_chunks,
                             float lr, float lrwd, float eps, int cautious, float* scratch, hipStream_t stream,
                             const ScalarHyper* hdev = nullptr);

hipError_t launch_scalar_update(const ScalarItem* items, const int32_t* prefix, int n_items, int total_chunks,
                                int algo, int hyperball, ScalarHyper h, float* scratch, hipStream_t stream,
                                const ScalarHyper* hdev = nullptr);

hipError_t launch_calibration_copy(const void* src, void* dst, size_t bytes, hipStream_t stream);
// mode 1: read a; mode 2: b <- a + b, c <- (a + b) ^ a (two reads, two writes)
hipError_t launch_calibration_stream(int mode, const void* a, void* b, void* c, size_t bytes, hipStream_t stream);

}  // namespace archscale
