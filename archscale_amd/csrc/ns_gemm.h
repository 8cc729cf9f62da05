// Internal interface between the Newton-Schulz GEMM kernels and the C-ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace archscale {

// MODE_SYRKT: as MODE_SYRK, but P = Q is given K-major ([K][M] row-major, ldp = leading dimension; P == Q required)
enum { MODE_SYRK = 0, MODE_SYRK2 = 1, MODE_BX = 2, MODE_SYRKT = 3 };

// C[m][n] = sum_k P[m][k] * Q[n][k]; all leading dimensions / strides in elements.
struct GemmParams {
  const __bf16* P;   // [batch][tilesM*BM][ldp]
  const __bf16* P2;  // second pass over K for P (low half of a split B), or null
  const __bf16* Q;   // [batch][tilesN*BN][ldq]
  long strideP, strideQ;
  int ldp, ldq;
  int K;             // reduction length, multiple of 64
  int tilesM, tilesN;
  int batch;
  const __bf16* E;   // epilogue addend, read as E[col][row..row+3]; MODE_BX: may be null (X' = B X, no addend)
  long strideE;
  int lde;
  __bf16* C;         // row-major output [row][col] (may be null in MODE_BX)
  __bf16* C2;        // low half of a split output (MODE_SYRK2 with split)
  long strideC;
  int ldc;
  __bf16* Ct;        // transposed output [col][row] (MODE_BX, may be null)
  long strideCt;
  int ldct;
  float alpha, beta;
  int out_shift;         // MODE_BX: the result is multiplied by 2^out_shift (0: as it is)
  float diag_add;        // MODE_SYRK2: added to the diagonal of the result (B + a I, so that B X needs no addend)
  const float* scale;    // per batch element, or null: SYRK / SYRKT multiply the product by scale^2, BX the result by scale
  int m_valid, n_valid;  // true extents for the bounds-checked final store
  int qt_first;          // quarter mode: first tile of this problem (in its own 2x coarser enumeration) that is covered
  // a launch may cover only tiles [t_first, t_first + t_count) of every matrix of the problem (in the matrix's own
  // enumeration; t_count = 0: all of them), the flat tile index of the launch then counts t_count tiles per matrix
  int t_first, t_count;
  // K-split (symmetric products of the 128x128 configuration only): `ksplit` > 1 blocks share every tile, block s of
  // them walks k-tiles [s KT / ksplit, (s + 1) KT / ksplit) and leaves its fp32 accumulators in sk_partial; the block
  // that finds itself last (sk_counter, one per tile, zero before the launch and zero again after it) adds the partial
  // results in the order s = 0, 1, ... and runs the epilogue.  The sums do not depend on which block came last.
  int ksplit;
  float* sk_partial;     // [tiles of this problem in the launch][ksplit][128 * 128] fp32, accumulator layout
  int* sk_counter;       // [tiles of this problem in the launch]
};

// Several independent problems of one kind (same tile configuration, mode, split and final flags) in ONE
// launch: block b works on problem g with tile_start[g] <= b < tile_start[g+1] (a problem with a K-split owns
// ksplit blocks per tile: block tile_start[g] + s * tiles + t is part s of tile t).  Passed by value as a kernel
// argument (about 1.5 KiB).
constexpr int MAX_GROUPS = 8;
// Quarter mode: the blocks of the launch are the four half-size tiles of each tile of a 2x coarser enumeration
// (tilesM, tilesN count the fine tiles; block 4q + s is quadrant s of coarse tile qt_first + q).  It lets the 128x128
// configuration finish the last, partly filled round of a 256x256 launch.
struct GroupedGemmParams {
  int n_groups;
  int quarter;
  int tile_start[MAX_GROUPS + 1];
  GemmParams g[MAX_GROUPS];
};

// number of block tiles of one problem
long ns_gemm_tiles(int mode, const GemmParams& p);

// tile: 256 (256x256 block tile, 8 waves) or 128 (128x128, 4 waves)
// f16: 0 = the workspace matrices of the launch are bfloat16; 1 = IEEE half (see GemmParams::out_shift), not with split;
// 2 = bfloat16 operands, IEEE-half result (MODE_BX, not the final launch)
// ksplit: some problem of the launch has GemmParams::ksplit > 1 (symmetric modes, tile 128, no hi+lo pair)
hipError_t launch_ns_gemm_grouped(int tile, int mode, bool split, bool final_, const GroupedGemmParams& gp,
                                  hipStream_t stream, int f16 = 0, bool ksplit = false);
// bytes of GemmParams::sk_partial per tile of a K-split launch
constexpr long SK_TILE_BYTES = 128L * 128 * 4;
hipError_t launch_ns_gemm(int tile, int mode, bool split, bool final_, const GemmParams& p, hipStream_t stream);

}  // namespace archscale
