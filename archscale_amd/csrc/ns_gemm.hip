// Newton-Schulz GEMMs for gfx950 (CDNA4): one MFMA kernel, three epilogues.
//
// The iteration  X <- aX + (bA + cA^2)X,  A = X X^T  keeps ONLY the transposed iterate X^T ([n_long][m]):
//   SYRKT  A  = X  * X^T         P = Q = X^T, a K-MAJOR operand ([k][m]); fragments by LDS transpose reads
//   SYRK2  B  = c*A*A + b*A      P = Q = A   (A symmetric, K-contiguous); optionally + a*I on the diagonal
//   BX     X' = a*X + B*X        P = B (symmetric), Q = X^T (K-contiguous); writes X'^T (and X' only for the caller);
//                                ADDEND = false: X' = B*X for a B that already carries a*I (no X tile in the epilogue)
// SYRK and SYRK2 compute upper-triangle tiles and mirror them.  SYRK (P = Q = X, K-contiguous) is the stand-alone
// symmetric rank-k product.  All modes share one main loop (replaces ns_line_1/ns_line_2 and the cuBLAS addmm of
// lit_gpt/optim/newton_schulz_triton.py:66-139, 181-266, 371-378 and the bf16 SYRK of
// emerging_optimizers/triton_kernels/syrk.py:104-185).
//
// Operands live in zero-padded workspace buffers whose extents are multiples of
// the tile sizes, so the main loop has no bounds checks; only the FINAL epilogue
// (which writes the caller's tensor) is bounds-checked.
//
// Data path: global -> LDS with direct 16-byte loads (no VGPR round trip), two
// LDS stages, XOR-swizzled 16-byte chunks so the 128-bit MFMA operand reads are
// bank-conflict free; v_mfma_f32_32x32x16_bf16 with fp32 accumulation.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <type_traits>

#include "ns_gemm.h"

// The epilogue arithmetic is written out with explicit fmaf() and the compiler forms no fused operations of its own:
// the same element is computed by different code depending on the grid (wave-local or block-cooperative epilogue,
// 256x256 or 128x128 configuration), and all of them have to round in the same places for the result of a matrix not to
// depend on how the launch was cut into blocks.  Left to itself the compiler fuses a multiply-add with the conversion
// to half in one path and not in the other.
#pragma clang fp contract(off)

namespace archscale {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

static constexpr int BK = 64;           // bf16 elements per k-tile: 128 bytes = 8 chunks of 16 B
static constexpr int ROW_BYTES = BK * 2;

__device__ __forceinline__ uint16_t bf16_bits(float f) {
  __bf16 h = (__bf16)f;  // round to nearest even
  return __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
  return __builtin_bit_cast(float, (uint32_t)b << 16);
}
// float -> half of a value that is ROUNDED TO FLOAT first: the empty asm keeps the compiler from merging the operation
// that produced `f` with the conversion (v_fma_mixlo_f16 rounds the exact multiply-add result once, a separate
// conversion rounds twice, and which of the two a code path got would otherwise depend on its shape)
__device__ __forceinline__ uint16_t f16_bits(float f) {
  asm("" : "+v"(f));
  return __builtin_bit_cast(uint16_t, (_Float16)f);
}
__device__ __forceinline__ float f16_to_f32(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ uint2 pack4(float a, float b, float c, float d) {
  uint2 r;
  r.x = (uint32_t)bf16_bits(a) | ((uint32_t)bf16_bits(b) << 16);
  r.y = (uint32_t)bf16_bits(c) | ((uint32_t)bf16_bits(d) << 16);
  return r;
}

// LDS placement of the 16-byte chunk (row r, k-chunk c) of a [rows][64] bf16 tile.
// XOR with (r>>1)&7 makes any 16 consecutive rows at one k-chunk hit 16 distinct
// 16-byte bank groups (rows alternate between the two 128-byte halves of the 64 banks).
__device__ __forceinline__ int lds_chunk_off(int r, int c) { return r * ROW_BYTES + ((c ^ ((r >> 1) & 7)) << 4); }

// F16 = 1: the workspace matrices (operands, addend, non-final outputs) are IEEE half instead of bfloat16 (the caller's
// tensors stay bfloat16); the host keeps them in range with power-of-two factors folded into alpha / beta / out_shift.
// F16 = 2: bfloat16 operands and addend, IEEE-half output (the step from a bfloat16 iteration to a half one).
// SK: problems of the launch may carry a K-split (GemmParams::ksplit; symmetric products, 128x128 configuration): the
// blocks that share a tile leave their fp32 accumulators in the workspace and the last one to arrive adds them up in
// the order of the parts and runs the epilogue.
template <int BM, int BN, int WM, int WN, int MODE, bool SPLIT, bool FINAL, bool ADDEND, int F16, bool SK>
__global__ void __launch_bounds__((BM / WM) * (BN / WN) * 64)
ns_gemm_kernel(const GroupedGemmParams gp) {
  static_assert(!(F16 && SPLIT), "the hi+lo pair is a bfloat16 device");
  static_assert(!SK || (BM == 128 && !SPLIT && !FINAL && MODE != MODE_BX), "the K-split serves symmetric products in the small configuration");
  static_assert(F16 != 2 || (MODE == MODE_BX && !FINAL), "only X' changes its storage type");
  constexpr bool IN16 = F16 == 1, OUT16 = F16 != 0;
  constexpr int NW = (BM / WM) * (BN / WN);
  constexpr int WAVES_N = BN / WN;
  constexpr int FM = WM / 32, FN = WN / 32;
  constexpr int PBYTES = BM * ROW_BYTES, QBYTES = BN * ROW_BYTES, STAGE = PBYTES + QBYTES;
  constexpr int JP = BM / 8 / NW, JQ = BN / 8 / NW;  // 8-row slabs (1 KiB) per wave
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile rows must split over waves");
  // MODE_SYRKT is MODE_SYRK with the operand given K-major: P = Q = X^T stored [K][M] (leading dimension ldp), so the
  // iteration needs no row-major copy of X at all; the MFMA fragments then come from LDS transpose reads
  constexpr bool KMAJ = (MODE == MODE_SYRKT);
  constexpr bool SYRK_PLAIN = (MODE == MODE_SYRK || MODE == MODE_SYRKT);   // alpha * product, no addend
  constexpr bool SYM = (SYRK_PLAIN || MODE == MODE_SYRK2);
  // SPLIT means "B is a hi+lo pair": SYRK2 WRITES the pair, BX READS it as a second pass over K
  constexpr bool KSPLIT = SPLIT && MODE == MODE_BX;
  // element codecs: workspace data is half or bfloat16; the final launch writes the caller's bfloat16
  auto dec = [](uint32_t bits) { return IN16 ? f16_to_f32((uint16_t)bits) : bf16_to_f32((uint16_t)bits); };
  auto enc = [](float f) { return (OUT16 && !FINAL) ? f16_bits(f) : bf16_bits(f); };
  auto pk4 = [&](float a, float b, float c, float d) {
    uint2 r;
    r.x = (uint32_t)enc(a) | ((uint32_t)enc(b) << 16);
    r.y = (uint32_t)enc(c) | ((uint32_t)enc(d) << 16);
    return r;
  };

  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hi = lane >> 5;

  // ---- block -> (problem, matrix, tile).  Workgroups are dealt round-robin to the 8 XCDs; runs of 32
  // consecutive logical tiles (neighbouring tiles of one matrix: shared operand panels) are kept on ONE
  // XCD, i.e. in one L2, and successive runs go to successive XCDs so that long and short tiles of a
  // grouped launch spread evenly over the chip.  The grid is a multiple of 8*32.
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int logical = (((slot >> 5) << 3) + xcd) * 32 + (slot & 31);
  if (logical >= gp.tile_start[gp.n_groups]) return;
  int grp = 0;
  while (grp + 1 < gp.n_groups && logical >= gp.tile_start[grp + 1]) ++grp;
  const GemmParams p = gp.g[grp];
  int local = logical - gp.tile_start[grp];
  int ks = 0;   // part of the K range this block walks
  if constexpr (SK) {
    const int launch_tiles = (gp.tile_start[grp + 1] - gp.tile_start[grp]) / p.ksplit;
    ks = local / launch_tiles;
    local -= ks * launch_tiles;
  }
  const int sk_tile = local;   // this tile among the problem's tiles in the launch
  // grid the tile index is decoded in: the problem's own, or the 2x coarser one whose tiles this launch quarters
  int dM = p.tilesM, dN = p.tilesN, quadrant = 0;
  if (gp.quarter) {
    quadrant = local & 3;
    local = p.qt_first + (local >> 2);
    dM >>= 1;
    dN >>= 1;
  }
  const int tiles_per_mat = SYM ? (dM * (dM + 1)) / 2 : dM * dN;
  // the launch may cover only tiles [t_first, t_first + t_count) of every matrix
  const int per_mat = p.t_count > 0 ? p.t_count : tiles_per_mat;
  const int b = local / per_mat;
  int t = p.t_first + (local - b * per_mat);
  int ti, tj;
  if (SYM && dM > 8) {
    // A large upper triangle in blocks of 4 x 4 tiles, block row by block row (a diagonal block holds the 10 tiles of
    // its own upper triangle): the 32 tiles that an XCD works on at a time are two neighbouring blocks, whose operand
    // panels are 4 + 8 row panels of the one matrix.  Row by row a run would be one row panel against 32 others.
    // The last block column is `last` (1 to 4) tiles wide, and the last diagonal block a triangle of that side.
    const int nb = (dM + 3) >> 2, last = dM - 4 * (nb - 1);
    int bi = 0, rowcount = 10 + (nb - 2) * 16 + 4 * last;
    while (bi < nb - 1 && t >= rowcount) { t -= rowcount; ++bi; rowcount -= 16; }
    const int side = bi == nb - 1 ? last : 4;
    if (t < side * (side + 1) / 2) {
      int i = 0, rowlen = side;                               // rows of the triangle hold side, side - 1, ... tiles
      while (t >= rowlen) { t -= rowlen; ++i; --rowlen; }
      ti = 4 * bi + i;
      tj = 4 * bi + i + t;
    } else {
      t -= 10;
      const int bj = bi + 1 + (t >> 4) < nb - 1 ? bi + 1 + (t >> 4) : nb - 1;
      const int w = t - 16 * (bj - bi - 1);                   // 0 .. 4 x (width of block bj) - 1
      ti = 4 * bi + (w & 3);
      tj = 4 * bj + (w >> 2);
    }
  } else if (SYM) {
    ti = 0;
    int rowlen = dM;
    while (t >= rowlen) { t -= rowlen; ++ti; --rowlen; }
    tj = ti + t;
  } else if (dM > 8) {
    // A wide tile grid in blocks of 4 x 4 tiles, the blocks of one block row (4 row panels of P) one after the other:
    // the 32 tiles that an XCD works on at a time are two neighbouring blocks, 4 row panels of P and 8 of Q, 12 panels
    // per k-step.  Whole columns of dM tiles at a time would stream dM + 32 / dM panels (33 for dM = 32, 24 for 22).
    // The last block row and the last block of a row are as narrow as the grid leaves them (1 to 4 tiles).
    const int nbi = (dM + 3) >> 2, nbj = (dN + 3) >> 2;
    int bi = t / (4 * dN);
    if (bi >= nbi) bi = nbi - 1;
    const int r = t - bi * 4 * dN;
    const int h = dM - 4 * bi < 4 ? dM - 4 * bi : 4;
    int bj = r / (4 * h);
    if (bj >= nbj) bj = nbj - 1;
    const int q = r - bj * 4 * h;
    const int qc = q / h;
    ti = 4 * bi + (q - qc * h);
    tj = 4 * bj + qc;
  } else {
    tj = t / dM;   // up to 8 row panels: whole columns, 8 x 4 tiles per XCD for dM = 8
    ti = t - tj * dM;
  }
  if (gp.quarter) {
    ti = 2 * ti + (quadrant >> 1);
    tj = 2 * tj + (quadrant & 1);
    if (SYM && ti > tj) return;   // lower quadrant of a diagonal tile: its mirror image covers it
  }
  const int R0 = ti * BM, C0 = tj * BN;

  const char* Pb = KMAJ ? (const char*)(p.P + (size_t)b * p.strideP + R0)
                        : (const char*)(p.P + (size_t)b * p.strideP + (size_t)R0 * p.ldp);
  const char* P2b = KSPLIT ? (const char*)(p.P2 + (size_t)b * p.strideP + (size_t)R0 * p.ldp) : nullptr;
  const char* Qb = KMAJ ? (const char*)(p.Q + (size_t)b * p.strideQ + C0)
                        : (const char*)(p.Q + (size_t)b * p.strideQ + (size_t)C0 * p.ldq);
  int KT = p.K / BK;
  if constexpr (SK) {
    // part ks of ksplit: k-tiles [ks KT / ksplit, (ks + 1) KT / ksplit), at least one (the host checks KT >= ksplit)
    const int kt0 = (int)((long)ks * KT / p.ksplit), kt1 = (int)((long)(ks + 1) * KT / p.ksplit);
    Pb += KMAJ ? (size_t)kt0 * BK * p.ldp * 2 : (size_t)kt0 * ROW_BYTES;
    Qb += KMAJ ? (size_t)kt0 * BK * p.ldq * 2 : (size_t)kt0 * ROW_BYTES;
    KT = kt1 - kt0;
  }

  // per-lane byte offsets of the global chunks this lane copies (k-tile 0)
  uint32_t offP[JP], offQ[JQ];
  if constexpr (!KMAJ) {
#pragma unroll
    for (int j = 0; j < JP; ++j) {
      const int r = (wave * JP + j) * 8 + (lane >> 3);
      const int src = (lane & 7) ^ ((r >> 1) & 7);
      offP[j] = (uint32_t)r * (uint32_t)p.ldp * 2u + (uint32_t)src * 16u;
    }
#pragma unroll
    for (int j = 0; j < JQ; ++j) {
      const int r = (wave * JQ + j) * 8 + (lane >> 3);
      const int src = (lane & 7) ^ ((r >> 1) & 7);
      offQ[j] = (uint32_t)r * (uint32_t)p.ldq * 2u + (uint32_t)src * 16u;
    }
  } else {
    // K-major tile in LDS: 64 k-rows of BM*2 bytes; the 16-byte chunk c of row k sits at chunk c ^ ((k & 3) << 2), so
    // that four consecutive k-rows of one 64-byte column segment cover all 64 banks (what a transpose read touches)
    constexpr int CPRK = BM / 8;   // chunks per k-row
#pragma unroll
    for (int j = 0; j < JP; ++j) {
      const int pidx = (wave * JP + j) * 64 + lane, k = pidx / CPRK, cpos = pidx % CPRK;
      offP[j] = (uint32_t)k * (uint32_t)p.ldp * 2u + (uint32_t)((cpos ^ ((k & 3) << 2)) * 16);
    }
#pragma unroll
    for (int j = 0; j < JQ; ++j) {
      const int pidx = (wave * JQ + j) * 64 + lane, k = pidx / CPRK, cpos = pidx % CPRK;
      offQ[j] = (uint32_t)k * (uint32_t)p.ldq * 2u + (uint32_t)((cpos ^ ((k & 3) << 2)) * 16);
    }
  }

  const int KT_ALL = KSPLIT ? 2 * KT : KT;

  // copy j (of JP + JQ per wave) of k-tile kt: one 1 KiB slab (8 rows x 128 B) straight into stage kt & 1
  constexpr int NGL = JP + JQ;
  auto gload = [&](int kt, int j) {
    const char* pb = Pb;
    int kk = kt;
    if (KSPLIT && kt >= KT) { pb = P2b; kk = kt - KT; }
    const size_t koffP = KMAJ ? (size_t)kk * BK * p.ldp * 2 : (size_t)kk * ROW_BYTES;
    const size_t koffQ = KMAJ ? (size_t)kk * BK * p.ldq * 2 : (size_t)kk * ROW_BYTES;
    char* sP = smem + (kt & 1) * STAGE;
    char* sQ = sP + PBYTES;
    if (j < JP) __builtin_amdgcn_global_load_lds((gptr_t)(pb + offP[j] + koffP), (lptr_t)(sP + (wave * JP + j) * 1024), 16, 0, 0);
    else __builtin_amdgcn_global_load_lds((gptr_t)(Qb + offQ[j - JP] + koffQ), (lptr_t)(sQ + (wave * JQ + (j - JP)) * 1024), 16, 0, 0);
  };

  f32x16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int wr0 = (wave / WAVES_N) * WM;  // wave origin inside the block tile
  const int wc0 = (wave % WAVES_N) * WN;
  // Diagonal tile of a symmetric product: a wave whose sub-tile lies wholly BELOW the diagonal computes nothing (it
  // only takes part in the copies and the barriers); its part of the tile is the mirror image of the sub-tiles that
  // lie wholly ABOVE the diagonal, and those waves write it (two of eight waves idle in the 256x256 configuration, one
  // of four in the 128x128 one: a quarter of the tile's matrix-core work).
  static_assert((BM == 256 && BN == 256 && WM == 128 && WN == 64) || (BM == 128 && BN == 128 && WM == 64 && WN == 64),
                "checked for these two: the idle sub-tiles together are exactly the mirror image of the sub-tiles above the diagonal");
  const bool diag = SYM && (ti == tj);
  const bool idle = diag && (wc0 + WN <= wr0);
  const bool above = diag && (wr0 + WM <= wc0);
  // operand read offsets: row (w0 + i*32 + l32), chunk (2*kk + hi)
  int rdP[4], rdQ[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    rdP[kk] = lds_chunk_off(wr0 + l32, 2 * kk + hi);
    rdQ[kk] = lds_chunk_off(wc0 + l32, 2 * kk + hi);
  }
  // K-major operands: a 16-lane group reads 4 k-rows x 16 columns with one LDS transpose read; lane s = 4e + a of the
  // group points at columns 4a..4a+3 of row k0 + e and receives, as lane 4a' + b', the 4 k-values of column 4a' + b'.
  // Two such reads (k0, k0 + 4) make the 8 k-values of an MFMA operand; k0 = 16*kk + 8*(lane/32) is added below.
  int trP[FM], trQ[FN];
  if constexpr (KMAJ) {
    const int g = lane >> 4, s16 = lane & 15, e = s16 >> 2, a = s16 & 3;
    const int krow = 8 * (g >> 1) + e;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const int m = wr0 + i * 32 + (g & 1) * 16 + 4 * a;
      trP[i] = krow * (BM * 2) + (((m >> 3) ^ (e << 2)) << 4) + ((m & 7) << 1);
    }
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      const int n = wc0 + j * 32 + (g & 1) * 16 + 4 * a;
      trQ[j] = krow * (BN * 2) + (((n >> 3) ^ (e << 2)) << 4) + ((n & 7) << 1);
    }
  }

  // ---- main loop.  A k-tile is four k-steps of FM*FN MFMAs; the operand fragments of a k-step are
  // double-buffered in registers.  Every memory instruction is pinned behind an MFMA of its own:
  //   * an LDS fragment read of the NEXT k-step after each of the first FM+FN MFMAs of a k-step;
  //   * the global->LDS copies of a k-tile spread over the MFMAs of COPY_PHASES k-steps.  Issued back to
  //     back, the copies hold the wave until the texture unit has accepted all of them (about as long as
  //     the MFMAs of half a k-tile), and nothing overlaps.
  // The loop is rotated by one k-step: the barrier that publishes k-tile kt+1 sits between k-steps 2 and 3
  // of k-tile kt, so the MFMAs of k-step 3 run over the first fragment reads of the new tile and over the
  // first copies of k-tile kt+2 into the stage that the barrier has just freed.
  constexpr int NMF = FM * FN, NRD = FM + FN;
  constexpr int COPY_PHASES = 2;
  constexpr int GPP = (NGL + COPY_PHASES - 1) / COPY_PHASES;
  constexpr int G1 = GPP < NGL ? GPP : NGL, G2 = 2 * GPP < NGL ? 2 * GPP : NGL, G3 = 3 * GPP < NGL ? 3 * GPP : NGL;
  static_assert(G1 == 4 || G1 == 8 || G1 == 16, "the first wait below is written for these counts");
  bf16x8 af[2][FM], bq[2][FN];
  // The transpose reads are inline assembly: the compiler makes the builtin wait for every outstanding global->LDS
  // copy (vmcnt(0)) before each read.  The compiler therefore does not know that their results arrive late.  The raw
  // results stay in variables of their own (afr / bqr, one 64-bit pair per read) that nothing touches until the explicit
  // s_waitcnt lgkmcnt(0) before the first MFMA of the k-step; that wait is followed by empty asm statements that take
  // every raw result as a read-write operand, so each use (the packing into an MFMA operand included) depends on a
  // statement that comes after the wait.
  typedef unsigned long long u64;
  u64 afr[2][KMAJ ? FM : 1][2], bqr[2][KMAJ ? FN : 1][2];
  auto tr8 = [&](const char* base, int pitch, int kk, u64 (&raw)[2]) {
    const uint32_t a0 = (uint32_t)(uintptr_t)base + (uint32_t)(16 * kk * pitch);
    const uint32_t a1 = a0 + (uint32_t)(4 * pitch);
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(raw[0]) : "v"(a0));
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(raw[1]) : "v"(a1));
  };
  auto fread = [&](int buf, const char* sP, const char* sQ, int kk, int r) {
    if constexpr (!KMAJ) {
      if (r < FM) af[buf][r] = *(const bf16x8*)(sP + rdP[kk] + r * 32 * ROW_BYTES);
      else bq[buf][r - FM] = *(const bf16x8*)(sQ + rdQ[kk] + (r - FM) * 32 * ROW_BYTES);
    } else {
      if (r < FM) tr8(sP + trP[r], BM * 2, kk, afr[buf][r]);
      else tr8(sQ + trQ[r - FM], BN * 2, kk, bqr[buf][r - FM]);
    }
  };
  // K-major operands: wait for the transpose reads of fragment buffer `buf`, then pack them
  auto land = [&](int buf) {
    if constexpr (KMAJ) {
      typedef u64 u64x2 __attribute__((ext_vector_type(2)));
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int i = 0; i < FM; ++i) asm volatile("" : "+v"(afr[buf][i][0]), "+v"(afr[buf][i][1]));
#pragma unroll
      for (int j = 0; j < FN; ++j) asm volatile("" : "+v"(bqr[buf][j][0]), "+v"(bqr[buf][j][1]));
#pragma unroll
      for (int i = 0; i < FM; ++i) { const u64x2 v = {afr[buf][i][0], afr[buf][i][1]}; af[buf][i] = __builtin_bit_cast(bf16x8, v); }
#pragma unroll
      for (int j = 0; j < FN; ++j) { const u64x2 v = {bqr[buf][j][0], bqr[buf][j][1]}; bq[buf][j] = __builtin_bit_cast(bf16x8, v); }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // one k-step: MFMAs on fragment buffer CBUF (when COMPUTE), reads of k-step RKK of the stage at (rP, rQ)
  // into buffer RBUF (when READ), copies [G0, G1) of k-tile gt
  auto phase = [&](auto compute, auto read, auto cbuf_, auto rbuf_, const char* rP, const char* rQ, auto rkk_, int gt,
                   auto g0_, auto g1_) {
    constexpr bool COMPUTE = decltype(compute)::value, READ = decltype(read)::value;
    constexpr int cbuf = decltype(cbuf_)::value, rbuf = decltype(rbuf_)::value, rkk = decltype(rkk_)::value;
    constexpr int g0 = decltype(g0_)::value, g1 = decltype(g1_)::value;
    if constexpr (COMPUTE) land(cbuf);
#pragma unroll
    for (int q = 0; q < NMF; ++q) {
      if (COMPUTE)
        acc[q / FN][q % FN] = IN16 ? __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, af[cbuf][q / FN]), __builtin_bit_cast(f16x8, bq[cbuf][q % FN]), acc[q / FN][q % FN], 0, 0, 0)
                                  : __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[cbuf][q / FN], bq[cbuf][q % FN], acc[q / FN][q % FN], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      const int g_lo = g0 + (q * (g1 - g0) + NMF - 1) / NMF, g_hi = g0 + ((q + 1) * (g1 - g0) + NMF - 1) / NMF;
      if (READ && q < NRD) fread(rbuf, rP, rQ, rkk, q);
#pragma unroll
      for (int g = 0; g < NGL; ++g)
        if (g >= g_lo && g < g_hi) gload(gt, g);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using Yes = std::true_type;
  using No = std::false_type;
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  using C1 = std::integral_constant<int, G1>;
  using C2 = std::integral_constant<int, G2>;
  using C3 = std::integral_constant<int, G3>;
  using C4 = std::integral_constant<int, NGL>;
  // k-steps 0..2 of k-tile kt (with the rest of the copies of kt+1), barrier, k-step 3 (with the first
  // copies of kt+2).  COPY_REST / NEXT / COPY_FIRST: k-tiles kt+1 / kt+1 / kt+2 exist.  ACTIVE = false is the same
  // sequence of copies, waits and barriers without the fragment reads and the MFMAs: what a wave runs whose sub-tile
  // lies below the diagonal of a symmetric product (one code path, so the barriers of the two kinds of wave cannot
  // drift apart).
  auto ktile = [&](int kt, auto copy_rest, auto next, auto copy_first, auto active) {
    constexpr bool COPY_REST = decltype(copy_rest)::value, NEXT = decltype(next)::value, COPY_FIRST = decltype(copy_first)::value;
    using Act = std::integral_constant<bool, decltype(active)::value>;
    const char* sP = smem + (kt & 1) * STAGE;
    const char* sQ = sP + PBYTES;
    const char* nP = smem + ((kt + 1) & 1) * STAGE;
    const char* nQ = nP + PBYTES;
    if constexpr (COPY_REST) {
      phase(Act{}, Act{}, I0{}, I1{}, sP, sQ, I1{}, kt + 1, C1{}, C2{});
      phase(Act{}, Act{}, I1{}, I0{}, sP, sQ, I2{}, kt + 1, C2{}, C3{});
      phase(Act{}, Act{}, I0{}, I1{}, sP, sQ, I3{}, kt + 1, C3{}, C4{});
    } else {
      phase(Act{}, Act{}, I0{}, I1{}, sP, sQ, I1{}, 0, I0{}, I0{});
      phase(Act{}, Act{}, I1{}, I0{}, sP, sQ, I2{}, 0, I0{}, I0{});
      phase(Act{}, Act{}, I0{}, I1{}, sP, sQ, I3{}, 0, I0{}, I0{});
    }
    if constexpr (NEXT) {
      // this wave's copies of kt+1 have landed and its reads of kt are done; after the barrier that holds for all
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (COPY_FIRST) phase(Act{}, Act{}, I1{}, I0{}, nP, nQ, I0{}, kt + 2, I0{}, C1{});
      else phase(Act{}, Act{}, I1{}, I0{}, nP, nQ, I0{}, 0, I0{}, I0{});
    } else {
      phase(Act{}, No{}, I1{}, I0{}, nP, nQ, I0{}, 0, I0{}, I0{});
    }
  };
  // the whole K range: ACTIVE waves multiply, the others only copy and meet the barriers
  auto k_range = [&](auto active) {
    using Act = std::integral_constant<bool, decltype(active)::value>;
    if constexpr (Act::value) {
#pragma unroll
      for (int r = 0; r < NRD; ++r) fread(0, smem, smem + PBYTES, 0, r);
    }
    for (int kt = 0; kt + 2 < KT_ALL; ++kt) ktile(kt, Yes{}, Yes{}, Yes{}, Act{});
    if (KT_ALL > 1) ktile(KT_ALL - 2, Yes{}, Yes{}, No{}, Act{});
    ktile(KT_ALL - 1, No{}, No{}, No{}, Act{});
  };

#pragma unroll
  for (int g = 0; g < NGL; ++g) gload(0, g);
  if (KT_ALL > 1) {
#pragma unroll
    for (int g = 0; g < G1; ++g) gload(1, g);
    // k-tile 0 has landed once at most the G1 younger copies are outstanding
    if constexpr (G1 == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else if constexpr (G1 == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __syncthreads();
  if (!idle) k_range(Yes{});
  else k_range(No{});

  // ---- epilogue.  acc[i][j][e] of lane l is element
  //   rl = wr0 + i*32 + 8*(e/4) + 4*(l/32) + e%4  (row in the tile),   cl = wc0 + j*32 + l%32  (column)
  // so a lane owns 4 consecutive rows of one column.  Every global access of the epilogue goes through
  // LDS (the operand stages are dead by now) so that it is a 16-byte, row-contiguous access:
  //   * the addend tile is copied in as its transposed image  S[cl][rl]  (it is read as E[col][row..row+3]);
  //   * the transposed output (mirror of a symmetric product, X'^T) is staged as S[cl][rl] with 8-byte
  //     LDS writes and flushed row by row;
  //   * the row-major output is staged as D[rl][cl] with 2-byte LDS writes and flushed row by row.
  // Scattered 8-byte / 2-byte global accesses straight from the accumulator layout flood L2 with
  // partial-line requests and cost a quarter of the kernel.
  static_assert(BM == BN, "square block tiles");
  constexpr int NT = NW * 64;
  if constexpr (SK) {
    if (p.ksplit > 1) {
      // Every part leaves its accumulators in the workspace (accumulator layout: one word per lane and accumulator
      // register, so every access of a wave is a run of 256 bytes), waits until they have arrived, and counts itself in.
      // The block that finds itself last adds ALL parts in the order 0, 1, ... (its own from memory like the others: the
      // sum of a tile is the same whichever block came last) and goes on to the epilogue; the others are done.  Nobody
      // waits for anybody.  The partial results travel as system-scope accesses (written through, read past the
      // caches): the eight L2 caches of the chip are not coherent with each other, and the alternative - a release /
      // acquire fence per block - writes back and invalidates a whole L2 each time (measured: the product twice as slow).
      __shared__ int sk_last;
      float* part = p.sk_partial + (size_t)sk_tile * p.ksplit * (BM * BN);
      if (!idle) {
        float* dst = part + (size_t)ks * (BM * BN);
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e)
              __hip_atomic_store(dst + ((i * FN + j) * 16 + e) * NT + tid, acc[i][j][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this lane's stores have been acknowledged
      __syncthreads();
      if (tid == 0) {
        const int old = __hip_atomic_fetch_add(p.sk_counter + sk_tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int last = old == p.ksplit - 1;
        if (last) __hip_atomic_store(p.sk_counter + sk_tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
        sk_last = last;
      }
      __syncthreads();
      if (!sk_last) return;
      if (!idle) {
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
        for (int sidx = 0; sidx < p.ksplit; ++sidx) {
          const float* src = part + (size_t)sidx * (BM * BN);
#pragma unroll
          for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
              for (int e = 0; e < 16; ++e)
                acc[i][j][e] += __hip_atomic_load(src + ((i * FN + j) * 16 + e) * NT + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
      }
    }
  }
  constexpr int TPITCH = BN * 2;            // bytes per staged row (both images)
  constexpr int CPRT = BN / 8;              // 16-byte chunks per staged row
  constexpr int PASSES = (BM * BN / 8) / NT;
  static_assert(BM * BN * 2 <= 2 * STAGE, "staging tile must fit in the operand stages");
  // optional per-matrix scale of the operand that was left out of it (deferred normalisation): the product of two
  // such operands carries sc^2, a product with one of them (and its addend) carries sc
  const float sc = p.scale ? p.scale[b] : 1.f;
  const float bx_sc = sc * __builtin_ldexpf(1.f, p.out_shift);   // MODE_BX: scale of the result (a power of two from the host)
  const float alpha = SYRK_PLAIN ? p.alpha * sc * sc : p.alpha, beta = p.beta;
  // A diagonal tile of a product of a matrix with ITSELF is symmetric bit for bit as it comes out of the matrix cores
  // (element (i,j) and element (j,i) are the same products summed in the same order over k), so it takes the wave-local
  // epilogue below like any other tile and writes one image.  A diagonal tile of P Q^T with two different (commuting,
  // symmetric) matrices is symmetric only up to rounding: it keeps its upper half and reflects it.
  const bool self_product = p.P == p.Q && p.strideP == p.strideQ && p.ldp == p.ldq;
  // (the instantiation that writes a hi+lo pair keeps the reflecting path for every diagonal tile: its epilogue has no
  // registers to spare for the diagonal term in the wave-local one)
  const bool reflect = diag && (!self_product || (SPLIT && MODE == MODE_SYRK2));
  // S[cl][rl]: chunk index XOR cl, so the 32 lanes of an 8-byte access (32 different cl) spread over all banks
  auto s_off = [](int cl, int rl) { return cl * TPITCH + ((((rl >> 3) ^ cl) & (CPRT - 1)) << 4) + ((rl & 7) << 1); };
  auto s_chunk = [](int cl, int ch) { return cl * TPITCH + (((ch ^ cl) & (CPRT - 1)) << 4); };
  // D[rl][cl]: 64-byte halves of a row swapped on rows with bit 2 set, so the two half-waves of a 2-byte
  // access (rows r and r+4) hit different banks
  auto d_off = [](int rl, int byte_in_row) { return rl * TPITCH + (byte_in_row ^ (((rl >> 2) & 1) << 6)); };

  // row-contiguous copy of a staged image to global memory; `swz` maps (staged row, chunk) -> LDS offset
  auto flush = [&](auto swz, __bf16* dst, long bstride, int ld, int row0, int col0, int rows_valid, int cols_valid) {
    __bf16* base = dst + (size_t)b * bstride;
    const bool vec_ok = !FINAL || ((ld & 7) == 0 && (bstride & 7) == 0 && (((uintptr_t)dst) & 15) == 0);
#pragma unroll 4
    for (int t = 0; t < PASSES; ++t) {
      const int q = t * NT + tid;
      const int sr = q / CPRT, ch = q - sr * CPRT;
      const uint4 val = *(const uint4*)(smem + swz(sr, ch));
      const int row = row0 + sr, col = col0 + ch * 8;
      if (!FINAL) {
        *(uint4*)(base + (size_t)row * ld + col) = val;
      } else if (row < rows_valid) {  // caller's tensor: true extents, arbitrary leading dimension
        if (vec_ok && col + 7 < cols_valid) {
          *(uint4*)(base + (size_t)row * ld + col) = val;
        } else {
          const uint32_t w[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
          for (int k = 0; k < 8; ++k)
            if (col + k < cols_valid) ((uint16_t*)base)[(size_t)row * ld + col + k] = (uint16_t)(w[k >> 1] >> ((k & 1) * 16));
        }
      }
    }
  };
  auto s_swz = [&](int sr, int ch) { return s_chunk(sr, ch); };
  auto d_swz = [&](int sr, int ch) { return d_off(sr, ch * 16); };

  __syncthreads();  // every wave is done reading the operand stages

  if (!reflect) {
    if (idle) return;
    // ---- wave-local epilogue (every tile except the diagonal tiles of a product of two different matrices).
    // Each wave stages its own WM x WN sub-tile in its own LDS region as the transposed image
    // W[c][r] (c = column in the sub-tile, r = row), so nothing below needs a block barrier:
    //   addend in:   16-byte direct copies of E[col][row..] rows into W, read back 8 bytes per lane
    //   W <- values: 8-byte LDS writes (a lane owns 4 consecutive r of one c)
    //   transposed / mirrored image out: 16-byte reads of W rows -> 16-byte stores, 256 B contiguous per row
    //   row-major image out: LDS transpose reads (ds_read_b64_tr_b16: a lane receives 4 consecutive c of one
    //     r; two of them make 16 bytes) -> 16-byte stores, 64 B contiguous per row
    constexpr int WROW = WM * 2;                  // bytes per W row
    constexpr int RCH = WM / 8;                   // 16-byte chunks per W row
    constexpr int WBYTES = WN * WROW;
    constexpr int WSLABS = WBYTES / 1024;         // 64-chunk slabs of one region
    static_assert(NW * WBYTES <= 2 * STAGE, "wave regions must fit in the operand stages");
    char* W = smem + wave * WBYTES;
    // chunk swizzle: 4 consecutive rows of W land in 4 different pairs of 16-byte bank groups
    auto sw = [](int c) { return (((c & 7) << 1) | ((c >> 3) & 1)) & (RCH - 1); };
    auto w_off = [&](int c, int r) { return c * WROW + ((((r >> 3) ^ sw(c)) & (RCH - 1)) << 4) + ((r & 7) << 1); };
    const int wrow0 = R0 + wr0, wcol0 = C0 + wc0;  // global origin of this wave's sub-tile

    // MODE_BX without an addend (ADDEND = false): a*I was folded into B's diagonal by the product that made B
    constexpr bool has_e = !SYRK_PLAIN && (MODE != MODE_BX || ADDEND);
    if constexpr (has_e) {
      const char* Eb = (const char*)(p.E + (size_t)b * p.strideE + (size_t)wcol0 * p.lde + wrow0);
#pragma unroll
      for (int t = 0; t < WSLABS; ++t) {
        const int q = t * 64 + lane;
        const int c = q / RCH, ch = (q % RCH) ^ sw(c);
        __builtin_amdgcn_global_load_lds((gptr_t)(Eb + ((size_t)c * p.lde + ch * 8) * 2), (lptr_t)(W + t * 1024), 16, 0, 0);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    if constexpr (MODE == MODE_BX && !has_e) {
      if (bx_sc != 1.f) {
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] *= bx_sc;
      }
    } else
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        const int c = j * 32 + l32;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int r = i * 32 + 8 * g + 4 * hi;
          if (SYRK_PLAIN) {
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[i][j][4 * g + q] *= alpha;
          } else {
            const uint2 e = *(const uint2*)(W + w_off(c, r));
            const float e0 = dec(e.x & 0xffff), e1 = dec(e.x >> 16);
            const float e2 = dec(e.y & 0xffff), e3 = dec(e.y >> 16);
            if (MODE == MODE_SYRK2) {
              acc[i][j][4 * g + 0] = fmaf(alpha, acc[i][j][4 * g + 0], beta * e0);
              acc[i][j][4 * g + 1] = fmaf(alpha, acc[i][j][4 * g + 1], beta * e1);
              acc[i][j][4 * g + 2] = fmaf(alpha, acc[i][j][4 * g + 2], beta * e2);
              acc[i][j][4 * g + 3] = fmaf(alpha, acc[i][j][4 * g + 3], beta * e3);
            } else {
              acc[i][j][4 * g + 0] = fmaf(alpha, e0, acc[i][j][4 * g + 0]) * bx_sc;
              acc[i][j][4 * g + 1] = fmaf(alpha, e1, acc[i][j][4 * g + 1]) * bx_sc;
              acc[i][j][4 * g + 2] = fmaf(alpha, e2, acc[i][j][4 * g + 2]) * bx_sc;
              acc[i][j][4 * g + 3] = fmaf(alpha, e3, acc[i][j][4 * g + 3]) * bx_sc;
            }
          }
        }
      }

    if constexpr (MODE == MODE_SYRK2 && !SPLIT) {
      // B + a I: in a diagonal tile (R0 == C0) the diagonal of the matrix runs through the 32x32 blocks (j + d32, j) of
      // this wave's sub-tile with 32 d32 == wc0 - wr0, where it is the element with 8*g + q == l32 - 4*hi.  Only those
      // blocks are touched, with a select per element.
      const int d32 = (wc0 - wr0) / 32;   // wave-uniform
      if (diag && d32 >= 0 && (wc0 - wr0) % 32 == 0) {
        const int t = l32 - 4 * hi;
        const float da = p.diag_add;
#pragma unroll
        for (int dd = 0; dd < FM; ++dd)
          if (dd == d32) {
#pragma unroll
            for (int j = 0; j < FN; ++j)
              if (j + dd < FM) {
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[j + dd][j][e] += (8 * (e >> 2) + (e & 3) == t) ? da : 0.f;
              }
          }
      }
    }

    auto store_wave = [&](__bf16* Cdst, int lane) {
      const int l32 = lane & 31, hi = lane >> 5;
      // W[c][r] <- bf16(acc)
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g)
            *(uint2*)(W + w_off(j * 32 + l32, i * 32 + 8 * g + 4 * hi)) =
                pk4(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
      // transposed / mirrored image: rows of W
      __bf16* Tdst = SYM ? Cdst : p.Ct;
      if (Tdst && (!diag || above)) {   // in a diagonal tile: only the image of the idle waves' part
        const long tbs = SYM ? p.strideC : p.strideCt;
        const int tld = SYM ? p.ldc : p.ldct;
        __bf16* base = Tdst + (size_t)b * tbs;
        const bool vec_ok = !FINAL || ((tld & 7) == 0 && (tbs & 7) == 0 && (((uintptr_t)Tdst) & 15) == 0);
#pragma unroll
        for (int t = 0; t < WSLABS; ++t) {
          const int q = t * 64 + lane;
          const int c = q / RCH, ch = q % RCH;
          const uint4 val = *(const uint4*)(W + c * WROW + (((ch ^ sw(c)) & (RCH - 1)) << 4));
          const int orow = wcol0 + c, ocol = wrow0 + ch * 8;   // row of the transposed image = column of the tile
          if (!FINAL) {
            *(uint4*)(base + (size_t)orow * tld + ocol) = val;
          } else if (orow < p.n_valid) {
            if (vec_ok && ocol + 7 < p.m_valid) {
              *(uint4*)(base + (size_t)orow * tld + ocol) = val;
            } else {
              const uint32_t w[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
              for (int k = 0; k < 8; ++k)
                if (ocol + k < p.m_valid) ((uint16_t*)base)[(size_t)orow * tld + ocol + k] = (uint16_t)(w[k >> 1] >> ((k & 1) * 16));
            }
          }
        }
      }
      // row-major image: transpose reads.  In a 16-lane group, source lane s points at W[c0 + s/4][r0 + 4*(s%4) ..+3];
      // lane L of the group then holds W[c0 .. c0+3][r0 + L].
      if (SYM || p.C) {
        __bf16* base = Cdst + (size_t)b * p.strideC;
        const bool vec_ok = !FINAL || ((p.ldc & 7) == 0 && (p.strideC & 7) == 0 && (((uintptr_t)Cdst) & 15) == 0);
        const int grp = lane >> 4, s = lane & 15;
#pragma unroll
        for (int rb = 0; rb < WM / 16; ++rb)
#pragma unroll
          for (int cb = 0; cb < WN / 32; ++cb) {
            const int c0 = cb * 32 + grp * 8;
            const s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) s16x4*)(W + w_off(c0 + (s >> 2), rb * 16 + 4 * (s & 3))));
            const s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) s16x4*)(W + w_off(c0 + 4 + (s >> 2), rb * 16 + 4 * (s & 3))));
            uint4 val;
            val.x = (uint32_t)(uint16_t)lo4[0] | ((uint32_t)(uint16_t)lo4[1] << 16);
            val.y = (uint32_t)(uint16_t)lo4[2] | ((uint32_t)(uint16_t)lo4[3] << 16);
            val.z = (uint32_t)(uint16_t)hi4[0] | ((uint32_t)(uint16_t)hi4[1] << 16);
            val.w = (uint32_t)(uint16_t)hi4[2] | ((uint32_t)(uint16_t)hi4[3] << 16);
            const int orow = wrow0 + rb * 16 + s, ocol = wcol0 + c0;
            if (!FINAL) {
              *(uint4*)(base + (size_t)orow * p.ldc + ocol) = val;
            } else if (orow < p.m_valid) {
              if (vec_ok && ocol + 7 < p.n_valid) {
                *(uint4*)(base + (size_t)orow * p.ldc + ocol) = val;
              } else {
                const uint32_t w[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
                for (int k = 0; k < 8; ++k)
                  if (ocol + k < p.n_valid) ((uint16_t*)base)[(size_t)orow * p.ldc + ocol + k] = (uint16_t)(w[k >> 1] >> ((k & 1) * 16));
              }
            }
          }
      }
    };

    store_wave(p.C, lane);
    if (SPLIT && MODE == MODE_SYRK2) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[i][j][e] -= bf16_to_f32(bf16_bits(acc[i][j][e]));
      __builtin_amdgcn_sched_barrier(0);
      // the second copy of the store code gets its lane id through an opaque move, so that its addresses are computed
      // here and not hoisted above the first copy (where they cost hundreds of spilled registers)
      int lane2 = lane;
      asm volatile("" : "+v"(lane2));
      store_wave(p.C2, lane2);
    }
    return;
  }

  // ---- block-cooperative epilogue for the diagonal tiles of a symmetric product (the upper half is
  // reflected across waves so that the product is bit-symmetric)

  // 1. fold the addend into the accumulators: acc <- alpha*acc + beta*E (SYRK2), acc + alpha*E (BX), alpha*acc (SYRK)
  if (!SYRK_PLAIN) {
    // E[C0 + cl][R0 + rl] -> S[cl][rl], two staged rows (1 KiB) per wave-wide copy
    const char* Eb = (const char*)(p.E + (size_t)b * p.strideE + (size_t)C0 * p.lde + R0);
#pragma unroll
    for (int t = 0; t < PASSES; ++t) {
      const int slab = wave * PASSES + t;                  // 64 chunks
      const int q = slab * 64 + lane;
      const int sr = q / CPRT, cpos = q - sr * CPRT;
      const int src = (cpos ^ sr) & (CPRT - 1);
      __builtin_amdgcn_global_load_lds((gptr_t)(Eb + ((size_t)sr * p.lde + src * 8) * 2), (lptr_t)(smem + slab * 1024), 16, 0, 0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      const int cl = wc0 + j * 32 + l32;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int rl = wr0 + i * 32 + 8 * g + 4 * hi;
        if (SYRK_PLAIN) {
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[i][j][4 * g + q] *= alpha;
        } else {
          const uint2 e = *(const uint2*)(smem + s_off(cl, rl));
          const float e0 = dec(e.x & 0xffff), e1 = dec(e.x >> 16);
          const float e2 = dec(e.y & 0xffff), e3 = dec(e.y >> 16);
          if (MODE == MODE_SYRK2) {
            acc[i][j][4 * g + 0] = fmaf(alpha, acc[i][j][4 * g + 0], beta * e0);
            acc[i][j][4 * g + 1] = fmaf(alpha, acc[i][j][4 * g + 1], beta * e1);
            acc[i][j][4 * g + 2] = fmaf(alpha, acc[i][j][4 * g + 2], beta * e2);
            acc[i][j][4 * g + 3] = fmaf(alpha, acc[i][j][4 * g + 3], beta * e3);
            // diagonal of the matrix (this path runs on diagonal tiles only: R0 == C0)
#pragma unroll
            for (int q = 0; q < 4; ++q)
              if (rl + q == cl) acc[i][j][4 * g + q] += p.diag_add;
          } else {
            acc[i][j][4 * g + 0] = fmaf(alpha, e0, acc[i][j][4 * g + 0]) * bx_sc;
            acc[i][j][4 * g + 1] = fmaf(alpha, e1, acc[i][j][4 * g + 1]) * bx_sc;
            acc[i][j][4 * g + 2] = fmaf(alpha, e2, acc[i][j][4 * g + 2]) * bx_sc;
            acc[i][j][4 * g + 3] = fmaf(alpha, e3, acc[i][j][4 * g + 3]) * bx_sc;
          }
        }
      }
    }
  if (!SYRK_PLAIN) __syncthreads();  // the addend image is consumed; LDS is free again

  // stores the accumulators as bf16 to Cdst (row-major image) and to its transposed / mirrored image
  auto store_all = [&](__bf16* Cdst, int lane) {
    const int l32 = lane & 31, hi = lane >> 5;
    // 2. transposed image
    const bool want_t = SYM ? !diag : (p.Ct != nullptr);
    if (want_t) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          const int cl = wc0 + j * 32 + l32;
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int rl = wr0 + i * 32 + 8 * g + 4 * hi;
            *(uint2*)(smem + s_off(cl, rl)) =
                pk4(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
          }
        }
      __syncthreads();
      if (SYM) flush(s_swz, Cdst, p.strideC, p.ldc, C0, R0, 0, 0);
      else flush(s_swz, p.Ct, p.strideCt, p.ldct, C0, R0, p.n_valid, p.m_valid);
      __syncthreads();
    }
    // 3. row-major image
    if (SYM || p.C) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          const int cl = wc0 + j * 32 + l32;
#pragma unroll
          for (int g = 0; g < 4; ++g) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int rl = wr0 + i * 32 + 8 * g + 4 * hi + q;
              const uint16_t bits = enc(acc[i][j][4 * g + q]);
              if (!diag) {
                *(uint16_t*)(smem + d_off(rl, cl * 2)) = bits;
              } else if (cl >= rl) {
                // diagonal tile: keep the upper half and reflect it, so the product is bit-symmetric
                *(uint16_t*)(smem + d_off(rl, cl * 2)) = bits;
                *(uint16_t*)(smem + d_off(cl, rl * 2)) = bits;
              }
            }
          }
        }
      __syncthreads();
      flush(d_swz, Cdst, p.strideC, p.ldc, R0, C0, p.m_valid, p.n_valid);
    }
  };

  store_all(p.C, lane);
  if (SPLIT && MODE == MODE_SYRK2) {
    __builtin_amdgcn_sched_barrier(0);
    // low half of the bf16 split: acc <- acc - bf16(acc), stored the same way to C2
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] -= bf16_to_f32(bf16_bits(acc[i][j][e]));
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    int lane2 = lane;
    asm volatile("" : "+v"(lane2));   // as above: keep the second copy's addresses out of the first copy
    store_all(p.C2, lane2);
  }
}

// ---------------------------------------------------------------------------
// launch
// ---------------------------------------------------------------------------
long ns_gemm_tiles(int mode, const GemmParams& p) {
  const bool sym = (mode == MODE_SYRK || mode == MODE_SYRK2 || mode == MODE_SYRKT);
  return (long)p.batch * (sym ? (long)p.tilesM * (p.tilesM + 1) / 2 : (long)p.tilesM * p.tilesN);
}

template <int BM, int BN, int WM, int WN, int MODE, bool SPLIT, bool FINAL, bool ADDEND = true, int F16 = 0, bool SK = false>
static hipError_t launch_one(const GroupedGemmParams& gp, hipStream_t stream) {
  constexpr int NT = (BM / WM) * (BN / WN) * 64;
  constexpr int SMEM = 2 * (BM + BN) * ROW_BYTES;
  auto kern = ns_gemm_kernel<BM, BN, WM, WN, MODE, SPLIT, FINAL, ADDEND, F16, SK>;
  // the dynamic-LDS limit is an attribute of the function on ONE device: set it once per device and instantiation
  // (the call is idempotent, so two threads that race on the first launch only repeat it)
  static std::atomic<bool> attr_set[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const bool slot = dev >= 0 && dev < 64;
  if (!slot || !attr_set[dev].load(std::memory_order_acquire)) {
    e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
    if (e != hipSuccess) return e;
    if (slot) attr_set[dev].store(true, std::memory_order_release);
  }
  const long tiles = gp.tile_start[gp.n_groups];
  if (tiles <= 0) return hipSuccess;
  const long grid = (tiles + 255) / 256 * 256;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), SMEM, stream, gp);
  return hipGetLastError();
}

template <int BM, int BN, int WM, int WN, int F16>
static hipError_t launch_cfg(int mode, bool split, bool final_, const GroupedGemmParams& p, hipStream_t s) {
  if (F16 && split) return hipErrorInvalidValue;
  if constexpr (F16 == 2) {
    if (mode != MODE_BX || final_) return hipErrorInvalidValue;
    return p.g[0].E ? launch_one<BM, BN, WM, WN, MODE_BX, false, false, true, 2>(p, s)
                    : launch_one<BM, BN, WM, WN, MODE_BX, false, false, false, 2>(p, s);
  } else {
    switch (mode) {
      case MODE_SYRK:
        return launch_one<BM, BN, WM, WN, MODE_SYRK, false, false, true, F16>(p, s);
      case MODE_SYRKT:
        return launch_one<BM, BN, WM, WN, MODE_SYRKT, false, false, true, F16>(p, s);
      case MODE_SYRK2:
        if constexpr (!F16) {
          if (split) return launch_one<BM, BN, WM, WN, MODE_SYRK2, true, false>(p, s);
        }
        return launch_one<BM, BN, WM, WN, MODE_SYRK2, false, false, true, F16>(p, s);
      case MODE_BX:
        if constexpr (!F16) {
          if (split) {
            if (p.g[0].E)
              return final_ ? launch_one<BM, BN, WM, WN, MODE_BX, true, true>(p, s)
                            : launch_one<BM, BN, WM, WN, MODE_BX, true, false>(p, s);
            return final_ ? launch_one<BM, BN, WM, WN, MODE_BX, true, true, false>(p, s)
                          : launch_one<BM, BN, WM, WN, MODE_BX, true, false, false>(p, s);
          }
        }
        if (p.g[0].E)
          return final_ ? launch_one<BM, BN, WM, WN, MODE_BX, false, true, true, F16>(p, s)
                        : launch_one<BM, BN, WM, WN, MODE_BX, false, false, true, F16>(p, s);
        return final_ ? launch_one<BM, BN, WM, WN, MODE_BX, false, true, false, F16>(p, s)
                      : launch_one<BM, BN, WM, WN, MODE_BX, false, false, false, F16>(p, s);
    }
    return hipErrorInvalidValue;
  }
}

// the symmetric products of the 128x128 configuration with a K-split
template <int F16>
static hipError_t launch_ksplit(int mode, const GroupedGemmParams& p, hipStream_t s) {
  switch (mode) {
    case MODE_SYRK: return launch_one<128, 128, 64, 64, MODE_SYRK, false, false, true, F16, true>(p, s);
    case MODE_SYRKT: return launch_one<128, 128, 64, 64, MODE_SYRKT, false, false, true, F16, true>(p, s);
    case MODE_SYRK2: return launch_one<128, 128, 64, 64, MODE_SYRK2, false, false, true, F16, true>(p, s);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_ns_gemm_grouped(int tile, int mode, bool split, bool final_, const GroupedGemmParams& gp,
                                  hipStream_t stream, int f16, bool ksplit) {
  if (gp.n_groups < 1 || gp.n_groups > MAX_GROUPS) return hipErrorInvalidValue;
  const bool sym = (mode == MODE_SYRK || mode == MODE_SYRK2 || mode == MODE_SYRKT);
  if (ksplit && (!sym || tile != 128 || split || final_ || f16 == 2)) return hipErrorInvalidValue;
  for (int i = 0; i < gp.n_groups; ++i) {
    const GemmParams& g = gp.g[i];
    if (g.K % BK != 0 || g.K <= 0 || gp.tile_start[i + 1] < gp.tile_start[i]) return hipErrorInvalidValue;
    if (mode == MODE_SYRK2 && !g.E) return hipErrorInvalidValue;
    if (mode == MODE_BX && (g.E == nullptr) != (gp.g[0].E == nullptr)) return hipErrorInvalidValue;  // one kernel per launch
    long blocks = (long)gp.tile_start[i + 1] - gp.tile_start[i];
    if (!ksplit) {
      if (g.ksplit > 1) return hipErrorInvalidValue;
    } else {
      // every part walks at least one k-tile; the parts of a tile find their partial results and their counter
      if (g.ksplit < 1 || g.ksplit > g.K / BK || blocks % g.ksplit) return hipErrorInvalidValue;
      if (g.ksplit > 1 && (!g.sk_partial || !g.sk_counter || ((uintptr_t)g.sk_partial & 15))) return hipErrorInvalidValue;
      blocks /= g.ksplit;
    }
    // every block must decode to a tile inside the problem
    if (g.t_first < 0 || g.t_count < 0 || (g.t_count == 0 && g.t_first != 0)) return hipErrorInvalidValue;
    if (!gp.quarter) {
      const long per = ns_gemm_tiles(mode, g) / g.batch;
      if (g.t_count ? (g.t_first + g.t_count > per || blocks > (long)g.batch * g.t_count) : blocks > ns_gemm_tiles(mode, g))
        return hipErrorInvalidValue;
    } else {
      if ((g.tilesM & 1) || (!sym && (g.tilesN & 1)) || g.qt_first < 0 || (blocks & 3)) return hipErrorInvalidValue;
      const long cm = g.tilesM / 2, cn = g.tilesN / 2;
      const long per = sym ? cm * (cm + 1) / 2 : cm * cn;
      if (g.t_count && g.t_first + g.t_count > per) return hipErrorInvalidValue;
      const long coarse = (long)g.batch * (g.t_count ? g.t_count : per);
      if (g.qt_first + blocks / 4 > coarse) return hipErrorInvalidValue;
    }
  }
  if (ksplit) {
    if (f16 == 1) return launch_ksplit<1>(mode, gp, stream);
    return launch_ksplit<0>(mode, gp, stream);
  }
  if (f16 == 1) {
    if (tile == 256) return launch_cfg<256, 256, 128, 64, 1>(mode, split, final_, gp, stream);
    if (tile == 128) return launch_cfg<128, 128, 64, 64, 1>(mode, split, final_, gp, stream);
  } else if (f16 == 2) {
    if (tile == 256) return launch_cfg<256, 256, 128, 64, 2>(mode, split, final_, gp, stream);
    if (tile == 128) return launch_cfg<128, 128, 64, 64, 2>(mode, split, final_, gp, stream);
  } else if (f16 == 0) {
    if (tile == 256) return launch_cfg<256, 256, 128, 64, 0>(mode, split, final_, gp, stream);
    if (tile == 128) return launch_cfg<128, 128, 64, 64, 0>(mode, split, final_, gp, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_ns_gemm(int tile, int mode, bool split, bool final_, const GemmParams& p, hipStream_t stream) {
  GroupedGemmParams gp = {};
  gp.n_groups = 1;
  gp.g[0] = p;
  const long tiles = ns_gemm_tiles(mode, p);
  if (tiles > 0x7ffffff0L) return hipErrorInvalidValue;
  gp.tile_start[1] = (int)tiles;
  return launch_ns_gemm_grouped(tile, mode, split, final_, gp, stream);
}

}  // namespace archscale
