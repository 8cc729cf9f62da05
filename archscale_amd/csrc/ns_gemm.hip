// Newton-Schulz GEMMs for gfx950 (CDNA4): one "NT" MFMA kernel, three epilogues.
//
// Every product of the quintic iteration  X <- aX + (bA + cA^2)X,  A = X X^T  is
// written as  C[m][n] = sum_k P[m][k] * Q[n][k]  with BOTH operands K-contiguous:
//   SYRK   A  = X  * X^T         P = Q = X   (m x n_long)      upper-triangle tiles, mirrored store
//   SYRK2  B  = c*A*A + b*A      P = Q = A   (A symmetric)     upper-triangle tiles, mirrored store
//   BX     X' = a*X + B*X        P = B (symmetric), Q = X^T    writes X' and X'^T
// Keeping X and X^T side by side is what makes the third product K-contiguous too,
// so all three share one inner loop (replaces ns_line_1/ns_line_2 and the cuBLAS
// addmm of lit_gpt/optim/newton_schulz_triton.py:66-139, 181-266, 371-378 and the
// bf16 SYRK of emerging_optimizers/triton_kernels/syrk.py:104-185).
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

#include "ns_gemm.h"

namespace archscale {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

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

template <int BM, int BN, int WM, int WN, int MODE, bool SPLIT, bool FINAL>
__global__ void __launch_bounds__((BM / WM) * (BN / WN) * 64)
ns_gemm_kernel(const GemmParams p) {
  constexpr int NW = (BM / WM) * (BN / WN);
  constexpr int WAVES_N = BN / WN;
  constexpr int FM = WM / 32, FN = WN / 32;
  constexpr int PBYTES = BM * ROW_BYTES, QBYTES = BN * ROW_BYTES, STAGE = PBYTES + QBYTES;
  constexpr int JP = BM / 8 / NW, JQ = BN / 8 / NW;  // 8-row slabs (1 KiB) per wave
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile rows must split over waves");
  constexpr bool SYM = (MODE == MODE_SYRK || MODE == MODE_SYRK2);
  // SPLIT means "B is a hi+lo pair": SYRK2 WRITES the pair, BX READS it as a second pass over K
  constexpr bool KSPLIT = SPLIT && MODE == MODE_BX;

  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hi = lane >> 5;

  // ---- block -> (matrix, tile) : consecutive logical tiles share an XCD (and its L2)
  const int nblk = gridDim.x;  // multiple of 8
  const int per_xcd = nblk >> 3;
  const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int tiles_per_mat = SYM ? (p.tilesM * (p.tilesM + 1)) / 2 : p.tilesM * p.tilesN;
  if (logical >= p.batch * tiles_per_mat) return;
  const int b = logical / tiles_per_mat;
  int t = logical - b * tiles_per_mat;
  int ti, tj;
  if (SYM) {
    ti = 0;
    int rowlen = p.tilesM;
    while (t >= rowlen) { t -= rowlen; ++ti; --rowlen; }
    tj = ti + t;
  } else {
    tj = t / p.tilesM;
    ti = t - tj * p.tilesM;
  }
  const int R0 = ti * BM, C0 = tj * BN;

  const char* Pb = (const char*)(p.P + (size_t)b * p.strideP + (size_t)R0 * p.ldp);
  const char* P2b = KSPLIT ? (const char*)(p.P2 + (size_t)b * p.strideP + (size_t)R0 * p.ldp) : nullptr;
  const char* Qb = (const char*)(p.Q + (size_t)b * p.strideQ + (size_t)C0 * p.ldq);

  // per-lane byte offsets of the global chunks this lane copies (k-tile 0)
  uint32_t offP[JP], offQ[JQ];
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

  const int KT = p.K / BK;
  const int KT_ALL = KSPLIT ? 2 * KT : KT;

  auto issue = [&](int kt, int stage) {
    const char* pb = Pb;
    int kk = kt;
    if (KSPLIT && kt >= KT) { pb = P2b; kk = kt - KT; }
    const uint32_t koff = (uint32_t)kk * ROW_BYTES;
    char* sP = smem + stage * STAGE;
    char* sQ = sP + PBYTES;
#pragma unroll
    for (int j = 0; j < JP; ++j)
      __builtin_amdgcn_global_load_lds((gptr_t)(pb + offP[j] + koff), (lptr_t)(sP + (wave * JP + j) * 1024), 16, 0, 0);
#pragma unroll
    for (int j = 0; j < JQ; ++j)
      __builtin_amdgcn_global_load_lds((gptr_t)(Qb + offQ[j] + koff), (lptr_t)(sQ + (wave * JQ + j) * 1024), 16, 0, 0);
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
  // operand read offsets: row (w0 + i*32 + l32), chunk (2*kk + hi)
  int rdP[4], rdQ[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    rdP[kk] = lds_chunk_off(wr0 + l32, 2 * kk + hi);
    rdQ[kk] = lds_chunk_off(wc0 + l32, 2 * kk + hi);
  }

  issue(0, 0);
  for (int kt = 0; kt < KT_ALL; ++kt) {
    const int stage = kt & 1;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's copies for `stage` have landed
    __syncthreads();                             // everyone's have; everyone is done reading the other stage
    if (kt + 1 < KT_ALL) issue(kt + 1, stage ^ 1);
    const char* sP = smem + stage * STAGE;
    const char* sQ = sP + PBYTES;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      bf16x8 af[FM], bq[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) af[i] = *(const bf16x8*)(sP + rdP[kk] + i * 32 * ROW_BYTES);
#pragma unroll
      for (int j = 0; j < FN; ++j) bq[j] = *(const bf16x8*)(sQ + rdQ[kk] + j * 32 * ROW_BYTES);
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bq[j], acc[i][j], 0, 0, 0);
    }
  }

  // ---- epilogue.  acc[i][j][e] of lane l is element
  //   row = R0 + wr0 + i*32 + 8*(e/4) + 4*(l/32) + e%4,   col = C0 + wc0 + j*32 + l%32
  // so each lane owns 4 consecutive rows of one column: the TRANSPOSED image is an 8-byte store.
  const float alpha = p.alpha, beta = p.beta;
  const bool diag = SYM && (ti == tj);
#pragma unroll
  for (int i = 0; i < FM; ++i) {
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      const int col = C0 + wc0 + j * 32 + l32;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int row = R0 + wr0 + i * 32 + 8 * g + 4 * hi;
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = acc[i][j][4 * g + q];

        if (MODE == MODE_SYRK || MODE == MODE_SYRK2) {
          __bf16* C = p.C + (size_t)b * p.strideC;
          __bf16* C2 = SPLIT ? p.C2 + (size_t)b * p.strideC : nullptr;
          float lo[4];
          if (MODE == MODE_SYRK2) {
            // addend A[row+q][col] == A[col][row+q] (A is stored exactly symmetric)
            const uint2 e = *(const uint2*)(p.E + (size_t)b * p.strideE + (size_t)col * p.lde + row);
            const float a0 = bf16_to_f32(e.x & 0xffff), a1 = bf16_to_f32(e.x >> 16);
            const float a2 = bf16_to_f32(e.y & 0xffff), a3 = bf16_to_f32(e.y >> 16);
            v[0] = alpha * v[0] + beta * a0;
            v[1] = alpha * v[1] + beta * a1;
            v[2] = alpha * v[2] + beta * a2;
            v[3] = alpha * v[3] + beta * a3;
          } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] *= alpha;
          }
          if (SPLIT) {
#pragma unroll
            for (int q = 0; q < 4; ++q) lo[q] = v[q] - bf16_to_f32(bf16_bits(v[q]));
          }
          if (!diag) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              ((uint16_t*)C)[(size_t)(row + q) * p.ldc + col] = bf16_bits(v[q]);
              if (SPLIT) ((uint16_t*)C2)[(size_t)(row + q) * p.ldc + col] = bf16_bits(lo[q]);
            }
            *(uint2*)(C + (size_t)col * p.ldc + row) = pack4(v[0], v[1], v[2], v[3]);
            if (SPLIT) *(uint2*)(C2 + (size_t)col * p.ldc + row) = pack4(lo[0], lo[1], lo[2], lo[3]);
          } else {
            // diagonal tile: keep the upper half and reflect it, so the result is bit-symmetric
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              if (col >= row + q) {
                ((uint16_t*)C)[(size_t)(row + q) * p.ldc + col] = bf16_bits(v[q]);
                ((uint16_t*)C)[(size_t)col * p.ldc + row + q] = bf16_bits(v[q]);
                if (SPLIT) {
                  ((uint16_t*)C2)[(size_t)(row + q) * p.ldc + col] = bf16_bits(lo[q]);
                  ((uint16_t*)C2)[(size_t)col * p.ldc + row + q] = bf16_bits(lo[q]);
                }
              }
            }
          }
        } else {  // MODE_BX: v = acc + alpha * X[row+q][col], X[row+q][col] == Xt[col][row+q]
          const uint2 e = *(const uint2*)(p.E + (size_t)b * p.strideE + (size_t)col * p.lde + row);
          v[0] += alpha * bf16_to_f32(e.x & 0xffff);
          v[1] += alpha * bf16_to_f32(e.x >> 16);
          v[2] += alpha * bf16_to_f32(e.y & 0xffff);
          v[3] += alpha * bf16_to_f32(e.y >> 16);
          if (!FINAL) {
            if (p.C) {
              uint16_t* C = (uint16_t*)(p.C + (size_t)b * p.strideC);
#pragma unroll
              for (int q = 0; q < 4; ++q) C[(size_t)(row + q) * p.ldc + col] = bf16_bits(v[q]);
            }
            if (p.Ct) *(uint2*)(p.Ct + (size_t)b * p.strideCt + (size_t)col * p.ldct + row) = pack4(v[0], v[1], v[2], v[3]);
          } else {
            // caller's tensor: true extents, arbitrary leading dimension
            if (p.C) {
              uint16_t* C = (uint16_t*)(p.C + (size_t)b * p.strideC);
              if (col < p.n_valid) {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                  if (row + q < p.m_valid) C[(size_t)(row + q) * p.ldc + col] = bf16_bits(v[q]);
              }
            }
            if (p.Ct && col < p.n_valid) {
              __bf16* Ct = p.Ct + (size_t)b * p.strideCt + (size_t)col * p.ldct + row;
              if (row + 3 < p.m_valid && (p.ldct & 3) == 0 && (p.strideCt & 3) == 0) {
                *(uint2*)Ct = pack4(v[0], v[1], v[2], v[3]);
              } else {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                  if (row + q < p.m_valid) ((uint16_t*)Ct)[q] = bf16_bits(v[q]);
              }
            }
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// launch
// ---------------------------------------------------------------------------
template <int BM, int BN, int WM, int WN, int MODE, bool SPLIT, bool FINAL>
static hipError_t launch_one(const GemmParams& p, hipStream_t stream) {
  constexpr int NT = (BM / WM) * (BN / WN) * 64;
  constexpr int SMEM = 2 * (BM + BN) * ROW_BYTES;
  auto kern = ns_gemm_kernel<BM, BN, WM, WN, MODE, SPLIT, FINAL>;
  static bool attr_set = false;  // idempotent; a benign race only repeats the call
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  const bool sym = (MODE == MODE_SYRK || MODE == MODE_SYRK2);
  const long tiles = (long)p.batch * (sym ? (long)p.tilesM * (p.tilesM + 1) / 2 : (long)p.tilesM * p.tilesN);
  if (tiles <= 0) return hipSuccess;
  const long grid = (tiles + 7) / 8 * 8;
  if (grid > 0x7fffffffL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NT), SMEM, stream, p);
  return hipGetLastError();
}

template <int BM, int BN, int WM, int WN>
static hipError_t launch_cfg(int mode, bool split, bool final_, const GemmParams& p, hipStream_t s) {
  switch (mode) {
    case MODE_SYRK:
      return launch_one<BM, BN, WM, WN, MODE_SYRK, false, false>(p, s);
    case MODE_SYRK2:
      return split ? launch_one<BM, BN, WM, WN, MODE_SYRK2, true, false>(p, s)
                   : launch_one<BM, BN, WM, WN, MODE_SYRK2, false, false>(p, s);
    case MODE_BX:
      if (split)
        return final_ ? launch_one<BM, BN, WM, WN, MODE_BX, true, true>(p, s)
                      : launch_one<BM, BN, WM, WN, MODE_BX, true, false>(p, s);
      return final_ ? launch_one<BM, BN, WM, WN, MODE_BX, false, true>(p, s)
                    : launch_one<BM, BN, WM, WN, MODE_BX, false, false>(p, s);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_ns_gemm(int tile, int mode, bool split, bool final_, const GemmParams& p, hipStream_t stream) {
  if (p.K % BK != 0 || p.K <= 0) return hipErrorInvalidValue;
  if (tile == 256) return launch_cfg<256, 256, 128, 64>(mode, split, final_, p, stream);
  if (tile == 128) return launch_cfg<128, 128, 64, 64>(mode, split, final_, p, stream);
  return hipErrorInvalidValue;
}

}  // namespace archscale
