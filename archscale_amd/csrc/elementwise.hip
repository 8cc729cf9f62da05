// HBM-bound kernels of the Muon / MuonH step for gfx950: multi-tensor momentum,
// Frobenius norms, normalise + transpose into the padded Newton-Schulz workspace,
// and the plain-Muon / MuonH weight updates.
//
// All multi-tensor kernels are driven by a device table of items (one contiguous
// range each) and a prefix array of chunk counts: block c finds its item by binary
// search, so ONE launch covers every matrix of every shape (replaces the
// per-parameter compiled foreach graphs of lit_gpt/optim/muon.py:653-818).
// Reductions are two-stage and ordered (per-chunk partials, then one block per
// item sums them in index order), so results do not depend on scheduling.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "elementwise.h"

namespace archscale {

static constexpr int EW_THREADS = 256;
static constexpr int EW_VEC = 8;                                   // elements per thread per trip
static constexpr int EW_TRIPS = MUON_CHUNK_ELEMS / (EW_THREADS * EW_VEC);
static_assert(EW_TRIPS * EW_THREADS * EW_VEC == MUON_CHUNK_ELEMS, "chunk must be a whole number of trips");

// ---------------------------------------------------------------------------
// small helpers
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint16_t f2bf(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
__device__ __forceinline__ float bf2f(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }

// Every kernel of this file streams: an element is touched once per launch and the tensors of a step are far larger
// than the caches, so all 16-byte accesses carry the non-temporal hint (measured on a 2-read / 2-write stream of
// 1 GiB arrays: 5.87 TB/s with it, 5.57 TB/s without; a plain copy 6.29 against 5.72 TB/s).
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x4 stream_load16(const void* p) { return __builtin_nontemporal_load((const u32x4*)p); }
__device__ __forceinline__ void stream_store16(void* p, u32x4 v) { __builtin_nontemporal_store(v, (u32x4*)p); }

template <int DT> struct Elem;  // DT_BF16 / DT_F32 access of 8 consecutive elements
template <> struct Elem<DT_BF16> {
  typedef uint16_t T;
  static __device__ __forceinline__ void load8(const void* p, long i, float (&v)[8]) {
    const u32x4 r = stream_load16((const uint16_t*)p + i);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) { v[2 * k] = bf2f(w[k] & 0xffff); v[2 * k + 1] = bf2f(w[k] >> 16); }
  }
  static __device__ __forceinline__ void store8(void* p, long i, const float (&v)[8]) {
    u32x4 r;
    r.x = f2bf(v[0]) | ((uint32_t)f2bf(v[1]) << 16);
    r.y = f2bf(v[2]) | ((uint32_t)f2bf(v[3]) << 16);
    r.z = f2bf(v[4]) | ((uint32_t)f2bf(v[5]) << 16);
    r.w = f2bf(v[6]) | ((uint32_t)f2bf(v[7]) << 16);
    stream_store16((uint16_t*)p + i, r);
  }
  static __device__ __forceinline__ float load1(const void* p, long i) { return bf2f(((const uint16_t*)p)[i]); }
  static __device__ __forceinline__ void store1(void* p, long i, float v) { ((uint16_t*)p)[i] = f2bf(v); }
  static __device__ __forceinline__ float round(float v) { return bf2f(f2bf(v)); }
};
template <> struct Elem<DT_F32> {
  typedef float T;
  static __device__ __forceinline__ void load8(const void* p, long i, float (&v)[8]) {
    const f32x4 a = __builtin_nontemporal_load((const f32x4*)((const float*)p + i));
    const f32x4 b = __builtin_nontemporal_load((const f32x4*)((const float*)p + i + 4));
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  static __device__ __forceinline__ void store8(void* p, long i, const float (&v)[8]) {
    const f32x4 a = {v[0], v[1], v[2], v[3]}, b = {v[4], v[5], v[6], v[7]};
    __builtin_nontemporal_store(a, (f32x4*)((float*)p + i));
    __builtin_nontemporal_store(b, (f32x4*)((float*)p + i + 4));
  }
  static __device__ __forceinline__ float load1(const void* p, long i) { return ((const float*)p)[i]; }
  static __device__ __forceinline__ void store1(void* p, long i, float v) { ((float*)p)[i] = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};

__device__ __forceinline__ bool aligned16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

// item that owns global chunk c: largest i with prefix[i] <= c
__device__ __forceinline__ int find_item(const int32_t* __restrict__ prefix, int n_items, int c) {
  int lo = 0, hi = n_items;  // invariant: prefix[lo] <= c < prefix[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (prefix[mid] <= c) lo = mid; else hi = mid;
  }
  return lo;
}

// ordered block reduction of up to 3 values; result valid in thread 0
template <int N>
__device__ __forceinline__ void block_reduce(float (&v)[N], float* smem /* N * 4 floats */) {
#pragma unroll
  for (int k = 0; k < N; ++k) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v[k] += __shfl_down(v[k], off, 64);
  }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (lane == 0) {
#pragma unroll
    for (int k = 0; k < N; ++k) smem[k * 4 + w] = v[k];
  }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int k = 0; k < N; ++k) v[k] = (smem[k * 4 + 0] + smem[k * 4 + 1]) + (smem[k * 4 + 2] + smem[k * 4 + 3]);
  }
}

// ---------------------------------------------------------------------------
// 1. momentum:  M <- c_mm*M + c_mg*G ;  U <- c_um*M + c_ug*G   (G optionally += l2*W first)
//    lit_gpt: (mu, 1, mu|1, 1|0)  (muon.py:665-679);  emerging: (b, 1-b, b|1, 1-b|0)
//    (orthogonalized_optimizer.py:193-199, mixin.py:48-49 for the l2 term)
// ---------------------------------------------------------------------------
// SS: also accumulate the sum of squares of the update as stored (rounded to U's dtype) into `ss`
template <int GD, int MD, int UD, bool SS = false>
__device__ __forceinline__ void momentum_range(const PreItem& it, long begin, long end, const MomentumCoef c, bool vec_ok,
                                               float* ss = nullptr) {
  const void* g = it.g; void* m = it.m; void* u = it.u;
  if (vec_ok) {
    // every load of the chunk first, then the arithmetic and the stores: the stores may alias the loads as far as the
    // compiler knows, and a load that waits for the previous trip's stores leaves the memory pipeline half empty
    float gv[EW_TRIPS][8], mv[EW_TRIPS][8];
#pragma unroll
    for (int t = 0; t < EW_TRIPS; ++t) {
      const long i = begin + ((long)t * EW_THREADS + threadIdx.x) * EW_VEC;
      if (i < end) {
        Elem<GD>::load8(g, i, gv[t]);
        Elem<MD>::load8(m, i, mv[t]);
      }
    }
#pragma unroll
    for (int t = 0; t < EW_TRIPS; ++t) {
      const long i = begin + ((long)t * EW_THREADS + threadIdx.x) * EW_VEC;
      if (i < end) {
        float uv[8];
        if (c.l2 != 0.f) {
          float wv[8];
          if (it.w_dtype == DT_BF16) Elem<DT_BF16>::load8(it.w, i, wv); else Elem<DT_F32>::load8(it.w, i, wv);
#pragma unroll
          for (int k = 0; k < 8; ++k) gv[t][k] = Elem<GD>::round(gv[t][k] + c.l2 * wv[k]);
          Elem<GD>::store8(const_cast<void*>(g), i, gv[t]);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const float gm = Elem<MD>::round(gv[t][k]);            // G cast to M's dtype (muon.py:666)
          const float mn = Elem<MD>::round(fmaf(c.mm, mv[t][k], c.mg * gm));
          mv[t][k] = mn;
          uv[k] = fmaf(c.um, mn, c.ug * gm);
          if (SS) { const float x = Elem<UD>::round(uv[k]); *ss += x * x; }
        }
        Elem<MD>::store8(m, i, mv[t]);
        Elem<UD>::store8(u, i, uv);
      }
    }
  } else {
    for (long i = begin + threadIdx.x; i < end; i += EW_THREADS) {
      float gv = Elem<GD>::load1(g, i);
      if (c.l2 != 0.f) {
        const float wv = it.w_dtype == DT_BF16 ? Elem<DT_BF16>::load1(it.w, i) : Elem<DT_F32>::load1(it.w, i);
        gv = Elem<GD>::round(gv + c.l2 * wv);
        Elem<GD>::store1(const_cast<void*>(g), i, gv);
      }
      const float gm = Elem<MD>::round(gv);
      const float mn = Elem<MD>::round(fmaf(c.mm, Elem<MD>::load1(m, i), c.mg * gm));
      Elem<MD>::store1(m, i, mn);
      const float uv = fmaf(c.um, mn, c.ug * gm);
      Elem<UD>::store1(u, i, uv);
      if (SS) { const float x = Elem<UD>::round(uv); *ss += x * x; }
    }
  }
}

__global__ void __launch_bounds__(EW_THREADS)
momentum_kernel(const PreItem* __restrict__ items, const int32_t* __restrict__ prefix, int n_items, MomentumCoef c) {
  const int chunk = blockIdx.x;
  const int ii = find_item(prefix, n_items, chunk);
  const PreItem it = items[ii];
  const long begin = (long)(chunk - prefix[ii]) * MUON_CHUNK_ELEMS;
  const long end = begin + MUON_CHUNK_ELEMS < it.numel ? begin + MUON_CHUNK_ELEMS : it.numel;
  const bool vec_ok = aligned16(it.g) && aligned16(it.m) && aligned16(it.u) && (c.l2 == 0.f || aligned16(it.w)) &&
                      (it.numel % EW_VEC == 0);
  const int key = (it.g_dtype << 2) | (it.m_dtype << 1) | it.u_dtype;
  switch (key) {
    case 0: momentum_range<DT_BF16, DT_BF16, DT_BF16>(it, begin, end, c, vec_ok); break;
    case 1: momentum_range<DT_BF16, DT_BF16, DT_F32>(it, begin, end, c, vec_ok); break;
    case 2: momentum_range<DT_BF16, DT_F32, DT_BF16>(it, begin, end, c, vec_ok); break;
    case 3: momentum_range<DT_BF16, DT_F32, DT_F32>(it, begin, end, c, vec_ok); break;
    case 4: momentum_range<DT_F32, DT_BF16, DT_BF16>(it, begin, end, c, vec_ok); break;
    case 5: momentum_range<DT_F32, DT_BF16, DT_F32>(it, begin, end, c, vec_ok); break;
    case 6: momentum_range<DT_F32, DT_F32, DT_BF16>(it, begin, end, c, vec_ok); break;
    default: momentum_range<DT_F32, DT_F32, DT_F32>(it, begin, end, c, vec_ok); break;
  }
}

hipError_t launch_momentum(const PreItem* items, const int32_t* prefix, int n_items, int total_chunks,
                           MomentumCoef c, hipStream_t stream) {
  if (total_chunks <= 0) return hipSuccess;
  hipLaunchKernelGGL(momentum_kernel, dim3(total_chunks), dim3(EW_THREADS), 0, stream, items, prefix, n_items, c);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// 2. per-matrix Frobenius norm of a strided batch -> scale[b] = 1/(|X|+eps) or 1/max(|X|,eps)
//    (muon.py:883-888; F.normalize semantics for spectral_ball_utils.py:46)
// ---------------------------------------------------------------------------
template <int DT, bool CAST_FIRST>
__global__ void __launch_bounds__(EW_THREADS)
sumsq_partial_kernel(const void* __restrict__ in, long batch_stride, int rows, int cols, int ld,
                     int chunks_per_mat, float* __restrict__ partial) {
  __shared__ float red[4];
  const int b = blockIdx.y, chunk = blockIdx.x;
  const char* base = (const char*)in + (size_t)b * batch_stride * sizeof(typename Elem<DT>::T);
  const long numel = (long)rows * cols;
  const long begin = (long)chunk * MUON_CHUNK_ELEMS;
  const long end = begin + MUON_CHUNK_ELEMS < numel ? begin + MUON_CHUNK_ELEMS : numel;
  float s[1] = {0.f};
  const bool dense = (ld == cols);
  if (dense && aligned16(base) && numel % EW_VEC == 0) {
#pragma unroll
    for (int t = 0; t < EW_TRIPS; ++t) {
      const long i = begin + ((long)t * EW_THREADS + threadIdx.x) * EW_VEC;
      if (i < end) {
        float v[8];
        Elem<DT>::load8(base, i, v);
#pragma unroll
        for (int k = 0; k < 8; ++k) { const float x = CAST_FIRST ? bf2f(f2bf(v[k])) : v[k]; s[0] += x * x; }
      }
    }
  } else {
    for (long i = begin + threadIdx.x; i < end; i += EW_THREADS) {
      const long r = i / cols, cc = i - r * cols;
      float x = Elem<DT>::load1(base, r * ld + cc);
      if (CAST_FIRST) x = bf2f(f2bf(x));
      s[0] += x * x;
    }
  }
  block_reduce<1>(s, red);
  if (threadIdx.x == 0) partial[(size_t)b * chunks_per_mat + chunk] = s[0];
}

__global__ void __launch_bounds__(EW_THREADS)
norm_scale_kernel(const float* __restrict__ partial, int chunks_per_mat, float eps, int eps_mode,
                  float* __restrict__ scale, float* __restrict__ pow2) {
  __shared__ float red[4];
  const int b = blockIdx.x;
  float s[1] = {0.f};
  for (int i = threadIdx.x; i < chunks_per_mat; i += EW_THREADS) s[0] += partial[(size_t)b * chunks_per_mat + i];
  block_reduce<1>(s, red);
  if (threadIdx.x == 0) {
    const float n = sqrtf(s[0]);
    const float sc = eps_mode == EPS_ADD ? 1.f / (n + eps) : 1.f / fmaxf(n, eps);
    if (!pow2) {
      scale[b] = sc;
    } else {
      // sc = pow2 * scale with pow2 a power of two (applied to the copy of the input, exactly) and scale in [0.7, 1.5]
      const bool ok = sc > 0.f && sc < 3.0e38f;
      const float p = ok ? exp2f(rintf(log2f(sc))) : sc;
      pow2[b] = p;
      scale[b] = ok ? sc / p : 1.f;
    }
  }
}

// ---------------------------------------------------------------------------
// 3. normalise + lay out:  D[b][r][c] = bf16(s_b * in[b][r][c]) (or half(2^shift * s_b * in)),  T[b][c][r] = same value,
//    both zero-padded to the tile multiples the GEMMs assume (replaces the
//    X/(norm+eps), .mT and .contiguous() of newton_schulz_triton.py:358-366).
// ---------------------------------------------------------------------------
template <int DT, bool CAST_FIRST>
__global__ void __launch_bounds__(256)
normalize_layout_kernel(const void* __restrict__ in, const LayoutPtrs ptrs, long in_bstride, int rows, int cols, int ld,
                        const float* __restrict__ scale,
                        uint16_t* __restrict__ D, long d_bstride, int ldd, int d_rows, int d_cols,
                        uint16_t* __restrict__ T, long t_bstride, int ldt, int out_f16, int out_shift,
                        float* __restrict__ tile_sumsq) {
  // 64x64 tile; d_rows/d_cols are the padded extents (multiples of 64)
  __shared__ uint16_t tile[64][66];
  __shared__ float red[4];
  float ss[1] = {0.f};
  const int b = blockIdx.z;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  // the matrices of the batch: equally spaced from `in`, or (in == null) separate allocations listed in `ptrs`
  const char* base = in ? (const char*)in + (size_t)b * in_bstride * sizeof(typename Elem<DT>::T) : (const char*)ptrs.p[b];
  const float s = scale ? scale[b] : 1.f;
  const float fs = __builtin_ldexpf(1.f, out_shift);
  const int tr = threadIdx.x >> 3;        // 0..31
  const int tc = (threadIdx.x & 7) * 8;   // 0..56
  const bool vec = aligned16(base) && (ld % 8 == 0) && (!in || in_bstride % 8 == 0);
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int r = r0 + tr + h * 32, c = c0 + tc;
    float v[8];
    if (r < rows && c + 7 < cols && vec) {
      Elem<DT>::load8(base, (long)r * ld + c, v);
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = (r < rows && c + k < cols) ? Elem<DT>::load1(base, (long)r * ld + c + k) : 0.f;
    }
    uint16_t o[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float x = CAST_FIRST ? bf2f(f2bf(v[k])) : v[k];
      // half output: times 2^out_shift, which keeps the normalised entries in the normal range of the format
      o[k] = out_f16 ? __builtin_bit_cast(uint16_t, (_Float16)(x * s * fs)) : f2bf(x * s);
      tile[tr + h * 32][tc + k] = o[k];
      if (tile_sumsq) { const float w = out_f16 ? x * s : bf2f(o[k]); ss[0] += w * w; }
    }
    if (D && r < d_rows && c < d_cols) {
      u32x4 pk;
      pk.x = o[0] | ((uint32_t)o[1] << 16); pk.y = o[2] | ((uint32_t)o[3] << 16);
      pk.z = o[4] | ((uint32_t)o[5] << 16); pk.w = o[6] | ((uint32_t)o[7] << 16);
      stream_store16(D + (size_t)b * d_bstride + (size_t)r * ldd + c, pk);
    }
  }
  if (tile_sumsq) {   // sum of squares of what this block wrote (every block of the grid: one value per 64x64 tile)
    block_reduce<1>(ss, red);
    if (threadIdx.x == 0)
      tile_sumsq[((size_t)b * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x] = ss[0];
  }
  if (!T) return;
  __syncthreads();
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int c = c0 + tr + h * 32;  // row of T
    const int r = r0 + tc;           // 8 consecutive columns of T
    uint16_t o[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) o[k] = tile[tc + k][tr + h * 32];
    if (c < d_cols && r < d_rows) {
      u32x4 pk;
      pk.x = o[0] | ((uint32_t)o[1] << 16); pk.y = o[2] | ((uint32_t)o[3] << 16);
      pk.z = o[4] | ((uint32_t)o[5] << 16); pk.w = o[6] | ((uint32_t)o[7] << 16);
      stream_store16(T + (size_t)b * t_bstride + (size_t)c * ldt + r, pk);
    }
  }
}

hipError_t launch_norm_scale(const void* in, int in_dtype, int cast_first, long in_bstride, int ld, int batch,
                             int rows, int cols, float eps, int eps_mode, float* partial, float* scale,
                             hipStream_t stream, float* pow2) {
  const long numel = (long)rows * cols;
  const int cpm = (int)((numel + MUON_CHUNK_ELEMS - 1) / MUON_CHUNK_ELEMS);
  if (batch > 65535) return hipErrorInvalidValue;
  dim3 g1(cpm, batch);
#define ARCHSCALE_SS(DT, CF)                                                                                  \
  hipLaunchKernelGGL((sumsq_partial_kernel<DT, CF>), g1, dim3(EW_THREADS), 0, stream, in, in_bstride, rows,   \
                     cols, ld, cpm, partial)
  if (in_dtype == DT_BF16) ARCHSCALE_SS(DT_BF16, false);
  else if (cast_first) ARCHSCALE_SS(DT_F32, true);
  else ARCHSCALE_SS(DT_F32, false);
#undef ARCHSCALE_SS
  hipLaunchKernelGGL(norm_scale_kernel, dim3(batch), dim3(EW_THREADS), 0, stream, partial, cpm, eps, eps_mode,
                     scale, pow2);
  return hipGetLastError();
}

namespace {
hipError_t launch_layout_impl(const void* in, const LayoutPtrs& ptrs, int in_dtype, int cast_first, long in_bstride, int ld,
                              int batch, int rows, int cols, const float* scale, void* D, long d_bstride, int ldd,
                              int d_rows, int d_cols, void* T, long t_bstride, int ldt, hipStream_t stream, int out_f16,
                              int out_shift, float* tile_sumsq) {
  if (batch > 65535 || d_rows / 64 > 65535 || d_rows % 64 || d_cols % 64) return hipErrorInvalidValue;
  dim3 g3(d_cols / 64, d_rows / 64, batch);
#define ARCHSCALE_NL(DT, CF)                                                                                   \
  hipLaunchKernelGGL((normalize_layout_kernel<DT, CF>), g3, dim3(256), 0, stream, in, ptrs, in_bstride, rows,  \
                     cols, ld, scale, (uint16_t*)D, d_bstride, ldd, d_rows, d_cols, (uint16_t*)T, t_bstride,   \
                     ldt, out_f16, out_shift, tile_sumsq)
  if (in_dtype == DT_BF16) ARCHSCALE_NL(DT_BF16, false);
  else if (cast_first) ARCHSCALE_NL(DT_F32, true);
  else ARCHSCALE_NL(DT_F32, false);
#undef ARCHSCALE_NL
  return hipGetLastError();
}
}  // namespace

hipError_t launch_layout(const void* in, int in_dtype, int cast_first, long in_bstride, int ld, int batch, int rows,
                         int cols, const float* scale, void* D, long d_bstride, int ldd, int d_rows, int d_cols,
                         void* T, long t_bstride, int ldt, hipStream_t stream, int out_f16, int out_shift,
                         float* tile_sumsq) {
  if (!in) return hipErrorInvalidValue;
  return launch_layout_impl(in, LayoutPtrs{}, in_dtype, cast_first, in_bstride, ld, batch, rows, cols, scale, D, d_bstride,
                            ldd, d_rows, d_cols, T, t_bstride, ldt, stream, out_f16, out_shift, tile_sumsq);
}

hipError_t launch_layout_ptrs(const LayoutPtrs& ptrs, int n_mats, int in_dtype, int ld, int rows, int cols, void* D,
                              long d_bstride, int ldd, int d_rows, int d_cols, void* T, long t_bstride, int ldt,
                              hipStream_t stream, float* tile_sumsq) {
  if (n_mats < 1 || n_mats > LAYOUT_PTRS_MAX) return hipErrorInvalidValue;
  for (int i = 0; i < n_mats; ++i)
    if (!ptrs.p[i]) return hipErrorInvalidValue;
  return launch_layout_impl(nullptr, ptrs, in_dtype, 0, 0, ld, n_mats, rows, cols, nullptr, D, d_bstride, ldd, d_rows,
                            d_cols, T, t_bstride, ldt, stream, 0, 0, tile_sumsq);
}

// ---------------------------------------------------------------------------
// 3b. momentum fused with the layout pass: M <- c_mm*M + c_mg*G, U = c_um*M + c_ug*G as in momentum_kernel, but U is
//     never stored in the parameter's orientation: its bf16 rounding goes straight into the Newton-Schulz operand
//     (the matrix as it is, or its transpose, zero-padded) UNNORMALISED, with per-tile sums of squares; the
//     normalisation 1/(|U| + eps) is applied by the first iteration's GEMM epilogues.  One launch covers up to
//     MOMLAY_MAX matrices of one shape (their tensors are separate allocations: pointers by value).
// ---------------------------------------------------------------------------
// tile of one block of the transposing pass: MOMLAY_TILE x MOMLAY_TILE elements (8 elements per thread and pass), so that
// a row of it is 256 contiguous bytes in the source and in the transposed image.  Measured alternatives were 5 to 20 %
// slower: 64 x 256, 256 x 64 and 32 x 512 tiles; the loads of all eight passes before the first store; and the transposed
// store through LDS transpose reads (16-byte LDS writes, ds_read_b64_tr_b16), which leaves a wave writing 64 bytes to
// each of 16 image rows per instruction instead of 256 bytes to each of 4 (4.75 against 5.26 TB/s): the stores, not
// the 2-byte LDS accesses, are what this pass is sensitive to.
constexpr int MOMLAY_TPR = MOMLAY_TILE / 8;          // threads per tile row (8 elements each)
constexpr int MOMLAY_RPP = 256 / MOMLAY_TPR;         // tile rows per pass of the block
constexpr int MOMLAY_PASSES = MOMLAY_TILE / MOMLAY_RPP;
constexpr int MOMLAY_BATCH = 4;                      // passes whose loads are issued before any of their stores

// one matrix of a fused momentum launch, as the block sees it
struct MomMat {
  const char* g; char* m; const void* w;
  int rows, cols, transpose, ldd, w_dtype;
  uint16_t* dst;      // image of this matrix
  MomentumCoef c;
};

template <int GD, int MD>
__device__ __forceinline__ void momlay_tile(const MomMat& p, int r0, int c0,
                                            uint16_t (&tile)[MOMLAY_TILE][MOMLAY_TILE + 2], float& sumsq) {
  const char* g = p.g;
  char* m = p.m;
  const void* w = p.w;
  const int tr = threadIdx.x / MOMLAY_TPR, tc = (threadIdx.x % MOMLAY_TPR) * 8;
  const int c = c0 + tc;
  const bool vec = aligned16(g) && aligned16(m) && (p.cols % 8 == 0) && (p.c.l2 == 0.f || aligned16(w));
  const bool cols_in = vec && c + 7 < p.cols;
#pragma unroll
  for (int hb = 0; hb < MOMLAY_PASSES; hb += MOMLAY_BATCH) {
    // all loads of the batch first: the stores below may alias them as far as the compiler knows
    float gv[MOMLAY_BATCH][8], mv[MOMLAY_BATCH][8];
#pragma unroll
    for (int j = 0; j < MOMLAY_BATCH; ++j) {
      const int r = r0 + tr + (hb + j) * MOMLAY_RPP;
      if (r < p.rows && cols_in) {
        const long i = (long)r * p.cols + c;
        Elem<GD>::load8(g, i, gv[j]);
        Elem<MD>::load8(m, i, mv[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < MOMLAY_BATCH; ++j) {
      const int r = r0 + tr + (hb + j) * MOMLAY_RPP;
      float uv[8];
      if (r < p.rows && cols_in) {
        const long i = (long)r * p.cols + c;
        if (p.c.l2 != 0.f) {
          float wv[8];
          if (p.w_dtype == DT_BF16) Elem<DT_BF16>::load8(w, i, wv); else Elem<DT_F32>::load8(w, i, wv);
#pragma unroll
          for (int k = 0; k < 8; ++k) gv[j][k] = Elem<GD>::round(gv[j][k] + p.c.l2 * wv[k]);
          Elem<GD>::store8(const_cast<char*>(g), i, gv[j]);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const float gm = Elem<MD>::round(gv[j][k]);
          const float mn = Elem<MD>::round(fmaf(p.c.mm, mv[j][k], p.c.mg * gm));
          mv[j][k] = mn;
          uv[k] = fmaf(p.c.um, mn, p.c.ug * gm);
        }
        Elem<MD>::store8(m, i, mv[j]);
      } else {
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          uv[k] = 0.f;
          if (r < p.rows && c + k < p.cols) {
            const long i = (long)r * p.cols + c + k;
            float gs = Elem<GD>::load1(g, i);
            if (p.c.l2 != 0.f) {
              const float wv = p.w_dtype == DT_BF16 ? Elem<DT_BF16>::load1(w, i) : Elem<DT_F32>::load1(w, i);
              gs = Elem<GD>::round(gs + p.c.l2 * wv);
              Elem<GD>::store1(const_cast<char*>(g), i, gs);
            }
            const float gm = Elem<MD>::round(gs);
            const float mn = Elem<MD>::round(fmaf(p.c.mm, Elem<MD>::load1(m, i), p.c.mg * gm));
            Elem<MD>::store1(m, i, mn);
            uv[k] = fmaf(p.c.um, mn, p.c.ug * gm);
          }
        }
      }
      uint16_t o[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        o[k] = f2bf(uv[k]);
        const float x = bf2f(o[k]);
        sumsq += x * x;
        tile[tr + (hb + j) * MOMLAY_RPP][tc + k] = o[k];
      }
      if (!p.transpose) {
        u32x4 pk;
        pk.x = o[0] | ((uint32_t)o[1] << 16); pk.y = o[2] | ((uint32_t)o[3] << 16);
        pk.z = o[4] | ((uint32_t)o[5] << 16); pk.w = o[6] | ((uint32_t)o[7] << 16);
        stream_store16(p.dst + (size_t)r * p.ldd + c, pk);
      }
    }
  }
}

// Tile passes of up to MOMG_MAX_MATS matrices of up to MOMG_MAX_CLS shape classes in ONE launch: block b works on
// matrix i with blk_start[i] <= b < blk_start[i + 1], on tile b - blk_start[i] of it (tiles along the source columns
// first).  A class of 32 small matrices alone is a launch of 60 us, a tenth of which is ramp and drain.
__global__ void __launch_bounds__(256)
momentum_layout_kernel(const MomGroupParams p) {
  __shared__ uint16_t tile[MOMLAY_TILE][MOMLAY_TILE + 2];
  __shared__ float red[4];
  const int i = find_item(p.blk_start, p.n_mats, blockIdx.x);
  const int local = blockIdx.x - p.blk_start[i];
  const MomClass& k = p.cls[p.cls_of[i]];
  const int idx = p.idx_in_cls[i];
  const int ty = local / k.tiles_x, tx = local - ty * k.tiles_x;
  const int r0 = ty * MOMLAY_TILE, c0 = tx * MOMLAY_TILE;   // tile of the padded source orientation
  MomMat mt;
  mt.g = (const char*)p.g[i]; mt.m = (char*)p.m[i]; mt.w = p.w[i];
  mt.rows = k.rows; mt.cols = k.cols; mt.transpose = k.transpose; mt.ldd = k.ldd; mt.w_dtype = p.w_dtype;
  mt.dst = k.dst + (size_t)idx * k.d_bstride;
  mt.c = p.c;
  float s[1] = {0.f};
  const int key = (p.g_dtype << 1) | p.m_dtype;
  switch (key) {
    case 0: momlay_tile<DT_BF16, DT_BF16>(mt, r0, c0, tile, s[0]); break;
    case 1: momlay_tile<DT_BF16, DT_F32>(mt, r0, c0, tile, s[0]); break;
    case 2: momlay_tile<DT_F32, DT_BF16>(mt, r0, c0, tile, s[0]); break;
    default: momlay_tile<DT_F32, DT_F32>(mt, r0, c0, tile, s[0]); break;
  }
  __syncthreads();
  if (mt.transpose) {
    const int tr = threadIdx.x / MOMLAY_TPR, tc = (threadIdx.x % MOMLAY_TPR) * 8;
#pragma unroll
    for (int h = 0; h < MOMLAY_PASSES; ++h) {
      const int c = c0 + tr + h * MOMLAY_RPP;   // row of the transposed image
      const int r = r0 + tc;                    // 8 consecutive columns of it
      uint16_t o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = tile[tc + e][tr + h * MOMLAY_RPP];
      u32x4 pk;
      pk.x = o[0] | ((uint32_t)o[1] << 16); pk.y = o[2] | ((uint32_t)o[3] << 16);
      pk.z = o[4] | ((uint32_t)o[5] << 16); pk.w = o[6] | ((uint32_t)o[7] << 16);
      stream_store16(mt.dst + (size_t)c * mt.ldd + r, pk);
    }
  }
  block_reduce<1>(s, red);
  if (threadIdx.x == 0) k.partial[(size_t)idx * k.blocks_per_mat + local] = s[0];
}

// The same when the operand image is the matrix itself (no transposition, no padding: dst has the layout of the
// source): linear chunks of MUON_CHUNK_ELEMS like momentum_kernel, one partial sum of squares per chunk.
__global__ void __launch_bounds__(EW_THREADS)
momentum_linear_kernel(const MomGroupParams p) {
  __shared__ float red[4];
  const int i = find_item(p.blk_start, p.n_mats, blockIdx.x);
  const int chunk = blockIdx.x - p.blk_start[i];
  const MomClass& k = p.cls[p.cls_of[i]];
  const int idx = p.idx_in_cls[i];
  PreItem it;
  it.g = p.g[i]; it.m = p.m[i]; it.w = p.w[i];
  it.u = k.dst + (size_t)idx * k.d_bstride;
  it.numel = (long)k.rows * k.cols;
  it.g_dtype = p.g_dtype; it.m_dtype = p.m_dtype; it.u_dtype = DT_BF16; it.w_dtype = p.w_dtype;
  const long begin = (long)chunk * MUON_CHUNK_ELEMS;
  const long end = begin + MUON_CHUNK_ELEMS < it.numel ? begin + MUON_CHUNK_ELEMS : it.numel;
  const bool vec_ok = aligned16(it.g) && aligned16(it.m) && aligned16(it.u) && (p.c.l2 == 0.f || aligned16(it.w)) &&
                      (it.numel % EW_VEC == 0);
  float s[1] = {0.f};
  switch ((p.g_dtype << 1) | p.m_dtype) {
    case 0: momentum_range<DT_BF16, DT_BF16, DT_BF16, true>(it, begin, end, p.c, vec_ok, &s[0]); break;
    case 1: momentum_range<DT_BF16, DT_F32, DT_BF16, true>(it, begin, end, p.c, vec_ok, &s[0]); break;
    case 2: momentum_range<DT_F32, DT_BF16, DT_BF16, true>(it, begin, end, p.c, vec_ok, &s[0]); break;
    default: momentum_range<DT_F32, DT_F32, DT_BF16, true>(it, begin, end, p.c, vec_ok, &s[0]); break;
  }
  block_reduce<1>(s, red);
  if (threadIdx.x == 0) k.partial[(size_t)idx * k.blocks_per_mat + chunk] = s[0];
}

int momentum_class_blocks(const MomClass& k, int linear) {
  if (linear) return (int)(((long)k.rows * k.cols + MUON_CHUNK_ELEMS - 1) / MUON_CHUNK_ELEMS);
  return (k.d_rows / MOMLAY_TILE) * (k.d_cols / MOMLAY_TILE);
}

hipError_t launch_momentum_group(const MomGroupParams& p, hipStream_t stream) {
  if (p.n_mats < 1 || p.n_mats > MOMG_MAX_MATS || p.n_cls < 1 || p.n_cls > MOMG_MAX_CLS || p.blk_start[0] != 0)
    return hipErrorInvalidValue;
  for (int c = 0; c < p.n_cls; ++c) {
    const MomClass& k = p.cls[c];
    if (k.rows < 1 || k.cols < 1 || !k.dst || !k.partial || k.blocks_per_mat != momentum_class_blocks(k, p.linear))
      return hipErrorInvalidValue;
    if (p.linear) {
      if (k.transpose || k.d_bstride < (long)k.rows * k.cols) return hipErrorInvalidValue;
    } else if (k.d_rows % MOMLAY_TILE || k.d_cols % MOMLAY_TILE || k.rows > k.d_rows || k.cols > k.d_cols ||
               k.tiles_x != k.d_cols / MOMLAY_TILE) {
      return hipErrorInvalidValue;
    }
  }
  // every block must decode to a tile (chunk) inside its matrix
  for (int i = 0; i < p.n_mats; ++i) {
    if (p.cls_of[i] >= p.n_cls || !p.g[i] || !p.m[i] || (p.c.l2 != 0.f && !p.w[i])) return hipErrorInvalidValue;
    if (p.blk_start[i + 1] - p.blk_start[i] != p.cls[p.cls_of[i]].blocks_per_mat) return hipErrorInvalidValue;
  }
  const int blocks = p.blk_start[p.n_mats];
  if (blocks <= 0) return hipErrorInvalidValue;
  if (p.linear) hipLaunchKernelGGL(momentum_linear_kernel, dim3(blocks), dim3(EW_THREADS), 0, stream, p);
  else hipLaunchKernelGGL(momentum_layout_kernel, dim3(blocks), dim3(256), 0, stream, p);
  return hipGetLastError();
}

// scale[b] from per-tile (or per-chunk) partial sums written by another kernel
hipError_t launch_norm_scale_from_partials(const float* partial, int partials_per_mat, int batch, float eps, int eps_mode,
                                           float* scale, hipStream_t stream) {
  if (batch < 1 || partials_per_mat < 1) return hipErrorInvalidValue;
  hipLaunchKernelGGL(norm_scale_kernel, dim3(batch), dim3(EW_THREADS), 0, stream, partial, partials_per_mat, eps, eps_mode,
                     scale, (float*)nullptr);
  return hipGetLastError();
}

__global__ void __launch_bounds__(EW_THREADS)
norm_scale_groups_kernel(const NormGroupParams p, float eps, int eps_mode) {
  __shared__ float red[4];
  const int i = find_item(p.mat_start, p.n, blockIdx.x);
  const NormGroup& g = p.g[i];
  const int b = blockIdx.x - p.mat_start[i];
  float s[1] = {0.f};
  for (int t = threadIdx.x; t < g.per_mat; t += EW_THREADS) s[0] += g.partial[(size_t)b * g.per_mat + t];
  block_reduce<1>(s, red);
  if (threadIdx.x == 0) {
    const float n = sqrtf(s[0]);
    g.scale[b] = eps_mode == EPS_ADD ? 1.f / (n + eps) : 1.f / fmaxf(n, eps);
  }
}

hipError_t launch_norm_scale_groups(const NormGroupParams& p, float eps, int eps_mode, hipStream_t stream) {
  if (p.n < 1 || p.n > NORMG_MAX || p.mat_start[0] != 0) return hipErrorInvalidValue;
  for (int i = 0; i < p.n; ++i)
    if (!p.g[i].partial || !p.g[i].scale || p.g[i].per_mat < 1 || p.mat_start[i + 1] <= p.mat_start[i]) return hipErrorInvalidValue;
  hipLaunchKernelGGL(norm_scale_groups_kernel, dim3(p.mat_start[p.n]), dim3(EW_THREADS), 0, stream, p, eps, eps_mode);
  return hipGetLastError();
}

__global__ void __launch_bounds__(256) zero_i32_kernel(int* __restrict__ p, long n) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0;
}

hipError_t launch_zero_i32(int* p, long n, hipStream_t stream) {
  if (!p || n <= 0 || n > 0x7fffffffL * 256) return hipErrorInvalidValue;
  hipLaunchKernelGGL(zero_i32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, p, n);
  return hipGetLastError();
}

// strided copy of the leading rows x cols corner of a padded bf16 buffer into a caller tensor
__global__ void __launch_bounds__(256)
unpad_copy_kernel(const uint16_t* __restrict__ src, long s_bstride, int lds_, uint16_t* __restrict__ dst,
                  long d_bstride, int ldd, int rows, int cols) {
  const int b = blockIdx.z;
  const int r = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int c = blockIdx.x * 64 + (threadIdx.x & 63);
  if (r < rows && c < cols) dst[(size_t)b * d_bstride + (size_t)r * ldd + c] = src[(size_t)b * s_bstride + (size_t)r * lds_ + c];
}

hipError_t launch_unpad_copy(const void* src, long s_bstride, int lds_, void* dst, long d_bstride, int ldd,
                             int batch, int rows, int cols, hipStream_t stream) {
  if (batch > 65535 || (rows + 3) / 4 > 65535) return hipErrorInvalidValue;
  dim3 g((cols + 63) / 64, (rows + 3) / 4, batch);
  hipLaunchKernelGGL(unpad_copy_kernel, g, dim3(256), 0, stream, (const uint16_t*)src, s_bstride, lds_,
                     (uint16_t*)dst, d_bstride, ldd, rows, cols);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// 4. weight updates
//    x' = weight-decayed x (muon.py:703-718): plain x*(1-lr*wd), or cautious
//         x - lr*wd*x*[x*u >= 0]
//    plain Muon   X <- x' - lr*ratio*U                              (muon.py:720-722)
//    MuonH        X <- r*(x' - lr*s*U), s=|x'|/max(|U|,eps), r=|x'|/max(|x'-lr*s*U|,eps)
//                                                                   (muon.py:614-639, 725-818)
//    MuonH needs |x'|^2, |U|^2, <x',U> first; |x'-tU|^2 follows in closed form.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float decayed(float x, float u, float lrwd, int cautious) {
  if (cautious) return (x * u >= 0.f) ? x - lrwd * x : x;
  return x * (1.f - lrwd);
}

template <int WD>
__device__ __forceinline__ void post_reduce_range(const PostItem& it, long begin, long end, float lrwd, int cautious,
                                                  bool vec_ok, float (&s)[3]) {
  if (vec_ok) {
#pragma unroll
    for (int t = 0; t < EW_TRIPS; ++t) {
      const long i = begin + ((long)t * EW_THREADS + threadIdx.x) * EW_VEC;
      if (i < end) {
        float x[8], u[8];
        Elem<WD>::load8(it.w, i, x);
        Elem<DT_BF16>::load8(it.u, i, u);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const float xd = decayed(x[k], u[k], lrwd, cautious);
          s[0] += xd * xd; s[1] += u[k] * u[k]; s[2] += xd * u[k];
        }
      }
    }
  } else {
    for (long i = begin + threadIdx.x; i < end; i += EW_THREADS) {
      const float u = Elem<DT_BF16>::load1(it.u, i);
      const float xd = decayed(Elem<WD>::load1(it.w, i), u, lrwd, cautious);
      s[0] += xd * xd; s[1] += u * u; s[2] += xd * u;
    }
  }
}

__global__ void __launch_bounds__(EW_THREADS)
post_reduce_kernel(const PostItem* __restrict__ items, const int32_t* __restrict__ prefix, int n_items,
                   float lrwd, int cautious, float* __restrict__ partial /* [total_chunks][3] */,
                   const ScalarHyper* __restrict__ hdev) {
  __shared__ float red[12];
  if (hdev) { lrwd = hdev->lr_wd; cautious = hdev->cautious; }   // hyper-parameters from device memory
  const int chunk = blockIdx.x;
  const int ii = find_item(prefix, n_items, chunk);
  const PostItem it = items[ii];
  const long begin = (long)(chunk - prefix[ii]) * MUON_CHUNK_ELEMS;
  const long end = begin + MUON_CHUNK_ELEMS < it.numel ? begin + MUON_CHUNK_ELEMS : it.numel;
  const bool vec_ok = aligned16(it.w) && aligned16(it.u) && (it.numel % EW_VEC == 0);
  float s[3] = {0.f, 0.f, 0.f};
  if (it.w_dtype == DT_BF16) post_reduce_range<DT_BF16>(it, begin, end, lrwd, cautious, vec_ok, s);
  else post_reduce_range<DT_F32>(it, begin, end, lrwd, cautious, vec_ok, s);
  block_reduce<3>(s, red);
  if (threadIdx.x == 0) {
    partial[(size_t)chunk * 3 + 0] = s[0];
    partial[(size_t)chunk * 3 + 1] = s[1];
    partial[(size_t)chunk * 3 + 2] = s[2];
  }
}

// one block per item: (alpha, beta) with X <- alpha*x' + beta*U
__global__ void __launch_bounds__(EW_THREADS)
muonh_coef_kernel(const int32_t* __restrict__ prefix, const float* __restrict__ partial, float lr, float eps,
                  float2* __restrict__ coef, const ScalarHyper* __restrict__ hdev) {
  __shared__ double red[3][4];
  if (hdev) { lr = hdev->lr; eps = hdev->eps; }
  const int ii = blockIdx.x;
  double s[3] = {0.0, 0.0, 0.0};
  for (int c = prefix[ii] + threadIdx.x; c < prefix[ii + 1]; c += EW_THREADS) {
    s[0] += partial[(size_t)c * 3 + 0];
    s[1] += partial[(size_t)c * 3 + 1];
    s[2] += partial[(size_t)c * 3 + 2];
  }
#pragma unroll
  for (int k = 0; k < 3; ++k)
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s[k] += __shfl_down(s[k], off, 64);
  if ((threadIdx.x & 63) == 0) { red[0][threadIdx.x >> 6] = s[0]; red[1][threadIdx.x >> 6] = s[1]; red[2][threadIdx.x >> 6] = s[2]; }
  __syncthreads();
  if (threadIdx.x == 0) {
    const double xx = red[0][0] + red[0][1] + red[0][2] + red[0][3];
    const double uu = red[1][0] + red[1][1] + red[1][2] + red[1][3];
    const double xu = red[2][0] + red[2][1] + red[2][2] + red[2][3];
    const double xn = sqrt(xx), un = sqrt(uu);
    const double e = (double)eps;
    const double t = (double)lr * xn / (un > e ? un : e);            // step along U
    double yy = xx - 2.0 * t * xu + t * t * uu;                      // |x' - tU|^2
    if (yy < 0.0) yy = 0.0;
    const double yn = sqrt(yy);
    const double r = xn / (yn > e ? yn : e);
    coef[ii] = make_float2((float)r, (float)(-r * t));
  }
}

template <int WD, bool HAS_COEF>
__device__ __forceinline__ void post_apply_range(const PostItem& it, long begin, long end, float lrwd, int cautious,
                                                 bool vec_ok, float alpha, float beta) {
  if (vec_ok) {
    float x[EW_TRIPS][8], u[EW_TRIPS][8];   // all loads of the chunk before the first store (see momentum_range)
#pragma unroll
    for (int t = 0; t < EW_TRIPS; ++t) {
      const long i = begin + ((long)t * EW_THREADS + threadIdx.x) * EW_VEC;
      if (i < end) {
        Elem<WD>::load8(it.w, i, x[t]);
        Elem<DT_BF16>::load8(it.u, i, u[t]);
      }
    }
#pragma unroll
    for (int t = 0; t < EW_TRIPS; ++t) {
      const long i = begin + ((long)t * EW_THREADS + threadIdx.x) * EW_VEC;
      if (i < end) {
#pragma unroll
        for (int k = 0; k < 8; ++k) x[t][k] = alpha * decayed(x[t][k], u[t][k], lrwd, cautious) + beta * u[t][k];
        Elem<WD>::store8(it.w, i, x[t]);
      }
    }
  } else {
    for (long i = begin + threadIdx.x; i < end; i += EW_THREADS) {
      const float u = Elem<DT_BF16>::load1(it.u, i);
      Elem<WD>::store1(it.w, i, alpha * decayed(Elem<WD>::load1(it.w, i), u, lrwd, cautious) + beta * u);
    }
  }
}

__global__ void __launch_bounds__(EW_THREADS)
post_apply_kernel(const PostItem* __restrict__ items, const int32_t* __restrict__ prefix, int n_items,
                  float lr, float lrwd, int cautious, const float2* __restrict__ coef,
                  const ScalarHyper* __restrict__ hdev) {
  if (hdev) { lr = hdev->lr; lrwd = hdev->lr_wd; cautious = hdev->cautious; }
  const int chunk = blockIdx.x;
  const int ii = find_item(prefix, n_items, chunk);
  const PostItem it = items[ii];
  const long begin = (long)(chunk - prefix[ii]) * MUON_CHUNK_ELEMS;
  const long end = begin + MUON_CHUNK_ELEMS < it.numel ? begin + MUON_CHUNK_ELEMS : it.numel;
  const bool vec_ok = aligned16(it.w) && aligned16(it.u) && (it.numel % EW_VEC == 0);
  float alpha = 1.f, beta = -lr * it.lr_ratio;
  if (coef) { const float2 c = coef[ii]; alpha = c.x; beta = c.y; }
  if (it.w_dtype == DT_BF16) post_apply_range<DT_BF16, true>(it, begin, end, lrwd, cautious, vec_ok, alpha, beta);
  else post_apply_range<DT_F32, true>(it, begin, end, lrwd, cautious, vec_ok, alpha, beta);
}

hipError_t launch_post_plain(const PostItem* items, const int32_t* prefix, int n_items, int total_chunks,
                             float lr, float lrwd, int cautious, hipStream_t stream, const ScalarHyper* hdev) {
  if (total_chunks <= 0) return hipSuccess;
  hipLaunchKernelGGL(post_apply_kernel, dim3(total_chunks), dim3(EW_THREADS), 0, stream, items, prefix, n_items,
                     lr, lrwd, cautious, (const float2*)nullptr, hdev);
  return hipGetLastError();
}

hipError_t launch_post_muonh(const PostItem* items, const int32_t* prefix, int n_items, int total_chunks,
                             float lr, float lrwd, float eps, int cautious, float* scratch, hipStream_t stream,
                             const ScalarHyper* hdev) {
  if (total_chunks <= 0) return hipSuccess;
  float* partial = scratch;                                             // 3 * total_chunks
  float2* coef = (float2*)(scratch + (size_t)3 * total_chunks + ((total_chunks & 1) ? 1 : 0));  // 8-byte aligned
  hipLaunchKernelGGL(post_reduce_kernel, dim3(total_chunks), dim3(EW_THREADS), 0, stream, items, prefix, n_items,
                     lrwd, cautious, partial, hdev);
  hipLaunchKernelGGL(muonh_coef_kernel, dim3(n_items), dim3(EW_THREADS), 0, stream, prefix, partial, lr, eps, coef, hdev);
  hipLaunchKernelGGL(post_apply_kernel, dim3(total_chunks), dim3(EW_THREADS), 0, stream, items, prefix, n_items,
                     lr, lrwd, cautious, (const float2*)coef, hdev);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// 5. AdamW / hyperball-AdamW / Lion for the non-matrix parameter groups (lit_gpt/optim/scalar_opts.py:118-443)
//    phase 0: one-pass update (AdamW, Lion)
//    phase 1: hyperball pass 1 - update M, V in place, reduce |x'|^2, |U|^2, <x',U> with U = M/denom/bias1
//    phase 2: hyperball pass 2 - recompute U from the updated M, V and apply X <- alpha*x' + beta*U
// ---------------------------------------------------------------------------
__device__ __forceinline__ void load8_rt(const void* p, int dt, long i, float (&v)[8]) {
  if (dt == DT_BF16) Elem<DT_BF16>::load8(p, i, v); else Elem<DT_F32>::load8(p, i, v);
}
__device__ __forceinline__ void store8_rt(void* p, int dt, long i, const float (&v)[8]) {
  if (dt == DT_BF16) Elem<DT_BF16>::store8(p, i, v); else Elem<DT_F32>::store8(p, i, v);
}
__device__ __forceinline__ float load1_rt(const void* p, int dt, long i) {
  return dt == DT_BF16 ? Elem<DT_BF16>::load1(p, i) : Elem<DT_F32>::load1(p, i);
}
__device__ __forceinline__ void store1_rt(void* p, int dt, long i, float v) {
  if (dt == DT_BF16) Elem<DT_BF16>::store1(p, i, v); else Elem<DT_F32>::store1(p, i, v);
}
__device__ __forceinline__ float round_rt(float v, int dt) { return dt == DT_BF16 ? bf2f(f2bf(v)) : v; }

// one element; returns the new weight, updates m, v (as rounded to their dtypes), accumulates sums
template <int ALGO, int PHASE>
__device__ __forceinline__ float scalar_elem(float x, float g, float& m, float& v, const ScalarHyper& h, int m_dt,
                                             int v_dt, float alpha, float beta, float (&s)[3]) {
  float u;
  if (ALGO == ALGO_LION) {
    const float gm = round_rt(g, m_dt);
    const float t = m + h.w1 * (gm - m);                       // lerp(M, G, 1-beta1)
    u = (t > 0.f) ? 1.f : ((t < 0.f) ? -1.f : 0.f);
    m = round_rt(m + h.w2 * (gm - m), m_dt);                   // M <- lerp(M, G, 1-beta2)
    const float xd = decayed(x, u, h.lr_wd, h.cautious);
    return xd - h.lr * u;
  }
  if (PHASE != 2) {
    const float gm = round_rt(g, m_dt);
    m = round_rt(m + h.w1 * (gm - m), m_dt);                   // M <- lerp(M, G, 1-beta1)
    const float g2 = round_rt(gm * gm, v_dt);
    v = round_rt(v + h.w2 * (g2 - v), v_dt);                   // V <- lerp(V, G*G, 1-beta2)
  }
  const float dir = m / (sqrtf(v) / h.bias2_sqrt + h.eps);     // M / (sqrt(V/bias2) + eps)
  if (PHASE == 0) {
    const float xd = decayed(x, dir, h.lr_wd, h.cautious);
    return xd - (h.lr / h.bias1) * dir;
  }
  u = dir / h.bias1;
  const float xd = decayed(x, u, h.lr_wd, h.cautious);
  if (PHASE == 1) { s[0] += xd * xd; s[1] += u * u; s[2] += xd * u; return x; }
  return alpha * xd + beta * u;
}

template <int ALGO, int PHASE>
__global__ void __launch_bounds__(EW_THREADS)
scalar_update_kernel(const ScalarItem* __restrict__ items, const int32_t* __restrict__ prefix, int n_items,
                     ScalarHyper h, float* __restrict__ partial, const float2* __restrict__ coef,
                     const ScalarHyper* __restrict__ hdev) {
  __shared__ float red[12];
  if (hdev) h = *hdev;   // hyper-parameters from device memory
  const int chunk = blockIdx.x;
  const int ii = find_item(prefix, n_items, chunk);
  const ScalarItem it = items[ii];
  const long begin = (long)(chunk - prefix[ii]) * MUON_CHUNK_ELEMS;
  const long end = begin + MUON_CHUNK_ELEMS < it.numel ? begin + MUON_CHUNK_ELEMS : it.numel;
  const bool has_v = ALGO == ALGO_ADAMW;
  const bool vec_ok = aligned16(it.w) && aligned16(it.g) && aligned16(it.m) && (!has_v || aligned16(it.v)) &&
                      (it.numel % EW_VEC == 0);
  float alpha = 1.f, beta = 0.f;
  if (PHASE == 2) { const float2 c = coef[ii]; alpha = c.x; beta = c.y; }
  float s[3] = {0.f, 0.f, 0.f};
  if (vec_ok) {
    // two trips at a time: every load of the pair before its first store (the stores may alias the loads as far as
    // the compiler knows, and a load that waits for the previous trip's stores leaves the memory pipeline half empty)
    // (plain AdamW moves four arrays per element and is faster one trip at a time: 5.0 against 4.6 TB/s)
    constexpr int PAIR = (ALGO == ALGO_ADAMW && PHASE == 0) ? 1 : 2;
    static_assert(EW_TRIPS % PAIR == 0, "trips come in pairs");
#pragma unroll
    for (int t0 = 0; t0 < EW_TRIPS; t0 += PAIR) {
      float x[PAIR][8], g[PAIR][8], m[PAIR][8], v[PAIR][8];
#pragma unroll
      for (int u = 0; u < PAIR; ++u) {
        const long i = begin + ((long)(t0 + u) * EW_THREADS + threadIdx.x) * EW_VEC;
        if (i < end) {
          load8_rt(it.w, it.w_dtype, i, x[u]);
          load8_rt(it.m, it.m_dtype, i, m[u]);
          if (PHASE != 2) load8_rt(it.g, it.g_dtype, i, g[u]);
          if (has_v) load8_rt(it.v, it.v_dtype, i, v[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < PAIR; ++u) {
        const long i = begin + ((long)(t0 + u) * EW_THREADS + threadIdx.x) * EW_VEC;
        if (i < end) {
#pragma unroll
          for (int k = 0; k < 8; ++k) {
            if (PHASE == 2) g[u][k] = 0.f;
            if (!has_v) v[u][k] = 0.f;
            x[u][k] = scalar_elem<ALGO, PHASE>(x[u][k], g[u][k], m[u][k], v[u][k], h, it.m_dtype, it.v_dtype, alpha, beta, s);
          }
          if (PHASE != 1) store8_rt(it.w, it.w_dtype, i, x[u]);
          if (PHASE != 2) {
            store8_rt(it.m, it.m_dtype, i, m[u]);
            if (has_v) store8_rt(it.v, it.v_dtype, i, v[u]);
          }
        }
      }
    }
  } else {
    for (long i = begin + threadIdx.x; i < end; i += EW_THREADS) {
      float x = load1_rt(it.w, it.w_dtype, i), m = load1_rt(it.m, it.m_dtype, i);
      float g = PHASE != 2 ? load1_rt(it.g, it.g_dtype, i) : 0.f;
      float v = has_v ? load1_rt(it.v, it.v_dtype, i) : 0.f;
      x = scalar_elem<ALGO, PHASE>(x, g, m, v, h, it.m_dtype, it.v_dtype, alpha, beta, s);
      if (PHASE != 1) store1_rt(it.w, it.w_dtype, i, x);
      if (PHASE != 2) {
        store1_rt(it.m, it.m_dtype, i, m);
        if (has_v) store1_rt(it.v, it.v_dtype, i, v);
      }
    }
  }
  if (PHASE == 1) {
    block_reduce<3>(s, red);
    if (threadIdx.x == 0) {
      partial[(size_t)chunk * 3 + 0] = s[0];
      partial[(size_t)chunk * 3 + 1] = s[1];
      partial[(size_t)chunk * 3 + 2] = s[2];
    }
  }
}

hipError_t launch_scalar_update(const ScalarItem* items, const int32_t* prefix, int n_items, int total_chunks,
                                int algo, int hyperball, ScalarHyper h, float* scratch, hipStream_t stream,
                                const ScalarHyper* hdev) {
  if (total_chunks <= 0) return hipSuccess;
  dim3 grid(total_chunks), block(EW_THREADS);
  if (algo == ALGO_LION) {
    hipLaunchKernelGGL((scalar_update_kernel<ALGO_LION, 0>), grid, block, 0, stream, items, prefix, n_items, h,
                       (float*)nullptr, (const float2*)nullptr, hdev);
  } else if (!hyperball) {
    hipLaunchKernelGGL((scalar_update_kernel<ALGO_ADAMW, 0>), grid, block, 0, stream, items, prefix, n_items, h,
                       (float*)nullptr, (const float2*)nullptr, hdev);
  } else {
    float* partial = scratch;
    float2* coef = (float2*)(scratch + (size_t)3 * total_chunks + ((total_chunks & 1) ? 1 : 0));
    hipLaunchKernelGGL((scalar_update_kernel<ALGO_ADAMW, 1>), grid, block, 0, stream, items, prefix, n_items, h,
                       partial, (const float2*)nullptr, hdev);
    hipLaunchKernelGGL(muonh_coef_kernel, dim3(n_items), block, 0, stream, prefix, partial, h.lr, h.eps, coef, hdev);
    hipLaunchKernelGGL((scalar_update_kernel<ALGO_ADAMW, 2>), grid, block, 0, stream, items, prefix, n_items, h,
                       (float*)nullptr, (const float2*)coef, hdev);
  }
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// plain copy of known size: calibrates the HBM byte counters (FETCH_SIZE / WRITE_SIZE) of a profiling run
// ---------------------------------------------------------------------------
// four 16-byte loads in flight per lane before their stores, non-temporal both ways, one 16 KiB piece per block:
// the fastest of the plain copies tried on this hardware (6.29 TB/s on 1 GiB; 5.38 TB/s as a grid-stride loop of single
// accesses)
constexpr int CAL_UNROLL = 4;
__global__ void __launch_bounds__(256)
calibration_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, long n16) {
  const long stride = (long)gridDim.x * blockDim.x * CAL_UNROLL;
  for (long base = (long)blockIdx.x * CAL_UNROLL * blockDim.x + threadIdx.x; base < n16; base += stride) {
    u32x4 v[CAL_UNROLL];
#pragma unroll
    for (int u = 0; u < CAL_UNROLL; ++u) {
      const long i = base + (long)u * blockDim.x;
      if (i < n16) v[u] = stream_load16(src + i);
    }
#pragma unroll
    for (int u = 0; u < CAL_UNROLL; ++u) {
      const long i = base + (long)u * blockDim.x;
      if (i < n16) stream_store16(dst + i, v[u]);
    }
  }
}

// The same access pattern as a pure read (mode 1: the words are folded into a checksum that is written only if it
// equals a value the fill pattern never produces) and as the momentum kernel's mix of two reads and two writes
// (mode 2: b <- a + b, c <- (a + b) xor a): the rates these reach are what an HBM-bound kernel of that mix can reach.
template <int MODE>
__global__ void __launch_bounds__(256)
calibration_stream_kernel(const u32x4* __restrict__ a, u32x4* __restrict__ b, u32x4* __restrict__ c, long n16) {
  const long stride = (long)gridDim.x * blockDim.x * CAL_UNROLL;
  uint32_t fold = 0;
  for (long base = (long)blockIdx.x * CAL_UNROLL * blockDim.x + threadIdx.x; base < n16; base += stride) {
    u32x4 va[CAL_UNROLL], vb[CAL_UNROLL];
#pragma unroll
    for (int u = 0; u < CAL_UNROLL; ++u) {
      const long i = base + (long)u * blockDim.x;
      if (i < n16) {
        va[u] = stream_load16(a + i);
        if (MODE == 2) vb[u] = stream_load16(b + i);
      }
    }
#pragma unroll
    for (int u = 0; u < CAL_UNROLL; ++u) {
      const long i = base + (long)u * blockDim.x;
      if (i < n16) {
        if (MODE == 1) {
          fold ^= va[u].x ^ va[u].y ^ va[u].z ^ va[u].w;
        } else {
          const u32x4 sum = va[u] + vb[u];
          stream_store16(b + i, sum);
          stream_store16(c + i, sum ^ va[u]);
        }
      }
    }
  }
  if (MODE == 1 && fold == 0x9e3779b9u) ((uint32_t*)b)[0] = fold;
}

hipError_t launch_calibration_stream(int mode, const void* a, void* b, void* c, size_t bytes, hipStream_t stream) {
  const long n16 = (long)(bytes / 16);
  if (n16 <= 0) return hipSuccess;
  long blocks = (n16 + 256 * CAL_UNROLL - 1) / (256 * CAL_UNROLL);
  if (blocks > (1L << 20)) blocks = 1L << 20;
  if (mode == 1)
    hipLaunchKernelGGL(calibration_stream_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, stream, (const u32x4*)a, (u32x4*)b,
                       (u32x4*)c, n16);
  else if (mode == 2)
    hipLaunchKernelGGL(calibration_stream_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, stream, (const u32x4*)a, (u32x4*)b,
                       (u32x4*)c, n16);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launch_calibration_copy(const void* src, void* dst, size_t bytes, hipStream_t stream) {
  const long n16 = (long)(bytes / 16);
  if (n16 <= 0) return hipSuccess;
  long blocks = (n16 + 256 * CAL_UNROLL - 1) / (256 * CAL_UNROLL);
  if (blocks > (1L << 20)) blocks = 1L << 20;
  hipLaunchKernelGGL(calibration_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const u32x4*)src,
                     (u32x4*)dst, n16);
  return hipGetLastError();
}

}  // namespace archscale
