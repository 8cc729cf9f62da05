// Spectral-norm estimate by power iteration and the MuonBall weight update for gfx950.
//
// The reference estimates the top singular value of every weight matrix W with `steps` rounds of
//   v <- normalize(W^T (W v)),  v0 = 1,   sigma = |W v|
// (emerging_optimizers/orthogonalized_optimizers/spectral_ball_utils.py:151-166): two matrix-vector
// products over W per round, 100 passes over all weights for the default 50 rounds.  Here the Gram
// matrix of the SHORT side, G = X X^T with X = W (rows <= cols) or W^T (rows > cols), is formed once on
// the matrix cores (the SYRK kernel of the Newton-Schulz iteration), and the rounds run on G:
//   rows >  cols:  G = W^T W,  x0 = 1,      x = G^steps x0,        sigma^2 = x^T G x / x^T x
//   rows <= cols:  G = W W^T,  x0 = W 1,    x = G^(steps-1) x0,    sigma^2 = |G x|^2 / x^T G x
// which is the same vector sequence ((W^T W)^k 1 = W^T (W W^T)^(k-1) W 1) at 1/2 .. 1/11 of the memory
// traffic per round.  The normalisation between two rounds only scales the vector, so all applications but the last
// (whose Rayleigh quotient is the result, and is taken with G itself) may be grouped: with G2 = G^2 and G4 = G2^2,
// formed once by the same SYRK kernel, 50 rounds are 12 passes over G4, one over G2 or G and the final one over G
// instead of 50 or 51 passes over G.  G carries a power-of-two factor (mean eigenvalue about 1) that keeps its powers
// in the bf16 range; the result is divided by it.  A rounding error in G2 / G4 perturbs the direction only, and the quotient is
// second-order in it.  Vectors stay in fp32 (the reference rounds them to bf16 every round); every application is ONE
// launch over all matrices of all shape classes; norms are ordered two-stage reductions.
//
// The weight update fuses decoupled weight decay, retraction to the spectral sphere and the step:
//   W <- f * decay * W - lr * ratio * Phi,   f from sigma(decay * W) = decay * sigma(W)
// (muon_ball.py:60-142, spectral_ball_utils.py:168-212, orthogonalized_optimizer.py:184-228).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>

#include "spectral.h"

namespace archscale {

namespace {

__device__ __forceinline__ float bf2f_(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }
__device__ __forceinline__ uint16_t f2bf_(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return __shfl(v, 0, 64);
}

// block -> (class, matrix, 16-row strip)
__device__ __forceinline__ bool locate(const SnParams& sp, int& g, int& b, int& s) {
  const int blk = blockIdx.x;
  if (blk >= sp.blk_start[sp.n]) return false;
  g = 0;
  while (g + 1 < sp.n && blk >= sp.blk_start[g + 1]) ++g;
  const int local = blk - sp.blk_start[g];
  b = local / sp.c[g].nblk;
  s = local - b * sp.c[g].nblk;
  return true;
}

// dot products of 4 consecutive rows of a row-major bf16 matrix (leading dimension ld, a multiple of 8)
// with an fp32 vector, over n_cols columns (a multiple of 8); result broadcast to all lanes
__device__ __forceinline__ void rows4_dot(const uint16_t* __restrict__ row0, long ld, const float* __restrict__ x,
                                          int n_cols, int lane, float (&acc)[4]) {
  acc[0] = acc[1] = acc[2] = acc[3] = 0.f;
  for (int j = lane * 8; j < n_cols; j += 512) {
    float xv[8];
    if (x) {
      const float4 a = *(const float4*)(x + j), c = *(const float4*)(x + j + 4);
      xv[0] = a.x; xv[1] = a.y; xv[2] = a.z; xv[3] = a.w; xv[4] = c.x; xv[5] = c.y; xv[6] = c.z; xv[7] = c.w;
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k) xv[k] = 1.f;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint4 r = *(const uint4*)(row0 + (size_t)i * ld + j);
      const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        acc[i] += bf2f_(w[k] & 0xffff) * xv[2 * k];
        acc[i] += bf2f_(w[k] >> 16) * xv[2 * k + 1];
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = wave_sum(acc[i]);
}

// sums `n` (S, D) pairs in a fixed lane-strided order; result in all lanes
__device__ __forceinline__ void sum_pairs(const float* __restrict__ part, int n, int lane, float& S, float& D) {
  float s = 0.f, d = 0.f;
  for (int i = lane; i < n; i += 64) { s += part[2 * i]; d += part[2 * i + 1]; }
  S = wave_sum(s);
  D = wave_sum(d);
}

}  // namespace

// x0 = X 1 (row sums of the short-side-first operand) or 1;  z[0] <- x0, z[1] <- 0, part[0] <- (|x0|^2 per strip, 0)
__global__ void __launch_bounds__(256)
sn_init_kernel(const SnParams sp) {
  __shared__ float red[8];
  int g, b, s;
  if (!locate(sp, g, b, s)) return;
  const SnClass c = sp.c[g];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r0 = s * SN_ROWS + wave * 4;
  float v[4];
  if (c.tall) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = 1.f;
  } else {
    rows4_dot((const uint16_t*)c.X + (size_t)b * c.d_p * c.L_p + (size_t)r0 * c.L_p, c.L_p, nullptr, c.L_p, lane, v);
  }
  float S = 0.f;
  float* z0 = c.z + (size_t)b * c.d_p;
  float* z1 = c.z + ((size_t)c.batch + b) * c.d_p;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float val = (r0 + i < c.d) ? v[i] : 0.f;
    if (lane == 0) { z0[r0 + i] = val; z1[r0 + i] = 0.f; }
    S += val * val;
  }
  if (lane == 0) red[wave] = S;
  __syncthreads();
  if (threadIdx.x == 0) {
    float* p = c.part + ((size_t)b * c.nblk + s) * 2;
    p[0] = (red[0] + red[1]) + (red[2] + red[3]);
    p[1] = 0.f;
  }
}

// z[dst] <- M z[src] / max(|z[src]|, 1e-12);  part[dst] <- per strip (|z[dst]|^2,  z[src]^T z[dst] / |z[src]|)
// M = G, G2 or G4 (which = 0, 1, 2) and the source buffer are given per kind of class (wide, tall), whose sequences
// differ; which < 0: the classes of that kind sit this launch out.
__global__ void __launch_bounds__(256)
sn_step_kernel(const SnParams sp, int src_wide, int which_wide, int src_tall, int which_tall) {
  __shared__ float red[8];
  int g, b, s;
  if (!locate(sp, g, b, s)) return;
  const SnClass c = sp.c[g];
  const int src = c.tall ? src_tall : src_wide, which = c.tall ? which_tall : which_wide;
  if (which < 0) return;
  const __bf16* M = which == 0 ? c.G : (which == 1 ? c.G2 : c.G4);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int dst = src ^ 1;
  const float* zin = c.z + ((size_t)src * c.batch + b) * c.d_p;
  float* zout = c.z + ((size_t)dst * c.batch + b) * c.d_p;
  const float* pin = c.part + (((size_t)src * c.batch + b) * c.nblk) * 2;
  float Sin, Din;
  sum_pairs(pin, c.nblk, lane, Sin, Din);
  const float inv = 1.f / fmaxf(sqrtf(Sin), 1e-12f);
  const int r0 = s * SN_ROWS + wave * 4;
  float acc[4];
  rows4_dot((const uint16_t*)M + (size_t)b * c.d_p * c.d_p + (size_t)r0 * c.d_p, c.d_p, zin, c.d_p, lane, acc);
  float S = 0.f, D = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float out = (r0 + i < c.d) ? acc[i] * inv : 0.f;
    if (lane == 0) zout[r0 + i] = out;
    S += out * out;
    D += zin[r0 + i] * inv * out;
  }
  if (lane == 0) { red[wave] = S; red[4 + wave] = D; }
  __syncthreads();
  if (threadIdx.x == 0) {
    float* p = c.part + (((size_t)dst * c.batch + b) * c.nblk + s) * 2;
    p[0] = (red[0] + red[1]) + (red[2] + red[3]);
    p[1] = (red[4] + red[5]) + (red[6] + red[7]);
  }
}

// sigma[b] from the partials of the last round
__global__ void __launch_bounds__(64)
sn_final_kernel(const SnParams sp, int src_wide, int src_tall) {
  // one wave per matrix: blocks are numbered class by class
  int blk = blockIdx.x, g = 0;
  while (g < sp.n && blk >= sp.c[g].batch) { blk -= sp.c[g].batch; ++g; }
  if (g >= sp.n) return;
  const SnClass c = sp.c[g];
  const int src = c.tall ? src_tall : src_wide;
  const int lane = threadIdx.x;
  float S, D;
  sum_pairs(c.part + (((size_t)src * c.batch + blk) * c.nblk) * 2, c.nblk, lane, S, D);
  const float s2 = c.tall ? D : (D > 0.f ? S / D : 0.f);
  const float xs = c.xscale[blk];   // G = xs^2 X X^T
  if (lane == 0) c.sigma[blk] = xs > 0.f ? sqrtf(fmaxf(s2, 0.f)) / xs : 0.f;
}

// xscale[b]: one wave per matrix, blocks numbered class by class; the tile sums are added in a fixed order
__global__ void __launch_bounds__(64)
sn_xscale_kernel(const SnParams sp) {
  int blk = blockIdx.x, g = 0;
  while (g < sp.n && blk >= sp.c[g].batch) { blk -= sp.c[g].batch; ++g; }
  if (g >= sp.n) return;
  const SnClass c = sp.c[g];
  const float* part = c.xpart + (size_t)blk * c.xtiles;
  float t = 0.f;
  for (int i = threadIdx.x; i < c.xtiles; i += 64) t += part[i];
  t = wave_sum(t);
  // a power of two: X and G are scaled exactly
  // (exponent clamped: xscale^2 multiplies an fp32 accumulator)
  if (threadIdx.x == 0)
    c.xscale[blk] = t > 0.f ? exp2f(fminf(fmaxf(rintf(0.5f * log2f((float)c.d / t)), -60.f), 60.f)) : 0.f;
}

int spectral_power_levels(int steps) {
  // G^4 pays from about a dozen applications on (two symmetric products against 3/4 of the passes), G^2 from half of that
  return steps >= 16 ? 2 : (steps >= 6 ? 1 : 0);
}

hipError_t launch_spectral_xscale(const SnParams& sp, hipStream_t stream) {
  if (sp.n < 1 || sp.n > SN_MAX_CLASSES) return hipErrorInvalidValue;
  int matrices = 0;
  for (int g = 0; g < sp.n; ++g) {
    if (sp.c[g].batch <= 0 || !sp.c[g].xscale || !sp.c[g].xpart || sp.c[g].xtiles < 1) return hipErrorInvalidValue;
    matrices += sp.c[g].batch;
  }
  hipLaunchKernelGGL(sn_xscale_kernel, dim3(matrices), dim3(64), 0, stream, sp);
  return hipGetLastError();
}

// The vectors of a finished iteration of ONE class: short_out[b][0..d) = z_short[b] and long_out[b][0..L) = X_b^T z_prev[b]
// (X_b: d_p x L_p, zero padded; one lane owns 8 consecutive columns and walks down the rows)
__global__ void __launch_bounds__(256)
sn_vectors_kernel(const uint16_t* __restrict__ X, const float* __restrict__ z_prev, const float* __restrict__ z_short,
                  float* __restrict__ short_out, float* __restrict__ long_out, int d, int d_p, int L, int L_p) {
  const int b = blockIdx.y;
  const long t = (long)blockIdx.x * 256 + threadIdx.x;
  if (t < d) short_out[(size_t)b * d + t] = z_short[(size_t)b * d_p + t];
  const long j0 = t * 8;
  if (j0 >= L_p) return;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const uint16_t* col = X + (size_t)b * d_p * L_p + j0;
  const float* zp = z_prev + (size_t)b * d_p;
  for (int i = 0; i < d; ++i) {
    const uint4 r = *(const uint4*)(col + (size_t)i * L_p);
    const float zi = zp[i];
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      acc[2 * k] += bf2f_((uint16_t)(w[k] & 0xffff)) * zi;
      acc[2 * k + 1] += bf2f_((uint16_t)(w[k] >> 16)) * zi;
    }
  }
#pragma unroll
  for (int k = 0; k < 8; ++k)
    if (j0 + k < L) long_out[(size_t)b * L + j0 + k] = acc[k];
}

hipError_t launch_spectral_vectors(const SnClass& c, int L, int src_final, float* short_out, float* long_out,
                                   hipStream_t stream) {
  if (!short_out || !long_out || c.batch <= 0 || c.batch > 65535 || c.d <= 0 || c.d > c.d_p || L <= 0 || L > c.L_p ||
      c.L_p % 8 || (src_final != 0 && src_final != 1))
    return hipErrorInvalidValue;
  const float* z_final = c.z + (size_t)src_final * c.batch * c.d_p;
  const float* z_prev = c.z + (size_t)(src_final ^ 1) * c.batch * c.d_p;
  // wide matrices (G = W W^T): the short vector is the LAST iterate, G^steps W 1 (the reference's u); tall ones
  // (G = W^T W): the one before it, G^steps 1 (the reference's v); the long vector is X^T times the one before the last
  const float* z_short = c.tall ? z_prev : z_final;
  const long lanes = std::max((long)c.L_p / 8, (long)c.d);
  const unsigned blocks = (unsigned)((lanes + 255) / 256);
  hipLaunchKernelGGL(sn_vectors_kernel, dim3(blocks, c.batch), dim3(256), 0, stream, (const uint16_t*)c.X, z_prev, z_short,
                     short_out, long_out, c.d, c.d_p, L, c.L_p);
  return hipGetLastError();
}

hipError_t launch_spectral_iterate(const SnParams& sp, int steps, hipStream_t stream, int* final_src) {
  if (sp.n < 1 || sp.n > SN_MAX_CLASSES || steps < 1) return hipErrorInvalidValue;
  const int blocks = sp.blk_start[sp.n];
  int matrices = 0;
  bool have2 = true, have4 = true, any[2] = {false, false};
  for (int g = 0; g < sp.n; ++g) {
    const SnClass& c = sp.c[g];
    if (c.batch <= 0 || c.d <= 0 || c.d_p % 128 || c.L_p % 8 || c.d > c.d_p || c.nblk * SN_ROWS != c.d_p || !c.xscale)
      return hipErrorInvalidValue;
    matrices += c.batch;
    have2 = have2 && c.G2 != nullptr;
    have4 = have4 && c.G4 != nullptr;
    any[c.tall ? 1 : 0] = true;
  }
  if (blocks <= 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(sn_init_kernel, dim3(blocks), dim3(256), 0, stream, sp);
  // applications before the final one: `steps` for tall matrices (one more than for wide ones, see the file comment),
  // as many as possible with the highest power
  int seq[2][3];   // per kind: how many applications of G4, G2, G, in this order
  int len[2];
  for (int kind = 0; kind < 2; ++kind) {
    int n = kind ? steps : steps - 1;
    seq[kind][0] = have4 ? n / 4 : 0; n -= 4 * seq[kind][0];
    seq[kind][1] = have2 ? n / 2 : 0; n -= 2 * seq[kind][1];
    seq[kind][2] = n;
    len[kind] = any[kind] ? seq[kind][0] + seq[kind][1] + seq[kind][2] : 0;
  }
  auto which_at = [&](int kind, int i) {   // matrix of application i of a kind; -1 past its end
    if (i >= len[kind]) return -1;
    if (i < seq[kind][0]) return 2;
    if (i < seq[kind][0] + seq[kind][1]) return 1;
    return 0;
  };
  int src[2] = {0, 0};
  const int launches = len[0] > len[1] ? len[0] : len[1];
  for (int i = 0; i <= launches; ++i) {
    // the last launch is the final application of G for both kinds
    const int w0 = i == launches ? (any[0] ? 0 : -1) : which_at(0, i), w1 = i == launches ? (any[1] ? 0 : -1) : which_at(1, i);
    hipLaunchKernelGGL(sn_step_kernel, dim3(blocks), dim3(256), 0, stream, sp, src[0], w0, src[1], w1);
    if (w0 >= 0) src[0] ^= 1;
    if (w1 >= 0) src[1] ^= 1;
  }
  hipLaunchKernelGGL(sn_final_kernel, dim3(matrices), dim3(64), 0, stream, sp, src[0], src[1]);
  if (final_src) { final_src[0] = src[0]; final_src[1] = src[1]; }
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// MuonBall weight update over a table of strided 2-D blocks
// ---------------------------------------------------------------------------
namespace {

__device__ __forceinline__ int find_item_(const int32_t* __restrict__ prefix, int n_items, int c) {
  int lo = 0, hi = n_items;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (prefix[mid] <= c) lo = mid; else hi = mid;
  }
  return lo;
}

template <bool WBF16>
__device__ __forceinline__ void ball_range(const muon_ball_item& it, long begin, long end, float fw, float fp) {
  const bool vec_ok = (it.cols % 8 == 0) && (it.ld_w % 8 == 0) && (it.ld_phi % 8 == 0) &&
                      ((((uintptr_t)it.w) & (WBF16 ? 15 : 31)) == 0) && ((((uintptr_t)it.phi) & 15) == 0);
  if (vec_ok) {
    for (long i = begin + (long)threadIdx.x * 8; i < end; i += 256 * 8) {
      const long r = i / it.cols, c = i - r * it.cols;
      const uint4 pv = *(const uint4*)((const uint16_t*)it.phi + r * it.ld_phi + c);
      const uint32_t pw[4] = {pv.x, pv.y, pv.z, pv.w};
      float ph[8];
#pragma unroll
      for (int k = 0; k < 4; ++k) { ph[2 * k] = bf2f_(pw[k] & 0xffff); ph[2 * k + 1] = bf2f_(pw[k] >> 16); }
      if (WBF16) {
        uint16_t* wp = (uint16_t*)it.w + r * it.ld_w + c;
        const uint4 wv = *(const uint4*)wp;
        const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
        uint32_t o[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float a = fw * bf2f_(ww[k] & 0xffff) - fp * ph[2 * k];
          const float b = fw * bf2f_(ww[k] >> 16) - fp * ph[2 * k + 1];
          o[k] = (uint32_t)f2bf_(a) | ((uint32_t)f2bf_(b) << 16);
        }
        *(uint4*)wp = make_uint4(o[0], o[1], o[2], o[3]);
      } else {
        float* wp = (float*)it.w + r * it.ld_w + c;
        float4 a = *(const float4*)wp, b = *(const float4*)(wp + 4);
        a.x = fw * a.x - fp * ph[0]; a.y = fw * a.y - fp * ph[1]; a.z = fw * a.z - fp * ph[2]; a.w = fw * a.w - fp * ph[3];
        b.x = fw * b.x - fp * ph[4]; b.y = fw * b.y - fp * ph[5]; b.z = fw * b.z - fp * ph[6]; b.w = fw * b.w - fp * ph[7];
        *(float4*)wp = a;
        *(float4*)(wp + 4) = b;
      }
    }
  } else {
    for (long i = begin + threadIdx.x; i < end; i += 256) {
      const long r = i / it.cols, c = i - r * it.cols;
      const float ph = bf2f_(((const uint16_t*)it.phi)[r * it.ld_phi + c]);
      if (WBF16) {
        uint16_t* wp = (uint16_t*)it.w + r * it.ld_w + c;
        *wp = f2bf_(fw * bf2f_(*wp) - fp * ph);
      } else {
        float* wp = (float*)it.w + r * it.ld_w + c;
        *wp = fw * *wp - fp * ph;
      }
    }
  }
}

}  // namespace

__global__ void __launch_bounds__(256)
ball_apply_kernel(const muon_ball_item* __restrict__ items, const int32_t* __restrict__ prefix, int n_items, float lr,
                  float decay, int retract_mode, float retract_step, float* __restrict__ log_out) {
  const int chunk = blockIdx.x;
  const int ii = find_item_(prefix, n_items, chunk);
  const muon_ball_item it = items[ii];
  const long numel = (long)it.rows * it.cols;
  const long begin = (long)(chunk - prefix[ii]) * MUON_CHUNK_ELEMS;
  const long end = begin + MUON_CHUNK_ELEMS < numel ? begin + MUON_CHUNK_ELEMS : numel;
  // spectral norm of the decayed weights; retraction factor (spectral_ball_utils.py:168-212)
  const float sigma = it.sigma ? decay * *it.sigma : 0.f;
  float f, bias = 0.f;
  if (!it.sigma) {
    f = 1.f;   // a block that is not retracted
  } else if (retract_mode == MUON_RETRACT_HARD) {
    f = it.radius / (fmaxf(sigma, 0.f) + 1e-8f);
  } else {
    bias = sigma > it.radius ? -1.f : 1.f;
    f = 1.f + retract_step * bias;
  }
  if (log_out && chunk == prefix[ii] && threadIdx.x == 0) { log_out[2 * ii] = sigma; log_out[2 * ii + 1] = bias; }
  const float fw = f * decay, fp = lr * it.lr_ratio;
  if (it.w_dtype == MUON_DTYPE_BF16) ball_range<true>(it, begin, end, fw, fp);
  else ball_range<false>(it, begin, end, fw, fp);
}

hipError_t launch_ball_apply(const muon_ball_item* items, const int32_t* prefix, int n_items, int total_chunks, float lr,
                             float decay, int retract_mode, float retract_step, float* log_out, hipStream_t stream) {
  if (total_chunks <= 0) return hipSuccess;
  hipLaunchKernelGGL(ball_apply_kernel, dim3(total_chunks), dim3(256), 0, stream, items, prefix, n_items, lr, decay,
                     retract_mode, retract_step, log_out);
  return hipGetLastError();
}

}  // namespace archscale
