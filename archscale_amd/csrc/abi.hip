// extern "C" entry points declared in include/archscale_muon.h: argument checks,
// workspace carving and the launch sequence of one Newton-Schulz call.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <mutex>
#include <vector>

#include "../../include/archscale_muon.h"
#include "elementwise.h"
#include "ns_gemm.h"

using namespace archscale;

namespace {

inline long round_up(long v, long m) { return (v + m - 1) / m * m; }

// Geometry of one batched Newton-Schulz problem inside the padded workspace.
struct NsPlan {
  int tile;      // 256 or 128: square block tile of all three GEMMs
  int m, n;      // short / long side of a matrix
  int Mp, Np;    // padded to the tile
  int cpm;       // norm chunks per matrix
  size_t off_x[2], off_xt[2], off_a, off_bh, off_bl, off_partial, off_scale, total;
};

int pick_tile(int m, int n) {
  const char* env = getenv("ARCHSCALE_MUON_TILE");
  if (env) {
    const int t = atoi(env);
    if (t == 128 || t == 256) return t;
  }
  // padded work, with the small tile charged for its lower arithmetic intensity
  auto cost = [&](int t, double penalty) {
    const double Mp = (double)round_up(m, t), Np = (double)round_up(n, t);
    return Mp * Mp * (3.0 * Np + Mp) * penalty;
  };
  return cost(256, 1.0) <= cost(128, 1.25) ? 256 : 128;
}

NsPlan make_plan(int batch, int rows, int cols, int prec_mode) {
  NsPlan p;
  p.m = rows < cols ? rows : cols;
  p.n = rows < cols ? cols : rows;
  p.tile = pick_tile(p.m, p.n);
  p.Mp = (int)round_up(p.m, p.tile);
  p.Np = (int)round_up(p.n, p.tile);
  p.cpm = (int)(((long)rows * cols + MUON_CHUNK_ELEMS - 1) / MUON_CHUNK_ELEMS);
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = (size_t)round_up((long)(off + bytes), 256); return o; };
  const size_t xb = (size_t)batch * p.Mp * p.Np * 2, ab = (size_t)batch * p.Mp * p.Mp * 2;
  p.off_x[0] = take(xb); p.off_xt[0] = take(xb);
  p.off_x[1] = take(xb); p.off_xt[1] = take(xb);
  p.off_a = take(ab);
  p.off_bh = take(ab);
  p.off_bl = prec_mode == MUON_PREC_BF16_BSPLIT ? take(ab) : 0;
  p.off_partial = take((size_t)batch * p.cpm * sizeof(float));
  p.off_scale = take((size_t)batch * sizeof(float));
  p.total = off;
  return p;
}

inline long sym_tiles(int t) { return (long)t * (t + 1) / 2; }

// Optional per-launch timing of the Newton-Schulz GEMMs (muon_profile_begin / muon_profile_collect):
// one pair of HIP events around every GEMM launch, on the stream the kernel runs on.
struct ProfRec {
  hipEvent_t start, stop;
  int key;  // tile*100 + mode*10 + split*2 + final
  double flops_algorithmic, flops_issued;
};
std::mutex g_prof_mutex;
std::vector<ProfRec> g_prof;
bool g_prof_on = false;

hipError_t timed_gemm(int tile, int mode, bool split, bool final_, const GemmParams& g, hipStream_t stream,
                      double flops_algorithmic, double flops_issued) {
  if (!g_prof_on) return launch_ns_gemm(tile, mode, split, final_, g, stream);
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  ProfRec r;
  r.key = tile * 100 + mode * 10 + (split ? 2 : 0) + (final_ ? 1 : 0);
  r.flops_algorithmic = flops_algorithmic;
  r.flops_issued = flops_issued;
  hipError_t e;
  if ((e = hipEventCreate(&r.start)) != hipSuccess) return e;
  if ((e = hipEventCreate(&r.stop)) != hipSuccess) return e;
  if ((e = hipEventRecord(r.start, stream)) != hipSuccess) return e;
  e = launch_ns_gemm(tile, mode, split, final_, g, stream);
  hipError_t e2 = hipEventRecord(r.stop, stream);
  g_prof.push_back(r);
  return e != hipSuccess ? e : e2;
}

}  // namespace

extern "C" {

int muon_abi_version(void) { return MUON_ABI_VERSION; }

const char* muon_status_string(int status) {
  if (status == 0) return "success";
  if (status == MUON_E_ARG) return "invalid argument (null pointer, non-positive extent or unknown enum)";
  if (status == MUON_E_WORKSPACE) return "workspace too small or not 256-byte aligned";
  if (status == MUON_E_UNSUPPORTED) return "unsupported configuration";
  if (status > 0) return hipGetErrorString((hipError_t)status);
  return "unknown status";
}

size_t muon_ns_workspace_bytes(int batch, int rows, int cols, int prec_mode) {
  if (batch <= 0 || rows <= 0 || cols <= 0) return 0;
  return make_plan(batch, rows, cols, prec_mode).total;
}

void muon_ns_flops(int batch, int rows, int cols, int iters, int prec_mode, double* dense, double* symmetric,
                   double* issued) {
  const NsPlan p = make_plan(batch, rows, cols, prec_mode);
  const double m = p.m, n = p.n, bi = (double)batch * iters;
  if (dense) *dense = bi * (4.0 * m * m * n + 2.0 * m * m * m);
  if (symmetric) *symmetric = bi * (3.0 * m * m * n + m * m * m);
  if (issued) {
    const double t = p.tile, tm = p.Mp / p.tile, tn = p.Np / p.tile;
    const double st = (double)sym_tiles(p.Mp / p.tile);
    const double passes = prec_mode == MUON_PREC_BF16_BSPLIT ? 2.0 : 1.0;
    *issued = bi * 2.0 * t * t * (st * p.Np + st * p.Mp + tm * tn * p.Mp * passes);
  }
}

int muon_ns_batched(const void* in_dev, int in_dtype, int64_t in_batch_stride, int in_ld, void* out_dev,
                    int64_t out_batch_stride, int out_ld, int batch, int rows, int cols, const float* abc_host,
                    int iters, float eps, int eps_mode, int prec_mode, int flags, void* ws_dev, size_t ws_bytes,
                    void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!in_dev || !out_dev || !abc_host || !ws_dev) return MUON_E_ARG;
  if (batch <= 0 || rows <= 0 || cols <= 0 || iters <= 0) return MUON_E_ARG;
  if (in_ld < cols || out_ld < cols) return MUON_E_ARG;
  if (in_dtype != MUON_DTYPE_BF16 && in_dtype != MUON_DTYPE_F32) return MUON_E_ARG;
  if (eps_mode != MUON_EPS_ADD && eps_mode != MUON_EPS_CLAMP) return MUON_E_ARG;
  if (prec_mode != MUON_PREC_BF16 && prec_mode != MUON_PREC_BF16_BSPLIT) return MUON_E_ARG;
  const NsPlan pl = make_plan(batch, rows, cols, prec_mode);
  if (ws_bytes < pl.total || ((uintptr_t)ws_dev & 255)) return MUON_E_WORKSPACE;
  // byte offsets inside one matrix are 32-bit in the GEMM loader
  if ((double)pl.Mp * pl.Np * 2.0 >= 4294967296.0) return MUON_E_UNSUPPORTED;

  char* ws = (char*)ws_dev;
  __bf16* X[2] = {(__bf16*)(ws + pl.off_x[0]), (__bf16*)(ws + pl.off_x[1])};
  __bf16* Xt[2] = {(__bf16*)(ws + pl.off_xt[0]), (__bf16*)(ws + pl.off_xt[1])};
  __bf16* A = (__bf16*)(ws + pl.off_a);
  __bf16* Bh = (__bf16*)(ws + pl.off_bh);
  __bf16* Bl = prec_mode == MUON_PREC_BF16_BSPLIT ? (__bf16*)(ws + pl.off_bl) : nullptr;
  float* partial = (float*)(ws + pl.off_partial);
  float* scale = (float*)(ws + pl.off_scale);
  const bool split = Bl != nullptr;
  const bool tall = rows > cols;
  const long xs = (long)pl.Mp * pl.Np, as = (long)pl.Mp * pl.Mp;

  // normalise; the input's own orientation goes to X (wide) or X^T (tall), its transpose to the other
  const int cast_first = (flags & MUON_NS_CAST_INPUT_FIRST) ? 1 : 0;
  hipError_t e = launch_norm_scale(in_dev, in_dtype, cast_first, in_batch_stride, in_ld, batch, rows, cols, eps,
                                   eps_mode, partial, scale, stream);
  if (e != hipSuccess) return (int)e;
  if (!tall)
    e = launch_layout(in_dev, in_dtype, cast_first, in_batch_stride, in_ld, batch, rows, cols, scale, X[0], xs,
                      pl.Np, pl.Mp, pl.Np, Xt[0], xs, pl.Mp, stream);
  else
    e = launch_layout(in_dev, in_dtype, cast_first, in_batch_stride, in_ld, batch, rows, cols, scale, Xt[0], xs,
                      pl.Mp, pl.Np, pl.Mp, X[0], xs, pl.Np, stream);
  if (e != hipSuccess) return (int)e;

  const int tm = pl.Mp / pl.tile, tn = pl.Np / pl.tile;
  int cur = 0;
  for (int it = 0; it < iters; ++it) {
    const float a = abc_host[3 * it], b = abc_host[3 * it + 1], c = abc_host[3 * it + 2];
    const bool last = it == iters - 1;
    GemmParams g = {};
    g.batch = batch;
    // A = X X^T
    g.P = X[cur]; g.Q = X[cur]; g.strideP = g.strideQ = xs; g.ldp = g.ldq = pl.Np; g.K = pl.Np;
    g.tilesM = g.tilesN = tm;
    g.C = A; g.strideC = as; g.ldc = pl.Mp; g.alpha = 1.f; g.beta = 0.f;
    const double bm = (double)batch, dm = pl.m, dn = pl.n, tl = pl.tile;
    const double st = (double)sym_tiles(tm);
    if ((e = timed_gemm(pl.tile, MODE_SYRK, false, false, g, stream, bm * dm * dm * dn,
                        bm * 2.0 * tl * tl * st * pl.Np)) != hipSuccess) return (int)e;
    // B = c A A + b A
    g.P = A; g.Q = A; g.strideP = g.strideQ = as; g.ldp = g.ldq = pl.Mp; g.K = pl.Mp;
    g.E = A; g.strideE = as; g.lde = pl.Mp;
    g.C = Bh; g.C2 = Bl; g.alpha = c; g.beta = b;
    if ((e = timed_gemm(pl.tile, MODE_SYRK2, split, false, g, stream, bm * dm * dm * dm,
                        bm * 2.0 * tl * tl * st * pl.Mp)) != hipSuccess) return (int)e;
    // X' = a X + B X
    g.P = Bh; g.P2 = Bl; g.Q = Xt[cur]; g.strideP = as; g.strideQ = xs; g.ldp = pl.Mp; g.ldq = pl.Mp; g.K = pl.Mp;
    g.tilesM = tm; g.tilesN = tn;
    g.E = Xt[cur]; g.strideE = xs; g.lde = pl.Mp;
    g.alpha = a; g.beta = 0.f; g.C2 = nullptr;
    if (!last) {
      g.C = X[cur ^ 1]; g.strideC = xs; g.ldc = pl.Np;
      g.Ct = Xt[cur ^ 1]; g.strideCt = xs; g.ldct = pl.Mp;
    } else {
      g.m_valid = pl.m; g.n_valid = pl.n;
      if (!tall) { g.C = (__bf16*)out_dev; g.strideC = out_batch_stride; g.ldc = out_ld; g.Ct = nullptr; }
      else { g.C = nullptr; g.Ct = (__bf16*)out_dev; g.strideCt = out_batch_stride; g.ldct = out_ld; }
    }
    if ((e = timed_gemm(pl.tile, MODE_BX, split, last, g, stream, bm * 2.0 * dm * dm * dn,
                        bm * 2.0 * tl * tl * tm * tn * pl.Mp * (split ? 2.0 : 1.0))) != hipSuccess) return (int)e;
    cur ^= 1;
  }
  return 0;
}

size_t muon_syrk_workspace_bytes(int batch, int n, int k) {
  if (batch <= 0 || n <= 0 || k <= 0) return 0;
  const int tile = pick_tile(n, k);
  const size_t Np = (size_t)round_up(n, tile), Kp = (size_t)round_up(k, 64);
  return (size_t)round_up((long)(batch * Np * Kp * 2), 256) + 2 * (size_t)round_up((long)(batch * Np * Np * 2), 256);
}

int muon_syrk(const void* a_dev, int64_t a_batch_stride, int lda, const void* c_dev, int64_t c_batch_stride, int ldc,
              void* d_dev, int64_t d_batch_stride, int ldd, int batch, int n, int k, float alpha, float beta,
              void* ws_dev, size_t ws_bytes, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!a_dev || !d_dev || !ws_dev || batch <= 0 || n <= 0 || k <= 0 || lda < k || ldd < n) return MUON_E_ARG;
  if (c_dev && ldc < n) return MUON_E_ARG;
  if (ws_bytes < muon_syrk_workspace_bytes(batch, n, k) || ((uintptr_t)ws_dev & 255)) return MUON_E_WORKSPACE;
  const int tile = pick_tile(n, k);
  const int Np = (int)round_up(n, tile), Kp = (int)round_up(k, 64);
  if ((double)Np * Kp * 2.0 >= 4294967296.0) return MUON_E_UNSUPPORTED;
  char* ws = (char*)ws_dev;
  __bf16* Ap = (__bf16*)ws;
  __bf16* Cp = (__bf16*)(ws + round_up((long)batch * Np * Kp * 2, 256));
  __bf16* Dp = (__bf16*)((char*)Cp + round_up((long)batch * Np * Np * 2, 256));
  hipError_t e = launch_layout(a_dev, MUON_DTYPE_BF16, 0, a_batch_stride, lda, batch, n, k, nullptr, Ap,
                               (long)Np * Kp, Kp, Np, Kp, nullptr, 0, 0, stream);
  if (e != hipSuccess) return (int)e;
  if (c_dev) {
    e = launch_layout(c_dev, MUON_DTYPE_BF16, 0, c_batch_stride, ldc, batch, n, n, nullptr, Cp, (long)Np * Np, Np, Np,
                      Np, nullptr, 0, 0, stream);
    if (e != hipSuccess) return (int)e;
  }
  GemmParams g = {};
  g.batch = batch;
  g.P = Ap; g.Q = Ap; g.strideP = g.strideQ = (long)Np * Kp; g.ldp = g.ldq = Kp; g.K = Kp;
  g.tilesM = g.tilesN = Np / tile;
  g.C = Dp; g.strideC = (long)Np * Np; g.ldc = Np;
  g.alpha = alpha; g.beta = c_dev ? beta : 0.f;
  g.E = Cp; g.strideE = (long)Np * Np; g.lde = Np;
  e = launch_ns_gemm(tile, c_dev ? MODE_SYRK2 : MODE_SYRK, false, false, g, stream);
  if (e != hipSuccess) return (int)e;
  return (int)launch_unpad_copy(Dp, (long)Np * Np, Np, d_dev, d_batch_stride, ldd, batch, n, n, stream);
}

int muon_calibration_copy(const void* src_dev, void* dst_dev, size_t bytes, void* stream) {
  if (!src_dev || !dst_dev || (bytes & 15) || ((uintptr_t)src_dev & 15) || ((uintptr_t)dst_dev & 15)) return MUON_E_ARG;
  return (int)launch_calibration_copy(src_dev, dst_dev, bytes, (hipStream_t)stream);
}

int muon_profile_begin(void) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  for (auto& r : g_prof) { (void)hipEventDestroy(r.start); (void)hipEventDestroy(r.stop); }
  g_prof.clear();
  g_prof_on = true;
  return 0;
}

int muon_profile_collect(float* ms_host, int32_t* key_host, double* flops_algorithmic_host,
                         double* flops_issued_host, int capacity) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  g_prof_on = false;
  int n = 0;
  for (auto& r : g_prof) {
    float ms = 0.f;
    hipError_t e = hipEventSynchronize(r.stop);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, r.start, r.stop);
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
    if (e != hipSuccess) { g_prof.clear(); return -(int)e - 1000; }
    if (n < capacity) {
      if (ms_host) ms_host[n] = ms;
      if (key_host) key_host[n] = r.key;
      if (flops_algorithmic_host) flops_algorithmic_host[n] = r.flops_algorithmic;
      if (flops_issued_host) flops_issued_host[n] = r.flops_issued;
    }
    ++n;
  }
  g_prof.clear();
  return n;
}

int muon_momentum(const muon_pre_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                  float c_mm, float c_mg, float c_um, float c_ug, float l2, void* stream) {
  if (n_items == 0) return 0;
  if (!items_dev || !prefix_dev || n_items < 0 || total_chunks < n_items) return MUON_E_ARG;
  MomentumCoef c = {c_mm, c_mg, c_um, c_ug, l2};
  return (int)launch_momentum(items_dev, prefix_dev, n_items, total_chunks, c, (hipStream_t)stream);
}

int muon_update_plain(const muon_post_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                      float lr, float lr_wd, int cautious, void* stream) {
  if (n_items == 0) return 0;
  if (!items_dev || !prefix_dev || n_items < 0 || total_chunks < n_items) return MUON_E_ARG;
  return (int)launch_post_plain(items_dev, prefix_dev, n_items, total_chunks, lr, lr_wd, cautious,
                                (hipStream_t)stream);
}

size_t muon_muonh_scratch_floats(int n_items, int total_chunks) {
  if (n_items <= 0 || total_chunks <= 0) return 0;
  return (size_t)3 * total_chunks + 1 + (size_t)2 * n_items;
}

int muon_update_muonh(const muon_post_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                      float lr, float lr_wd, float eps, int cautious, float* scratch_dev, void* stream) {
  if (n_items == 0) return 0;
  if (!items_dev || !prefix_dev || !scratch_dev || n_items < 0 || total_chunks < n_items) return MUON_E_ARG;
  if ((uintptr_t)scratch_dev & 7) return MUON_E_WORKSPACE;
  return (int)launch_post_muonh(items_dev, prefix_dev, n_items, total_chunks, lr, lr_wd, eps, cautious, scratch_dev,
                                (hipStream_t)stream);
}

}  // extern "C"
