// extern "C" entry points declared in include/archscale_muon.h: argument checks,
// workspace carving and the launch sequence of one Newton-Schulz call.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <math.h>
#include <stdlib.h>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <vector>

#include "../../include/archscale_muon.h"
#include "elementwise.h"
#include "ns_gemm.h"
#include "spectral.h"

using namespace archscale;

namespace {

inline long round_up(long v, long m) { return (v + m - 1) / m * m; }

// Geometry of one batched Newton-Schulz problem inside the padded workspace.
struct NsPlan {
  int tile;      // 256 or 128: square block tile of all three GEMMs
  int m, n;      // short / long side of a matrix
  int Mp, Np;    // padded to the tile
  int cpm;       // norm chunks per matrix
  size_t off_xt[2], off_a, off_bh, off_bl, off_partial, off_scale, off_skpart, off_skcnt, total;
  int sk_quadrants;   // K-split: 128x128 quadrants per matrix that have partial results (0: none)
};

// The ARCHSCALE_MUON_* environment is read ONCE, when the first call needs it (debugging switches: a tile configuration
// forced for every problem, the quartered last round or the K-split switched off); later changes are not seen.
struct EnvSwitches {
  int tile;       // 0, 128 or 256
  bool quarter;
  int ksplit;     // 0: no K-split
  EnvSwitches() : tile(0), quarter(true), ksplit(1) {
    if (const char* k = getenv("ARCHSCALE_MUON_KSPLIT")) ksplit = atoi(k);   // 0: off; 2, 4, 8: that many parts wherever the rule splits
    if (const char* t = getenv("ARCHSCALE_MUON_TILE")) {
      const int v = atoi(t);
      if (v == 128 || v == 256) tile = v;
    }
    if (const char* q = getenv("ARCHSCALE_MUON_QUARTER")) quarter = atoi(q) != 0;
  }
};
const EnvSwitches& env_switches() {
  static const EnvSwitches e;
  return e;
}

int pick_tile(int m, int n) {
  if (env_switches().tile) return env_switches().tile;
  // padded work, with the small tile charged for its lower arithmetic intensity
  auto cost = [&](int t, double penalty) {
    const double Mp = (double)round_up(m, t), Np = (double)round_up(n, t);
    return Mp * Mp * (3.0 * Np + Mp) * penalty;
  };
  return cost(256, 1.0) <= cost(128, 1.25) ? 256 : 128;
}

inline long sym_tiles(int t) { return (long)t * (t + 1) / 2; }

// K-split of a symmetric product of ONE matrix, a pure function of the matrix's own shape (so a matrix takes the same
// path, and gives the same bits, alone and in any batch).  With tm = tiles of 256 along the short side and KT k-tiles of
// 64: the first `full` = floor(T / 256) * 256 upper-triangle tiles (whole rounds of the chip when the matrix is alone)
// run as they are; the remaining `rem` run as 128x128 quadrants, `parts` blocks per quadrant, each walking KT / parts
// k-tiles.  Only long reductions (KT >= 128, i.e. K >= 8192) of matrices with at least 16 tiles left over are split: the
// partial results cost 64 KiB of traffic per block each way, which a block of 32 or more k-tiles hides, and a batch of
// many small matrices (whose launches are full anyway) must not pay for it.  Measured on single matrices (us per
// product, 2 / 4 / 8 parts against none): the 136 tiles of a 4096 x 14336 matrix 330 / 315 / 366 against 378, the 16 tiles
// left over by an 8192 x 8192 matrix 55 / 40 / 43 against 83; a batch of eight 8192 x 8192 matrices, which needs no split,
// pays 1.5 % of its time for the partial results.
struct SkRule { int full, rem, parts; };
constexpr int SK_PARTS = 4, SK_MIN_KT = 128, SK_MIN_REM = 16;
SkRule sk_rule(int tm, int KT) {
  const int T = (int)sym_tiles(tm);
  SkRule r = {T, 0, 1};
  const int full = T / 256 * 256, rem = T - full;
  // (a tile configuration forced through the environment, a debugging switch, also switches the split off)
  if (env_switches().ksplit == 0 || env_switches().tile != 0 || KT < SK_MIN_KT || rem < SK_MIN_REM) return r;
  int parts = SK_PARTS;
  if (env_switches().ksplit > 1 && KT / env_switches().ksplit >= 16) parts = env_switches().ksplit;   // (experiments)
  return SkRule{full, rem, parts};
}
// the two reduction lengths of a matrix's symmetric products: the long side (A = X X^T) and the short side (the m x m products)
struct SkShape { SkRule long_k, short_k; bool any; };
SkShape sk_shape(int m, int n) {
  const int tm = (int)(round_up(m, 256) / 256);
  SkShape s;
  s.long_k = sk_rule(tm, (int)(round_up(n, 256) / 64));
  s.short_k = sk_rule(tm, (int)(round_up(m, 256) / 64));
  s.any = s.long_k.rem > 0 || s.short_k.rem > 0;
  return s;
}

NsPlan make_plan(int batch, int rows, int cols, int prec_mode, int tile = 0) {
  NsPlan p;
  p.m = rows < cols ? rows : cols;
  p.n = rows < cols ? cols : rows;
  p.tile = tile ? tile : pick_tile(p.m, p.n);
  const SkShape sk = sk_shape(p.m, p.n);
  // a shape with a K-split is enumerated in tiles of 256 whatever the configuration of the call
  const int pad = sk.any ? 256 : p.tile;
  p.Mp = (int)round_up(p.m, pad);
  p.Np = (int)round_up(p.n, pad);
  p.cpm = (int)(((long)rows * cols + MUON_CHUNK_ELEMS - 1) / MUON_CHUNK_ELEMS);
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = (size_t)round_up((long)(off + bytes), 256); return o; };
  // a class whose long side is at least twice the short one may finish on the Gram side (see ns_grouped_impl): the idle
  // X^T buffer then holds two more m x m matrices per matrix
  const size_t ab = (size_t)batch * p.Mp * p.Mp * 2;
  const size_t xb = std::max((size_t)batch * p.Mp * p.Np * 2, p.n >= 2 * p.m ? 2 * ab : (size_t)0);
  p.off_xt[0] = take(xb);
  p.off_xt[1] = take(xb);
  p.off_a = take(ab);
  p.off_bh = take(ab);
  p.off_bl = prec_mode == MUON_PREC_BF16_BSPLIT ? take(ab) : 0;
  // norm partials: one per 8192-element chunk (separate norm pass) or one per tile of the fused momentum pass (at most one per 64x64 elements)
  const size_t tiles64 = (size_t)(p.Mp / 64) * (p.Np / 64);
  p.off_partial = take((size_t)batch * std::max((size_t)p.cpm, tiles64) * sizeof(float));
  p.off_scale = take((size_t)2 * batch * sizeof(float));   // deferred factor and the power of two applied to the copy
  // K-split: fp32 partial results ([matrix][quadrant][part]) and one counter per quadrant
  p.sk_quadrants = 4 * std::max(sk.long_k.rem, sk.short_k.rem);
  const int parts = std::max(sk.long_k.rem ? sk.long_k.parts : 0, sk.short_k.rem ? sk.short_k.parts : 0);
  p.off_skpart = take((size_t)batch * p.sk_quadrants * parts * SK_TILE_BYTES);
  p.off_skcnt = take((size_t)batch * p.sk_quadrants * sizeof(int));
  p.total = off;
  return p;
}
// matrix-core work of the upper-triangle tiles, in tiles: a diagonal tile runs three quarters of its MFMAs (the waves
// whose sub-tiles lie wholly below the diagonal sit out)
inline double sym_tiles_issued(int t) { return (double)sym_tiles(t) - 0.25 * t; }

// workspace bound of one problem: the larger of the two tile configurations (a call with few tiles in total takes the
// small one, see ns_grouped_impl)
size_t plan_bytes_bound(int batch, int rows, int cols, int prec_mode) {
  if (env_switches().tile) return make_plan(batch, rows, cols, prec_mode).total;
  return std::max(make_plan(batch, rows, cols, prec_mode, 256).total, make_plan(batch, rows, cols, prec_mode, 128).total);
}

constexpr int MAX_DEVICES = 64;

// compute units of the CURRENT device (cached per device; a racing first call only repeats the query)
int compute_units() {
  static std::atomic<int> cached[MAX_DEVICES];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  const bool slot = dev >= 0 && dev < MAX_DEVICES;
  int v = slot ? cached[dev].load(std::memory_order_relaxed) : 0;
  if (v > 0) return v;
  if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) return 256;
  if (slot) cached[dev].store(v, std::memory_order_relaxed);
  return v;
}

// Optional per-launch timing (muon_profile_begin / muon_profile_collect): one pair of HIP events around every
// Newton-Schulz GEMM launch and every fused momentum launch, on the stream the kernel runs on.  The events come from a
// pool that muon_profile_begin creates, so a timed call creates nothing; launches beyond the pool run untimed.
// Profiling is a single-threaded debugging mode: every timed launch takes one process-wide lock.
struct ProfRec {
  int key;  // tile*100 + mode*10 + 4*(BX without addend) + split*2 + final; PROF_KEY_MOMENTUM_LAYOUT for the fused momentum
  double work_algorithmic, work_issued;   // FLOPs of a GEMM launch; bytes of a momentum launch
};
constexpr int PROF_POOL = 1024;
constexpr int PROF_KEY_MOMENTUM_LAYOUT = 90000;
std::mutex g_prof_mutex;
std::vector<hipEvent_t> g_prof_start, g_prof_stop;   // the pool
std::vector<ProfRec> g_prof;                         // g_prof[i] used events i
std::atomic<bool> g_prof_on{false};

// runs `launch` between two pooled events when profiling is on
template <class F>
hipError_t timed_launch(int key, double work_algorithmic, double work_issued, hipStream_t stream, F&& launch) {
  if (!g_prof_on.load(std::memory_order_acquire)) return launch();
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  const size_t i = g_prof.size();
  if (!g_prof_on || i >= g_prof_start.size()) return launch();
  hipError_t e = hipEventRecord(g_prof_start[i], stream);
  if (e != hipSuccess) return e;
  e = launch();
  const hipError_t e2 = hipEventRecord(g_prof_stop[i], stream);
  g_prof.push_back(ProfRec{key, work_algorithmic, work_issued});
  return e != hipSuccess ? e : e2;
}

hipError_t timed_gemm(int tile, int mode, bool split, bool final_, const GroupedGemmParams& g, hipStream_t stream,
                      double flops_algorithmic, double flops_issued, int f16 = 0) {
  const int key = tile * 100 + mode * 10 + ((mode == MODE_BX && !g.g[0].E) ? 4 : 0) + (split ? 2 : 0) + (final_ ? 1 : 0);
  return timed_launch(key, flops_algorithmic, flops_issued, stream,
                      [&] { return launch_ns_gemm_grouped(tile, mode, split, final_, g, stream, f16); });
}

// One product over all problems of a 256-tile launch.  When the last round of the grid would hold only a few tiles, the
// full rounds run as they are and the tiles of the last round are handed, as four 128x128 quadrants each, to the small
// configuration: a quarter of the time per block instead of a whole round for a few tiles.  The small configuration
// runs at about half the rate of the large one, so this pays for at most QUARTER_MAX_TAIL tiles (measured: a tail of
// 160 tiles on the depth-16 set costs 83 us quartered against 57 us as it is; tails of 16 and 128 tiles of single
// 8192x8192 and 4096x14336 matrices: 10.33 -> 9.80 ms and 4.58 -> 4.44 ms per call); a launch smaller than one round
// is quartered as a whole up to QUARTER_MAX_ALONE tiles.  ARCHSCALE_MUON_QUARTER=0 switches it off.
constexpr int QUARTER_MAX_TAIL = 128, QUARTER_MAX_ALONE = 176;
hipError_t launch_rounds(int tile, int mode, bool split, bool final_, const GroupedGemmParams& gp, hipStream_t stream,
                         double fa, double fi, int f16) {
  const bool enabled = env_switches().quarter;
  const int total = gp.tile_start[gp.n_groups];
  const int round = 256;
  const int full = total / round * round, tail = total - full;
  if (!enabled || tile != 256 || tail == 0 || tail > (full > 0 ? QUARTER_MAX_TAIL : QUARTER_MAX_ALONE))
    return timed_gemm(tile, mode, split, final_, gp, stream, fa, fi, f16);
  const double share = (double)full / total;
  if (full > 0) {
    GroupedGemmParams m = gp;
    for (int i = 0; i <= gp.n_groups; ++i) m.tile_start[i] = std::min(gp.tile_start[i], full);
    hipError_t e = timed_gemm(tile, mode, split, final_, m, stream, fa * share, fi * share, f16);
    if (e != hipSuccess) return e;
  }
  GroupedGemmParams q = {};
  q.quarter = 1;
  for (int i = 0; i < gp.n_groups; ++i) {
    const int s = gp.tile_start[i], e = gp.tile_start[i + 1];
    const int f = std::max(s, full);
    if (e <= f) continue;
    GemmParams g = gp.g[i];
    g.tilesM *= 2;
    g.tilesN *= 2;
    g.qt_first = f - s;
    q.g[q.n_groups] = g;
    q.tile_start[q.n_groups + 1] = q.tile_start[q.n_groups] + 4 * (e - f);
    ++q.n_groups;
  }
  return timed_gemm(128, mode, split, final_, q, stream, fa * (1.0 - share), fi * (1.0 - share), f16);
}

}  // namespace

// Scratch of muon_ns_batched_static: a device array that exists from the moment the code object is loaded, so that entry
// point allocates nothing.  In host code this NAME is only a handle for hipGetSymbolAddress; kernels and copies get the
// device address that the lookup returns (one per device: every GPU holds its own copy of the array).
static __device__ __align__(256) unsigned char scratch[MUON_NS_STATIC_SCRATCH_BYTES];

namespace {
// per device: the array's address, and what orders calls that come in on different streams (the event marks the end
// of the last call's work; a call on another stream waits for it on the device, so two streams that share the array
// take turns instead of racing).  Created once per device, on the first call.
struct StaticScratch {
  void* ptr = nullptr;
  hipEvent_t done = nullptr;
  hipStream_t last = nullptr;
  bool has_last = false;
};
std::mutex g_scratch_mutex;   // held while a call on the array is being enqueued
StaticScratch g_scratch[MAX_DEVICES];

// the array of the CURRENT device (address looked up once per device); the caller holds g_scratch_mutex
int static_scratch(StaticScratch** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= MAX_DEVICES) return MUON_E_UNSUPPORTED;
  StaticScratch& st = g_scratch[dev];
  if (!st.ptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr || ((uintptr_t)ptr & 255)) return MUON_E_WORKSPACE;
    hipEvent_t ev = nullptr;
    e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
    if (e != hipSuccess) return (int)e;
    st.done = ev;
    st.ptr = ptr;
  }
  *out = &st;
  return 0;
}
}  // namespace

extern "C" {

int muon_abi_version(void) { return MUON_ABI_VERSION; }

const char* muon_status_string(int status) {
  if (status == 0) return "success";
  if (status == MUON_E_ARG) return "invalid argument (null pointer, non-positive extent or unknown enum)";
  if (status == MUON_E_WORKSPACE) return "workspace too small or not 256-byte aligned";
  if (status == MUON_E_UNSUPPORTED) return "unsupported configuration";
  if (status == MUON_E_STATIC_LIMIT)
    return "the problem needs more than MUON_NS_STATIC_SCRATCH_BYTES of workspace; call muon_ns_batched with a workspace of muon_ns_workspace_bytes()";
  if (status > 0) return hipGetErrorString((hipError_t)status);
  return "unknown status";
}

size_t muon_ns_workspace_bytes(int batch, int rows, int cols, int prec_mode) {
  if (batch <= 0 || rows <= 0 || cols <= 0) return 0;
  return plan_bytes_bound(batch, rows, cols, prec_mode);
}

void muon_ns_flops(int batch, int rows, int cols, int iters, int prec_mode, double* dense, double* symmetric,
                   double* issued) {
  const NsPlan p = make_plan(batch, rows, cols, prec_mode);
  const double m = p.m, n = p.n, bi = (double)batch * iters;
  if (dense) *dense = bi * (4.0 * m * m * n + 2.0 * m * m * m);
  if (symmetric) *symmetric = bi * (3.0 * m * m * n + m * m * m);
  if (issued) {
    const double t = p.tile, tm = p.Mp / p.tile, tn = p.Np / p.tile;
    const double st = sym_tiles_issued(p.Mp / p.tile);
    const double passes = prec_mode == MUON_PREC_BF16_BSPLIT ? 2.0 : 1.0;
    *issued = bi * 2.0 * t * t * (st * p.Np + st * p.Mp + tm * tn * p.Mp * passes);
  }
}

void muon_ns_ksplit_info(int rows, int cols, int* info) {
  if (!info) return;
  for (int i = 0; i < 6; ++i) info[i] = 0;
  if (rows <= 0 || cols <= 0) return;
  const SkShape s = sk_shape(rows < cols ? rows : cols, rows < cols ? cols : rows);
  info[0] = s.long_k.full; info[1] = s.long_k.rem; info[2] = s.long_k.parts;
  info[3] = s.short_k.full; info[4] = s.short_k.rem; info[5] = s.short_k.parts;
}

// plan + carved workspace pointers of one problem of a grouped call
namespace {
struct NsProblem {
  muon_ns_problem q;
  NsPlan pl;
  __bf16 *Xt[2], *A, *Bh, *Bl;   // Xt: the iterate as X^T, [b][Np][Mp] (long side first), ping-pong
  float *partial, *scale, *pow2;
  float* sk_partial;   // K-split: partial results and counters (null when the shape has none)
  int* sk_counter;
  bool tall;
  bool gram_tail;   // the last two iterations run on the Gram side (n >= 2m): one B X product instead of two
  bool defer;   // the operand of the first iteration is the input as it is; its epilogues apply 1/(|X| + eps)
  int sx;   // half-precision mode: the iterate is kept times 2^sx (its rms entry starts at about 2^-3)
};

int check_problem(const muon_ns_problem& q, bool no_input = false) {
  if ((!q.in && !no_input) || !q.out) return MUON_E_ARG;
  if (q.batch <= 0 || q.rows <= 0 || q.cols <= 0) return MUON_E_ARG;
  if (q.in_ld < q.cols || q.out_ld < q.cols) return MUON_E_ARG;
  if (q.in_dtype != MUON_DTYPE_BF16 && q.in_dtype != MUON_DTYPE_F32) return MUON_E_ARG;
  return 0;
}
}  // namespace

size_t muon_ns_grouped_workspace_bytes(const muon_ns_problem* problems_host, int n_problems, int prec_mode) {
  if (!problems_host || n_problems <= 0) return 0;
  size_t total = 0;
  for (int i = 0; i < n_problems; ++i) {
    const muon_ns_problem& q = problems_host[i];
    if (q.batch <= 0 || q.rows <= 0 || q.cols <= 0) return 0;
    total += plan_bytes_bound(q.batch, q.rows, q.cols, prec_mode);
  }
  return total;
}

namespace {
// The grouped Newton-Schulz call.  With `fused` (one entry per problem) the operand is not read from problems[i].in:
// the momentum update of the matrices listed there produces it (unnormalised; the first iteration's epilogues apply
// the scale), see momentum_layout_kernel.
int ns_grouped_impl(const muon_ns_problem* problems_host, const muon_mns_problem* fused, MomentumCoef mc, int n_problems,
                    const float* abc_host, int iters, float eps, int eps_mode, int prec_mode, int flags, void* ws_dev,
                    size_t ws_bytes, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!problems_host || n_problems <= 0 || !abc_host || !ws_dev || iters <= 0) return MUON_E_ARG;
  if (eps_mode != MUON_EPS_ADD && eps_mode != MUON_EPS_CLAMP) return MUON_E_ARG;
  if (prec_mode != MUON_PREC_BF16 && prec_mode != MUON_PREC_BF16_BSPLIT && prec_mode != MUON_PREC_F16) return MUON_E_ARG;
  const bool f16 = prec_mode == MUON_PREC_F16;
  // power-of-two factors of the half-precision workspace: A is kept times 2^SA, B times 2^SB, X times 2^sx (per problem)
  const int SA = f16 ? 8 : 0, SB = f16 ? 6 : 0;
  if ((uintptr_t)ws_dev & 255) return MUON_E_WORKSPACE;
  const bool split_any = prec_mode == MUON_PREC_BF16_BSPLIT;
  const int split_tail = (flags >> 8) & 0xff;   // 0: every iteration keeps B as a hi+lo pair; t: only the last t
  if (flags & ~(MUON_NS_CAST_INPUT_FIRST | MUON_NS_NO_NORMALIZE | MUON_NS_NO_DIAG_FOLD | MUON_NS_NO_GRAM_TAIL |
                MUON_NS_GRAM_TAIL | 0xff00))
    return MUON_E_ARG;
  if ((flags & MUON_NS_NO_GRAM_TAIL) && (flags & MUON_NS_GRAM_TAIL)) return MUON_E_ARG;
  const bool normalize = !(flags & MUON_NS_NO_NORMALIZE);
  if (!normalize && fused) return MUON_E_ARG;
  bool split = split_any;
  const int cast_first = (flags & MUON_NS_CAST_INPUT_FIRST) ? 1 : 0;

  std::vector<NsProblem> pr(n_problems);
  size_t off = 0;
  // A call whose smallest launch (the symmetric products) would not even occupy half of the compute units with 256x256
  // tiles takes the 128x128 configuration for every problem: four times the blocks, a quarter of the time per block.
  long sym_blocks = 0;
  for (int i = 0; i < n_problems; ++i) {
    const muon_ns_problem& q = problems_host[i];
    if (q.batch <= 0 || q.rows <= 0 || q.cols <= 0) return MUON_E_ARG;
    const NsPlan pl = make_plan(q.batch, q.rows, q.cols, prec_mode);
    sym_blocks += (long)q.batch * sym_tiles(pl.Mp / pl.tile);
  }
  const int force_tile = (!env_switches().tile && sym_blocks * 2 < compute_units()) ? 128 : 0;
  for (int i = 0; i < n_problems; ++i) {
    NsProblem& P = pr[i];
    P.q = problems_host[i];
    const int st = check_problem(P.q, fused != nullptr);
    if (st) return st;
    P.pl = make_plan(P.q.batch, P.q.rows, P.q.cols, prec_mode, force_tile);
    // byte offsets inside one matrix are 32-bit in the GEMM loader
    if ((double)P.pl.Mp * P.pl.Np * 2.0 >= 4294967296.0) return MUON_E_UNSUPPORTED;
    if (off + P.pl.total > ws_bytes) return MUON_E_WORKSPACE;
    char* ws = (char*)ws_dev + off;
    off += P.pl.total;
    P.Xt[0] = (__bf16*)(ws + P.pl.off_xt[0]); P.Xt[1] = (__bf16*)(ws + P.pl.off_xt[1]);
    P.A = (__bf16*)(ws + P.pl.off_a);
    P.Bh = (__bf16*)(ws + P.pl.off_bh);
    P.Bl = split_any ? (__bf16*)(ws + P.pl.off_bl) : nullptr;
    P.partial = (float*)(ws + P.pl.off_partial);
    P.scale = (float*)(ws + P.pl.off_scale);
    P.pow2 = P.scale + P.q.batch;
    P.sk_partial = P.pl.sk_quadrants ? (float*)(ws + P.pl.off_skpart) : nullptr;
    P.sk_counter = P.pl.sk_quadrants ? (int*)(ws + P.pl.off_skcnt) : nullptr;
    // a square matrix counts as tall: orthogonalising X^T and transposing the result is the same map, and a tall
    // matrix enters the workspace as it is (a linear pass instead of a tile transpose)
    P.tall = P.q.rows >= P.q.cols;
    // An input that is bfloat16 already (or is rounded to it before its norm) goes into the workspace EXACTLY and the
    // factor is applied by the first iteration's epilogues, as after the fused momentum (all but a power of two, which
    // the copy takes exactly and which keeps the products of the first iteration in range): rounding the normalised copy a
    // second time is what a matrix with a few dominant singular values is sensitive to (Gaussian plus a 30x rank-one
    // spike, error against an fp32 run: 5.2e-2 -> 5.0e-3 in bfloat16, 6.7e-3 -> 1.8e-3 with the half workspace).
    P.defer = fused || (normalize && (P.q.in_dtype == MUON_DTYPE_BF16 || cast_first));
    const int l2 = (int)floor(0.5 * log2((double)P.pl.m * (double)P.pl.n)) - 3;
    P.sx = l2 > 0 ? l2 : 0;   // used by the iterations that keep the iterate in half
    P.gram_tail = false;
  }
  // the half workspace starts with a bfloat16 iteration when the scale is deferred (see the iteration below); one
  // kernel type per launch, so either every problem of the call defers or none does
  bool defer_all = true;
  for (const NsProblem& P : pr) defer_all = defer_all && P.defer;
  if (f16 && !defer_all)
    for (NsProblem& P : pr) P.defer = false;
  // launch order inside a grouped kernel: problems with the longest tiles first, so the tail of the
  // grid is made of short tiles
  std::vector<int> order(n_problems);
  for (int i = 0; i < n_problems; ++i) order[i] = i;
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) {
    return (long)pr[a].pl.Mp * pr[a].pl.Np > (long)pr[b].pl.Mp * pr[b].pl.Np;
  });

  hipError_t e;
  // K-split counters start at zero (every launch leaves them at zero again); the workspace is the caller's and holds anything
  for (const NsProblem& P : pr)
    if (P.sk_counter && (e = launch_zero_i32(P.sk_counter, (long)P.q.batch * P.pl.sk_quadrants, stream)) != hipSuccess) return (int)e;
  // normalise into X^T (long side first): a wide input is transposed on the way, a tall one is copied as it is
  for (int i = 0; i < n_problems && !fused; ++i) {
    const NsProblem& P = pr[i];
    const NsPlan& pl = P.pl;
    const long xs = (long)pl.Mp * pl.Np;
    const float* sc = !normalize ? nullptr : (P.defer ? P.pow2 : P.scale);   // null: copy unscaled
    const int to_half = (f16 && !P.defer) ? 1 : 0;
    if (normalize) {
      e = launch_norm_scale(P.q.in, P.q.in_dtype, cast_first, P.q.in_batch_stride, P.q.in_ld, P.q.batch, P.q.rows,
                            P.q.cols, eps, eps_mode, P.partial, P.scale, stream, P.defer ? P.pow2 : nullptr);
      if (e != hipSuccess) return (int)e;
    }
    if (!P.tall)
      e = launch_layout(P.q.in, P.q.in_dtype, cast_first, P.q.in_batch_stride, P.q.in_ld, P.q.batch, P.q.rows,
                        P.q.cols, sc, nullptr, 0, 0, pl.Mp, pl.Np, P.Xt[0], xs, pl.Mp, stream, to_half, to_half ? P.sx : 0);
    else
      e = launch_layout(P.q.in, P.q.in_dtype, cast_first, P.q.in_batch_stride, P.q.in_ld, P.q.batch, P.q.rows,
                        P.q.cols, sc, P.Xt[0], xs, pl.Mp, pl.Np, pl.Mp, nullptr, 0, 0, stream, to_half, to_half ? P.sx : 0);
    if (e != hipSuccess) return (int)e;
  }
  // fused staging: momentum of every matrix, its bf16 update written unnormalised into X^T, norms from tile partials.
  // The matrices of ALL problems share launches (up to MOMG_MAX_MATS matrices of MOMG_MAX_CLS classes each): one
  // sequence of launches for the matrices that take the linear pass, one for those that take the tile pass.
  if (fused) {
    std::vector<int> blocks_per_mat(n_problems);
    for (int pass = 0; pass < 2; ++pass) {   // 0: linear pass, 1: tile pass (transposition and / or padding)
      MomGroupParams mp = {};
      double bytes = 0.0;
      auto flush = [&]() -> hipError_t {
        if (mp.n_mats == 0) return hipSuccess;
        const double b = bytes;
        hipError_t err = timed_launch(PROF_KEY_MOMENTUM_LAYOUT, b, b, stream, [&] { return launch_momentum_group(mp, stream); });
        mp = MomGroupParams{};
        bytes = 0.0;
        return err;
      };
      for (int i = 0; i < n_problems; ++i) {
        const NsProblem& P = pr[i];
        const NsPlan& pl = P.pl;
        const muon_mns_problem& f = fused[i];
        // a tall matrix whose extents need no padding goes into the workspace as it is: a linear pass, partials per chunk
        const bool linear = P.tall && P.q.rows == pl.Np && P.q.cols == pl.Mp;
        if (linear != (pass == 0)) continue;
        MomClass k = {};
        k.rows = P.q.rows; k.cols = P.q.cols;
        k.transpose = P.tall ? 0 : 1;
        k.d_rows = P.tall ? pl.Np : pl.Mp; k.d_cols = P.tall ? pl.Mp : pl.Np;   // padded extents of the matrix itself
        k.ldd = pl.Mp; k.d_bstride = (long)pl.Mp * pl.Np;
        k.tiles_x = k.d_cols / MOMLAY_TILE;
        k.blocks_per_mat = momentum_class_blocks(k, linear ? 1 : 0);
        k.dst = (uint16_t*)P.Xt[0];
        k.partial = P.partial;
        blocks_per_mat[i] = k.blocks_per_mat;
        int cls = -1;
        for (int b = 0; b < P.q.batch; ++b) {
          const bool dtypes_differ = mp.n_mats > 0 && (mp.g_dtype != f.g_dtype || mp.m_dtype != f.m_dtype || mp.w_dtype != f.w_dtype);
          if (mp.n_mats == MOMG_MAX_MATS || dtypes_differ || (cls < 0 && mp.n_cls == MOMG_MAX_CLS) ||
              (long)mp.blk_start[mp.n_mats] + k.blocks_per_mat > 0x7ffffff0L) {
            if ((e = flush()) != hipSuccess) return (int)e;
            cls = -1;
          }
          if (mp.n_mats == 0) {
            mp.linear = linear ? 1 : 0;
            mp.g_dtype = f.g_dtype; mp.m_dtype = f.m_dtype; mp.w_dtype = f.w_dtype;
            mp.c = mc;
          }
          if (cls < 0) {
            cls = mp.n_cls++;
            mp.cls[cls] = k;
          }
          const int j = mp.n_mats++;
          mp.cls_of[j] = (uint8_t)cls;
          mp.idx_in_cls[j] = b;
          mp.blk_start[j + 1] = mp.blk_start[j] + k.blocks_per_mat;
          mp.g[j] = f.g_ptrs[b];
          mp.m[j] = f.m_ptrs[b];
          mp.w[j] = f.w_ptrs ? f.w_ptrs[b] : nullptr;
          // algorithmic bytes: G read, M read and written, the operand image written (2 bytes each)
          bytes += (double)P.q.rows * P.q.cols *
                   ((f.g_dtype == MUON_DTYPE_F32 ? 4 : 2) + 2 * (f.m_dtype == MUON_DTYPE_F32 ? 4 : 2) + 2);
        }
      }
      if ((e = flush()) != hipSuccess) return (int)e;
    }
    // 1 / (|U| + eps) of every matrix of every problem from the partial sums: one launch per NORMG_MAX problems
    NormGroupParams ng = {};
    for (int i = 0; i <= n_problems; ++i) {
      if (i == n_problems || ng.n == NORMG_MAX) {
        if (ng.n > 0 && (e = launch_norm_scale_groups(ng, eps, eps_mode, stream)) != hipSuccess) return (int)e;
        ng = NormGroupParams{};
        if (i == n_problems) break;
      }
      NormGroup& g = ng.g[ng.n];
      g.partial = pr[i].partial; g.per_mat = blocks_per_mat[i]; g.scale = pr[i].scale;
      ng.mat_start[ng.n + 1] = ng.mat_start[ng.n] + pr[i].q.batch;
      ++ng.n;
    }
  }

  // one product of the iteration for every problem that `fill` accepts: problems that share a tile configuration go
  // into one launch (at most MAX_GROUPS per launch)
  auto run_mode = [&](int mode, bool split_launch, bool final_, int ws16, auto&& fill) -> hipError_t {
    const bool sym = mode != MODE_BX;
    // tiles of symmetric products that take a K-split (see sk_rule), of every problem: one launch of its own
    GroupedGemmParams sk = {};
    sk.quarter = 1;
    double sk_fa = 0.0, sk_fi = 0.0;
    auto flush_sk = [&]() -> hipError_t {
      if (sk.n_groups == 0) return hipSuccess;
      const int key = 128 * 100 + mode * 10;
      const GroupedGemmParams launch = sk;
      hipError_t err = timed_launch(key, sk_fa, sk_fi, stream, [&] {
        return launch_ns_gemm_grouped(128, mode, false, false, launch, stream, ws16, true);
      });
      sk = GroupedGemmParams{};
      sk.quarter = 1;
      sk_fa = sk_fi = 0.0;
      return err;
    };
    for (int tile : {256, 128}) {
      GroupedGemmParams gp = {};
      double fa = 0.0, fi = 0.0;
      auto flush = [&]() -> hipError_t {
        if (gp.n_groups == 0) return hipSuccess;
        hipError_t err = launch_rounds(tile, mode, split_launch, final_, gp, stream, fa, fi, ws16);
        gp = GroupedGemmParams{};
        fa = fi = 0.0;
        return err;
      };
      for (int oi = 0; oi < n_problems; ++oi) {
        const NsProblem& P = pr[order[oi]];
        if (P.pl.tile != tile) continue;
        GemmParams g = {};
        double a_fl = 0.0, i_fl = 0.0;
        if (!fill(P, g, a_fl, i_fl)) continue;
        long tiles = ns_gemm_tiles(mode, g);
        if (sym && P.pl.sk_quadrants > 0 && !split_launch) {
          // the shape has a K-split for some reduction length: this product's own rule, in tiles of 256
          const SkRule r = sk_rule(P.pl.Mp / 256, g.K / 64);
          if (r.rem > 0) {
            GemmParams q = g;
            q.tilesM = q.tilesN = P.pl.Mp / 128;          // quarter mode counts the fine tiles
            q.qt_first = 0;
            q.t_first = r.full; q.t_count = r.rem;
            q.ksplit = r.parts;
            q.sk_partial = P.sk_partial; q.sk_counter = P.sk_counter;
            const long blocks = 4L * g.batch * r.rem * r.parts;
            if (blocks + sk.tile_start[sk.n_groups] > 0x7ffffff0L || sk.n_groups == MAX_GROUPS) {
              hipError_t err = flush_sk();
              if (err != hipSuccess) return err;
            }
            if (blocks > 0x7ffffff0L) return hipErrorInvalidValue;
            sk.g[sk.n_groups] = q;
            sk.tile_start[sk.n_groups + 1] = sk.tile_start[sk.n_groups] + (int)blocks;
            ++sk.n_groups;
            const double share = (double)r.rem / (r.full + r.rem);
            sk_fa += a_fl * share; sk_fi += i_fl * share;
            a_fl *= 1.0 - share; i_fl *= 1.0 - share;
            if (r.full == 0) continue;
            // the whole rounds run as they are; a forced small configuration never gets here (it has fewer than 128 tiles)
            if (tile != 256) return hipErrorInvalidValue;
            g.t_first = 0; g.t_count = r.full;
            tiles = (long)g.batch * r.full;
          }
        }
        if (tiles + gp.tile_start[gp.n_groups] > 0x7ffffff0L || gp.n_groups == MAX_GROUPS) {
          hipError_t err = flush();
          if (err != hipSuccess) return err;
        }
        if (tiles > 0x7ffffff0L) return hipErrorInvalidValue;
        gp.g[gp.n_groups] = g;
        gp.tile_start[gp.n_groups + 1] = gp.tile_start[gp.n_groups] + (int)tiles;
        ++gp.n_groups;
        fa += a_fl;
        fi += i_fl;
      }
      hipError_t err = flush();
      if (err != hipSuccess) return err;
    }
    return flush_sk();
  };

  // ---- storage of the iteration's matrices, per iteration.  MUON_PREC_F16: half from the first iteration on, or from
  // the second one when the scale is deferred - the unnormalised operand cannot go into half as it is (its magnitude is
  // the gradient's), so the first iteration then runs on it in bfloat16 with the deferred scale and its last product
  // writes X' as scaled half; the operand of that iteration is the exact bfloat16 update, and A and B of ONE early
  // iteration in bfloat16 cost nothing measurable (error against an fp32 run, CPU model, 512x2048 / 1024x1024 / 64x129:
  // constant row 2.15 / 2.01 / 2.27e-3 against 2.16 / 2.03 / 2.22e-3 with all five in half; a second bfloat16 iteration
  // would cost 3.3 / 3.7 / 9.2e-3).
  // MUON_PREC_BF16 with at least three iterations: the LAST TWO iterations run in half as well ("tail").  Their
  // matrices are bounded whatever the input was, the rounding of the last iterations dominates the error of the result
  // (CPU model, quintic schedule, error against an fp64 run: Gaussian 4.5e-3 -> 3.3e-3, 300x rank-one spike
  // 1.9e-2 -> 1.6e-2), and half is what makes the Gram-side tail below as accurate as the iteration on X.
  auto fold_ok = [&](int it) {
    return !(flags & MUON_NS_NO_DIAG_FOLD) && it > 0 && fabsf(abc_host[3 * it]) <= 4.2f;
  };
  // (an input that is not normalised is not bounded: no half storage that the caller did not ask for)
  // On by default under MUON_PREC_BF16, where it lowers the error on every spectrum tried; under MUON_PREC_F16 it costs
  // 1-2 % of accuracy (polar-express msign table, whose spectrum is not settled two iterations before the end:
  // 1.9e-3 -> 2.4e-3), so there the caller has to ask for it.
  const bool tail_wanted = (flags & MUON_NS_NO_GRAM_TAIL) ? false : ((flags & MUON_NS_GRAM_TAIL) ? true : !f16);
  // (half storage holds B + aI times 2^6: with |A| <= 1.5 after the normalisation that is in range for any table whose
  // last two rows keep 1.5 |b| + 2.25 |c| + |a| under 500 - every table of the reference is under 25; a custom table beyond
  // that keeps its last iterations in bfloat16)
  auto half_range_ok = [&](int it) {
    return 1.5f * fabsf(abc_host[3 * it + 1]) + 2.25f * fabsf(abc_host[3 * it + 2]) + fabsf(abc_host[3 * it]) <= 500.f;
  };
  const bool tail = tail_wanted && normalize && !split_any && iters >= 3 && fold_ok(iters - 2) && fold_ok(iters - 1) &&
                    half_range_ok(iters - 2) && half_range_ok(iters - 1);
  const int first_half_it = f16 ? (defer_all ? 1 : 0) : (tail ? iters - 2 : iters);
  // ---- Gram-side tail.  With P_k = a_k I + b_k A_k + c_k A_k^2 (symmetric, a polynomial in A_k = X_k X_k^T, so all of
  // them commute) the last two iterations are  X_N = P_N P_{N-1} X_{N-2}  with  A_{N-1} = P_{N-1} A_{N-2} P_{N-1}:
  // three more m x m symmetric products (T = P A, A' = T P, Q = P' P) replace one B X and one X X^T product, which
  // saves 3 m^2 (n - m) multiply-adds per matrix - 11 % of a 2048 x 5632 matrix's iteration.  Taken for the classes
  // with n >= 2m.  Only the LAST two iterations: earlier, the spectrum still spans orders of magnitude and squaring it
  // pushes the small singular values under the rounding of the Gram matrix (CPU model, fusing three iterations:
  // log-spaced spectrum 3e-2 -> 1.6e-1).  With the tail in half the result is as close to an fp64 run as the iteration
  // on X (Gaussian 3.26e-3 / 3.28e-3, 300x spike 1.62e-2 / 1.62e-2, log-spaced spectrum 3.00e-2 / 3.01e-2, low rank
  // plus noise 4.54e-2 / 4.54e-2 without / with it; MUON_PREC_F16: 1.74 / 1.77e-3, 3.9 / 4.0e-3, 4.2 / 4.5e-3, 7.2 / 7.3e-3).
  bool any_tail = false, all_tail = true;
  for (NsProblem& P : pr) {
    P.gram_tail = tail && P.pl.n >= 2 * P.pl.m;
    any_tail = any_tail || P.gram_tail;
    all_tail = all_tail && P.gram_tail;
  }
  const int SH_A = 8, SH_B = 6;   // powers of two carried by A and by B, T, Q in half storage

  struct ItCfg { float a, b, c; bool last, half_ops, half_out, fold, split; int SAi, SBi, ws16, bx16; };
  auto it_cfg = [&](int it) {
    ItCfg k;
    k.a = abc_host[3 * it]; k.b = abc_host[3 * it + 1]; k.c = abc_host[3 * it + 2];
    k.last = it == iters - 1;
    k.half_ops = it >= first_half_it;
    k.half_out = !k.last && it + 1 >= first_half_it;
    k.split = split_any && (split_tail == 0 || it >= iters - split_tail);
    // a*I folded into B (diagonal entries of B + aI are rounded like any other entry): X' = (B + aI) X needs no addend.
    // Not for a large `a` (first row of the polar-express table), whose rounding on the diagonal would show, and not in
    // the first iteration: a matrix with a few dominant singular values has a tiny A after the normalisation, and
    // B_ii would vanish below half an ulp of `a`.  With the hi+lo pair the folded diagonal is exact; an iteration of a
    // split call that keeps B in plain bf16 is not folded (constant coefficients on small matrices: 8.4e-3 -> 1.1e-2
    // for 64x129 when it is).
    k.fold = fold_ok(it) && (!split_any || k.split);
    k.SAi = k.half_ops ? SH_A : 0;
    k.SBi = k.half_ops ? SH_B : 0;
    k.ws16 = k.half_ops ? 1 : 0;
    k.bx16 = k.half_ops ? 1 : (k.half_out ? 2 : 0);   // 2: bfloat16 operands, the next iterate in half
    return k;
  };
  // A = X X^T of the iterate in Xt[src], from X^T (K-major operand)
  auto syrkt = [&](int it, int src, auto&& want) -> hipError_t {
    const ItCfg k = it_cfg(it);
    return run_mode(MODE_SYRKT, false, false, k.ws16, [&](const NsProblem& P, GemmParams& g, double& fa, double& fi) {
      if (!want(P)) return false;
      const NsPlan& pl = P.pl;
      const long xs = (long)pl.Mp * pl.Np, as = (long)pl.Mp * pl.Mp;
      g.batch = P.q.batch;
      g.P = P.Xt[src]; g.Q = P.Xt[src]; g.strideP = g.strideQ = xs; g.ldp = g.ldq = pl.Mp; g.K = pl.Np;
      g.tilesM = g.tilesN = pl.Mp / pl.tile;
      g.C = P.A; g.strideC = as; g.ldc = pl.Mp; g.alpha = ldexpf(1.f, k.SAi - 2 * (k.half_ops ? P.sx : 0)); g.beta = 0.f;
      g.scale = (P.defer && it == 0) ? P.scale : nullptr;
      const double bm = P.q.batch, dm = pl.m, dn = pl.n, tl = pl.tile;
      fa = bm * dm * dm * dn;
      fi = bm * 2.0 * tl * tl * sym_tiles_issued(pl.Mp / pl.tile) * pl.Np;
      return true;
    });
  };
  // B = c A A + b A (+ a I) into dst(P) (and the low half of the pair into P.Bl)
  auto syrk2 = [&](int it, auto&& want, auto&& dst) -> hipError_t {
    const ItCfg k = it_cfg(it);
    return run_mode(MODE_SYRK2, k.split, false, k.ws16, [&](const NsProblem& P, GemmParams& g, double& fa, double& fi) {
      if (!want(P)) return false;
      const NsPlan& pl = P.pl;
      const long as = (long)pl.Mp * pl.Mp;
      g.batch = P.q.batch;
      g.P = P.A; g.Q = P.A; g.strideP = g.strideQ = as; g.ldp = g.ldq = pl.Mp; g.K = pl.Mp;
      g.tilesM = g.tilesN = pl.Mp / pl.tile;
      g.E = P.A; g.strideE = as; g.lde = pl.Mp;
      g.C = dst(P); g.C2 = P.Bl; g.strideC = as; g.ldc = pl.Mp;
      g.alpha = ldexpf(k.c, k.SBi - 2 * k.SAi); g.beta = ldexpf(k.b, k.SBi - k.SAi);
      g.diag_add = k.fold ? ldexpf(k.a, k.SBi) : 0.f;
      const double bm = P.q.batch, dm = pl.m, tl = pl.tile;
      fa = bm * dm * dm * dm;
      fi = bm * 2.0 * tl * tl * sym_tiles_issued(pl.Mp / pl.tile) * pl.Mp;
      return true;
    });
  };
  // symmetric product of two symmetric m x m matrices in half storage: dst = 2^shift * L * R (upper triangle computed
  // and mirrored; L and R commute)
  auto symprod = [&](auto&& want, auto&& lhs, auto&& rhs, auto&& dst, int shift) -> hipError_t {
    return run_mode(MODE_SYRK, false, false, 1, [&](const NsProblem& P, GemmParams& g, double& fa, double& fi) {
      if (!want(P)) return false;
      const NsPlan& pl = P.pl;
      const long as = (long)pl.Mp * pl.Mp;
      g.batch = P.q.batch;
      g.P = lhs(P); g.Q = rhs(P); g.strideP = g.strideQ = as; g.ldp = g.ldq = pl.Mp; g.K = pl.Mp;
      g.tilesM = g.tilesN = pl.Mp / pl.tile;
      g.C = dst(P); g.strideC = as; g.ldc = pl.Mp;
      g.alpha = ldexpf(1.f, shift); g.beta = 0.f;
      const double bm = P.q.batch, dm = pl.m, tl = pl.tile;
      fa = bm * dm * dm * dm;
      fi = bm * 2.0 * tl * tl * sym_tiles_issued(pl.Mp / pl.tile) * pl.Mp;
      return true;
    });
  };
  // X' = a X + B X with B = lhs(P) and X^T in Xt[src_of(P)]; the next iterate goes to the other X^T buffer, the last
  // one to the caller
  auto bx = [&](int it, auto&& src_of, auto&& want, auto&& lhs) -> hipError_t {
    const ItCfg k = it_cfg(it);
    return run_mode(MODE_BX, k.split, k.last, k.bx16, [&](const NsProblem& P, GemmParams& g, double& fa, double& fi) {
      if (!want(P)) return false;
      const int src = src_of(P);
      const NsPlan& pl = P.pl;
      const long xs = (long)pl.Mp * pl.Np, as = (long)pl.Mp * pl.Mp;
      g.batch = P.q.batch;
      g.P = lhs(P); g.P2 = P.Bl; g.Q = P.Xt[src]; g.strideP = as; g.strideQ = xs; g.ldp = pl.Mp; g.ldq = pl.Mp;
      g.K = pl.Mp;
      g.tilesM = pl.Mp / pl.tile; g.tilesN = pl.Np / pl.tile;
      g.E = k.fold ? nullptr : P.Xt[src]; g.strideE = xs; g.lde = pl.Mp;
      g.alpha = ldexpf(k.a, k.SBi); g.beta = 0.f;
      // B carries 2^SB, a half operand 2^sx, a half result 2^sx; the caller's result carries nothing
      g.out_shift = -k.SBi - (k.half_ops ? P.sx : 0) + (k.half_out ? P.sx : 0);
      g.scale = (P.defer && it == 0) ? P.scale : nullptr;
      if (!k.last) {
        g.Ct = P.Xt[src ^ 1]; g.strideCt = xs; g.ldct = pl.Mp;   // only X'^T: no product reads a row-major X
      } else {
        g.m_valid = pl.m; g.n_valid = pl.n;
        if (!P.tall) { g.C = (__bf16*)P.q.out; g.strideC = P.q.out_batch_stride; g.ldc = P.q.out_ld; }
        else { g.Ct = (__bf16*)P.q.out; g.strideCt = P.q.out_batch_stride; g.ldct = P.q.out_ld; }
      }
      const double bm = P.q.batch, dm = pl.m, dn = pl.n, tl = pl.tile;
      fa = bm * 2.0 * dm * dm * dn;
      fi = bm * 2.0 * tl * tl * (double)(pl.Mp / pl.tile) * (pl.Np / pl.tile) * pl.Mp * (k.split ? 2.0 : 1.0);
      return true;
    });
  };
  auto every = [](const NsProblem&) { return true; };
  auto on_gram = [](const NsProblem& P) { return P.gram_tail; };
  auto plain = [](const NsProblem& P) { return !P.gram_tail; };
  auto in_bh = [](const NsProblem& P) { return P.Bh; };

  int cur = 0;
  const int n_plain_iters = any_tail ? iters - 2 : iters;
  for (int it = 0; it < n_plain_iters; ++it) {
    if ((e = syrkt(it, cur, every)) != hipSuccess) return (int)e;
    if ((e = syrk2(it, every, in_bh)) != hipSuccess) return (int)e;
    if ((e = bx(it, [&](const NsProblem&) { return cur; }, every, in_bh)) != hipSuccess) return (int)e;
    cur ^= 1;
  }
  if (any_tail) {
    // X_{N-2} is in Xt[cur] (half); the idle buffer Xt[cur ^ 1] of a fused problem holds T / Q and P_N
    const int i1 = iters - 2, i2 = iters - 1;
    auto buf_t = [&](const NsProblem& P) { return P.Xt[cur ^ 1]; };
    auto buf_p2 = [&](const NsProblem& P) { return P.Xt[cur ^ 1] + (size_t)P.q.batch * P.pl.Mp * P.pl.Mp; };
    auto in_a = [](const NsProblem& P) { return P.A; };
    if ((e = syrkt(i1, cur, every)) != hipSuccess) return (int)e;                                  // A1 = X X^T
    if ((e = syrk2(i1, every, in_bh)) != hipSuccess) return (int)e;                                // P1 (in Bh)
    if ((e = symprod(on_gram, in_bh, in_a, buf_t, SH_B - SH_B - SH_A)) != hipSuccess) return (int)e;  // T = P1 A1
    if (!all_tail && (e = bx(i1, [&](const NsProblem&) { return cur; }, plain, in_bh)) != hipSuccess) return (int)e;  // X' = P1 X
    if ((e = symprod(on_gram, buf_t, in_bh, in_a, SH_A - 2 * SH_B)) != hipSuccess) return (int)e;    // A2 = T P1
    if (!all_tail && (e = syrkt(i2, cur ^ 1, plain)) != hipSuccess) return (int)e;                 // A2 = X' X'^T
    // P2: next to T for a fused problem (P1 is still needed), over P1 otherwise
    if ((e = syrk2(i2, every, [&](const NsProblem& P) { return P.gram_tail ? buf_p2(P) : P.Bh; })) != hipSuccess) return (int)e;
    if ((e = symprod(on_gram, buf_p2, in_bh, buf_t, SH_B - 2 * SH_B)) != hipSuccess) return (int)e;   // Q = P2 P1 (over T)
    // the result, one launch for all: Q X_{N-2} for a fused problem, P2 X_{N-1} otherwise
    e = bx(i2, [&](const NsProblem& P) { return P.gram_tail ? cur : cur ^ 1; }, every,
           [&](const NsProblem& P) { return P.gram_tail ? buf_t(P) : P.Bh; });
    if (e != hipSuccess) return (int)e;
  }
  return 0;
}
}  // namespace

int muon_ns_grouped(const muon_ns_problem* problems_host, int n_problems, const float* abc_host, int iters, float eps,
                    int eps_mode, int prec_mode, int flags, void* ws_dev, size_t ws_bytes, void* stream) {
  return ns_grouped_impl(problems_host, nullptr, MomentumCoef{}, n_problems, abc_host, iters, eps, eps_mode, prec_mode,
                         flags, ws_dev, ws_bytes, stream);
}

int muon_momentum_ns_grouped(const muon_mns_problem* problems_host, int n_problems, float c_mm, float c_mg, float c_um,
                             float c_ug, float l2, const float* abc_host, int iters, float eps, int eps_mode,
                             int prec_mode, int flags, void* ws_dev, size_t ws_bytes, void* stream) {
  if (!problems_host || n_problems <= 0) return MUON_E_ARG;
  if (flags & MUON_NS_CAST_INPUT_FIRST) return MUON_E_ARG;   // the update is always rounded to bf16 before its norm here
  std::vector<muon_ns_problem> q(n_problems);
  for (int i = 0; i < n_problems; ++i) {
    const muon_mns_problem& f = problems_host[i];
    if (!f.g_ptrs || !f.m_ptrs || (l2 != 0.f && !f.w_ptrs) || !f.out || f.batch <= 0) return MUON_E_ARG;
    for (int d : {f.g_dtype, f.m_dtype})
      if (d != MUON_DTYPE_BF16 && d != MUON_DTYPE_F32) return MUON_E_ARG;
    if (l2 != 0.f && f.w_dtype != MUON_DTYPE_BF16 && f.w_dtype != MUON_DTYPE_F32) return MUON_E_ARG;
    for (int b = 0; b < f.batch; ++b)
      if (!f.g_ptrs[b] || !f.m_ptrs[b] || (l2 != 0.f && !f.w_ptrs[b])) return MUON_E_ARG;
    q[i].in = nullptr; q[i].out = f.out;
    q[i].in_batch_stride = 0; q[i].out_batch_stride = f.out_batch_stride;
    q[i].in_dtype = MUON_DTYPE_BF16; q[i].in_ld = f.cols; q[i].out_ld = f.out_ld;
    q[i].batch = f.batch; q[i].rows = f.rows; q[i].cols = f.cols;
  }
  const MomentumCoef mc = {c_mm, c_mg, c_um, c_ug, l2};
  return ns_grouped_impl(q.data(), problems_host, mc, n_problems, abc_host, iters, eps, eps_mode, prec_mode, flags, ws_dev,
                         ws_bytes, stream);
}

int muon_ns_batched(const void* in_dev, int in_dtype, int64_t in_batch_stride, int in_ld, void* out_dev,
                    int64_t out_batch_stride, int out_ld, int batch, int rows, int cols, const float* abc_host,
                    int iters, float eps, int eps_mode, int prec_mode, int flags, void* ws_dev, size_t ws_bytes,
                    void* stream) {
  muon_ns_problem q;
  q.in = in_dev; q.out = out_dev;
  q.in_batch_stride = in_batch_stride; q.out_batch_stride = out_batch_stride;
  q.in_dtype = in_dtype; q.in_ld = in_ld; q.out_ld = out_ld;
  q.batch = batch; q.rows = rows; q.cols = cols;
  if (!ws_dev) return MUON_E_ARG;
  return muon_ns_grouped(&q, 1, abc_host, iters, eps, eps_mode, prec_mode, flags, ws_dev, ws_bytes, stream);
}

int muon_ns_batched_static(const void* in_dev, int in_dtype, int64_t in_batch_stride, int in_ld, void* out_dev,
                           int64_t out_batch_stride, int out_ld, int batch, int rows, int cols, const float* abc_host,
                           int iters, float eps, int eps_mode, int prec_mode, int flags, void* stream_) {
  if (batch <= 0 || rows <= 0 || cols <= 0) return MUON_E_ARG;
  if (prec_mode != MUON_PREC_BF16 && prec_mode != MUON_PREC_BF16_BSPLIT && prec_mode != MUON_PREC_F16) return MUON_E_ARG;
  if (plan_bytes_bound(batch, rows, cols, prec_mode) > (size_t)MUON_NS_STATIC_SCRATCH_BYTES) return MUON_E_STATIC_LIMIT;
  hipStream_t stream = (hipStream_t)stream_;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  StaticScratch* sc = nullptr;
  const int st = static_scratch(&sc);
  if (st) return st;
  // Calls on one stream are ordered by the stream.  A call on ANOTHER stream than the last one first waits (on the
  // device) for the end of that call, so the two do not overlap on the array.  Not under stream capture: a captured call
  // is replayed later, in an order that only the caller knows, and an event recorded outside the capture cannot be
  // waited for inside it; replays that overlap other users of the array are the caller's to order.
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  hipError_t e = hipStreamIsCapturing(stream, &capture);
  if (e != hipSuccess) return (int)e;
  const bool eager = capture == hipStreamCaptureStatusNone;
  if (eager && sc->has_last && sc->last != stream && (e = hipStreamWaitEvent(stream, sc->done, 0)) != hipSuccess) return (int)e;
  // every byte of the workspace that a kernel reads is written earlier in the same call (the layout pass writes the
  // zero padding, the products write whole tiles, the K-split counters are cleared by a kernel), so nothing left over
  // from the previous call has to be cleared
  const int rc = muon_ns_batched(in_dev, in_dtype, in_batch_stride, in_ld, out_dev, out_batch_stride, out_ld, batch, rows,
                                 cols, abc_host, iters, eps, eps_mode, prec_mode, flags, sc->ptr,
                                 MUON_NS_STATIC_SCRATCH_BYTES, stream_);
  if (eager) {
    // (also after a failed call: some of its launches may be in flight)
    if ((e = hipEventRecord(sc->done, stream)) != hipSuccess) return rc ? rc : (int)e;
    sc->last = stream;
    sc->has_last = true;
  }
  return rc;
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

int muon_scalar_update(const muon_scalar_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                       int algo, int hyperball, float lr, float beta1, float beta2, float lr_wd, float eps, int step,
                       int cautious, float* scratch_dev, void* stream) {
  if (n_items == 0) return 0;
  if (!items_dev || !prefix_dev || n_items < 0 || total_chunks < n_items || step < 1) return MUON_E_ARG;
  if (algo != MUON_ALGO_ADAMW && algo != MUON_ALGO_LION) return MUON_E_ARG;
  if (hyperball && (algo != MUON_ALGO_ADAMW || !scratch_dev || ((uintptr_t)scratch_dev & 7))) return MUON_E_ARG;
  ScalarHyper h;
  h.lr = lr; h.lr_wd = lr_wd; h.eps = eps;
  h.w1 = 1.f - beta1; h.w2 = 1.f - beta2;
  h.bias1 = (float)(1.0 - pow((double)beta1, (double)step));
  h.bias2_sqrt = (float)sqrt(1.0 - pow((double)beta2, (double)step));
  h.cautious = cautious;
  return (int)launch_scalar_update(items_dev, prefix_dev, n_items, total_chunks, algo, hyperball, h, scratch_dev,
                                   (hipStream_t)stream);
}

int muon_scalar_update_dev(const muon_scalar_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                           int algo, int hyperball, const muon_hyper* hyper_dev, float* scratch_dev, void* stream) {
  if (n_items == 0) return 0;
  if (!items_dev || !prefix_dev || !hyper_dev || n_items < 0 || total_chunks < n_items) return MUON_E_ARG;
  if (((uintptr_t)hyper_dev & 3) != 0) return MUON_E_ARG;
  if (algo != MUON_ALGO_ADAMW && algo != MUON_ALGO_LION) return MUON_E_ARG;
  if (hyperball && (algo != MUON_ALGO_ADAMW || !scratch_dev || ((uintptr_t)scratch_dev & 7))) return MUON_E_ARG;
  return (int)launch_scalar_update(items_dev, prefix_dev, n_items, total_chunks, algo, hyperball, ScalarHyper{}, scratch_dev,
                                   (hipStream_t)stream, hyper_dev);
}

// ---- MuonBall -------------------------------------------------------------------------------------------
namespace {
struct SnPlan {
  NsPlan pl;
  size_t off_x, off_g, off_g2, off_g4, off_xscale, off_xpart, off_z, off_part, total;
};
SnPlan make_sn_plan(int batch, int rows, int cols) {
  SnPlan s;
  s.pl = make_plan(batch, rows, cols, MUON_PREC_BF16);
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = (size_t)round_up((long)(off + bytes), 256); return o; };
  s.off_x = take((size_t)batch * s.pl.Mp * s.pl.Np * 2);
  s.off_g = take((size_t)batch * s.pl.Mp * s.pl.Mp * 2);
  s.off_g2 = take((size_t)batch * s.pl.Mp * s.pl.Mp * 2);   // G^2 and G^4 of the grouped rounds (used from 6 / 16 rounds on)
  s.off_g4 = take((size_t)batch * s.pl.Mp * s.pl.Mp * 2);
  s.off_xscale = take((size_t)batch * sizeof(float));
  s.off_xpart = take((size_t)batch * (s.pl.Mp / 64) * (s.pl.Np / 64) * sizeof(float));
  s.off_z = take((size_t)2 * batch * s.pl.Mp * sizeof(float));
  s.off_part = take((size_t)2 * batch * (s.pl.Mp / SN_ROWS) * 2 * sizeof(float));
  s.total = off;
  return s;
}
int check_sn_problem(const muon_sn_problem& q) {
  if (!q.w_ptrs || !q.sigma_out) return MUON_E_ARG;
  if (q.batch <= 0 || q.rows <= 0 || q.cols <= 0 || q.ld < q.cols) return MUON_E_ARG;
  if (q.dtype != MUON_DTYPE_BF16 && q.dtype != MUON_DTYPE_F32) return MUON_E_ARG;
  if (q.flags & ~MUON_SN_TRANSPOSED) return MUON_E_ARG;
  for (int b = 0; b < q.batch; ++b)
    if (!q.w_ptrs[b]) return MUON_E_ARG;
  return 0;
}
}  // namespace

size_t muon_spectral_norm_workspace_bytes(const muon_sn_problem* problems_host, int n_problems) {
  if (!problems_host || n_problems <= 0) return 0;
  size_t total = 0;
  for (int i = 0; i < n_problems; ++i) {
    const muon_sn_problem& q = problems_host[i];
    if (q.batch <= 0 || q.rows <= 0 || q.cols <= 0) return 0;
    total += make_sn_plan(q.batch, q.rows, q.cols).total;
  }
  return total;
}

namespace {
int spectral_norm_impl(const muon_sn_problem* problems_host, int n_problems, int steps, void* ws_dev, size_t ws_bytes,
                       void* stream_, float* short_out, float* long_out);
}

int muon_spectral_norm(const muon_sn_problem* problems_host, int n_problems, int steps, void* ws_dev, size_t ws_bytes,
                       void* stream) {
  return spectral_norm_impl(problems_host, n_problems, steps, ws_dev, ws_bytes, stream, nullptr, nullptr);
}

int muon_power_iteration(const void* const* w_ptrs_host, int dtype, int ld, int batch, int rows, int cols, int steps,
                         float* sigma_out_dev, float* u_out_dev, float* v_out_dev, void* ws_dev, size_t ws_bytes,
                         void* stream) {
  if (!u_out_dev || !v_out_dev) return MUON_E_ARG;
  muon_sn_problem q = {};
  q.w_ptrs = w_ptrs_host; q.sigma_out = sigma_out_dev;
  q.dtype = dtype; q.ld = ld; q.batch = batch; q.rows = rows; q.cols = cols; q.flags = 0;
  // the short-side vector is u for a wide matrix and v for a tall one
  const bool tall = rows > cols;
  return spectral_norm_impl(&q, 1, steps, ws_dev, ws_bytes, stream, tall ? v_out_dev : u_out_dev,
                            tall ? u_out_dev : v_out_dev);
}

namespace {
int spectral_norm_impl(const muon_sn_problem* problems_host, int n_problems, int steps, void* ws_dev, size_t ws_bytes,
                       void* stream_, float* short_out, float* long_out) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!problems_host || n_problems <= 0 || steps < 1 || !ws_dev) return MUON_E_ARG;
  if ((short_out || long_out) && (n_problems != 1 || !short_out || !long_out)) return MUON_E_ARG;
  if ((uintptr_t)ws_dev & 255) return MUON_E_WORKSPACE;
  // tall: the matrix meant (after MUON_SN_TRANSPOSED) has more rows than columns; use_t: its short-side-first copy is
  // the transpose of the stored block
  struct Prob { muon_sn_problem q; SnPlan sp; __bf16 *X, *G, *G2, *G4; float *xscale, *xpart, *z, *part; bool tall, use_t; };
  const int levels = spectral_power_levels(steps);
  std::vector<Prob> pr(n_problems);
  size_t off = 0;
  for (int i = 0; i < n_problems; ++i) {
    Prob& P = pr[i];
    P.q = problems_host[i];
    const int st = check_sn_problem(P.q);
    if (st) return st;
    P.sp = make_sn_plan(P.q.batch, P.q.rows, P.q.cols);
    if ((double)P.sp.pl.Mp * P.sp.pl.Np * 2.0 >= 4294967296.0) return MUON_E_UNSUPPORTED;
    if (off + P.sp.total > ws_bytes) return MUON_E_WORKSPACE;
    char* ws = (char*)ws_dev + off;
    off += P.sp.total;
    P.X = (__bf16*)(ws + P.sp.off_x);
    P.G = (__bf16*)(ws + P.sp.off_g);
    P.G2 = levels >= 1 ? (__bf16*)(ws + P.sp.off_g2) : nullptr;
    P.G4 = levels >= 2 ? (__bf16*)(ws + P.sp.off_g4) : nullptr;
    P.xscale = (float*)(ws + P.sp.off_xscale);
    P.xpart = (float*)(ws + P.sp.off_xpart);
    P.z = (float*)(ws + P.sp.off_z);
    P.part = (float*)(ws + P.sp.off_part);
    const bool transposed = (P.q.flags & MUON_SN_TRANSPOSED) != 0;
    P.tall = transposed ? P.q.cols > P.q.rows : P.q.rows > P.q.cols;
    P.use_t = transposed != P.tall;
  }
  hipError_t e;
  // bf16 copy of every matrix with its short side first, zero padded to the GEMM tile, and its sums of squares per tile
  for (const Prob& P : pr) {
    const NsPlan& pl = P.sp.pl;
    const long xs = (long)pl.Mp * pl.Np;
    const size_t xt = (size_t)(pl.Mp / 64) * (pl.Np / 64);
    // one launch per LAYOUT_PTRS_MAX matrices of the class (the matrices are separate allocations: pointers by value)
    for (int b0 = 0; b0 < P.q.batch; b0 += LAYOUT_PTRS_MAX) {
      LayoutPtrs lp = {};
      const int nb = std::min(LAYOUT_PTRS_MAX, P.q.batch - b0);
      for (int k = 0; k < nb; ++k) lp.p[k] = P.q.w_ptrs[b0 + k];
      __bf16* dst = P.X + (size_t)b0 * xs;
      if (!P.use_t)
        e = launch_layout_ptrs(lp, nb, P.q.dtype, P.q.ld, P.q.rows, P.q.cols, dst, xs, pl.Np, pl.Mp, pl.Np, nullptr, 0, 0,
                               stream, P.xpart + (size_t)b0 * xt);
      else
        e = launch_layout_ptrs(lp, nb, P.q.dtype, P.q.ld, P.q.rows, P.q.cols, nullptr, 0, 0, pl.Np, pl.Mp, dst, xs, pl.Np,
                               stream, P.xpart + (size_t)b0 * xt);
      if (e != hipSuccess) return (int)e;
    }
  }
  // a symmetric product for every problem, problems of one tile size sharing launches: dst = scale^2 * src src^T
  // (src: [d_p][K] row-major per matrix)
  auto gram = [&](auto&& src_of, auto&& k_of, auto&& dst_of, auto&& scale_of) -> int {
    for (int tile : {256, 128}) {
      GroupedGemmParams gp = {};
      auto flush = [&]() -> hipError_t {
        if (gp.n_groups == 0) return hipSuccess;
        hipError_t err = launch_ns_gemm_grouped(tile, MODE_SYRK, false, false, gp, stream);
        gp = GroupedGemmParams{};
        return err;
      };
      for (const Prob& P : pr) {
        const NsPlan& pl = P.sp.pl;
        if (pl.tile != tile) continue;
        GemmParams g = {};
        const int K = k_of(P);
        g.batch = P.q.batch;
        g.P = src_of(P); g.Q = g.P; g.strideP = g.strideQ = (long)pl.Mp * K; g.ldp = g.ldq = K; g.K = K;
        g.tilesM = g.tilesN = pl.Mp / pl.tile;
        g.C = dst_of(P); g.strideC = (long)pl.Mp * pl.Mp; g.ldc = pl.Mp; g.alpha = 1.f; g.beta = 0.f;
        g.scale = scale_of(P);
        const long tiles = ns_gemm_tiles(MODE_SYRK, g);
        if (tiles > 0x7ffffff0L) return MUON_E_UNSUPPORTED;
        if (gp.n_groups == MAX_GROUPS || tiles + gp.tile_start[gp.n_groups] > 0x7ffffff0L) {
          if ((e = flush()) != hipSuccess) return (int)e;
        }
        gp.g[gp.n_groups] = g;
        gp.tile_start[gp.n_groups + 1] = gp.tile_start[gp.n_groups] + (int)tiles;
        ++gp.n_groups;
      }
      if ((e = flush()) != hipSuccess) return (int)e;
    }
    return 0;
  };
  // the classes in launches of at most SN_MAX_CLASSES
  auto for_class_chunks = [&](auto&& run) -> int {
    SnParams sp = {};
    for (size_t i = 0; i <= pr.size(); ++i) {
      if (i == pr.size() || sp.n == SN_MAX_CLASSES ||
          (long)pr[i].q.batch * (pr[i].sp.pl.Mp / SN_ROWS) + sp.blk_start[sp.n] > 0x3ffffff0L) {
        if (sp.n > 0 && (e = run(sp)) != hipSuccess) return (int)e;
        sp = SnParams{};
        if (i == pr.size()) break;
      }
      const Prob& P = pr[i];
      const NsPlan& pl = P.sp.pl;
      const long blocks = (long)P.q.batch * (pl.Mp / SN_ROWS);
      if (blocks > 0x3ffffff0L) return MUON_E_UNSUPPORTED;
      SnClass& c = sp.c[sp.n];
      c.X = P.X; c.G = P.G; c.G2 = P.G2; c.G4 = P.G4;
      c.xscale = P.xscale; c.xpart = P.xpart; c.xtiles = (pl.Mp / 64) * (pl.Np / 64);
      c.z = P.z; c.part = P.part; c.sigma = P.q.sigma_out;
      c.batch = P.q.batch; c.d = pl.m; c.d_p = pl.Mp; c.L_p = pl.Np; c.nblk = pl.Mp / SN_ROWS; c.tall = P.tall ? 1 : 0;
      sp.blk_start[sp.n + 1] = sp.blk_start[sp.n] + (int)blocks;
      ++sp.n;
    }
    return 0;
  };
  int st;
  // G = s^2 X X^T with s a power of two near sqrt(d) / |X|_F (mean eigenvalue about 1: no power of G leaves the bf16 range)
  if ((st = for_class_chunks([&](const SnParams& sp) { return launch_spectral_xscale(sp, stream); })) != 0) return st;
  if ((st = gram([](const Prob& P) { return P.X; }, [](const Prob& P) { return P.sp.pl.Np; },
                 [](const Prob& P) { return P.G; }, [](const Prob& P) { return (const float*)P.xscale; })) != 0)
    return st;
  // G2 = G^2, G4 = G2^2
  if (levels >= 1) {
    if ((st = gram([](const Prob& P) { return P.G; }, [](const Prob& P) { return P.sp.pl.Mp; },
                   [](const Prob& P) { return P.G2; }, [](const Prob&) { return (const float*)nullptr; })) != 0)
      return st;
  }
  if (levels >= 2) {
    if ((st = gram([](const Prob& P) { return P.G2; }, [](const Prob& P) { return P.sp.pl.Mp; },
                   [](const Prob& P) { return P.G4; }, [](const Prob&) { return (const float*)nullptr; })) != 0)
      return st;
  }
  // the rounds: every application of G (or of a power of it) is one launch over all classes
  int final_src[2] = {0, 0};
  SnParams last = {};
  if ((st = for_class_chunks([&](const SnParams& sp) {
         last = sp;
         return launch_spectral_iterate(sp, steps, stream, final_src);
       })) != 0)
    return st;
  if (short_out) {   // one problem, one class: its singular vectors from the iterates that are still in the workspace
    const SnClass& c = last.c[0];
    const int L = pr[0].sp.pl.n;
    if ((e = launch_spectral_vectors(c, L, final_src[c.tall ? 1 : 0], short_out, long_out, stream)) != hipSuccess) return (int)e;
  }
  return 0;
}
}  // namespace

int muon_ball_apply(const muon_ball_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks, float lr,
                    float decay, int retract_mode, float retract_step, float* log_out_dev, void* stream) {
  if (n_items == 0) return 0;
  if (!items_dev || !prefix_dev || n_items < 0 || total_chunks < n_items) return MUON_E_ARG;
  if (retract_mode != MUON_RETRACT_HARD && retract_mode != MUON_RETRACT_DYNAMIC) return MUON_E_ARG;
  return (int)launch_ball_apply(items_dev, prefix_dev, n_items, total_chunks, lr, decay, retract_mode, retract_step,
                                log_out_dev, (hipStream_t)stream);
}

int muon_calibration_copy(const void* src_dev, void* dst_dev, size_t bytes, void* stream) {
  if (!src_dev || !dst_dev || (bytes & 15) || ((uintptr_t)src_dev & 15) || ((uintptr_t)dst_dev & 15)) return MUON_E_ARG;
  return (int)launch_calibration_copy(src_dev, dst_dev, bytes, (hipStream_t)stream);
}

int muon_calibration_stream(int mode, const void* a_dev, void* b_dev, void* c_dev, size_t bytes, void* stream) {
  if (mode == MUON_STREAM_COPY) return muon_calibration_copy(a_dev, b_dev, bytes, stream);
  if (mode != MUON_STREAM_READ && mode != MUON_STREAM_MIX) return MUON_E_ARG;
  if (!a_dev || !b_dev || (bytes & 15) || ((uintptr_t)a_dev & 15) || ((uintptr_t)b_dev & 15)) return MUON_E_ARG;
  if (mode == MUON_STREAM_MIX && (!c_dev || ((uintptr_t)c_dev & 15))) return MUON_E_ARG;
  return (int)launch_calibration_stream(mode, a_dev, b_dev, c_dev, bytes, (hipStream_t)stream);
}

int muon_profile_begin(void) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  g_prof.clear();
  while ((int)g_prof_start.size() < PROF_POOL) {
    hipEvent_t a, b;
    hipError_t e = hipEventCreate(&a);
    if (e != hipSuccess) return (int)e;
    if ((e = hipEventCreate(&b)) != hipSuccess) { (void)hipEventDestroy(a); return (int)e; }
    g_prof_start.push_back(a);
    g_prof_stop.push_back(b);
  }
  g_prof.reserve(PROF_POOL);
  g_prof_on.store(true, std::memory_order_release);
  return 0;
}

int muon_profile_collect(float* ms_host, int32_t* key_host, double* flops_algorithmic_host,
                         double* flops_issued_host, int capacity) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  g_prof_on.store(false, std::memory_order_release);
  int n = 0;
  for (size_t i = 0; i < g_prof.size(); ++i) {
    float ms = 0.f;
    hipError_t e = hipEventSynchronize(g_prof_stop[i]);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, g_prof_start[i], g_prof_stop[i]);
    if (e != hipSuccess) { g_prof.clear(); return -(int)e - 1000; }
    if (n < capacity) {
      if (ms_host) ms_host[n] = ms;
      if (key_host) key_host[n] = g_prof[i].key;
      if (flops_algorithmic_host) flops_algorithmic_host[n] = g_prof[i].work_algorithmic;
      if (flops_issued_host) flops_issued_host[n] = g_prof[i].work_issued;
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

int muon_update_plain_dev(const muon_post_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                          const muon_hyper* hyper_dev, void* stream) {
  if (n_items == 0) return 0;
  if (!items_dev || !prefix_dev || !hyper_dev || n_items < 0 || total_chunks < n_items) return MUON_E_ARG;
  if (((uintptr_t)hyper_dev & 3) != 0) return MUON_E_ARG;
  return (int)launch_post_plain(items_dev, prefix_dev, n_items, total_chunks, 0.f, 0.f, 0, (hipStream_t)stream, hyper_dev);
}

int muon_update_muonh_dev(const muon_post_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                          const muon_hyper* hyper_dev, float* scratch_dev, void* stream) {
  if (n_items == 0) return 0;
  if (!items_dev || !prefix_dev || !hyper_dev || !scratch_dev || n_items < 0 || total_chunks < n_items) return MUON_E_ARG;
  if (((uintptr_t)hyper_dev & 3) != 0) return MUON_E_ARG;
  if ((uintptr_t)scratch_dev & 7) return MUON_E_WORKSPACE;
  return (int)launch_post_muonh(items_dev, prefix_dev, n_items, total_chunks, 0.f, 0.f, 0.f, 0, scratch_dev,
                                (hipStream_t)stream, hyper_dev);
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
