/* C ABI of the MI355X (gfx950) Muon / MuonH hot path.
 *
 * Plain pointers and sizes only: every pointer named *_dev is DEVICE memory owned by
 * the caller; the library never allocates or frees device memory and never
 * synchronises the host.  All work is enqueued on the stream argument (a
 * hipStream_t passed as void*; NULL = the default stream).
 *
 * Return value of every int function: 0 = success, < 0 = MUON_E_* argument error,
 * > 0 = a hipError_t from a launch.  Nothing throws or aborts.
 *
 * Reference file:line citations are relative to the microsoft/ArchScale checkout.
 */
#ifndef ARCHSCALE_MUON_H
#define ARCHSCALE_MUON_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MUON_ABI_VERSION 3

/* element types of caller tensors */
#define MUON_DTYPE_BF16 0
#define MUON_DTYPE_F32 1

/* how eps enters the Frobenius normalisation */
#define MUON_EPS_ADD 0   /* X / (|X| + eps)      lit_gpt/optim/muon.py:888 */
#define MUON_EPS_CLAMP 1 /* X / max(|X|, eps)    emerging_optimizers/.../spectral_ball_utils.py:46 */

/* precision of B = bA + cA^2 as an operand of B*X */
#define MUON_PREC_BF16 0       /* one bf16 rounding per GEMM epilogue (rounding points of newton_schulz_triton.py:374-378);
                                  the last two iterations round to IEEE half instead unless MUON_NS_NO_GRAM_TAIL is set */
#define MUON_PREC_BF16_BSPLIT 1 /* DIAGNOSTIC mode, superseded by MUON_PREC_F16 (faster: one walk over K per product; a
                                  third of the error): B kept as a bf16 hi+lo pair, B*X accumulates both */
#define MUON_PREC_F16 2         /* the iterate and both Gram-side matrices are kept in IEEE half inside the workspace (inputs
                                   and the result stay bfloat16), each times a power of two that keeps it in the normal
                                   range: eight times the mantissa of bfloat16 at the same matrix-core rate, no hi+lo pair
                                   needed for any of the reference's coefficient tables (muon_momentum_ns_grouped runs the
                                   first iteration in bfloat16 on the unnormalised update and goes to half from there) */

/* flags of muon_ns_batched */
#define MUON_NS_CAST_INPUT_FIRST 1 /* fp32 input: round to bf16 BEFORE taking the norm (muon.py:883-888); default is
                                      normalise in fp32, then round (spectral_ball_utils.py:46-54) */
#define MUON_NS_NO_NORMALIZE 2     /* iterate on the input as it is (no Frobenius normalisation; eps is ignored): one call
                                      with iters = 1 is newton_schulz_step_tsyrk
                                      (emerging_optimizers/orthogonalized_optimizers/muon_utils.py:262-287) */
#define MUON_NS_NO_DIAG_FOLD 4     /* always compute X' = aX + BX with the addend; by default an iteration after the first
                                      with |a| <= 4.2 stores B + aI (the diagonal rounded to bf16 like every other entry
                                      of B; with MUON_PREC_BF16_BSPLIT only in the iterations that keep the hi+lo pair,
                                      where it is exact) and computes X' = (B + aI) X, which saves reading X a second
                                      time */
#define MUON_NS_NO_GRAM_TAIL 8      /* keep the last two iterations as plain iterations in the storage type of prec_mode */
#define MUON_NS_GRAM_TAIL 16        /* take the tail described below also under MUON_PREC_F16 */
/* The tail: a call with at least three iterations whose last two rows have |a| <= 4.2 and 1.5 |b| + 2.25 |c| + |a| <= 500
 * (the range of the half storage; every table of the reference is under 25) (MUON_NS_NO_DIAG_FOLD not set,
 * input normalised, no hi+lo pair) (1) keeps the matrices of the last two iterations in IEEE half also under
 * MUON_PREC_BF16, and (2) for every problem with long side >= 2 x short side finishes on the Gram side:
 * X_N = (P_N P_{N-1}) X_{N-2} with A_{N-1} = P_{N-1} A_{N-2} P_{N-1}, P = aI + bA + cA^2 - three m x m symmetric
 * products instead of one B X and one X X^T product (3 m^2 (n - m) multiply-adds less per matrix).  Default: on under
 * MUON_PREC_BF16 (error against an fp64 run lower than with five plain bfloat16 iterations on every spectrum tried:
 * Gaussian, rank-one spikes, log-spaced, low rank plus noise), off under MUON_PREC_F16 (there it costs 1-2 % of
 * accuracy, 25 % with the polar-express table of msign). */
#define MUON_NS_BSPLIT_TAIL(t) (((t) & 0xff) << 8) /* with MUON_PREC_BF16_BSPLIT: only the last t iterations keep B as a
                                                      hi+lo pair (0 = all); the rounding of B in the last iterations
                                                      dominates the error of the result */

#define MUON_E_ARG (-1)        /* null pointer, non-positive extent, bad enum */
#define MUON_E_WORKSPACE (-2)  /* workspace too small or misaligned */
#define MUON_E_UNSUPPORTED (-3)
#define MUON_E_STATIC_LIMIT (-4) /* muon_ns_batched_static: the problem needs more than MUON_NS_STATIC_SCRATCH_BYTES */

/* elements covered by one block of the multi-tensor kernels; chunk prefixes are in these units */
#define MUON_CHUNK_ELEMS 8192

int muon_abi_version(void);
const char* muon_status_string(int status);

/* ---- Newton-Schulz -------------------------------------------------------------------------
 * Replaces zeropower_via_newtonschulz5 (lit_gpt/optim/muon.py:869-897, lit_gpt/legacy_optim.py:187-213),
 * newton_schulz_triton (lit_gpt/optim/newton_schulz_triton.py:344-382: ns_line_1, ns_line_2, addmm/baddbmm),
 * _small_msign (emerging_optimizers/orthogonalized_optimizers/spectral_ball_utils.py:37-74) and
 * newton_schulz / newton_schulz_step_tsyrk (.../muon_utils.py:68-164, 262-287).
 *
 * in  : [batch] matrices of rows x cols, leading dimension in_ld, batch stride in_batch_stride (elements),
 *       dtype in_dtype.  Not modified.
 * out : bf16, same logical shape, leading dimension out_ld, batch stride out_batch_stride.  May alias `in`
 *       only if in_dtype is bf16 and the strides are equal.
 * abc : HOST array of 3*iters floats, one (a, b, c) row per iteration (the reference has three different
 *       tables; none is compiled in).
 * Each matrix is normalised by its own Frobenius norm, tall matrices (rows > cols) are iterated transposed
 * and returned in the caller's orientation (a square matrix too: orthogonalising the transpose and transposing the
 * result is the same map, and its memory image is then the operand of the iteration as it is).  A bf16 input (or an fp32 one with MUON_NS_CAST_INPUT_FIRST) is not rounded
 * a second time after the normalisation: the workspace takes it times a power of two, exactly, and the rest of the
 * factor is applied in fp32 by the products of the first iteration.
 * ws  : device workspace of at least muon_ns_workspace_bytes(...) bytes, 256-byte aligned.
 */
size_t muon_ns_workspace_bytes(int batch, int rows, int cols, int prec_mode);

int muon_ns_batched(const void* in_dev, int in_dtype, int64_t in_batch_stride, int in_ld,
                    void* out_dev, int64_t out_batch_stride, int out_ld,
                    int batch, int rows, int cols,
                    const float* abc_host, int iters, float eps, int eps_mode, int prec_mode, int flags,
                    void* ws_dev, size_t ws_bytes, void* stream);

/* muon_ns_batched for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as
 * muon_ns_batched, without the workspace: the library's own scratch is a device array of
 * MUON_NS_STATIC_SCRATCH_BYTES that is part of the loaded code object (every GPU the library runs on holds it until
 * the process ends), and the call performs no hipMalloc / hipFree and calls no allocating library routine.
 * A problem whose muon_ns_workspace_bytes(batch, rows, cols, prec_mode) exceeds MUON_NS_STATIC_SCRATCH_BYTES is
 * rejected with MUON_E_STATIC_LIMIT before anything is launched.  All calls on one GPU share that GPU's array:
 * calls on one stream are ordered by the stream; a call on another stream than the previous one first waits, on the
 * device, for the end of that one (an event that the library records after every eager call), so streams and host
 * threads that share the array take turns.  A call under stream capture records and waits for nothing: replays of a
 * captured call that overlap other users of the array on the same GPU race, and ordering them is the caller's job.
 * The first call on a device looks the array's address up (hipGetSymbolAddress) and creates that event; make that call
 * outside a capture. */
#define MUON_NS_STATIC_SCRATCH_BYTES (64u << 20)
int muon_ns_batched_static(const void* in_dev, int in_dtype, int64_t in_batch_stride, int in_ld,
                           void* out_dev, int64_t out_batch_stride, int out_ld,
                           int batch, int rows, int cols,
                           const float* abc_host, int iters, float eps, int eps_mode, int prec_mode, int flags,
                           void* stream);

/* The same for several independent batches of different shapes at once (all shape classes of an optimizer
 * step): each product of the iteration is ONE kernel launch over the tiles of every problem, so there are
 * 15 GEMM launches per call whatever the number of shapes, and the tail of one shape's grid is filled by the
 * next.  Replaces the per-parameter task loop of lit_gpt/optim/muon.py:211-333 around the calls above.
 * problems_host is a HOST array; the workspace is muon_ns_grouped_workspace_bytes(...) bytes. */
typedef struct muon_ns_problem {
  const void* in; /* device, [batch] rows x cols, dtype in_dtype */
  void* out;      /* device, bf16 */
  int64_t in_batch_stride, out_batch_stride; /* elements */
  int32_t in_dtype, in_ld, out_ld, batch, rows, cols;
} muon_ns_problem;

size_t muon_ns_grouped_workspace_bytes(const muon_ns_problem* problems_host, int n_problems, int prec_mode);

int muon_ns_grouped(const muon_ns_problem* problems_host, int n_problems,
                    const float* abc_host, int iters, float eps, int eps_mode, int prec_mode, int flags,
                    void* ws_dev, size_t ws_bytes, void* stream);

/* Algorithmic work of `iters` PLAIN iterations, for roofline accounting: dense-count FLOPs (what a GEMM library
 * executes), symmetric-count FLOPs (upper-triangle SYRK minimum) and FLOPs this library issues for them (tiles incl.
 * padding, three quarters of a diagonal tile, the second pass of the B split).  A call that takes the Gram-side tail
 * (see the flags above) replaces one B X and one X X^T product of every problem with long side >= 2 x short side by three
 * m x m symmetric products; that is not counted here - the per-launch records of muon_profile_collect are the
 * authoritative count of what a call issued. */
void muon_ns_flops(int batch, int rows, int cols, int iters, int prec_mode,
                   double* dense, double* symmetric, double* issued);

/* How the symmetric products of ONE rows x cols matrix are cut along K (no counterpart in the reference; its Triton
 * kernels take one program per output tile, lit_gpt/optim/newton_schulz_triton.py:51-53).  A matrix that leaves few
 * upper-triangle tiles over after whole rounds of the chip and has a long reduction (K >= 8192) runs those leftover tiles
 * as 128 x 128 quadrants with several blocks per quadrant, each over a part of K; the partial sums are added in the order
 * of the parts, so the result is deterministic, and the rule looks at the matrix's own shape only, so a matrix gives
 * the same bits alone and in any batch.  info (6 ints, HOST): for the reduction over the long side (A = X X^T) and
 * then for the reduction over the short side (the m x m products): tiles of 256 x 256 that run whole, leftover tiles
 * that are cut, parts per quadrant (1 = no cut).  muon_ns_workspace_bytes already includes the partial results. */
void muon_ns_ksplit_info(int rows, int cols, int* info);

/* Per-launch timing of the Newton-Schulz GEMM kernels, for roofline accounting (no counterpart in the
 * reference).  Between muon_profile_begin() and muon_profile_collect() every GEMM launch of muon_ns_batched is
 * bracketed by a pair of HIP events on its stream.  muon_profile_collect waits for them, writes up to `capacity`
 * records to the HOST arrays (any may be NULL) and returns the number of launches recorded (< 0 on error):
 *   ms                elapsed milliseconds of the launch
 *   key               tile*100 + mode*10 + 4*noaddend + split*2 + final  (mode 0 = X X^T, 1 = cAA+bA, 2 = aX + BX,
 *                     3 = X X^T from the transposed iterate; noaddend: an X' = (B + aI) X launch)
 *   flops_algorithmic minimum FLOPs of the product (symmetric products counted once)
 *   flops_issued      FLOPs of the matrix-core instructions actually issued (whole tiles; three quarters of a diagonal
 *                     tile of a symmetric product)
 */
int muon_profile_begin(void);
int muon_profile_collect(float* ms_host, int32_t* key_host, double* flops_algorithmic_host,
                         double* flops_issued_host, int capacity);

/* dst <- src, `bytes` (multiple of 16) of device memory with one plain copy kernel.  No counterpart in the
 * reference: a copy of known size is the yardstick that scales the HBM byte counters of a profiling run. */
int muon_calibration_copy(const void* src_dev, void* dst_dev, size_t bytes, void* stream);

/* Streaming yardsticks with the access pattern of the copy above (no counterpart in the reference): what this GPU's
 * memory delivers to a kernel that only reads (MUON_STREAM_READ: `bytes` of a; b receives nothing but must be valid), that
 * copies (MUON_STREAM_COPY: b <- a) or that has the fused momentum kernel's mix of two reads and two writes
 * (MUON_STREAM_MIX: b <- a + b, c <- (a + b) xor a, as 32-bit words).  The rates of the HBM-bound kernels are reported
 * beside these.  All buffers `bytes` long (a multiple of 16), 16-byte aligned; c_dev only for MUON_STREAM_MIX. */
#define MUON_STREAM_COPY 0
#define MUON_STREAM_READ 1
#define MUON_STREAM_MIX 2
int muon_calibration_stream(int mode, const void* a_dev, void* b_dev, void* c_dev, size_t bytes, void* stream);

/* ---- single products on caller tensors ------------------------------------------------------
 * D = alpha * A A^T + beta * C, A [batch] n x k (bf16, row-major, ld lda), C symmetric n x n or NULL, D n x n,
 * both triangles written.  Replaces ns_line_1 / ns_line_2 (newton_schulz_triton.py:142-178, 269-310) and
 * tsyrk_ex (emerging_optimizers/triton_kernels/syrk.py:188-261).
 */
size_t muon_syrk_workspace_bytes(int batch, int n, int k);
int muon_syrk(const void* a_dev, int64_t a_batch_stride, int lda,
              const void* c_dev, int64_t c_batch_stride, int ldc,
              void* d_dev, int64_t d_batch_stride, int ldd,
              int batch, int n, int k, float alpha, float beta,
              void* ws_dev, size_t ws_bytes, void* stream);

/* ---- multi-tensor momentum ------------------------------------------------------------------
 * For every item:  M <- c_mm*M + c_mg*G ;  U <- c_um*M + c_ug*G   (G rounded to M's dtype first).
 *   lit_gpt Muon   (lit_gpt/optim/muon.py:653-681):  c_mm=mu, c_mg=1, (c_um,c_ug) = (mu,1) nesterov | (1,0)
 *   emerging Muon  (emerging_optimizers/.../orthogonalized_optimizer.py:193-199):
 *                  c_mm=beta, c_mg=1-beta, (c_um,c_ug) = (beta,1-beta) nesterov | (1,0)
 * l2 != 0 first does G <- G + l2*W in place (emerging_optimizers/mixin.py:48-49).
 * items/prefix are DEVICE arrays; prefix[i] = first chunk of item i, prefix[n_items] = total_chunks,
 * an item of numel elements owns ceil(numel / MUON_CHUNK_ELEMS) chunks.
 */
typedef struct muon_pre_item {
  const void* g; /* gradient (read; written only when l2 != 0) */
  void* m;       /* momentum buffer, in place */
  void* u;       /* output */
  const void* w; /* weights, only read when l2 != 0 */
  int64_t numel;
  int32_t g_dtype, m_dtype, u_dtype, w_dtype;
} muon_pre_item;

int muon_momentum(const muon_pre_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                  float c_mm, float c_mg, float c_um, float c_ug, float l2, void* stream);

/* ---- momentum fused into the Newton-Schulz call ---------------------------------------------------------------
 * muon_momentum followed by muon_ns_grouped, without the bf16 update U ever being stored in the parameter's
 * orientation: the momentum kernel writes bf16(U) straight into the (transposed, zero-padded) operand of the iteration
 * with per-tile sums of squares, and the normalisation 1/(|bf16(U)| + eps) (lit_gpt/optim/muon.py:883-888) is applied by
 * the first iteration's GEMM epilogues.  Saves one write and two reads of U per step.  Momentum semantics and
 * coefficients as muon_momentum (muon.py:653-681); a problem is one shape class whose `batch` matrices (rows x cols,
 * contiguous) are given by HOST arrays of device pointers; `out` receives the result as in muon_ns_problem.
 * Workspace: muon_ns_grouped_workspace_bytes of the same shapes.  MUON_NS_CAST_INPUT_FIRST is implied, not accepted.
 */
typedef struct muon_mns_problem {
  const void* const* g_ptrs; /* gradients (read; written when l2 != 0) */
  void* const* m_ptrs;       /* momentum, in place */
  const void* const* w_ptrs; /* weights, read only when l2 != 0 (may be null otherwise) */
  void* out;                 /* bf16, [batch][rows][out_ld] */
  int64_t out_batch_stride;
  int32_t out_ld;
  int32_t g_dtype, m_dtype, w_dtype, batch, rows, cols, reserved;
} muon_mns_problem;

int muon_momentum_ns_grouped(const muon_mns_problem* problems_host, int n_problems, float c_mm, float c_mg, float c_um,
                             float c_ug, float l2, const float* abc_host, int iters, float eps, int eps_mode,
                             int prec_mode, int flags, void* workspace_dev, size_t workspace_bytes, void* stream);

/* ---- multi-tensor weight updates ------------------------------------------------------------
 * x' = x*(1 - lr_wd), or with cautious != 0:  x' = x - lr_wd*x where x*u >= 0  (muon.py:703-718).
 * muon_update_plain:  W <- x' - lr*lr_ratio*U                                   (muon.py:720-722;
 *                     emerging_optimizers/.../orthogonalized_optimizer.py:225-228 with lr_ratio = scale factor)
 * muon_update_muonh:  W <- r*(x' - lr*s*U),  s = |x'|/max(|U|,eps),  r = |x'|/max(|x' - lr*s*U|,eps),
 *                     norms over the whole item                                 (muon.py:614-639, 725-818).
 * scratch_dev: muon_muonh_scratch_floats(n_items, total_chunks) floats, 8-byte aligned.
 */
typedef struct muon_post_item {
  void* w;       /* weights, in place */
  const void* u; /* orthogonalised update, bf16 */
  int64_t numel;
  float lr_ratio; /* adjusted_lr / lr for this tensor (plain update only) */
  int32_t w_dtype;
} muon_post_item;

int muon_update_plain(const muon_post_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                      float lr, float lr_wd, int cautious, void* stream);

size_t muon_muonh_scratch_floats(int n_items, int total_chunks);
int muon_update_muonh(const muon_post_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                      float lr, float lr_wd, float eps, int cautious, float* scratch_dev, void* stream);

/* ---- AdamW / hyperball-AdamW / Lion for the non-matrix groups of the same optimizer ----------------
 * One multi-tensor launch (three for hyperball) over every parameter of a group, replacing the foreach graphs of
 * lit_gpt/optim/scalar_opts.py:118-251 (adamw_update_foreach, lion_update_foreach) and 254-443 (hyperball AdamW:
 * step of relative size lr along the bias-corrected Adam direction, then renormalisation to the previous norm).
 *   AdamW:  M <- lerp(M, G, 1-beta1); V <- lerp(V, G*G, 1-beta2); dir = M / (sqrt(V / (1-beta2^step)) + eps);
 *           W <- x' - lr / (1-beta1^step) * dir            (x' = weight-decayed W, plain or cautious)
 *   Lion:   U = sign(lerp(M, G, 1-beta1)); M <- lerp(M, G, 1-beta2); W <- x' - lr * U
 * scratch_dev: only for hyperball, muon_muonh_scratch_floats(n_items, total_chunks) floats.
 */
#define MUON_ALGO_ADAMW 0
#define MUON_ALGO_LION 1

typedef struct muon_scalar_item {
  void* w;       /* weights, in place */
  const void* g; /* gradient */
  void* m;       /* first moment / momentum, in place */
  void* v;       /* second moment (AdamW), in place; unused for Lion */
  int64_t numel;
  int32_t w_dtype, g_dtype, m_dtype, v_dtype;
} muon_scalar_item;

int muon_scalar_update(const muon_scalar_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                       int algo, int hyperball, float lr, float beta1, float beta2, float lr_wd, float eps, int step,
                       int cautious, float* scratch_dev, void* stream);

/* ---- hyper-parameters from device memory ---------------------------------------------------------------------
 * The training loop rewrites the learning rate (and, under batch ramp-up, weight decay and eps) of every param group
 * before each step (pretrain.py:829-877), and the bias corrections of AdamW change with the step count.  Scalars that
 * are kernel arguments are frozen into a captured HIP graph; the *_dev variants below read them from a muon_hyper block
 * in DEVICE memory instead, which the caller refreshes with one small asynchronous copy before each replay, outside the
 * graph.  Same kernels and same arithmetic as the by-value entry points (bit-identical results for equal values).
 *   muon_update_plain_dev  uses lr, lr_wd, cautious           (replaces the scalars of muon_update_plain)
 *   muon_update_muonh_dev  uses lr, lr_wd, eps, cautious      (muon_update_muonh)
 *   muon_scalar_update_dev uses every field                    (muon_scalar_update; the host computes
 *                          w1 = 1 - beta1, w2 = 1 - beta2 in float, bias1 = 1 - beta1^step and
 *                          bias2_sqrt = sqrt(1 - beta2^step) in double, rounded to float)
 */
typedef struct muon_hyper {
  float lr, lr_wd, eps;
  float w1, w2;            /* 1 - beta1, 1 - beta2 */
  float bias1, bias2_sqrt; /* 1 - beta1^step, sqrt(1 - beta2^step) */
  int32_t cautious;
} muon_hyper;

int muon_update_plain_dev(const muon_post_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                          const muon_hyper* hyper_dev, void* stream);
int muon_update_muonh_dev(const muon_post_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                          const muon_hyper* hyper_dev, float* scratch_dev, void* stream);
int muon_scalar_update_dev(const muon_scalar_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks,
                           int algo, int hyperball, const muon_hyper* hyper_dev, float* scratch_dev, void* stream);

/* ---- MuonBall: spectral norm by power iteration, retraction and update ---------------------------------
 * muon_spectral_norm estimates the top singular value of every matrix of every shape class with the vector
 * sequence of power_iteration (emerging_optimizers/orthogonalized_optimizers/spectral_ball_utils.py:151-166:
 * v <- normalize(W^T (W v)) `steps` times from v = 1, sigma = |W v|), run on the Gram matrix of the short side
 * (one SYRK on the matrix cores per call, then launches over all matrices with fp32 vectors; from 6 / 16 rounds on the
 * Gram matrix is squared once / twice, so that one pass stands for two / four rounds: the normalisation between
 * rounds only scales the vector; the last application, whose quotient is the result, is always the Gram matrix's).
 * A problem is one shape class: `batch` matrices rows x cols with leading dimension ld, given by a HOST array of
 * device pointers (the parameters of a model are separate allocations); the matrix is read as bf16 (fp32 input is
 * rounded first, as the reference does, :158).  sigma_out: device, `batch` floats per problem.
 * MUON_SN_TRANSPOSED in flags: the matrix meant is the TRANSPOSE of the stored rows x cols block (the reference
 * hands W_expert.t() to the iteration, muon_ball.py:441-485; before convergence the estimate depends on the side the
 * all-ones start vector lives on).
 */
#define MUON_SN_TRANSPOSED 1
typedef struct muon_sn_problem {
  const void* const* w_ptrs; /* host array of `batch` device pointers */
  float* sigma_out;          /* device */
  int32_t dtype, ld, batch, rows, cols, flags;
} muon_sn_problem;

size_t muon_spectral_norm_workspace_bytes(const muon_sn_problem* problems_host, int n_problems);
int muon_spectral_norm(const muon_sn_problem* problems_host, int n_problems, int steps, void* workspace_dev,
                       size_t workspace_bytes, void* stream);

/* power_iteration with its singular vectors (spectral_ball_utils.py:151-166 returns (sigma, u, v)): one shape class
 * as in muon_sn_problem (w_ptrs_host: HOST array of `batch` device pointers; dtype, ld, rows, cols as there), sigma as
 * muon_spectral_norm computes it, plus the vectors of the same sequence, UNNORMALISED, in fp32:
 *   u_out_dev [batch][rows]  proportional to W v_steps,   v_out_dev [batch][cols]  proportional to v_steps = (W^T W)^steps 1
 * (the short-side one is the last Gram-side iterate, the long-side one a single pass over the bf16 copy of W).
 * Workspace: muon_spectral_norm_workspace_bytes of the same problem. */
int muon_power_iteration(const void* const* w_ptrs_host, int dtype, int ld, int batch, int rows, int cols, int steps,
                         float* sigma_out_dev, float* u_out_dev, float* v_out_dev, void* workspace_dev,
                         size_t workspace_bytes, void* stream);

/* muon_ball_apply: for every item (a strided rows x cols block of a weight tensor)
 *   W <- f * decay * W - lr * lr_ratio * Phi
 * decay = 1 - lr*wd (decoupled) or 1 - wd (independent) or 1 (emerging_optimizers/mixin.py:33-52, applied before the
 * power iteration in the reference, orthogonalized_optimizer.py:184-190: sigma(decay*W) = decay*sigma(W));
 * f = R / (max(sigma,0) + 1e-8) (MUON_RETRACT_HARD) or 1 + retract_step * bias, bias = -1 if sigma > R else +1
 * (MUON_RETRACT_DYNAMIC; retract_step = alpha*lr) (spectral_ball_utils.py:168-212); Phi = msign(momentum) in bf16,
 * lr_ratio = the shape scale factor (muon_ball.py:349-352, 636-637; p.add_(update, alpha=-lr) :228).
 * log_out_dev (nullable): 2 floats per item, (sigma of the decayed weights, bias).
 */
#define MUON_RETRACT_HARD 0
#define MUON_RETRACT_DYNAMIC 1

typedef struct muon_ball_item {
  void* w;            /* weights, in place */
  const void* phi;    /* orthogonalised update, bf16 */
  const float* sigma; /* device: spectral norm of this block's matrix BEFORE weight decay; null = no retraction (f = 1) */
  int64_t ld_w, ld_phi;
  int32_t rows, cols;
  float radius;   /* target spectral norm R (compute_target_radius, spectral_ball_utils.py:432-440) */
  float lr_ratio; /* get_spectral_ball_scale_factor (:442-466) */
  int32_t w_dtype, reserved;
} muon_ball_item;

int muon_ball_apply(const muon_ball_item* items_dev, const int32_t* prefix_dev, int n_items, int total_chunks, float lr,
                    float decay, int retract_mode, float retract_step, float* log_out_dev, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ARCHSCALE_MUON_H */
