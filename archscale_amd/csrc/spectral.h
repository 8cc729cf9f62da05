// Internal interface between the spectral-norm / MuonBall kernels and the C-ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/archscale_muon.h"

namespace archscale {

constexpr int SN_ROWS = 16;         // rows of the Gram matrix per block (4 waves x 4 rows)
constexpr int SN_MAX_CLASSES = 8;   // shape classes per launch (passed by value)

// One shape class of the power iteration inside the workspace.  X is the zero-padded bf16 copy of the matrices with
// the SHORT side first (d_p x L_p), G = X X^T (d_p x d_p), both row-major; d_p is a multiple of 128, L_p of 8.
// G is formed as xscale^2 X X^T with xscale a power of two near sqrt(d) / |X|_F (mean eigenvalue about 1), so that
// G2 = G^2 and G4 = G2^2 (bf16) stay in range whatever the magnitude of the weights; they let one application stand for
// two or four: the rounds are x <- G x up to the normalisation, so G^k x costs k/4 passes over a matrix of the same
// size.  G2 / G4 are null when the call does not use them.
struct SnClass {
  const __bf16* X;
  const __bf16* G;
  const __bf16* G2;
  const __bf16* G4;
  float* xscale;       // [batch], written by launch_spectral_xscale; the result is divided by it
  const float* xpart;  // [batch][xtiles] sums of squares of X per 64x64 tile (from the layout kernel)
  int xtiles;
  float* z;      // [2][batch][d_p]
  float* part;   // [2][batch][nblk][2]
  float* sigma;  // [batch], result
  int batch, d, d_p, L_p, nblk, tall;
};

struct SnParams {
  int n;
  int blk_start[SN_MAX_CLASSES + 1];  // blocks of class g: batch * nblk
  SnClass c[SN_MAX_CLASSES];
};

// how many of the powers G^2, G^4 a call with `steps` rounds uses (0, 1 or 2): each costs one symmetric product
int spectral_power_levels(int steps);

// xscale[b] = 2^round(log2 sqrt(d / |X_b|_F^2)) for every matrix of every class (0 for a zero matrix)
hipError_t launch_spectral_xscale(const SnParams& sp, hipStream_t stream);

// init + the applications of G that `steps` rounds stand for (`steps` for wide matrices, `steps + 1` for tall ones, the
// last one always G itself; the others G^4, G^2 or G as far as the class has them) + final
// final_src (optional, two ints): which of the two z buffers holds the last iterate of the wide / of the tall classes
hipError_t launch_spectral_iterate(const SnParams& sp, int steps, hipStream_t stream, int* final_src = nullptr);

// after launch_spectral_iterate, for one class: short_out[b][d] = the short-side singular vector (unnormalised: u of a
// wide matrix, v of a tall one), long_out[b][L] = X^T times the iterate before the last (v of a wide matrix, u of a
// tall one, unnormalised); L = the true long extent
hipError_t launch_spectral_vectors(const SnClass& c, int L, int src_final, float* short_out, float* long_out,
                                   hipStream_t stream);

hipError_t launch_ball_apply(const muon_ball_item* items, const int32_t* prefix, int n_items, int total_chunks, float lr,
                             float decay, int retract_mode, float retract_step, float* log_out, hipStream_t stream);

}  // namespace archscale
